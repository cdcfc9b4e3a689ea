"""Norms over the model's width.

LayerNorm (`"layer"`): out = (x - mean) / sqrt(mean((x - mean)^2) + eps) * gain + bias, all in float32; it also
norms a weighted sum of several residual streams (what a hyper-connected sublayer reads).

RMSNorm: out = x * 1/sqrt(mean(x^2) + eps) * gain, eps inside the root, the gain multiplied
last, no (1 + gain) offset (src/model/simd.rs:75-110,
arch/lib/transformer.json5:9-11)."""
from __future__ import annotations

from typing import List, Optional

import torch

from ..weights.loader import FLOAT32, TensorDecl, WeightStore
from .base import Norm, Runtime, register_norm


@register_norm("rms")
class RMSNorm(Norm):
    def tensor_decls(self) -> List[TensorDecl]:
        return [TensorDecl(self.spec.weight, (self.width,), FLOAT32, init="gain")]

    def bind(self, weights: WeightStore, rt: Runtime) -> None:
        self.rt = rt
        self.gain = weights[self.spec.weight]

    def fold_gain(self) -> torch.Tensor:
        """Hands the gain over to whoever multiplies it into the matrices that read the normed
        rows; from then on this norm only divides by the root mean square."""
        gain, self.gain = self.gain, None
        return gain

    def small_tensors(self):
        return [] if self.gain is None else [self.gain]

    def emit(self, plan) -> int:
        return plan.rms_norm(self.gain, self.spec.eps)


@register_norm("group_rms")
class GroupRMSNorm(Norm):
    """The row in `groups` equal consecutive parts, each divided by its own sqrt(mean(part^2) + eps); then the whole times
    the gain.  One part is the plain RMS norm (whose kernels and gain folding `"rms"` keeps for itself)."""

    def __init__(self, spec, width):
        super().__init__(spec, width)
        self.groups = int(spec.groups)
        if self.groups < 1 or width % self.groups:
            raise ValueError(f"a row of {width} values cannot be normed in {self.groups} equal parts")

    def tensor_decls(self) -> List[TensorDecl]:
        return [TensorDecl(self.spec.weight, (self.width,), FLOAT32, init="gain")]

    def bind(self, weights: WeightStore, rt: Runtime) -> None:
        self.rt = rt
        self.gain = weights[self.spec.weight]

    def small_tensors(self):
        return [self.gain]

    def emit(self, plan) -> int:
        return plan.group_rms_norm(self.gain, self.spec.eps, self.groups)


@register_norm("layer")
class LayerNorm(Norm):
    def tensor_decls(self) -> List[TensorDecl]:
        decls = [TensorDecl(self.spec.weight, (self.width,), FLOAT32, init="gain")]
        if self.spec.bias is not None:
            decls.append(TensorDecl(self.spec.bias, (self.width,), FLOAT32, init="bias"))
        return decls

    def bind(self, weights: WeightStore, rt: Runtime) -> None:
        self.rt = rt
        self.gain = weights[self.spec.weight]
        self.bias = weights[self.spec.bias] if self.spec.bias is not None else None

    def small_tensors(self):
        return [t for t in (self.gain, self.bias) if t is not None]

    def emit(self, plan) -> int:
        return plan.layer_norm(self.gain, self.bias, self.spec.eps)
