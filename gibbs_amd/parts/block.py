"""Arrangements of a layer's parts.

`pre_norm` is LFM2's (arch/families/lfm2.json5:77-88):
    x = x + mixer(norm(x));   x = x + ffn(norm(x))
The residual stream x is float32.  In the native step each residual add is fused into the norm that
follows it, so a half of the block hands its delta on instead of adding it.

In bfloat16 the block folds each norm's gain into the matrices that read the normed rows (the
reference's graph passes fold norm gains into weights too, src/graph/passes/mod.rs).
A step of single decoded tokens (up to `Runtime.fused_decode_rows` rows) then takes the parts' fused
decode kernels: the product itself computes 1/rms of its input rows, and the last product of each
half adds its result into the stream, so a half of a layer is two or three kernels.  Whether a step
does is decided where the step runs (csrc/step_plan.hip), per half, from the step's shape, the
norm (its gain folded) and the part (sizes that its fused kernels take).
"""
from __future__ import annotations

import torch

from ..weights.loader import FLOAT32, TensorDecl
from .base import Block, Connection, Runtime, register_arrangement, register_connection


@register_arrangement("pre_norm")
class PreNormBlock(Block):
    def __init__(self, spec, hidden, layer_index):
        super().__init__(spec, hidden, layer_index)
        missing = [r for r in spec.PRE_NORM_ROLES if r not in self.named]
        if missing:
            raise ValueError(f"a pre-norm block needs the parts {list(spec.PRE_NORM_ROLES)}; layer {spec.name!r} lacks {missing}")

    def bind(self, weights, rt: Runtime) -> None:
        super().bind(weights, rt)
        self._fold(self.mixer_norm, self.mixer)
        self._fold(self.ffn_norm, self.ffn)
        if self.rt.act_dtype == torch.bfloat16:
            self.mixer.pack_matrices()
            self.ffn.pack_matrices()

    def _fold(self, norm, part) -> bool:
        if self.rt.act_dtype != torch.bfloat16 or not self.rt.fold_gains:
            return False
        if not (hasattr(norm, "fold_gain") and hasattr(part, "fold_input_gain")):
            return False
        part.fold_input_gain(norm.fold_gain())
        return True

    def emit(self, plan, caches) -> None:
        plan.half(self.mixer_norm.emit(plan), self.mixer.emit(plan, caches["mixer"]))
        plan.half(self.ffn_norm.emit(plan), self.ffn.emit(plan))


@register_arrangement("parallel_norms")
class ParallelNormsBlock(Block):
    """Mixer and feed-forward side by side, each on a norm of its own of the same stream:

        x = x + mixer(norm1(x)) + ffn(norm2(x))

    Roles: `norm1`, then either `mixer`, or a pair of mixers `left` and `right` that read the same normed rows,
    each result normed over the width by `left_out` / `right_out` and the two averaged; `norm2` and `ffn` may
    be missing (a layer without a feed-forward).  The average's half is multiplied into the two out-norms'
    gains when the weights are bound (exact: a power of two).

    The feed-forward is laid down as a half of its own, x += ffn(norm2(x)), between the mixer's norm and the
    mixer itself: the mixer's rows were normed before that half touched the stream, so both still read the
    same x, and in bfloat16 the half takes the fused few-row kernels (norm2's gain folded into the gate and up
    matrices) as a pre-norm block's does.  The mixers run norm, body and add operations."""

    def __init__(self, spec, hidden, layer_index):
        super().__init__(spec, hidden, layer_index)
        self.pair = "left" in self.named
        want = ["norm1"] + (["left", "right", "left_out", "right_out"] if self.pair else ["mixer"])
        want += ["norm2"] if "ffn" in self.named else []
        missing = [r for r in want if r not in self.named]
        if missing:
            raise ValueError(f"layer {spec.name!r} lacks the parts {missing}")

    def bind(self, weights, rt: Runtime) -> None:
        super().bind(weights, rt)
        if self.pair:
            for norm in (self.left_out, self.right_out):
                norm.gain = norm.gain * 0.5
        if "ffn" in self.named and rt.act_dtype == torch.bfloat16:
            if rt.fold_gains and hasattr(self.norm2, "fold_gain") and hasattr(self.ffn, "fold_input_gain"):
                self.ffn.fold_input_gain(self.norm2.fold_gain())
            self.ffn.pack_matrices()

    def emit(self, plan, caches) -> None:
        h = plan.normed(self.norm1.emit(plan))
        if "ffn" in self.named:
            plan.half(self.norm2.emit(plan), self.ffn.emit(plan))
        if self.pair:
            left = plan.apply(self.left.emit(plan, caches["left"]), h)
            right = plan.apply(self.right.emit(plan, caches["right"]), h)
            plan.drop(h)
            plan.add_normed(self.left_out.emit(plan), left)      # (normed and added in float32, in one pass each)
            plan.add_normed(self.right_out.emit(plan), right)
        else:
            delta = plan.apply(self.mixer.emit(plan, caches["mixer"]), h)
            plan.drop(h)
            plan.add(delta)


@register_arrangement("sandwich")
class SandwichBlock(Block):
    """Sublayers with a norm on both sides, the normed result times a constant:

        x = x + mult * norm1b(mixer(norm1(x)));   x = x + mult * norm2b(ffn(norm2(x)))

    Roles: `norm1`, `mixer`, `norm1b`, and optionally `norm2`, `ffn`, `norm2b` (a layer without a feed-forward), and
    optionally `mixer_input`: a part with state of its own (kind `conv_input`) through which the mixer reads its normed
    rows, x = x + mult * norm1b(mixer(mixer_input(norm1(x)))).
    `mult` is the layer spec's `params["residual_mult"]` (default 1); it is multiplied into the gains of the norms
    behind the sublayers when the weights are bound.  The norm of a sublayer's result and its addition into the
    float32 stream are one pass (`plan.add_normed`)."""

    def __init__(self, spec, hidden, layer_index):
        super().__init__(spec, hidden, layer_index)
        self.has_ffn = "ffn" in self.named
        self.mult = float(spec.params.get("residual_mult", 1.0))
        want = ["norm1", "mixer", "norm1b"] + (["norm2", "norm2b"] if self.has_ffn else [])
        missing = [r for r in want if r not in self.named]
        if missing:
            raise ValueError(f"layer {spec.name!r} lacks the parts {missing}")

    def bind(self, weights, rt: Runtime) -> None:
        super().bind(weights, rt)
        if self.mult != 1.0:
            for norm in [self.norm1b] + ([self.norm2b] if self.has_ffn else []):
                norm.gain = (norm.gain * self.mult).contiguous()
        if rt.act_dtype == torch.bfloat16:       # (tile-ordered copies for the few-row products of decode steps)
            self.mixer.pack_matrices()
            if self.has_ffn:
                self.ffn.pack_matrices()

    def emit(self, plan, caches) -> None:
        subs = [(self.norm1, lambda: self.mixer.emit(plan, caches["mixer"]), self.norm1b, self.named.get("mixer_input"))]
        if self.has_ffn:
            subs.append((self.norm2, lambda: self.ffn.emit(plan), self.norm2b, None))
        for before, body, after, through in subs:
            h = plan.normed(before.emit(plan))
            if through is not None:
                seen = plan.filtered(through.emit(plan, caches["mixer_input"]), h)
                plan.drop(h)
                h = seen
            delta = plan.apply(body(), h)
            plan.drop(h)
            plan.add_normed(after.emit(plan), delta)


@register_connection("hyper")
class HyperConnection(Connection):
    """A sublayer over S residual streams x_1 .. x_S: it reads u = sum_s in[s] x_s and, with its result y, writes all
    streams at once from the old ones, x_t <- sum_s mix[s, t] x_s + out[t] y (`mix` indexed [from, to]).  The three
    tensors are float32; the streams and both sums are float32 in either precision of a run."""

    def tensor_decls(self):
        t, S = self.spec.tensors, self.streams
        return [TensorDecl(t["in"], (S,), FLOAT32, init="gain"), TensorDecl(t["out"], (S,), FLOAT32, init="gain"),
                TensorDecl(t["mix"], (S, S), FLOAT32)]

    def bind(self, weights, rt: Runtime) -> None:
        self.rt = rt
        t = self.spec.tensors
        self.w_in, self.w_mix, self.w_out = weights[t["in"]], weights[t["mix"]].contiguous(), weights[t["out"]]

    def small_tensors(self):
        return [self.w_in, self.w_mix, self.w_out]

    def emit(self, plan) -> int:
        return plan.hyper(self.w_in, self.w_mix, self.w_out)


@register_arrangement("sublayers")
class SublayersBlock(Block):
    """Pre-norm sublayers, each of which may be missing but the first: x += mixer(norm1(x)); x += ffn(norm2(x)).

    Roles: `norm1`, `mixer`, and optionally `norm2` with `ffn`.  With `connection1` (and `connection2` for the
    feed-forward) the model has several residual streams, and a sublayer reads and writes them through its
    connection instead of adding into one: y = sublayer(norm(read(streams))); write(streams, y)."""

    def __init__(self, spec, hidden, layer_index):
        super().__init__(spec, hidden, layer_index)
        self.has_ffn = "ffn" in self.named
        self.connected = "connection1" in self.named
        want = ["norm1", "mixer"] + (["norm2"] if self.has_ffn else []) + (["connection2"] if self.has_ffn and self.connected else [])
        missing = [r for r in want if r not in self.named]
        if missing:
            raise ValueError(f"layer {spec.name!r} lacks the parts {missing}")

    def streams(self) -> int:
        return self.connection1.streams if self.connected else 1

    def emit(self, plan, caches) -> None:
        subs = [(self.norm1, lambda: self.mixer.emit(plan, caches["mixer"]), "connection1")]
        if self.has_ffn:
            subs.append((self.norm2, lambda: self.ffn.emit(plan), "connection2"))
        for norm, body, role in subs:
            if self.connected:
                c = self.named[role].emit(plan)
                h = plan.streams_normed(norm.emit(plan), c)
                delta = plan.apply(body(), h)
                plan.drop(h)
                plan.streams_add(c, delta)
            else:
                plan.half(norm.emit(plan), body())
