"""A short causal convolution beside the identity on the rows that a mixer is about to read.

    h_t <- h_t + sum_j taps[:, j] * h_(t - K + 1 + j)        (per channel of the model's width; zeros before a sequence's start)

taps [hidden, K], the last one the current token's, no bias.  The last K - 1 rows that a request brought are part of its
state (float32 in its slot), so a prompt may be cut anywhere.  It is a part of a layer like a mixer (it owns state), but
what it makes is not added to the residual stream: an arrangement lays it down between a norm and the mixer that
reads the normed rows (`plan.filtered`).  The kernel is the framework's causal convolution (csrc/recurrent.hip) without
activation and with the input added.
"""
from __future__ import annotations

from typing import List, Sequence

import torch

from ..cache.needs import StateNeed
from ..weights.loader import FLOAT32, TensorDecl, WeightStore
from .base import Mixer, Runtime, register_mixer

INPUT_STATE = "conv_input"


@register_mixer("conv_input")
class ConvInput(Mixer):
    def __init__(self, spec, hidden, layer_index):
        super().__init__(spec, hidden, layer_index)
        self.taps = int(spec.params["taps"])
        if self.taps < 1:
            raise ValueError(f"a convolution of {self.taps} taps")

    def state_needs(self) -> Sequence[StateNeed]:
        return (StateNeed(INPUT_STATE, (self.taps - 1, self.hidden)),) if self.taps > 1 else ()

    def tensor_decls(self) -> List[TensorDecl]:
        return [TensorDecl(self.spec.tensors["taps"], (self.hidden, self.taps), FLOAT32)]

    def bind(self, weights: WeightStore, rt: Runtime) -> None:
        self.rt = rt
        self.w_taps = weights[self.spec.tensors["taps"]].contiguous()
        self._no_state = torch.zeros(1, 1, max(self.hidden, 1), dtype=torch.float32, device=rt.device) if self.taps == 1 else None

    def small_tensors(self):
        return [self.w_taps]

    def state_bytes(self) -> int:
        return 2 * 4 * (self.taps - 1) * self.hidden

    def emit(self, plan, cache) -> int:
        state = cache.states[INPUT_STATE] if self.taps > 1 else self._no_state      # (one tap: no rows are kept)
        return plan.conv_input(taps=self.w_taps, kernel=self.taps, state=state)
