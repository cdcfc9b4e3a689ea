"""State-space mixer: a decayed outer-product state per head with one decay per head and token.

One projection of the normed rows gives [z: inner | x: inner | B: groups * state | C: groups * state | dt: heads], inner =
heads * vdim.  x, B and C together pass a short causal convolution per channel (taps [channels, K], the last one the
current token's, with a bias, zeros before a sequence's start) and silu.  dt <- softplus(dt + dt_bias).  Per head h
(reading B and C of group h // (heads / groups)), with a state S [state, vdim] that starts at zero and ' for transposed:

    S = exp(-exp(A_log_h) dt) S + B (dt x)';    y = S' C + D_h x

y (heads side by side) is multiplied by silu(z), normed in `norm_groups` equal parts (each by its own root mean square,
eps inside the root), multiplied by a gain [inner] and projected back.  S and the convolution's last K - 1 inputs live in
the request's slot as float32; dt, the decay, the rule, the gate and the norm are float32 in both precisions of a run.
The rule's kernel is the framework's recurrence (csrc/recurrent.hip: the delta rule's walk without its correction).
"""
from __future__ import annotations

from typing import List, Sequence

from ..cache.needs import StateNeed
from ..weights.loader import FLOAT32, TensorDecl, WeightStore
from .base import Mixer, Runtime, register_mixer

CONV_STATE, RULE_STATE = "ssd_conv", "ssd_rule"


@register_mixer("ssd")
class SsdMixer(Mixer):
    def __init__(self, spec, hidden, layer_index):
        super().__init__(spec, hidden, layer_index)
        p = spec.params
        self.heads, self.vdim, self.state, self.groups = int(p["heads"]), int(p["vdim"]), int(p["state"]), int(p["groups"])
        self.taps, self.norm_groups, self.norm_eps = int(p["taps"]), int(p.get("norm_groups", 1)), float(p["norm_eps"])
        self.inner = self.heads * self.vdim
        self.conv_channels = self.inner + 2 * self.groups * self.state
        if self.heads % self.groups:
            raise ValueError(f"{self.heads} heads are not a multiple of {self.groups} groups")
        if self.inner % self.norm_groups:
            raise ValueError(f"{self.inner} channels cannot be normed in {self.norm_groups} equal parts")
        if self.taps < 1 or not 0 < self.state <= 256:
            raise ValueError(f"taps {self.taps} must be at least 1 and the state size {self.state} at most 256")

    def state_needs(self) -> Sequence[StateNeed]:
        needs = [StateNeed(RULE_STATE, (self.heads, self.state, self.vdim))]
        if self.taps > 1:
            needs.append(StateNeed(CONV_STATE, (self.taps - 1, self.conv_channels)))
        return tuple(needs)

    def tensor_decls(self) -> List[TensorDecl]:
        t, W = self.spec.tensors, self.hidden
        return [TensorDecl(t["in"], (2 * self.inner + 2 * self.groups * self.state + self.heads, W)),
                TensorDecl(t["conv"], (self.conv_channels, self.taps), FLOAT32),
                TensorDecl(t["conv_bias"], (self.conv_channels,), FLOAT32, init="bias"),
                TensorDecl(t["dt_bias"], (self.heads,), FLOAT32, init="bias"), TensorDecl(t["A_log"], (self.heads,), FLOAT32, init="bias"),
                TensorDecl(t["D"], (self.heads,), FLOAT32, init="gain"), TensorDecl(t["norm"], (self.inner,), FLOAT32, init="gain"),
                TensorDecl(t["o"], (W, self.inner))]

    def bind(self, weights: WeightStore, rt: Runtime) -> None:
        self.rt = rt
        t = self.spec.tensors
        self.w_in, self.w_out = weights[t["in"]].contiguous(), weights[t["o"]].contiguous()
        self.conv_taps, self.conv_bias = weights[t["conv"]].contiguous(), weights[t["conv_bias"]].contiguous()
        self.dt_bias, self.a_log, self.skip, self.gain = weights[t["dt_bias"]], weights[t["A_log"]], weights[t["D"]], weights[t["norm"]]

    def matrices(self):
        return [self.w_in, self.w_out]

    def product_shapes(self):
        return [(2 * self.inner + 2 * self.groups * self.state + self.heads, self.hidden), (self.hidden, self.inner)]

    def small_tensors(self):
        return [self.conv_taps, self.conv_bias, self.dt_bias, self.a_log, self.skip, self.gain]

    def state_bytes(self) -> int:
        """Bytes of state that a decoded token reads and writes."""
        return 2 * 4 * (self.heads * self.state * self.vdim + (self.taps - 1) * self.conv_channels)

    def emit(self, plan, cache) -> int:
        rule = cache.states[RULE_STATE]
        conv = cache.states[CONV_STATE] if self.taps > 1 else rule      # (one tap: no inputs are kept)
        return plan.ssd(self, conv_state=conv, rule_state=rule)
