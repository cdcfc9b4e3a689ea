"""Mixture-of-experts feed-forward: every row goes through `top` of `experts` small gated feed-forwards.

Router logits z = W_router h + b in float32 (h as the step holds it); a row's experts are the `top` largest logits
(the lower index among equals) and their weights the softmax over those logits alone; an expert is
down(act(gate h) * (up h)) without biases; the row's result is the weighted sum of its experts' results.  With
`shared` a further expert of its own width runs for every row and is added, times sigmoid(w_gate . h), one number
per row (`shared: {"inter": F, "activation": .., "gate": bool}`).

`scores: "softmax_all"` is another router: scores s = softmax(z) over all router outputs, the `top` largest of
s + correction (tensor `correction`, one number per output, seen by the choice alone), weights the chosen experts' s
divided by their sum (+ 1e-20).  `identity: n`: the router has `experts + n` outputs, and the last n of them are experts
without matrices whose result is the row itself.  `shared.gate: False` adds the shared expert as it is.

The experts' matrices are kept stacked, [experts, F, hidden] and [experts, hidden, F]: the step sorts its (row,
choice) pairs by expert on the device and runs the experts' products over tiles of pairs (csrc/moe.hip), so the
host never learns which experts a step uses."""
from __future__ import annotations

from typing import List

import torch

from .. import ops
from ..weights.loader import FLOAT32, TensorDecl, WeightStore
from .base import FeedForward, Runtime, register_feed_forward


@register_feed_forward("moe")
class MoeFeedForward(FeedForward):
    def __init__(self, spec, hidden):
        super().__init__(spec, hidden)
        p = spec.params
        self.experts, self.top, self.inter = int(p["experts"]), int(p["top"]), int(p["inter"])
        self.activation = p.get("activation", "silu")
        self.router_bias_name = spec.tensors.get("router_bias")
        self.scores = p.get("scores", "softmax_top")
        self.identity = int(p.get("identity", 0))
        self.outputs = self.experts + self.identity         # rows of the router
        if self.scores not in ("softmax_top", "softmax_all") or self.identity < 0:
            raise ValueError(f"router scores {self.scores!r} ('softmax_top' or 'softmax_all') with {self.identity} identity experts")
        if self.scores == "softmax_all":
            self.router_bias_name = spec.tensors.get("correction")
        shared = p.get("shared")
        self.shared_inter = int(shared["inter"]) if shared else 0
        self.shared_activation = (shared or {}).get("activation", self.activation)
        self.shared_gated = bool((shared or {}).get("gate", True))
        if not 1 <= self.top <= self.outputs:
            raise ValueError(f"{self.top} of {self.outputs} experts a token")
        if self.outputs > 1024:
            raise ValueError(f"{self.experts} experts are more than the router's kernel takes (1024)")
        for act in (self.activation, self.shared_activation):
            if act not in ops.ACTIVATIONS:
                raise ValueError(f"feed-forward activation {act!r} is not implemented")
        t = spec.tensors
        if len(t["gate"]) != self.experts or len(t["up"]) != self.experts or len(t["down"]) != self.experts:
            raise ValueError("a mixture of experts names one gate, up and down tensor per expert")

    def tensor_decls(self) -> List[TensorDecl]:
        t, H, F = self.spec.tensors, self.hidden, self.inter
        decls = [TensorDecl(t["router"], (self.outputs, H), FLOAT32)]
        if self.router_bias_name is not None:
            decls.append(TensorDecl(self.router_bias_name, (self.outputs,), FLOAT32, init="bias"))
        for e in range(self.experts):
            decls += [TensorDecl(t["gate"][e], (F, H)), TensorDecl(t["up"][e], (F, H)), TensorDecl(t["down"][e], (H, F))]
        if self.shared_inter:
            S = self.shared_inter
            decls += [TensorDecl(t["shared_gate"], (S, H)), TensorDecl(t["shared_up"], (S, H)), TensorDecl(t["shared_down"], (H, S))]
            if self.shared_gated:
                decls.append(TensorDecl(t["shared_weight"], (1, H), FLOAT32))
        return decls

    def bind(self, weights: WeightStore, rt: Runtime) -> None:
        self.rt = rt
        t = self.spec.tensors
        self.router = weights[t["router"]].contiguous()
        self.router_bias = weights[self.router_bias_name].contiguous() if self.router_bias_name is not None else None
        self.w_gate = torch.stack([weights[n] for n in t["gate"]]).contiguous()
        self.w_up = torch.stack([weights[n] for n in t["up"]]).contiguous()
        self.w_down = torch.stack([weights[n] for n in t["down"]]).contiguous()
        self.shared_gate_up = self.shared_down = self.shared_gate = None
        if self.shared_inter:
            self.shared_gate_up = torch.cat([weights[t["shared_gate"]], weights[t["shared_up"]]], dim=0).contiguous()
            self.shared_down = weights[t["shared_down"]].contiguous()
            if self.shared_gated:
                self.shared_gate = weights[t["shared_weight"]].reshape(-1).contiguous()

    def matrices(self):
        """What a row is multiplied with: the router, its `top` experts (counted as the first ones) and the shared expert."""
        top = min(self.top, self.experts)
        own = [self.router, self.w_gate[:top], self.w_up[:top], self.w_down[:top]]
        return own + [m for m in (self.shared_gate_up, self.shared_down) if m is not None]

    def product_shapes(self):
        shapes = [(self.outputs, self.hidden)] + [(2 * self.inter, self.hidden), (self.hidden, self.inter)] * min(self.top, self.experts)
        if self.shared_inter:
            shapes += [(2 * self.shared_inter, self.hidden), (self.hidden, self.shared_inter)]
        return shapes

    def small_tensors(self):
        return [t for t in (self.router_bias, self.shared_gate) if t is not None]

    def emit(self, plan) -> int:
        return plan.moe(self)
