"""Typed configuration of Ruzinex: a decoder of attention layers whose sublayers are normed on both sides.

  layer       x += m norm1b(mixer(norm1(x)));  x += m norm2b(ff(norm2(x)))  with RMS norms and one multiplier m for the
              whole model (`residual_mult`); a layer may have no feed-forward
  mixer       grouped-query attention: biases on the q, k and v projections; the first `rot.dims` channels of every
              head of q and k turned by position (pairs (i, i + dims/2), frequencies base^(-2i/dims) divided by
              `rot.scaling.factor`); scores times `scale`; a learned sink per head in the softmax's denominator;
              values of a head size of their own; value mixing: every layer that says `v_mix`, but the first of them,
              caches and uses (1 - lambda) v + lambda v_first, v_first being the first such layer's values of the token
  feed-forward  dense: down(gelu_tanh(gate h) * (up h));  or a mixture of experts: router logits with a bias, the `top`
              largest, weights by the softmax over those alone, experts down(silu(gate h) * (up h)), and a shared expert
              times sigmoid(w . h)
  output      the model's norm, then the token table again as the head

config.json gives every size and constant; what the design fixes (the activations, the pairing of the rotation, that
the head is the table) is written here.  Positions have no limit of the model's own: `MAX_POSITIONS` is the framework's.
"""
from __future__ import annotations

import copy
from typing import Any, Dict, Mapping, Optional, Sequence, Tuple

from .base import ArchConfig, ConfigError, require
from .spec import FeedForwardSpec, LayerSpec, MixerSpec, ModelSpec, NormSpec, PositionSpec

MAX_POSITIONS = 1 << 20
DENSE_ACTIVATION = "gelu_tanh"
EXPERT_ACTIVATION = "silu"
VALUE_MIX_KEY = 0          # one family of value-mixing layers a model


def _has(tensors, name: str) -> bool:
    return tensors is not None and name in tensors


class RuzinexConfig(ArchConfig):
    architecture = "Ruzinex"

    def __init__(self, cfg: Dict[str, Any], absent: Sequence[str] = (), unread: Sequence[Tuple[str, Tuple[int, ...]]] = ()):
        self.cfg = cfg
        self.absent = frozenset(absent)     # optional tensors that the checkpoint does not hold (a router's bias, a shared expert's gate, a sink)
        self.unread = tuple(unread)         # (name, shape) of checkpoint tensors of parts that a layer does not have

    def __eq__(self, other) -> bool:
        return isinstance(other, RuzinexConfig) and self.cfg == other.cfg

    # ------------------------------------------------------------------ reading
    @classmethod
    def from_dict(cls, cfg: Mapping[str, Any], tensors: Optional[Mapping[str, Sequence[int]]] = None) -> "RuzinexConfig":
        c = copy.deepcopy(dict(cfg))
        width, vocab = int(require(c, "width")), int(require(c, "vocab"))
        if _has(tensors, "embed") and tuple(int(s) for s in tensors["embed"]) != (vocab, width):
            raise ConfigError(f"config.json says embed is {[vocab, width]}, the checkpoint holds {list(tensors['embed'])}")
        float(require(c, "norm.eps"))
        float(c.get("residual_mult", 1.0))
        layers = require(c, "layers")
        if not isinstance(layers, list) or not layers:
            raise ConfigError("config.json: layers must be a non-empty list")
        absent, unread, mixed = [], [], None
        for i, layer in enumerate(layers):
            if layer.get("type") != "attention":
                raise ConfigError(f"layer {i}: mixer type {layer.get('type')!r} is not 'attention'")
            m = layer.get("mixer")
            if not isinstance(m, dict):
                raise ConfigError(f"layer {i}: no mixer sizes")
            for key in ("heads", "kv_heads", "dim", "vdim", "scale"):
                require(m, key)
            if int(m["heads"]) % int(m["kv_heads"]):
                raise ConfigError(f"layer {i}: {m['heads']} heads are not a multiple of {m['kv_heads']} kv heads")
            rot = m.get("rot")
            if rot is not None:
                dims = int(require(rot, "dims"))
                if dims:
                    float(require(rot, "base"))
                if dims % 2 or not 0 <= dims <= int(m["dim"]):
                    raise ConfigError(f"layer {i}: {dims} rotated dimensions of a head of {m['dim']}")
                factor = (rot.get("scaling") or {}).get("factor")
                if factor is not None and not float(factor) > 0:
                    raise ConfigError(f"layer {i}: a scaling factor of {factor}")
            if m.get("v_mix"):
                size = (int(m["kv_heads"]), int(m["vdim"]))
                if mixed is not None and mixed != size:
                    raise ConfigError(f"layer {i}: value mixing needs {mixed[0]} value heads of {mixed[1]}, this layer has {size[0]} of {size[1]}")
                mixed = size
            elif tensors is not None and f"l{i}.mix.vmix" in tensors:
                unread.append((f"l{i}.mix.vmix", tuple(int(s) for s in tensors[f"l{i}.mix.vmix"])))
            if tensors is not None:
                absent += [n for n in (f"l{i}.mix.sink", f"l{i}.mix.q.b") if n not in tensors]
            mlp = layer.get("mlp")
            if mlp is None:
                if tensors is not None:
                    unread += [(n, tuple(int(s) for s in tensors[n])) for n in (f"l{i}.norm2", f"l{i}.norm2b") if n in tensors]
            elif mlp.get("kind") == "dense":
                int(require(mlp, "ff"))
            elif mlp.get("kind") == "moe":
                int(require(mlp, "expert.ff"))
                experts, top = int(require(mlp, "router.experts")), int(require(mlp, "router.top"))
                if not 1 <= top <= experts:
                    raise ConfigError(f"layer {i}: {top} of {experts} experts a token")
                if mlp.get("shared") is not None:
                    int(require(mlp, "shared.ff"))
                if tensors is not None:
                    absent += [n for n in (f"l{i}.mlp.router.b", f"l{i}.mlp.shared.sg") if n not in tensors]
            else:
                raise ConfigError(f"layer {i}: feed-forward kind {mlp.get('kind')!r} is neither 'dense' nor 'moe'")
        return cls(c, absent, unread)

    def to_dict(self) -> dict:
        return copy.deepcopy(self.cfg)

    def derived(self) -> dict:
        first = next((i for i, layer in enumerate(self.cfg["layers"]) if layer["mixer"].get("v_mix")), None)
        return {"value_mix_source": first, "max_positions": MAX_POSITIONS}

    # ------------------------------------------------------------------ the model it describes
    def _mixer(self, i: int, m: Mapping[str, Any], publishes: Optional[bool]) -> MixerSpec:
        p = f"l{i}.mix."
        params = {"heads": int(m["heads"]), "kv_heads": int(m["kv_heads"]), "head_dim": int(m["dim"]), "v_head_dim": int(m["vdim"]),
                  "scale": float(m["scale"]), "bias": (p + "q.b") not in self.absent, "sink": (p + "sink") not in self.absent,
                  "value_mix": None if publishes is None else {"key": VALUE_MIX_KEY, "publish": publishes}}
        names = {"q_proj": p + "q", "k_proj": p + "k", "v_proj": p + "v", "out_proj": p + "o", "q_bias": p + "q.b", "k_bias": p + "k.b",
                 "v_bias": p + "v.b", "sink": p + "sink", "value_mix": p + "vmix"}
        position = None
        rot = m.get("rot")
        if rot is not None and int(rot["dims"]) > 0:
            position = PositionSpec("rope", {"theta": float(rot["base"]), "rotary_dim": int(rot["dims"]), "variant": "half_split",
                                             "precision": "f64", "scaling_factor": float((rot.get("scaling") or {}).get("factor", 1.0))})
        return MixerSpec("attention", params, names, position=position)

    def _feed_forward(self, i: int, mlp: Mapping[str, Any]) -> FeedForwardSpec:
        p = f"l{i}.mlp."
        if mlp["kind"] == "dense":
            return FeedForwardSpec("glu", {"inter": int(mlp["ff"]), "activation": DENSE_ACTIVATION},
                                   {"gate": p + "gate", "up": p + "up", "down": p + "down"})
        n = int(mlp["router"]["experts"])
        shared = mlp.get("shared")
        params = {"experts": n, "top": int(mlp["router"]["top"]), "inter": int(mlp["expert"]["ff"]), "activation": EXPERT_ACTIVATION,
                  "shared": None if shared is None else {"inter": int(shared["ff"]), "activation": EXPERT_ACTIVATION,
                                                         "gate": (p + "shared.sg") not in self.absent}}
        names = {"router": p + "router", "gate": tuple(f"{p}e{e}.gate" for e in range(n)), "up": tuple(f"{p}e{e}.up" for e in range(n)),
                 "down": tuple(f"{p}e{e}.down" for e in range(n)), "shared_gate": p + "shared.gate", "shared_up": p + "shared.up",
                 "shared_down": p + "shared.down", "shared_weight": p + "shared.sg"}
        if (p + "router.b") not in self.absent:
            names["router_bias"] = p + "router.b"
        return FeedForwardSpec("moe", params, names)

    def model_spec(self) -> ModelSpec:
        c = self.cfg
        width, eps = int(c["width"]), float(c["norm"]["eps"])
        mult = float(c.get("residual_mult", 1.0))
        layers, seen_mix = [], False
        for i, layer in enumerate(c["layers"]):
            name, m = f"l{i}", layer["mixer"]
            publishes = None
            if m.get("v_mix"):
                publishes, seen_mix = not seen_mix, True
            parts = [("norm1", NormSpec("rms", eps, f"{name}.norm1")), ("mixer", self._mixer(i, m, publishes)),
                     ("norm1b", NormSpec("rms", eps, f"{name}.norm1b"))]
            if layer.get("mlp") is not None:
                parts += [("norm2", NormSpec("rms", eps, f"{name}.norm2")), ("ffn", self._feed_forward(i, layer["mlp"])),
                          ("norm2b", NormSpec("rms", eps, f"{name}.norm2b"))]
            layers.append(LayerSpec(name, "sandwich", parts=parts, params={"residual_mult": mult}))
        return ModelSpec(
            architecture=self.architecture, hidden=width, vocab=int(c["vocab"]), layers=tuple(layers), order=tuple(range(len(layers))),
            embedding="embed", final_norm=NormSpec("rms", eps, "final.norm"), head=None, max_position=MAX_POSITIONS,
            unread_tensors=self.unread)
