"""Typed configuration of Litizen: a decoder whose layers mix tokens by windowed attention, chunked attention or a
state-space recurrence, in any order, every sublayer normed on both sides.

  embedding   the table's row times `embedding.scale`
  layer       x += norm1b(mixer(h + conv(h))) with h = norm1(x) and conv a causal convolution over time per channel
              (`canon.taps` taps, tensor `canon1`, its last taps - 1 inputs part of a request's state);
              x += norm2b(ff(norm2(x))) (`mlp: null`: no feed-forward).  Every norm of the model's width is an RMS norm in
              `norm.groups` equal consecutive parts, each divided by its own root mean square
  attention   grouped heads; the values are the keys as projected; q and k normed per head with a gain before the rotation of
              their first `rot.dims` channels (pairs (i, i + dims/2)); scores times `scale` over the last `mask.size`
              positions; one added to the softmax's denominator; the heads' outputs times sigmoid(W_g h)
  attention_2 values of their own, turned by their position over all channels (frequencies `rot.base`^(-2m/vdim)) and
              cached so, every head's output turned back by the query's position; scores capped by `softcap`; a row sees
              the keys of its own stretch of `mask.size` positions counted from 0; a learned sink per head; the same gate
  mamba2      state-space mixer: `heads` x `vdim` channels, `groups` of B and C of size `state`, a convolution of `conv`
              taps with bias and silu over x, B, C, the gated read-out normed in `norm_groups` parts
  feed-forward  dense, down(silu(gate h) * (up h)); or experts: scores by a softmax over all router outputs, the `top`
              largest of score + correction, weights the chosen scores over their sum; the router's last `identity` outputs
              are experts that return their input; a shared expert of the same form is added for every token
  output      the model's norm, the head, then logits <- `logit_softcap` * tanh(logits / `logit_softcap`)

config.json gives every size and constant; what the design fixes (the activations, the pairing of the rotation, the
constant under the weights' sum, that the attention's sink is zero) is written here or in the parts.  Optional tensors (the
convolution in front of a mixer, a correction of the router's scores, a sink, the q/k gains, the gate, an untied head)
are decided by what the checkpoint holds.
"""
from __future__ import annotations

import copy
from typing import Any, Dict, Mapping, Optional, Sequence, Tuple

from .base import ArchConfig, ConfigError, require
from .spec import FeedForwardSpec, LayerSpec, MixerSpec, ModelSpec, NormSpec, PositionSpec

MAX_POSITIONS = 1 << 20
ACTIVATION = "silu"
MIXER_TYPES = ("attention", "attention_2", "mamba2")


class LitizenConfig(ArchConfig):
    architecture = "Litizen"

    def __init__(self, cfg: Dict[str, Any], absent: Sequence[str] = (), unread: Sequence[Tuple[str, Tuple[int, ...]]] = ()):
        self.cfg = cfg
        self.absent = frozenset(absent)     # optional tensors that the checkpoint does not hold
        self.unread = tuple(unread)         # (name, shape) of checkpoint tensors of parts that a layer does not have

    def __eq__(self, other) -> bool:
        return isinstance(other, LitizenConfig) and self.cfg == other.cfg

    # ------------------------------------------------------------------ reading
    @classmethod
    def from_dict(cls, cfg: Mapping[str, Any], tensors: Optional[Mapping[str, Sequence[int]]] = None) -> "LitizenConfig":
        c = copy.deepcopy(dict(cfg))
        width, vocab = int(require(c, "width")), int(require(c, "vocab"))
        if tensors is not None and "embed" in tensors and tuple(int(s) for s in tensors["embed"]) != (vocab, width):
            raise ConfigError(f"config.json says embed is {[vocab, width]}, the checkpoint holds {list(tensors['embed'])}")
        float(require(c, "norm.eps"))
        groups = int((c.get("norm") or {}).get("groups", 1))
        if groups < 1 or width % groups:
            raise ConfigError(f"norm.groups: a width of {width} in {groups} equal parts")
        taps = (c.get("canon") or {}).get("taps")
        if taps is not None and int(taps) < 1:
            raise ConfigError(f"canon.taps: {taps}")
        if float(c.get("logit_softcap") or 0.0) < 0:
            raise ConfigError(f"logit_softcap: {c['logit_softcap']}")
        layers = require(c, "layers")
        if not isinstance(layers, list) or not layers:
            raise ConfigError("config.json: layers must be a non-empty list")
        optional, unread = ["head"], []
        for i, layer in enumerate(layers):
            kind, m = layer.get("type"), layer.get("mixer")
            if kind not in MIXER_TYPES:
                raise ConfigError(f"layer {i}: mixer type {kind!r} is none of {list(MIXER_TYPES)}")
            if not isinstance(m, dict):
                raise ConfigError(f"layer {i}: no mixer sizes")
            p = f"l{i}."
            optional.append(p + "canon1")
            if kind == "mamba2":
                for key in ("heads", "vdim", "state", "groups", "conv"):
                    if int(require(m, key)) < 1:
                        raise ConfigError(f"layer {i}: {key} = {m[key]}")
                if int(m["heads"]) % int(m["groups"]):
                    raise ConfigError(f"layer {i}: {m['heads']} heads are not a multiple of {m['groups']} groups")
                if (int(m["heads"]) * int(m["vdim"])) % int(m.get("norm_groups", 1)):
                    raise ConfigError(f"layer {i}: {int(m['heads']) * int(m['vdim'])} channels in {m['norm_groups']} equal parts")
            else:
                for key in ("heads", "kv_heads", "dim", "vdim", "scale"):
                    require(m, key)
                if int(m["heads"]) % int(m["kv_heads"]):
                    raise ConfigError(f"layer {i}: {m['heads']} heads are not a multiple of {m['kv_heads']} kv heads")
                rot = m.get("rot")
                dims = int((rot or {}).get("dims", 0))
                if dims % 2 or not 0 <= dims <= int(m["dim"]):
                    raise ConfigError(f"layer {i}: {dims} rotated dimensions of a head of {m['dim']}")
                if dims or kind == "attention_2":
                    float(require(rot or {}, "base"))
                size = (m.get("mask") or {}).get("size")
                if size is not None and int(size) < 1:
                    raise ConfigError(f"layer {i}: mask.size = {size}")
                if kind == "attention" and int(m["vdim"]) != int(m["dim"]):
                    raise ConfigError(f"layer {i}: the values are the keys, of size {m['dim']}; vdim says {m['vdim']}")
                if kind == "attention_2" and int(m["vdim"]) % 2:
                    raise ConfigError(f"layer {i}: values of size {m['vdim']} cannot be turned in pairs")
                optional += [p + "mix.g"] + ([p + "mix.q.norm", p + "mix.k.norm"] if kind == "attention" else [p + "mix.sink"])
            mlp = layer.get("mlp")
            if mlp is None:
                if tensors is not None:      # (a layer without a feed-forward whose checkpoint holds that sublayer's norms all the same)
                    unread += [(n, tuple(int(s) for s in tensors[n])) for n in (p + "norm2", p + "norm2b") if n in tensors]
                continue
            if mlp.get("kind") == "dense":
                int(require(mlp, "ff"))
            elif mlp.get("kind") == "moe":
                int(require(mlp, "expert.ff"))
                experts, top = int(require(mlp, "router.experts")), int(require(mlp, "router.top"))
                identity = int(mlp["router"].get("identity", 0))
                if experts < 1 or identity < 0 or not 1 <= top <= experts + identity:
                    raise ConfigError(f"layer {i}: {top} of {experts} + {identity} experts a token")
                if mlp.get("shared") is not None:
                    int(require(mlp, "shared.ff"))
                optional.append(p + "mlp.correction")
            else:
                raise ConfigError(f"layer {i}: feed-forward kind {mlp.get('kind')!r} is neither 'dense' nor 'moe'")
        absent = [n for n in optional if tensors is not None and n not in tensors]
        if taps is None:
            absent += [n for n in optional if n.endswith(".canon1") and n not in absent]
        elif tensors is not None and any(n.endswith(".canon1") for n in absent) and not all(f"l{i}.canon1" in absent for i in range(len(layers))):
            raise ConfigError("the checkpoint holds an input convolution for some layers and not for others")
        return cls(c, absent, unread)

    def to_dict(self) -> dict:
        return copy.deepcopy(self.cfg)

    def derived(self) -> dict:
        kinds = [layer["type"] for layer in self.cfg["layers"]]
        return {"max_positions": MAX_POSITIONS, "layers_by_type": {k: kinds.count(k) for k in MIXER_TYPES}}

    # ------------------------------------------------------------------ the model it describes
    def _has(self, name: str) -> bool:
        return name not in self.absent

    def _attention(self, i: int, kind: str, m: Mapping[str, Any], eps: float) -> MixerSpec:
        p = f"l{i}.mix."
        size = (m.get("mask") or {}).get("size")
        params = {"heads": int(m["heads"]), "kv_heads": int(m["kv_heads"]), "head_dim": int(m["dim"]), "v_head_dim": int(m["vdim"]),
                  "scale": float(m["scale"]), "gate": self._has(p + "g")}
        names = {"q_proj": p + "q", "k_proj": p + "k", "out_proj": p + "o", "gate_proj": p + "g"}
        rot = m.get("rot") or {}
        if kind == "attention":
            params.update(values_from_keys=True, sink="zero", window=None if size is None else int(size))
            if self._has(p + "q.norm"):
                params.update(qk_norm="before", qk_norm_eps=eps)
                names.update(q_norm=p + "q.norm", k_norm=p + "k.norm")
        else:
            params.update(sink=self._has(p + "sink"), chunk=0 if size is None else int(size), softcap=float(m.get("softcap") or 0.0),
                          value_rotation={"theta": float(rot["base"])})
            names.update(v_proj=p + "v", sink=p + "sink")
        position = None
        if int(rot.get("dims", 0)) > 0:
            position = PositionSpec("rope", {"theta": float(rot["base"]), "rotary_dim": int(rot["dims"]), "variant": "half_split", "precision": "f64"})
        return MixerSpec("attention", params, names, position=position)

    def _state_space(self, i: int, m: Mapping[str, Any], eps: float) -> MixerSpec:
        p = f"l{i}.mix."
        params = {"heads": int(m["heads"]), "vdim": int(m["vdim"]), "state": int(m["state"]), "groups": int(m["groups"]),
                  "taps": int(m["conv"]), "norm_groups": int(m.get("norm_groups", 1)), "norm_eps": eps}
        names = {"in": p + "in", "conv": p + "conv", "conv_bias": p + "conv.b", "dt_bias": p + "dt_bias", "A_log": p + "A_log", "D": p + "D",
                 "norm": p + "norm", "o": p + "o"}
        return MixerSpec("ssd", params, names)

    def _feed_forward(self, i: int, mlp: Mapping[str, Any]) -> FeedForwardSpec:
        p = f"l{i}.mlp."
        if mlp["kind"] == "dense":
            return FeedForwardSpec("glu", {"inter": int(mlp["ff"]), "activation": ACTIVATION}, {"gate": p + "gate", "up": p + "up", "down": p + "down"})
        n = int(mlp["router"]["experts"])
        shared = mlp.get("shared")
        params = {"experts": n, "top": int(mlp["router"]["top"]), "inter": int(mlp["expert"]["ff"]), "activation": ACTIVATION,
                  "scores": "softmax_all", "identity": int(mlp["router"].get("identity", 0)),
                  "shared": None if shared is None else {"inter": int(shared["ff"]), "activation": ACTIVATION, "gate": False}}
        names = {"router": p + "router", "gate": tuple(f"{p}e{e}.gate" for e in range(n)), "up": tuple(f"{p}e{e}.up" for e in range(n)),
                 "down": tuple(f"{p}e{e}.down" for e in range(n)), "shared_gate": p + "shared.gate", "shared_up": p + "shared.up",
                 "shared_down": p + "shared.down"}
        if self._has(p + "correction"):
            names["correction"] = p + "correction"
        return FeedForwardSpec("moe", params, names)

    def norm(self, name: str) -> NormSpec:
        eps, groups = float(self.cfg["norm"]["eps"]), int(self.cfg["norm"].get("groups", 1))
        return NormSpec("rms", eps, name) if groups == 1 else NormSpec("group_rms", eps, name, groups=groups)

    def model_spec(self) -> ModelSpec:
        c = self.cfg
        eps = float(c["norm"]["eps"])
        taps = (c.get("canon") or {}).get("taps")
        layers = []
        for i, layer in enumerate(c["layers"]):
            name, kind, m = f"l{i}", layer["type"], layer["mixer"]
            mixer = self._state_space(i, m, eps) if kind == "mamba2" else self._attention(i, kind, m, eps)
            parts = [("norm1", self.norm(f"{name}.norm1"))]
            if taps is not None and self._has(f"{name}.canon1"):
                parts.append(("mixer_input", MixerSpec("conv_input", {"taps": int(taps)}, {"taps": f"{name}.canon1"})))
            parts += [("mixer", mixer), ("norm1b", self.norm(f"{name}.norm1b"))]
            if layer.get("mlp") is not None:
                parts += [("norm2", self.norm(f"{name}.norm2")), ("ffn", self._feed_forward(i, layer["mlp"])), ("norm2b", self.norm(f"{name}.norm2b"))]
            layers.append(LayerSpec(name, "sandwich", parts=parts))
        return ModelSpec(
            architecture=self.architecture, hidden=int(c["width"]), vocab=int(c["vocab"]), layers=tuple(layers), order=tuple(range(len(layers))),
            embedding="embed", final_norm=self.norm("final.norm"), head="head" if self._has("head") else None, max_position=MAX_POSITIONS,
            embedding_scale=float((c.get("embedding") or {}).get("scale", 1.0)), logit_softcap=float(c.get("logit_softcap") or 0.0),
            unread_tensors=self.unread)
