"""Grouped-query attention mixer over the paged cache.

In the reference's order (arch/lib/transformer.json5:46-87): q, k, v
projections; optional RMSNorm of every head of q and k with one [head_dim] gain (`qk_norm:
"before"` the rotation, as LFM2 has it, arch/families/lfm2.json5:80-83);
position encoding of q and k; k, v written to the cache at their positions; causal attention of
each row over the keys up to its own position (within `window`, if given), query head h reading
kv head h // (heads / kv_heads) with scale `scale`; output projection.  A mixer whose params
name `kv_source` projects no k, v and reads that layer's pages (the reference's `write: false`).

The position encoding is asked how it works (`PositionEncoding`): a rotation goes to the kernels
as tables and every fast path stays open; an encoding that changes q and k itself (`apply`) is
called back between the q/k norm and the cache write, and one that biases the scores by distance
(`score_slopes`) takes the plain attention kernel, which knows such a bias.  Which kernels a step
takes is decided where the step runs (csrc/step_plan.hip).

Further options, each a parameter of the spec: `bias` (q, k and v projections have biases: tensors `q_bias`,
`k_bias`, `v_bias`), `sink` (a learned number per head, tensor `sink`, whose exponential joins the softmax's
denominator without key or value and without the score's scale), `v_head_dim` (values of a head size of their
own), and `value_mix` = {"key": k, "publish": bool}: the layer that publishes hands its values of the step's rows
to the later layers of the same key, which cache and use  v <- (1 - lambda) v + lambda v_published  with their
own lambda (tensor `value_mix`, one number; the publishing layer declares it too and never reads it).

With those options (they share the preparation of the step's rows) go further ones: `qk_norm: "before"` (tensors `q_norm`,
`k_norm` [head_dim], eps `qk_norm_eps`); `values_from_keys` (no value projection: a position's value is its key as
projected, before norm and rotation); `value_rotation: {"theta": base}` (values are turned by their position over all of
their channels, pair m by p * base^(-2m / v_head_dim) in the rotation's pairing, cached so, and every head's output is
turned back by the query's position); `chunk: n` (a row sees the keys of its own stretch of n positions, counted from
position 0, instead of a window); `softcap: c` (scores become c tanh(s / c) after the scale); `sink: "zero"` (a sink whose
number is 0 and not learned: one added to the softmax's denominator); `gate` (tensor `gate_proj` [heads * v_head_dim,
hidden]: the heads' outputs times sigmoid(W_g h), h the rows that the projections read, before the out-projection).
"""
from __future__ import annotations

from typing import List, Optional

import torch

from .. import ops
from ..cache.needs import CacheNeed
from ..weights.loader import FLOAT32, TensorDecl, WeightStore
from .base import Mixer, Runtime, build_position, register_mixer


@register_mixer("attention")
class AttentionMixer(Mixer):
    def __init__(self, spec, hidden, layer_index):
        super().__init__(spec, hidden, layer_index)
        p = spec.params
        self.heads, self.kv_heads, self.head_dim = int(p["heads"]), int(p["kv_heads"]), int(p["head_dim"])
        self.scale = float(p["scale"])
        self.window = p.get("window")
        self.qk_norm = p.get("qk_norm")
        self.qk_norm_eps = float(p.get("qk_norm_eps", 0.0))
        self.source = p.get("kv_source")
        # values of a head size of their own; q and k divided by their root mean square without a gain
        # (`qk_norm: "unit"`); q times 1 + coef * log(1 + (position + 1) div every) (`q_temperature`)
        self.v_head_dim = int(p.get("v_head_dim") or self.head_dim)
        self.q_temperature = p.get("q_temperature")
        self.has_bias, self.has_sink = bool(p.get("bias")), bool(p.get("sink"))
        self.zero_sink = p.get("sink") == "zero"
        self.value_mix = p.get("value_mix")
        self.values_from_keys = bool(p.get("values_from_keys"))
        self.value_rotation = p.get("value_rotation")
        self.chunk = int(p.get("chunk") or 0)
        self.softcap = float(p.get("softcap") or 0.0)
        self.gated = bool(p.get("gate"))
        self.gated_options = bool(self.values_from_keys or self.value_rotation or self.chunk or self.softcap or self.gated or self.zero_sink)
        if self.gated_options and (self.source is not None or self.q_temperature is not None or self.qk_norm == "unit"):
            raise ValueError("values from keys, turned values, chunks, capped scores and a gate go with a mixer that owns its pages and has no unit norm or temperature")
        if self.chunk and self.window is not None:
            raise ValueError("an attention sees a window or chunks, not both")
        if self.values_from_keys and (self.v_head_dim > self.head_dim or self.value_mix is not None or self.value_rotation):
            raise ValueError("values that are the keys are no larger than they, and neither mixed nor turned")
        if self.value_rotation and (self.v_head_dim % 2 or self.value_mix is not None):
            raise ValueError("turned values have an even size and are not mixed")
        if self.value_mix is not None and (self.source is not None or int(self.value_mix["key"]) < 0):
            raise ValueError("value mixing needs a key >= 0 and a mixer that owns its pages")
        if (self.has_bias or self.has_sink or self.value_mix is not None) and (self.qk_norm == "unit" or self.q_temperature is not None
                                                                              or self.source is not None):
            raise ValueError("projection biases, a sink and value mixing go with neither a unit norm nor a temperature nor another layer's cache")
        if self.heads % self.kv_heads:
            raise ValueError(f"{self.heads} heads are not a multiple of {self.kv_heads} kv heads")
        if self.qk_norm not in (None, "before", "unit"):
            raise ValueError(f"qk_norm {self.qk_norm!r} is not implemented (None, 'before' or 'unit')")
        if self.window is not None and int(self.window) <= 0:
            raise ValueError(f"attention window {self.window} must be positive")
        self.position = build_position(spec.position, self.head_dim)
        if hasattr(self.position, "for_heads"):          # (an encoding with a column per head)
            self.position.for_heads(self.heads)

    # ------------------------------------------------------------------ what it asks for
    def cache_need(self) -> Optional[CacheNeed]:
        if self.source is not None:
            return None
        hd, vd = self.stored_dims()
        return CacheNeed(self.kv_heads, hd, None if self.window is None else int(self.window), None if vd == hd else vd)

    def stored_dims(self):
        """(key, value) head sizes as projected and cached: the mixer's own, or, once it is bound for a bfloat16 run with
        keys and values of different sizes (or sizes that are no multiple of 16), one common size with zeros behind each
        head's channels, which the matrix-core attention kernels take."""
        pad = getattr(self, "padded_dim", None)
        return (pad, pad) if pad else (self.head_dim, self.v_head_dim)

    def _pad_heads(self, w: torch.Tensor, heads: int, dim: int, pad: int, rows: bool) -> torch.Tensor:
        """[heads * dim, in] -> [heads * pad, in] (rows) or [out, heads * dim] -> [out, heads * pad], zeros behind each head."""
        if rows:
            out = torch.zeros((heads, pad, w.shape[1]), dtype=w.dtype, device=w.device)
            out[:, :dim] = w.view(heads, dim, w.shape[1])
            return out.view(heads * pad, w.shape[1])
        out = torch.zeros((w.shape[0], heads, pad), dtype=w.dtype, device=w.device)
        out[:, :, :dim] = w.view(w.shape[0], heads, dim)
        return out.view(w.shape[0], heads * pad)

    def attention_flops(self, keys: float) -> float:
        """Multiply-adds x 2 of scores and weighted values when the step's rows see `keys` keys in all."""
        return 2.0 * keys * self.heads * (self.head_dim + self.v_head_dim)

    def kv_source(self) -> Optional[int]:
        return self.source

    def tensor_decls(self) -> List[TensorDecl]:
        t, H, hd, vd = self.spec.tensors, self.hidden, self.head_dim, self.v_head_dim
        decls = [TensorDecl(t["q_proj"], (self.heads * hd, H))]
        if self.source is None:
            decls.append(TensorDecl(t["k_proj"], (self.kv_heads * hd, H)))
            if not self.values_from_keys:
                decls.append(TensorDecl(t["v_proj"], (self.kv_heads * vd, H)))
        if self.gated:
            decls.append(TensorDecl(t["gate_proj"], (self.heads * vd, H)))
        decls.append(TensorDecl(t["out_proj"], (H, self.heads * vd)))
        if self.qk_norm == "before":
            decls.append(TensorDecl(t["q_norm"], (hd,), FLOAT32, init="gain"))
            if self.source is None:
                decls.append(TensorDecl(t["k_norm"], (hd,), FLOAT32, init="gain"))
        if self.has_bias:
            decls += [TensorDecl(t["q_bias"], (self.heads * hd,), FLOAT32, init="bias"),
                      TensorDecl(t["k_bias"], (self.kv_heads * hd,), FLOAT32, init="bias"),
                      TensorDecl(t["v_bias"], (self.kv_heads * vd,), FLOAT32, init="bias")]
        if self.has_sink and not self.zero_sink:
            decls.append(TensorDecl(t["sink"], (self.heads,), FLOAT32, init="bias"))
        if self.value_mix is not None:
            decls.append(TensorDecl(t["value_mix"], (), FLOAT32, init="bias"))
        if self.position is not None:
            decls += self.position.tensor_decls()
        return decls

    def projection_options(self) -> bool:
        """Options that take the preparation of the step's rows with biases, partial rotation and value mixing."""
        rotated_own_values = (self.v_head_dim != self.head_dim and self.qk_norm is None and self.q_temperature is None
                              and self.spec.position is not None and self.spec.position.kind == "rope")
        return self.has_bias or self.has_sink or self.value_mix is not None or rotated_own_values or self.gated_options

    def bind(self, weights: WeightStore, rt: Runtime) -> None:
        self.rt = rt
        t = self.spec.tensors
        wq, w_out = weights[t["q_proj"]], weights[t["out_proj"]]
        # A bfloat16 run of an attention that takes the general preparation of its rows anyway (a unit norm, a score table)
        # stores every head of q, k and v at one size that the matrix-core kernels take: a multiple of 16 that holds the
        # larger of the two, zeros behind each head's channels (rows of zeros in the projections, columns of zeros in the
        # out-projection: products with them are exactly zero).
        self.padded_dim = None
        pad = -(-max(self.head_dim, self.v_head_dim) // 16) * 16
        if (rt.act_dtype == torch.bfloat16 and self.source is None and (self.qk_norm == "unit" or self.projection_options())
                and pad <= 128 and (self.head_dim, self.v_head_dim) != (pad, pad)):
            self.padded_dim = pad
            wq = self._pad_heads(wq, self.heads, self.head_dim, pad, rows=True)
            w_out = self._pad_heads(w_out, self.heads, self.v_head_dim, pad, rows=False)
        if self.source is None:
            # one product for q, k and v: rows [Wq; Wk; Wv]
            wk = weights[t["k_proj"]]
            wv = None if self.values_from_keys else weights[t["v_proj"]]
            wg = weights[t["gate_proj"]] if self.gated else None
            if self.padded_dim:
                wk = self._pad_heads(wk, self.kv_heads, self.head_dim, pad, rows=True)
                wv = None if wv is None else self._pad_heads(wv, self.kv_heads, self.v_head_dim, pad, rows=True)
                wg = None if wg is None else self._pad_heads(wg, self.heads, self.v_head_dim, pad, rows=True)
            # (rows [q | k | v, unless the values are the keys | gate])
            self.w_qkv = torch.cat([w for w in (wq, wk, wv, wg) if w is not None], dim=0).contiguous()
        else:
            self.w_qkv = wq
        self.w_out = w_out.contiguous()
        self.p_qkv = self.p_out = None
        # biases in the layout of a projected row (heads as they are stored), the sink and the mixing weight
        self.proj_bias = self.sinks = self.mix_weight = None
        if self.has_bias:
            def stored(b, heads, dim, size):
                out = torch.zeros((heads, size), dtype=torch.float32, device=b.device)
                out[:, :dim] = b.view(heads, dim)
                return out.view(-1)
            hd_s, vd_s = self.stored_dims()
            self.proj_bias = torch.cat([stored(weights[t["q_bias"]], self.heads, self.head_dim, hd_s),
                                        stored(weights[t["k_bias"]], self.kv_heads, self.head_dim, hd_s),
                                        stored(weights[t["v_bias"]], self.kv_heads, self.v_head_dim, vd_s)]).contiguous()
        if self.zero_sink:
            self.sinks = torch.zeros(self.heads, dtype=torch.float32, device=rt.device)
        elif self.has_sink:
            self.sinks = weights[t["sink"]].contiguous()
        self.v_inv_freq = None
        if self.value_rotation:
            from .rope import rope_inv_freq
            self.v_inv_freq = torch.from_numpy(rope_inv_freq(self.v_head_dim, float(self.value_rotation["theta"]))).to(rt.device)
        if self.value_mix is not None and not self.value_mix.get("publish"):
            self.mix_weight = weights[t["value_mix"]].reshape(1).contiguous()
        self.q_gain = weights[t["q_norm"]] if self.qk_norm == "before" else None
        self.k_gain = weights[t["k_norm"]] if self.qk_norm == "before" and self.source is None else None
        self.rot, self.slopes, self.pos_hook, self.score_bias = None, None, False, None
        if self.position is not None:
            self.position.bind(weights, rt)
            self.rot = self.position.rotation()
            self.slopes = self.position.score_slopes(self.heads)
            self.score_bias = self.position.score_table(self.heads)
            self.pos_hook = self.rot is None and self.position.transforms_rows()
        # (the matrix-core kernels add the bias to unscaled scores, head by head)
        self.score_bias_over_scale = None
        if self.score_bias is not None and rt.act_dtype == torch.bfloat16 and self.scale > 0:
            self.score_bias_over_scale = (self.score_bias.t() / self.scale).contiguous()
        if self.slopes is not None and (self.slopes.dtype != torch.float32 or tuple(self.slopes.shape) != (self.heads,)):
            raise ValueError(f"score slopes must be float32 [{self.heads}]")

    def matrices(self):
        return [self.w_qkv, self.w_out]

    def product_shapes(self):
        kv = self.kv_heads * (self.head_dim + (0 if self.values_from_keys else self.v_head_dim)) if self.source is None else 0
        gate = self.heads * self.v_head_dim if self.gated else 0
        return [(self.heads * self.head_dim + kv + gate, self.hidden), (self.hidden, self.heads * self.v_head_dim)]

    def small_tensors(self):
        own = [t for t in (self.q_gain, self.k_gain, self.slopes, self.proj_bias, self.sinks, self.mix_weight, self.v_inv_freq) if t is not None]   # (a score table is the position's)
        return own + ([] if self.position is None else list(self.position.small_tensors()))

    def fold_input_gain(self, gain: torch.Tensor) -> None:
        """The preceding norm's gain, multiplied into the columns of the q, k, v projections."""
        self.w_qkv = (self.w_qkv.float() * gain[None, :]).to(self.w_qkv.dtype)

    def pack_matrices(self) -> None:
        self.p_qkv = ops.PackedWeight(self.w_qkv)
        self.p_out = ops.PackedWeight(self.w_out)

    def extras(self) -> bool:
        """Options that take the general preparation of the step's rows (no rotation, no gains)."""
        return not self.projection_options() and (self.v_head_dim != self.head_dim or self.qk_norm == "unit"
                                                  or self.q_temperature is not None or self.score_bias is not None)

    def emit(self, plan, cache) -> int:
        hd, vd = self.stored_dims()
        if cache.kpages is None or cache.vpages.shape[-1] != vd or cache.kpages.shape[-1] != hd:
            raise ValueError("the attention mixer's pages do not have its head sizes")
        hook = self.position.apply if self.pos_hook else None
        body = self._emit_body(plan, cache, hook, hd)
        if self.extras():
            temp = self.q_temperature or {"coef": 0.0, "every": 0}
            plan.attention_extras(body, v_head_dim=vd, unit_qk=self.qk_norm == "unit", temp_coef=float(temp["coef"]),
                                  temp_every=int(temp["every"]), bias=self.score_bias, bias_over_scale=self.score_bias_over_scale,
                                  norm_dim=self.head_dim)
        if self.projection_options():
            if hook is not None or self.slopes is not None or self.score_bias is not None:
                raise ValueError("projection biases, a sink and value mixing go with a rotation or no position encoding")
            mix = self.value_mix
            plan.attention_projection(body, v_head_dim=vd, bias=self.proj_bias, sink=self.sinks,
                                      keep_mode=0 if mix is None else (1 if mix.get("publish") else 2),
                                      keep_key=-1 if mix is None else int(mix["key"]), value_dim=self.v_head_dim, weight=self.mix_weight)
            if self.gated_options or self.qk_norm == "before":
                plan.attention_gated(body, q_gain=self.q_gain, k_gain=self.k_gain, qk_eps=self.qk_norm_eps, norm_dim=self.head_dim,
                                     values_from_keys=self.values_from_keys, v_inv_freq=self.v_inv_freq, v_rot=self.v_head_dim,
                                     chunk=self.chunk, softcap=self.softcap, gate=self.gated)
        return body

    def _emit_body(self, plan, cache, hook, head_dim: int) -> int:
        # (with the projection options the q/k gains travel with them: the body's own are those of the fast paths)
        prep = self.projection_options()
        return plan.attention(w_qkv=self.w_qkv, p_qkv=self.p_qkv, w_out=self.w_out, p_out=self.p_out, heads=self.heads,
                              kv_heads=self.kv_heads, head_dim=head_dim, scale=self.scale, window=self.window,
                              q_gain=None if prep else self.q_gain, k_gain=None if prep else self.k_gain, qk_eps=self.qk_norm_eps, rotation=self.rot,
                              kpages=cache.kpages, vpages=cache.vpages, group=cache.group, owns=self.source is None,
                              slopes=self.slopes, rows_hook=hook)
