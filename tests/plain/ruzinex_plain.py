"""Plain Ruzinex forward pass: whole sequences, no cache, one function per mechanism.

Written from the design's equations in float64 (rotation angles in float32, as the design computes them).
Nothing from the product package is imported; the engine is held against this in both of its precisions.

Notation: T tokens, W model width; a linear weight is stored [out, in] and applied as h @ W.T.  A layer is two
sandwiched sublayers, x += m norm_after(sublayer(norm_before(x))), the second of which may be missing.
"""
from __future__ import annotations

import math

import numpy as np

F64 = np.float64


# --------------------------------------------------------------------------- small functions
def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def silu(z):
    return z * sigmoid(z)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + np.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def rms_norm(x, gain, eps):
    """x / sqrt(mean(x^2) + eps) * gain over the last axis."""
    return x / np.sqrt((x * x).mean(-1, keepdims=True) + eps) * gain


# --------------------------------------------------------------------------- rotation
def rotate(x, positions, base: float, dims: int, factor: float = 1.0) -> np.ndarray:
    """Turns the pairs (i, i + dims/2) of the first `dims` entries of the last axis of x [T, heads, n] by the angle
    float32(p) * float32(base^(-2i/dims) / factor); the other entries pass."""
    half = dims // 2
    i = np.arange(half, dtype=F64)
    freq = (float(base) ** (-2.0 * i / dims) / float(factor)).astype(np.float32)
    ang = (np.asarray(positions, dtype=np.float32)[:, None] * freq[None, :]).astype(np.float32).astype(F64)
    cos, sin = np.cos(ang)[:, None, :], np.sin(ang)[:, None, :]
    out = x.astype(F64).copy()
    u, v = x[..., :half], x[..., half:dims]
    out[..., :half] = u * cos - v * sin
    out[..., half:dims] = v * cos + u * sin
    return out


# --------------------------------------------------------------------------- attention
def sink_softmax_attention(q, k, v, scale: float, sink=None) -> np.ndarray:
    """Causal attention of q [T, H, D] over k [T, G, D], v [T, G, V]; query head h reads kv head h // (H / G).  With
    `sink` [H] the softmax's denominator also holds exp(sink[h]): a term without key or value that is not scaled."""
    T, H, _ = q.shape
    G = k.shape[1]
    out = np.zeros((T, H, v.shape[2]), dtype=F64)
    for h in range(H):
        g = h // (H // G)
        s = (q[:, h] @ k[:, g].T) * scale
        s = np.where(np.tril(np.ones((T, T), dtype=bool)), s, -np.inf)
        m = s.max(-1, keepdims=True)
        if sink is not None:
            m = np.maximum(m, sink[h])
        e = np.exp(s - m)
        den = e.sum(-1, keepdims=True)
        if sink is not None:
            den = den + np.exp(sink[h] - m)
        out[:, h] = (e / den) @ v[:, g]
    return out


def attention_mixer(h, w, p: str, m: dict, positions, v_first=None):
    """The attention mixer of the tensors `p`* on the normed rows h [T, W]; returns (delta, the values as cached).
    `v_first`: the values of the first value-mixing layer (None in that layer and without value mixing)."""
    H, G, D, V = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    T = h.shape[0]
    q = (h @ w[p + "q"].T + w[p + "q.b"]).reshape(T, H, D)
    k = (h @ w[p + "k"].T + w[p + "k.b"]).reshape(T, G, D)
    v = (h @ w[p + "v"].T + w[p + "v.b"]).reshape(T, G, V)
    rot = m.get("rot")
    if rot is not None and int(rot.get("dims", 0)) > 0:
        factor = float((rot.get("scaling") or {}).get("factor", 1.0))
        q = rotate(q, positions, float(rot["base"]), int(rot["dims"]), factor)
        k = rotate(k, positions, float(rot["base"]), int(rot["dims"]), factor)
    if v_first is not None:
        lam = float(w[p + "vmix"])
        v = (1.0 - lam) * v + lam * v_first
    o = sink_softmax_attention(q, k, v, float(m["scale"]), w.get(p + "sink"))
    return o.reshape(T, H * V) @ w[p + "o"].T, v


# --------------------------------------------------------------------------- feed-forwards
def gated(h, w, p: str, act):
    """down(act(gate h) * (up h)) of the tensors `p`gate, up, down."""
    return (act(h @ w[p + "gate"].T) * (h @ w[p + "up"].T)) @ w[p + "down"].T


def route(h, router, bias, top: int):
    """(chosen experts [T, top], their weights [T, top]): the `top` largest logits of router h + bias, and the softmax
    over those logits alone."""
    z = h @ router.T + bias
    chosen = np.argsort(-z, axis=-1, kind="stable")[:, :top]
    zc = np.take_along_axis(z, chosen, -1)
    e = np.exp(zc - zc.max(-1, keepdims=True))
    return chosen, e / e.sum(-1, keepdims=True)


def route_margin(h, router, bias, top: int):
    """How clear every row's choice is: the gap between its last chosen logit and the next one, in units of the row's
    spread of logits (infinite when every expert is chosen)."""
    z = np.sort(h @ router.T + bias, axis=-1)[:, ::-1]
    if top >= z.shape[1]:
        return np.full(z.shape[0], np.inf)
    return (z[:, top - 1] - z[:, top]) / (z.std(-1) + 1e-30)


def expert_feed_forward(h, w, p: str, mlp: dict, margins_out=None):
    """Weighted sum of each token's chosen experts, plus the shared expert times sigmoid(sg h) where the layer has one."""
    n, top = int(mlp["router"]["experts"]), int(mlp["router"]["top"])
    chosen, weight = route(h, w[p + "router"], w[p + "router.b"], top)
    if margins_out is not None:
        margins_out.append(route_margin(h, w[p + "router"], w[p + "router.b"], top))
    out = np.zeros((h.shape[0], w[p + "e0.down"].shape[0]), dtype=F64)
    for e in range(n):
        rows, slot = np.nonzero(chosen == e)
        if rows.size:
            out[rows] += weight[rows, slot][:, None] * gated(h[rows], w, f"{p}e{e}.", silu)
    if mlp.get("shared") is not None:
        out = out + sigmoid(h @ w[p + "shared.sg"].T) * gated(h, w, p + "shared.", silu)
    return out


def feed_forward(h, w, p: str, mlp: dict, margins_out=None):
    if mlp["kind"] == "dense":
        return gated(h, w, p, gelu_tanh)
    if mlp["kind"] == "moe":
        return expert_feed_forward(h, w, p, mlp, margins_out)
    raise ValueError(mlp["kind"])


# --------------------------------------------------------------------------- the model
def forward(cfg: dict, w: dict, tokens, layers_out=None, margins_out=None) -> np.ndarray:
    """Logits [T, vocab] of one sequence.  `layers_out`: a list that takes the residual stream after every layer;
    `margins_out`: a list that takes every expert layer's `route_margin` of the tokens."""
    tokens = np.asarray(tokens, dtype=np.int64)
    positions = np.arange(len(tokens))
    eps, mult = float(cfg["norm"]["eps"]), float(cfg.get("residual_mult", 1.0))
    x = w["embed"][tokens].astype(F64)
    v_first = None
    for i, layer in enumerate(cfg["layers"]):
        if layer["type"] != "attention":
            raise ValueError(layer["type"])
        p, m = f"l{i}.", layer["mixer"]
        mixes = bool(m.get("v_mix"))
        d, v = attention_mixer(rms_norm(x, w[p + "norm1"], eps), w, p + "mix.", m, positions, v_first if mixes else None)
        if mixes and v_first is None:
            v_first = v
        x = x + mult * rms_norm(d, w[p + "norm1b"], eps)
        if layer.get("mlp") is not None:
            d = feed_forward(rms_norm(x, w[p + "norm2"], eps), w, p + "mlp.", layer["mlp"], margins_out)
            x = x + mult * rms_norm(d, w[p + "norm2b"], eps)
        if layers_out is not None:
            layers_out.append(x.copy())
    return rms_norm(x, w["final.norm"], eps) @ w["embed"].T
