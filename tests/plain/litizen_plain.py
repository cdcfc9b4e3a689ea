"""Plain Litizen forward pass: whole sequences, no cache, one function per mechanism.

Written from the design's equations in float64 (rotation angles in float32, as the design computes them).  Nothing
from the product package is imported; the engine is held against this in both of its precisions.

Notation: T tokens, W model width; a linear weight is stored [out, in] and applied as h @ W.T.  A layer is two
sublayers normed on both sides, x += norm_after(sublayer(norm_before(x))); the second may be missing.  What the mixer
reads passes a short causal convolution over time first, h <- h + conv(h).
"""
from __future__ import annotations

import numpy as np

F64 = np.float64


# --------------------------------------------------------------------------- small functions
def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def silu(z):
    return z * sigmoid(z)


def softplus(z):
    return np.maximum(z, 0.0) + np.log1p(np.exp(-np.abs(z)))


def group_rms_norm(x, gain, eps: float, groups: int) -> np.ndarray:
    """The last axis in `groups` equal consecutive parts, each divided by its own sqrt(mean(part^2) + eps); the whole
    times `gain`."""
    shape = x.shape
    parts = x.reshape(shape[:-1] + (groups, shape[-1] // groups))
    parts = parts / np.sqrt((parts * parts).mean(-1, keepdims=True) + eps)
    return parts.reshape(shape) * gain


def causal_conv(x, taps, bias=None) -> np.ndarray:
    """y[t, c] = sum_j taps[c, j] x[t - (K - 1) + j, c] (+ bias[c]): the last tap is the current token's, zeros before
    the sequence's start.  x [T, C], taps [C, K]."""
    T, C = x.shape
    K = taps.shape[1]
    padded = np.concatenate([np.zeros((K - 1, C), dtype=F64), x.astype(F64)], axis=0)
    y = np.zeros((T, C), dtype=F64)
    for j in range(K):
        y += padded[j:j + T] * taps[:, j][None, :]
    return y if bias is None else y + bias[None, :]


def input_conv(h, taps) -> np.ndarray:
    """What a mixer reads: h + conv(h)."""
    return h + causal_conv(h, taps)


# --------------------------------------------------------------------------- rotation
def angles(positions, base: float, dims: int) -> np.ndarray:
    """float32(p) * float32(base^(-2i/dims)), i = 0 .. dims/2 - 1, as float64 [T, dims/2]."""
    i = np.arange(dims // 2, dtype=F64)
    freq = (float(base) ** (-2.0 * i / dims)).astype(np.float32)
    return (np.asarray(positions, dtype=np.float32)[:, None] * freq[None, :]).astype(np.float32).astype(F64)


def rotate(x, positions, base: float, dims: int, sign: float = 1.0) -> np.ndarray:
    """Turns the pairs (i, i + dims/2) of the first `dims` entries of the last axis of x [T, heads, n] by the angle of
    the row's position times `sign`; the other entries pass."""
    half = dims // 2
    ang = angles(positions, base, dims) * sign
    cos, sin = np.cos(ang)[:, None, :], np.sin(ang)[:, None, :]
    out = x.astype(F64).copy()
    u, v = x[..., :half], x[..., half:dims]
    out[..., :half] = u * cos - v * sin
    out[..., half:dims] = v * cos + u * sin
    return out


# --------------------------------------------------------------------------- attention
def visible_window(T: int, size: int) -> np.ndarray:
    """[i, j]: 0 <= i - j < size."""
    d = np.arange(T)[:, None] - np.arange(T)[None, :]
    return (d >= 0) & (d < size)


def visible_chunk(T: int, size: int) -> np.ndarray:
    """[i, j]: j <= i and both in the same stretch of `size` positions counted from 0."""
    i, j = np.arange(T)[:, None], np.arange(T)[None, :]
    return (j <= i) & (i // size == j // size)


def masked_attention(q, k, v, scale: float, visible, sink=None, softcap=None) -> np.ndarray:
    """Attention of q [T, H, D] over k [T, G, D], v [T, G, V] where `visible` [T, T] says so; query head h reads kv head
    h // (H / G).  Scores are (q . k) scale, then capped as cap tanh(s / cap) if `softcap`.  `sink` [H]: the softmax's
    denominator also holds exp(sink[h]), a term without key or value that is neither scaled nor capped."""
    T, H, _ = q.shape
    G = k.shape[1]
    out = np.zeros((T, H, v.shape[2]), dtype=F64)
    for h in range(H):
        g = h // (H // G)
        s = (q[:, h] @ k[:, g].T) * scale
        if softcap:
            s = softcap * np.tanh(s / softcap)
        s = np.where(visible, s, -np.inf)
        m = s.max(-1, keepdims=True)
        if sink is not None:
            m = np.maximum(m, sink[h])
        e = np.exp(s - m)
        den = e.sum(-1, keepdims=True)
        if sink is not None:
            den = den + np.exp(sink[h] - m)
        out[:, h] = (e / den) @ v[:, g]
    return out


def window_attention_mixer(h, w, p: str, m: dict, positions, eps: float) -> np.ndarray:
    """Mixer 'attention': the values are the keys as projected; q and k normed per head, then turned; a sliding
    window; one added to the softmax's denominator; a sigmoid gate on the heads' outputs."""
    H, G, D, V = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    T = h.shape[0]
    q = (h @ w[p + "q"].T).reshape(T, H, D)
    k = (h @ w[p + "k"].T).reshape(T, G, D)
    v = k.copy()
    if p + "q.norm" in w:
        q = group_rms_norm(q, w[p + "q.norm"], eps, 1)
        k = group_rms_norm(k, w[p + "k.norm"], eps, 1)
    rot = m.get("rot")
    if rot is not None and int(rot.get("dims", 0)) > 0:
        q = rotate(q, positions, float(rot["base"]), int(rot["dims"]))
        k = rotate(k, positions, float(rot["base"]), int(rot["dims"]))
    size = (m.get("mask") or {}).get("size")
    o = masked_attention(q, k, v, float(m["scale"]), visible_window(T, T if size is None else int(size)), sink=np.zeros(H, dtype=F64))
    o = o.reshape(T, H * V) * sigmoid(h @ w[p + "g"].T)
    return o @ w[p + "o"].T


def chunk_attention_mixer(h, w, p: str, m: dict, positions) -> np.ndarray:
    """Mixer 'attention_2': values of their own, turned by their position over all of their channels and the heads'
    outputs turned back by the query's position; capped scores; chunks; a learned sink; a sigmoid gate."""
    H, G, D, V = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    T = h.shape[0]
    q = (h @ w[p + "q"].T).reshape(T, H, D)
    k = (h @ w[p + "k"].T).reshape(T, G, D)
    v = (h @ w[p + "v"].T).reshape(T, G, V)
    rot = m["rot"]
    base = float(rot["base"])
    if int(rot.get("dims", 0)) > 0:
        q = rotate(q, positions, base, int(rot["dims"]))
        k = rotate(k, positions, base, int(rot["dims"]))
    v = rotate(v, positions, base, V)
    size = (m.get("mask") or {}).get("size")
    o = masked_attention(q, k, v, float(m["scale"]), visible_chunk(T, T if size is None else int(size)), sink=w.get(p + "sink"),
                         softcap=m.get("softcap"))
    o = rotate(o, positions, base, V, sign=-1.0)
    o = o.reshape(T, H * V) * sigmoid(h @ w[p + "g"].T)
    return o @ w[p + "o"].T


# --------------------------------------------------------------------------- state-space mixer
def ssd_scan(x, B, C, dt, a_log, D_skip, groups: int) -> np.ndarray:
    """Per head h (group h // (H / groups)), with a state S [N, P] that starts at zero:
    S_t = exp(-exp(a_log_h) dt_t) S_(t-1) + dt_t B_t x_t';  y_t = S_t' C_t + D_h x_t.
    x [T, H, P], B and C [T, groups, N], dt [T, H]."""
    T, H, P = x.shape
    N = B.shape[2]
    y = np.zeros((T, H, P), dtype=F64)
    for h in range(H):
        g = h // (H // groups)
        S = np.zeros((N, P), dtype=F64)
        rate = np.exp(a_log[h])
        for t in range(T):
            S = np.exp(-rate * dt[t, h]) * S + dt[t, h] * np.outer(B[t, g], x[t, h])
            y[t, h] = S.T @ C[t, g] + D_skip[h] * x[t, h]
    return y


def mamba2_mixer(h, w, p: str, m: dict, eps: float) -> np.ndarray:
    H, P, N, G = int(m["heads"]), int(m["vdim"]), int(m["state"]), int(m["groups"])
    inner = H * P
    T = h.shape[0]
    zxbcdt = h @ w[p + "in"].T
    z, xbc, dt = zxbcdt[:, :inner], zxbcdt[:, inner:2 * inner + 2 * G * N], zxbcdt[:, 2 * inner + 2 * G * N:]
    xbc = silu(causal_conv(xbc, w[p + "conv"], w[p + "conv.b"]))
    x = xbc[:, :inner].reshape(T, H, P)
    B = xbc[:, inner:inner + G * N].reshape(T, G, N)
    C = xbc[:, inner + G * N:].reshape(T, G, N)
    dt = softplus(dt + w[p + "dt_bias"][None, :])
    y = ssd_scan(x, B, C, dt, w[p + "A_log"], w[p + "D"], G).reshape(T, inner)
    y = group_rms_norm(y * silu(z), w[p + "norm"], eps, int(m["norm_groups"]))
    return y @ w[p + "o"].T


# --------------------------------------------------------------------------- feed-forwards
def gated_ff(h, gate, up, down) -> np.ndarray:
    return (silu(h @ gate.T) * (h @ up.T)) @ down.T


def route(h, router, correction, top: int):
    """Scores s = softmax(router h) over all experts; the `top` largest of s + correction (the lower index among
    equals); weights: the chosen experts' s divided by their sum (+ 1e-20).  -> (chosen [T, top], weights [T, top])."""
    z = h @ router.T
    z = z - z.max(-1, keepdims=True)
    s = np.exp(z)
    s = s / s.sum(-1, keepdims=True)
    chosen = np.argsort(-(s + correction[None, :]), axis=-1, kind="stable")[:, :top]
    picked = np.take_along_axis(s, chosen, axis=-1)
    return chosen, picked / (picked.sum(-1, keepdims=True) + 1e-20)


def route_margin(h, router, correction, top: int) -> np.ndarray:
    """Per row, how far the last chosen expert's score + correction lies above the best one that was not chosen (inf
    where every expert is chosen): a choice closer than the rounding of h may fall the other way in another precision."""
    z = h @ router.T
    z = z - z.max(-1, keepdims=True)
    s = np.exp(z)
    s = np.sort(s / s.sum(-1, keepdims=True) + correction[None, :], axis=-1)[:, ::-1]
    return s[:, top - 1] - s[:, top] if top < s.shape[1] else np.full(h.shape[0], np.inf)


def moe_ff(h, w, p: str, mlp: dict, margins_out=None) -> np.ndarray:
    """Experts 0 .. E-1 are gated feed-forwards; the last `identity` router outputs are experts that return their input."""
    E, top = int(mlp["router"]["experts"]), int(mlp["router"]["top"])
    correction = w.get(p + "correction", np.zeros(w[p + "router"].shape[0]))
    chosen, weights = route(h, w[p + "router"], correction, top)
    if margins_out is not None:
        margins_out.append(route_margin(h, w[p + "router"], correction, top))
    out = np.zeros_like(h, dtype=F64)
    for t in range(h.shape[0]):
        for e, wt in zip(chosen[t], weights[t]):
            if e >= E:
                out[t] += wt * h[t]
            else:
                q = f"{p}e{e}."
                out[t] += wt * gated_ff(h[t:t + 1], w[q + "gate"], w[q + "up"], w[q + "down"])[0]
    if mlp.get("shared") is not None:
        out += gated_ff(h, w[p + "shared.gate"], w[p + "shared.up"], w[p + "shared.down"])
    return out


def feed_forward(h, w, p: str, mlp: dict, margins_out=None) -> np.ndarray:
    if mlp["kind"] == "dense":
        return gated_ff(h, w[p + "gate"], w[p + "up"], w[p + "down"])
    return moe_ff(h, w, p, mlp, margins_out)


# --------------------------------------------------------------------------- the model
def forward(cfg: dict, weights: dict, tokens, return_layers: bool = False, margins_out=None):
    """Logits [T, vocab] of one sequence (and the residual stream after every layer, [layers, T, W]).  `margins_out`: a list
    that receives every expert layer's `route_margin` per token."""
    w = {k: np.asarray(v, dtype=F64) for k, v in weights.items()}
    eps, groups = float(cfg["norm"]["eps"]), int(cfg["norm"].get("groups", 1))
    T = len(tokens)
    positions = np.arange(T)
    x = w["embed"][np.asarray(tokens)] * float(cfg.get("embedding", {}).get("scale", 1.0))
    norm = lambda v, name: group_rms_norm(v, w[name], eps, groups)
    after = []
    for i, layer in enumerate(cfg["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        h = norm(x, p + "norm1")
        if p + "canon1" in w:
            h = input_conv(h, w[p + "canon1"])
        if layer["type"] == "attention":
            d = window_attention_mixer(h, w, p + "mix.", m, positions, eps)
        elif layer["type"] == "attention_2":
            d = chunk_attention_mixer(h, w, p + "mix.", m, positions)
        elif layer["type"] == "mamba2":
            d = mamba2_mixer(h, w, p + "mix.", m, eps)
        else:
            raise ValueError(layer["type"])
        x = x + norm(d, p + "norm1b")
        if layer.get("mlp") is not None:
            x = x + norm(feed_forward(norm(x, p + "norm2"), w, p + "mlp.", layer["mlp"], margins_out), p + "norm2b")
        after.append(x.copy())
    logits = norm(x, "final.norm") @ w["head" if "head" in w else "embed"].T
    cap = cfg.get("logit_softcap")
    if cap:
        logits = cap * np.tanh(logits / cap)
    return (logits, np.stack(after)) if return_layers else logits
