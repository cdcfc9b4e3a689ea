"""Small Litizen configurations that differ in every size and option, model folders made from them through the
framework's random-weights mode, and the plain implementation's logits for them."""
from __future__ import annotations

import json
import os

import numpy as np

from tests.plain import litizen_plain as Z


def window_attention(heads, kv, dim, scale, size=None, rot=None):
    m = {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": dim, "scale": scale}
    if size is not None:
        m["mask"] = {"size": size}
    if rot is not None:
        m["rot"] = {"base": rot[0], "dims": rot[1]}
    return {"type": "attention", "mixer": m}


def chunk_attention(heads, kv, dim, vdim, scale, base, dims=0, size=None, softcap=None):
    m = {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "scale": scale, "rot": {"base": base, "dims": dims}}
    if size is not None:
        m["mask"] = {"size": size}
    if softcap is not None:
        m["softcap"] = softcap
    return {"type": "attention_2", "mixer": m}


def state_space(heads, vdim, state, groups, conv, norm_groups):
    return {"type": "mamba2", "mixer": {"heads": heads, "vdim": vdim, "state": state, "groups": groups, "conv": conv, "norm_groups": norm_groups}}


def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(experts, identity, top, ff, shared=None):
    m = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "identity": identity, "top": top}}
    if shared is not None:
        m["shared"] = {"ff": shared}
    return m


def with_mlp(layer, mlp):
    return dict(layer, mlp=mlp)


# A: no size a multiple of 8 where it can be avoided (the plain kernels in both precisions); norms in five parts; two taps;
# a window of 7, chunks of 13, a state-space layer whose groups, heads and norm parts all differ; identity experts among
# the chosen; a layer without a feed-forward.
LITIZEN_A = {
    "architecture": "Litizen", "vocab": 211, "width": 100, "norm": {"eps": 1e-5, "groups": 5}, "canon": {"taps": 2},
    "embedding": {"scale": 2.5}, "logit_softcap": 8.0,
    "layers": [
        with_mlp(window_attention(6, 3, 20, 0.25, size=7, rot=(1000.0, 10)), dense(150)),
        with_mlp(state_space(4, 10, 12, 2, 4, 2), moe(5, 2, 3, 30, shared=44)),
        with_mlp(chunk_attention(6, 2, 12, 10, 0.3, 300.0, dims=12, size=13, softcap=5.0), None),
        with_mlp(state_space(6, 6, 7, 3, 2, 3), moe(3, 1, 2, 50)),
    ],
}
# B: aligned sizes, norms in one part (the plain RMS norm's kernels), four taps, keys and values of 64 and 32 (in bfloat16 the
# matrix-core attention kernels), no cap on scores or logits, no scale on the embedding, experts without identity and
# without a shared expert, one expert a token.
LITIZEN_B = {
    "architecture": "Litizen", "vocab": 256, "width": 128, "norm": {"eps": 1e-6, "groups": 1}, "canon": {"taps": 4},
    "layers": [
        with_mlp(chunk_attention(8, 2, 64, 64, 0.125, 10000.0, dims=32, size=64), moe(8, 0, 2, 64)),
        with_mlp(window_attention(8, 8, 32, 0.18, size=48, rot=(10000.0, 32)), dense(256)),
        with_mlp(state_space(4, 32, 64, 1, 2, 1), moe(4, 1, 1, 32, shared=64)),
    ],
}
# C: sizes in steps of 8 that are no multiples of 16, values larger than keys in the chunked layer (stored at one padded
# size in bfloat16), one tap everywhere (no state for the convolutions), a window of one token, chunks of five, every
# router output chosen.
LITIZEN_C = {
    "architecture": "Litizen", "vocab": 97, "width": 72, "norm": {"eps": 1e-5, "groups": 3}, "canon": {"taps": 1},
    "embedding": {"scale": 0.5}, "logit_softcap": 30.0,
    "layers": [
        with_mlp(chunk_attention(4, 4, 24, 40, 0.2, 100.0, dims=8, size=5, softcap=30.0), dense(40)),
        with_mlp(window_attention(3, 1, 40, 0.15, size=1, rot=(100.0, 40)), None),
        with_mlp(state_space(3, 8, 16, 3, 1, 3), moe(3, 3, 6, 16)),
    ],
}
# D: no input convolution, no rotation in the windowed layer and none of q and k in the chunked one, no masks (every
# earlier token is seen), heads of 128, a state of 128.
LITIZEN_D = {
    "architecture": "Litizen", "vocab": 64, "width": 48, "norm": {"eps": 1e-6, "groups": 2},
    "layers": [
        with_mlp(window_attention(2, 1, 128, 0.09), dense(48)),
        with_mlp(chunk_attention(5, 1, 16, 16, 0.25, 1e4), moe(2, 0, 1, 24, shared=8)),
        with_mlp(state_space(2, 64, 128, 1, 3, 4), dense(24)),
    ],
}
MODELS = {"A": LITIZEN_A, "B": LITIZEN_B, "C": LITIZEN_C, "D": LITIZEN_D}


def single_layer(layer, mlp=None, width=100, groups=5, taps=3) -> dict:
    """A model of one layer with the mixer of `layer` and the feed-forward `mlp`."""
    return {"architecture": "Litizen", "vocab": 131, "width": width, "norm": {"eps": 1e-5, "groups": groups}, "canon": {"taps": taps},
            "embedding": {"scale": 1.5}, "logit_softcap": 12.0, "layers": [with_mlp(layer, mlp)]}


def make_model_dir(folder: str, cfg: dict, name: str, seed: int = 0, std: float = 0.1, bias_std: float = 0.5, gain_std: float = 0.3) -> str:
    """Writes a model of configuration `cfg` through the framework's random-weights mode: matrices in bfloat16, so that
    both precisions of the engine and the plain implementation start from the same values; gains, biases, sinks, taps and
    corrections spread widely so that leaving one out shows."""
    from gibbs_amd.config import config_from_dict
    from gibbs_amd.parts import DecoderModel
    from gibbs_amd.weights import write_random_model
    config = config_from_dict(cfg)
    decls = DecoderModel(config.model_spec()).tensor_decls()
    path = os.path.join(folder, f"litizen_{name}_{seed}")
    write_random_model(path, config, decls, seed=seed, dtype="bfloat16", std=std, gain_std=gain_std, bias_std=bias_std)
    return path


def settle_choices(model_dir: str, folder: str) -> str:
    """A copy of a model folder whose routers always choose clearly: the corrections of a layer's outputs lie 0.3 apart (in a
    shuffled order), and the router's matrix is a twentieth of what it was, so that the scores stay near one over the number
    of outputs and every token of a layer takes the same experts, with weights that still differ from token to token.
    Another precision cannot choose differently on such a model, so all of its rows can be held to a bound."""
    import shutil
    from safetensors.torch import load_file, save_file
    path = os.path.join(folder, os.path.basename(model_dir) + "_settled")
    os.makedirs(path, exist_ok=True)
    shutil.copy(os.path.join(model_dir, "config.json"), os.path.join(path, "config.json"))
    w = load_file(os.path.join(model_dir, "model.safetensors"))
    rng = np.random.default_rng(11)
    for name in sorted(w):
        if name.endswith(".mlp.correction"):
            n = w[name].numel()
            w[name] = w[name].new_tensor(rng.permutation(n) * 0.3)
            w[name[:-len("correction")] + "router"] = w[name[:-len("correction")] + "router"] * 0.05
    save_file(w, os.path.join(path, "model.safetensors"))
    return path


def tokens(seed: int, n: int, vocab: int) -> list:
    return np.random.default_rng(seed).integers(0, vocab, size=n).tolist()


def load_model_dir(model_dir: str):
    """(config, name -> float64 array) of a model folder, read with the safetensors package."""
    from safetensors.torch import load_file
    with open(os.path.join(model_dir, "config.json")) as f:
        cfg = json.load(f)
    w = {k: v.double().numpy() for k, v in load_file(os.path.join(model_dir, "model.safetensors")).items()}
    return cfg, w


def clear_tokens(model_dir: str, seed: int, n: int, vocab: int, clear: float, tries: int = 6) -> list:
    """Of a few random sequences, the one whose first unclear choice of experts (`plain_margins` below `clear`) comes latest:
    what follows such a token in a sequence may depend on a choice that another precision makes differently."""
    best, best_at = None, -1
    for k in range(tries):
        ids = tokens(seed * 1000 + k, n, vocab)
        unclear = np.nonzero(plain_margins(model_dir, ids) < clear)[0]
        at = int(unclear[0]) if unclear.size else n
        if at > best_at:
            best, best_at = ids, at
        if at == n:
            break
    return best


_models: dict = {}
_logits: dict = {}
_margins: dict = {}


def plain_logits(model_dir: str, ids) -> np.ndarray:
    key = (model_dir, tuple(ids))
    if key not in _logits:
        if model_dir not in _models:
            _models[model_dir] = load_model_dir(model_dir)
        cfg, w = _models[model_dir]
        margins = []
        _logits[key] = Z.forward(cfg, w, list(ids), margins_out=margins)
        _margins[key] = np.min(margins, axis=0) if margins else np.full(len(ids), np.inf)
    return _logits[key]


def plain_margins(model_dir: str, ids) -> np.ndarray:
    """Per token, how clear the least clear choice of experts among the model's layers is (`Z.route_margin`)."""
    plain_logits(model_dir, ids)
    return _margins[(model_dir, tuple(ids))]
