"""Small Ruzinex configurations that differ in every size and option, model folders made from them through the
framework's random-weights mode, and the plain implementation's logits for them."""
from __future__ import annotations

import json
import os

import numpy as np

from tests.plain import ruzinex_plain as Z


def _mix(heads, kv, dim, vdim, scale, rot=None, v_mix=False):
    m = {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "scale": scale}
    if rot is not None:
        base, dims, factor = rot
        m["rot"] = {"base": base, "dims": dims}
        if factor is not None:
            m["rot"]["scaling"] = {"factor": factor}
    if v_mix:
        m["v_mix"] = True
    return m


def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(experts, top, ff, shared=None):
    m = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}
    if shared is not None:
        m["shared"] = {"ff": shared}
    return m


def _layer(mixer, mlp):
    return {"type": "attention", "mixer": mixer, "mlp": mlp}


# A: no size a multiple of 8 where it can be avoided (the plain kernels in both precisions); values smaller than keys; the
# second layer is the first that mixes values (it publishes), the first layer does not; a layer without a feed-forward;
# three of three experts; sizes of the mixers differ between layers.
RUZINEX_A = {
    "architecture": "Ruzinex", "vocab": 211, "width": 100, "norm": {"eps": 1e-5}, "residual_mult": 1.3,
    "layers": [
        _layer(_mix(6, 3, 20, 12, 0.2, rot=(1000.0, 10, 4.0)), dense(150)),
        _layer(_mix(6, 3, 20, 12, 0.25, rot=(1000.0, 20, None), v_mix=True), moe(5, 2, 30, shared=44)),
        _layer(_mix(3, 3, 14, 12, 0.3, rot=(300.0, 6, 2.0), v_mix=True), None),
        _layer(_mix(9, 3, 12, 12, 0.22, rot=(50000.0, 12, 1.5), v_mix=True), moe(3, 3, 50)),
    ],
}
# B: aligned sizes, keys and values of one size (in bfloat16 the matrix-core attention kernels without padding and the
# matrix-core expert products), full rotation without scaling, every layer mixes values, one expert of eight.
RUZINEX_B = {
    "architecture": "Ruzinex", "vocab": 256, "width": 128, "norm": {"eps": 1e-6}, "residual_mult": 0.5,
    "layers": [
        _layer(_mix(8, 2, 64, 64, 0.125, rot=(10000.0, 64, None), v_mix=True), moe(8, 1, 64, shared=64)),
        _layer(_mix(8, 2, 64, 64, 0.125, rot=(10000.0, 64, None), v_mix=True), dense(256)),
        _layer(_mix(8, 2, 32, 64, 0.18, rot=(10000.0, 16, 8.0), v_mix=True), moe(16, 4, 32)),
    ],
}
# C: values larger than keys (in bfloat16 stored at one padded size), no grouping of heads, no value mixing, no
# multiplier, dense layers only, sizes that are multiples of 8 but not of 16.
RUZINEX_C = {
    "architecture": "Ruzinex", "vocab": 97, "width": 72, "norm": {"eps": 1e-5},
    "layers": [
        _layer(_mix(4, 4, 24, 40, 0.2, rot=(100.0, 8, 2.0)), dense(40)),
        _layer(_mix(3, 1, 40, 24, 0.15, rot=(100.0, 40, 3.0)), dense(104)),
    ],
}
# D: no rotation at all, one kv head, a single expert, one layer that publishes its values and none that mixes them,
# heads of 128 with values of 16.
RUZINEX_D = {
    "architecture": "Ruzinex", "vocab": 64, "width": 48, "norm": {"eps": 1e-6}, "residual_mult": 0.9,
    "layers": [
        _layer(_mix(5, 1, 16, 16, 0.25), moe(1, 1, 24, shared=8)),
        _layer(_mix(2, 1, 128, 16, 0.09, rot=(1e6, 32, 8.0), v_mix=True), dense(48)),
    ],
}
MODELS = {"A": RUZINEX_A, "B": RUZINEX_B, "C": RUZINEX_C, "D": RUZINEX_D}


def single_layer(mlp, v_mix_layers=0, width=100) -> dict:
    """A model of one attention layer (and `v_mix_layers` more that mix its values), with the feed-forward `mlp`."""
    mixer = _mix(6, 2, 20, 12, 0.2, rot=(1000.0, 10, 4.0), v_mix=v_mix_layers > 0)
    layers = [_layer(mixer, mlp)] + [_layer(dict(mixer), None) for _ in range(v_mix_layers)]
    return {"architecture": "Ruzinex", "vocab": 131, "width": width, "norm": {"eps": 1e-5}, "residual_mult": 0.8, "layers": layers}


def make_model_dir(folder: str, cfg: dict, name: str, seed: int = 0, std: float = 0.1, bias_std: float = 0.7,
                   gain_std: float = 0.3) -> str:
    """Writes a model of configuration `cfg` through the framework's random-weights mode: matrices in bfloat16, so that
    both precisions of the engine and the plain implementation start from the same values; gains, biases, sinks and
    mixing weights spread widely so that leaving one out shows."""
    from gibbs_amd.config import config_from_dict
    from gibbs_amd.parts import DecoderModel
    from gibbs_amd.weights import write_random_model
    config = config_from_dict(cfg)
    decls = DecoderModel(config.model_spec()).tensor_decls()
    path = os.path.join(folder, f"ruzinex_{name}_{seed}")
    write_random_model(path, config, decls, seed=seed, dtype="bfloat16", std=std, gain_std=gain_std, bias_std=bias_std)
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
