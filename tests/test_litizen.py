"""Litizen without a GPU: the configuration reader, the model it describes, the tensors it declares, and the plain
implementation's mechanisms against hand-made cases."""
import copy

import numpy as np
import pytest

from tests import litizen_helpers as LH
from tests.plain import litizen_plain as Z


def test_registry_and_layers():
    from gibbs_amd.config import LitizenConfig, config_from_dict
    cfg = config_from_dict(LH.LITIZEN_A)
    assert isinstance(cfg, LitizenConfig) and cfg.to_dict() == LH.LITIZEN_A
    spec = cfg.model_spec()
    assert spec.order == (0, 1, 2, 3) and spec.head == "head" and spec.embedding == "embed" and spec.streams == 1
    assert spec.embedding_scale == 2.5 and spec.logit_softcap == 8.0
    assert [ls.arrangement for ls in spec.layers] == ["sandwich"] * 4
    assert [r for r, _ in spec.layers[0].parts] == ["norm1", "mixer_input", "mixer", "norm1b", "norm2", "ffn", "norm2b"]
    assert [r for r, _ in spec.layers[2].parts] == ["norm1", "mixer_input", "mixer", "norm1b"]
    assert [spec.layers[i].part("mixer").kind for i in range(4)] == ["attention", "ssd", "attention", "ssd"]
    assert cfg.derived()["layers_by_type"] == {"attention": 1, "attention_2": 1, "mamba2": 2}
    d = config_from_dict(LH.LITIZEN_D).model_spec()
    assert d.embedding_scale == 1.0 and d.logit_softcap == 0.0 and [r for r, _ in d.layers[0].parts][:2] == ["norm1", "mixer"]


def test_constants_come_from_the_configuration():
    from gibbs_amd.config import config_from_dict
    spec = config_from_dict(LH.LITIZEN_A).model_spec()
    n = spec.layers[0].part("norm1")
    assert (n.kind, n.eps, n.groups) == ("group_rms", 1e-5, 5) and spec.final_norm.groups == 5
    assert config_from_dict(LH.LITIZEN_B).model_spec().final_norm.kind == "rms"
    assert spec.layers[1].part("mixer_input").params == {"taps": 2}
    w, s, c = spec.layers[0].part("mixer"), spec.layers[1].part("mixer"), spec.layers[2].part("mixer")
    assert w.params["heads"] == 6 and w.params["kv_heads"] == 3 and w.params["head_dim"] == 20 and w.params["v_head_dim"] == 20
    assert w.params["window"] == 7 and w.params["values_from_keys"] and w.params["sink"] == "zero" and w.params["gate"]
    assert w.params["qk_norm"] == "before" and w.params["qk_norm_eps"] == 1e-5 and w.params["scale"] == 0.25
    assert w.position.params == {"theta": 1000.0, "rotary_dim": 10, "variant": "half_split", "precision": "f64"}
    assert c.params["chunk"] == 13 and c.params["softcap"] == 5.0 and c.params["value_rotation"] == {"theta": 300.0} and c.params["sink"] is True
    assert c.params["v_head_dim"] == 10 and "window" not in c.params and c.position.params["rotary_dim"] == 12
    assert s.params == {"heads": 4, "vdim": 10, "state": 12, "groups": 2, "taps": 4, "norm_groups": 2, "norm_eps": 1e-5}
    ff0, ff1, ff3 = spec.layers[0].part("ffn"), spec.layers[1].part("ffn"), spec.layers[3].part("ffn")
    assert ff0.kind == "glu" and ff0.params == {"inter": 150, "activation": "silu"}
    assert ff1.kind == "moe" and ff1.params["experts"] == 5 and ff1.params["identity"] == 2 and ff1.params["top"] == 3
    assert ff1.params["scores"] == "softmax_all" and ff1.params["shared"] == {"inter": 44, "activation": "silu", "gate": False}
    assert ff3.params["shared"] is None and ff3.params["identity"] == 1
    d = config_from_dict(LH.LITIZEN_D).model_spec()
    assert d.layers[0].part("mixer").position is None and d.layers[0].part("mixer").params["window"] is None
    assert d.layers[1].part("mixer").position is None and d.layers[1].part("mixer").params["chunk"] == 0


def test_declared_tensors_cache_and_state():
    from gibbs_amd.config import config_from_dict
    from gibbs_amd.parts import DecoderModel
    model = DecoderModel(config_from_dict(LH.LITIZEN_A).model_spec())
    shapes = {d.name: d.shape for d in model.tensor_decls()}
    assert shapes["embed"] == (211, 100) and shapes["head"] == (211, 100) and shapes["final.norm"] == (100,)
    assert shapes["l0.canon1"] == (100, 2) and shapes["l3.canon1"] == (100, 2)
    assert shapes["l0.mix.q"] == (120, 100) and shapes["l0.mix.k"] == (60, 100) and "l0.mix.v" not in shapes and "l0.mix.sink" not in shapes
    assert shapes["l0.mix.q.norm"] == (20,) and shapes["l0.mix.k.norm"] == (20,) and shapes["l0.mix.g"] == (120, 100) and shapes["l0.mix.o"] == (100, 120)
    assert shapes["l2.mix.v"] == (20, 100) and shapes["l2.mix.sink"] == (6,) and shapes["l2.mix.g"] == (60, 100) and "l2.mix.q.norm" not in shapes
    assert shapes["l1.mix.in"] == (2 * 40 + 2 * 24 + 4, 100) and shapes["l1.mix.conv"] == (88, 4) and shapes["l1.mix.conv.b"] == (88,)
    assert shapes["l1.mix.A_log"] == (4,) and shapes["l1.mix.D"] == (4,) and shapes["l1.mix.dt_bias"] == (4,) and shapes["l1.mix.norm"] == (40,)
    assert shapes["l1.mlp.router"] == (7, 100) and shapes["l1.mlp.correction"] == (7,) and shapes["l1.mlp.e4.down"] == (100, 30) and "l1.mlp.e5.up" not in shapes
    assert shapes["l1.mlp.shared.up"] == (44, 100) and "l3.mlp.shared.up" not in shapes and "l2.norm2" not in shapes
    owners = model.cache_owners()
    assert owners[:4] == [(0, "mixer_input"), (0, "mixer"), (1, "mixer_input"), (1, "mixer")]
    need = dict(zip(owners, model.cache_needs()))
    assert (need[(0, "mixer")].kv_heads, need[(0, "mixer")].head_dim, need[(0, "mixer")].window) == (3, 20, 7)
    assert (need[(2, "mixer")].kv_heads, need[(2, "mixer")].head_dim, need[(2, "mixer")].value_dim, need[(2, "mixer")].window) == (2, 12, 10, None)
    assert need[(1, "mixer")] is None and need[(0, "mixer_input")] is None
    states = dict(zip(owners, model.state_needs()))
    assert [(s.name, s.shape) for s in states[(0, "mixer_input")]] == [("conv_input", (1, 100))]
    assert sorted((s.name, s.shape) for s in states[(1, "mixer")]) == [("ssd_conv", (3, 88)), ("ssd_rule", (4, 12, 10))]
    one_tap = DecoderModel(config_from_dict(LH.LITIZEN_C).model_spec())
    assert all(not s for o, s in zip(one_tap.cache_owners(), one_tap.state_needs()) if o[1] == "mixer_input")


def test_what_the_checkpoint_holds_decides_the_optional_tensors():
    from gibbs_amd.config import config_from_dict
    from gibbs_amd.parts import DecoderModel
    full = {d.name: d.shape for d in DecoderModel(config_from_dict(LH.LITIZEN_A).model_spec()).tensor_decls()}
    gone = ("head", "l1.mlp.correction", "l2.mix.sink", "l0.mix.q.norm", "l0.mix.k.norm", "l2.mix.g") + tuple(f"l{i}.canon1" for i in range(4))
    table = {k: v for k, v in full.items() if k not in gone}
    spec = config_from_dict(LH.LITIZEN_A, tensors=table).model_spec()
    names = {d.name for d in DecoderModel(spec).tensor_decls()}
    assert names == set(table) and spec.head is None
    assert "mixer_input" not in [r for r, _ in spec.layers[0].parts]
    assert spec.layers[0].part("mixer").params.get("qk_norm") is None and spec.layers[2].part("mixer").params["sink"] is False
    assert spec.layers[2].part("mixer").params["gate"] is False and "correction" not in spec.layers[1].part("ffn").tensors
    # a layer without a feed-forward whose checkpoint holds that sublayer's norms: declared, and read by nobody
    more = dict(full, **{"l2.norm2": (100,), "l2.norm2b": (100,)})
    spec = config_from_dict(LH.LITIZEN_A, tensors=more).model_spec()
    assert {d.name for d in DecoderModel(spec).tensor_decls()} == set(more) and [r for r, _ in spec.layers[2].parts][-1] == "norm1b"


@pytest.mark.parametrize("change, words", [
    (lambda c: c["layers"][0].__setitem__("type", "conv"), "mixer type"),
    (lambda c: c["layers"][0]["mixer"].__setitem__("kv_heads", 4), "multiple"),
    (lambda c: c["layers"][0]["mixer"].__setitem__("vdim", 12), "values are the keys"),
    (lambda c: c["layers"][0]["mixer"]["rot"].__setitem__("dims", 22), "rotated"),
    (lambda c: c["layers"][2]["mixer"].__setitem__("vdim", 9), "pairs"),
    (lambda c: c["layers"][1]["mixer"].__setitem__("groups", 3), "groups"),
    (lambda c: c["layers"][1]["mixer"].__setitem__("norm_groups", 3), "equal parts"),
    (lambda c: c["layers"][1]["mlp"]["router"].__setitem__("top", 8), "experts a token"),
    (lambda c: c["norm"].__setitem__("groups", 7), "equal parts"),
    (lambda c: c.pop("width"), "width"),
])
def test_refused_configurations(change, words):
    from gibbs_amd.config import ConfigError, config_from_dict
    cfg = copy.deepcopy(LH.LITIZEN_A)
    change(cfg)
    with pytest.raises(ConfigError, match=words):
        config_from_dict(cfg)


# ----------------------------------------------------------------------------------------------- the plain mechanisms
def test_norm_in_groups():
    x = np.array([[3.0, 4.0, 0.0, 0.0, 100.0, 0.0]])
    out = Z.group_rms_norm(x, np.array([1.0, 1.0, 2.0, 2.0, 1.0, 0.5]), 1e-12, 3)
    want = np.array([[3.0 / np.sqrt(12.5), 4.0 / np.sqrt(12.5), 0.0, 0.0, np.sqrt(2.0), 0.0]])
    assert np.allclose(out, want)
    assert np.allclose(Z.group_rms_norm(x, np.ones(6), 1e-5, 1), x / np.sqrt((x * x).mean() + 1e-5))


def test_convolution_reaches_back_and_starts_from_zeros():
    x = np.arange(1.0, 6.0)[:, None] * np.array([[1.0, 10.0]])
    taps = np.array([[0.5, 0.25, 2.0], [0.0, 1.0, 0.0]])
    y = Z.causal_conv(x, taps, bias=np.array([0.0, 1.0]))
    assert np.allclose(y[:, 0], [2.0, 4.25, 7.0, 9.75, 12.5]) and np.allclose(y[:, 1], [1.0, 11.0, 21.0, 31.0, 41.0])
    assert np.allclose(Z.input_conv(x, taps)[:, 0], x[:, 0] + y[:, 0])


def test_masks_at_their_edges():
    w, c = Z.visible_window(10, 3), Z.visible_chunk(10, 4)
    assert w[5].nonzero()[0].tolist() == [3, 4, 5] and w[1].nonzero()[0].tolist() == [0, 1] and Z.visible_window(4, 1).sum() == 4
    assert c[5].nonzero()[0].tolist() == [4, 5] and c[7].nonzero()[0].tolist() == [4, 5, 6, 7] and c[8].nonzero()[0].tolist() == [8]
    assert c[3].nonzero()[0].tolist() == [0, 1, 2, 3]


def test_a_sink_counts_once_and_the_cap_bounds_the_scores():
    q = np.array([[[2.0, 0.0]], [[2.0, 0.0]]])
    k = np.array([[[1.0, 0.0]], [[50.0, 0.0]]])
    v = np.array([[[1.0]], [[3.0]]])
    out = Z.masked_attention(q, k, v, 0.5, Z.visible_window(2, 2), sink=np.zeros(1))
    assert np.isclose(out[0, 0, 0], np.e / (1.0 + np.e))                       # one key with score 1 beside the sink's exp(0)
    capped = Z.masked_attention(q, k, v, 0.5, Z.visible_window(2, 2), sink=np.array([0.0]), softcap=2.0)
    s0, s1 = 2.0 * np.tanh(0.5), 2.0 * np.tanh(25.0)
    assert np.isclose(capped[1, 0, 0], (np.exp(s0) * 1.0 + np.exp(s1) * 3.0) / (1.0 + np.exp(s0) + np.exp(s1)))
    none = Z.masked_attention(q, k, v, 0.5, Z.visible_window(2, 2))
    assert np.isclose(none[0, 0, 0], 1.0)


def test_turned_values_come_back_as_a_function_of_the_distance():
    """Values turned by their own position and the output turned back by the query's: with one visible key the result is
    the value turned by minus the distance, wherever the pair sits in the sequence."""
    rng = np.random.default_rng(0)
    v = rng.normal(size=(1, 1, 8))
    outs = []
    for j, i in ((3, 5), (40, 42)):
        turned = Z.rotate(v, [j], 100.0, 8)
        outs.append(Z.rotate(turned, [i], 100.0, 8, sign=-1.0))
    assert np.allclose(outs[0], outs[1], atol=1e-5) and not np.allclose(outs[0], v)
    assert np.allclose(Z.rotate(Z.rotate(v, [7], 100.0, 8), [7], 100.0, 8, sign=-1.0), v, atol=1e-6)
    part = Z.rotate(v, [9], 100.0, 4)
    assert np.array_equal(part[..., 4:], v[..., 4:]) and not np.allclose(part[..., :4], v[..., :4])


def test_the_recurrence_against_its_closed_form():
    """With constant decay a per token, y_t = sum_s a^(t - s) dt (B_s . C_t) x_s + D x_t."""
    rng = np.random.default_rng(1)
    T, H, P, N = 6, 2, 3, 4
    x, B, C = rng.normal(size=(T, H, P)), rng.normal(size=(T, 1, N)), rng.normal(size=(T, 1, N))
    dt, a_log, D = np.full((T, H), 0.3), np.array([0.2, -0.5]), np.array([1.5, -2.0])
    y = Z.ssd_scan(x, B, C, dt, a_log, D, 1)
    for h in range(H):
        a = np.exp(-np.exp(a_log[h]) * 0.3)
        for t in range(T):
            want = D[h] * x[t, h] + sum(a ** (t - s) * 0.3 * (B[s, 0] @ C[t, 0]) * x[s, h] for s in range(t + 1))
            assert np.allclose(y[t, h], want)


def test_choice_by_score_plus_correction_weights_by_score_alone():
    h = np.eye(3)
    router = np.array([[2.0, 0.0, 0.0], [1.0, 0.0, 0.0], [0.0, 0.0, 0.0], [-1.0, 0.0, 0.0]])
    corr = np.array([0.0, 0.0, 0.0, 1.0])
    chosen, weights = Z.route(h[:1], router, corr, 2)
    s = np.exp([2.0, 1.0, 0.0, -1.0]) / np.exp([2.0, 1.0, 0.0, -1.0]).sum()
    assert chosen[0].tolist() == [3, 0]                                     # the last output wins by its correction alone
    assert np.allclose(weights[0], [s[3] / (s[3] + s[0]), s[0] / (s[3] + s[0])])
    tied, _ = Z.route(h[1:2], router, np.zeros(4), 2)
    assert tied[0].tolist() == [0, 1]                                       # equal scores: the lower index
    assert np.isinf(Z.route_margin(h[:1], router, corr, 4)).all() and Z.route_margin(h[1:2], router, np.zeros(4), 2)[0] == 0.0


def test_identity_experts_return_their_input():
    rng = np.random.default_rng(2)
    W, F = 6, 4
    w = {"m.router": np.zeros((3, W)), "m.correction": np.array([0.0, 5.0, 4.0]),
         "m.e0.gate": rng.normal(size=(F, W)), "m.e0.up": rng.normal(size=(F, W)), "m.e0.down": rng.normal(size=(W, F))}
    h = rng.normal(size=(2, W))
    mlp = {"kind": "moe", "expert": {"ff": F}, "router": {"experts": 1, "identity": 2, "top": 2}}
    assert np.allclose(Z.moe_ff(h, w, "m.", mlp), h)                        # two identity experts of weight one half each
    mlp["router"]["top"] = 3
    third = Z.gated_ff(h, w["m.e0.gate"], w["m.e0.up"], w["m.e0.down"]) / 3.0 + 2.0 * h / 3.0
    assert np.allclose(Z.moe_ff(h, w, "m.", mlp), third)


def test_plain_forward_runs_every_configuration(tmp_path):
    for name, cfg in LH.MODELS.items():
        d = LH.make_model_dir(str(tmp_path), cfg, name, seed=3)
        ids = LH.tokens(1, 30, cfg["vocab"])
        logits = LH.plain_logits(d, ids)
        assert logits.shape == (30, cfg["vocab"]) and np.isfinite(logits).all()
        cap = cfg.get("logit_softcap")
        assert cap is None or np.abs(logits).max() < cap
        # what a position's logits are does not depend on what follows it
        assert np.allclose(LH.plain_logits(d, ids[:17]), logits[:17], atol=1e-9)
