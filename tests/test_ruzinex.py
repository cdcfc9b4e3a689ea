"""Ruzinex without a GPU: the configuration reader, the model it describes, the tensors it declares, and the plain
implementation's mechanisms against hand-made cases."""
import copy

import numpy as np
import pytest

from tests import ruzinex_helpers as ZH
from tests.plain import ruzinex_plain as Z


def test_registry_and_layers():
    from gibbs_amd.config import RuzinexConfig, config_from_dict
    cfg = config_from_dict(ZH.RUZINEX_A)
    assert isinstance(cfg, RuzinexConfig) and cfg.to_dict() == ZH.RUZINEX_A
    spec = cfg.model_spec()
    assert spec.order == (0, 1, 2, 3) and spec.head is None and spec.embedding == "embed" and spec.streams == 1
    assert [ls.arrangement for ls in spec.layers] == ["sandwich"] * 4 and spec.layers[0].params == {"residual_mult": 1.3}
    assert [r for r, _ in spec.layers[0].parts] == ["norm1", "mixer", "norm1b", "norm2", "ffn", "norm2b"]
    assert [r for r, _ in spec.layers[2].parts] == ["norm1", "mixer", "norm1b"]
    assert cfg.derived()["value_mix_source"] == 1
    assert config_from_dict(ZH.RUZINEX_C).model_spec().layers[0].params == {"residual_mult": 1.0}


def test_constants_come_from_the_configuration():
    from gibbs_amd.config import config_from_dict
    spec = config_from_dict(ZH.RUZINEX_A).model_spec()
    m0, m1, m2 = (spec.layers[i].part("mixer") for i in range(3))
    assert m0.params["heads"] == 6 and m0.params["kv_heads"] == 3 and m0.params["head_dim"] == 20 and m0.params["v_head_dim"] == 12
    assert m0.params["scale"] == 0.2 and m0.params["bias"] and m0.params["sink"] and m0.params["value_mix"] is None
    assert m0.position.params == {"theta": 1000.0, "rotary_dim": 10, "variant": "half_split", "precision": "f64", "scaling_factor": 4.0}
    assert m1.position.params["scaling_factor"] == 1.0 and m1.position.params["rotary_dim"] == 20
    assert m1.params["value_mix"] == {"key": 0, "publish": True} and m2.params["value_mix"] == {"key": 0, "publish": False}
    ff0, ff1, ff3 = spec.layers[0].part("ffn"), spec.layers[1].part("ffn"), spec.layers[3].part("ffn")
    assert ff0.kind == "glu" and ff0.params == {"inter": 150, "activation": "gelu_tanh"}
    assert ff1.kind == "moe" and ff1.params["experts"] == 5 and ff1.params["top"] == 2 and ff1.params["inter"] == 30
    assert ff1.params["shared"] == {"inter": 44, "activation": "silu", "gate": True} and ff1.params["activation"] == "silu"
    assert ff3.params["shared"] is None and ff3.params["top"] == 3
    assert config_from_dict(ZH.RUZINEX_D).model_spec().layers[0].part("mixer").position is None


def test_declared_tensors():
    from gibbs_amd.config import config_from_dict
    from gibbs_amd.parts import DecoderModel
    model = DecoderModel(config_from_dict(ZH.RUZINEX_A).model_spec())
    shapes = {d.name: d.shape for d in model.tensor_decls()}
    assert shapes["embed"] == (211, 100) and shapes["final.norm"] == (100,) and "head" not in shapes
    assert shapes["l0.mix.q"] == (120, 100) and shapes["l0.mix.k"] == (60, 100) and shapes["l0.mix.v"] == (36, 100)
    assert shapes["l0.mix.q.b"] == (120,) and shapes["l0.mix.v.b"] == (36,) and shapes["l0.mix.sink"] == (6,) and shapes["l0.mix.o"] == (100, 72)
    assert "l0.mix.vmix" not in shapes and shapes["l1.mix.vmix"] == () and shapes["l2.mix.vmix"] == ()
    assert shapes["l1.mlp.router"] == (5, 100) and shapes["l1.mlp.router.b"] == (5,) and shapes["l1.mlp.e4.down"] == (100, 30)
    assert shapes["l1.mlp.shared.up"] == (44, 100) and shapes["l1.mlp.shared.sg"] == (1, 100) and "l3.mlp.shared.sg" not in shapes
    assert "l2.norm2" not in shapes and shapes["l2.norm1b"] == (100,) and shapes["l3.norm2b"] == (100,)
    need = model.cache_needs()
    assert (need[0].kv_heads, need[0].head_dim, need[0].value_dim, need[0].window) == (3, 20, 12, None)
    assert (need[2].kv_heads, need[2].head_dim, need[2].value_dim) == (3, 14, 12) and all(not s for s in model.state_needs())


def test_what_the_checkpoint_holds_decides_the_optional_tensors():
    from gibbs_amd.config import config_from_dict
    from gibbs_amd.parts import DecoderModel
    from gibbs_amd.weights.loader import check_table
    full = DecoderModel(config_from_dict(ZH.RUZINEX_A).model_spec())
    table = {d.name: d.shape for d in full.tensor_decls()}
    # a mixing weight in a layer that does not mix, and second norms in a layer without a feed-forward: held, not read
    table.update({"l0.mix.vmix": (), "l2.norm2": (100,), "l2.norm2b": (100,)})
    del table["l1.mlp.router.b"], table["l1.mlp.shared.sg"]
    cfg = config_from_dict(ZH.RUZINEX_A, tensors=table)
    model = DecoderModel(cfg.model_spec())
    check_table(model.tensor_decls(), table)
    ff = cfg.model_spec().layers[1].part("ffn")
    assert "router_bias" not in ff.tensors and ff.params["shared"]["gate"] is False


def test_bad_configurations_are_refused():
    from gibbs_amd.config import ConfigError, config_from_dict
    def broken(change):
        c = copy.deepcopy(ZH.RUZINEX_A)
        change(c)
        with pytest.raises(ConfigError):
            config_from_dict(c)
    broken(lambda c: c["layers"][0].update(type="recurrent"))
    broken(lambda c: c["layers"][0]["mixer"].update(kv_heads=4))
    broken(lambda c: c["layers"][0]["mixer"]["rot"].update(dims=22))
    broken(lambda c: c["layers"][1]["mlp"]["router"].update(top=6))
    broken(lambda c: c["layers"][3]["mixer"].update(vdim=13))          # its values no longer fit the ones it mixes in
    broken(lambda c: c["layers"][2]["mixer"].update(heads=4, kv_heads=2, vdim=18))   # as many numbers, in other heads
    broken(lambda c: c["layers"][0]["mlp"].update(kind="sparse"))
    broken(lambda c: c.pop("width"))


# ----------------------------------------------------------------------------------------------- the plain mechanisms
def test_rotation_pairs_scaling_and_the_channels_that_pass():
    x = np.arange(1.0, 13.0).reshape(1, 1, 12).repeat(3, 0)
    out = Z.rotate(x, [0, 3, 8], 100.0, 4, factor=2.0)
    assert np.array_equal(out[0], x[0]) and np.array_equal(out[:, :, 4:], x[:, :, 4:])
    for t, p in ((1, 3), (2, 8)):
        for i in range(2):
            a = np.float32(p) * np.float32(100.0 ** (-2.0 * i / 4) / 2.0)
            u, v = x[t, 0, i], x[t, 0, i + 2]
            assert abs(out[t, 0, i] - (u * np.cos(a) - v * np.sin(a))) < 1e-6 and abs(out[t, 0, i + 2] - (v * np.cos(a) + u * np.sin(a))) < 1e-6
    # a scaled position is the unscaled rotation of position / factor
    assert np.allclose(Z.rotate(x, [0, 4, 8], 100.0, 4, factor=4.0)[1:], Z.rotate(x, [0, 1, 2], 100.0, 4)[1:], atol=1e-6)


def test_the_sink_counts_once_and_is_not_scaled():
    rng = np.random.default_rng(0)
    q, k, v = rng.normal(size=(5, 4, 6)), rng.normal(size=(5, 2, 6)), rng.normal(size=(5, 2, 3))
    plain = Z.sink_softmax_attention(q, k, v, 0.3)
    assert np.allclose(plain[0], v[0][[0, 0, 1, 1]])                      # the first token sees itself only; heads 0, 1 read kv head 0
    sunk = Z.sink_softmax_attention(q, k, v, 0.3, sink=np.array([-50.0, 0.0, 50.0, 2.0]))
    assert np.allclose(sunk[:, 0], plain[:, 0]) and np.abs(sunk[:, 2]).max() < 1e-15
    s = (q[3, 1] @ k[:4, 0].T) * 0.3
    w = np.exp(s) / (np.exp(s).sum() + np.exp(0.0))
    assert np.allclose(sunk[3, 1], w @ v[:4, 0])


def test_routing_takes_the_largest_and_normalises_over_them_alone():
    h = np.eye(4)
    router = np.array([[1.0, 0, 0, 5], [3.0, 0, 0, 5], [2.0, 1, 0, -1], [0.0, 1, 0, 5]])
    chosen, weight = Z.route(h, router, np.array([0.0, 0.0, 0.5, 0.0]), 2)
    assert chosen[0].tolist() == [1, 2] and chosen[1].tolist() == [2, 3]
    assert chosen[3].tolist() == [0, 1]                                   # equal logits: the lower indices
    assert np.allclose(weight[0], np.exp([3.0, 2.5]) / np.exp([3.0, 2.5]).sum()) and np.allclose(weight.sum(-1), 1.0)
    one, w1 = Z.route(h, router, np.zeros(4), 1)
    assert one[:, 0].tolist() == [1, 2, 0, 0] and np.array_equal(w1, np.ones((4, 1)))


def test_value_mixing_reads_the_first_mixing_layers_values():
    """With lambda = 1 in a later layer its own value projection does not matter at all."""
    import tempfile
    cfg = ZH.single_layer(None, v_mix_layers=1)
    rng = np.random.default_rng(1)
    with tempfile.TemporaryDirectory() as tmp:
        d = ZH.make_model_dir(tmp, cfg, "vm", seed=3)
        cfg2, w = ZH.load_model_dir(d)
    ids = ZH.tokens(2, 12, 131)
    w["l1.mix.vmix"] = np.array(1.0)
    base = Z.forward(cfg2, w, ids)
    w2 = dict(w)
    w2["l1.mix.v"] = rng.normal(size=w["l1.mix.v"].shape)
    assert np.allclose(Z.forward(cfg2, w2, ids), base)
    w2["l1.mix.vmix"] = np.array(0.5)
    assert not np.allclose(Z.forward(cfg2, w2, ids), base)
