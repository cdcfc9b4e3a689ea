"""Ruzinex on the GPU against the plain implementation, in 32-bit and in bfloat16: each mechanism alone; whole prompts;
most of a prompt in one step and its last tokens one by one; portions of changing size down to two tokens; mixed
batches in a pool so small that pages and slots are used again; long decoding; the first tokens; kernels with inputs
made so that one far key, a sink, a bias, a mixing weight or a router's choice stands out; generation through the
scheduler, the replay program and the command line."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

from tests import ruzinex_helpers as ZH
from tests.plain import ruzinex_plain as Z
from tests.test_engine_gpu import mixed_schedule, portions, run_steps

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
DTYPES = ["float32", "bfloat16"]
NAMES = ["A", "B", "C", "D"]
LENGTHS = {"A": 150, "B": 330, "C": 120, "D": 90}
# bfloat16 against the plain implementation, per row: relative L2 error of the logits.  A router's choice between two
# experts whose logits differ by less than the rounding of its input may fall the other way than in float64: rows whose
# least clear choice (`route_margin`) is below CLEAR_CHOICE are not held to the bound, and of the others one in a
# hundred may exceed it (a row that attends to a token whose choice fell the other way).
BF16_REL_L2 = 0.05
BF16_ROWS_OVER = 0.01
CLEAR_CHOICE = 0.03


@pytest.fixture(scope="module")
def dirs(tmp_path_factory):
    root = tmp_path_factory.mktemp("ruzinex")
    out = {n: ZH.make_model_dir(str(root), ZH.MODELS[n], n, seed=21 + i) for i, n in enumerate(NAMES)}
    out["attention"] = ZH.make_model_dir(str(root), ZH.single_layer(None), "attention", seed=5)
    out["value_mix"] = ZH.make_model_dir(str(root), ZH.single_layer(None, v_mix_layers=2), "value_mix", seed=6)
    out["dense"] = ZH.make_model_dir(str(root), ZH.single_layer(ZH.dense(77)), "dense", seed=7)
    out["experts"] = ZH.make_model_dir(str(root), ZH.single_layer(ZH.moe(7, 3, 36, shared=20)), "experts", seed=8)
    out["experts_aligned"] = ZH.make_model_dir(str(root), ZH.single_layer(ZH.moe(4, 2, 64), width=128), "experts_aligned", seed=9)
    return out


def make_engine(model_dir, dtype, **kw):
    from gibbs_amd import Engine
    kw.setdefault("max_tokens", 2048)
    kw.setdefault("max_requests", 4)
    return Engine(model_dir, dtype=dtype, **kw)


def close(got, want, dtype, what, margins=None):
    got, want = np.asarray(got, dtype=np.float64), np.asarray(want, dtype=np.float64)
    assert got.shape == want.shape, (what, got.shape, want.shape)
    if dtype == "float32":
        err = np.abs(got - want).max(-1)
        bound = 2e-5 * np.abs(want).max()
        assert err.max() <= bound, f"{what}: max error {err.max():.3e} at row {int(err.argmax())} above {bound:.3e}; first bad row {int((err > bound).argmax())}"
        return
    rel = np.sqrt(((got - want) ** 2).sum(-1) / (want ** 2).sum(-1))
    assert np.isfinite(rel).all(), what
    clear = np.ones(rel.size, dtype=bool) if margins is None else np.asarray(margins) >= CLEAR_CHOICE
    assert clear.sum() >= 0.5 * rel.size, f"{what}: only {int(clear.sum())} of {rel.size} rows have clear choices of experts"
    over = (rel > BF16_REL_L2) & clear
    allowed = 0 if margins is None or np.isinf(margins).all() else max(1, int(BF16_ROWS_OVER * rel.size))
    assert over.sum() <= allowed, \
        f"{what}: relative L2 error {rel[clear].max():.3e}; {int(over.sum())} of {int(clear.sum())} rows with clear choices over; first bad row {int(over.argmax())}"


def check(model_dir, seqs, got, dtype, what):
    for rid, ids in seqs.items():
        want = ZH.plain_logits(model_dir, ids)
        places = sorted(p for r, p in got if r == rid)
        assert places, f"{what}: no logits for {rid}"
        close(np.stack([got[(rid, p)] for p in places]), want[places], dtype, f"{what} request {rid}", ZH.plain_margins(model_dir, ids)[places])


def vocab_of(model_dir):
    with open(os.path.join(model_dir, "config.json")) as f:
        return json.load(f)["vocab"]


# ----------------------------------------------------------------------------------------------- whole models
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("kind", ["attention", "value_mix", "dense", "experts", "experts_aligned"])
def test_each_mechanism_alone(dirs, kind, dtype):
    d = dirs[kind]
    ids = ZH.tokens(1, 90, vocab_of(d))
    eng = make_engine(d, dtype)
    got = run_steps(eng, [([("r", ids[:61], list(range(61)))], []), ([("r", ids[61:], list(range(29)))], ["r"])])
    check(d, {"r": ids}, got, dtype, f"{kind} alone {dtype}")
    assert eng.cache.free_slots() == 4


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", NAMES)
def test_whole(dirs, name, dtype):
    d = dirs[name]
    ids = ZH.tokens(2, LENGTHS[name], vocab_of(d))
    eng = make_engine(d, dtype)
    got = run_steps(eng, [([("r", ids, list(range(len(ids))))], ["r"])])
    check(d, {"r": ids}, got, dtype, f"whole {name} {dtype}")
    eng.cache.check()
    assert all(eng.cache.free_pages(g) == eng.cache.pools[g].num_pages for g in range(eng.cache.n_groups))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", NAMES)
def test_bulk_then_last_tokens_one_by_one(dirs, name, dtype):
    d = dirs[name]
    ids = ZH.tokens(3, LENGTHS[name], vocab_of(d))
    cut = len(ids) - 40
    steps = [([("r", ids[:cut], list(range(cut)))], [])] + [([("r", [t], [0])], []) for t in ids[cut:]]
    got = run_steps(make_engine(d, dtype), steps)
    check(d, {"r": ids}, got, dtype, f"bulk+tail {name} {dtype}")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", NAMES)
def test_changing_portions_down_to_two_tokens(dirs, name, dtype):
    d = dirs[name]
    ids = ZH.tokens(4, LENGTHS[name], vocab_of(d))
    cuts = portions(len(ids) - 9, [7, 2, 13, 3, 2, 64, 5, 2, 17, 1, 2]) + [(len(ids) - 9 + i, len(ids) - 8 + i) for i in range(9)]
    steps = [([("r", ids[a:b], list(range(b - a)))], []) for a, b in cuts]
    got = run_steps(make_engine(d, dtype), steps)
    check(d, {"r": ids}, got, dtype, f"portions {name} {dtype}")


@pytest.mark.parametrize("name", NAMES)
def test_cutting_and_batching_change_nothing_in_32_bit(dirs, name):
    """Products add in ascending k, the attention takes keys in blocks aligned to absolute positions, and an expert's
    result for a row does not depend on which other rows the expert serves: 32-bit logits do not depend on how the prompt
    was cut or on what else was in the batch, beyond rounding."""
    d = dirs[name]
    ids = ZH.tokens(5, 77, vocab_of(d))
    other = ZH.tokens(6, 41, vocab_of(d))
    whole = run_steps(make_engine(d, "float32"), [([("r", ids, list(range(77)))], [])])
    eng = make_engine(d, "float32")
    steps = [([("o", other[:20], []), ("r", ids[:2], [0, 1])], []), ([("r", ids[2:50], list(range(48))), ("o", other[20:21], [])], []),
             ([("o", other[21:], []), ("r", ids[50:51], [0])], ["o"]), ([("r", ids[51:], list(range(26)))], [])]
    cut = run_steps(eng, steps)
    for p in range(77):
        assert np.abs(cut[("r", p)] - whole[("r", p)]).max() <= 2e-6 * np.abs(whole[("r", p)]).max(), p


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", NAMES)
def test_mixed_batches_with_pages_and_slots_used_again(dirs, name, dtype):
    d = dirs[name]
    rng = np.random.default_rng(7)
    seqs = {f"q{i}": ZH.tokens(100 + i, int(n), vocab_of(d)) for i, n in enumerate([70, 45, 90, 33, 64, 81, 50, 3, 2])}
    steps = mixed_schedule(seqs, rng)
    assert max(len(e) for e, _ in steps) >= 3
    assert any(len(t) > 1 for e, _ in steps for _, t, _ in e) and any(len(t) == 1 for e, _ in steps for _, t, _ in e)
    eng = make_engine(d, dtype, max_tokens=384, max_requests=4, page_size=16)
    assert sum(-(-len(s) // 16) for s in seqs.values()) > eng.cache.pools[0].num_pages, "the pool must be too small to avoid reuse"
    got = run_steps(eng, steps)
    check(d, seqs, got, dtype, f"mixed {name} {dtype}")
    eng.cache.check()
    assert eng.cache.free_slots() == 4 and all(eng.cache.free_pages(g) == eng.cache.pools[g].num_pages for g in range(eng.cache.n_groups))


@pytest.mark.parametrize("dtype", DTYPES)
def test_long_decoding(dirs, dtype):
    d = dirs["A"]
    ids = ZH.tokens(9, 330, vocab_of(d))
    steps = [([("r", ids[:5], list(range(5)))], [])] + [([("r", [t], [0])], []) for t in ids[5:]]
    got = run_steps(make_engine(d, dtype), steps)
    check(d, {"r": ids}, got, dtype, f"long decoding {dtype}")


@pytest.mark.parametrize("dtype", DTYPES)
def test_first_tokens(dirs, dtype):
    """Sequences of one, two, three and five tokens, side by side and one token at a time: a single visible key beside
    the sink, values mixed with the first layer's from the first token on."""
    d = dirs["A"]
    seqs = {f"s{n}": ZH.tokens(20 + n, n, vocab_of(d)) for n in (1, 2, 3, 5)}
    got = run_steps(make_engine(d, dtype), [([(r, ids, list(range(len(ids)))) for r, ids in seqs.items()], list(seqs))])
    check(d, seqs, got, dtype, f"first tokens together {dtype}")
    eng = make_engine(d, dtype)
    for r, ids in seqs.items():
        got = run_steps(eng, [([(r, ids[:1], [0])], [])] + [([(r, [t], [0])], []) for t in ids[1:]])
        check(d, {r: ids}, got, dtype, f"first tokens one by one {dtype}")
        eng.release(r)


# ----------------------------------------------------------------------------------------------- kernels with made-up inputs
def _dev(a, dtype=torch.float32):
    return torch.tensor(np.asarray(a), dtype=dtype, device="cuda")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("mode", ["publish", "mix", "none"])
@pytest.mark.parametrize("sizes", [(3, 2, 12, 24, 20, 6, 5), (3, 2, 32, 24, 16, 16, 8), (5, 1, 64, 64, 64, 64, 0)])
def test_projected_rows_bias_rotation_value_mixing_and_cache_write(dtype, mode, sizes):
    """Rows [q | k | v] with heads of 12 (6 of them rotated) and values of 20 stored as 24, and sizes in steps of 8 that take
    the kernel with 16-byte accesses in bfloat16 (part of a head rotated, and all of it): biases, the rotation with scaled
    frequencies at positions on both sides of page borders and far out, the values published or mixed, pages written."""
    from gibbs_amd.ops.lib import call, dtype_code, ptr, stream
    rng = np.random.default_rng(1)
    nh, nkv, hd, vd, vt, rot, extra = sizes
    ps = 16
    pos = _dev([0, 15, 16, 17, 31, 250, 70000], torch.int32)
    n = pos.numel()
    ld = (nh + nkv) * hd + nkv * vd + extra
    rows = _dev(rng.normal(size=(n, ld)), dtype)
    before = rows.float().cpu().numpy().astype(np.float64)
    bias = _dev(rng.normal(size=(nh + nkv) * hd + nkv * vd))
    inv = _dev((1000.0 ** (-2.0 * np.arange(rot // 2) / rot) / 4.0).astype(np.float32))
    n_pages = 70000 // ps + 1
    kpages = torch.zeros((n_pages, nkv, ps, hd), dtype=dtype, device="cuda")
    vpages = torch.zeros((n_pages, nkv, ps, vd), dtype=dtype, device="cuda")
    table = torch.arange(n_pages - 1, -1, -1, dtype=torch.int32, device="cuda").view(1, n_pages).contiguous()
    req = torch.zeros(n, dtype=torch.int32, device="cuda")
    keep = _dev(rng.normal(size=(n, nkv * vt)), dtype)
    kept = keep.float().cpu().numpy().astype(np.float64).reshape(n, nkv, vt)
    lam = _dev([0.3])
    call("gibbs_qkv_prepare", ptr(rows), ld, ptr(kpages), ptr(vpages), dtype_code(dtype), ptr(bias), ptr(inv), rot, 0, None, 0,
         ptr(keep), {"none": 0, "publish": 1, "mix": 2}[mode], vt, ptr(lam), ptr(pos), ptr(req), ptr(table), n_pages, ps, n_pages,
         n, nh, nkv, hd, vd, stream())
    tol = 3e-6 if dtype == torch.float32 else 2e-2
    b = bias.cpu().numpy().astype(np.float64)
    places = pos.tolist()
    q = Z.rotate((before[:, :nh * hd] + b[:nh * hd]).reshape(n, nh, hd), places, 1000.0, rot, 4.0)
    k = Z.rotate((before[:, nh * hd:(nh + nkv) * hd] + b[nh * hd:(nh + nkv) * hd]).reshape(n, nkv, hd), places, 1000.0, rot, 4.0)
    v = (before[:, (nh + nkv) * hd:(nh + nkv) * hd + nkv * vd] + b[(nh + nkv) * hd:]).reshape(n, nkv, vd)
    if mode == "mix":
        v[:, :, :vt] = 0.7 * v[:, :, :vt] + 0.3 * kept
    after = rows.float().cpu().numpy()
    assert np.abs(after[:, :nh * hd].reshape(n, nh, hd) - q).max() <= tol * 4
    assert extra == 0 or np.array_equal(after[:, -extra:], before[:, -extra:].astype(np.float32))
    for i, p in enumerate(places):
        page = n_pages - 1 - p // ps
        assert np.abs(kpages[page, :, p % ps].float().cpu().numpy() - k[i]).max() <= tol * 4, p
        assert np.abs(vpages[page, :, p % ps].float().cpu().numpy() - v[i]).max() <= tol * 4, p
    if mode == "publish":
        assert np.abs(keep.float().cpu().numpy().reshape(n, nkv, vt) - v[:, :, :vt]).max() <= tol * 4
    else:
        assert np.array_equal(keep.float().cpu().numpy().reshape(n, nkv, vt), kept.astype(np.float32))
    assert int((kpages != 0).any(-1).sum()) == n * nkv            # nothing else was written


@pytest.mark.parametrize("kernel", ["plain32", "plain16", "plain16_own_values", "decode", "prefill"])
def test_grouped_heads_far_keys_page_borders_and_the_sink(kernel):
    """Six query heads over two kv heads whose values have a size of their own (the plain kernel) or the keys' (the
    matrix-core kernels), pages of 16 scattered over the pool.  One key is made to dominate head 4 (kv head 1): at page
    borders, inside a page, at the sequence's first token and 700 tokens back; then a sink that outweighs every key must
    shrink its head's output and leave the others alone."""
    from gibbs_amd import ops
    rng = np.random.default_rng(0)
    dtype = torch.float32 if kernel == "plain32" else torch.bfloat16
    tol = 2e-5 if kernel == "plain32" else 3e-2
    T, nh, nkv, hd, ps, n_pages = 720, 6, 2, 32, 16, 64
    vd = 20 if kernel in ("plain32", "plain16_own_values") else hd
    order = rng.permutation(n_pages)[:-(-T // ps)].tolist()
    table = _dev([order], torch.int32)
    keys = _dev(rng.normal(size=(T, nkv, hd)) * 0.1, dtype)
    vals = _dev(rng.normal(size=(T, nkv, vd)), dtype)
    p = T - 1
    q = _dev(rng.normal(size=(1, nh * hd)) * 0.1, dtype)
    qh = q.float().cpu().numpy().reshape(nh, hd).astype(np.float64)

    def pages_of(rows):
        pages = torch.full((n_pages, nkv, ps, rows.shape[-1]), 7.0, dtype=dtype, device="cuda")
        for t in range(T):
            pages[order[t // ps], :, t % ps] = rows[t]
        return pages

    def run(k_rows, sink):
        kp, vp = pages_of(k_rows), pages_of(vals)
        sk = None if sink is None else _dev(sink)
        pos, req = _dev([p], torch.int32), torch.zeros(1, dtype=torch.int32, device="cuda")
        if kernel.startswith("plain"):
            out = ops.attention_plain(q, 1, nh, nkv, hd, kp, vp, table, 1, pos, req, 1.0, sink=sk)
        elif kernel == "decode":
            out = ops.attention_decode(q, 1, nh, nkv, hd, kp, vp, table, 1, pos, req, 1.0, max_seq=T, n_splits=3, sink=sk)
        else:
            n = 40
            qs = torch.zeros((n, nh * hd), dtype=dtype, device="cuda")
            qs[-1] = q[0]
            out = ops.attention_prefill(qs, n, nh, nkv, hd, kp, vp, table, 1, _dev([0, n], torch.int32), _dev([T - n], torch.int32), 1.0,
                                        max_seq=T, sink=sk)[-1:]
        return out.float().cpu().numpy().reshape(nh, vd)

    def want(k_rows, sink):
        kk, vv = k_rows.float().cpu().numpy().astype(np.float64), vals.float().cpu().numpy().astype(np.float64)
        qq = np.repeat(qh[None], T, 0)
        return Z.sink_softmax_attention(qq, kk, vv, 1.0, sink)[-1]

    for far in (0, 15, 16, 19, p - 16, p):
        k_rows = keys.clone()
        k_rows[far, 1] = (q[0, 4 * hd:5 * hd].float() / q[0, 4 * hd:5 * hd].float().norm() ** 2 * 14.0).to(dtype)    # head 4: q . k = 14
        got = run(k_rows, None)
        assert np.abs(got - want(k_rows, None)).max() <= tol * 4, far
        assert np.abs(got[4] - vals[far, 1].float().cpu().numpy()).max() < 0.2, f"head 4 does not see the key at {far}"
    sink = np.array([9.0, -30.0, 0.5, 3.0, 12.0, 0.0])
    got, without = run(keys, sink), run(keys, None)
    assert np.abs(got - want(keys, sink)).max() <= tol * 4
    assert np.abs(got[4]).max() < 0.01 * np.abs(without[4]).max() + tol and np.abs(got[1] - without[1]).max() <= tol * 4


@pytest.mark.parametrize("case", [(torch.float32, 52, 7, 3, 100, 30), (torch.bfloat16, 52, 7, 3, 100, 30), (torch.bfloat16, 300, 8, 2, 128, 64),
                                  (torch.bfloat16, 300, 3, 2, 1056, 512),
                                  (torch.bfloat16, 9, 16, 4, 64, 32), (torch.float32, 3, 1, 1, 24, 8)])
def test_experts_route_group_products_and_combine(case):
    """The router's choices and weights (with made-up logits that tie), the pairs sorted by expert, both products and the
    weighted sum with a shared expert, against the plain functions; few pairs (tiles of 16) and many (tiles of 64); plain
    products in 32-bit and for sizes that are not aligned, the matrix cores otherwise."""
    from gibbs_amd.ops.lib import call, dtype_code, library, ptr, stream
    dtype, n, E, top, W, F = case
    rng = np.random.default_rng(3)
    h = _dev(rng.normal(size=(n, W)), dtype)
    router = rng.normal(size=(E, W))
    if E > 2:
        router[2] = router[1]                                    # two experts with equal logits: the lower index wins
    router, rb = _dev(router), _dev(rng.normal(size=E) * 0.0)
    sgw = _dev(rng.normal(size=W) * 0.3)
    gate, up, down = _dev(rng.normal(size=(E, F, W)) * 0.1, dtype), _dev(rng.normal(size=(E, F, W)) * 0.1, dtype), _dev(rng.normal(size=(E, W, F)) * 0.1, dtype)
    chosen = torch.empty((n, top), dtype=torch.int32, device="cuda")
    weight = torch.empty((n, top), dtype=torch.float32, device="cuda")
    sgate = torch.empty(n, dtype=torch.float32, device="cuda")
    call("gibbs_moe_route", ptr(h), W, dtype_code(dtype), ptr(router), ptr(rb), ptr(sgw), ptr(chosen), ptr(weight), ptr(sgate), n, W, E, top, stream())
    hh = h.float().cpu().numpy().astype(np.float64)
    want_c, want_w = Z.route(hh, router.cpu().numpy().astype(np.float64), rb.cpu().numpy().astype(np.float64), top)
    z = hh @ router.cpu().numpy().astype(np.float64).T
    sure = np.ones(n, dtype=bool)
    if E > top:                                                   # rows whose last choice is clear of the next logit
        srt = np.sort(z, -1)[:, ::-1]
        sure = (srt[:, top - 1] - srt[:, top]) > 1e-3
        if E > 2:
            sure |= np.isin(want_c[:, -1], [1]) & (np.abs(z[:, 1] - z[:, 2]) < 1e-9)
    got_c = chosen.cpu().numpy()
    assert np.array_equal(got_c[sure], want_c[sure])
    assert np.abs(weight.cpu().numpy()[sure] - want_w[sure]).max() <= 1e-5
    assert np.abs(sgate.cpu().numpy() - Z.sigmoid(hh @ sgw.cpu().numpy().astype(np.float64))).max() <= 1e-5
    lib = library()
    pairs = n * top
    bm = lib.gibbs_moe_tile(pairs, E)
    assert bm == (128 if n == 300 else 16)
    cap = lib.gibbs_moe_capacity(pairs, E, bm)
    sorted_pair = torch.empty(cap, dtype=torch.int32, device="cuda")
    place = torch.empty(pairs, dtype=torch.int32, device="cuda")
    tile_expert = torch.empty(cap // bm, dtype=torch.int32, device="cuda")
    call("gibbs_moe_group", ptr(chosen), pairs, E, bm, ptr(sorted_pair), ptr(place), ptr(tile_expert), cap, stream())
    sp, pl, te = sorted_pair.cpu().numpy(), place.cpu().numpy(), tile_expert.cpu().numpy()
    assert sorted(sp[sp >= 0].tolist()) == list(range(pairs)) and np.array_equal(sp[pl], np.arange(pairs))
    flat = got_c.reshape(-1)
    for m in np.nonzero(sp >= 0)[0]:
        assert te[m // bm] == flat[sp[m]]
    mid = torch.zeros((cap, F), dtype=dtype, device="cuda")
    y = torch.zeros((cap, W), dtype=dtype, device="cuda")
    call("gibbs_moe_gemm", ptr(h), W, top, ptr(sorted_pair), ptr(tile_expert), cap, bm, ptr(gate), ptr(up), ptr(mid), F, dtype_code(dtype), F, W, 0, stream())
    call("gibbs_moe_gemm", ptr(mid), F, 0, ptr(sorted_pair), ptr(tile_expert), cap, bm, ptr(down), None, ptr(y), W, dtype_code(dtype), W, F, 0, stream())
    shared = _dev(rng.normal(size=(n, W)), dtype)
    out = torch.empty((n, W), dtype=dtype, device="cuda")
    call("gibbs_moe_combine", ptr(y), ptr(place), ptr(weight), ptr(shared), ptr(sgate), ptr(out), dtype_code(dtype), n, top, W, stream())
    g64, u64, d64 = (t.float().cpu().numpy().astype(np.float64) for t in (gate, up, down))
    wt = weight.cpu().numpy().astype(np.float64)
    want = sgate.cpu().numpy().astype(np.float64)[:, None] * shared.float().cpu().numpy().astype(np.float64)
    for r in range(n):
        for c in range(top):
            e = got_c[r, c]
            want[r] += wt[r, c] * ((Z.silu(hh[r] @ g64[e].T) * (hh[r] @ u64[e].T)) @ d64[e].T)
    tol = 2e-5 if dtype == torch.float32 else 3e-2
    assert np.abs(out.float().cpu().numpy() - want).max() <= tol * max(1.0, np.abs(want).max())


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("shared", ["gated", "plain", "none"])
def test_experts_sum_inside_the_sublayer_boundary(dtype, shared):
    """x += gain_b * rms_norm(sum_s w[n][s] y[place[n][s]] + g[n] shared[n]) and out = gain_a * rms_norm(x) in one kernel, against
    numpy; places are scattered over more rows than are used, and one row's weights leave a single choice."""
    from gibbs_amd.ops.lib import call, dtype_code, ptr, stream
    rng = np.random.default_rng(11)
    n, top, W, places = 37, 3, 200, 150
    y = _dev(rng.normal(size=(places, W)), dtype)
    place = rng.permutation(places)[:n * top].reshape(n, top).astype(np.int32)
    weight = rng.random(size=(n, top)).astype(np.float32)
    weight[5] = [0.0, 1.0, 0.0]
    sh = _dev(rng.normal(size=(n, W)), dtype) if shared != "none" else None
    g = _dev(rng.random(size=n)) if shared == "gated" else None
    x0 = rng.normal(size=(n, W)).astype(np.float32)
    gain_b, gain_a = rng.normal(size=W).astype(np.float32), rng.normal(size=W).astype(np.float32)
    x = _dev(x0)
    out = torch.empty((n, W), dtype=dtype, device="cuda")
    gb, ga, pl, wt = _dev(gain_b), _dev(gain_a), torch.tensor(place, device="cuda"), _dev(weight)
    call("gibbs_rmsnorm_rows_mix_add_norm", ptr(x), ptr(y), ptr(pl), ptr(wt), top, ptr(sh) if sh is not None else None,
         ptr(g) if g is not None else None, ptr(gb), 1e-5, ptr(ga), 1e-6, ptr(out), dtype_code(dtype), n, W, stream())
    y64 = y.float().cpu().numpy().astype(np.float64)
    v = (weight.astype(np.float64)[:, :, None] * y64[place]).sum(1)
    if sh is not None:
        v += (g.cpu().numpy().astype(np.float64)[:, None] if g is not None else 1.0) * sh.float().cpu().numpy().astype(np.float64)
    want_x = x0 + Z.rms_norm(v, gain_b.astype(np.float64), 1e-5)
    want_out = Z.rms_norm(want_x, gain_a.astype(np.float64), 1e-6)
    assert np.abs(x.cpu().numpy() - want_x).max() <= 2e-5
    assert np.abs(out.float().cpu().numpy() - want_out).max() <= (2e-5 if dtype == torch.float32 else 2e-2) * max(1.0, np.abs(want_out).max())


def test_a_rows_experts_do_not_depend_on_its_neighbours():
    """32-bit: the same row alone and among 200 others gives the same bits."""
    from gibbs_amd import Engine
    import tempfile
    with tempfile.TemporaryDirectory() as tmp:
        d = ZH.make_model_dir(tmp, ZH.single_layer(ZH.moe(6, 2, 40, shared=16)), "rows", seed=4)
        eng = Engine(d, dtype="float32", max_tokens=1024, max_requests=4)
        ff = eng.model.blocks[0].ffn
        rng = np.random.default_rng(5)
        h = _dev(rng.normal(size=(201, 100)))
        many = ff.forward(h, None).clone()
        one = ff.forward(h[77:78].contiguous(), None)
        assert torch.equal(many[77:78], one)


# ----------------------------------------------------------------------------------------------- entry points
def plain_greedy(model_dir, prompt, n):
    seq, out = list(prompt), []
    for _ in range(n):
        t = int(np.argmax(ZH.plain_logits(model_dir, seq)[-1]))
        out.append(t); seq.append(t)
    return out


@pytest.mark.parametrize("dtype", DTYPES)
def test_greedy_generation_through_the_scheduler(dirs, dtype):
    """`generate` (scheduler, prompt steps, bursts of captured decode steps) gives the plain implementation's greedy
    tokens; in bfloat16 wherever the plain logits' lead exceeds the precision's error."""
    from gibbs_amd import Engine, generate
    held = 0
    for name, lens in (("A", [7, 13, 2]), ("C", [5])):
        d = dirs[name]
        eng = Engine(d, dtype=dtype, max_tokens=512, max_requests=4)
        prompts = [ZH.tokens(40 + i, n, vocab_of(d)) for i, n in enumerate(lens)]
        outs = generate(eng, prompts, max_tokens=20, temperature=0.0, ignore_eos=True)
        for p, o in zip(prompts, outs):
            assert o.finish_reason == "length" and len(o.tokens) == 20
            if dtype == "float32":
                assert o.tokens == plain_greedy(d, p, 20)
                held += 20
                continue
            logits = ZH.plain_logits(d, list(p) + list(o.tokens))
            for i, t in enumerate(o.tokens):
                row = logits[len(p) - 1 + i]
                best, second = np.sort(row)[[-1, -2]]
                margin = 2 * 0.04 * np.abs(row).max()
                if best - second > margin:
                    held += 1
                    assert t == int(np.argmax(row)), f"token {i}"
                else:
                    assert row[t] >= best - margin, f"token {i}"
        eng.cache.check()
        assert eng.cache.free_slots() == 4
    assert held >= 20


def test_decode_bursts_change_nothing(dirs):
    from gibbs_amd import Engine, Generator, SamplingParams
    d = dirs["B"]
    prompts = [ZH.tokens(70 + i, n, vocab_of(d)) for i, n in enumerate([9, 21, 5])]
    runs = []
    for burst in (0, 16):
        eng = Engine(d, dtype="float32", max_tokens=1024, max_requests=4)
        gen = Generator(eng, decode_burst=burst, eos_token_ids=())
        rids = [gen.submit(p, SamplingParams(temperature=0.0, max_new_tokens=n), rid=f"r{i}") for i, (p, n) in enumerate(zip(prompts, [60, 20, 9]))]
        res = gen.run()
        runs.append([res[r].tokens for r in rids])
    assert runs[0] == runs[1]
    assert runs[0][0] == plain_greedy(d, prompts[0], 60)


@pytest.mark.parametrize("dtype", DTYPES)
def test_replay_program(dirs, dtype, tmp_path):
    d = dirs["C"]
    ids = ZH.tokens(50, 40, vocab_of(d))
    other = ZH.tokens(51, 9, vocab_of(d))
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": ids[:17], "want": [0, 16]}, {"id": "b", "tokens": other[:2], "want": []}], "end": []},
             {"step": 1, "entries": [{"id": "b", "tokens": other[2:], "want": [6]}], "end": ["b"]},
             {"step": 2, "entries": [{"id": "a", "tokens": ids[17:39], "want": [21]}], "end": []},
             {"step": 3, "entries": [{"id": "a", "tokens": ids[39:], "want": [0]}], "end": ["a"]}]
    out = tmp_path / "out"
    proc = subprocess.run([os.path.join(ROOT, "bin", "trace_run"), "--model", d, "--dtype", dtype, "--out", str(out), "--max-tokens", "128"],
                          input="\n".join(json.dumps(s) for s in steps) + "\n", capture_output=True, text=True, timeout=600)
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert [l for l in proc.stdout.splitlines() if l.startswith("done")] == [f"done {i}" for i in range(4)]
    want_a, want_b = ZH.plain_logits(d, ids), ZH.plain_logits(d, other)
    read = lambda i: np.fromfile(out / f"{i}.f32", dtype="<f4").reshape(-1, vocab_of(d))
    close(read(0), want_a[[0, 16]], dtype, "step 0")
    close(read(1), want_b[[8]], dtype, "step 1")
    close(read(2), want_a[[38]], dtype, "step 2")
    close(read(3), want_a[[39]], dtype, "step 3")


def test_command_line(dirs):
    d = dirs["A"]
    prompt = ZH.tokens(60, 6, vocab_of(d))
    proc = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "gibbs"), "--model", d, "--dtype", "float32", "--prompt-ids",
                           ",".join(map(str, prompt)), "--max-tokens", "8", "--temperature", "0", "--ignore-eos"],
                          capture_output=True, text=True, timeout=600)
    assert proc.returncode == 0, proc.stderr[-2000:]
    line = proc.stdout.split("✨ Output:\n")[1].splitlines()[0]
    assert [int(t) for t in line.split()] == plain_greedy(d, prompt, 8)
    proc = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "gibbs"), "--model", d, "--arch-dump"], capture_output=True, text=True, timeout=600)
    dump = json.loads(proc.stdout)
    assert dump["architecture"] == "Ruzinex" and dump["unconsumed"] == [] and dump["missing"] == []
    assert dump["derived"]["value_mix_source"] == 1
