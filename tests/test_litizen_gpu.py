"""Litizen on the GPU against the plain implementation, in 32-bit and in bfloat16: each mechanism alone; whole prompts;
most of a prompt in one step and its last tokens one by one; portions of changing size down to two tokens; mixed
batches in a pool so small that pages and slots are used again; long decoding; the first tokens; kernels with inputs
made so that one key at a window's or a chunk's edge, a sink, a state written long ago or a router's choice stands
out; generation through the scheduler, the replay program and the command line."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

from tests import litizen_helpers as LH
from tests.plain import litizen_plain as Z
from tests.test_engine_gpu import mixed_schedule, portions, run_steps

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
DTYPES = ["float32", "bfloat16"]
NAMES = ["A", "B", "C", "D"]
LENGTHS = {"A": 150, "B": 230, "C": 120, "D": 90}
# bfloat16 against the plain implementation, per row: relative L2 error of the logits.  A router's choice between two
# experts whose scores differ by less than the rounding of its input may fall the other way than in float64, and with a
# norm behind the experts that changes the token's whole row, which every later token may read through a window or a state:
# a sequence is held to the bound up to its first token whose least clear choice (`route_margin`) is below CLEAR_CHOICE
# (sequences are picked so that this comes late, `clear_tokens`).  So that every row of every test is held to the bound
# in bfloat16 as well, each model also runs in a copy whose routers always choose clearly (`settle_choices`).
# A sublayer's result is normed before it is added: where it nearly cancels for a token, the division by its root mean
# square amplifies the rounding of its operands (measured: single rows at 7 to 35 % among rows at 1 to 3 %, with clear
# choices of experts and 1e-5 in 32-bit): a few rows in a hundred may exceed the bound, none by more than BF16_WORST.
BF16_REL_L2 = 0.06
BF16_ROWS_OVER = 0.03
BF16_WORST = 0.5
CLEAR_CHOICE = 0.01


@pytest.fixture(scope="module")
def dirs(tmp_path_factory):
    root = tmp_path_factory.mktemp("litizen")
    out = {n: LH.make_model_dir(str(root), LH.MODELS[n], n, seed=31 + i) for i, n in enumerate(NAMES)}
    out.update({n + "_settled": LH.settle_choices(out[n], str(root)) for n in NAMES})
    one = LH.single_layer
    out["window"] = LH.make_model_dir(str(root), one(LH.window_attention(6, 2, 20, 0.2, size=9, rot=(1000.0, 10))), "window", seed=5)
    out["chunk"] = LH.make_model_dir(str(root), one(LH.chunk_attention(6, 3, 20, 12, 0.2, 1000.0, dims=8, size=11, softcap=4.0)), "chunk", seed=6)
    out["chunk_aligned"] = LH.make_model_dir(str(root), one(LH.chunk_attention(4, 2, 32, 32, 0.17, 1e4, dims=32, size=40, softcap=6.0), width=64, groups=2),
                                             "chunk_aligned", seed=10)
    out["state_space"] = LH.make_model_dir(str(root), one(LH.state_space(5, 8, 12, 5, 3, 2)), "state_space", seed=7)
    out["dense"] = LH.make_model_dir(str(root), one(LH.state_space(2, 10, 8, 1, 2, 1), LH.dense(77)), "dense", seed=8)
    out["experts"] = LH.make_model_dir(str(root), one(LH.state_space(2, 10, 8, 1, 2, 1), LH.moe(7, 2, 3, 36, shared=20)), "experts", seed=9)
    out["experts_settled"] = LH.settle_choices(out["experts"], str(root))
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
        bound = 3e-5 * np.abs(want).max()
        assert err.max() <= bound, f"{what}: max error {err.max():.3e} at row {int(err.argmax())} above {bound:.3e}; first bad row {int((err > bound).argmax())}"
        return
    rel = np.sqrt(((got - want) ** 2).sum(-1) / (want ** 2).sum(-1))
    assert np.isfinite(rel).all(), what
    over = rel > BF16_REL_L2
    assert over.sum() <= max(2, int(BF16_ROWS_OVER * rel.size)) and rel.max() <= BF16_WORST, \
        f"{what}: relative L2 error {rel.max():.3e}; {int(over.sum())} of {rel.size} rows over; first bad row {int(over.argmax())}"


def check(model_dir, seqs, got, dtype, what):
    compared = total = 0
    for rid, ids in seqs.items():
        want = LH.plain_logits(model_dir, ids)
        places = sorted(p for r, p in got if r == rid)
        assert places, f"{what}: no logits for {rid}"
        total += len(places)
        if dtype != "float32":
            unclear = np.nonzero(LH.plain_margins(model_dir, ids) < CLEAR_CHOICE)[0]
            places = [p for p in places if not unclear.size or p < unclear[0]]
            if not places:
                continue
        compared += len(places)
        close(np.stack([got[(rid, p)] for p in places]), want[places], dtype, f"{what} request {rid}")
    assert compared == total or not model_dir.endswith("_settled"), f"{what}: {total - compared} rows of a model with settled choices were not compared"


def variants(dirs, name, dtype):
    """The model's folder, and for bfloat16 also its copy with settled choices of experts."""
    return [dirs[name]] + ([dirs[name + "_settled"]] if dtype == "bfloat16" and name + "_settled" in dirs else [])


def pick(model_dir, seed, n):
    return LH.clear_tokens(model_dir, seed, n, vocab_of(model_dir), CLEAR_CHOICE)


def vocab_of(model_dir):
    with open(os.path.join(model_dir, "config.json")) as f:
        return json.load(f)["vocab"]


# ----------------------------------------------------------------------------------------------- whole models
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("kind", ["window", "chunk", "chunk_aligned", "state_space", "dense", "experts"])
def test_each_mechanism_alone(dirs, kind, dtype):
    for d in variants(dirs, kind, dtype):
        ids = pick(d, 1, 90)
        eng = make_engine(d, dtype)
        got = run_steps(eng, [([("r", ids[:61], list(range(61)))], []), ([("r", ids[61:], list(range(29)))], ["r"])])
        check(d, {"r": ids}, got, dtype, f"{kind} alone {dtype}")
        assert eng.cache.free_slots() == 4


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", NAMES)
def test_whole(dirs, name, dtype):
    for d in variants(dirs, name, dtype):
        ids = pick(d, 2, LENGTHS[name])
        eng = make_engine(d, dtype)
        got = run_steps(eng, [([("r", ids, list(range(len(ids))))], ["r"])])
        check(d, {"r": ids}, got, dtype, f"whole {name} {dtype}")
        eng.cache.check()
        assert all(eng.cache.free_pages(g) == eng.cache.pools[g].num_pages for g in range(eng.cache.n_groups))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", NAMES)
def test_bulk_then_last_tokens_one_by_one(dirs, name, dtype):
    """The decoded tokens pass every window's and several chunks' edges."""
    for d in variants(dirs, name, dtype):
        ids = pick(d, 3, LENGTHS[name])
        cut = len(ids) - 70
        steps = [([("r", ids[:cut], list(range(cut)))], [])] + [([("r", [t], [0])], []) for t in ids[cut:]]
        got = run_steps(make_engine(d, dtype), steps)
        check(d, {"r": ids}, got, dtype, f"bulk+tail {name} {dtype}")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", NAMES)
def test_changing_portions_down_to_two_tokens(dirs, name, dtype):
    """Portions shorter than the convolutions' taps, and cuts in the middle of pages, windows and chunks."""
    for d in variants(dirs, name, dtype):
        ids = pick(d, 4, LENGTHS[name])
        cuts = portions(len(ids) - 9, [7, 2, 13, 3, 2, 64, 5, 2, 17, 1, 2]) + [(len(ids) - 9 + i, len(ids) - 8 + i) for i in range(9)]
        steps = [([("r", ids[a:b], list(range(b - a)))], []) for a, b in cuts]
        got = run_steps(make_engine(d, dtype), steps)
        check(d, {"r": ids}, got, dtype, f"portions {name} {dtype}")


@pytest.mark.parametrize("name", NAMES)
def test_cutting_and_batching_change_nothing_in_32_bit(dirs, name):
    """Products add in ascending k, the attention takes keys in blocks aligned to absolute positions, the recurrence
    walks a request's tokens in order, the norms' sums depend on the row alone, and an expert's result for a row does not
    depend on which other rows the expert serves: 32-bit logits do not depend on how the prompt was cut or on what else
    was in the batch, beyond rounding."""
    d = dirs[name]
    ids = LH.tokens(5, 77, vocab_of(d))
    other = LH.tokens(6, 41, vocab_of(d))
    whole = run_steps(make_engine(d, "float32"), [([("r", ids, list(range(77)))], [])])
    eng = make_engine(d, "float32")
    steps = [([("o", other[:20], []), ("r", ids[:2], [0, 1])], []), ([("r", ids[2:50], list(range(48))), ("o", other[20:21], [])], []),
             ([("o", other[21:], []), ("r", ids[50:51], [0])], ["o"]), ([("r", ids[51:], list(range(26)))], [])]
    cut = run_steps(eng, steps)
    for p in range(77):
        assert np.abs(cut[("r", p)] - whole[("r", p)]).max() <= 4e-6 * np.abs(whole[("r", p)]).max(), p


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", NAMES)
def test_mixed_batches_with_pages_and_slots_used_again(dirs, name, dtype):
    for d in variants(dirs, name, dtype):
        rng = np.random.default_rng(7)
        seqs = {f"q{i}": pick(d, 100 + i, int(n)) for i, n in enumerate([70, 45, 90, 33, 64, 81, 50, 3, 2])}
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
    for d in variants(dirs, "A", dtype):
        ids = pick(d, 9, 300)
        steps = [([("r", ids[:5], list(range(5)))], [])] + [([("r", [t], [0])], []) for t in ids[5:]]
        got = run_steps(make_engine(d, dtype), steps)
        check(d, {"r": ids}, got, dtype, f"long decoding {dtype}")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["A", "B"])
def test_first_tokens(dirs, name, dtype):
    """Sequences of one, two, three and five tokens, side by side and one token at a time: a single visible key beside
    the sink, convolutions that reach before the sequence's start, an empty state."""
    d = variants(dirs, name, dtype)[-1]
    seqs = {f"s{n}": pick(d, 20 + n, n) for n in (1, 2, 3, 5)}
    got = run_steps(make_engine(d, dtype), [([(r, ids, list(range(len(ids)))) for r, ids in seqs.items()], list(seqs))])
    check(d, seqs, got, dtype, f"first tokens together {dtype}")
    eng = make_engine(d, dtype)
    for r, ids in seqs.items():
        got = run_steps(eng, [([(r, ids[:1], [0])], [])] + [([(r, [t], [0])], []) for t in ids[1:]])
        check(d, {r: ids}, got, dtype, f"first tokens one by one {dtype}")
        eng.release(r)


# ----------------------------------------------------------------------------------------------- kernels with made-up inputs
_alive = []


def _dev(a, dtype=torch.float32):
    """A device tensor of `a` that lives until the module is done: kernels are handed raw addresses, and a tensor that is
    made inside a call's argument list would be given back before the kernel has run."""
    t = torch.tensor(np.asarray(a), dtype=dtype, device="cuda")
    _alive.append(t)
    if len(_alive) > 4000:
        torch.cuda.synchronize()
        del _alive[:2000]
    return t


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("case", [(100, 5, 1), (100, 1, 4), (96, 8, 3), (4096, 4, 4), (48, 48, 2), (90, 5, 3), (9000, 2, 8)])
def test_norm_in_groups_alone_added_and_both(dtype, case):
    """x += norm(delta) in `gd` parts and out = norm(x) in `gn` parts, each alone and in one pass; a part whose values are
    a thousand times the others' must not change its neighbours' scale; the tail's gather of rows."""
    from gibbs_amd.ops.lib import call, dtype_code, ptr, stream
    H, gd, gn = case
    rng = np.random.default_rng(2)
    n = 7
    x0 = rng.normal(size=(n, H))
    x0[:, :H // gn] *= 1000.0
    delta = rng.normal(size=(n, H))
    delta[:, -(H // gd):] *= 1000.0
    gain_d, gain_n = rng.normal(size=H) + 1.0, rng.normal(size=H) + 1.0
    x = _dev(x0)
    dl = _dev(delta, dtype)
    out = torch.empty((n, H), dtype=dtype, device="cuda")
    call("gibbs_group_rmsnorm", ptr(x), ptr(dl), 1, n * H, ptr(_dev(gain_d)), 1e-5, gd, ptr(_dev(gain_n)), 1e-6, gn, ptr(out), dtype_code(dtype),
         None, n, H, stream())
    want_x = x0.astype(np.float32).astype(np.float64) + Z.group_rms_norm(dl.float().cpu().numpy().astype(np.float64), gain_d.astype(np.float32), 1e-5, gd)
    want_out = Z.group_rms_norm(want_x, gain_n.astype(np.float32), 1e-6, gn)
    tol = 1e-5 if dtype == torch.float32 else 1e-2
    assert np.abs(x.cpu().numpy() - want_x).max() <= 1e-5 * np.abs(want_x).max()
    assert np.abs(out.float().cpu().numpy() - want_out).max() <= tol * np.abs(want_out).max()
    # the norm alone, of chosen rows
    rows = _dev([5, 0, 5], torch.int32)
    some = torch.empty((3, H), dtype=dtype, device="cuda")
    call("gibbs_group_rmsnorm", ptr(x), None, 0, 0, None, 0.0, 0, ptr(_dev(gain_n)), 1e-6, gn, ptr(some), dtype_code(dtype), ptr(rows), 3, H, stream())
    assert np.abs(some.float().cpu().numpy() - want_out[[5, 0, 5]]).max() <= tol * np.abs(want_out).max()
    # the addition alone, from two float32 partial sums
    x2 = _dev(x0)
    halves = _dev(np.stack([delta * 0.25, delta * 0.75]))
    call("gibbs_group_rmsnorm", ptr(x2), ptr(halves), 2, n * H, ptr(_dev(gain_d)), 1e-5, gd, None, 0.0, 0, None, dtype_code(dtype), None, n, H, stream())
    want2 = x0.astype(np.float32).astype(np.float64) + Z.group_rms_norm(delta.astype(np.float32).astype(np.float64), gain_d.astype(np.float32), 1e-5, gd)
    assert np.abs(x2.cpu().numpy() - want2).max() <= 2e-5 * np.abs(want2).max()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("taps", [1, 2, 3, 5])
def test_convolution_beside_the_identity_through_short_portions_and_a_reused_slot(dtype, taps):
    """Two requests side by side in portions of 1, 2, 1, 4, ... rows (shorter than the taps), states in scattered slots;
    then a new request in a slot that was used (cleared by the caller, as the cache manager does): zeros before its start."""
    from gibbs_amd.ops.lib import call, dtype_code, ptr, stream
    rng = np.random.default_rng(3)
    C, T = 37, 23
    w = rng.normal(size=(C, taps))
    seqs = [rng.normal(size=(T, C)), rng.normal(size=(T - 5, C))]
    state = torch.zeros((4, max(taps - 1, 1), C), dtype=torch.float32, device="cuda")
    slots = [2, 0]
    got = [[], []]
    at = [0, 0]
    sizes = [1, 2, 1, 4, 1, 1, 3, 7, 2, 30]
    step = 0
    while any(at[r] < len(seqs[r]) for r in range(2)):
        rows, cu, req, live = [], [0], [], []
        for r in range(2):
            n = min(sizes[(step + r) % len(sizes)], len(seqs[r]) - at[r])
            if n <= 0:
                continue
            live.append((r, n))
            rows.append(seqs[r][at[r]:at[r] + n])
            req += [len(live) - 1] * n
            cu.append(cu[-1] + n)
        x = _dev(np.concatenate(rows), dtype)
        out = torch.empty_like(x)
        single = all(n == 1 for _, n in live)
        call("gibbs_causal_conv", ptr(x), C, dtype_code(dtype), ptr(_dev(w)), None, ptr(state), state.stride(0), ptr(_dev(req, torch.int32)),
             ptr(_dev(cu, torch.int32)), ptr(_dev([slots[r] for r, _ in live], torch.int32)), ptr(out), 0, C, x.shape[0], len(live), C, taps, 0, 1, 1,
             int(single), stream())
        o = out.float().cpu().numpy()
        for i, (r, n) in enumerate(live):
            got[r].append(o[cu[i]:cu[i + 1]])
            at[r] += n
        step += 1
    tol = 2e-5 if dtype == torch.float32 else 3e-2
    for r in range(2):
        seen = _dev(seqs[r], dtype).float().cpu().numpy().astype(np.float64)
        want = Z.input_conv(seen, w.astype(np.float32).astype(np.float64))
        assert np.abs(np.concatenate(got[r]) - want).max() <= tol * np.abs(want).max(), r
    state[2].zero_()
    x = _dev(seqs[1][:3], dtype)
    out = torch.empty_like(x)
    call("gibbs_causal_conv", ptr(x), C, dtype_code(dtype), ptr(_dev(w)), None, ptr(state), state.stride(0), ptr(_dev([0, 0, 0], torch.int32)),
         ptr(_dev([0, 3], torch.int32)), ptr(_dev([2], torch.int32)), ptr(out), 0, C, 3, 1, C, taps, 0, 1, 1, 0, stream())
    want = Z.input_conv(x.float().cpu().numpy().astype(np.float64), w.astype(np.float32).astype(np.float64))
    assert np.abs(out.float().cpu().numpy() - want).max() <= tol * np.abs(want).max()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("sizes", [(3, 3, 12, 12, 12, 6, True), (6, 2, 20, 12, 12, 10, False), (4, 2, 32, 48, 40, 16, False), (2, 1, 64, 64, 64, 64, True)])
def test_projected_rows_norm_rotation_turned_values_and_the_way_back(dtype, sizes):
    """Rows [q | k | (v) | gate]: q and k normed over the head's true size with a gain, then turned; values that are the
    keys as projected, or values of their own turned over all of their true channels (stored wider with zeros behind),
    written to their pages at positions on both sides of page borders and far out; then an output turned back and gated."""
    from gibbs_amd.ops.lib import call, dtype_code, ptr, stream
    rng = np.random.default_rng(1)
    nh, nkv, hd, vd, vt, rot, from_k = sizes
    ps = 16
    pos = _dev([0, 15, 16, 17, 31, 250, 70000], torch.int32)
    places = pos.tolist()
    n = pos.numel()
    ld = (nh + nkv) * hd + (0 if from_k else nkv * vd) + nh * vd + 3
    raw = rng.normal(size=(n, ld))
    if not from_k:                                                   # channels behind a value's true size are zeros
        v_view = raw[:, (nh + nkv) * hd:(nh + nkv) * hd + nkv * vd].reshape(n, nkv, vd)
        v_view[:, :, vt:] = 0.0
    rows = _dev(raw, dtype)
    before = rows.float().cpu().numpy().astype(np.float64)
    qg, kg = rng.normal(size=hd) + 1.0, rng.normal(size=hd) + 1.0
    inv = _dev((1000.0 ** (-2.0 * np.arange(rot // 2) / rot)).astype(np.float32))
    v_inv = None if from_k else _dev((1000.0 ** (-2.0 * np.arange(vt // 2) / vt)).astype(np.float32))
    n_pages = 70000 // ps + 1
    kpages = torch.zeros((n_pages, nkv, ps, hd), dtype=dtype, device="cuda")
    vpages = torch.zeros((n_pages, nkv, ps, vd), dtype=dtype, device="cuda")
    table = torch.arange(n_pages - 1, -1, -1, dtype=torch.int32, device="cuda").view(1, n_pages).contiguous()
    req = torch.zeros(n, dtype=torch.int32, device="cuda")
    call("gibbs_qkv_prepare_full", ptr(rows), ld, ptr(kpages), ptr(vpages), dtype_code(dtype), None, ptr(inv), rot, 0, None, 0, None, 0, vt, None,
         ptr(pos), ptr(req), ptr(table), n_pages, ps, n_pages, n, nh, nkv, hd, vd, ptr(_dev(qg)), ptr(_dev(kg)), 1e-5, hd, int(from_k),
         ptr(v_inv), vt, stream())
    tol = 1e-5 if dtype == torch.float32 else 4e-2
    qg32, kg32 = qg.astype(np.float32).astype(np.float64), kg.astype(np.float32).astype(np.float64)
    q0 = before[:, :nh * hd].reshape(n, nh, hd)
    k0 = before[:, nh * hd:(nh + nkv) * hd].reshape(n, nkv, hd)
    q = Z.rotate(Z.group_rms_norm(q0, qg32, 1e-5, 1), places, 1000.0, rot)
    k = Z.rotate(Z.group_rms_norm(k0, kg32, 1e-5, 1), places, 1000.0, rot)
    if from_k:
        v = k0[:, :, :vd]
    else:
        v = before[:, (nh + nkv) * hd:(nh + nkv) * hd + nkv * vd].reshape(n, nkv, vd).copy()
        v[:, :, :vt] = Z.rotate(v[:, :, :vt], places, 1000.0, vt)
    after = rows.float().cpu().numpy()
    assert np.abs(after[:, :nh * hd].reshape(n, nh, hd) - q).max() <= tol * 4
    assert np.array_equal(after[:, -3:], before[:, -3:].astype(np.float32))
    for i, p in enumerate(places):
        page = n_pages - 1 - p // ps
        assert np.abs(kpages[page, :, p % ps].float().cpu().numpy() - k[i]).max() <= tol * 4, p
        assert np.abs(vpages[page, :, p % ps].float().cpu().numpy() - v[i]).max() <= tol * 4, p
    assert int((kpages != 0).any(-1).sum()) == n * nkv            # nothing else was written
    # the way back: an output turned by minus its position, then gated (the gate's columns are the row's last nh * vd + 3)
    att0 = rng.normal(size=(n, nh, vd))
    att = _dev(att0.reshape(n, nh * vd), dtype)
    gate_off = ld - 3 - nh * vd
    call("gibbs_attention_finish", ptr(att), nh * vd, rows.data_ptr() + gate_off * rows.element_size(), ld, vd, dtype_code(dtype), ptr(pos),
         ptr(v_inv), vt, 0, n, nh, vd, vt, stream())
    a64 = att0.astype(np.float32).astype(np.float64) if dtype == torch.float32 else _dev(att0, dtype).float().cpu().numpy().astype(np.float64)
    want = a64.copy()
    if not from_k:
        want[:, :, :vt] = Z.rotate(a64[:, :, :vt], places, 1000.0, vt, sign=-1.0)
    gate = before[:, gate_off:gate_off + nh * vd].reshape(n, nh, vd)
    want[:, :, :vt] = want[:, :, :vt] * Z.sigmoid(gate[:, :, :vt])
    assert np.abs(att.float().cpu().numpy().reshape(n, nh, vd) - want).max() <= tol * 4


@pytest.mark.parametrize("kernel", ["plain32", "plain16", "decode", "decode_lanes", "prefill"])
@pytest.mark.parametrize("mask", ["window", "chunk"])
def test_keys_just_inside_and_just_outside_a_window_and_a_chunk(kernel, mask):
    """Four query heads over two kv heads, pages of 16 scattered over the pool, 700 keys.  One key is made to dominate head 2:
    where the mask lets the last row see it (the window's first key, the chunk's first key, a page's border, the row itself) the
    head's output is that key's value, one key earlier it is not; a zero sink takes its share; capped scores."""
    from gibbs_amd import ops
    rng = np.random.default_rng(0)
    dtype = torch.float32 if kernel == "plain32" else torch.bfloat16
    tol = 3e-5 if kernel == "plain32" else 3e-2
    T, nh, nkv, hd, ps, n_pages = 700, 4, 2, 32, 16, 64
    size = 75 if mask == "window" else 180
    p = T - 1
    first_seen = p - size + 1 if mask == "window" else p - p % size
    order = rng.permutation(n_pages)[:-(-T // ps)].tolist()
    table = _dev([order], torch.int32)
    keys = _dev(rng.normal(size=(T, nkv, hd)) * 0.1, dtype)
    vals = _dev(rng.normal(size=(T, nkv, hd)), dtype)
    q = _dev(rng.normal(size=(1, nh * hd)) * 0.1, dtype)
    qh = q.float().cpu().numpy().reshape(nh, hd).astype(np.float64)
    softcap = 20.0
    sink = _dev(np.zeros(nh))

    def pages_of(rows):
        pages = torch.full((n_pages, nkv, ps, rows.shape[-1]), 7.0, dtype=dtype, device="cuda")
        for t in range(T):
            pages[order[t // ps], :, t % ps] = rows[t]
        return pages

    kw = {"window": size} if mask == "window" else {"chunk": size}

    def run(k_rows):
        kp, vp = pages_of(k_rows), pages_of(vals)
        pos, req = _dev([p], torch.int32), torch.zeros(1, dtype=torch.int32, device="cuda")
        if kernel.startswith("plain"):
            out = ops.attention_plain(q, 1, nh, nkv, hd, kp, vp, table, 1, pos, req, 1.0, sink=sink, softcap=softcap, **kw)
        elif kernel.startswith("decode"):
            out = ops.attention_decode(q, 1, nh, nkv, hd, kp, vp, table, 1, pos, req, 1.0, max_seq=T, n_splits=3, sink=sink, softcap=softcap,
                                       kind="valu" if kernel == "decode_lanes" else "auto", **kw)
        else:
            n = 40
            qs = torch.zeros((n, nh * hd), dtype=dtype, device="cuda")
            qs[-1] = q[0]
            out = ops.attention_prefill(qs, n, nh, nkv, hd, kp, vp, table, 1, _dev([0, n], torch.int32), _dev([T - n], torch.int32), 1.0,
                                        max_seq=T, sink=sink, softcap=softcap, **kw)[-1:]
        return out.float().cpu().numpy().reshape(nh, hd)

    def want(k_rows):
        kk, vv = k_rows.float().cpu().numpy().astype(np.float64), vals.float().cpu().numpy().astype(np.float64)
        visible = Z.visible_window(T, size) if mask == "window" else Z.visible_chunk(T, size)
        return Z.masked_attention(np.repeat(qh[None], T, 0), kk, vv, 1.0, visible, sink=np.zeros(nh), softcap=softcap)[-1]

    for far in (first_seen - 1, first_seen, first_seen + 1, (first_seen // ps + 1) * ps, (first_seen // ps + 1) * ps - 1, p):
        k_rows = keys.clone()
        k_rows[far, 1] = (q[0, 2 * hd:3 * hd].float() / q[0, 2 * hd:3 * hd].float().norm() ** 2 * 14.0).to(dtype)    # head 2: q . k = 14
        got = run(k_rows)
        assert np.abs(got - want(k_rows)).max() <= tol * 4, far
        hit = np.abs(got[2] - vals[far, 1].float().cpu().numpy()).max() < 0.2
        assert hit == (far >= first_seen), f"head 2 and the key at {far} (the first key seen is {first_seen})"


@pytest.mark.parametrize("sizes", [(3, 3, 7, 10), (4, 2, 40, 56), (2, 1, 128, 64), (8, 2, 16, 24), (2, 1, 200, 8)])
def test_state_written_long_ago_read_back_through_portions_and_a_reused_slot(sizes):
    """The state-space rule alone: one token's write (all other tokens' B are zero, decays of nearly one) is read back 400
    tokens later by a C that matches it, through portions of 1 to 150 tokens; the same walk in one step gives the same
    bits; a second request in another slot does not see it, and a slot that is cleared starts from zero."""
    from gibbs_amd.ops.lib import call, ptr, stream
    H, G, D, V = sizes
    rng = np.random.default_rng(4)
    T = 420
    B = np.zeros((T, G, D)); C = np.zeros((T, G, D))
    x = rng.normal(size=(T, H, V)); dt = np.full((T, H), 0.5)
    mark = rng.normal(size=D); mark /= np.linalg.norm(mark)
    B[10, :] = mark
    C[410, :] = mark
    B[11:400:7] = rng.normal(size=(len(range(11, 400, 7)), G, D)) * 0.01
    a_log = np.full(H, -9.0)                                         # decay exp(-exp(-9) * 0.5) a token: nearly one
    decay = np.exp(-np.exp(a_log)[None, :] * dt)
    want = Z.ssd_scan(x, B, C, dt, a_log, np.zeros(H), G)

    def run(cuts, slot, state):
        outs = []
        for a, b in cuts:
            n = b - a
            bc = _dev(np.concatenate([B[a:b].reshape(n, -1), C[a:b].reshape(n, -1)], axis=1))
            xdt = _dev((x[a:b] * dt[a:b, :, None]).reshape(n, -1))
            o = torch.empty((n, H * V), dtype=torch.float32, device="cuda")
            call("gibbs_ssd_rule", bc.data_ptr() + G * D * 4, ptr(bc), 2 * G * D, ptr(xdt), H * V, ptr(_dev(decay[a:b])), ptr(state), state.stride(0),
                 ptr(_dev([0, n], torch.int32)), ptr(_dev([slot], torch.int32)), ptr(o), 1, H, G, D, V, stream())
            outs.append(o.cpu().numpy())
        return np.concatenate(outs)

    state = torch.zeros((3, H * D * V), dtype=torch.float32, device="cuda")
    whole = run([(0, T)], 1, state)
    assert np.abs(whole.reshape(T, H, V) - want).max() <= 2e-5 * np.abs(want).max()
    assert np.abs(want[410]).max() > 0.1 and np.abs(whole.reshape(T, H, V)[410] - want[410]).max() <= 1e-4 * np.abs(want[410]).max()
    cuts, at = [], 0
    for s in [1, 2, 150, 3, 1, 1, 64, 9, 100, 2, 500]:
        if at >= T:
            break
        cuts.append((at, min(T, at + s)))
        at = cuts[-1][1]
    state2 = torch.zeros_like(state)
    assert np.array_equal(run(cuts, 2, state2), whole)
    assert torch.equal(state2[2], state[1]) and not state2[0].any() and not state2[1].any()
    state2[2].zero_()
    assert np.array_equal(run([(0, 30)], 2, state2), whole[:30])


@pytest.mark.parametrize("case", [(torch.float32, 52, 5, 2, 3, 100, 30, True), (torch.bfloat16, 52, 5, 2, 3, 100, 30, True),
                                  (torch.bfloat16, 300, 8, 0, 2, 128, 64, False), (torch.float32, 40, 2, 3, 5, 24, 8, True),
                                  (torch.bfloat16, 9, 16, 1, 4, 64, 32, True), (torch.bfloat16, 1200, 4, 2, 2, 64, 32, False)])
def test_scores_over_all_experts_corrections_identity_experts_and_the_sum(case):
    """Scores by a softmax over all router outputs, the choice by score + correction (made so that it differs from the
    choice by score alone), weights from the scores without it; identity experts among the chosen; both products and the
    weighted sum with a shared expert that has no gate, against the plain functions."""
    from gibbs_amd.ops.lib import call, dtype_code, library, ptr, stream
    dtype, n, E, ident, top, W, F, with_shared = case
    R = E + ident
    rng = np.random.default_rng(3)
    h = _dev(rng.normal(size=(n, W)), dtype)
    router = _dev(rng.normal(size=(R, W)) * 0.3)
    corr = rng.normal(size=R) * 0.5
    corr[-1] += 0.7                                               # the last output (an identity expert, if any) is chosen often
    corr = _dev(corr)
    gate, up, down = _dev(rng.normal(size=(E, F, W)) * 0.1, dtype), _dev(rng.normal(size=(E, F, W)) * 0.1, dtype), _dev(rng.normal(size=(E, W, F)) * 0.1, dtype)
    chosen = torch.empty((n, top), dtype=torch.int32, device="cuda")
    weight = torch.empty((n, top), dtype=torch.float32, device="cuda")
    call("gibbs_moe_route_mode", ptr(h), W, dtype_code(dtype), ptr(router), ptr(corr), None, ptr(chosen), ptr(weight), None, n, W, R, top, 1, stream())
    hh = h.float().cpu().numpy().astype(np.float64)
    r64, c64 = router.cpu().numpy().astype(np.float64), corr.cpu().numpy().astype(np.float64)
    want_c, want_w = Z.route(hh, r64, c64, top)
    sure = Z.route_margin(hh, r64, c64, top) > 1e-4
    plain_c, _ = Z.route(hh, r64, np.zeros(R), top)
    assert top == R or (np.sort(want_c, -1) != np.sort(plain_c, -1)).any(), "the correction must change some choice"
    got_c, got_w = chosen.cpu().numpy(), weight.cpu().numpy()
    assert sure.sum() >= 0.9 * n
    assert np.array_equal(got_c[sure], want_c[sure])
    assert np.abs(got_w[sure] - want_w[sure]).max() <= 2e-5
    assert ident == 0 or (got_c >= E).any()
    lib = library()
    pairs = n * top
    bm = lib.gibbs_moe_tile(pairs, E)
    cap = lib.gibbs_moe_capacity(pairs, E, bm)
    sorted_pair = torch.empty(cap, dtype=torch.int32, device="cuda")
    place = torch.empty(pairs, dtype=torch.int32, device="cuda")
    tile_expert = torch.empty(cap // bm, dtype=torch.int32, device="cuda")
    call("gibbs_moe_group", ptr(chosen), pairs, E, bm, ptr(sorted_pair), ptr(place), ptr(tile_expert), cap, stream())
    assert np.array_equal(place.cpu().numpy() < 0, got_c.reshape(-1) >= E)
    mid = torch.zeros((cap, F), dtype=dtype, device="cuda")
    y = torch.zeros((cap, W), dtype=dtype, device="cuda")
    call("gibbs_moe_gemm", ptr(h), W, top, ptr(sorted_pair), ptr(tile_expert), cap, bm, ptr(gate), ptr(up), ptr(mid), F, dtype_code(dtype), F, W, 0, stream())
    call("gibbs_moe_gemm", ptr(mid), F, 0, ptr(sorted_pair), ptr(tile_expert), cap, bm, ptr(down), None, ptr(y), W, dtype_code(dtype), W, F, 0, stream())
    shared = _dev(rng.normal(size=(n, W)), dtype) if with_shared else None
    out = torch.empty((n, W), dtype=dtype, device="cuda")
    call("gibbs_moe_combine_self", ptr(y), ptr(place), ptr(weight), ptr(shared), None, ptr(h), ptr(out), dtype_code(dtype), n, top, W, stream())
    g64, u64, d64 = (t.float().cpu().numpy().astype(np.float64) for t in (gate, up, down))
    want = np.zeros((n, W))
    for i in range(n):
        for e, wt in zip(got_c[i], got_w[i].astype(np.float64)):
            want[i] += wt * (hh[i] if e >= E else Z.gated_ff(hh[i:i + 1], g64[e], u64[e], d64[e])[0])
    if with_shared:
        want += shared.float().cpu().numpy().astype(np.float64)
    tol = 2e-5 if dtype == torch.float32 else 3e-2
    assert np.abs(out.float().cpu().numpy() - want).max() <= tol * np.abs(want).max()


@pytest.mark.parametrize("sizes", [(3, 3, 7, 10), (4, 2, 40, 56), (2, 1, 200, 72), (8, 2, 128, 64)])
def test_one_token_per_request_against_the_walk(sizes):
    """Three requests that bring one token each, for 20 steps, through the kernel for such steps and through the walk: the
    states are equal to the bit (the same arithmetic per element), the read-outs to rounding; slots are scattered."""
    from gibbs_amd.ops.lib import call, ptr, stream
    H, G, D, V = sizes
    rng = np.random.default_rng(8)
    R, steps = 3, 20
    slots = _dev([2, 0, 3], torch.int32)
    cu = _dev([0, 1, 2, 3], torch.int32)
    state_a = _dev(rng.normal(size=(5, H * D * V + 3)))
    state_b = state_a.clone()
    for _ in range(steps):
        bc = _dev(rng.normal(size=(R, 2 * G * D)))
        xdt = _dev(rng.normal(size=(R, H * V)))
        decay = _dev(rng.uniform(0.2, 1.0, size=(R, H)))
        out_a = torch.empty((R, H * V), dtype=torch.float32, device="cuda")
        out_b = torch.empty_like(out_a)
        call("gibbs_ssd_rule", bc.data_ptr() + G * D * 4, ptr(bc), 2 * G * D, ptr(xdt), H * V, ptr(decay), ptr(state_a), state_a.stride(0), ptr(cu), ptr(slots),
             ptr(out_a), R, H, G, D, V, stream())
        call("gibbs_ssd_step", bc.data_ptr() + G * D * 4, ptr(bc), 2 * G * D, ptr(xdt), H * V, ptr(decay), ptr(state_b), state_b.stride(0), ptr(slots),
             ptr(out_b), R, H, G, D, V, stream())
        assert torch.equal(state_a, state_b)
        assert (out_a - out_b).abs().max() <= 2e-5 * out_a.abs().max()
    assert torch.equal(state_a[1], state_b[1]) and torch.equal(state_a[4], state_b[4])      # slots of no request are untouched


@pytest.mark.parametrize("sizes", [(3, 3, 8, 12, 300), (4, 2, 40, 56, 257), (2, 1, 128, 64, 640), (2, 2, 20, 100, 450), (1, 1, 4, 4, 64)])
def test_the_rule_in_chunks_against_the_walk(sizes):
    """One request's long stretch of rows through the rule in chunks of 64 tokens (sizes that are no multiples of 64,
    more columns than a workgroup takes, a last chunk that is not full), from a state that an earlier call left: the plain
    recurrence's read-outs and state, and the token-by-token kernel's, to rounding; decays from nearly one down to 1e-4 a token."""
    from gibbs_amd.ops.lib import call, library, ptr, stream
    H, G, D, V, T = sizes
    rng = np.random.default_rng(6)
    first = 37
    n = first + T
    B, C, x = rng.normal(size=(n, G, D)), rng.normal(size=(n, G, D)), rng.normal(size=(n, H, V))
    dt = rng.uniform(0.05, 1.5, size=(n, H))
    a_log = np.linspace(-6.0, 1.8, H)
    log_decay = -np.exp(a_log)[None, :] * dt
    want = Z.ssd_scan(x, B, C, dt, a_log, np.zeros(H), G)
    bc = _dev(np.concatenate([B.reshape(n, -1), C.reshape(n, -1)], axis=1))
    xdt = _dev((x * dt[:, :, None]).reshape(n, -1))
    decay, logd = _dev(np.exp(log_decay)), _dev(log_decay)
    slot = _dev([1], torch.int32)

    def walk(state, a, b, out):
        call("gibbs_ssd_rule", bc[a:b].data_ptr() + G * D * 4, bc[a:b].data_ptr(), 2 * G * D, xdt[a:b].data_ptr(), H * V, decay[a:b].data_ptr(), ptr(state),
             state.stride(0), ptr(_dev([0, b - a], torch.int32)), ptr(slot), out[a:b].data_ptr(), 1, H, G, D, V, stream())

    state_w = torch.zeros((3, H * D * V + 5), dtype=torch.float32, device="cuda")
    out_w = torch.zeros((n, H * V), dtype=torch.float32, device="cuda")
    walk(state_w, 0, first, out_w)
    state_c = state_w.clone()
    out_c = out_w.clone()
    walk(state_w, first, n, out_w)
    floats = library().gibbs_ssd_chunked_workspace(T, H, D, V)
    assert floats > 0
    work = torch.full((floats,), float("nan"), dtype=torch.float32, device="cuda")
    call("gibbs_ssd_chunked", bc[first:].data_ptr() + G * D * 4, bc[first:].data_ptr(), 2 * G * D, xdt[first:].data_ptr(), H * V, logd[first:].data_ptr(),
         ptr(state_c), state_c.stride(0), ptr(slot), out_c[first:].data_ptr(), ptr(work), T, H, G, D, V, stream())
    scale = np.abs(want).max()
    assert np.abs(out_w.cpu().numpy().reshape(n, H, V) - want).max() <= 3e-5 * scale
    assert np.abs(out_c.cpu().numpy().reshape(n, H, V) - want).max() <= 3e-5 * scale
    assert torch.isfinite(state_c).all() and (state_c[1] - state_w[1]).abs().max() <= 3e-5 * state_w[1].abs().max()
    assert not state_c[0].any() and not state_c[2].any() and not state_c[1, H * D * V:].any()


@pytest.mark.parametrize("dtype", DTYPES)
def test_a_long_prompt_whole_in_portions_and_decoded(dirs, dtype, tmp_path):
    """A prompt long enough for the state-space rule's chunks (600 tokens in one step), the same prompt in portions that are
    too short for them, and its last tokens one by one: all against the plain logits."""
    cfg = {"architecture": "Litizen", "vocab": 150, "width": 64, "norm": {"eps": 1e-5, "groups": 2}, "canon": {"taps": 3},
           "layers": [LH.with_mlp(LH.state_space(4, 16, 24, 2, 4, 2), LH.dense(96)), LH.with_mlp(LH.chunk_attention(4, 2, 16, 16, 0.25, 1e4, dims=8, size=150), None),
                      LH.with_mlp(LH.state_space(3, 8, 128, 1, 2, 1), LH.dense(64))]}
    d = LH.make_model_dir(str(tmp_path), cfg, "long", seed=12)
    ids = LH.tokens(8, 600, 150)
    want = [0, 63, 64, 255, 256, 300, 511, 512, 598, 599]
    whole = run_steps(make_engine(d, dtype), [([("r", ids, want)], ["r"])])
    check(d, {"r": ids}, whole, dtype, f"long prompt whole {dtype}")
    cuts = portions(560, [200, 90, 255, 15]) + [(560 + i, 561 + i) for i in range(40)]
    cut = run_steps(make_engine(d, dtype), [([("r", ids[a:b], [p - a for p in want if a <= p < b])], []) for a, b in cuts])
    check(d, {"r": ids}, cut, dtype, f"long prompt in portions {dtype}")
    assert sorted(cut) == sorted(whole)


# ----------------------------------------------------------------------------------------------- entry points
def plain_greedy(model_dir, prompt, n):
    ids = list(prompt)
    for _ in range(n):
        ids.append(int(np.argmax(LH.plain_logits(model_dir, ids)[-1])))
    return ids[len(prompt):]


@pytest.mark.parametrize("dtype", DTYPES)
def test_greedy_generation_through_the_scheduler(dirs, dtype):
    """`generate` (scheduler, prompt steps, bursts of captured decode steps) gives the plain implementation's greedy
    tokens; in bfloat16 wherever the plain logits' lead exceeds the precision's error."""
    from gibbs_amd import Engine, generate
    held = 0
    for name, lens in (("A", [7, 13, 2]), ("D", [5])):
        d = dirs[name]
        eng = Engine(d, dtype=dtype, max_tokens=512, max_requests=4)
        prompts = [LH.tokens(40 + i, n, vocab_of(d)) for i, n in enumerate(lens)]
        outs = generate(eng, prompts, max_tokens=20, temperature=0.0, ignore_eos=True)
        for p, o in zip(prompts, outs):
            assert o.finish_reason == "length" and len(o.tokens) == 20
            if dtype == "float32":
                assert o.tokens == plain_greedy(d, p, 20)
                held += 20
                continue
            logits = LH.plain_logits(d, list(p) + list(o.tokens))
            for i, t in enumerate(o.tokens):
                row = logits[len(p) - 1 + i]
                best, second = np.sort(row)[[-1, -2]]
                margin = 2 * 0.05 * np.abs(row).max()
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
    prompts = [LH.tokens(70 + i, n, vocab_of(d)) for i, n in enumerate([9, 21, 5])]
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
    d = dirs["C"]                  # (every router output is chosen there: no choice can fall the other way)
    ids = pick(d, 50, 40)
    other = pick(d, 51, 9)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": ids[:17], "want": [0, 16]}, {"id": "b", "tokens": other[:2], "want": []}], "end": []},
             {"step": 1, "entries": [{"id": "b", "tokens": other[2:], "want": [6]}], "end": ["b"]},
             {"step": 2, "entries": [{"id": "a", "tokens": ids[17:39], "want": [21]}], "end": []},
             {"step": 3, "entries": [{"id": "a", "tokens": ids[39:], "want": [0]}], "end": ["a"]}]
    out = tmp_path / "out"
    proc = subprocess.run([os.path.join(ROOT, "bin", "trace_run"), "--model", d, "--dtype", dtype, "--out", str(out), "--max-tokens", "128"],
                          input="\n".join(json.dumps(s) for s in steps) + "\n", capture_output=True, text=True, timeout=600)
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert [l for l in proc.stdout.splitlines() if l.startswith("done")] == [f"done {i}" for i in range(4)]
    want_a, want_b = LH.plain_logits(d, ids), LH.plain_logits(d, other)
    read = lambda i: np.fromfile(out / f"{i}.f32", dtype="<f4").reshape(-1, vocab_of(d))
    close(read(0), want_a[[0, 16]], dtype, "step 0")
    close(read(1), want_b[[8]], dtype, "step 1")
    close(read(2), want_a[[38]], dtype, "step 2")
    close(read(3), want_a[[39]], dtype, "step 3")


def test_command_line(dirs):
    d = dirs["A"]
    prompt = LH.tokens(60, 6, vocab_of(d))
    proc = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "gibbs"), "--model", d, "--dtype", "float32", "--prompt-ids",
                           ",".join(map(str, prompt)), "--max-tokens", "8", "--temperature", "0", "--ignore-eos"],
                          capture_output=True, text=True, timeout=600)
    assert proc.returncode == 0, proc.stderr[-2000:]
    line = proc.stdout.split("✨ Output:\n")[1].splitlines()[0]
    assert [int(t) for t in line.split()] == plain_greedy(d, prompt, 8)
    proc = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "gibbs"), "--model", d, "--arch-dump"], capture_output=True, text=True, timeout=600)
    dump = json.loads(proc.stdout)
    assert dump["architecture"] == "Litizen" and dump["unconsumed"] == [] and dump["missing"] == []
    assert dump["derived"]["layers_by_type"] == {"attention": 1, "attention_2": 1, "mamba2": 2}
