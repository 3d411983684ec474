"""Pins the CPU oracle (oracle/moe_oracle.c) with checks that do not retype its formulas:
library routines (numpy fp64 matmul, scipy softmax, numpy stable argsort, torch.ldexp, glibc qsort),
exact rational arithmetic, closed-form special cases and integer invariants.  CPU only."""
import os

import numpy as np
import pytest
import scipy.special

from conftest import GOLDEN


def bf16_round(oracle, a):
    return oracle.bf16_to_f32(oracle.f32_to_bf16(np.asarray(a, dtype=np.float32)))


# ---- matmul: src/run.cpp:341-354 -----------------------------------------------------------------
def test_matmul_matches_fp64_library_gemv(oracle):
    rng = np.random.default_rng(0)
    for n, d in [(1, 1), (7, 3), (64, 33), (2880, 32), (2880, 257)]:
        x = rng.standard_normal(n).astype(np.float32)
        w = bf16_round(oracle, rng.standard_normal((d, n)) * 0.02)
        got = oracle.matmul(x, w)
        # float products widened to double, summed by the library in fp64, rounded once
        want = (w * x[None, :]).astype(np.float64).sum(axis=1)
        assert got.dtype == np.float32
        np.testing.assert_allclose(got, want, rtol=2e-7, atol=1e-30)


def test_matmul_product_is_rounded_to_fp32_before_widening(oracle):
    # (1 + 2^-12)^2 = 1 + 2^-11 + 2^-24: an fp32 multiply drops the last term, an fp64 multiply keeps
    # it.  4096 such products minus 4098 leave exactly 0 in the first case and 2^-12 in the second.
    a = np.float32(1 + 2.0 ** -12)
    n = 1 << 12
    x = np.concatenate([np.full(n, a, dtype=np.float32), [np.float32(1.0)]])
    w = np.concatenate([np.full(n, a, dtype=np.float32), [np.float32(-4098.0)]])[None, :]
    assert np.float64(a) * np.float64(a) * n - 4098.0 == 2.0 ** -12
    assert oracle.matmul(x, w)[0] == 0.0


def test_matmul_accumulates_in_fp64(oracle):
    # 1 + 2^-30 + ... : fp32 accumulation would drop every small term
    n = 1025
    x = np.ones(n, dtype=np.float32)
    w = np.full((1, n), 2.0 ** -30, dtype=np.float32)
    w[0, 0] = 1.0
    got = oracle.matmul(x, w)[0]
    assert got == np.float32(1.0 + 1024 * 2.0 ** -30)
    assert got != np.float32(1.0)


def test_matmul_one_hot_and_zero(oracle):
    rng = np.random.default_rng(1)
    w = rng.standard_normal((9, 40)).astype(np.float32)
    assert np.array_equal(oracle.matmul(np.zeros(40, np.float32), w), np.zeros(9, np.float32))
    for k in (0, 17, 39):
        x = np.zeros(40, np.float32)
        x[k] = 1.0
        assert np.array_equal(oracle.matmul(x, w), w[:, k])


def test_matmul_is_not_transposed(oracle):
    w = np.arange(6, dtype=np.float32).reshape(2, 3)  # (out=2, in=3)
    x = np.array([1, 10, 100], dtype=np.float32)
    assert np.array_equal(oracle.matmul(x, w), np.array([210, 543], dtype=np.float32))


# ---- top-k: src/run.cpp:357-404 ------------------------------------------------------------------
def test_topk_matches_stable_argsort(oracle):
    rng = np.random.default_rng(2)
    for E, K in [(4, 1), (32, 4), (128, 4), (7, 7), (1024, 8)]:
        for _ in range(20):
            s = rng.standard_normal(E).astype(np.float32)
            v, i = oracle.topk(s, K)
            want = np.argsort(-s, kind="stable")[:K]
            assert np.array_equal(i, want)
            assert np.array_equal(v, s[want])


def test_topk_ties_keep_lower_index_first(oracle):
    s = np.array([1, 5, 5, 3, 5, 3, 0, 5], dtype=np.float32)
    v, i = oracle.topk(s, 6)
    assert i.tolist() == [1, 2, 4, 7, 3, 5]
    assert v.tolist() == [5, 5, 5, 5, 3, 3]
    v, i = oracle.topk(np.zeros(32, np.float32), 4)
    assert i.tolist() == [0, 1, 2, 3]
    s = np.array([0.0, -0.0, 0.0, -0.0], dtype=np.float32)  # signed zeros compare equal
    assert oracle.topk(s, 4)[1].tolist() == [0, 1, 2, 3]


def test_topk_agrees_with_glibc_qsort(oracle):
    """The reference sorts with qsort(3); on this libc that is a stable merge sort, so the
    explicit stable rule gives the same order, ties included."""
    rng = np.random.default_rng(3)
    for E in (32, 128):
        for _ in range(200):
            s = rng.integers(-3, 4, size=E).astype(np.float32)  # many ties
            assert np.array_equal(oracle.topk(s, 4)[1], oracle.topk(s, 4, use_qsort=True)[1])
            assert np.array_equal(oracle.topk(s, E)[1], oracle.topk(s, E, use_qsort=True)[1])


def test_topk_rejects_bad_arguments(oracle):
    with pytest.raises(ValueError):
        oracle.topk(np.zeros(4, np.float32), 5)


# ---- softmax: src/run.cpp:321-339 ----------------------------------------------------------------
def test_softmax_matches_scipy(oracle):
    rng = np.random.default_rng(4)
    for size in (1, 2, 4, 8, 33):
        x = (rng.standard_normal(size) * 3).astype(np.float32)
        got = oracle.softmax(x)
        want = scipy.special.softmax(x.astype(np.float64))
        # x - max is rounded to fp32 before expf: |x - max| * 2^-24 of relative error on top of the final rounding
        np.testing.assert_allclose(got, want, rtol=2e-6)
        assert abs(got.astype(np.float64).sum() - 1) < 1e-6
        assert np.array_equal(np.argsort(-got, kind="stable"), np.argsort(-x, kind="stable"))
    assert np.array_equal(oracle.softmax(np.array([3.0], np.float32)), np.array([1.0], np.float32))
    np.testing.assert_array_equal(oracle.softmax(np.full(4, 1000.0, np.float32)), np.full(4, 0.25, np.float32))


# ---- SwiGLU: src/run.cpp:666-689 -----------------------------------------------------------------
def test_swiglu_special_cases(oracle):
    def one(g, u, lim=7.0):
        return float(oracle.swiglu(np.array([g, u], np.float32), lim)[0])

    sig = lambda z: 1.0 / (1.0 + np.exp(-z))
    assert one(0.0, 3.0) == 0.0                       # g = 0
    assert one(2.0, -1.0) == 0.0                      # u = -1
    assert one(100.0, 1.0) == pytest.approx(7.0 * sig(1.702 * 7.0) * 2.0, rel=1e-6)   # gate clamps at +7
    assert one(3.0, 50.0) == pytest.approx(3.0 * sig(1.702 * 3.0) * 8.0, rel=1e-6)    # up clamps at +7
    assert one(3.0, -50.0) == pytest.approx(3.0 * sig(1.702 * 3.0) * -6.0, rel=1e-6)  # up clamps at -7
    assert one(-60.0, 2.0) == pytest.approx(0.0, abs=1e-30)  # no lower clamp on gate: g*sigmoid -> 0
    assert one(-8.0, 1.0) == pytest.approx(-8.0 * sig(1.702 * -8.0) * 2.0, rel=1e-5)  # gate NOT clamped at -7
    assert one(1.0, 0.0) == pytest.approx(sig(1.702), rel=1e-6)


def test_swiglu_deinterleaves_gate_even_up_odd(oracle):
    rng = np.random.default_rng(5)
    I = 16
    m = rng.standard_normal(2 * I).astype(np.float32)
    g = np.minimum(m[0::2].astype(np.float64), 7.0)
    u = np.clip(m[1::2].astype(np.float64), -7.0, 7.0)
    want = g / (1 + np.exp(-1.702 * g)) * (u + 1)
    np.testing.assert_allclose(oracle.swiglu(m), want, rtol=2e-6, atol=1e-7)


# ---- rmsnorm: src/run.cpp:306-319 ----------------------------------------------------------------
def test_rmsnorm_matches_fp64(oracle):
    rng = np.random.default_rng(6)
    x = rng.standard_normal(2880).astype(np.float32) * 3
    w = bf16_round(oracle, 1 + 0.1 * rng.standard_normal(2880))
    want = w * x.astype(np.float64) / np.sqrt((x.astype(np.float64) ** 2).mean() + 1e-5)
    np.testing.assert_allclose(oracle.rmsnorm(x, w), want, rtol=3e-7)
    np.testing.assert_array_equal(oracle.rmsnorm(np.zeros(8, np.float32), np.ones(8, np.float32)), np.zeros(8))


# ---- MXFP4 dequant: export_model_bin.py:75-133 ---------------------------------------------------
def test_dequant_exhaustive_against_exact_rationals(oracle):
    table = np.load(os.path.join(GOLDEN, "mxfp4_table.npy"))
    got = np.array([[oracle.mxfp4_to_bf16_bits(c, s) for s in range(256)] for c in range(16)], dtype=np.uint16)
    assert np.array_equal(got, table)


def test_dequant_exhaustive_against_torch_ldexp():
    """The reference computes lut[idx] then torch.ldexp(sub, exp, out=sub) on bf16
    (export_model_bin.py:122-129); run that library routine on every (code, scale) pair."""
    import torch
    table = np.load(os.path.join(GOLDEN, "mxfp4_table.npy"))
    lut = torch.tensor([0, .5, 1, 1.5, 2, 3, 4, 6, -0., -.5, -1, -1.5, -2, -3, -4, -6], dtype=torch.bfloat16)
    for s in range(256):
        col = lut.clone()
        torch.ldexp(col, torch.full((16,), s - 127, dtype=torch.int32), out=col)
        bits = col.view(torch.int16).numpy().view(np.uint16)
        nan = np.isnan(col.float().numpy())
        assert np.array_equal(bits[~nan], table[:, s][~nan]), s
        assert np.all((table[:, s][nan] & 0x7FFF) > 0x7F80)


def test_dequant_nibble_and_block_order(oracle):
    # byte b of a block holds element 2b in its low nibble and 2b+1 in its high nibble; blocks follow
    # each other along the row (export_model_bin.py:122-127, 133)
    blocks = np.zeros((1, 2, 16), dtype=np.uint8)
    scales = np.array([[127, 128]], dtype=np.uint8)
    blocks[0, 0, 0] = 0x42   # element 0 = code 2 (1.0), element 1 = code 4 (2.0)
    blocks[0, 0, 15] = 0xF1  # element 30 = code 1 (0.5), element 31 = code 15 (-6.0)
    blocks[0, 1, 1] = 0x07   # second block, element 2 = code 7 (6.0) * 2^1, element 3 = 0
    out = oracle.bf16_to_f32(oracle.dequant_mxfp4(blocks, scales))[0]
    want = np.zeros(64, np.float32)
    want[0], want[1], want[30], want[31], want[32 + 2] = 1.0, 2.0, 0.5, -6.0, 12.0
    assert np.array_equal(out, want)


def test_dequant_random_matches_table(oracle):
    rng = np.random.default_rng(7)
    table = np.load(os.path.join(GOLDEN, "mxfp4_table.npy"))
    blocks = rng.integers(0, 256, size=(3, 5, 90, 16), dtype=np.uint8)
    scales = rng.integers(0, 256, size=(3, 5, 90), dtype=np.uint8)
    got = oracle.dequant_mxfp4(blocks, scales).reshape(3, 5, 90, 32)
    lo, hi = blocks & 0xF, blocks >> 4
    s = scales[..., None]
    assert np.array_equal(got[..., 0::2], table[lo, s])
    assert np.array_equal(got[..., 1::2], table[hi, s])
    # the one-pass fp32 form (what fills the CPU path's fp32 expert tensors) is the same values widened; NaN codes
    # (scale 255) compare as bit patterns
    wide = oracle.dequant_mxfp4_f32(blocks, scales)
    assert np.array_equal(wide.view(np.uint32), got.reshape(wide.shape).astype(np.uint32) << 16)
    into = np.full((3, 5, 90 * 32), 3.0, dtype=np.float32)
    assert oracle.dequant_mxfp4_f32(blocks, scales, out=into) is into
    assert np.array_equal(into.view(np.uint32), wide.view(np.uint32))


# ---- bucketing: src/hip/scheduler.hip:11-61 ------------------------------------------------------
def test_bucket_invariants(oracle):
    rng = np.random.default_rng(8)
    for T, K, E in [(1, 1, 1), (5, 2, 4), (64, 4, 32), (300, 4, 128), (77, 8, 8)]:
        topk_i = np.stack([rng.permutation(E)[:K] for _ in range(T)]).astype(np.int32)
        topk_v = rng.random((T, K)).astype(np.float32)
        off, tok, wts, slot = oracle.bucket(topk_i, topk_v, E)
        counts = np.bincount(topk_i.ravel(), minlength=E)
        assert np.array_equal(off, np.concatenate([[0], np.cumsum(counts)]))
        for e in range(E):
            seg = tok[off[e]:off[e + 1]]
            assert np.array_equal(seg, np.sort(np.nonzero((topk_i == e).any(axis=1))[0]))
        # round trip through slot_of
        assert np.array_equal(tok[slot], np.repeat(np.arange(T), K).reshape(T, K))
        assert np.array_equal(wts[slot], topk_v)
        assert np.array_equal(np.sort(slot.ravel()), np.arange(T * K))


def test_bucket_empty_experts_and_skew(oracle):
    topk_i = np.tile(np.array([[7, 2]], np.int32), (10, 1))
    off, tok, wts, slot = oracle.bucket(topk_i, np.ones((10, 2), np.float32), 9)
    assert off.tolist() == [0, 0, 0, 10, 10, 10, 10, 10, 20, 20]
    assert tok.tolist() == list(range(10)) * 2


# ---- heavy / light work queues: src/hip/scheduler.hip:112-184 -------------------------------------
def numpy_classify(off, cutoff, f_sparse, f_default):
    """The rule from its description, with library calls only: active experts split by a row threshold."""
    ne = np.diff(off)
    act = np.nonzero(ne > 0)[0]
    if len(act) == 0:
        return np.zeros((0, 3), np.int32), np.zeros((0, 3), np.int32), (0, 0, 0, 0, 0)
    avg = np.float32(ne[act].sum()) / np.float32(len(act))
    factor = np.float32(1.0 if len(act) <= cutoff else f_sparse if len(act) <= 12 else f_default)
    thresh = int(np.ceil(np.float32(factor * avg)))
    heavy = act if len(act) <= cutoff else act[ne[act] >= thresh]
    light = np.setdiff1d(act, heavy)
    q = lambda sel: np.stack([sel, off[sel], ne[sel]], axis=1).astype(np.int32).reshape(-1, 3)
    return q(heavy), q(light), (len(heavy), len(light), int(ne[heavy].max()) if len(heavy) else 0, len(act), int(ne.sum()))


def test_classify_queues_against_numpy(oracle):
    rng = np.random.default_rng(12)
    cases = [np.zeros(9, np.int64)]                                   # no rows at all
    cases.append(np.concatenate([[0], np.cumsum([5, 0, 0, 7, 0, 1])]))  # 3 active <= cutoff 6: all heavy
    cases.append(np.concatenate([[0], np.cumsum([10, 10, 10, 10, 10, 10, 10, 15, 14, 0])]))  # 9 active: sparse factor 1.5
    for E in (13, 32, 128, 200):
        for _ in range(4):
            counts = rng.integers(0, 40, size=E) * (rng.random(E) < rng.choice([0.2, 0.6, 1.0]))
            cases.append(np.concatenate([[0], np.cumsum(counts)]))
    # a bucket exactly at the threshold and one row below it (13 active experts, default factor 1.25)
    counts = np.array([8] * 11 + [10, 9])        # mean 8.2308, 1.25 * mean = 10.29 -> threshold 11
    cases.append(np.concatenate([[0], np.cumsum(counts)]))
    counts = np.array([8] * 11 + [12, 4])        # mean 8 -> threshold exactly 10
    cases.append(np.concatenate([[0], np.cumsum(counts)]))
    for off in cases:
        off = np.asarray(off, dtype=np.int32)
        for cutoff, fs, fd in [(6, 1.5, 1.25), (0, 2.0, 1.0), (3, 1.0, 3.0)]:
            h, l, st = oracle.classify_queues(off, cutoff, fs, fd)
            rh, rl, rst = numpy_classify(off, cutoff, fs, fd)
            assert np.array_equal(h, rh) and np.array_equal(l, rl) and st == rst, (off.tolist(), cutoff, fs, fd)
            # partition of the active experts, ascending inside each queue
            both = np.concatenate([h[:, 0], l[:, 0]])
            assert np.array_equal(np.sort(both), np.nonzero(np.diff(off) > 0)[0])
            assert np.all(np.diff(h[:, 0]) > 0) and np.all(np.diff(l[:, 0]) > 0)


# ---- whole block: src/run.cpp:628-707 ------------------------------------------------------------
def fp64_block(t, wr, br, w1, b1, w2, b2, K, limit=7.0):
    """Independent composition in numpy fp64 (library matmul, library sort)."""
    t64 = t.astype(np.float64)
    scores = t64 @ wr.astype(np.float64).T + br
    idx = np.argsort(-scores.astype(np.float32), axis=1, kind="stable")[:, :K]
    out = np.zeros_like(t64)
    for b in range(t.shape[0]):
        sel = scores[b, idx[b]]
        p = np.exp(sel - sel.max())
        p /= p.sum()
        for k in range(K):
            e = idx[b, k]
            m = w1[e].astype(np.float64) @ t64[b] + b1[e]
            g = np.minimum(m[0::2], limit)
            u = np.clip(m[1::2], -limit, limit)
            h = g / (1 + np.exp(-1.702 * g)) * (u + 1)
            out[b] += p[k] * (w2[e].astype(np.float64) @ h + b2[e])
    return out, idx


def random_block(oracle, rng, T, H, I, E, scale=0.1):
    bf = lambda a: bf16_round(oracle, a)
    return dict(t=rng.standard_normal((T, H)).astype(np.float32),
                wr=bf(rng.standard_normal((E, H)) * scale), br=bf(rng.standard_normal(E) * scale),
                w1=bf(rng.standard_normal((E, 2 * I, H)) * scale), b1=bf(rng.standard_normal((E, 2 * I)) * scale),
                w2=bf(rng.standard_normal((E, H, I)) * scale), b2=bf(rng.standard_normal((E, H)) * scale))


@pytest.mark.parametrize("T,H,I,E,K", [(1, 8, 4, 1, 1), (6, 64, 32, 4, 2), (9, 96, 80, 16, 4), (4, 128, 64, 32, 4)])
def test_block_matches_fp64_composition(oracle, T, H, I, E, K):
    d = random_block(oracle, np.random.default_rng(T * 131 + E), T, H, I, E)
    y, ti, tv = oracle.moe_block(d["t"], d["wr"], d["br"], d["w1"], d["b1"], d["w2"], d["b2"], K)
    want, idx = fp64_block(d["t"], d["wr"], d["br"], d["w1"], d["b1"], d["w2"], d["b2"], K)
    assert np.array_equal(ti, idx)
    np.testing.assert_allclose(y, want, rtol=2e-5, atol=2e-6)
    np.testing.assert_allclose(tv.sum(axis=1), 1.0, rtol=1e-6)


def test_block_single_expert_is_a_dense_mlp(oracle):
    d = random_block(oracle, np.random.default_rng(11), 3, 32, 16, 1)
    y, ti, tv = oracle.moe_block(d["t"], d["wr"], d["br"], d["w1"], d["b1"], d["w2"], d["b2"], 1)
    assert np.all(ti == 0) and np.all(tv == 1.0)
    for b in range(3):
        m = oracle.matmul(d["t"][b], d["w1"][0]) + d["b1"][0]
        h = oracle.swiglu(m)
        assert np.array_equal(y[b], oracle.matmul(h, d["w2"][0]) + d["b2"][0])


def test_block_tokens_are_independent(oracle):
    d = random_block(oracle, np.random.default_rng(12), 7, 64, 32, 8)
    args = (d["wr"], d["br"], d["w1"], d["b1"], d["w2"], d["b2"], 4)
    y, ti, tv = oracle.moe_block(d["t"], *args)
    perm = np.random.default_rng(0).permutation(7)
    y2, ti2, tv2 = oracle.moe_block(d["t"][perm], *args)
    assert np.array_equal(y2, y[perm]) and np.array_equal(ti2, ti[perm]) and np.array_equal(tv2, tv[perm])


def test_block_golden_fixture(oracle):
    g = np.load(os.path.join(GOLDEN, "tiny_block.npz"))
    y, ti, tv, sc = oracle.moe_block(g["t"], g["w_router"], g["b_router"], g["w_mlp1"], g["b_mlp1"], g["w_mlp2"],
                                     g["b_mlp2"], int(g["K"]), want_scores=True)
    assert np.array_equal(ti, g["topk_i"])
    assert np.array_equal(sc, g["router_score"])
    np.testing.assert_allclose(tv, g["topk_v"], rtol=1e-6)
    np.testing.assert_allclose(y, g["e_agg"], rtol=1e-5, atol=1e-7)


def test_layer_is_norm_block_residual(oracle):
    d = random_block(oracle, np.random.default_rng(13), 4, 64, 32, 8)
    rms_w = bf16_round(oracle, 1 + 0.1 * np.random.default_rng(1).standard_normal(64))
    x1, ti, tv = oracle.moe_layer(d["t"], rms_w, d["wr"], d["br"], d["w1"], d["b1"], d["w2"], d["b2"], 4)
    tn = np.stack([oracle.rmsnorm(r, rms_w) for r in d["t"]])
    y, ti2, _ = oracle.moe_block(tn, d["wr"], d["br"], d["w1"], d["b1"], d["w2"], d["b2"], 4)
    assert np.array_equal(ti, ti2)
    assert np.array_equal(x1, d["t"] + y)
