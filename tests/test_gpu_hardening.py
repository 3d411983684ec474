"""Parity checks that go through the matrix-core path itself rather than beside it.

One-hot rows: a bf16 activation row that is 1.0 in column k and 0 elsewhere makes the down
projection return W2_e[:, k] + b2_e, every product exact and every partial sum a single value, so
the fused MXFP4 dequantisation is compared BIT FOR BIT with the reference dequantisation
(tools/model_export/gpt-oss-20b/export_model_bin.py:95-133) through the GEMM kernels' own weight and
scale addressing, in every kernel family.

Screening bound: the two-pass router may only drop an expert whose approximate score is more than
twice its error bound below the K-th best.  The bound is checked against exact scores on inputs made
to stress it."""
import zlib

import numpy as np
import pytest
import torch

import hostgen

pytestmark = pytest.mark.gpu


def say(*a):
    print(*a, flush=True)


def bf16_rows_one_hot(cols, width, dev):
    h = torch.zeros((len(cols), width), dtype=torch.bfloat16, device=dev)
    h[torch.arange(len(cols), device=dev), torch.as_tensor(cols, device=dev)] = 1.0
    return h


def routing(T, E, K, seed):
    """K distinct experts per token, every expert used, bucket sizes uneven."""
    rng = np.random.default_rng(seed)
    p = rng.dirichlet(np.ones(E) * 0.7)
    ti = np.stack([rng.choice(E, size=K, replace=False, p=p) for _ in range(T)]).astype(np.int32)
    ti[: E // K + 1] = (np.arange((E // K + 1) * K) % E).reshape(-1, K)   # every expert at least once
    return ti


# T, H, I, E, K : I is the contraction length of the down GEMM (320 = ragged last MX stage; 2880 real)
# the last two: buckets of 100 / 200 rows (bf16: the 128-token-block kernel with one block a compute unit), whose
# three-stage ring leaves two stages (2880 = 22.5 stages of 128) / one stage (448 = 3.5) after its whole turns
# the last: 80 000 assignment rows, more than one grid dimension holds (the row moves into and out of slot order
# run in slabs of 65535 rows)
ONE_HOT = [(70, 128, 320, 8, 4), (33, 192, 2880, 4, 2), (300, 64, 320, 4, 4), (129, 2880, 2880, 8, 4),
           (400, 2880, 2880, 8, 2), (200, 64, 448, 2, 2), (20000, 64, 64, 16, 4)]


@pytest.mark.parametrize("fmt", ["mxfp4", "bf16"])
@pytest.mark.parametrize("T,H,I,E,K", ONE_HOT)
def test_one_hot_rows_through_the_block_down_gemm(pkg, wl, oracle, dev, T, H, I, E, K, fmt):
    shape = wl.MoeShape("onehot", T=T, H=H, I=I, E=E, K=K, fmt=fmt, seed=I + T)
    say("one-hot down GEMM", shape)
    blk, raw = wl.make_device_layer(shape, oracle.normal_table(), dev, keep_canonical=True)
    hw = hostgen.host_layer(oracle, wl, shape)            # fp32 values of the reference dequantisation
    ti = routing(T, E, K, seed=T)
    A = T * K
    # column k of assignment a: sweep all columns, and hit the last MX block and the last element
    cols = (np.arange(A) * 37 + 5) % I
    cols[:4] = [0, I - 1, I - 32, 31]
    h = bf16_rows_one_hot(cols, I, dev)
    want = hw["w_mlp2"][ti.ravel(), :, cols] + hw["b_mlp2"][ti.ravel()]   # fp32 add of two bf16 values
    ti_d = torch.from_numpy(ti).to(dev)
    flags = {"size rule": 0,
             "64-token blocks, bucketing in the expert kernels": pkg.MOE_FLAG_FORCE_STREAM | pkg.MOE_FLAG_FORCE_DIRECT,
             "64-token blocks, bucketing launch": pkg.MOE_FLAG_FORCE_STREAM | pkg.MOE_FLAG_FORCE_BUCKET_LAUNCH,
             "128-token blocks": pkg.MOE_FLAG_FORCE_TILED}
    if A > 4096:  # past the longest assignment list a block scans itself: the flag is ignored, same path as the next
        del flags["64-token blocks, bucketing in the expert kernels"]
    for name, f in flags.items():
        y = blk.down_gemm(ti_d, h, flags=f)
        torch.cuda.synchronize()
        got = y.cpu().numpy()
        assert np.array_equal(got.view(np.uint32), want.astype(np.float32).view(np.uint32)), \
            "%s: %d of %d values differ" % (name, int((got != want).sum()), got.size)
    say("  all four kernel choices return W2[:, k] + b2 bit for bit (%d rows x %d)" % (A, H))


@pytest.mark.parametrize("fmt", ["mxfp4", "bf16"])
def test_one_hot_rows_through_the_scatter_entry(pkg, wl, oracle, dev, fmt):
    """The same through moe_mlp2_scatter[_mxfp4] (work queue, fp32 rows, atomic scatter): router
    weight 1, e_agg zero, one assignment per token, so every output row is one row of W2 + b2."""
    T, H, I, E = 90, 128, 320, 8
    shape = wl.MoeShape("onehot_q", T=T, H=H, I=I, E=E, K=1, fmt=fmt, seed=77)
    blk, raw = wl.make_device_layer(shape, oracle.normal_table(), dev, keep_canonical=True)
    hw = hostgen.host_layer(oracle, wl, shape)
    rng = np.random.default_rng(3)
    ex = rng.integers(0, E, T).astype(np.int32)
    cols = (np.arange(T) * 13 + 1) % I
    order = np.argsort(ex, kind="stable")                 # bucket order: by expert, ascending token
    off = np.concatenate([[0], np.cumsum(np.bincount(ex, minlength=E))]).astype(np.int32)
    gate = torch.zeros((T, I), dtype=torch.float32, device=dev)
    gate[torch.arange(T, device=dev), torch.from_numpy(cols[order]).to(dev)] = 1.0
    tok = torch.from_numpy(order.astype(np.int32)).to(dev)
    wts = torch.ones(T, dtype=torch.float32, device=dev)
    off_d = torch.from_numpy(off).to(dev)
    wq = torch.empty(3 * E, dtype=torch.int32, device=dev)
    wc = torch.zeros(1, dtype=torch.int32, device=dev)
    pkg.build_work_queue(off_d, E, wq, wc)
    e_agg = torch.zeros((T, H), dtype=torch.float32, device=dev)
    n_work = int(wc.item())
    max_ne = int(np.diff(off).max())
    if fmt == "bf16":
        pkg.moe_mlp2_scatter(wq, 0, n_work, gate, tok, wts, e_agg, raw["w_mlp2"], raw["b_mlp2"], I, H, H * I, H,
                             max_ne, 0)
    else:
        pkg.moe_mlp2_scatter_mxfp4(wq, 0, n_work, gate, tok, wts, e_agg, blk.tensors["w_mlp2"],
                                   blk.tensors["w_mlp2_scales"], raw["b_mlp2"], I, H, H, max_ne, 0)
    torch.cuda.synchronize()
    want = hw["w_mlp2"][ex, :, cols] + hw["b_mlp2"][ex]
    got = e_agg.cpu().numpy()
    assert np.array_equal(got.view(np.uint32), want.astype(np.float32).view(np.uint32))


def exact_scores(oracle, x, w_bits, b_bits):
    f = oracle.bf16_to_f32
    return np.stack([oracle.matmul(x[t], f(w_bits)) for t in range(x.shape[0])]) + f(b_bits)


ADVERSARIAL = ["same sign", "wide range", "extreme rows", "near ties", "random"]


@pytest.mark.parametrize("case", ADVERSARIAL)
@pytest.mark.parametrize("T,H,E,K", [(2048, 2880, 32, 4), (512, 2880, 128, 4), (1100, 320, 250, 8)])
def test_two_pass_router_bound_holds_with_margin(pkg, oracle, dev, T, H, E, K, case):
    """|approximate - exact| <= 0.5 * bound for every (token, expert): the screening pass may use the
    whole bound, so half of it is a safety factor of two."""
    # a seed that is the same in every process (str hashes are salted per process)
    rng = np.random.default_rng(zlib.crc32(repr((T, E, case)).encode()))
    x = rng.standard_normal((T, H)).astype(np.float32)
    w = rng.standard_normal((E, H)) * 0.02
    b = rng.standard_normal(E) * 0.02
    if case == "same sign":          # every product positive: nothing cancels, the sums are as large as they get
        x, w = np.abs(x), np.abs(w)
    elif case == "wide range":       # |x| spans 2^12 inside every row, the largest values anywhere in it
        x *= np.exp2(rng.integers(-6, 7, size=(T, H))).astype(np.float32)
    elif case == "extreme rows":     # router rows of very different norms, some at the top of the bf16 range used
        w *= np.exp2(rng.integers(-10, 11, size=(E, 1)))
        x[::3] *= 64.0
    elif case == "near ties":        # many experts within a few bf16 steps of one another
        base = rng.standard_normal(H) * 0.05
        w[: E // 2] = base
        b[: E // 2] = b[0]
    w_bits = oracle.f32_to_bf16(w)
    if case == "near ties":
        for e in range(1, E // 2):
            w_bits[e, (7 * e) % H] += 1
    b_bits = oracle.f32_to_bf16(b)
    to = lambda a, bf=False: (torch.from_numpy(np.ascontiguousarray(a)).view(torch.int16).view(torch.bfloat16)
                              if bf else torch.from_numpy(np.ascontiguousarray(a))).to(dev)
    tv, ti, approx, bound, n_cand = pkg.router_two_pass_report(to(x), to(w_bits, True), to(b_bits, True), K)
    torch.cuda.synchronize()
    sub = np.arange(0, T, max(1, T // 256))
    ref = exact_scores(oracle, x[sub], w_bits, b_bits)
    err = np.abs(approx.cpu().numpy()[sub].astype(np.float64) - ref.astype(np.float64)).max(axis=1)
    bd = bound.cpu().numpy()[sub].astype(np.float64)
    ratio = float((err / bd).max())
    say("  %-12s T=%d E=%d: max |approx - exact| / bound = %.3f, candidates per token mean %.2f max %d"
        % (case, T, E, ratio, float(n_cand.float().mean()), int(n_cand.max())))
    assert ratio <= 0.5
    # and the selection is the exact one (ties to the lower index)
    want_i = np.argsort(-ref, axis=1, kind="stable")[:, :K]
    assert np.array_equal(ti.cpu().numpy()[sub], want_i)
