"""GPU parity tests: every call goes through the C ABI (libmoe_gfx950.so) and is compared with
the CPU oracle on the same seeded inputs.  Bars: dequantised weights, top-k indices and bucketing
bit-exact; fp32 block outputs within 1e-2 of max|ref| (bf16 MFMA operands, fp32 accumulation)."""
import os

import numpy as np
import pytest
import torch

import hostgen
from conftest import GOLDEN

pytestmark = pytest.mark.gpu

OUT_TOL = 1e-2  # max|y - ref| / max|ref|


def to_dev(a, dev, bf16_bits=False):
    t = torch.from_numpy(np.ascontiguousarray(a))
    if bf16_bits:
        t = t.view(torch.int16).view(torch.bfloat16) if a.dtype == np.uint16 else t
    return t.to(dev)


def bits_of(t):
    return t.view(torch.int16).cpu().numpy().view(np.uint16)


def say(*a):
    print(*a, flush=True)


# ---- synthetic generator -------------------------------------------------------------------------
def test_device_generator_matches_host(pkg, wl, oracle, dev):
    table = oracle.normal_table()
    td = wl.normal_table_device(table, dev)
    n = 100003
    x = torch.empty(n, dtype=torch.float32, device=dev)
    pkg.synth_normal_f32(x, td, 1.0, 5, 1)
    assert np.array_equal(x.cpu().numpy(), oracle.synth_normal_f32((n,), 1.0, 5, 1))
    w = torch.empty(n, dtype=torch.bfloat16, device=dev)
    pkg.synth_normal_bf16(w, td, 0.02, 5, 4)
    assert np.array_equal(bits_of(w), oracle.synth_normal_bf16((n,), 0.02, 5, 4))
    b = torch.empty(n, dtype=torch.uint8, device=dev)
    pkg.synth_bytes(b, 5, 6)
    assert np.array_equal(b.cpu().numpy(), oracle.synth_bytes((n,), 5, 6))
    pkg.synth_range_bytes(b, 5, 8, 119, 9)
    assert np.array_equal(b.cpu().numpy(), oracle.synth_range_bytes((n,), 5, 8, 119, 9))


def test_checksum_matches_host_sum(pkg, oracle, dev):
    """moe_synth_checksum = sum of the buffer's 32-bit words mod 2^64: against numpy on the host generator's bytes
    (the device buffer is filled by the device generator), from one 16-byte word, over sizes that end inside a
    thread's chunk, up to more chunks than the launch has blocks; all-ones words so that the 64-bit carry matters;
    bad sizes and alignments refused."""
    out = torch.empty(pkg.SYNTH_CHECKSUM_WORDS, dtype=torch.int64, device=dev)
    for n16 in (1, 255, 256, 1023, 1024, 1025, 5000, 1024 * 2048 + 5, 3 * 1024 * 2048 + 777):
        n = n16 * 16
        print("checksum of", n, "bytes", flush=True)
        b = torch.empty(n, dtype=torch.uint8, device=dev)
        pkg.synth_bytes(b, 9, 3)
        got = int(pkg.synth_checksum(b, out=out)[0].item()) & ((1 << 64) - 1)
        want = int(oracle.synth_bytes((n,), 9, 3).view(np.uint32).sum(dtype=np.uint64))
        assert got == want, n16
    ones = torch.full((1 << 20,), -1, dtype=torch.int32, device=dev)  # 2^20 words of 0xFFFFFFFF: sum needs 52 bits
    assert int(pkg.synth_checksum(ones)[0].item()) == (1 << 20) * 0xFFFFFFFF
    with pytest.raises(Exception) as e:
        pkg.synth_checksum(ones.view(torch.uint8)[:24])
    assert e.value.code == -2  # not a multiple of 16 bytes
    with pytest.raises(Exception) as e:
        pkg.synth_checksum(ones.view(torch.uint8)[4:36])
    assert e.value.code == -6  # source not 16-byte aligned


def test_device_attributes_are_those_of_the_part(pkg, dev):
    a = pkg.device_attributes()
    pr = torch.cuda.get_device_properties(0)
    assert a["compute_units"] == pr.multi_processor_count and a["compute_units"] >= 64
    assert 500_000 <= a["clock_khz"] <= 4_000_000 and a["memory_clock_khz"] > 0
    assert a["memory_bus_bits"] >= 1024 and a["l2_bytes"] >= 1 << 20


# ---- MXFP4 ---------------------------------------------------------------------------------------
def test_dequant_exhaustive_bit_exact(pkg, dev):
    """Every (code, scale byte) pair through moe_dequant_mxfp4 against the exact-rational table."""
    table = np.load(os.path.join(GOLDEN, "mxfp4_table.npy"))
    # block s, byte b: low nibble = code b, high nibble = code 15-b, scale byte s
    blocks = np.zeros((256, 16), dtype=np.uint8)
    for b in range(16):
        blocks[:, b] = b | ((15 - b) << 4)
    scales = np.arange(256, dtype=np.uint8)
    out = bits_of(pkg.dequant_mxfp4(to_dev(blocks, dev), to_dev(scales, dev))).reshape(256, 32)
    for b in range(16):
        assert np.array_equal(out[:, 2 * b], table[b, :]), "low nibble code %d" % b
        assert np.array_equal(out[:, 2 * b + 1], table[15 - b, :]), "high nibble code %d" % (15 - b)


def test_fused_path_conversion_exhaustive(pkg, dev):
    """The conversion the fused GEMM uses (moe_mxfp4_tiled_to_bf16) on every code and every scale
    byte; it must be bit-exact wherever the workloads live (scale bytes 1..254, a superset of the
    119..127 the configs draw from)."""
    table = np.load(os.path.join(GOLDEN, "mxfp4_table.npy"))
    E, rows, K = 1, 64, 256 * 32  # one row per scale byte would do; use a full 64-row group
    blocks = np.zeros((E, rows, 256, 16), dtype=np.uint8)
    for b in range(16):
        blocks[..., b] = ((b + np.arange(rows)[None, :, None]) % 16) | (((15 - b + np.arange(rows)[None, :, None]) % 16) << 4)
    scales = np.broadcast_to(np.arange(256, dtype=np.uint8), (E, rows, 256)).copy()
    tb, ts = pkg.mxfp4_repack(to_dev(blocks, dev), to_dev(scales, dev))
    out = bits_of(pkg.mxfp4_tiled_to_bf16(tb, ts, E, rows, K)).reshape(rows, 256, 32)
    want = np.empty_like(out)
    lo, hi = blocks[0] & 0xF, blocks[0] >> 4
    want[..., 0::2] = table[lo, scales[0][..., None]]
    want[..., 1::2] = table[hi, scales[0][..., None]]
    bad_scales = sorted(set(np.argwhere(out != want)[:, 1].tolist()))
    say("fused-path conversion: scale bytes that differ from the reference dequant:", bad_scales)
    assert all(s in (0, 255) for s in bad_scales), bad_scales


@pytest.mark.parametrize("E,rows,K", [(1, 64, 32), (2, 128, 128), (3, 64, 320), (2, 192, 2880)])
def test_repack_round_trip_and_tiled_dequant(pkg, oracle, dev, E, rows, K):
    rng = np.random.default_rng(E * 1000 + K)
    blocks = rng.integers(0, 256, size=(E, rows, K // 32, 16), dtype=np.uint8)
    scales = rng.integers(110, 135, size=(E, rows, K // 32), dtype=np.uint8)
    db, ds = to_dev(blocks, dev), to_dev(scales, dev)
    tb, ts = pkg.mxfp4_repack(db, ds)
    ub, us = pkg.mxfp4_unpack(tb, ts, E, rows, K)
    assert torch.equal(ub, db) and torch.equal(us, ds)
    want = oracle.dequant_mxfp4(blocks, scales)
    assert np.array_equal(bits_of(pkg.mxfp4_tiled_to_bf16(tb, ts, E, rows, K)), want)
    assert np.array_equal(bits_of(pkg.dequant_mxfp4(db, ds)), want)
    # The scale slots of MX blocks that do not exist (a ragged last group of four stages) must hold 0 whatever the
    # destination held before: the expert kernels rely on that byte (a factor of exactly 0) to drop what the lanes past
    # the last block of a row load.  Every real scale here is non-zero, so the non-zero bytes are exactly the real ones.
    bb, sb = pkg.mxfp4_tiled_bytes(rows, K)
    dirty = (torch.full((E * bb,), 0xFF, dtype=torch.uint8, device=dev), torch.full((E * sb,), 0xFF, dtype=torch.uint8, device=dev))
    tb2, ts2 = pkg.mxfp4_repack(db, ds, out=dirty)
    assert torch.equal(tb2, tb) and torch.equal(ts2, ts)
    assert int((ts2 != 0).sum().item()) == E * rows * (K // 32)


# ---- router --------------------------------------------------------------------------------------
@pytest.mark.parametrize("T,H,E,K", [(1, 64, 4, 2), (5, 2880, 32, 4), (256, 2880, 32, 4), (130, 2880, 128, 4),
                                     (700, 512, 64, 8), (3, 128, 1024, 8)])
def test_router_logits_topk_softmax(pkg, oracle, dev, T, H, E, K):
    rng = np.random.default_rng(T + E)
    x = rng.standard_normal((T, H)).astype(np.float32)
    w_bits = oracle.f32_to_bf16(rng.standard_normal((E, H)) * 0.02)
    b_bits = oracle.f32_to_bf16(rng.standard_normal(E) * 0.02)
    w, b = oracle.bf16_to_f32(w_bits), oracle.bf16_to_f32(b_bits)
    want = np.stack([oracle.matmul(x[t], w) + b for t in range(T)])
    scores = torch.empty((T, E), dtype=torch.float32, device=dev)
    pkg.gemm_router(scores, to_dev(x, dev), to_dev(w_bits, dev, True), to_dev(b_bits, dev, True), T, H, E)
    got = scores.cpu().numpy()
    assert np.array_equal(got, want), "router logits differ in %d places" % (got != want).sum()
    tv = torch.empty((T, K), dtype=torch.float32, device=dev)
    ti = torch.empty((T, K), dtype=torch.int32, device=dev)
    pkg.topk(tv, ti, scores, T, E, K)
    ref = [oracle.topk(want[t], K) for t in range(T)]
    assert np.array_equal(ti.cpu().numpy(), np.stack([r[1] for r in ref]))
    assert np.array_equal(tv.cpu().numpy(), np.stack([r[0] for r in ref]))
    pkg.softmax(tv, T, K)
    np.testing.assert_allclose(tv.cpu().numpy(), np.stack([oracle.softmax(r[0]) for r in ref]), rtol=2e-6)


def test_topk_ties_go_to_lower_index(pkg, oracle, dev):
    rng = np.random.default_rng(0)
    for E, K in [(32, 4), (128, 4), (200, 8)]:
        s = rng.integers(-2, 3, size=(64, E)).astype(np.float32)
        s[0] = 0.0
        s[1] = np.where(np.arange(E) % 2 == 0, 0.0, -0.0)
        tv = torch.empty((64, K), dtype=torch.float32, device=dev)
        ti = torch.empty((64, K), dtype=torch.int32, device=dev)
        pkg.topk(tv, ti, to_dev(s, dev), 64, E, K)
        want = np.stack([oracle.topk(s[t], K)[1] for t in range(64)])
        assert np.array_equal(ti.cpu().numpy(), want)
        assert ti[0].tolist() == list(range(K))


# ---- bucketing -----------------------------------------------------------------------------------
@pytest.mark.parametrize("T,K,E", [(1, 1, 1), (7, 2, 4), (256, 4, 32), (4096, 4, 32), (1024, 4, 128), (1500, 8, 1000),
                                   (1025, 4, 8), (5000, 4, 32), (65535, 2, 16)])
def test_bucketing_bit_exact(pkg, oracle, dev, T, K, E):
    rng = np.random.default_rng(T + E)
    p = 1.0 / np.arange(1, E + 1) ** 1.2
    p /= p.sum()
    topk_i = np.stack([rng.choice(E, size=K, replace=False, p=p) for _ in range(T)]).astype(np.int32)
    topk_v = rng.random((T, K)).astype(np.float32)
    off = torch.empty(E + 1, dtype=torch.int32, device=dev)
    tok = torch.empty(T * K, dtype=torch.int32, device=dev)
    wts = torch.empty(T * K, dtype=torch.float32, device=dev)
    slot = torch.empty(T * K, dtype=torch.int32, device=dev)
    pkg.bucket_by_expert(to_dev(topk_i, dev), to_dev(topk_v, dev), T, K, E, off, tok, wts, slot)
    r_off, r_tok, r_wts, r_slot = oracle.bucket(topk_i, topk_v, E)
    assert np.array_equal(off.cpu().numpy(), r_off)
    assert np.array_equal(tok.cpu().numpy(), r_tok)
    assert np.array_equal(wts.cpu().numpy(), r_wts)
    assert np.array_equal(slot.cpu().numpy().reshape(T, K), r_slot)
    wq = torch.full((3 * E,), -1, dtype=torch.int32, device=dev)
    wc = torch.zeros(1, dtype=torch.int32, device=dev)
    pkg.build_work_queue(off, E, wq, wc)
    counts = np.diff(r_off)
    active = np.nonzero(counts)[0]
    assert int(wc.item()) == len(active)
    q = wq.cpu().numpy()[: 3 * len(active)].reshape(-1, 3)
    assert np.array_equal(q[:, 0], active) and np.array_equal(q[:, 1], r_off[active]) and np.array_equal(q[:, 2], counts[active])


@pytest.mark.parametrize("T,K,E", [(1, 1, 1), (5, 2, 4), (256, 4, 32), (1024, 4, 128), (4100, 4, 32), (777, 8, 200)])
def test_reference_signature_bucketing_steps(pkg, oracle, dev, T, K, E):
    """count -> scan -> compact -> classify under the reference kernels' argument lists
    (src/hip/scheduler.hip:11, 33, 48, 112) against the oracle, bit for bit."""
    rng = np.random.default_rng(3 * T + E)
    p = 1.0 / np.arange(1, E + 1) ** 1.2
    p /= p.sum()
    topk_i = np.stack([rng.choice(E, size=K, replace=False, p=p) for _ in range(T)]).astype(np.int32)
    topk_v = rng.random((T, K)).astype(np.float32)
    A = T * K
    i32 = lambda n, v=0: torch.full((n,), v, dtype=torch.int32, device=dev)
    a_e, a_t, counts, off = i32(A, -1), i32(A, -1), i32(E), i32(E + 1, -1)
    a_w = torch.zeros(A, dtype=torch.float32, device=dev)
    d_i, d_v = to_dev(topk_i, dev), to_dev(topk_v, dev)
    pkg.count_tokens_per_expert(d_i, d_v, T, K, a_e, a_t, a_w, counts, E)
    assert np.array_equal(a_e.cpu().numpy(), topk_i.ravel())
    assert np.array_equal(a_t.cpu().numpy(), np.repeat(np.arange(T), K))
    assert np.array_equal(a_w.cpu().numpy(), topk_v.ravel())
    assert np.array_equal(counts.cpu().numpy(), np.bincount(topk_i.ravel(), minlength=E))
    pkg.exclusive_scan_expert_offsets(counts, off, E)
    r_off, r_tok, r_wts, _ = oracle.bucket(topk_i, topk_v, E)
    assert np.array_equal(off.cpu().numpy(), r_off)
    assert not counts.cpu().numpy().any()
    tok, wts = i32(A, -1), torch.zeros(A, dtype=torch.float32, device=dev)
    pkg.compact_by_expert(a_e, a_t, a_w, A, off, counts, tok, wts, E)
    assert np.array_equal(tok.cpu().numpy(), r_tok)
    assert np.array_equal(wts.cpu().numpy(), r_wts)
    assert np.array_equal(counts.cpu().numpy(), np.diff(r_off))      # as after the reference's slot claims
    for cutoff, fs, fd in [(6, 1.5, 1.25), (0, 2.0, 1.0)]:           # the reference's constants (src/forward.cpp:36-44) first
        wq_h, wq_l = i32(3 * E, -1), i32(3 * E, -1)
        stats = torch.zeros(3, dtype=torch.int64, device=dev)
        pkg.classify_and_build_queues(off, E, cutoff, fs, fd, wq_h, wq_l, stats)
        r_h, r_l, r_st = oracle.classify_queues(r_off, cutoff, fs, fd)
        st32 = stats.cpu().numpy().view(np.int32)
        got = (int(st32[0]), int(st32[1]), int(st32[2]), int(st32[3]), int(stats.cpu().numpy()[2]))
        assert got == r_st
        assert np.array_equal(wq_h.cpu().numpy()[: 3 * r_st[0]].reshape(-1, 3), r_h)
        assert np.array_equal(wq_l.cpu().numpy()[: 3 * r_st[1]].reshape(-1, 3), r_l)


# ---- whole block, small shapes (oracle on every token) ---------------------------------------------
SMALL = [
    # T, H, I, E, K, fmt
    (1, 64, 64, 4, 2, "bf16"),
    (48, 256, 128, 8, 4, "bf16"),
    (48, 256, 128, 8, 4, "mxfp4"),
    (130, 320, 192, 16, 4, "mxfp4"),     # K=320 -> ragged last MX chunk (10 blocks), I=192 -> 6 blocks
    (130, 320, 192, 16, 4, "bf16"),
    (300, 128, 64, 4, 4, "mxfp4"),       # every token uses every expert: 300 rows per expert, 5 token blocks
    (33, 192, 64, 128, 4, "bf16"),       # most experts empty
    (17, 2880, 2880, 4, 2, "mxfp4"),     # real row/contraction lengths, few experts
    (64, 512, 256, 8, 4, "mxfp4"),       # contraction lengths that are whole groups of four stages / two stages
    (64, 512, 256, 8, 4, "bf16"),
    # large buckets: every token-tile count from 1 to 8 in the 128-token-block kernels
    (300, 128, 64, 4, 4, "bf16"),
    (700, 320, 192, 8, 4, "mxfp4"),      # ragged last MX chunk on the gate/up side
    (700, 320, 192, 8, 4, "bf16"),
    (210, 256, 128, 4, 2, "mxfp4"),      # ~105 rows per expert: one partly filled 128-token block each
    (97, 576, 320, 2, 2, "mxfp4"),       # 97 rows per expert, rows not a multiple of 512
    # bf16 buckets of 80+ rows (one-block-a-CU kernel): contraction lengths of 2 / 5 and 4 / 7 stages of 128,
    # i.e. one or two stages left after the whole turns of its three-stage ring, many token blocks in flight
    (700, 192, 64, 64, 8, "bf16"),
    (400, 576, 448, 8, 2, "bf16"),
    (97, 576, 832, 2, 2, "bf16"),
    # 56 and 52 row tiles over three row blocks (19, 19, 18 and 18, 17, 17): bf16 blocks that start or end inside a row unit
    (40, 832, 448, 4, 2, "bf16"),
]


@pytest.mark.parametrize("T,H,I,E,K,fmt", SMALL)
def test_block_small(pkg, wl, oracle, dev, T, H, I, E, K, fmt):
    shape = wl.MoeShape("small", T=T, H=H, I=I, E=E, K=K, fmt=fmt, seed=T + H)
    say("block_small", shape)
    table = oracle.normal_table()
    blk, raw = wl.make_device_layer(shape, table, dev)
    x = wl.make_device_input(shape, table, dev)
    scores = torch.empty((T, E), dtype=torch.float32, device=dev)
    y, ti, tv = blk.forward(x, router_score=scores)
    torch.cuda.synchronize()
    hw = hostgen.host_layer(oracle, wl, shape)
    xh = hostgen.host_input(oracle, wl, shape)
    assert np.array_equal(x.cpu().numpy(), xh)
    ref_y, ref_i, ref_v, ref_s = hostgen.oracle_block(oracle, shape, hw, xh)
    assert np.array_equal(scores.cpu().numpy(), ref_s)
    assert np.array_equal(ti.cpu().numpy(), ref_i)
    np.testing.assert_allclose(tv.cpu().numpy(), ref_v, rtol=2e-6)
    err = hostgen.rel_err(y.cpu().numpy(), ref_y)
    say("  rel err %.3e" % err)
    assert err <= OUT_TOL
    # strict router order gives the same routing, and the whole call is deterministic
    y2, ti2, tv2 = blk.forward(x, flags=pkg.MOE_FLAG_ROUTER_STRICT_ORDER)
    assert torch.equal(ti2, ti) and torch.equal(y2, y) and torch.equal(tv2, tv)
    # both kernel families on every shape, and the streaming family with either way of bucketing
    # (inside the expert kernels / by the bucketing launch), whichever the size rule picked above
    by_family = {}
    for name, flag in (("64-token blocks, bucketing in the expert kernels",
                        pkg.MOE_FLAG_FORCE_STREAM | pkg.MOE_FLAG_FORCE_DIRECT),
                       ("both GEMMs in one launch",
                        pkg.MOE_FLAG_FORCE_STREAM | pkg.MOE_FLAG_FORCE_DIRECT | pkg.MOE_FLAG_FUSED_GEMM_LAUNCH),
                       ("64-token blocks, bucketing launch",
                        pkg.MOE_FLAG_FORCE_STREAM | pkg.MOE_FLAG_FORCE_BUCKET_LAUNCH),
                       ("128-token blocks", pkg.MOE_FLAG_FORCE_TILED)):
        yf, tif, _ = blk.forward(x, flags=flag)
        errf = hostgen.rel_err(yf.cpu().numpy(), ref_y)
        say("  %s: rel err %.3e rms %.3e" % (name, errf, hostgen.rms_err(yf.cpu().numpy(), ref_y)))
        assert torch.equal(tif, ti) and errf <= OUT_TOL
        by_family[name] = yf
    # the one-launch kernel multiplies and adds in the order of the two-launch kernels: same bits
    assert torch.equal(by_family["both GEMMs in one launch"],
                       by_family["64-token blocks, bucketing in the expert kernels"])


@pytest.mark.parametrize("T,H", [(40, 256), (130, 2880), (9, 4160)])
def test_next_norm_fused_into_combine(pkg, wl, oracle, dev, T, H):
    """residual add + the RMSNorm that follows, done by the block's last kernel: bit-identical to
    the block without it followed by moe_rmsnorm (rows longer than 4096 take that route inside)."""
    import ctypes
    shape = wl.MoeShape("nextnorm", T=T, H=H, I=64, E=8, K=4, fmt="bf16", seed=T)
    table = oracle.normal_table()
    blk, raw = wl.make_device_layer(shape, table, dev)
    t_in = wl.make_device_input(shape, table, dev)
    x0 = torch.randn((T, H), device=dev, generator=torch.Generator(device=dev).manual_seed(3)) * 2.0
    w_bits = oracle.f32_to_bf16(1 + 0.2 * np.random.default_rng(1).standard_normal(H))
    w_d = to_dev(w_bits, dev, True)
    # separate: block with residual, then the norm
    xa = x0.clone()
    ya, tia, tva = blk.forward(t_in, residual_x=xa)
    na = torch.empty_like(xa)
    pkg.rmsnorm(na, xa, w_d, T, H)
    # fused
    xb = x0.clone()
    nb = torch.full_like(xb, float("nan"))
    yb, tib, tvb = blk.forward(t_in, residual_x=xb, next_norm_weight=w_d, next_norm_out=nb)
    torch.cuda.synchronize()
    assert torch.equal(ya, yb) and torch.equal(xa, xb) and torch.equal(tia, tib)
    assert torch.equal(na, nb)
    ref = np.stack([oracle.rmsnorm(r, oracle.bf16_to_f32(w_bits)) for r in xa.cpu().numpy()])
    np.testing.assert_allclose(nb.cpu().numpy(), ref, rtol=3e-7, atol=1e-9)
    # a caller compiled against the struct without the two members still works
    p = blk.params(t_in, torch.empty_like(ya), tia, tva, residual_x=x0.clone())
    p.struct_bytes = pkg.BlockParams.next_norm_weight.offset
    assert pkg.lib.moe_block_forward(ctypes.byref(p), torch.cuda.current_stream().cuda_stream) == 0
    # both members or neither, and the norm needs the residual
    p = blk.params(t_in, torch.empty_like(ya), tia, tva, residual_x=x0.clone(), next_norm_weight=w_d)
    assert pkg.lib.moe_block_forward(ctypes.byref(p), None) == -1
    p = blk.params(t_in, torch.empty_like(ya), tia, tva, next_norm_weight=w_d, next_norm_out=nb)
    assert pkg.lib.moe_block_forward(ctypes.byref(p), None) == -1


def _random_shapes(n, seed):
    rng = np.random.default_rng(seed)
    out = []
    for i in range(n):
        E = int(rng.choice([2, 3, 5, 8, 13, 32, 40]))
        K = int(rng.integers(1, min(8, E) + 1))
        T = int(rng.choice([1, 2, 7, 31, 64, 65, 129, 257, 400]))
        H = 64 * int(rng.integers(1, 9))
        I = 64 * int(rng.integers(1, 5))
        out.append((T, H, I, E, K, "bf16" if i % 2 else "mxfp4"))
    return out


@pytest.mark.parametrize("T,H,I,E,K,fmt", _random_shapes(24, seed=20))
def test_block_random_shapes(pkg, wl, oracle, dev, T, H, I, E, K, fmt):
    """Seeded random small shapes (one and many tokens, K from 1 to 8, expert counts that are no power
    of two), each through the size rule's choice and through both forced kernel families."""
    shape = wl.MoeShape("rand", T=T, H=H, I=I, E=E, K=K, fmt=fmt, seed=1000 + T + 7 * H + E)
    say("block_random", shape)
    table = oracle.normal_table()
    blk, raw = wl.make_device_layer(shape, table, dev)
    x = wl.make_device_input(shape, table, dev)
    hw = hostgen.host_layer(oracle, wl, shape)
    ref_y, ref_i, ref_v, _ = hostgen.oracle_block(oracle, shape, hw, hostgen.host_input(oracle, wl, shape))
    for flags in (0, pkg.MOE_FLAG_FORCE_STREAM | pkg.MOE_FLAG_FORCE_DIRECT,
                  pkg.MOE_FLAG_FORCE_STREAM | pkg.MOE_FLAG_FORCE_DIRECT | pkg.MOE_FLAG_FUSED_GEMM_LAUNCH,
                  pkg.MOE_FLAG_FORCE_STREAM | pkg.MOE_FLAG_FORCE_BUCKET_LAUNCH, pkg.MOE_FLAG_FORCE_TILED):
        y, ti, tv = blk.forward(x, flags=flags)
        torch.cuda.synchronize()
        assert np.array_equal(ti.cpu().numpy(), ref_i), flags
        np.testing.assert_allclose(tv.cpu().numpy(), ref_v, rtol=2e-6)
        err = hostgen.rel_err(y.cpu().numpy(), ref_y)
        assert err <= OUT_TOL, (flags, err)


def _random_bucket_shapes(n, seed):
    rng = np.random.default_rng(seed)
    out = []
    for i in range(n):
        E = int(rng.choice([2, 3, 4, 6, 8, 12]))
        K = int(rng.integers(1, min(4, E) + 1))
        T = int(rng.choice([90, 130, 200, 333, 512, 700, 1025, 1500]))
        H = 64 * int(rng.integers(1, 13))
        I = 64 * int(rng.integers(1, 13))
        out.append((T, H, I, E, K, ["bf16", "mxfp4"][i % 2]))
    return out


@pytest.mark.parametrize("T,H,I,E,K,fmt", _random_bucket_shapes(20, seed=31))
def test_block_random_long_buckets(pkg, wl, oracle, dev, T, H, I, E, K, fmt):
    """Seeded random shapes with few experts and up to 1500 tokens: buckets of tens to hundreds of rows
    (several token blocks per expert, every 128-token-block kernel), contraction lengths of 1 to 6 stages
    of 128 with and without a ragged last one; the size rule's choice and every forced family."""
    shape = wl.MoeShape("randlong", T=T, H=H, I=I, E=E, K=K, fmt=fmt, seed=2000 + T + 3 * H + I + E)
    say("block_random_long", shape, "rows per expert %.0f" % (T * K / E))
    table = oracle.normal_table()
    blk, raw = wl.make_device_layer(shape, table, dev)
    x = wl.make_device_input(shape, table, dev)
    hw = hostgen.host_layer(oracle, wl, shape)
    ref_y, ref_i, ref_v, _ = hostgen.oracle_block(oracle, shape, hw, hostgen.host_input(oracle, wl, shape))
    families = [0, pkg.MOE_FLAG_FORCE_STREAM | pkg.MOE_FLAG_FORCE_BUCKET_LAUNCH, pkg.MOE_FLAG_FORCE_TILED]
    if T * K <= 4096:  # the longest assignment list a block scans itself
        families.append(pkg.MOE_FLAG_FORCE_STREAM | pkg.MOE_FLAG_FORCE_DIRECT)
        families.append(pkg.MOE_FLAG_FORCE_STREAM | pkg.MOE_FLAG_FORCE_DIRECT | pkg.MOE_FLAG_FUSED_GEMM_LAUNCH)
    for flags in families:
        y, ti, tv = blk.forward(x, flags=flags)
        torch.cuda.synchronize()
        assert np.array_equal(ti.cpu().numpy(), ref_i), flags
        np.testing.assert_allclose(tv.cpu().numpy(), ref_v, rtol=2e-6)
        err = hostgen.rel_err(y.cpu().numpy(), ref_y)
        assert err <= OUT_TOL, (flags, err)


@pytest.mark.parametrize("fmt", ["bf16", "mxfp4"])
@pytest.mark.parametrize("T,zipf_s", [(1000, 8.0), (257, 10.0)])
def test_block_extreme_routing_skew(pkg, wl, oracle, dev, T, zipf_s, fmt):
    """A router bias that sends nearly every token to the same four experts: buckets as long as the batch
    next to empty and one-row buckets, through every kernel family; oracle on 200 tokens."""
    shape = wl.MoeShape("skew", T=T, H=512, I=256, E=32, K=4, fmt=fmt, zipf_s=zipf_s, seed=3)
    table = oracle.normal_table()
    blk, raw = wl.make_device_layer(shape, table, dev)
    x = wl.make_device_input(shape, table, dev)
    hw = hostgen.host_layer(oracle, wl, shape)
    sub = np.sort(np.random.default_rng(0).choice(T, min(T, 200), replace=False))
    ref_y, ref_i, ref_v, _ = hostgen.oracle_block(oracle, shape, hw, hostgen.host_input(oracle, wl, shape)[sub])
    for flags in (0, pkg.MOE_FLAG_FORCE_STREAM | pkg.MOE_FLAG_FORCE_BUCKET_LAUNCH,
                  pkg.MOE_FLAG_FORCE_STREAM | pkg.MOE_FLAG_FORCE_DIRECT,
                  pkg.MOE_FLAG_FORCE_STREAM | pkg.MOE_FLAG_FORCE_DIRECT | pkg.MOE_FLAG_FUSED_GEMM_LAUNCH,
                  pkg.MOE_FLAG_FORCE_TILED):
        y, ti, tv = blk.forward(x, flags=flags)
        torch.cuda.synchronize()
        counts = np.bincount(ti.cpu().numpy().ravel(), minlength=shape.E)
        assert counts.max() >= 0.9 * T and (counts == 0).sum() >= 16   # the skew is what the test is about
        assert np.array_equal(ti.cpu().numpy()[sub], ref_i), flags
        np.testing.assert_allclose(tv.cpu().numpy()[sub], ref_v, rtol=2e-6)
        err = hostgen.rel_err(y.cpu().numpy()[sub], ref_y)
        assert err <= OUT_TOL, (flags, err)
    say("  skew T=%d %s: longest bucket %d rows, %d empty experts, rel err %.2e" %
        (T, fmt, counts.max(), (counts == 0).sum(), err))


def test_block_residual_and_rmsnorm_glue(pkg, wl, oracle, dev):
    shape = wl.MoeShape("glue", T=40, H=256, I=128, E=8, K=4, fmt="bf16", seed=3)
    table = oracle.normal_table()
    blk, raw = wl.make_device_layer(shape, table, dev)
    x = wl.make_device_input(shape, table, dev) * 3.0
    rms_bits = oracle.f32_to_bf16(1 + 0.1 * np.random.default_rng(0).standard_normal(shape.H))
    t = torch.empty_like(x)
    pkg.rmsnorm(t, x, to_dev(rms_bits, dev, True), shape.T, shape.H)
    xres = x.clone()
    y, ti, tv = blk.forward(t, residual_x=xres)
    hw = hostgen.host_layer(oracle, wl, shape)
    x_ref, ref_i, _ = oracle.moe_layer(x.cpu().numpy(), oracle.bf16_to_f32(rms_bits), hw["w_router"], hw["b_router"],
                                       hw["w_mlp1"], hw["b_mlp1"], hw["w_mlp2"], hw["b_mlp2"], shape.K)
    t_ref = np.stack([oracle.rmsnorm(r, oracle.bf16_to_f32(rms_bits)) for r in x.cpu().numpy()])
    np.testing.assert_allclose(t.cpu().numpy(), t_ref, rtol=3e-7, atol=1e-9)
    assert np.array_equal(ti.cpu().numpy(), ref_i)
    assert torch.equal(xres, x + y)
    assert hostgen.rel_err(xres.cpu().numpy(), x_ref) <= OUT_TOL


def test_two_pass_router_near_ties(pkg, oracle, dev):
    """Large batches take the two-pass router (fp32 screening, exact scores of the candidates).
    Router rows that are equal, or differ by one bf16 step in a few elements, put many tokens'
    K-th and (K+1)-th scores closer together than the screening error: indices must still be the
    oracle's, ties to the lower index, and the weights the exact softmax's."""
    T, H, I, E, K = 1024, 256, 64, 64, 4
    rng = np.random.default_rng(7)
    x = rng.standard_normal((T, H)).astype(np.float32)
    x[5] = 0.0                      # every score equals its bias
    x[6] = x[7]                     # duplicate tokens
    w = rng.standard_normal((E, H)) * 0.02
    base = rng.standard_normal(H) * 0.08
    w_bits = oracle.f32_to_bf16(w)
    base_bits = oracle.f32_to_bf16(base)
    for e in (3, 9, 10, 20, 41, 63):  # a family of near-copies that usually wins
        w_bits[e] = base_bits
    w_bits[10, 17] += 1             # one bf16 step up in one element
    w_bits[20, 100] -= 1
    w_bits[41, 0:4] += 1
    w_bits[63, 200] += 2
    b_bits = oracle.f32_to_bf16(rng.standard_normal(E) * 0.01)
    b_bits[[3, 9, 10, 20, 41, 63]] = b_bits[3]
    w1 = oracle.f32_to_bf16(rng.standard_normal((E, 2 * I, H)) * 0.05)
    b1 = oracle.f32_to_bf16(rng.standard_normal((E, 2 * I)) * 0.05)
    w2 = oracle.f32_to_bf16(rng.standard_normal((E, H, I)) * 0.05)
    b2 = oracle.f32_to_bf16(rng.standard_normal((E, H)) * 0.05)
    blk = pkg.MoeBlock(H, I, E, K, *[to_dev(a, dev, True) for a in (w_bits, b_bits, w1, b1, w2, b2)], max_tokens=T)
    xd = to_dev(x, dev)
    say("two-pass router, near ties")
    y, ti, tv = blk.forward(xd)                                            # two-pass
    scores = torch.empty((T, E), dtype=torch.float32, device=dev)
    y1, ti1, tv1 = blk.forward(xd, router_score=scores)                    # single exact pass
    torch.cuda.synchronize()
    f = oracle.bf16_to_f32
    ref_y, ref_i, ref_v, ref_s = oracle.moe_block(x, f(w_bits), f(b_bits), f(w1), f(b1), f(w2), f(b2), K, 7.0,
                                                  want_scores=True)
    assert np.array_equal(scores.cpu().numpy(), ref_s)
    top = np.sort(ref_s, axis=1)[:, ::-1]
    say("  tokens whose K-th and (K+1)-th exact scores are equal: %d, within 1e-4: %d"
        % (int((top[:, K - 1] == top[:, K]).sum()), int((top[:, K - 1] - top[:, K] < 1e-4).sum())))
    assert (top[:, K - 1] - top[:, K] < 1e-4).sum() > T // 10  # the case really is exercised
    assert np.array_equal(ti1.cpu().numpy(), ref_i)
    assert np.array_equal(ti.cpu().numpy(), ref_i)
    np.testing.assert_allclose(tv.cpu().numpy(), ref_v, rtol=2e-6)
    assert torch.equal(ti[6], ti[7]) and torch.equal(y[6], y[7])
    assert hostgen.rel_err(y.cpu().numpy(), ref_y) <= OUT_TOL


@pytest.mark.parametrize("T,H,I,E,K", [(300, 320, 64, 250, 4), (20000, 64, 64, 4, 2), (70, 128, 64, 1024, 8),
                                       (4100, 2880, 64, 17, 4)])
def test_two_pass_router_odd_shapes(pkg, oracle, dev, T, H, I, E, K):
    """The two-pass router at shapes that leave partial tiles everywhere: expert counts that are no
    multiple of 16, token counts that are no multiple of 64, one and many k-segments."""
    rng = np.random.default_rng(T + E)
    x = rng.standard_normal((T, H)).astype(np.float32)
    w_bits = oracle.f32_to_bf16(rng.standard_normal((E, H)) * 0.05)
    b_bits = oracle.f32_to_bf16(rng.standard_normal(E) * 0.05)
    w1 = oracle.f32_to_bf16(rng.standard_normal((E, 2 * I, H)) * 0.05)
    b1 = oracle.f32_to_bf16(rng.standard_normal((E, 2 * I)) * 0.05)
    w2 = oracle.f32_to_bf16(rng.standard_normal((E, H, I)) * 0.05)
    b2 = oracle.f32_to_bf16(rng.standard_normal((E, H)) * 0.05)
    blk = pkg.MoeBlock(H, I, E, K, *[to_dev(a, dev, True) for a in (w_bits, b_bits, w1, b1, w2, b2)], max_tokens=T)
    say("two-pass router", (T, H, I, E, K))
    y, ti, tv = blk.forward(to_dev(x, dev))
    torch.cuda.synchronize()
    f = oracle.bf16_to_f32
    # router and top-k of the oracle on every token (cheap); the whole block on a few
    want_s = np.stack([oracle.matmul(x[t], f(w_bits)) + f(b_bits) for t in range(0, T, max(1, T // 512))])
    sub = np.arange(0, T, max(1, T // 512))
    want_i = np.argsort(-want_s, axis=1, kind="stable")[:, :K]
    assert np.array_equal(ti.cpu().numpy()[sub], want_i)
    few = sub[:24]
    ref_y, ref_i, ref_v, _ = oracle.moe_block(x[few], f(w_bits), f(b_bits), f(w1), f(b1), f(w2), f(b2), K, 7.0,
                                              want_scores=True)
    assert np.array_equal(ti.cpu().numpy()[few], ref_i)
    np.testing.assert_allclose(tv.cpu().numpy()[few], ref_v, rtol=2e-6)
    assert hostgen.rel_err(y.cpu().numpy()[few], ref_y) <= OUT_TOL


# ---- the reference's own data flow: gather -> queue -> mlp1 -> mlp2 scatter -> vecadd -------------
@pytest.mark.parametrize("fmt", ["bf16", "mxfp4"])
def test_reference_call_sequence(pkg, wl, oracle, dev, fmt):
    shape = wl.MoeShape("seq", T=150, H=320, I=192, E=8, K=4, fmt=fmt, seed=9)
    T, H, I, E, K = shape.T, shape.H, shape.I, shape.E, shape.K
    table = oracle.normal_table()
    blk, raw = wl.make_device_layer(shape, table, dev)
    t = wl.make_device_input(shape, table, dev)
    y_fused, ti_fused, tv_fused = blk.forward(t)
    # step by step, as src/forward.cpp:317-514 issues it
    scores = torch.empty((T, E), dtype=torch.float32, device=dev)
    pkg.gemm_router(scores, t, raw["w_router"], raw["b_router"], T, H, E)
    tv = torch.empty((T, K), dtype=torch.float32, device=dev)
    ti = torch.empty((T, K), dtype=torch.int32, device=dev)
    pkg.topk(tv, ti, scores, T, E, K)
    pkg.softmax(tv, T, K)
    assert torch.equal(ti, ti_fused) and torch.equal(tv, tv_fused)
    A = T * K
    off = torch.empty(E + 1, dtype=torch.int32, device=dev)
    tok = torch.empty(A, dtype=torch.int32, device=dev)
    wts = torch.empty(A, dtype=torch.float32, device=dev)
    pkg.bucket_by_expert(ti, tv, T, K, E, off, tok, wts)
    x_by_expert = torch.empty((A, H), dtype=torch.float32, device=dev)
    pkg.gather_rows(t, tok, x_by_expert, A, H)
    assert torch.equal(x_by_expert, t[tok.long()])
    wq = torch.empty(3 * E, dtype=torch.int32, device=dev)
    wc = torch.zeros(1, dtype=torch.int32, device=dev)
    pkg.build_work_queue(off, E, wq, wc)
    n_work = int(wc.item())
    max_ne = int((off[1:] - off[:-1]).max().item())
    gate = torch.empty((A, I), dtype=torch.float32, device=dev)
    e_agg = torch.zeros((T, H), dtype=torch.float32, device=dev)
    x_res = torch.zeros((T, H), dtype=torch.float32, device=dev)
    if fmt == "bf16":
        pkg.moe_mlp1_swiglu(wq, 0, n_work, x_by_expert, gate, raw["w_mlp1"], raw["b_mlp1"], H, I, 2 * I * H, 2 * I,
                            shape.alpha, shape.swiglu_limit, max_ne, 0)
        pkg.moe_mlp2_scatter(wq, 0, n_work, gate, tok, wts, e_agg, raw["w_mlp2"], raw["b_mlp2"], I, H, H * I, H,
                             max_ne, 0)
    else:
        tns = blk.tensors
        pkg.moe_mlp1_swiglu_mxfp4(wq, 0, n_work, x_by_expert, gate, tns["w_mlp1"], tns["w_mlp1_scales"],
                                  raw["b_mlp1"], H, I, 2 * I, shape.alpha, shape.swiglu_limit, max_ne, 0)
        pkg.moe_mlp2_scatter_mxfp4(wq, 0, n_work, gate, tok, wts, e_agg, tns["w_mlp2"], tns["w_mlp2_scales"],
                                   raw["b_mlp2"], I, H, H, 16, 0)  # maxNe hint smaller than the truth: blocks loop
    pkg.vecadd_and_zero(x_res, e_agg, 1.0, T, H)
    assert float(e_agg.abs().max().item()) == 0.0
    hw = hostgen.host_layer(oracle, wl, shape)
    ref_y, ref_i, _, _ = hostgen.oracle_block(oracle, shape, hw, t.cpu().numpy())
    assert np.array_equal(ti.cpu().numpy(), ref_i)
    assert hostgen.rel_err(x_res.cpu().numpy(), ref_y) <= OUT_TOL
    assert hostgen.rel_err(y_fused.cpu().numpy(), ref_y) <= OUT_TOL
    # atomics reorder the fp32 sum over a token's experts; everything else is the same arithmetic
    # up to the fp32 (not bf16) intermediate kept by this data flow
    assert hostgen.rel_err(x_res.cpu().numpy(), y_fused.cpu().numpy()) <= 5e-3
