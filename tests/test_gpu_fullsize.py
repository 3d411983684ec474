"""GPU parity at the published configurations' full sizes.  The CPU oracle runs on a subset of the
tokens (the block treats every token independently, src/run.cpp:503, so a subset is exact), and
size-independent properties cover the rest: bit-exact dequantisation of the whole tensor, token
permutation equivariance, batch invariance, run-to-run determinism."""
import numpy as np
import pytest
import torch

import hostgen

pytestmark = pytest.mark.gpu
OUT_TOL = 1e-2  # max|y - ref| / max|ref|


def say(*a):
    print(*a, flush=True)


def run_block(wl, oracle, dev, shape):
    table = oracle.normal_table()
    blk, raw = wl.make_device_layer(shape, table, dev, keep_canonical=True)
    x = wl.make_device_input(shape, table, dev)
    y, ti, tv = blk.forward(x)
    torch.cuda.synchronize()
    return blk, raw, x, y, ti, tv


def check_tokens(wl, oracle, shape, x, y, ti, tv, tokens, hw=None):
    """Oracle on the listed tokens only."""
    ti_h = ti.cpu().numpy()
    if hw is None:
        hw = hostgen.host_layer(oracle, wl, shape, experts=np.unique(ti_h[tokens]))
    xs = x.cpu().numpy()[tokens]
    ref_y, ref_i, ref_v, _ = hostgen.oracle_block(oracle, shape, hw, xs)
    assert np.array_equal(ti_h[tokens], ref_i), "top-k indices differ"
    np.testing.assert_allclose(tv.cpu().numpy()[tokens], ref_v, rtol=2e-6)
    err = hostgen.rel_err(y.cpu().numpy()[tokens], ref_y)
    say("  %s: %d tokens checked, rel err %.3e (max|d|/max|ref|), %.3e (rms)" %
        (shape.name, len(tokens), err, hostgen.rms_err(y.cpu().numpy()[tokens], ref_y)))
    assert err <= OUT_TOL
    return hw


def properties(pkg, blk, x, y, ti, tv, shape):
    # run-to-run determinism
    y2, ti2, tv2 = blk.forward(x)
    assert torch.equal(y2, y) and torch.equal(ti2, ti) and torch.equal(tv2, tv)
    # a permutation of the tokens permutes the outputs, bit for bit
    perm = torch.randperm(shape.T, device=x.device, generator=torch.Generator(device=x.device).manual_seed(1))
    yp, tip, tvp = blk.forward(x[perm].contiguous())
    assert torch.equal(tip, ti[perm]) and torch.equal(tvp, tv[perm])
    assert torch.equal(yp, y[perm])
    # the router's strict summation order selects the same experts
    ys, tis, tvs = blk.forward(x, flags=pkg.MOE_FLAG_ROUTER_STRICT_ORDER)
    assert torch.equal(tis, ti)
    assert torch.allclose(tvs, tv, rtol=1e-6, atol=0)
    # decode-sized batches: both expert GEMMs in one launch give the bits of the two launches
    if shape.T * shape.K <= 4096 and shape.T * shape.K <= 48 * shape.E:
        yf, tif, tvf = blk.forward(x, flags=pkg.MOE_FLAG_FUSED_GEMM_LAUNCH)
        assert torch.equal(yf, y) and torch.equal(tif, ti) and torch.equal(tvf, tv)


def test_decode256_bf16_and_the_cpu_64_token_case(pkg, wl, oracle, dev):
    """Configs 1 and 2: the 20b-shaped block, bf16 experts; 64 tokens through the CPU path."""
    shape = wl.WORKLOADS["decode256_bf16"]
    blk, raw, x, y, ti, tv = run_block(wl, oracle, dev, shape)
    hw = hostgen.host_layer(oracle, wl, shape)
    check_tokens(wl, oracle, shape, x, y, ti, tv, np.arange(shape.T), hw)     # every token
    properties(pkg, blk, x, y, ti, tv, shape)
    # batch invariance: the first 64 tokens alone (the 64-token configuration) give the same rows, bit for bit
    y64, ti64, tv64 = blk.forward(x[:64].contiguous())
    assert torch.equal(ti64, ti[:64]) and torch.equal(tv64, tv[:64])
    assert torch.equal(y64, y[:64])


def test_decode256_mxfp4(pkg, wl, oracle, dev):
    """Config 3: MXFP4 experts; the whole dequantised tensor is compared bit for bit."""
    shape = wl.WORKLOADS["decode256_mxfp4"]
    blk, raw, x, y, ti, tv = run_block(wl, oracle, dev, shape)
    hw = hostgen.host_layer(oracle, wl, shape)
    for name, rows, K in (("w_mlp1", 2 * shape.I, shape.H), ("w_mlp2", shape.H, shape.I)):
        got = pkg.mxfp4_tiled_to_bf16(blk.tensors[name], blk.tensors[name + "_scales"], shape.E, rows, K)
        want = oracle.dequant_mxfp4(hw[name + "_blocks"], hw[name + "_scales"])
        assert np.array_equal(got.view(torch.int16).cpu().numpy().view(np.uint16), want), name
        assert np.array_equal(raw[name + "_blocks"].cpu().numpy(), hw[name + "_blocks"])
    check_tokens(wl, oracle, shape, x, y, ti, tv, np.arange(shape.T), hw)     # every token
    properties(pkg, blk, x, y, ti, tv, shape)


def test_prefill4096_mxfp4_zipf(pkg, wl, oracle, dev):
    """Config 4: 4096 tokens, Zipf-skewed routing."""
    shape = wl.WORKLOADS["prefill4096_mxfp4_zipf"]
    blk, raw, x, y, ti, tv = run_block(wl, oracle, dev, shape)
    counts = np.bincount(ti.cpu().numpy().ravel(), minlength=shape.E)
    say("  realised rows per expert (sorted):", np.sort(counts)[::-1].tolist())
    assert counts.max() > 8 * counts.min()  # the skew is real
    # 288 tokens: 96 from the largest bucket (first, middle and last rows of it), every token of the
    # smallest bucket up to 96, and a random rest
    ti_h = ti.cpu().numpy()
    rng = np.random.default_rng(0)
    big, small = int(np.argmax(counts)), int(np.argmin(counts))
    in_big = np.nonzero((ti_h == big).any(axis=1))[0]
    in_small = np.nonzero((ti_h == small).any(axis=1))[0][:96]
    pick_big = np.concatenate([in_big[:32], in_big[len(in_big) // 2 - 16: len(in_big) // 2 + 16], in_big[-32:]])
    tokens = np.unique(np.concatenate([pick_big, in_small]))
    rest = np.setdiff1d(np.arange(shape.T), tokens)
    tokens = np.sort(np.concatenate([tokens, rng.choice(rest, 288 - len(tokens), replace=False)]))
    say("  largest bucket: expert %d with %d rows; smallest: expert %d with %d rows" % (big, counts[big], small, counts[small]))
    check_tokens(wl, oracle, shape, x, y, ti, tv, tokens, hostgen.host_layer(oracle, wl, shape))
    properties(pkg, blk, x, y, ti, tv, shape)
    # the same tokens through the decode-sized kernels (64-token blocks) agree closely
    ys, tis, _ = blk.forward(x, flags=pkg.MOE_FLAG_FORCE_STREAM)
    assert torch.equal(tis, ti)
    assert hostgen.rel_err(ys.cpu().numpy(), y.cpu().numpy()) <= 1e-5


def test_prefill4096_bf16(pkg, wl, oracle, dev):
    """4096 tokens on the bf16 experts of the 20b-shaped block (512 rows an expert on average: the
    128-token-block kernel with one block a compute unit)."""
    shape = wl.WORKLOADS["prefill4096_bf16"]
    blk, raw, x, y, ti, tv = run_block(wl, oracle, dev, shape)
    tokens = np.sort(np.random.default_rng(2).choice(shape.T, 160, replace=False))
    check_tokens(wl, oracle, shape, x, y, ti, tv, tokens, hostgen.host_layer(oracle, wl, shape))
    properties(pkg, blk, x, y, ti, tv, shape)
    # the same tokens through the decode-sized kernels and through the 128-token-block kernel that
    # runs two blocks a compute unit (what 1000 of these tokens alone would get) agree closely
    ys, tis, _ = blk.forward(x, flags=pkg.MOE_FLAG_FORCE_STREAM)
    assert torch.equal(tis, ti)
    e_s = hostgen.rel_err(ys.cpu().numpy(), y.cpu().numpy())
    y1, ti1, _ = blk.forward(x[:600].contiguous(), flags=pkg.MOE_FLAG_FORCE_TILED)
    assert torch.equal(ti1, ti[:600])
    e_1 = hostgen.rel_err(y1.cpu().numpy(), y[:600].cpu().numpy())
    say("  against the 64-token-block kernels %.3e, against the two-blocks-a-unit kernel %.3e" % (e_s, e_1))
    assert e_s <= 1e-5
    assert e_1 <= 1e-3  # another summation order ahead of the bf16 rounding of the SwiGLU rows


@pytest.mark.parametrize("fmt", ["bf16", "mxfp4"])
def test_largest_batch(pkg, wl, oracle, dev, fmt):
    """The documented maximum of 65535 tokens per call (small H and I keep it cheap): every launch grid
    and the workspace carving at their limits; a spread of tokens against the oracle, the rest
    through the size-independent properties."""
    shape = wl.MoeShape("maxT", T=65535, H=64, I=64, E=16, K=2, fmt=fmt, seed=9)
    say("largest batch", shape)
    blk, raw, x, y, ti, tv = run_block(wl, oracle, dev, shape)
    tokens = np.unique(np.concatenate([np.arange(8), np.arange(65527, 65535),
                                       np.random.default_rng(1).integers(0, 65535, 48)]))
    check_tokens(wl, oracle, shape, x, y, ti, tv, tokens)
    counts = np.bincount(ti.cpu().numpy().ravel(), minlength=shape.E)
    assert counts.sum() == 65535 * 2
    properties(pkg, blk, x, y, ti, tv, shape)
    assert pkg.block_workspace_bytes(65536, 64, 64, 16, 2) == 0  # one more token is refused


def test_stack120b_mxfp4(pkg, wl, oracle, dev):
    """Config 5: 36 layers, 128 experts, 1024 tokens, all weights (~61 GB) resident on one GPU.
    Layer glue as the reference's: t = rmsnorm(x) (unit weight), x += moe(t)."""
    shape = wl.WORKLOADS["stack120b_mxfp4"]
    L = shape.layers
    table = oracle.normal_table()
    stack = wl.DeviceStack(shape, table, dev)
    x0 = wl.make_device_input(shape, table, dev)
    tokens = np.concatenate([[0, 1, 511, 1023], np.random.default_rng(5).choice(np.arange(2, 1023), 12, replace=False)])
    tokens = np.sort(tokens)                                   # 16 tokens
    checked = [0, 7, 14, 21, 28, L - 1]                        # six layers, each fed the GPU's own input
    ones = np.ones(shape.H, np.float32)

    def check_layer(layer, x_in, x_out):
        ti = stack.topk_i[layer].cpu().numpy()
        hw = hostgen.host_layer(oracle, wl, shape, layer=layer, experts=np.unique(ti[tokens]))
        ref_x, ref_i, _ = oracle.moe_layer(x_in.cpu().numpy()[tokens], ones, hw["w_router"], hw["b_router"],
                                           hw["w_mlp1"], hw["b_mlp1"], hw["w_mlp2"], hw["b_mlp2"], shape.K)
        assert np.array_equal(ti[tokens], ref_i), "layer %d: top-k indices differ" % layer
        xin = x_in.cpu().numpy()[tokens]
        # the layer's own contribution, not the residual stream it is added to (which dwarfs it later on)
        err = hostgen.rel_err(x_out.cpu().numpy()[tokens] - xin, ref_x - xin)
        say("  layer %d: %d tokens, rel err of the MoE contribution %.3e (max), %.3e (rms)" %
            (layer, len(tokens), err, hostgen.rms_err(x_out.cpu().numpy()[tokens] - xin, ref_x - xin)))
        assert err <= OUT_TOL

    x = x0.clone()
    stack.prepare(x)
    done = 0
    for layer in checked:
        stack.forward(start=done, stop=layer)
        torch.cuda.synchronize()
        x_before = x.clone()
        stack.forward(start=layer, stop=layer + 1)
        torch.cuda.synchronize()
        check_layer(layer, x_before, x)
        done = layer + 1
    x_final = x.clone()
    assert bool(torch.isfinite(x_final).all())

    # the whole stack in one go ends in the same bits
    x = x0.clone()
    stack.prepare(x)
    stack.forward()
    torch.cuda.synchronize()
    assert torch.equal(x, x_final)
    ti_all = stack.topk_i.cpu().numpy()
    active = [(np.bincount(ti_all[l].ravel(), minlength=shape.E) > 0).sum() for l in range(L)]
    say("  active experts per layer: min %d max %d" % (min(active), max(active)))
