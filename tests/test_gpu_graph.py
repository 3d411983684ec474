"""moe_block_forward inside a captured HIP graph: the entry allocates nothing, never synchronises and clears
its counters with kernels, so a serving loop may capture one call and replay it.  Every replay must return
the eager call's bits: replayed several times, with eager work on the same buffers and synchronisations
between the replays, for each kernel family the size rule can pick."""
import pytest
import torch

pytestmark = pytest.mark.gpu

# T, H, I, E, K, fmt -> bucketing inside the expert kernels / bucketing launch + 64-token blocks /
# 128-token blocks (both MXFP4 and the two bf16 kernels) / two-pass router
FUSED = 32  # MOE_FLAG_FUSED_GEMM_LAUNCH: both expert GEMMs in one launch (counters cleared by a kernel)
CASES = [
    (64, 256, 128, 8, 4, "mxfp4"),
    (64, 256, 128, 8, 4, "bf16"),
    (64, 256, 128, 8, 4, "mxfp4", FUSED),
    (96, 320, 192, 16, 4, "bf16", FUSED),
    (300, 192, 128, 8, 1, "mxfp4"),
    (260, 320, 192, 4, 1, "bf16"),      # 65 rows per expert: two blocks a compute unit
    (700, 320, 192, 8, 4, "bf16"),      # 350 rows per expert: one block a compute unit
    (700, 320, 192, 8, 4, "mxfp4"),
    (2100, 128, 64, 32, 2, "mxfp4"),    # T x E >= 65536: the two-pass router
    (1200, 128, 64, 128, 4, "mxfp4"),   # 4800 assignments, 37 rows per expert: bucketing launch + 64-token blocks
    (1200, 128, 64, 128, 4, "bf16"),
]


@pytest.mark.parametrize("case", CASES, ids=lambda c: "-".join(str(v) for v in c))
def test_graph_replays_equal_the_eager_call(pkg, wl, oracle, dev, case):
    T, H, I, E, K, fmt = case[:6]
    flags = case[6] if len(case) > 6 else 0
    assert FUSED == pkg.MOE_FLAG_FUSED_GEMM_LAUNCH
    shape = wl.MoeShape("graph", T=T, H=H, I=I, E=E, K=K, fmt=fmt, seed=5 + T)
    table = oracle.normal_table()
    blk, raw = wl.make_device_layer(shape, table, dev)
    x = wl.make_device_input(shape, table, dev)
    x_alt = x.flip(0).contiguous()
    e_agg = torch.empty((T, H), dtype=torch.float32, device=dev)
    ti = torch.empty((T, K), dtype=torch.int32, device=dev)
    tv = torch.empty((T, K), dtype=torch.float32, device=dev)
    x_in = x.clone()
    p = blk.params(x_in, e_agg, ti, tv, flags=flags)
    stream = torch.cuda.current_stream().cuda_stream
    print("graph", shape, blk.describe(p), flush=True)

    def eager(inp):
        x_in.copy_(inp)
        blk.launch(p, stream)
        torch.cuda.synchronize()
        return e_agg.clone(), ti.clone(), tv.clone()

    want = eager(x)
    want_alt = eager(x_alt)
    assert not torch.equal(want[0], want_alt[0])
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        blk.launch(p, torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    for rep in range(4):
        inp, ref = (x, want) if rep % 2 == 0 else (x_alt, want_alt)
        x_in.copy_(inp)
        e_agg.fill_(float("nan"))
        ti.fill_(-1)
        tv.fill_(float("nan"))
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(ti, ref[1]) and torch.equal(tv, ref[2]), rep
        assert torch.equal(e_agg, ref[0]), rep
        # eager work on the same buffers between the replays
        got = eager(inp)
        assert torch.equal(got[0], ref[0])


def test_two_streams_do_not_share_state(pkg, wl, oracle, dev):
    """Two calls with their own workspaces on two streams at once (default priority) give the bits each gives
    alone: the library keeps nothing between or across calls."""
    table = oracle.normal_table()
    jobs = []
    for T, H, I, E, K, fmt in ((256, 256, 128, 8, 4, "mxfp4"), (700, 320, 192, 8, 4, "bf16")):
        shape = wl.MoeShape("streams", T=T, H=H, I=I, E=E, K=K, fmt=fmt, seed=T)
        blk, raw = wl.make_device_layer(shape, table, dev)
        x = wl.make_device_input(shape, table, dev)
        out = (torch.empty((T, H), dtype=torch.float32, device=dev), torch.empty((T, K), dtype=torch.int32, device=dev),
               torch.empty((T, K), dtype=torch.float32, device=dev))
        p = blk.params(x, *out)
        blk.launch(p, torch.cuda.current_stream().cuda_stream)
        torch.cuda.synchronize()
        jobs.append((blk, raw, x, p, out, [o.clone() for o in out]))
    streams = [torch.cuda.Stream(device=dev), torch.cuda.Stream(device=dev)]
    torch.cuda.synchronize()
    for _ in range(20):
        for (blk, raw, x, p, out, alone), st in zip(jobs, streams):
            for o in out:
                o.zero_()
        torch.cuda.synchronize()
        for _ in range(3):
            for (blk, raw, x, p, out, alone), st in zip(jobs, streams):
                blk.launch(p, st.cuda_stream)
        torch.cuda.synchronize()
        for blk, raw, x, p, out, alone in jobs:
            assert all(torch.equal(o, a) for o, a in zip(out, alone))
