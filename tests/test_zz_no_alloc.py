"""moe_gemm_router_static (the entry point that allocates nothing: its fp64 partial sums live in a fixed
device array inside the library) against moe_gemm_router (caller-provided scratch), bit for bit.
Two calls in a row share the array; the second is smaller, so stale contents of the first must not leak."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def _router_inputs(T, H, E, seed, dev):
    g = torch.Generator(device="cpu").manual_seed(seed)
    x = torch.randn((T, H), generator=g, dtype=torch.float32)
    w = (0.02 * torch.randn((E, H), generator=g, dtype=torch.float32)).to(torch.bfloat16)
    b = (0.02 * torch.randn((E,), generator=g, dtype=torch.float32)).to(torch.bfloat16)
    return x.to(dev), w.to(dev), b.to(dev)


def test_static_router_matches_scratch_router_twice(pkg, dev):
    assert pkg.lib.moe_gemm_router_static_max_bytes() == 16 << 20
    # first call: 20b decode shape; second call: fewer tokens, fewer experts, shorter rows
    for T, H, E, seed in [(256, 2880, 32, 1), (37, 512, 8, 2)]:
        x, w, b = _router_inputs(T, H, E, seed, dev)
        want = torch.full((T, E), float("nan"), dtype=torch.float32, device=dev)
        got = torch.full((T, E), float("nan"), dtype=torch.float32, device=dev)
        pkg.gemm_router(want, x, w, b, T, H, E)
        pkg.gemm_router_static(got, x, w, b, T, H, E)
        torch.cuda.synchronize()
        assert not torch.isnan(want).any()
        assert np.array_equal(got.cpu().numpy().view(np.uint32), want.cpu().numpy().view(np.uint32)), (T, H, E)


def test_static_router_rejects_what_does_not_fit(pkg, dev):
    # 16 segments x 65536 tokens x 64 experts x 8 bytes is far beyond the fixed array
    rc = pkg.lib.moe_gemm_router_static(16, 16, 16, 16, 65536, 2880, 64, None)
    assert rc == -3
    with pytest.raises(pkg.MoeError):
        pkg._check("moe_gemm_router_static", rc)
