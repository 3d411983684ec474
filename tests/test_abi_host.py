"""Host-side checks that need no GPU: the C-ABI library loads, exports every symbol the header
declares, sizes workspaces, and rejects bad arguments before touching the device; the Python and C
sides of the synthetic generator agree; algorithmic byte/flop counts match the published table."""
import ctypes
import os
import re

import numpy as np
import pytest

from conftest import ROOT


def declared_functions():
    text = open(os.path.join(ROOT, "include", "moe_abi.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(moe_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol(pkg):
    names = declared_functions()
    assert len(names) >= 25
    raw = ctypes.CDLL(pkg.LIB_PATH)
    for n in names:
        assert hasattr(raw, n), "symbol %s declared in include/moe_abi.h is not exported" % n
    assert sorted(pkg.SIGNATURES) == names
    assert pkg.lib.moe_abi_version() == 1


def test_error_strings(pkg):
    assert pkg.lib.moe_error_string(0) == b"ok"
    for code in range(-6, 0):
        assert len(pkg.lib.moe_error_string(code)) > 3


def test_workspace_and_tiled_sizes(pkg):
    assert pkg.block_workspace_bytes(0, 2880, 2880, 32, 4) == 0
    assert pkg.block_workspace_bytes(256, 2881, 2880, 32, 4) == 0      # H % 64
    assert pkg.block_workspace_bytes(256, 2880, 2880, 2048, 4) == 0    # E > 1024
    assert pkg.block_workspace_bytes(256, 2880, 2880, 32, 33) == 0     # K > E
    n = pkg.block_workspace_bytes(256, 2880, 2880, 32, 4)
    A = 1024
    assert n >= A * 2880 * 2 + A * 2880 * 4 + 256 * 2880 * 2
    assert n % 256 == 0
    # tiled MXFP4: same block bytes as the checkpoint layout, scales padded to 16 per quad of chunks
    bb, sb = pkg.mxfp4_tiled_bytes(5760, 2880)
    assert bb == 5760 * 90 * 16
    assert sb == (5760 // 16) * 6 * 256
    assert pkg.mxfp4_tiled_bytes(5761, 2880) == (0, 0)
    assert pkg.mxfp4_tiled_bytes(5760, 2881) == (0, 0)


def test_entries_reject_bad_arguments_without_a_device(pkg):
    L = pkg.lib
    assert L.moe_topk(None, None, None, 1, 32, 4, None) == -1
    assert L.moe_topk(1, 1, 1, 1, 2048, 4, None) == -3
    assert L.moe_topk(1, 1, 1, 1, 4, 5, None) == -2
    assert L.moe_softmax(1, 4, 65, None) == -3
    assert L.moe_gemm_router(1, 1, 1, 1, 4, 2881, 32, 1, 1 << 30, None) == -2
    assert L.moe_gemm_router(16, 16, 16, 16, 4, 2880, 32, None, 0, None) == -4
    assert L.moe_gemm_router(16, 8, 16, 16, 4, 2880, 32, 16, 1 << 30, None) == -6
    assert L.moe_bucket_by_expert(1, 1, 4, 4, 2000, 1, 1, 1, None, None) == -3
    assert L.moe_gather_rows(1, 1, 1, 4, 6, None) == -2
    assert L.moe_count_tokens_per_expert(1, 1, 4, 4, 1, 1, 1, None, 32, None) == -1
    assert L.moe_count_tokens_per_expert(1, 1, 4, 4, 1, 1, 1, 1, 2000, None) == -3
    assert L.moe_exclusive_scan_expert_offsets(1, 1, 0, None) == -2
    assert L.moe_compact_by_expert(1, 1, 1, 16, 1, 1, 1, None, 32, None) == -1
    assert L.moe_classify_and_build_queues(1, 32, 6, 1.5, 1.25, 1, 1, None, None) == -1
    assert L.moe_dequant_mxfp4(8, 8, 4, 8, None) == -6      # blocks not 16-byte aligned
    assert L.moe_mxfp4_repack(16, 16, 1, 63, 64, 16, 16, None) == -2
    assert L.moe_block_forward(None, None) == -1
    p = pkg.BlockParams()
    p.struct_bytes = 8
    assert L.moe_block_forward(ctypes.byref(p), None) == -5
    p.struct_bytes = ctypes.sizeof(pkg.BlockParams)
    p.n_tokens, p.hidden_dim, p.intermediate_dim, p.n_experts, p.experts_per_token = 4, 64, 64, 4, 2
    assert L.moe_block_forward(ctypes.byref(p), None) == -1  # NULL tensors
    # several layers in one call: same checks per element, the array is walked by the caller's struct size
    assert L.moe_block_forward_layers(None, 2, None) == -1
    assert L.moe_block_forward_layers(ctypes.byref(p), 0, None) == -2
    two = pkg.pack_layer_params([p, p])
    assert ctypes.sizeof(two) == 2 * ctypes.sizeof(pkg.BlockParams)
    assert L.moe_block_forward_layers(ctypes.byref(two), 2, None) == -1  # NULL tensors in the first element
    two[0].struct_bytes = 8
    assert L.moe_block_forward_layers(ctypes.byref(two), 2, None) == -5
    assert L.moe_synth_checksum(None, 16, None, None) == -1
    assert L.moe_synth_checksum(16, 24, 16, None) == -2     # not a multiple of 16 bytes
    assert L.moe_synth_checksum(8, 32, 16, None) == -6      # source not 16-byte aligned
    with pytest.raises(pkg.MoeError):
        pkg._check("x", -2)


def test_python_hash_matches_c(oracle, wl):
    for seed, tid in [(0, 1), (7, 36), (123, 4)]:
        got = oracle.synth_bytes((64,), seed, tid)
        want = np.array([wl.synth_hash(seed, tid, i) >> 24 for i in range(64)], dtype=np.uint8)
        assert np.array_equal(got, want)


def test_synth_distributions(oracle):
    x = oracle.synth_normal_f32((1 << 18,), 1.0, 0, 1)
    assert abs(x.mean()) < 0.01 and abs(x.std() - 1) < 0.01
    w = oracle.bf16_to_f32(oracle.synth_normal_bf16((1 << 18,), 0.02, 0, 4))
    assert abs(w.std() - 0.02) < 3e-4
    s = oracle.synth_range_bytes((1 << 16,), 0, 8, 119, 9)
    assert s.min() == 119 and s.max() == 127
    assert np.bincount(s)[119:].min() > (1 << 16) / 9 * 0.9
    b = oracle.synth_bytes((1 << 16,), 0, 4)
    assert np.bincount(b & 0xF, minlength=16).min() > (1 << 16) / 16 * 0.9
    # streams differ by tensor id and by seed
    assert not np.array_equal(oracle.synth_bytes((64,), 0, 4), oracle.synth_bytes((64,), 0, 6))
    assert not np.array_equal(oracle.synth_bytes((64,), 0, 4), oracle.synth_bytes((64,), 1, 4))


def test_algorithmic_work_matches_published_table(wl):
    W = wl.WORKLOADS
    assert wl.algorithmic_bytes(W["decode256_bf16"]) == 1_599_160_384
    assert wl.algorithmic_bytes(W["decode256_mxfp4"]) == 429_649_984
    assert wl.algorithmic_bytes(W["prefill4096_mxfp4_zipf"]) == 518_123_584
    assert wl.algorithmic_bytes(W["stack120b_mxfp4"]) * 36 == 61_869_597_696
    assert wl.algorithmic_flops(W["decode256_bf16"]) == 4 * 256 * 2 * 24_883_200 + 2 * 256 * 2880 * 32
    assert abs(wl.algorithmic_flops(W["prefill4096_mxfp4_zipf"]) / 816.13e9 - 1) < 1e-3


def test_zipf_router_bias(wl):
    shape = wl.WORKLOADS["prefill4096_mxfp4_zipf"]
    bits = wl.zipf_router_bias_bits(shape)
    b = (bits.astype(np.uint32) << 16).view(np.float32)
    assert b.max() == 0.0 and len(np.unique(b)) == shape.E
    assert abs(b.min() - wl.ZIPF_BETA * -1.2 * np.log(32)) < 0.02


def test_cpp_host_headers_compile_link_and_check_arguments(pkg, tmp_path):
    """The C++ host side (drop-in wrappers under the reference's function names + the layer
    function) builds with a plain C++17 compiler against the C ABI and rejects null buffers."""
    import subprocess
    host = os.path.join(ROOT, "gpt-oss-amd_amd", "host")
    exe = str(tmp_path / "example_layer_loop")
    libdir = os.path.dirname(pkg.LIB_PATH)
    subprocess.run(["g++", "-std=c++17", "-Wall", "-Wextra", "-Werror", "-o", exe,
                    os.path.join(host, "example_layer_loop.cpp"), "-L" + libdir, "-lmoe_gfx950",
                    "-Wl,-rpath," + libdir], check=True, capture_output=True)
    r = subprocess.run([exe], capture_output=True, text=True)
    assert r.returncode == 0, r.stdout + r.stderr
    assert "workspace for B=256" in r.stdout
    # the same program describes a checkpoint file in either on-disk format
    import ckptgen
    tensors = ckptgen.make_tensors(ckptgen.TINY, seed=1, mxfp4=False)
    ckptgen.write_bin(tmp_path / "m.bin", ckptgen.TINY, tensors)
    r = subprocess.run([exe, str(tmp_path / "m.bin")], capture_output=True, text=True)
    assert r.returncode == 0 and "3 layers, 4 experts, H=64, I=32, dense experts" in r.stdout, r.stdout
    ckptgen.write_safetensors(tmp_path / "m.safetensors", ckptgen.make_tensors(ckptgen.TINY, seed=1, mxfp4=True))
    r = subprocess.run([exe, str(tmp_path / "m.safetensors")], capture_output=True, text=True)
    assert r.returncode == 0 and "MXFP4 experts" in r.stdout, r.stdout
    r = subprocess.run([exe, str(tmp_path / "absent.bin")], capture_output=True, text=True)
    assert r.returncode == 2 and "cannot be opened" in r.stdout
