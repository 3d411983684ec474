"""The C++ host side on the device, as a separate process (host/bin/moe_stack_main, built by
__graft_entry__.build()): a checkpoint file written here goes through moe_host::moe_upload_weights,
moe_host::forward_layers / forward() (the reference's per-step entry, src/forward.cpp:202-204) and the
decode loop of host/moe_getp.hpp (src/getp/run.cpp:467-659).  The residual stream after every layer is
compared with the CPU oracle; the decode loop's tokens and final states must not depend on the batch
size (compaction of the live batch, src/getp/run.cpp:573-588)."""
import os
import subprocess

import numpy as np
import pytest

import ckptgen
from conftest import ROOT

pytestmark = pytest.mark.gpu

EXE = os.path.join(ROOT, "gpt-oss-amd_amd", "host", "bin", "moe_stack_main")
OUT_TOL = 1e-2  # max|y - ref| / max|ref| of a layer's MoE contribution

CFG = dict(ckptgen.TINY, hidden_size=128, intermediate_size=64, num_experts=8, experts_per_token=4,
           num_hidden_layers=3)


def run(*args):
    assert os.path.exists(EXE), "%s is missing: run __graft_entry__.build()" % EXE
    print("run:", " ".join(str(a) for a in args), flush=True)
    return subprocess.run([EXE] + [str(a) for a in args], capture_output=True, text=True, timeout=120)


def write_model(tmp_path, fmt):
    if fmt == "mxfp4":
        tensors = ckptgen.make_tensors(CFG, seed=5, mxfp4=True)
        path = tmp_path / "model.safetensors"
        ckptgen.write_safetensors(path, tensors)
        return path, "safetensors:%d" % CFG["experts_per_token"], tensors
    tensors = ckptgen.make_tensors(CFG, seed=5, mxfp4=False)
    path = tmp_path / "model.bin"
    ckptgen.write_bin(path, CFG, tensors, bf16=(fmt == "bin_bf16"))
    return path, fmt, tensors


def layer_weights(tensors, l, mxfp4):
    p = "block.%d.mlp." % l
    if mxfp4:
        w1 = ckptgen.mxfp4_dequant(tensors[p + "mlp1_weight.blocks"], tensors[p + "mlp1_weight.scales"])
        w2 = ckptgen.mxfp4_dequant(tensors[p + "mlp2_weight.blocks"], tensors[p + "mlp2_weight.scales"])
    else:
        w1, w2 = tensors[p + "mlp1_weight"], tensors[p + "mlp2_weight"]
    return (tensors[p + "norm.scale"], tensors[p + "gate.weight"], tensors[p + "gate.bias"], w1, tensors[p + "mlp1_bias"],
            w2, tensors[p + "mlp2_bias"])


@pytest.mark.parametrize("fmt", ["bin_f32", "bin_bf16", "mxfp4"])
def test_cpp_forward_layer_by_layer_vs_oracle(oracle, dev, tmp_path, fmt):
    path, kind, tensors = write_model(tmp_path, fmt)
    T, H, L, K = 45, CFG["hidden_size"], CFG["num_hidden_layers"], CFG["experts_per_token"]
    x0 = (np.random.default_rng(2).standard_normal((T, H)) * 1.5).astype(np.float32)
    x0.tofile(tmp_path / "x.f32")
    r = run("layers", path, kind, tmp_path / "x.f32", T, tmp_path / "out.f32")
    assert r.returncode == 0, r.stdout + r.stderr
    assert "forward() equals the layer-by-layer result bit for bit" in r.stdout
    dump = np.fromfile(tmp_path / "out.f32", dtype=np.float32).reshape(L, T, H)
    x_in = x0
    for l in range(L):
        ref_x, ref_i, _ = oracle.moe_layer(x_in, *layer_weights(tensors, l, fmt == "mxfp4"), K)  # fed the GPU's own input
        d_ref, d_gpu = ref_x - x_in, dump[l] - x_in
        err = float(np.abs(d_gpu - d_ref).max() / np.abs(d_ref).max())
        print("  %s layer %d: rel err of the MoE contribution %.3e" % (fmt, l, err), flush=True)
        assert err <= OUT_TOL, (l, err)
        x_in = dump[l]


PROMPTS = ["abc", "hello", "xy", "prompt!", "q", "seven77", "ab", "longer one"]


def test_cpp_decode_loop_is_batch_invariant(dev, tmp_path):
    path, kind, _ = write_model(tmp_path, "mxfp4")
    with open(tmp_path / "in.txt", "w") as f:
        f.write("%d\n" % len(PROMPTS))
        f.writelines(p + "\n" for p in PROMPTS)
    steps, vocab, eos = 28, 8, 3
    outs = {}
    for batch in (8, 1, 3):
        out, fin, sizes = tmp_path / ("out%d.txt" % batch), tmp_path / ("fin%d.f32" % batch), tmp_path / ("sz%d.txt" % batch)
        r = run("getp", path, kind, tmp_path / "in.txt", out, steps, batch, vocab, eos, fin, sizes)
        assert r.returncode == 0, r.stdout + r.stderr
        outs[batch] = (open(out).read(), np.fromfile(fin, dtype=np.float32), [int(s) for s in open(sizes).read().split()])
    text8, fin8, sizes8 = outs[8]
    lines = text8.split("\n")[:-1]
    assert len(lines) == len(PROMPTS)
    toks = [[int(t) for t in l.split()] for l in lines]
    for p, t in zip(PROMPTS, toks):
        # a sequence generates until it samples the end token or runs out of steps (src/getp/run.cpp:556-558)
        assert 1 <= len(t) <= steps - len(p)
        assert all(0 <= v < vocab for v in t) and eos not in t[:-1]
        assert t[-1] == eos or len(t) == steps - len(p)
    # the live batch shrinks as sequences finish, and never grows
    assert sizes8[0] == len(PROMPTS) and sizes8[-1] < len(PROMPTS)
    assert all(a >= b for a, b in zip(sizes8, sizes8[1:]))
    assert len({len(t) + len(p) for p, t in zip(PROMPTS, toks)}) > 2, "sequences should finish at different steps"
    # one request at a time, or three: same tokens (the reference's verifier), same final state bits
    for batch in (1, 3):
        text, fin, sizes = outs[batch]
        r = run("verify", tmp_path / ("out%d.txt" % batch), tmp_path / "out8.txt")
        assert r.returncode == 0, r.stdout
        assert text == text8
        assert np.array_equal(fin.view(np.uint32), fin8.view(np.uint32)), "state rows depend on the batch size"
        assert max(sizes) <= batch
