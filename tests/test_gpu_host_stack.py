"""The C++ host side on the device, as a separate process (host/bin/moe_stack_main, built by
__graft_entry__.build()): a checkpoint file written here goes through moe_host::moe_upload_weights,
moe_host::forward_layers / forward() (the reference's per-step entry, src/forward.cpp:202-204) and the
decode loop of host/moe_getp.hpp (src/getp/run.cpp:467-659).  The residual stream after every layer is
compared with the CPU oracle; the decode loop is followed step by step by a Python restatement of
src/getp/run.cpp:545-617 over the oracle's layer function, and its tokens and final states must not depend
on the batch size (compaction of the live batch, src/getp/run.cpp:573-588)."""
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
    assert "forward() with the reference's seven arguments: same bits; a group of two shards is refused" in r.stdout
    dump = np.fromfile(tmp_path / "out.f32", dtype=np.float32).reshape(L, T, H)
    x_in = x0
    for l in range(L):
        ref_x, ref_i, _ = oracle.moe_layer(x_in, *layer_weights(tensors, l, fmt == "mxfp4"), K)  # fed the GPU's own input
        d_ref, d_gpu = ref_x - x_in, dump[l] - x_in
        err = float(np.abs(d_gpu - d_ref).max() / np.abs(d_ref).max())
        print("  %s layer %d: rel err of the MoE contribution %.3e" % (fmt, l, err), flush=True)
        assert err <= OUT_TOL, (l, err)
        x_in = dump[l]


@pytest.mark.parametrize("scratch", ["own", "static"])
def test_cpp_dropin_wrappers_in_the_reference_call_order(oracle, dev, tmp_path, scratch):
    """Every layer's MoE half issued call by call through the reference-named wrappers of host/moe_kernels.hpp
    (gemm_router, topk, softmax, the three bucketing kernels, gather_rows, the work queue, moe_mlp1_swiglu,
    moe_mlp2_scatter, vecadd_and_zero: src/forward.cpp:315-514), with a registered router scratch buffer and with
    the library's fixed array; compared with the oracle layer by layer and with the one-call block."""
    path, kind, tensors = write_model(tmp_path, "bin_bf16")
    T, H, L, K = 45, CFG["hidden_size"], CFG["num_hidden_layers"], CFG["experts_per_token"]
    x0 = (np.random.default_rng(2).standard_normal((T, H)) * 1.5).astype(np.float32)
    x0.tofile(tmp_path / "x.f32")
    r = run("dropin", path, kind, tmp_path / "x.f32", T, tmp_path / "dropin.f32", scratch)
    assert r.returncode == 0, r.stdout + r.stderr
    r2 = run("layers", path, kind, tmp_path / "x.f32", T, tmp_path / "layers.f32")
    assert r2.returncode == 0, r2.stdout + r2.stderr
    dump = np.fromfile(tmp_path / "dropin.f32", dtype=np.float32).reshape(L, T, H)
    block = np.fromfile(tmp_path / "layers.f32", dtype=np.float32).reshape(L, T, H)
    x_in = x0
    for l in range(L):
        ref_x, _, _ = oracle.moe_layer(x_in, *layer_weights(tensors, l, False), K)  # fed this path's own input
        d_ref, d_gpu = ref_x - x_in, dump[l] - x_in
        err = float(np.abs(d_gpu - d_ref).max() / np.abs(d_ref).max())
        print("  dropin (%s scratch) layer %d: rel err of the MoE contribution %.3e" % (scratch, l, err), flush=True)
        assert err <= OUT_TOL, (l, err)
        x_in = dump[l]
    # against the one-call block on the same input: the fp32 intermediate and the atomic combine order differ
    d_blk, d_seq = block[0] - x0, dump[0] - x0
    assert float(np.abs(d_seq - d_blk).max() / np.abs(d_blk).max()) <= 5e-3


def test_cpp_dropin_router_refuses_without_a_scratch_buffer(dev, tmp_path):
    """No registered buffer and no opt-in to the library's fixed array: gemm_router returns MOE_ERR_WORKSPACE."""
    path, kind, _ = write_model(tmp_path, "bin_bf16")
    T, H = 9, CFG["hidden_size"]
    np.zeros((T, H), np.float32).tofile(tmp_path / "x.f32")
    r = run("dropin", path, kind, tmp_path / "x.f32", T, tmp_path / "o.f32", "none")
    assert r.returncode == 0, r.stdout + r.stderr
    assert "gemm_router without a scratch buffer -> -4" in r.stdout


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


# ---- the decode loop against an oracle-side loop -----------------------------------------------------

def initial_state_row(request, H):
    """The stand-in for a prompt's embedding (host/moe_getp.hpp): FNV-1a of the bytes seeds a 32-bit xorshift."""
    h = 2166136261
    for c in request.encode():
        h = ((h ^ c) * 16777619) & 0xFFFFFFFF
    if h == 0:
        h = 1
    row = np.empty(H, dtype=np.float32)
    for i in range(H):
        h ^= (h << 13) & 0xFFFFFFFF
        h ^= h >> 17
        h ^= (h << 5) & 0xFFFFFFFF
        row[i] = np.float32(h - (1 << 32) if h >= (1 << 31) else h) * np.float32(1.0 / 2147483648.0)
    return row


def oracle_generate(prompts, steps, vocab, eos, H, forward):
    """generate() of the reference's batch runtime (src/getp/run.cpp:467-659) for one batch, restated:
    prompt tokens are the request's bytes, sequence b owns state row b, a step runs `forward(step, indices,
    rows_in)` on the rows of the sequences still running, and commit_generation (:545-571) gives each its
    next prompt token or the first maximum of the moving logit window, and ends it at the end token or when
    the steps run out.  Returns (outputs, step_sizes, per-step records, final rows)."""
    B = len(prompts)
    prompt_tokens = [list(p.encode()) or [0] for p in prompts]
    rows = np.stack([initial_state_row(p, H) for p in prompts])
    current = [pt[0] for pt in prompt_tokens]
    pos = [0] * B
    finished = [False] * B
    out = [[] for _ in range(B)]
    step_sizes, records = [], []
    active = B

    def commit(b, token, counted):
        nonlocal active
        if counted and pos[b] - len(prompt_tokens[b]) >= 0:
            out[b].append(token)
        if (token == eos or pos[b] + 1 >= steps) and not finished[b]:
            finished[b] = True
            active -= 1
        current[b] = token

    it = 0
    while active > 0:
        idx = [b for b in range(B) if not finished[b] and pos[b] + 1 < steps]      # :573-583
        if not idx:
            break
        step_sizes.append(len(idx))
        tokens_in = [current[b] for b in idx]
        rows_in = rows[idx].copy()
        rows_out = forward(len(records), idx, rows_in)
        rows[idx] = rows_out
        window = (it * vocab) % (H - vocab + 1)
        it += 1
        margins = []
        for i, b in enumerate(idx):                                                   # :603-617
            pos[b] += 1
            if pos[b] < len(prompt_tokens[b]):
                commit(b, prompt_tokens[b][pos[b]], False)
                margins.append(np.inf)
            else:
                logits = rows_out[i, window:window + vocab]
                top = int(np.argmax(logits))                                          # first maximum
                rest = np.delete(logits, top)
                margins.append(float(logits[top] - rest.max()) if len(rest) else np.inf)
                commit(b, top, True)
        records.append(dict(indices=idx, window=window, tokens_in=tokens_in, rows_in=rows_in, rows_out=rows_out,
                            tokens_out=[current[b] for b in idx], margins=margins))
    return out, step_sizes, records, rows


def read_trace(path, H):
    raw = np.fromfile(path, dtype=np.int32)
    steps, o = [], 0
    while o < len(raw):
        n, window = int(raw[o]), int(raw[o + 1])
        o += 2
        idx = raw[o:o + n].tolist(); o += n
        tok_in = raw[o:o + n].tolist(); o += n
        rin = raw[o:o + n * H].view(np.float32).reshape(n, H); o += n * H
        rout = raw[o:o + n * H].view(np.float32).reshape(n, H); o += n * H
        tok_out = raw[o:o + n].tolist(); o += n
        steps.append(dict(indices=idx, window=window, tokens_in=tok_in, rows_in=rin, rows_out=rout, tokens_out=tok_out))
    return steps


LONG_PROMPTS = PROMPTS + ["a prompt that is longer than the step budget allows!"]


def test_cpp_decode_loop_vs_oracle_loop(oracle, dev, tmp_path):
    """`moe_stack_main getp` with a step trace against the loop restated in Python over oracle.moe_layer:
    (1) fed the GPU's own rows as forward results, the restated loop must reproduce the GPU program's live
    batches, tokens, step sizes and output file exactly (the loop logic, no arithmetic involved);
    (2) every step's rows: the oracle's layers on the GPU's input rows give the GPU's output rows within the
    block tolerance, and wherever the oracle's logit window has a margin above twice that row's error the GPU
    sampled the oracle's token;  (3) a prompt that does not fit the step budget generates nothing and leaves
    an empty line."""
    path, kind, tensors = write_model(tmp_path, "mxfp4")
    H, L, K = CFG["hidden_size"], CFG["num_hidden_layers"], CFG["experts_per_token"]
    prompts = LONG_PROMPTS
    with open(tmp_path / "in.txt", "w") as f:
        f.write("%d\n" % len(prompts))
        f.writelines(p + "\n" for p in prompts)
    steps, vocab, eos, batch = 28, 8, 3, len(prompts)
    r = run("getp", path, kind, tmp_path / "in.txt", tmp_path / "out.txt", steps, batch, vocab, eos, tmp_path / "fin.f32",
            tmp_path / "sz.txt", tmp_path / "trace.bin")
    assert r.returncode == 0, r.stdout + r.stderr
    trace = read_trace(tmp_path / "trace.bin", H)
    gpu_sizes = [int(v) for v in open(tmp_path / "sz.txt").read().split()]
    gpu_lines = open(tmp_path / "out.txt").read().split("\n")[:-1]
    gpu_tokens = [[int(t) for t in l.split()] for l in gpu_lines]
    gpu_final = np.fromfile(tmp_path / "fin.f32", dtype=np.float32).reshape(len(prompts), H)
    assert len(gpu_lines) == len(prompts) and len(trace) == len(gpu_sizes)
    # the request file reader cuts a line to its slot of 8 x (steps + 1) - 1 characters: none is that long here
    assert gpu_tokens[-1] == [], "a prompt as long as the step budget generates nothing"

    # (1) the loop logic, replaying the GPU's rows
    def replay(step, idx, rows_in):
        assert idx == trace[step]["indices"], ("live batch differs at step", step)
        assert np.array_equal(rows_in, trace[step]["rows_in"]), ("state rows differ at step", step)
        return trace[step]["rows_out"]

    out, sizes, records, final = oracle_generate(prompts, steps, vocab, eos, H, replay)
    assert sizes == gpu_sizes
    assert out == gpu_tokens
    assert np.array_equal(final, gpu_final)
    for rec, tr in zip(records, trace):
        assert rec["window"] == tr["window"] and rec["tokens_in"] == tr["tokens_in"] and rec["tokens_out"] == tr["tokens_out"]

    # (2) the arithmetic of every step against the oracle's layers
    weights = [layer_weights(tensors, l, True) for l in range(L)]

    def oracle_forward(x):
        for w in weights:
            x = oracle.moe_layer(x, *w, K)[0]
        return x

    worst, decided, undecided = 0.0, 0, 0
    for rec in records:
        ref = oracle_forward(rec["rows_in"])
        gpu = rec["rows_out"]
        err = float(np.abs(gpu - ref).max() / np.abs(ref - rec["rows_in"]).max())
        worst = max(worst, err)
        assert err <= OUT_TOL, err
        w = rec["window"]
        for i, m in enumerate(rec["margins"]):
            if not np.isfinite(m):
                continue  # a prompt token was taken
            logits = ref[i, w:w + vocab]
            top = int(np.argmax(logits))
            margin = float(logits[top] - np.delete(logits, top).max())
            row_err = float(np.abs(gpu[i] - ref[i]).max())
            if margin > 2 * row_err:
                assert rec["tokens_out"][i] == top
                decided += 1
            else:
                undecided += 1
    print("  decode loop: %d steps, worst rel err of a step %.3e, %d sampled tokens pinned by the oracle, %d too close "
          "to call" % (len(records), worst, decided, undecided), flush=True)
    assert decided > 4 * max(1, undecided)


def test_cpp_synthetic_stack_equals_the_python_driven_stack(pkg, wl, dev):
    """`moe_stack_main synth` builds the synthetic MXFP4 stack the benchmark times (device generator, same stream ids)
    and runs it through the C++ forward(); the Python-driven DeviceStack over the same tensors must leave the same
    residual stream bit for bit (compared through moe_synth_checksum, which both sides compute on the device)."""
    import json
    import torch
    shape = wl.MoeShape("synth_small", T=48, H=256, I=128, E=8, K=2, fmt="mxfp4", layers=3)
    r = run("synth", shape.T, shape.H, shape.I, shape.E, shape.K, shape.layers, 2, 1)
    assert r.returncode == 0, r.stdout + r.stderr
    rec = json.loads(r.stdout.strip().splitlines()[-1])
    assert rec["layers"] == 3 and rec["ms_per_forward_events"] > 0 and rec["ms_per_forward_wall"] > 0
    table = pkg.normal_table()
    stack = wl.DeviceStack(shape, table, dev)
    x = wl.make_device_input(shape, table, dev)
    stack.prepare(x)
    stack.forward()
    torch.cuda.synchronize()
    assert bool(torch.isfinite(x).all()) and float(x.abs().max()) > 0
    got = int(pkg.synth_checksum(x)[0].item()) & ((1 << 64) - 1)
    assert got == rec["x_checksum_after_first_forward"]
