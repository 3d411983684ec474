"""Benchmark of the MoE expert block on one MI355X.

A step is one pass of the whole block (router -> top-k -> softmax -> bucketing -> gate/up GEMM +
SwiGLU -> down GEMM -> combine) over one batch of synthetic tokens already resident in HBM.
Headline workload: the gpt-oss-20b-shaped block at 256-token decode with bf16 experts.

Prints ONE JSON line.  `roofline` describes the dominant kernel of the headline workload (the gate/up
GEMM, 2/3 of the weight bytes): algorithmic bytes (decode shapes; flops for the prefill shape) of that
launch / its average duration from HIP events recorded on the launch stream, against the 8 TB/s HBM
peak (2.5 PFLOP/s bf16 MFMA peak).  Every workload under `also` carries the same object for its own
gate/up launch.  `cpu_baseline` is the CPU oracle (the OpenMP restatement of the reference's CPU
path) timed on the host cores on a bounded sample; nothing else in this file touches oracle/.
"""
import argparse
import importlib
import json
import os
import sys
import time

HBM_PEAK_GBS = 8000.0
MFMA_BF16_PEAK_TFLOPS = 2500.0


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default="decode256_bf16")
    ap.add_argument("--also", default="decode256_mxfp4,prefill4096_mxfp4_zipf,stack120b_mxfp4",
                    help="comma-separated extra workloads reported under 'also' ('' for none)")
    ap.add_argument("--cpu-tokens", type=int, default=256, help="tokens of the workload the CPU baseline runs")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--flags", type=int, default=0)
    ap.add_argument("--copy-calibration", action="store_true",
                    help="first run five plain 1 GiB device-to-device copies (a kernel of known traffic: 1 GiB read, "
                         "1 GiB written) so that rocprofv3 FETCH_SIZE / WRITE_SIZE readings can be scaled")
    ap.add_argument("--graph", action="store_true",
                    help="replay a captured HIP graph of one moe_block_forward call per step instead of plain launches "
                         "(measured: no faster, the kernels' own dependent latencies dominate)")
    return ap.parse_args()


def kernel_prefix(name):
    """Profiler-style kernel name up to the template arguments that identify it ("expert_x<1, 0")."""
    head, _, args = name.partition("<")
    return head + "<" + ", ".join(a.strip() for a in args.split(",")[:2])


def profiled_traffic(root, workload, kernel_name):
    """HBM-side bytes per launch of `kernel_name` from the committed rocprofv3 counter summary
    profiles/moe_block_<workload>.txt: 2 x FETCH_SIZE + WRITE_SIZE in KiB, the factors coming from the
    plain-copy calibration recorded in that file.  (None, reason) when the summary does not hold this
    kernel, which is what happens when the kernels changed after the summary was taken."""
    rel = os.path.join("profiles", "moe_block_%s.txt" % workload)
    path = os.path.join(root, rel)
    if not os.path.exists(path):
        return None, "no counter summary %s" % rel
    want = kernel_name.split("(")[0].strip()
    section, vals = None, {}
    for line in open(path):
        if line.startswith("== FETCH_SIZE"):
            section = "fetch"
        elif line.startswith("== WRITE_SIZE"):
            section = "write"
        elif line.startswith("=="):
            section = None
        elif section and line.startswith(want) and section not in vals:
            vals[section] = float(line.split("avg")[-1])
    if "fetch" not in vals or "write" not in vals:
        return None, "%s has no FETCH_SIZE / WRITE_SIZE rows for %s" % (rel, want)
    return (2.0 * vals["fetch"] + vals["write"]) * 1024.0, "%s (rocprofv3 --pmc runs, not measured in this run)" % rel


def roofline_of(root, shape, res):
    """The roofline object of one workload's gate/up launch."""
    bound = "mfma" if res["kernels"]["gate_up"].startswith("expert_prefill") else "hbm"
    kname = res["kernels"]["gate_up"]
    traffic, source = profiled_traffic(root, shape.name, kname)
    ms = res["mlp1"]["ms"]
    common = {"kernel": kname + " (gate/up GEMM + SwiGLU)", "kernel_ms": ms, "traffic": traffic, "traffic_source": source,
              "algorithmic_bytes": res["mlp1"]["bytes"], "algorithmic_flops": res["mlp1"]["flops"],
              "launches_per_step": res.get("layers", 1)}
    if bound == "hbm":
        achieved = res["mlp1"]["bytes"] / (ms * 1e-3) / 1e9
        return dict({"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": achieved / HBM_PEAK_GBS}, **common)
    achieved = res["mlp1"]["flops"] / (ms * 1e-3) / 1e12
    return dict({"bound": "mfma", "achieved": achieved, "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s",
                 "frac": achieved / MFMA_BF16_PEAK_TFLOPS}, **common)


def launch_work(wl, shape, active):
    """Algorithmic bytes and flops of the two GEMM launches of one block."""
    H, I, T = shape.H, shape.I, shape.T
    wpe = wl.weight_bytes_per_expert(shape)
    w1_bytes = wpe * 2 // 3
    return {"mlp1": {"bytes": active * (w1_bytes + 2 * I * 2) + T * H * 4, "flops": shape.K * T * 2 * (2 * I * H)},
            "mlp2": {"bytes": active * (wpe - w1_bytes + H * 2) + T * H * 4, "flops": shape.K * T * 2 * (H * I)}}


def measure(pkg, wl, torch, shape, table, steps, warmup, flags=0, use_graph=False):
    """Returns a dict of measurements for one single-block workload on cuda:0."""
    dev = torch.device("cuda:0")
    blk, raw = wl.make_device_layer(shape, table, dev)
    x = wl.make_device_input(shape, table, dev)
    T = shape.T
    e_agg = torch.empty((T, shape.H), dtype=torch.float32, device=dev)
    topk_i = torch.empty((T, shape.K), dtype=torch.int32, device=dev)
    topk_v = torch.empty((T, shape.K), dtype=torch.float32, device=dev)
    p = blk.params(x, e_agg, topk_i, topk_v, flags=flags)
    stream = torch.cuda.current_stream().cuda_stream

    # One step = one moe_block_forward call.  The entry allocates nothing and never synchronises, so a
    # serving loop can also capture it once and replay it (--graph).
    for _ in range(3):
        blk.launch(p, stream)
    torch.cuda.synchronize()
    graph = None
    if use_graph:
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            blk.launch(p, torch.cuda.current_stream().cuda_stream)
        torch.cuda.synchronize()

    def step():
        if graph is not None:
            graph.replay()
        else:
            blk.launch(p, stream)

    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    ms_per_step = (t1 - t0) * 1e3 / steps

    # second pass with HIP events at the stage boundaries (same stream)
    timer = pkg.StageTimer()
    stage_ms = [0.0] * len(pkg.STAGES)
    for _ in range(steps):
        timer.launch(p, stream)
        for i, v in enumerate(timer.read()):
            stage_ms[i] += v / steps
    timer.close()

    counts = torch.bincount(topk_i.flatten().long(), minlength=shape.E).cpu().numpy()
    active = int((counts > 0).sum())
    alg_bytes = wl.algorithmic_bytes(shape, active)
    alg_flops = wl.algorithmic_flops(shape)
    work = launch_work(wl, shape, active)
    res = {
        "workload": shape.name,
        "ms_per_step": ms_per_step,
        "tokens_per_s": T / (ms_per_step * 1e-3),
        "stage_ms": dict(zip(pkg.STAGES, [round(v, 5) for v in stage_ms])),
        "active_experts": active,
        "rows_per_expert_min_max": [int(counts.min()), int(counts.max())],
        "block_algorithmic_bytes": alg_bytes,
        "block_hbm_frac": alg_bytes / (ms_per_step * 1e-3) / (HBM_PEAK_GBS * 1e9),
        "block_mfma_frac": alg_flops / (ms_per_step * 1e-3) / (MFMA_BF16_PEAK_TFLOPS * 1e12),
        "kernels": blk.describe(p),
        "mlp1": dict(work["mlp1"], ms=stage_ms[3]),
        "mlp2": dict(work["mlp2"], ms=stage_ms[4]),
    }
    del blk, raw, x
    torch.cuda.empty_cache()
    return res


def measure_stack(pkg, wl, torch, shape, table, steps, warmup):
    """The 36-layer 120b-shaped stack: one step = all layers (rmsnorm -> MoE block -> residual)."""
    dev = torch.device("cuda:0")
    stack = wl.DeviceStack(shape, table, dev)
    x = wl.make_device_input(shape, table, dev)
    x0 = x.clone()
    stack.prepare(x)
    stream = torch.cuda.current_stream().cuda_stream
    for _ in range(warmup):
        x.copy_(x0)
        stack.forward(stream)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        stack.forward(stream)  # activations keep evolving; routing stays data-dependent and realistic
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) * 1e3 / steps

    # per-stage durations: every layer's launch with HIP events, averaged over the layers of a few passes
    timer = pkg.StageTimer()
    stage_ms = [0.0] * len(pkg.STAGES)
    passes = 2
    x.copy_(x0)
    pkg.rmsnorm(stack.t, stack.x, stack.rms_w, shape.T, shape.H, stream=stream)
    for _ in range(passes):
        for l in range(shape.layers):
            timer.launch(stack.params[l], stream)
            for i, v in enumerate(timer.read()):
                stage_ms[i] += v / (passes * shape.layers)
    timer.close()
    active = shape.E  # every expert of every layer is used at 1024 tokens x top-4 over 128 experts
    alg_bytes = wl.algorithmic_bytes(shape) * shape.layers
    alg_flops = wl.algorithmic_flops(shape) * shape.layers
    work = launch_work(wl, shape, active)
    res = {"workload": shape.name, "ms_per_step": ms, "tokens_per_s": shape.T / (ms * 1e-3), "layers": shape.layers,
           "steps": steps,
           "stage_ms": dict(zip(pkg.STAGES, [round(v, 5) for v in stage_ms])),
           "block_algorithmic_bytes": alg_bytes,
           "block_hbm_frac": alg_bytes / (ms * 1e-3) / (HBM_PEAK_GBS * 1e9),
           "block_mfma_frac": alg_flops / (ms * 1e-3) / (MFMA_BF16_PEAK_TFLOPS * 1e12),
           "weights_gb": round(shape.layers * shape.E * wl.weight_bytes_per_expert(shape) / 1e9, 2),
           "kernels": stack.blocks[0].describe(stack.params[0]),
           "mlp1": dict(work["mlp1"], ms=stage_ms[3]),
           "mlp2": dict(work["mlp2"], ms=stage_ms[4])}
    del stack
    torch.cuda.empty_cache()
    return res


def cpu_baseline(ge, wl, shape, n_tokens):
    """The CPU oracle on the first n_tokens of the workload, all host threads.  The only place where
    this file loads oracle/ (and the host generator the tests use to feed it)."""
    sys.path.insert(0, os.path.join(ge.ROOT, "tests"))
    import hostgen
    oracle = ge.import_oracle()
    hw = hostgen.host_layer(oracle, wl, shape)
    x = hostgen.host_input(oracle, wl, shape)[:n_tokens]
    hostgen.oracle_block(oracle, shape, hw, x[:2])  # warm the pages
    t0 = time.perf_counter()
    hostgen.oracle_block(oracle, shape, hw, x)
    dt = time.perf_counter() - t0
    return {"value": n_tokens / dt, "unit": "tokens/s", "cores": oracle.max_threads(), "kind": "port",
            "sample": "%d tokens of %s through oracle/moe_oracle.c (fp32 weights, OpenMP over output rows), %.2f s"
                      % (n_tokens, shape.name, dt)}


def main():
    args = parse()
    if args.gpus != 1:
        print("bench.py measures one MI355X; --gpus %d is not supported (the MoE block is built for a single GPU: "
              "no expert parallelism, no collectives)" % args.gpus, file=sys.stderr)
        sys.exit(2)
    import torch
    import __graft_entry__ as ge
    pkg = ge.import_package()
    wl = importlib.import_module("gpt_oss_amd_amd.workloads")
    table = pkg.normal_table()  # the synthetic generator's quantile table, built by the library

    if args.copy_calibration:
        src = torch.zeros(1 << 30, dtype=torch.uint8, device="cuda:0")
        dst = torch.empty_like(src)
        for _ in range(5):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
        torch.cuda.empty_cache()

    def run(shape, steps, warmup):
        if shape.layers > 1:
            # the stack: at least 20 timed steps (15 ms each)
            r = measure_stack(pkg, wl, torch, shape, table, max(20, steps // 10), 3)
        else:
            r = measure(pkg, wl, torch, shape, table, steps, warmup, args.flags, args.graph)
        r["roofline"] = roofline_of(ge.ROOT, shape, r)
        return r

    shape = wl.WORKLOADS[args.workload]
    head = run(shape, args.steps, args.warmup)

    also = []
    for name in [n for n in args.also.split(",") if n and n != args.workload]:
        # same step count as the headline workload, and at least 100 warm-up steps: the 0.12 ms MXFP4
        # decode step is 3 % slower in the first few milliseconds after a change of workload
        r = run(wl.WORKLOADS[name], args.steps, max(100, args.warmup))
        keep = ("workload", "ms_per_step", "tokens_per_s", "block_hbm_frac", "block_mfma_frac", "block_algorithmic_bytes",
                "stage_ms", "rows_per_expert_min_max", "layers", "steps", "weights_gb", "kernels", "roofline")
        also.append({k: r[k] for k in keep if k in r})

    cpu = None
    if not args.no_cpu_baseline:
        cpu = cpu_baseline(ge, wl, shape, min(args.cpu_tokens, shape.T))

    out = {
        "metric": "MoE-block tokens/sec at 1 GPU; % HBM peak (decode), % bf16 MFMA peak (prefill)",
        "value": head["tokens_per_s"],
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": head["ms_per_step"],
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": "%s: gpt-oss-20b-shaped MoE block, T=%d tokens, H=I=%d, E=%d, top-%d, %s experts"
                               % (shape.name, shape.T, shape.H, shape.E, shape.K, shape.fmt),
                   "tokens": shape.T, "active_experts": head.get("active_experts", shape.E)},
        "roofline": head["roofline"],
        "cpu_baseline": cpu,
        "block_hbm_frac": head["block_hbm_frac"],
        "block_mfma_frac": head["block_mfma_frac"],
        "stage_ms": head["stage_ms"],
        "kernels": head["kernels"],
        "launch": "HIP graph replay of one moe_block_forward call" if args.graph else "plain launches",
        "also": also,
    }
    print(json.dumps(out))


if __name__ == "__main__":
    main()
