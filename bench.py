"""Benchmark of the MoE expert block on one MI355X.

A step is one pass of the whole block (router -> top-k -> softmax -> bucketing -> gate/up GEMM +
SwiGLU -> down GEMM -> combine) over one batch of synthetic tokens already resident in HBM.
Headline workload: the gpt-oss-20b-shaped block at 256-token decode with bf16 experts.

Prints ONE JSON line.  `roofline` describes the dominant kernel of the headline workload (the gate/up
GEMM, 2/3 of the weight bytes): algorithmic bytes (decode shapes; flops for the prefill shape) of that
launch / its average duration from HIP events recorded on the launch stream, against the 8 TB/s HBM
peak (2.5 PFLOP/s bf16 MFMA peak).  `roofline.practical_peak` is measured in the same run: a plain
streaming read of 4 GiB through the library's checksum kernel (every byte fetched once, nothing
written), so the gap between a kernel and what this device's memory sustains can be read off beside
the gap to the nominal figure.  `device` holds the CU count and the clocks the device reports.
`ms_per_step` is the wall-clock mean over the timed steps (preceded by max(--warmup, 100) untimed ones:
the device's step time needs about 40 steps to settle after a change of workload); `step_ms` adds the
median and the minimum of per-step HIP-event times.  Every workload under `also` carries the same objects for its own
launches; the MXFP4 decode workload also runs with three copies of its expert tensors used in turn
(1.3 GB, five times the 256 MB Infinity Cache) next to the single-copy figure, and the 36-layer stack
is also timed through the C++ forward() of host/moe_forward.hpp (host/bin/moe_stack_main synth, a child
process) beside the Python-driven loop.  `cpu_baseline` (one per workload) is the CPU oracle (the
OpenMP restatement of the reference's CPU path) timed on the host cores on a bounded 64-token sample;
nothing else in this file touches oracle/.
"""
import argparse
import importlib
import json
import os
import sys
import time

SETTLE_STEPS = 100  # untimed steps every single-block workload runs before its timed ones, at least
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
    ap.add_argument("--cpu-tokens", type=int, default=64, help="tokens of each workload the CPU baseline runs")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-cpp-stack", action="store_true", help="skip the C++ forward() timing of the stack workload")
    ap.add_argument("--peak-gib", type=int, default=4, help="size of the buffer the practical read peak is measured on")
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


def roofline_of(root, shape, res, read_peak):
    """The roofline object of one workload's gate/up launch.  `read_peak`: the measured streaming-read rate."""
    kname = res["kernels"]["gate_up"]
    bound = "mfma" if kname.startswith("expert_prefill") else "hbm"
    traffic, source = profiled_traffic(root, shape.name, kname)
    ms, nbytes, flops, what = res["mlp1"]["ms"], res["mlp1"]["bytes"], res["mlp1"]["flops"], "gate/up GEMM + SwiGLU"
    if kname.startswith("expert_fused"):  # one launch holds both GEMMs; its time is reported as the gate/up stage
        nbytes, flops, what = nbytes + res["mlp2"]["bytes"], flops + res["mlp2"]["flops"], "gate/up GEMM + SwiGLU + down GEMM"
    common = {"kernel": "%s (%s)" % (kname, what), "kernel_ms": ms, "traffic": traffic, "traffic_source": source,
              "algorithmic_bytes": nbytes, "algorithmic_flops": flops, "launches_per_step": res.get("layers", 1),
              "practical_peak": read_peak["best_gbs"], "practical_peak_unit": "GB/s",
              "practical_peak_source": read_peak["what"]}
    achieved_gbs = nbytes / (ms * 1e-3) / 1e9
    if bound == "hbm":
        return dict({"bound": "hbm", "achieved": achieved_gbs, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": achieved_gbs / HBM_PEAK_GBS, "frac_of_practical_peak": achieved_gbs / read_peak["best_gbs"]},
                    **common)
    achieved = flops / (ms * 1e-3) / 1e12
    return dict({"bound": "mfma", "achieved": achieved, "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s",
                 "frac": achieved / MFMA_BF16_PEAK_TFLOPS}, **common)


def device_info(pkg, torch):
    """What the device reports about itself: the peaks above are the part's published ones, not derived from this."""
    pr = torch.cuda.get_device_properties(0)
    a = pkg.device_attributes()
    return {"name": pr.name, "gcn_arch": getattr(pr, "gcnArchName", None), "compute_units": a["compute_units"],
            "clock_mhz": a["clock_khz"] / 1e3, "memory_clock_mhz": a["memory_clock_khz"] / 1e3,
            "memory_bus_bits": a["memory_bus_bits"], "l2_bytes": a["l2_bytes"], "hbm_bytes": pr.total_memory}


def measure_read_peak(pkg, torch, gib, launches=10):
    """Streaming-read rate of device memory: moe_synth_checksum over `gib` GiB of generator bytes, each launch
    timed with HIP events on the launch stream."""
    dev = torch.device("cuda:0")
    n = gib << 30
    buf = torch.empty(n, dtype=torch.uint8, device=dev)
    pkg.synth_bytes(buf, 1, 1)
    out = torch.empty(pkg.SYNTH_CHECKSUM_WORDS, dtype=torch.int64, device=dev)
    for _ in range(3):
        pkg.synth_checksum(buf, out=out)
    torch.cuda.synchronize()
    first = int(out[0].item())
    ev = [torch.cuda.Event(enable_timing=True) for _ in range(launches + 1)]
    ev[0].record()
    for i in range(launches):
        pkg.synth_checksum(buf, out=out)
        ev[i + 1].record()
    torch.cuda.synchronize()
    assert int(out[0].item()) == first, "checksum changed between launches"
    ms = sorted(ev[i].elapsed_time(ev[i + 1]) for i in range(launches))
    del buf, out
    torch.cuda.empty_cache()
    return {"bytes": n, "launches": launches, "best_gbs": n / (ms[0] * 1e-3) / 1e9,
            "median_gbs": n / (ms[launches // 2] * 1e-3) / 1e9, "nominal_gbs": HBM_PEAK_GBS,
            "what": "moe_synth_checksum over %d GiB (16-byte loads, every byte once, no stores), best of %d launches, "
                    "HIP events" % (gib, launches)}


def step_stats(torch, step, steps):
    """Per-step durations from HIP events recorded after every step on the launch stream."""
    ev = [torch.cuda.Event(enable_timing=True) for _ in range(steps + 1)]
    torch.cuda.synchronize()
    ev[0].record()
    for i in range(steps):
        step()
        ev[i + 1].record()
    torch.cuda.synchronize()
    ms = sorted(ev[i].elapsed_time(ev[i + 1]) for i in range(steps))
    return {"mean": sum(ms) / steps, "median": ms[steps // 2], "min": ms[0], "max": ms[-1], "steps": steps,
            "clock": "HIP events after every step"}


def launch_work(wl, shape, active):
    """Algorithmic bytes and flops of the two GEMM launches of one block."""
    H, I, T = shape.H, shape.I, shape.T
    wpe = wl.weight_bytes_per_expert(shape)
    w1_bytes = wpe * 2 // 3
    return {"mlp1": {"bytes": active * (w1_bytes + 2 * I * 2) + T * H * 4, "flops": shape.K * T * 2 * (2 * I * H)},
            "mlp2": {"bytes": active * (wpe - w1_bytes + H * 2) + T * H * 4, "flops": shape.K * T * 2 * (H * I)}}


def measure(pkg, wl, torch, shape, table, steps, warmup, flags=0, use_graph=False, rotate=0):
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
    stats = step_stats(torch, step, steps)

    # the same step with `rotate` separate copies of the layer's tensors used in turn, so that no step finds
    # the previous step's weights in the Infinity Cache
    rotating = None
    if rotate > 1:
        copies = [(blk, raw, p)]
        for _ in range(rotate - 1):
            b2, r2 = wl.make_device_layer(shape, table, dev)
            copies.append((b2, r2, b2.params(x, e_agg, topk_i, topk_v, flags=flags)))
        turn = [0]

        def rotating_step():
            b, _, q = copies[turn[0] % rotate]
            turn[0] += 1
            b.launch(q, stream)

        for _ in range(max(warmup, rotate)):
            rotating_step()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            rotating_step()
        torch.cuda.synchronize()
        rot_ms = (time.perf_counter() - t0) * 1e3 / steps
        rotating = {"copies": rotate, "ms_per_step": rot_ms, "step_ms": step_stats(torch, rotating_step, steps),
                    "weight_bytes_in_rotation": rotate * shape.E * wl.weight_bytes_per_expert(shape)}
        del copies

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
        "step_ms": stats,
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
    if rotating:
        rotating["block_hbm_frac"] = alg_bytes / (rotating["ms_per_step"] * 1e-3) / (HBM_PEAK_GBS * 1e9)
        res["rotating_weights"] = rotating
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
    stats = step_stats(torch, lambda: stack.forward(stream), steps)

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
           "steps": steps, "step_ms": stats, "driver": "one moe_block_forward_layers call per step from Python (workloads.DeviceStack)",
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


def cpp_stack(ge, shape, steps, warmup, flags):
    """The same synthetic stack through the C++ host side: host/bin/moe_stack_main synth builds it with the device
    generator and times forward() (host/moe_forward.hpp).  A child process: this one keeps its own device state."""
    import subprocess
    exe = os.path.join(ge.PKG_DIR, "host", "bin", "moe_stack_main")
    if not os.path.exists(exe):
        return {"error": "%s is missing (run __graft_entry__.build())" % exe}
    cmd = [exe, "synth"] + [str(v) for v in (shape.T, shape.H, shape.I, shape.E, shape.K, shape.layers, steps, warmup, flags)]
    r = subprocess.run(cmd, capture_output=True, text=True, timeout=600)
    if r.returncode != 0:
        return {"error": "moe_stack_main synth exited with %d: %s" % (r.returncode, (r.stdout + r.stderr)[-300:])}
    rec = json.loads(r.stdout.strip().splitlines()[-1])
    ms = rec["ms_per_forward_wall"]
    return {"driver": "C++ forward() of host/moe_forward.hpp (moe_stack_main synth, child process)",
            "ms_per_step": ms, "ms_per_step_events": rec["ms_per_forward_events"], "steps": steps,
            "tokens_per_s": shape.T / (ms * 1e-3)}


class CpuBaseline:
    """The CPU oracle on the first n tokens of a workload, all host threads.  The only place where this file loads
    oracle/ (and the host generator the tests use to feed it).  Expert tensors (fp32 on the host, as the reference's
    CPU path holds them) are generated for the experts the sample routes to and shared between workloads that have
    the same expert streams."""

    def __init__(self, ge, wl):
        sys.path.insert(0, os.path.join(ge.ROOT, "tests"))
        import hostgen
        self.hostgen, self.wl, self.oracle = hostgen, wl, ge.import_oracle()
        self.cache_key, self.cache = None, None

    def run(self, shape, n_tokens):
        import numpy as np
        hostgen, oracle, wl = self.hostgen, self.oracle, self.wl
        n_tokens = min(n_tokens, shape.T)
        t_gen = time.perf_counter()
        x = hostgen.host_input(oracle, wl, shape)[:n_tokens]
        small = hostgen.host_layer(oracle, wl, shape, experts=[])  # router and biases; expert tensors untouched
        # which experts the sample needs: the oracle's own router on the host weights
        needed = set()
        for t in range(n_tokens):
            scores = oracle.matmul(x[t], small["w_router"]) + small["b_router"]
            needed.update(int(e) for e in oracle.topk(scores, shape.K)[1])
        needed = sorted(needed)
        key = (shape.fmt, shape.H, shape.I, shape.E, shape.seed)
        if self.cache_key != key:
            self.cache, self.cache_key = None, key
        have = set() if self.cache is None else self.cache["experts"]
        todo = [e for e in needed if e not in have]
        if self.cache is None:
            hw = hostgen.host_layer(oracle, wl, shape, experts=todo)
            self.cache = {"experts": set(todo), "w_mlp1": hw["w_mlp1"], "w_mlp2": hw["w_mlp2"]}
        elif todo:
            hw = hostgen.host_layer(oracle, wl, shape, experts=todo)
            for e in todo:
                self.cache["w_mlp1"][e], self.cache["w_mlp2"][e] = hw["w_mlp1"][e], hw["w_mlp2"][e]
            self.cache["experts"].update(todo)
            del hw
        hw = dict(small, w_mlp1=self.cache["w_mlp1"], w_mlp2=self.cache["w_mlp2"])
        t_gen = time.perf_counter() - t_gen
        hostgen.oracle_block(oracle, shape, hw, x[:2])  # warm the pages
        t0 = time.perf_counter()
        hostgen.oracle_block(oracle, shape, hw, x)
        dt = time.perf_counter() - t0
        layers = shape.layers
        sample = ("%d tokens of %s through oracle/moe_oracle.c (fp32 weights, OpenMP over output rows), %.2f s%s; "
                  "%d of %d experts generated on the host in %.1f s"
                  % (n_tokens, shape.name, dt,
                     "" if layers == 1 else " for layer 0 of %d, scaled by the layer count" % layers,
                     len(needed), shape.E, t_gen))
        return {"value": n_tokens / (dt * layers), "unit": "tokens/s", "cores": oracle.max_threads(), "kind": "port",
                "sample": sample}


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

    device = device_info(pkg, torch)
    cpu = None if args.no_cpu_baseline else CpuBaseline(ge, wl)
    measured = []  # (shape, result) of every workload: the roofline objects are filled in once the read peak is known

    def run(shape, steps, warmup):
        if shape.layers > 1:
            # the stack: at least 20 timed steps (15 ms each)
            stack_steps = max(20, steps // 10)
            r = measure_stack(pkg, wl, torch, shape, table, stack_steps, 3)
            if not args.no_cpp_stack:
                r["cpp_forward"] = cpp_stack(ge, shape, stack_steps, 3, args.flags)
        else:
            # decode shapes whose experts fit the Infinity Cache a few times over also run with rotating copies
            small = shape.E * wl.weight_bytes_per_expert(shape) < (1 << 30)
            r = measure(pkg, wl, torch, shape, table, steps, warmup, args.flags, args.graph,
                        rotate=3 if (small and shape.fmt == "mxfp4" and shape.T <= 1024) else 0)
        r["cpu_baseline"] = cpu.run(shape, args.cpu_tokens) if cpu else None
        measured.append((shape, r))
        return r

    # Untimed steps before the timed ones: --warmup of them, and never fewer than SETTLE_STEPS.  After a change of
    # workload this device needs some 40 steps (15 ms) before its step time settles (the first launches run 3-7 %
    # slower: 0.30-0.31 ms against 0.293 for the headline workload, measured step by step), and a caller that asks
    # for five warm-up steps would otherwise time that transient instead of the workload.  The timed region is
    # unchanged: exactly --steps steps between two synchronisations.
    settle = max(SETTLE_STEPS, args.warmup)
    shape = wl.WORKLOADS[args.workload]
    head = run(shape, args.steps, settle)
    extra = [run(wl.WORKLOADS[name], args.steps, settle) for name in args.also.split(",") if name and name != args.workload]
    # The streaming-read probe runs last: where a workload's tensors land in device memory depends on what the process
    # allocated and freed before it, and the step time follows (the headline workload takes 0.291 ms as the first
    # allocation of its process and 0.300 ms behind the probe's 4 GiB buffer: one box, alternating runs with a pause
    # between them; the other workloads measure the same either way).
    read_peak = measure_read_peak(pkg, torch, args.peak_gib)
    for sh, r in measured:
        r["roofline"] = roofline_of(ge.ROOT, sh, r, read_peak)
    also = []
    for r in extra:
        keep = ("workload", "ms_per_step", "step_ms", "tokens_per_s", "block_hbm_frac", "block_mfma_frac",
                "block_algorithmic_bytes", "stage_ms", "rows_per_expert_min_max", "layers", "steps", "weights_gb", "driver",
                "cpp_forward", "rotating_weights", "kernels", "roofline", "cpu_baseline")
        also.append({k: r[k] for k in keep if k in r})

    out = {
        "metric": "MoE-block tokens/sec at 1 GPU; % HBM peak (decode), % bf16 MFMA peak (prefill)",
        "value": head["tokens_per_s"],
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "untimed_steps_before_timing": settle,
        "ms_per_step": head["ms_per_step"],
        "step_ms": head["step_ms"],
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": "%s: gpt-oss-20b-shaped MoE block, T=%d tokens, H=I=%d, E=%d, top-%d, %s experts"
                               % (shape.name, shape.T, shape.H, shape.E, shape.K, shape.fmt),
                   "tokens": shape.T, "active_experts": head.get("active_experts", shape.E)},
        "roofline": head["roofline"],
        "cpu_baseline": head["cpu_baseline"],
        "device": device,
        "read_peak": read_peak,
        "block_hbm_frac": head["block_hbm_frac"],
        "block_mfma_frac": head["block_mfma_frac"],
        "stage_ms": head["stage_ms"],
        "kernels": head["kernels"],
        "rotating_weights": head.get("rotating_weights"),
        "launch": "HIP graph replay of one moe_block_forward call" if args.graph else "plain launches",
        "also": also,
    }
    print(json.dumps(out))


if __name__ == "__main__":
    main()
