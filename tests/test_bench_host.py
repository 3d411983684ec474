"""Host-side pieces of bench.py that need no GPU: the committed counter summaries must stay readable by the
traffic parser, --gpus above 1 must be refused, and the work figures that the roofline fractions are computed from
must be the ones the workload module publishes."""
import importlib.util
import os
import subprocess
import sys

import pytest

from conftest import ROOT


@pytest.fixture(scope="module")
def bench():
    spec = importlib.util.spec_from_file_location("bench_under_test", os.path.join(ROOT, "bench.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


@pytest.mark.parametrize("workload,kernel,lo,hi", [
    ("decode256_bf16", "expert_stream_direct_kernel<0, 0, 12, 2, false>", 1.0, 1.15),
    ("decode256_mxfp4", "expert_stream_direct_kernel<1, 0, 12, 2, true>", 1.0, 1.2),
    ("stack120b_mxfp4", "expert_stream_direct_kernel<1, 0, 12, 2, true>", 1.0, 1.4),
    ("prefill4096_mxfp4_zipf", "expert_prefill_kernel<1, 0, 4>", 2.0, 6.0),
])
def test_committed_profiles_give_the_traffic_of_the_gate_up_launch(bench, wl, workload, kernel, lo, hi):
    traffic, source = bench.profiled_traffic(ROOT, workload, kernel)
    assert traffic is not None, source
    assert source.startswith("profiles/moe_block_%s.txt" % workload)
    shape = wl.WORKLOADS[workload]
    alg = bench.launch_work(wl, shape, shape.E)["mlp1"]["bytes"]
    # measured HBM-side bytes of the launch against its algorithmic bytes: above 1, and within the range the
    # design document discusses for that kernel family
    assert lo <= traffic / alg <= hi, (traffic, alg)


def test_a_kernel_the_summary_does_not_hold_is_reported_not_guessed(bench):
    traffic, why = bench.profiled_traffic(ROOT, "decode256_bf16", "no_such_kernel<1>")
    assert traffic is None and "no FETCH_SIZE / WRITE_SIZE rows" in why
    traffic, why = bench.profiled_traffic(ROOT, "no_such_workload", "k")
    assert traffic is None and "no counter summary" in why


def test_more_than_one_gpu_is_refused():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True,
                       timeout=120)
    assert r.returncode == 2 and "one MI355X" in r.stderr and r.stdout.strip() == ""


def test_launch_work_adds_up_to_the_block(bench, wl):
    for name in ("decode256_bf16", "decode256_mxfp4", "stack120b_mxfp4"):
        shape = wl.WORKLOADS[name]
        work = bench.launch_work(wl, shape, shape.E)
        wpe = wl.weight_bytes_per_expert(shape)
        # both launches together: every expert's weights and biases once, the rows in and out once per launch
        total = work["mlp1"]["bytes"] + work["mlp2"]["bytes"]
        assert total == shape.E * (wpe + (2 * shape.I + shape.H) * 2) + 2 * shape.T * shape.H * 4
        assert work["mlp1"]["flops"] == 2 * work["mlp2"]["flops"]
