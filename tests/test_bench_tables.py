"""bench.py's table of measured HBM traffic (profiles/hbm_traffic.json) must describe the kernels that run now:
for the workloads whose dominant kernel has a geometry query, the recorded signature equals what the library
reports for that workload's row length, so a change of launch shape without a fresh measurement fails here
instead of printing a stale figure. No GPU needed."""
import json
import os

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def bench():
    import importlib.util

    spec = importlib.util.spec_from_file_location("bench_module", os.path.join(ROOT, "bench.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


# workload -> (row length, geometry kind of nhp_softmax_geometry, signature prefix)
GEOMETRY_WORKLOADS = {
    "pythia-1.4b": (2048, 2, "softmax_bwd causal "),
    "llama2-7b-c5": (8192, 2, "softmax_bwd causal "),
    "mistral-window": (8192, 2, "softmax_bwd causal "),
    "masked-c3": (2048, 4, "softmax_bwd plain "),
}


def test_traffic_table_matches_the_running_kernels(hotpath, bench):
    table = json.load(open(bench.TRAFFIC_TABLE))["workloads"]
    lib = hotpath.lib()
    for workload, (n, kind, prefix) in GEOMETRY_WORKLOADS.items():
        assert workload in table, workload
        now = prefix + bench.softmax_signature(lib, n, kind)
        assert table[workload]["signature"] == now, (workload, table[workload]["signature"], now)
        assert bench.measured_traffic(workload, now) == table[workload]["bytes"]
        # measured traffic can only exceed what the algorithm has to move, and not by much
        assert bench.measured_traffic(workload, now + " other") is None
    for workload, entry in table.items():
        assert os.path.exists(os.path.join(ROOT, "profiles", entry["source"])), entry["source"]
        assert entry["bytes"] > 0
    assert bench.measured_traffic("no-such-workload", "x") is None


def test_algorithmic_byte_formulas(bench):
    # the figures stated in the scope table for the Pythia-1.4B and Llama-2-7B shapes
    assert bench.causal_bytes(128, 2048) == (1610874880, 2148007936)
    assert bench.causal_bytes(64, 8192) == (12885426176, 17180917760)
    assert bench.rope_bytes(2048, 8, 16, 128, 32) == 134479872
    assert bench.tri(2048) == 2048 * 2049 // 2


@pytest.mark.gpu
def test_bench_measures_a_configuration_and_releases_its_tensors(bench):
    """bench.py's per-configuration measurement (what fills the `configs` object of its default line) on its two
    smallest workloads: every kernel reports bytes, a positive bracket and a fraction of the peak below 1, the
    16 launches of the [4,8,512,512] bracket are divided out, and the tensors are released afterwards."""
    import torch

    dev = torch.device("cuda:0")
    torch.cuda.synchronize()
    before = torch.cuda.memory_allocated(dev)
    c1 = bench.measure_workload("causal-c1", torch, dev, steps=2, warmup=1)
    k = c1["kernels"]["causal_softmax_fwd"]
    assert k["bytes"] == bench.causal_bytes(32, 512)[0] == 25182208
    assert 1.0 < k["us"] < 100.0 and 0.0 < k["frac_of_peak"] < 1.0
    rope = bench.measure_workload("rope-styles-1.4b", torch, dev, steps=2, warmup=1)
    assert set(rope["kernels"]) == {"rope_fwd_per_tensor", "rope_bwd_per_tensor", "rope_fwd_one_launch", "rope_bwd_one_launch"}
    for v in rope["kernels"].values():
        assert v["bytes"] > 2 * 2048 * 8 * 16 * 128 * 2 * 2 and 10.0 < v["us"] < 1000.0 and 0.0 < v["frac_of_peak"] < 1.0
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated(dev) <= before + (1 << 20)
