"""Host-side pieces of bench.py that need no GPU: the description of the host CPU that goes into cpu_baseline, and the
lookup of measured HBM traffic, which must answer None unless the kernel that ran is the one the figure was measured on."""
import json
import os
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)


def test_host_cpu_description():
    import bench
    c = bench.host_cpu()
    assert c["cpu_model"] and c["physical_cores_per_socket"] >= 1 and c["sockets"] >= 1 and c["numa_nodes"] >= 1
    assert c["physical_cores_per_socket"] * c["sockets"] <= c["logical_cpus"]


def test_measured_traffic_is_tied_to_the_kernel():
    import bench
    table = json.load(open(bench.TRAFFIC_FILE))
    for name, e in table["workloads"].items():
        assert name in bench.WORKLOADS
        assert e["hbm_bytes_per_launch"] == (e["fetch_kib"] + e["write_kib"]) * 1024
        assert bench.measured_traffic(name, e["kernel"]) == e["hbm_bytes_per_launch"]
        assert bench.measured_traffic(name, "some_other_kernel") is None
        assert os.path.exists(os.path.join(ROOT, e["summary"]))
    assert bench.measured_traffic("c1_fp32", "reduce_vec_kernel") is None or "c1_fp32" in table["workloads"]
    assert bench.measured_traffic("no_such_workload", "copy_kernel") is None


def test_other_workloads_schema():
    """The five entries a default run adds under "other_workloads", and the keys of an entry."""
    import bench
    assert bench.OTHER_WORKLOADS == ("c1_fp32", "c2_bf16", "c5_fp32", "c4_fused", "c4_three_step")
    e = bench.other_entry("c1_fp32", 0.0323, 201_326_592, "reduce_vec_kernel", 64, "bit-exact vs oracle: every element")
    assert tuple(e) == bench.OTHER_KEYS
    assert e["GBps"] == round(201_326_592 / 0.0323e-3 / 1e9, 1) and abs(e["frac"] - e["GBps"] / 8000.0) < 1e-4
    assert e["traffic"] == bench.measured_traffic("c1_fp32", "reduce_vec_kernel")
    assert bench.other_entry("c1_fp32", 1.0, 1, "another_kernel", 1, "")["traffic"] is None
    assert bench.other_entry("c4_three_step", 1.0, 1, "fusion_copy_kernel + reduce_multi_kernel + fusion_copy_kernel", 1, "")["traffic"] is None
    src = open(bench.__file__).read()
    for name in bench.OTHER_WORKLOADS:
        assert f'"{name}"' in src
