"""Runs the C++ self-checking harness (tests/cpp/ep_selftest), which drives include/mi_ep.hpp the
way the reference's main() drives its classes and prints the reference's one-JSON-object protocol."""
import json
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BINARY = os.path.join(ROOT, "tests", "cpp", "ep_selftest")


@pytest.mark.gpu
def test_selftest_binary_passes():
    assert os.path.exists(BINARY), "build with `make -C tests/cpp` (done by __graft_entry__.build())"
    proc = subprocess.run([BINARY], capture_output=True, text=True, timeout=300)
    print(proc.stderr)
    report = json.loads(proc.stdout)
    assert report["Correctness"] == "PASS" and proc.returncode == 0
    rows = report["metrics"]
    layout_rows = [r for r in rows if r["surface"] in ("get_dispatch_layout", "fused_layout")]
    assert len(layout_rows) == 14              # the reference's 7 benchmark cases on both surfaces
    assert {r["surface"] for r in rows} == {"get_dispatch_layout", "fused_layout", "dispatch", "combine",
                                            "host_get_dispatch_layout", "launch_floor"}
    assert all(r["latency_avg"] > 0 for r in rows)
    # every row that moves data carries its minimum HBM traffic, the rate that implies and the fraction
    # of the 8 TB/s peak (how large that fraction is belongs to the benchmark, not to this test)
    for r in rows:
        if r["surface"] == "launch_floor":
            continue
        assert r["throughput_avg"] > 0 and r["hbm_bytes"] > 0 and r["hbm_gbps"] > 0
        assert abs(r["roofline_frac"] - r["hbm_gbps"] / 8000.0) < 1e-4
        assert r["host_pointers"] == (r["surface"] == "host_get_dispatch_layout")
    assert len([r for r in rows if r["surface"] in ("dispatch", "combine") and r["data_size"] == 8192]) == 2
    print(proc.stdout)


def test_selftest_binary_skips_without_a_device():
    """Same protocol as the reference when no device is present: SKIP, exit code 0."""
    import torch
    if torch.cuda.is_available():
        pytest.skip("a device is present")
    if not os.path.exists(BINARY):
        pytest.skip("binary not built")
    proc = subprocess.run([BINARY], capture_output=True, text=True, timeout=60)
    assert proc.returncode == 0 and json.loads(proc.stdout)["Correctness"] == "SKIP"
