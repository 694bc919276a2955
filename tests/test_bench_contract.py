"""Host-side checks of bench.py that need no GPU: the workload table, the FLOP model behind the
reported metric, the roofline traffic figure read from the committed rocprofv3 summaries, and the
refusal of multi-GPU runs."""
import os
import subprocess
import sys

import bench

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_flop_model_of_the_headline_workload():
    """C3: 2*R*D*2H for the gate+up GEMM and 2*R*H*O for the down GEMM, R = T*K routed rows."""
    w = bench.WORKLOADS["c3_bf16"]
    f1, f2 = bench.flops_of(w)
    R = 16384 * 8
    assert f1 == 2.0 * R * 2048 * 2 * 1408 and f2 == 2.0 * R * 1408 * 2048
    assert abs((f1 + f2) / 1e12 - 2.2677) < 1e-3
    # the plain SiLU MLP of C2 has one hidden matrix
    g1, g2 = bench.flops_of(bench.WORKLOADS["c2_bf16"])
    assert g1 == 2.0 * 8192 * 2 * 1024 * 4096 and g2 == g1


def test_roofline_traffic_is_read_from_the_committed_profiles():
    for name in ("c3_bf16", "c4_fp8"):
        path = os.path.join(ROOT, "profiles", bench.PROFILE_OF[name])
        assert os.path.exists(path), path
        traffic = bench.measured_traffic_bytes(name)
        assert isinstance(traffic, int)
        # at least the algorithmic bytes of GEMM1 (tokens + weights + hidden), below 10x that
        w = bench.WORKLOADS[name]
        esize = 1 if w["dtype"] == "fp8" else 2
        algorithmic = (w["T"] * w["D"] + w["E"] * 2 * w["H"] * w["D"]) * esize + w["T"] * w["K"] * w["H"] * 2
        assert algorithmic <= traffic < 10 * algorithmic, (name, traffic, algorithmic)
    assert bench.measured_traffic_bytes("c2_bf16") is None       # no summary committed for it


def test_more_than_one_gpu_is_refused_with_a_message():
    res = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True,
                         text=True, timeout=300)
    assert res.returncode != 0
    assert "--gpus must be 1" in res.stderr and "ONE GPU" in res.stderr
