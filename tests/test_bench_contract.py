"""The parts of bench.py's contract that need no GPU: more than one GPU is refused with a
message, the workload constants are the ones the metric is quoted on, the profiled-traffic
reader understands the committed counter summary, and the CPU baseline leg runs the oracle."""
import os
import subprocess
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)
import bench  # noqa: E402


def test_more_than_one_gpu_is_refused_with_a_message():
    out = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert out.returncode != 0
    assert "one GPU" in out.stderr


def test_workload_constants():
    assert bench.XS == (32, 56, 56, 64) and bench.WS == (3, 3, 64, 64)
    assert bench.MACS_PER_PASS == 3_699_376_128
    assert bench.METRIC.endswith("MBM_7")


def test_measured_table_comes_from_the_library_generator_and_equals_the_reference_file():
    """bench.py and smoke() build MBM_7 with the library's generator (host code, no GPU needed):
    byte-identical to the reference's file, which stays test data only."""
    from approxtrain_amd import lut_gen
    from tests.util import lut_bytes
    assert np.array_equal(np.asarray(lut_gen.generate_builtin("MBM", 7, 1), np.uint8), lut_bytes("MBM", 7))
    src = open(os.path.join(ROOT, "bench.py")).read() + open(os.path.join(ROOT, "__graft_entry__.py")).read()
    assert "golden" not in src


def test_profiled_traffic_reads_the_committed_summary():
    t = bench.profiled_traffic()
    assert t is not None and t["bytes"] == t["read_bytes"] + t["written_bytes"]
    assert t["measured_in_run"] is False
    # at least the un-lowered input + output, far below an im2col-materialising lowering (231 MB more)
    assert 45e6 < t["bytes"] < 120e6


def test_cpu_baseline_leg_runs_the_oracle_on_a_sample():
    from oracle import cpu
    rng = np.random.default_rng(0)
    x = np.maximum(rng.standard_normal((1, 8, 8, 64)), 0).astype(np.float32)
    w = (rng.standard_normal(bench.WS) * 0.06).astype(np.float32)
    lut32 = cpu.expand_u8(cpu.lutgen("MBM", 7), 7)
    y = cpu.conv2d_fwd(lut32, 7, x, w, (1, 1), "SAME", threads=2)
    assert y.shape == (1, 8, 8, 64) and np.isfinite(y).all()
