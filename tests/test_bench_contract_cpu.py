"""bench.py contract pieces that need no GPU: more than one GPU is refused with a message, and
the algorithmic flop counts are the closed forms the roofline figures are quoted against."""
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_more_than_one_gpu_is_refused():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert r.returncode == 2
    assert "ONE GPU" in r.stderr and r.stdout.strip() == ""


def test_algorithmic_flops_closed_forms():
    sys.path.insert(0, ROOT)
    import bench

    fl = bench.algorithmic_flops(64, 2)
    feat = 1 + 64 + 64 * 64
    assert fl["fwd"] == 4 * feat * 65 == 1081860
    assert fl["bwd"] == 2 * (2 * feat * 65 + 2 * (feat - 1) * 65 + feat * 64) == 2696068
    assert fl["build"] + fl["fwd_apply"] == fl["fwd"]
    fl1 = bench.algorithmic_flops(64, 1)
    assert fl1["fwd"] == 16900 and fl1["bwd"] == 41860
    fl32 = bench.algorithmic_flops(32, 2)
    assert fl32["fwd"] == 139524 and fl32["bwd"] == 346564
