"""Runs the C++ planner / source-generator checks (tests/cpp/test_planner.cpp).  No GPU needed:
generated kernels are only compiled (hipRTC cross-compiles for gfx950)."""
import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)


def test_planner_and_generator():
    subprocess.check_call(["make", "-s", "-C", os.path.join(HERE, "cpp")])
    res = subprocess.run([os.path.join(HERE, "cpp", "build", "test_planner"),
                          os.path.join(ROOT, "aix_amd", "csrc", "hip", "aix_device.h")],
                         stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=600)
    print(res.stdout[-4000:])
    assert res.returncode == 0, res.stdout[-4000:]
    assert "all planner checks passed" in res.stdout
