"""Runs the host-only C++ checks: the planner / source generator (tests/cpp/test_planner.cpp; generated kernels are only
compiled, hipRTC cross-compiles for gfx950) and DeviceHIP's memory bookkeeping on a stub of the kernel layer
(tests/cpp/test_allocator.cpp).  No GPU needed.  With AIX_SANITIZERS=1 the same programs are also built and run under
AddressSanitizer + UndefinedBehaviorSanitizer and ThreadSanitizer (`make -C tests/cpp asan tsan`, about three minutes)."""
import os
import subprocess

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)


def test_planner_and_generator():
    subprocess.check_call(["make", "-s", "-C", os.path.join(HERE, "cpp"), os.path.join(HERE, "cpp", "build", "test_planner")])
    res = subprocess.run([os.path.join(HERE, "cpp", "build", "test_planner"),
                          os.path.join(ROOT, "aix_amd", "csrc", "hip", "aix_device.h")],
                         stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=600)
    print(res.stdout[-4000:])
    assert res.returncode == 0, res.stdout[-4000:]
    assert "all planner checks passed" in res.stdout


def test_allocator_on_the_stub_kernel_layer():
    subprocess.check_call(["make", "-s", "-C", os.path.join(HERE, "cpp"), os.path.join(HERE, "cpp", "build", "test_allocator")])
    res = subprocess.run([os.path.join(HERE, "cpp", "build", "test_allocator"), "threads"],
                         stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=600)
    assert res.returncode == 0 and "all allocator checks passed" in res.stdout, res.stdout[-4000:]


@pytest.mark.skipif(os.environ.get("AIX_SANITIZERS") != "1", reason="set AIX_SANITIZERS=1 to build and run the ASan/UBSan and TSan configurations")
def test_host_code_under_sanitizers():
    for target in ("asan", "tsan"):
        res = subprocess.run(["make", "-s", "-C", os.path.join(HERE, "cpp"), target], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=1800)
        assert res.returncode == 0 and "all allocator checks passed" in res.stdout, res.stdout[-4000:]
