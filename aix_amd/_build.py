"""Builds the HIP/C++ libraries in-tree with hipcc / g++ (no cmake, no JIT cache)."""
import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))


def library_path(name):
    return os.path.join(HERE, name)


def build(jobs=8, verbose=False):
    """Compile every HIP extension for gfx950 and the host library.  Always recompiles what is
    out of date; raises on the first compiler error."""
    cmd = ["make", "-C", os.path.join(HERE, "csrc"), f"-j{jobs}", "all"]
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if verbose or res.returncode != 0:
        print(res.stdout[-8000:])
    if res.returncode != 0:
        raise RuntimeError("building the aix_amd libraries failed")
