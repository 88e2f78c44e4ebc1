"""Builds the HIP/C++ libraries in-tree with hipcc / g++ (no cmake, no JIT cache)."""
import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))


def library_path(name):
    return os.path.join(HERE, name)


def build(jobs=8, verbose=False, force=False):
    """Compile every HIP extension for gfx950 and the host library; raises on the first compiler
    error.  force=True recompiles every source even where an up-to-date library is present."""
    cmd = ["make", "-C", os.path.join(HERE, "csrc"), f"-j{jobs}", "all"] + (["-B"] if force else [])
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if verbose or res.returncode != 0:
        print(res.stdout[-8000:])
    if res.returncode != 0:
        raise RuntimeError("building the aix_amd libraries failed")
