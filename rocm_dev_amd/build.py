"""Compiles libsgemm.so in-tree with hipcc for gfx950 (cross-compiles without a GPU)."""
import os
import subprocess

CSRC = os.path.join(os.path.dirname(os.path.abspath(__file__)), "csrc")
LIB_PATH = os.path.join(CSRC, "libsgemm.so")


def build(force=False, jobs=8, verbose=False):
    """Run ``make`` in csrc/.  ``force`` rebuilds every object."""
    if force:
        subprocess.run(["make", "-C", CSRC, "clean"], check=True, capture_output=True)
    res = subprocess.run(["make", "-C", CSRC, "-j%d" % jobs], capture_output=True, text=True)
    if verbose or res.returncode != 0:
        print(res.stdout)
        print(res.stderr)
    if res.returncode != 0 or not os.path.exists(LIB_PATH):
        raise RuntimeError("building libsgemm.so failed")
    return LIB_PATH
