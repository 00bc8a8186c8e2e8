"""Builds csrc/libdapple_hip.so with hipcc for gfx950 (cross-compiles without a GPU).

    python -m dapple_amd.build [--clean]
"""
import os
import subprocess
import sys

CSRC = os.path.join(os.path.dirname(os.path.abspath(__file__)), "csrc")


def build(clean=False, jobs=8, force=False):
    """force: recompile every source even where an up-to-date object is there (make -B)."""
    if clean:
        subprocess.check_call(["make", "-C", CSRC, "clean"])
    subprocess.check_call(["make", "-C", CSRC, "-j%d" % jobs] + (["-B"] if force else []))
    return os.path.join(CSRC, "libdapple_hip.so")


if __name__ == "__main__":
    print(build(clean="--clean" in sys.argv))
