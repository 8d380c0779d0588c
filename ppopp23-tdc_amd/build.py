"""Compile libtdc_amd.so for gfx950 with hipcc (in-tree, next to the Python layer)."""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))


def build(jobs=8, clean=False):
    csrc = os.path.join(HERE, "csrc")
    if clean:
        subprocess.check_call(["make", "-C", csrc, "clean"])
    subprocess.check_call(["make", "-C", csrc, f"-j{jobs}", "all"])
    return os.path.join(HERE, "tdc_amd", "libtdc_amd.so")


if __name__ == "__main__":
    print(build(clean="--clean" in sys.argv))
