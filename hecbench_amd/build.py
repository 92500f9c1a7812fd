"""Builds libhq.so in-tree with hipcc for gfx950 (python -m hecbench_amd.build)."""
import os
import subprocess
import sys

_HERE = os.path.dirname(os.path.abspath(__file__))


def build(clean=False, jobs=8):
    csrc = os.path.join(_HERE, "csrc")
    if clean:
        subprocess.run(["make", "-C", csrc, "clean"], check=True)
    subprocess.run(["make", "-C", csrc, f"-j{jobs}"], check=True)
    return os.path.join(_HERE, "libhq.so")


if __name__ == "__main__":
    print(build(clean="--clean" in sys.argv))
