"""Builds libspdnn.so and spdnn_network in-tree with hipcc for gfx950 (see csrc/Makefile)."""
import os
import subprocess

_HERE = os.path.dirname(os.path.abspath(__file__))


def build(clean=False, jobs=8):
    csrc = os.path.join(_HERE, "csrc")
    if clean:
        subprocess.run(["make", "-s", "-C", csrc, "clean"], check=True)
    subprocess.run(["make", "-s", "-C", csrc, "-j%d" % jobs, "all"], check=True)
    return os.path.join(_HERE, "libspdnn.so")
