"""Compile libcutt.so for gfx950 with the committed Makefile (hipcc + g++)."""
import os
import subprocess

_HERE = os.path.dirname(os.path.abspath(__file__))


def build(clean=True, jobs=8):
    csrc = os.path.join(_HERE, "csrc")
    if clean:
        subprocess.check_call(["make", "-s", "-C", csrc, "clean"])
    subprocess.check_call(["make", "-s", "-C", csrc, "-j%d" % jobs])
    path = os.path.join(_HERE, "libcutt.so")
    if not os.path.exists(path):
        raise RuntimeError("build did not produce %s" % path)
    return path
