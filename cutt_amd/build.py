"""Compile libcutt.so and the native drivers for gfx950 with the committed Makefiles (hipcc + g++)."""
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
    # native drivers (cutt_test, cutt_bench) link against the library just built
    drivers = os.path.join(_HERE, "drivers")
    if clean:
        subprocess.check_call(["make", "-s", "-C", drivers, "clean"])
    subprocess.check_call(["make", "-s", "-C", drivers, "-j%d" % jobs])
    for name in ("cutt_test", "cutt_bench"):
        if not os.path.exists(os.path.join(_HERE, "bin", name)):
            raise RuntimeError("build did not produce bin/%s" % name)
    return path
