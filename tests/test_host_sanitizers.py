"""The planner's host code under the compiler's sanitizers (no GPU needed): plan.cpp, model.cpp and
cutt_api.cpp are compiled with g++ -fsanitize=..., linked with the in-tree HIP objects, and a
stress program (planner_stress.cpp) plans random problems from four caller threads at once while
the planner itself estimates its candidates on helper threads."""
import os
import subprocess

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(ROOT, "cutt_amd", "csrc")
ROCM_LIB = "/opt/rocm/lib"


def hip_objects():
    objs = [os.path.join(CSRC, n) for n in ("hip_layer.o", "kernels.o")]
    if not all(os.path.exists(o) for o in objs):
        subprocess.check_call(["make", "-s", "-C", CSRC, "hip_layer.o", "kernels.o"])
    return objs


@pytest.mark.parametrize("name,flags,marks", [
    ("address+undefined", ["-fsanitize=address,undefined", "-fno-omit-frame-pointer"],
     ("ERROR: AddressSanitizer", "runtime error:")),
    ("thread", ["-fsanitize=thread"], ("WARNING: ThreadSanitizer",)),
])
def test_planner_under_sanitizer(tmp_path, name, flags, marks):
    exe = str(tmp_path / "planner_stress")
    srcs = [os.path.join(HERE, "planner_stress.cpp")] + [os.path.join(CSRC, n) for n in ("cutt_api.cpp", "plan.cpp", "model.cpp")]
    cmd = (["g++", "-O1", "-g", "-std=c++17", "-pthread"] + flags +
           ["-I" + os.path.join(ROOT, "include"), "-I" + CSRC] + srcs + hip_objects() +
           ["-L" + ROCM_LIB, "-lamdhip64", "-Wl,-rpath," + ROCM_LIB, "-o", exe])
    subprocess.check_call(cmd)
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=0:verify_asan_link_order=0")
    r = subprocess.run([exe, "25"], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, env=env, timeout=600)
    assert r.returncode == 0, r.stdout[-3000:]
    assert "done, refused 0" in r.stdout, r.stdout[-3000:]
    for mark in marks:
        assert mark not in r.stdout, r.stdout[-3000:]
