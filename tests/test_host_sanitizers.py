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
    objs = [os.path.join(CSRC, n) for n in ("hip_layer.o", "kernels.o", "count_kernels.o")]
    if not all(os.path.exists(o) for o in objs):
        subprocess.check_call(["make", "-s", "-C", CSRC, "hip_layer.o", "kernels.o", "count_kernels.o"])
    return objs


@pytest.mark.parametrize("name,flags,marks", [
    ("address+undefined", ["-fsanitize=address,undefined", "-fno-omit-frame-pointer"],
     ("ERROR: AddressSanitizer", "runtime error:")),
    ("thread", ["-fsanitize=thread"], ("WARNING: ThreadSanitizer",)),
])
def test_planner_under_sanitizer(tmp_path, name, flags, marks):
    exe = str(tmp_path / "planner_stress")
    srcs = [os.path.join(HERE, "planner_stress.cpp")] + [os.path.join(CSRC, n) for n in ("cutt_api.cpp", "plan.cpp", "model.cpp", "layer_math.cpp", "slab.cpp")]
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


FAKE_SRCS = [os.path.join(HERE, n) for n in ("plan_lifetime_stress.cpp", "fake_hip_layer.cpp")] + \
            [os.path.join(CSRC, n) for n in ("cutt_api.cpp", "plan.cpp", "model.cpp", "layer_math.cpp", "slab.cpp")]


def build_on_fake_layer(exe, flags):
    """The plan API (host code only) on top of a stand-in for the runtime half of its C-ABI layer."""
    subprocess.check_call(["g++", "-O1", "-g", "-std=c++17", "-pthread"] + flags +
                          ["-I" + os.path.join(ROOT, "include"), "-I" + CSRC] + FAKE_SRCS + ["-o", exe])


@pytest.mark.parametrize("name,flags,marks", [
    ("address+undefined", ["-fsanitize=address,undefined", "-fno-omit-frame-pointer"],
     ("ERROR: AddressSanitizer", "runtime error:")),
    ("thread", ["-fsanitize=thread"], ("WARNING: ThreadSanitizer",)),
])
def test_destroy_while_another_thread_executes(tmp_path, name, flags, marks):
    # cuttExecute holds the plan while it launches: a concurrent cuttDestroy frees it afterwards
    exe = str(tmp_path / "plan_lifetime_stress")
    build_on_fake_layer(exe, flags)
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=0", CUTT_PLAN_CACHE="0")
    r = subprocess.run([exe, "race", "150"], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, env=env,
                       timeout=600)
    assert r.returncode == 0, r.stdout[-3000:]
    assert "unexpected results 0" in r.stdout, r.stdout[-3000:]
    for mark in marks:
        assert mark not in r.stdout, r.stdout[-3000:]


def test_zeroed_device_properties_do_not_change_the_plan(tmp_path):
    # a runtime that reports 0 for clocks, bus width, CU count or L2 size gets MI355X defaults
    exe = str(tmp_path / "plan_lifetime_stress")
    build_on_fake_layer(exe, [])
    outs = []
    for zero in ("0", "1"):
        env = dict(os.environ, CUTT_FAKE_ZERO_PROPS=zero)
        r = subprocess.run([exe, "plans"], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, env=env,
                           timeout=300)
        assert r.returncode == 0, r.stdout[-3000:]
        outs.append(r.stdout)
    assert outs[0] == outs[1] and outs[0].count("method") == 8


def test_execute_no_alloc_allocates_nothing_and_builds_the_same_tables(tmp_path):
    # on the stand-in layer, which counts allocations and uploads and keeps the tables of the last launch
    exe = str(tmp_path / "plan_lifetime_stress")
    build_on_fake_layer(exe, ["-fsanitize=address,undefined", "-fno-omit-frame-pointer"])
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=0", CUTT_PLAN_CACHE="0")
    r = subprocess.run([exe, "noalloc"], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, env=env, timeout=300)
    assert r.returncode == 0, r.stdout[-3000:]
    assert "noalloc done, failures 0" in r.stdout and r.stdout.count("table entries equal") == 5, r.stdout[-3000:]
    assert "ERROR: AddressSanitizer" not in r.stdout and "runtime error:" not in r.stdout, r.stdout[-3000:]
