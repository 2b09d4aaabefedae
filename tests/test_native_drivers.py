"""The native drivers (cutt_test, cutt_bench) built beside the library.

On a machine without a GPU only their command lines are exercised (usage
paths return before any HIP call); on the GPU a shortened cutt_test and one
cutt_bench tensor run for real.
"""
import os
import subprocess

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
BIN = os.path.join(HERE, "..", "cutt_amd", "bin")


def run(name, *args, timeout=300):
    exe = os.path.join(BIN, name)
    if not os.path.exists(exe):
        pytest.fail("%s is not built; run __graft_entry__.build()" % exe)
    return subprocess.run([exe, *args], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=timeout)


def test_usage_without_gpu():
    r = run("cutt_bench")
    assert r.returncode == 1 and "-bench benchID" in r.stdout and "-measure" in r.stdout
    r = run("cutt_bench", "-elemsize", "3", "-bench", "6")
    assert r.returncode == 1
    r = run("cutt_bench", "-dim", "4", "5", "-permutation", "1")
    assert r.returncode == 1
    r = run("cutt_test", "-nonsense")
    assert r.returncode == 1 and "-device gpuid" in r.stdout


@pytest.mark.gpu
def test_cutt_test_short_run():
    # all eight groups; groups 2 and 8 with fewer random tensors per rank than the full run's 100 and 20
    r = run("cutt_test", "-samples", "5", "-seed", "3", timeout=600)
    assert r.returncode == 0, r.stdout[-2000:]
    assert "test OK" in r.stdout
    for k in range(1, 9):
        assert "test %d passed" % k in r.stdout


@pytest.mark.gpu
def test_cutt_test_with_measuring_planner():
    r = run("cutt_test", "-tests", "3,4,6,8", "-samples", "10", "-measure", timeout=600)
    assert r.returncode == 0, r.stdout[-2000:]
    assert "test OK" in r.stdout


@pytest.mark.gpu
def test_cutt_bench_single_tensor_and_memcpy():
    r = run("cutt_bench", "-dim", "1024", "64", "1024", "3", "-permutation", "2", "1", "0", "3", "-plantimer")
    assert r.returncode == 0, r.stdout[-2000:]
    assert "bench OK" in r.stdout and "method Tiled" in r.stdout and "plan took" in r.stdout
    r = run("cutt_bench", "-memcpy", "50000000", "-elemsize", "4")
    assert r.returncode == 0 and "bench OK" in r.stdout and "hipMemcpyDtoD average" in r.stdout


@pytest.mark.gpu
def test_cutt_bench_ttc_suite():
    r = run("cutt_bench", "-bench", "6", "-nomemcpy", timeout=600)
    assert r.returncode == 0, r.stdout[-2000:]
    assert "bench OK" in r.stdout
    assert r.stdout.count("number of elements") == 57


def _suite_summary(out):
    """(tensors, min % of memcpy) from the driver's closing line."""
    import re
    m = re.search(r"percent of same-size hipMemcpy .*: tensors (\d+) min ([0-9.]+) median ([0-9.]+)", out)
    assert m, out[-2000:]
    return int(m.group(1)), float(m.group(2)), float(m.group(3))


@pytest.mark.gpu
@pytest.mark.parametrize("planner", ["heuristic", "measure"])
def test_cutt_bench_random_suites_short(planner):
    # the reference's random-tensor suites with two tensors per rank (or per shape) instead of 50 / 500:
    # bench 3 (ranks 2-8 and 15, reference src/cutt_bench.cpp:414-431), bench 5 with extent ratio 10
    # (ranks 2-7, :455-546) and bench 7 (ranks 8 and 12 with four large extents, :688-728); every
    # tensor is checked on the device, and the 8-byte suites must stay above 70 % of the same-size copy
    extra = ["-measure"] if planner == "measure" else []
    for bench, tensors in (("3", 16), ("510", 12), ("7", 6)):
        r = run("cutt_bench", "-bench", bench, "-samples", "2", "-seed", "11", "-plantimer", *extra, timeout=600)
        assert r.returncode == 0, r.stdout[-2000:]
        assert "bench OK" in r.stdout and "plan took" in r.stdout
        n, worst, median = _suite_summary(r.stdout)
        print("bench %s %s: %d tensors, %% of memcpy min %.1f median %.1f" % (bench, planner, n, worst, median), flush=True)
        assert n >= tensors - 2   # bench 7 skips a shuffle that happens to be the identity
        assert worst >= 70.0, r.stdout[-3000:]


@pytest.mark.gpu
def test_rank_31_the_highest_rank_that_exists():
    # 31 extents of 2 = 2^31 four-byte elements (8.6 GB per buffer), random permutation; checked on
    # the device by closed form.  A rank-32 tensor would have 2^32 elements, beyond the API's limit.
    import os
    import numpy as np
    exe = os.path.join(BIN, "cutt_bench")
    perm = [str(int(p)) for p in np.random.default_rng(5).permutation(31)]
    for extra in ([], ["-measure"]):
        r = subprocess.run([exe, "-elemsize", "4", "-bufelems", "2147483648", "-dim"] + ["2"] * 31 + ["-permutation"] + perm +
                           ["-nomemcpy"] + extra, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=600)
        assert r.returncode == 0, r.stdout[-2000:]
        assert "bench OK" in r.stdout


@pytest.mark.gpu
def test_more_than_2_to_the_32_elements():
    # 65552 x 65536 four-byte elements (4.3e9, 17 GB per buffer) transposed: cut into four pieces, one launch
    # each, checked on the device by closed form (the checker's value pattern repeats every 2^32 elements;
    # tests/test_gpu_large.py checks the same tensor with a pattern that does not)
    import os
    exe = os.path.join(BIN, "cutt_bench")
    r = subprocess.run([exe, "-elemsize", "4", "-bufelems", "4296015872", "-dim", "65552", "65536", "-permutation", "1", "0",
                        "-nomemcpy"], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=600)
    assert r.returncode == 0, r.stdout[-2000:]
    assert "bench OK" in r.stdout and "pieces 4 shapes 1" in r.stdout


@pytest.mark.gpu
def test_tensor_above_4GB_uses_wide_offsets():
    # 671 088 640 doubles = 5.4 GB per buffer: byte offsets no longer fit 32 bits
    import os
    env = dict(os.environ, CUTT_FORCE_METHOD="packedsplit")
    exe = os.path.join(BIN, "cutt_bench")
    r = subprocess.run([exe, "-bufelems", "671088640", "-dim", "1024", "640", "1024", "-permutation", "2", "1", "0",
                        "-nomemcpy"], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=600, env=env)
    assert r.returncode == 0, r.stdout[-2000:]
    assert "bench OK" in r.stdout and "method PackedSplit" in r.stdout
    r = subprocess.run([exe, "-bufelems", "671088640", "-dim", "1024", "640", "1024", "-permutation", "2", "1", "0",
                        "-nomemcpy", "-measure"], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=600)
    assert r.returncode == 0, r.stdout[-2000:]
    assert "bench OK" in r.stdout


@pytest.mark.gpu
def test_tensor_of_2_to_31_elements_and_more():
    # 2 148 353 100 four-byte elements (8.6 GB per buffer) and 2 147 581 963 eight-byte ones
    # (17.2 GB per buffer): more than the reference's int volumes hold; checked on the device by
    # closed form like every other tensor of the driver.
    import os
    exe = os.path.join(BIN, "cutt_bench")
    big4 = ["-elemsize", "4", "-bufelems", "2148353100", "-dim", "1291", "1290", "1290", "-permutation", "2", "0", "1",
            "-nomemcpy"]
    for force, extra, want in ((None, [], "method "), ("tiled", [], "method Tiled"),
                               ("packedsplit", [], "method PackedSplit"), (None, ["-measure"], "method ")):
        env = dict(os.environ)
        if force:
            env["CUTT_FORCE_METHOD"] = force
        r = subprocess.run([exe] + big4 + extra, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True,
                           timeout=600, env=env)
        assert r.returncode == 0, r.stdout[-2000:]
        assert "bench OK" in r.stdout and want in r.stdout
    r = subprocess.run([exe, "-bufelems", "2147581963", "-dim", "46341", "46343", "-permutation", "1", "0", "-nomemcpy"],
                       stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=600)
    assert r.returncode == 0, r.stdout[-2000:]
    assert "bench OK" in r.stdout
