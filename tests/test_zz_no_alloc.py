"""cuttExecuteNoAlloc - plan and execute without allocating on the device - against the CPU oracle and
against cuttPlan + cuttExecute: same bytes, on calls in a row that reuse the library's static scratch
memory (the second with a smaller tensor and smaller tables), for every method; that the call neither
allocates device memory nor uploads tables (the layer's call counters and the device's free memory do
not move); and its refusals."""
import sys

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def say(msg):
    print(msg, flush=True)
    sys.stdout.flush()


@pytest.fixture(scope="module")
def gpu():
    import torch
    assert torch.cuda.is_available(), "these tests need the MI355X"
    import gpu_util
    import cutt_amd
    cutt_amd.lib()
    cutt_amd.set_method_override(0)
    return gpu_util


def both_ways(gpu, dim, perm, es, seed):
    """Output of cuttPlan + cuttExecute and of cuttExecuteNoAlloc for the same input."""
    import torch
    import cutt_amd as cutt
    vol = int(np.prod(dim, dtype=np.int64))
    data = gpu.seeded(vol, es, seed=seed)
    d_in = gpu.to_device(data)
    st = gpu.stream_handle()
    ref = torch.full_like(d_in, -1)
    rc, h = cutt.cuttPlan(len(dim), dim, perm, es, st)
    assert rc == cutt.CUTT_SUCCESS
    info = cutt.get_plan_info(h)
    gpu.run_plan(h, d_in, ref)
    assert cutt.cuttDestroy(h) == cutt.CUTT_SUCCESS
    out = torch.full_like(d_in, -1)
    say("cuttExecuteNoAlloc dim=%s perm=%s es=%d method %s lds %d" % (dim, perm, es, info.method_name, info.ldsBytes))
    torch.cuda.synchronize()
    calls = cutt.device_call_counts()
    free = torch.cuda.mem_get_info()[0]
    rc = cutt.cuttExecuteNoAlloc(len(dim), dim, perm, es, st, d_in.data_ptr(), out.data_ptr())
    assert rc == cutt.CUTT_SUCCESS, rc
    torch.cuda.synchronize()
    # nothing allocated, nothing uploaded: the library's own counters and the driver's free memory agree
    assert cutt.device_call_counts() == calls, (calls, cutt.device_call_counts())
    assert torch.cuda.mem_get_info()[0] == free
    return data, ref, out, info


def test_two_calls_in_a_row_second_smaller(gpu):
    import torch
    import oracle
    import cutt_amd as cutt
    # a large Packed plan (tables of 6545 elements), then a small one whose tables overwrite the
    # front of the same scratch memory, then the large one again
    cases = [((5, 7, 11, 13, 17, 109), (4, 2, 0, 5, 1, 3), 4), ((6, 5, 9, 31), (2, 0, 3, 1), 4),
             ((5, 7, 11, 13, 17, 109), (4, 2, 0, 5, 1, 3), 4)]
    methods = []
    for i, (dim, perm, es) in enumerate(cases):
        data, ref, out, info = both_ways(gpu, list(dim), list(perm), es, seed=10 + i)
        assert torch.equal(out, ref), (dim, perm, es)
        assert np.array_equal(gpu.to_host(out, es), oracle.transpose_mt(list(dim), list(perm), data, 8))
        methods.append(info.method)
    assert cutt.METHOD_PACKED in methods or cutt.METHOD_PACKEDSPLIT in methods


@pytest.mark.parametrize("method", ["tiled", "tiledcopy", "packed", "packedsplit", "trivial"])
def test_every_method(gpu, method):
    import torch
    import oracle
    import cutt_amd as cutt
    force = {"tiled": cutt.METHOD_TILED, "tiledcopy": cutt.METHOD_TILEDCOPY, "packed": cutt.METHOD_PACKED,
             "packedsplit": cutt.METHOD_PACKEDSPLIT, "trivial": 0}[method]
    shapes = {"tiled": ((300, 7, 290), (2, 1, 0), 8), "tiledcopy": ((130, 59, 88), (0, 2, 1), 4),
              "packed": ((12, 9, 31, 40), (2, 0, 3, 1), 8), "packedsplit": ((20000, 2, 50), (2, 1, 0), 8),
              "trivial": ((20, 30, 40), (0, 1, 2), 4)}
    dim, perm, es = shapes[method]
    cutt.set_method_override(force)
    try:
        data, ref, out, info = both_ways(gpu, list(dim), list(perm), es, seed=3)
    finally:
        cutt.set_method_override(0)
    assert info.method_name.lower() == method
    assert np.array_equal(gpu.to_host(out, es), oracle.transpose_mt(list(dim), list(perm), data, 8))
    assert torch.equal(out, ref)
    # a second, smaller call with the same method
    small = tuple(max(2, d // 2) for d in dim)
    cutt.set_method_override(force)
    try:
        data, ref, out, info = both_ways(gpu, list(small), list(perm), es, seed=4)
    finally:
        cutt.set_method_override(0)
    assert np.array_equal(gpu.to_host(out, es), oracle.transpose_mt(list(small), list(perm), data, 8))
    assert torch.equal(out, ref)


def test_the_counters_do_see_an_allocating_plan(gpu):
    # what the checks above rest on: cuttPlan of a plan with index tables allocates once and uploads once
    import cutt_amd as cutt
    cutt.set_method_override(cutt.METHOD_PACKED)
    try:
        before = cutt.device_call_counts()
        rc, h = cutt.cuttPlan(4, [12, 9, 31, 40], [2, 0, 3, 1], 8, gpu.stream_handle())
        assert rc == cutt.CUTT_SUCCESS
        after = cutt.device_call_counts()
        cutt.cuttDestroy(h)
    finally:
        cutt.set_method_override(0)
    assert after == (before[0] + 1, before[1] + 1)


def test_refusals(gpu, monkeypatch):
    import torch
    import cutt_amd as cutt
    a = torch.zeros(64 * 64, dtype=torch.int64, device="cuda")
    b = torch.zeros_like(a)
    st = gpu.stream_handle()
    assert cutt.cuttExecuteNoAlloc(2, [64, 64], [1, 0], 8, st, a.data_ptr(), a.data_ptr()) == cutt.CUTT_INVALID_PARAMETER
    assert cutt.cuttExecuteNoAlloc(2, [64, 64], [1, 1], 8, st, a.data_ptr(), b.data_ptr()) == cutt.CUTT_INVALID_PARAMETER
    assert cutt.cuttExecuteNoAlloc(2, [64, 64], [1, 0], 3, st, a.data_ptr(), b.data_ptr()) == cutt.CUTT_INVALID_PARAMETER
    assert cutt.cuttExecuteNoAlloc(2, [64, 64], [1, 0], 8, st, 0, b.data_ptr()) == cutt.CUTT_INVALID_PARAMETER
    # tables beyond the scratch memory: refused, nothing is launched
    monkeypatch.setenv("CUTT_NOALLOC_MAX_BYTES", "256")
    cutt.set_method_override(cutt.METHOD_PACKED)
    try:
        b.fill_(-1)
        rc = cutt.cuttExecuteNoAlloc(3, [16, 16, 16], [2, 1, 0], 8, st, a.data_ptr(), b.data_ptr())
    finally:
        cutt.set_method_override(0)
    torch.cuda.synchronize()
    assert rc == cutt.CUTT_INVALID_PARAMETER
    assert bool((b == -1).all())
