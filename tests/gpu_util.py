"""Helpers for the GPU parity tests: device buffers come from torch, the transpose
goes through the C-ABI of libcutt.so, the expectation from the CPU oracle."""
import numpy as np
import torch

import cutt_amd as cutt
import oracle

DTYPES = {4: (np.uint32, torch.int32), 8: (np.uint64, torch.int64)}


def to_device(a):
    """numpy array of uint32/uint64 -> device tensor holding the same bytes."""
    signed = a.view(np.int32 if a.itemsize == 4 else np.int64)
    return torch.from_numpy(signed).cuda()


def to_host(t, itemsize):
    return t.cpu().numpy().view(np.uint32 if itemsize == 4 else np.uint64)


def stream_handle():
    return torch.cuda.current_stream().cuda_stream


def seeded(vol, es, seed=0):
    rng = np.random.default_rng(seed)
    return rng.integers(0, 2 ** (8 * es) - 1, size=vol, dtype=np.uint64, endpoint=True).astype(DTYPES[es][0])


def run_plan(handle, d_in, d_out):
    rc = cutt.cuttExecute(handle, d_in.data_ptr(), d_out.data_ptr())
    assert rc == cutt.CUTT_SUCCESS, rc
    torch.cuda.synchronize()


def check_case(dim, perm, es, data=None, how="plan", candidate=None, expect=None):
    """Transpose on the GPU and compare bit-exact with the oracle.  Returns the plan info."""
    vol = int(np.prod([int(d) for d in dim], dtype=object))
    if data is None:
        data = seeded(vol, es, seed=vol % 9973)
    d_in = to_device(data)
    d_out = torch.full_like(d_in, -1)
    st = stream_handle()
    if how == "plan":
        rc, h = cutt.cuttPlan(len(dim), dim, perm, es, st)
    elif how == "measure":
        rc, h = cutt.cuttPlanMeasure(len(dim), dim, perm, es, st, d_in.data_ptr(), d_out.data_ptr())
    else:
        rc, h = cutt.cuttPlanFromCandidate(len(dim), dim, perm, es, st, candidate)
    assert rc == cutt.CUTT_SUCCESS, (rc, dim, perm, es, how)
    info = cutt.get_plan_info(h)
    d_out.fill_(-1)
    torch.cuda.synchronize()
    run_plan(h, d_in, d_out)
    assert cutt.cuttDestroy(h) == cutt.CUTT_SUCCESS
    got = to_host(d_out, es)
    if expect is None:
        expect = oracle.transpose_mt(dim, perm, data, 8) if vol > (1 << 22) else oracle.transpose(dim, perm, data)
    if not np.array_equal(got, expect):
        bad = np.nonzero(got != expect)[0]
        raise AssertionError("mismatch dim=%s perm=%s es=%d %s: %d wrong, first at %d" %
                             (dim, perm, es, info.as_dict(), bad.size, bad[0]))
    return info
