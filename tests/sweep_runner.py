"""Runs a list of transpose problems through both planners on the GPU, the way the reference's
benchmark times a tensor (reference src/cutt_bench.cpp:801-830: plan timed on the host clock; per
repetition output fill, device synchronise, event-timed cuttExecute), with a same-size
device-to-device hipMemcpy timed the same way in the same process.

Every output is checked on the device: the input holds each element's linear index, and the
expectation is torch's own permute + contiguous of that index tensor (an independent routine).
Shared by tests/test_gpu_c5_sweep.py and bench.py --sweep."""
import ctypes
import os
import time

import numpy as np
import torch

import cutt_amd as cutt


def _lib():
    lib = cutt.lib()
    lib.cuttHipMemcpyDtoDAsync.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p]
    lib.cuttHipMemcpyDtoDAsync.restype = ctypes.c_int
    return lib


def index_pattern(vol, es):
    """Device tensor whose element k holds k (as a 4- or 8-byte integer)."""
    return torch.arange(vol, dtype=torch.int32 if es == 4 else torch.int64, device="cuda")


def expected_on_device(d_in, dim, perm):
    """The transposed tensor by torch: dim[0] is fastest, so the C-ordered view has the dims reversed."""
    n = len(dim)
    view = d_in.view(*[int(d) for d in reversed(dim)])
    axes = [n - 1 - perm[n - 1 - b] for b in range(n)]
    return view.permute(*axes).contiguous().view(-1)


def timed_ms(fn, out, reps):
    times = []
    for _ in range(reps):
        out.fill_(-1)
        torch.cuda.synchronize()
        e0 = torch.cuda.Event(enable_timing=True)
        e1 = torch.cuda.Event(enable_timing=True)
        e0.record()
        fn()
        e1.record()
        e1.synchronize()
        times.append(e0.elapsed_time(e1))
    return times


def copy_kernel_plan(dim, es, st):
    """A plan of the library's own copy kernel for a tensor of this size (the identity permutation of the
    tensor seen as two ranks is a Trivial plan), the ceiling of what a streaming kernel reaches."""
    vol = int(np.prod(dim, dtype=np.int64))
    rc, h = cutt.cuttPlan(2, [int(dim[0]), vol // int(dim[0])], [0, 1], es, st)
    assert rc == cutt.CUTT_SUCCESS and cutt.get_plan_info(h).method_name == "Trivial"
    return h


def run_tensor(cfg, reps=4, planners=("plan", "measure"), log=None):
    """Returns a dict with one entry per planner: method, plan ms, best ms, GB/s, % of memcpy, % of the
    library's copy kernel, bit-exact.  The plans are created first and then timed in turn (plan, measure,
    plan, measure ...; the best run of each counts), so that a drift of the device's state between two
    blocks of repetitions cannot favour one of them."""
    lib = _lib()
    dim, perm, es = [int(d) for d in cfg["dim"]], [int(p) for p in cfg["perm"]], int(cfg["es"])
    vol = int(np.prod(dim, dtype=np.int64))
    nbytes = vol * es
    st = torch.cuda.current_stream().cuda_stream
    d_in = index_pattern(vol, es)
    d_out = torch.empty_like(d_in)
    want = expected_on_device(d_in, dim, perm)

    def copy():
        assert lib.cuttHipMemcpyDtoDAsync(d_out.data_ptr(), d_in.data_ptr(), nbytes, st) == 0
    copy_ms = min(timed_ms(copy, d_out, reps))
    hc = copy_kernel_plan(dim, es, st)

    def copy_kernel():
        assert cutt.cuttExecute(hc, d_in.data_ptr(), d_out.data_ptr()) == cutt.CUTT_SUCCESS
    kernel_ms = min(timed_ms(copy_kernel, d_out, reps))
    assert cutt.cuttDestroy(hc) == cutt.CUTT_SUCCESS
    res = dict(name=cfg.get("name", ""), dim=dim, perm=perm, es=es, elements=vol,
               memcpy_gbs=2.0 * nbytes / (copy_ms * 1e-3) / 1e9, copy_kernel_gbs=2.0 * nbytes / (kernel_ms * 1e-3) / 1e9)
    handles = {}
    for how in planners:
        if log:
            log("%s %s dim=%s perm=%s es=%d" % (res["name"], how, dim, perm, es))
        # plan-creation time is that of a first call: the library's cache of decisions is switched
        # off for the call (an earlier test of the same process may have planned this tensor)
        saved = os.environ.get("CUTT_PLAN_CACHE")
        os.environ["CUTT_PLAN_CACHE"] = "0"
        try:
            t0 = time.perf_counter()
            if how == "measure":
                rc, h = cutt.cuttPlanMeasure(len(dim), dim, perm, es, st, d_in.data_ptr(), d_out.data_ptr())
            else:
                rc, h = cutt.cuttPlan(len(dim), dim, perm, es, st)
            plan_ms = (time.perf_counter() - t0) * 1e3
        finally:
            if saved is None:
                del os.environ["CUTT_PLAN_CACHE"]
            else:
                os.environ["CUTT_PLAN_CACHE"] = saved
        assert rc == cutt.CUTT_SUCCESS, (rc, cfg, how)
        handles[how] = (h, plan_ms, cutt.get_plan_info(h))
    best = {how: float("inf") for how in planners}
    exact = {how: True for how in planners}
    for _ in range(reps):
        for how in planners:
            h = handles[how][0]

            def execute():
                assert cutt.cuttExecute(h, d_in.data_ptr(), d_out.data_ptr()) == cutt.CUTT_SUCCESS
            best[how] = min(best[how], timed_ms(execute, d_out, 1)[0])
            exact[how] = exact[how] and bool(torch.equal(d_out, want))
    for how in planners:
        h, plan_ms, info = handles[how]
        assert cutt.cuttDestroy(h) == cutt.CUTT_SUCCESS
        res[how] = dict(method=info.method_name, plan_ms=plan_ms, ms=best[how], gbs=2.0 * nbytes / (best[how] * 1e-3) / 1e9,
                        pct=100.0 * copy_ms / best[how], pct_kernel=100.0 * kernel_ms / best[how], exact=exact[how],
                        candidates=info.numCandidates, predicted_us=info.usPredicted)
    return res


def table(results, planners=("plan", "measure")):
    """Per-tensor text table and per-width summary lines."""
    lines = ["%-6s %-2s %-34s %-22s %7s %7s | %s" % ("name", "B", "dims", "permutation", "memcpy", "copyk",
                                                    " | ".join("%-11s %7s %6s %6s %8s" % (p, "GB/s", "%cpy", "%cpk", "plan ms") for p in planners))]
    for r in results:
        cols = []
        for p in planners:
            x = r[p]
            cols.append("%-11s %7.0f %6.1f %6.1f %8.2f" % (x["method"], x["gbs"], x["pct"], x["pct_kernel"], x["plan_ms"]))
        lines.append("%-6s %-2d %-34s %-22s %7.0f %7.0f | %s" % (r["name"], r["es"], " ".join(map(str, r["dim"])),
                                                               " ".join(map(str, r["perm"])), r["memcpy_gbs"], r["copy_kernel_gbs"],
                                                               " | ".join(cols)))
    for es in (8, 4):
        sel = [r for r in results if r["es"] == es]
        if not sel:
            continue
        for p in planners:
            pct = np.array([r[p]["pct"] for r in sel])
            pck = np.array([r[p]["pct_kernel"] for r in sel])
            pms = np.array([r[p]["plan_ms"] for r in sel])
            lines.append("%d-byte elements, %-7s: tensors %d, %% of memcpy min %.1f median %.1f max %.1f; %% of the copy kernel "
                         "min %.1f median %.1f max %.1f; plan ms median %.2f max %.2f" %
                         (es, p, len(sel), pct.min(), np.median(pct), pct.max(), pck.min(), np.median(pck), pck.max(),
                          np.median(pms), pms.max()))
    return "\n".join(lines)
