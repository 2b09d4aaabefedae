#!/usr/bin/env python3
"""Benchmark of the transpose path on one MI355X.

Default run (the contract line): configuration C2 - fp64, dims (1024, 64, 1024, 3),
permutation (2, 1, 0, 3), ~201 M elements - planned with cuttPlan, executed K
times through cuttExecute.  One "step" is one transpose of the whole tensor;
inputs are resident in HBM before the timed region.  The line also carries the
roofline of the transpose kernel (algorithmic bytes 2*N*sizeof / average launch
duration from HIP events on the plan's stream, against the 8 TB/s HBM peak),
the same-size device-to-device hipMemcpy measured in the same run, and a CPU
baseline (the oracle's multithreaded transpose on the host cores).

  python bench.py [--gpus 1] [--steps K] [--warmup W]
  python bench.py --all        # C1..C4 (+ forced PackedSplit on C4) -> bench_all.json in the --out folder
  python bench.py --sweep N    # first N tensors of the C5 sweep, cuttPlan and cuttPlanMeasure
"""
import argparse
import ctypes
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

import numpy as np

HBM_PEAK_GBS = 8000.0
# HBM bytes per launch of the C2 transpose kernel, from rocprofv3 counters (FETCH_SIZE and WRITE_SIZE
# in runs of their own, each scaled by what the counter reads for the same-size device-to-device
# copy).  A figure belongs to one launched kernel instance: it is reported only when the plan of
# this run has the signature (method, workgroups, tile order, super-tile shape, cache policy, rows
# in groups, digits of the workgroup number in tile order 7) the profile was taken on, together with
# the name of the profile; otherwise null.
C2_ADDRESS_BIT_DIGITS = "m2@1,k2@1,b2@1,b2@2,b2@4,b2@8,b2@32,b2@16,k2@2,m2@8,k2@8,b3@64,m2@4,k2@4,m2@2"
C2_TRAFFIC_PROFILES = {
    ("Tiled", 49152, 7, 1, 1, 3, 0, C2_ADDRESS_BIT_DIGITS): (3221375181, "profiles/tiledKernel_u64_C2_address_bit_order.txt"),
    ("Tiled", 49152, 5, 2, 8, 3, 0, ""): (3221443482, "profiles/tiledKernel_u64_C2_hbm_traffic_pmc.txt"),
    ("Tiled", 49152, 6, 2, 2, 3, 0, ""): (3221508198, "profiles/tiledKernel_u64_C2_order6_measured_plan.txt"),
}


def plan_signature(info):
    return (info.method_name, int(info.numBlocks), int(info.tiledOrder), int(info.superM), int(info.superK),
            int(info.cachePolicy), int(info.tiledGrouped), info.tileDigits.decode())


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def effective_gbs(cfg_bytes, ms):
    return 2.0 * cfg_bytes / (ms * 1e-3) / 1e9


class Runner:
    def __init__(self):
        import torch
        import cutt_amd
        if not torch.cuda.is_available():
            raise SystemExit("bench.py needs a GPU (torch.cuda.is_available() is False)")
        self.torch = torch
        self.cutt = cutt_amd
        self.lib = cutt_amd.lib()  # raises if libcutt.so has not been built
        self.lib.cuttHipMemcpyDtoDAsync.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p]
        self.lib.cuttHipMemcpyDtoDAsync.restype = ctypes.c_int
        torch.cuda.set_device(0)
        self.stream = torch.cuda.current_stream().cuda_stream

    def device_input(self, data):
        t = self.torch.from_numpy(data.view(np.int32 if data.itemsize == 4 else np.int64)).cuda()
        return t

    def time_calls(self, fn, reps, out=None):
        """Per-call milliseconds from HIP events on the current stream; the output buffer is
        overwritten before each call as the reference's benchmark does
        (reference src/cutt_bench.cpp:818-827)."""
        torch = self.torch
        times = []
        for _ in range(reps):
            if out is not None:
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

    def memcpy_ms(self, d_in, d_out, reps=8):
        nbytes = d_in.numel() * d_in.element_size()

        def fn():
            rc = self.lib.cuttHipMemcpyDtoDAsync(d_out.data_ptr(), d_in.data_ptr(), nbytes, self.stream)
            assert rc == 0
        return self.time_calls(fn, reps, out=d_out)

    def plan(self, cfg, how, d_in=None, d_out=None):
        c = self.cutt
        dim, perm, es = list(cfg["dim"]), list(cfg["perm"]), cfg["es"]
        t0 = time.perf_counter()
        if how == "measure":
            rc, h = c.cuttPlanMeasure(len(dim), dim, perm, es, self.stream, d_in.data_ptr(), d_out.data_ptr())
        else:
            rc, h = c.cuttPlan(len(dim), dim, perm, es, self.stream)
        ms = (time.perf_counter() - t0) * 1e3
        if rc != c.CUTT_SUCCESS:
            raise RuntimeError("planning failed with code %d for %s" % (rc, cfg))
        return h, ms

    def run_config(self, cfg, how="plan", reps=6, check=True, data=None, expect=None, force=0):
        """Plan, time and verify one configuration; returns a result dict."""
        import oracle
        c = self.cutt
        dim, perm, es = list(cfg["dim"]), list(cfg["perm"]), cfg["es"]
        vol = int(np.prod(dim, dtype=np.int64))
        nbytes = vol * es
        if data is None:
            import baseline_configs as bc
            data = bc.make_input(cfg)
        d_in = self.device_input(data)
        d_out = self.torch.empty_like(d_in)
        c.set_method_override(force)
        try:
            h, plan_ms = self.plan(cfg, how, d_in, d_out)
        finally:
            c.set_method_override(0)
        info = c.get_plan_info(h)
        times = self.time_calls(lambda: c.cuttExecute(h, d_in.data_ptr(), d_out.data_ptr()), reps, out=d_out)
        ok = None
        if check:
            got = d_out.cpu().numpy().view(data.dtype)
            if expect is None:
                expect = oracle.transpose_mt(dim, perm, data, min(16, os.cpu_count() or 1))
            ok = bool(np.array_equal(got, expect))
        c.cuttDestroy(h)
        cp = self.memcpy_ms(d_in, d_out)
        best, med = min(times), float(np.median(times))
        res = dict(name=cfg["name"], dim=dim, perm=perm, elem_bytes=es, elements=vol, planner=how,
                   method=info.method_name, numSplit=info.numSplit, blocks=info.numBlocks,
                   threads=info.numThreads, lds_bytes=info.ldsBytes, candidates=info.numCandidates,
                   plan_ms=round(plan_ms, 3), ms_min=round(best, 4), ms_median=round(med, 4),
                   gbs_best=round(effective_gbs(nbytes, best), 1), gbs_median=round(effective_gbs(nbytes, med), 1),
                   memcpy_gbs=round(effective_gbs(nbytes, min(cp)), 1),
                   pct_of_memcpy=round(100.0 * min(cp) / best, 1), predicted_us=round(info.usPredicted, 1),
                   bit_exact=ok)
        del d_in, d_out
        return res


def cpu_baseline(cfg, data, budget_s=20.0):
    """The oracle's multithreaded transpose on the host cores (reported baseline, kind 'port')."""
    import oracle
    dim, perm, es = list(cfg["dim"]), list(cfg["perm"]), cfg["es"]
    nbytes = data.size * es
    host_cores = os.cpu_count() or 1
    cores = min(16, host_cores)
    out = np.empty_like(data)
    best = None
    t_start = time.perf_counter()
    reps = 0
    while reps < 5 and (time.perf_counter() - t_start) < budget_s:
        t0 = time.perf_counter()
        oracle.transpose_mt(dim, perm, data, cores, out=out)
        dt = time.perf_counter() - t0
        best = dt if best is None else min(best, dt)
        reps += 1
    return dict(value=round(2.0 * nbytes / best / 1e9, 2), unit="GB/s", cores=cores, host_cores=host_cores, kind="port",
                sample="%d full passes of the same workload (%s, %d elements), best pass" % (reps, cfg["name"], data.size),
                note="the reference has no CPU transpose; this is the oracle's multithreaded C port")


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--all", action="store_true", help="run C1..C4 with both planners")
    ap.add_argument("--sweep", type=int, default=0, help="run the first N tensors of the C5 sweep")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline")
    ap.add_argument("--out", default=os.path.join(ROOT, "bench_out"), help="folder for the --all / --sweep result files")
    args = ap.parse_args()
    if args.gpus != 1:
        raise SystemExit("bench.py measures one GPU: a transpose plan is bound to a single device and this "
                         "build has no multi-GPU path (--gpus %d refused)" % args.gpus)

    import baseline_configs as bc
    r = Runner()
    torch, c = r.torch, r.cutt

    if args.all or args.sweep:
        os.makedirs(args.out, exist_ok=True)
        results = []
        if args.all:
            for cfg in bc.FIXED:
                data = bc.make_input(cfg)
                import oracle
                expect = oracle.transpose_mt(list(cfg["dim"]), list(cfg["perm"]), data, min(16, os.cpu_count() or 1))
                for how in ("plan", "measure"):
                    res = r.run_config(cfg, how, data=data, expect=expect)
                    log(json.dumps(res))
                    results.append(res)
                if cfg["name"] == "C4":
                    for how in ("plan", "measure"):
                        res = r.run_config(cfg, how, data=data, expect=expect, force=c.METHOD_PACKEDSPLIT)
                        res["forced"] = "PackedSplit"
                        log(json.dumps(res))
                        results.append(res)
            with open(os.path.join(args.out, "bench_all.json"), "w") as f:
                json.dump(results, f, indent=1)
        if args.sweep:
            import sweep_runner
            sres = [sweep_runner.run_tensor(cfg, reps=4, log=log) for cfg in bc.sweep()[: args.sweep]]
            log(sweep_runner.table(sres))
            with open(os.path.join(args.out, "bench_sweep.json"), "w") as f:
                json.dump(sres, f, indent=1)
        return

    # ---- the contract line: C2 through cuttPlan + cuttExecute ----
    cfg = bc.C2
    dim, perm, es = list(cfg["dim"]), list(cfg["perm"]), cfg["es"]
    data = bc.make_input(cfg)
    nbytes = data.size * es
    d_in = r.device_input(data)
    d_out = torch.full_like(d_in, -1)
    h, plan_ms = r.plan(cfg, "plan")
    info = c.get_plan_info(h)
    log("plan: %s blocks=%d threads=%d lds=%d candidates=%d plan_ms=%.2f" %
        (info.method_name, info.numBlocks, info.numThreads, info.ldsBytes, info.numCandidates, plan_ms))

    def step():
        rc = c.cuttExecute(h, d_in.data_ptr(), d_out.data_ptr())
        if rc != c.CUTT_SUCCESS:
            raise RuntimeError("cuttExecute failed: %d" % rc)

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    # timed region: exactly K steps launched back to back, bracketed by two HIP events on the
    # plan's stream: the kernel's average launch duration is their distance / K (an event between
    # every two launches would add about 10 us of barrier to every step)
    ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    ev0.record()
    for _ in range(args.steps):
        step()
    ev1.record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    ms_per_step = wall * 1e3 / args.steps
    avg_kernel_ms = ev0.elapsed_time(ev1) / args.steps

    # parity of the timed output against the oracle
    import oracle
    expect = oracle.transpose_mt(dim, perm, data, min(16, os.cpu_count() or 1))
    bit_exact = bool(np.array_equal(d_out.cpu().numpy().view(data.dtype), expect))
    if not bit_exact:
        raise SystemExit("bench output differs from the CPU oracle")

    # the same workload through the measuring planner (reported beside the contract value)
    hm, plan_ms_m = r.plan(cfg, "measure", d_in, d_out)
    info_m = c.get_plan_info(hm)
    ms_m = r.time_calls(lambda: c.cuttExecute(hm, d_in.data_ptr(), d_out.data_ptr()), 8, out=d_out)
    c.cuttDestroy(hm)

    # the same-size device-to-device copy, timed both ways: like the timed region above (K calls back
    # to back, wall clock) and with the reference's per-call protocol (output fill, synchronise,
    # event-timed call; best of 8)
    def copy_step():
        assert r.lib.cuttHipMemcpyDtoDAsync(d_out.data_ptr(), d_in.data_ptr(), nbytes, r.stream) == 0
    for _ in range(args.warmup):
        copy_step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        copy_step()
    torch.cuda.synchronize()
    copy_wall = time.perf_counter() - t0
    memcpy_gbs_loop = 2.0 * nbytes / (copy_wall / args.steps) / 1e9
    cp = r.memcpy_ms(d_in, d_out)
    memcpy_gbs = effective_gbs(nbytes, min(cp))
    # ... and the library's own copy kernel on the same bytes (the Trivial method: the identity permutation
    # of the buffer seen as two ranks), which is what a kernel that streams perfectly reaches on this
    # device - a higher and more honest ceiling than the runtime's copy
    rc, hk = c.cuttPlan(2, [dim[0], data.size // dim[0]], [0, 1], es, r.stream)
    if rc != c.CUTT_SUCCESS or c.get_plan_info(hk).method_name != "Trivial":
        raise SystemExit("no Trivial plan for the copy-kernel ceiling")

    def kernel_copy_step():
        assert c.cuttExecute(hk, d_in.data_ptr(), d_out.data_ptr()) == c.CUTT_SUCCESS
    for _ in range(args.warmup):
        kernel_copy_step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        kernel_copy_step()
    torch.cuda.synchronize()
    copy_kernel_gbs_loop = 2.0 * nbytes / ((time.perf_counter() - t0) / args.steps) / 1e9
    ck = r.time_calls(kernel_copy_step, 8, out=d_out)
    c.cuttDestroy(hk)
    exec_ms = r.time_calls(step, 8, out=d_out)   # the transpose with the per-call protocol
    c.cuttDestroy(h)
    value = 2.0 * nbytes / (wall / args.steps) / 1e9
    achieved = 2.0 * nbytes / (avg_kernel_ms * 1e-3) / 1e9
    traffic, traffic_source = C2_TRAFFIC_PROFILES.get(plan_signature(info), (None, None))
    line = {
        "metric": "effective transpose bandwidth GB/s (2×bytes/time) and % of D2D memcpy, 1 GPU",
        "value": round(value, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "u64", "data": "synthetic",
        "config": {"workload": "C2: fp64 dims (1024,64,1024,3) perm (2,1,0,3), 201326592 elements, value = linear index",
                   "planner": "cuttPlan", "method": info.method_name, "blocks": info.numBlocks,
                   "threads": info.numThreads, "tile_order": info.tiledOrder, "super_tile": [info.superM, info.superK],
                   "tile_digits": info.tileDigits.decode(),
                   "cache_policy": info.cachePolicy, "plan_ms": round(plan_ms, 2)},
        "pct_of_d2d_memcpy": round(100.0 * value / memcpy_gbs_loop, 1),
        "d2d_memcpy_GBs": round(memcpy_gbs_loop, 1),
        "pct_of_copy_kernel": round(100.0 * value / copy_kernel_gbs_loop, 1),
        "copy_kernel_GBs": round(copy_kernel_gbs_loop, 1),
        "per_call_protocol": {"transpose_GBs_best": round(effective_gbs(nbytes, min(exec_ms)), 1),
                              "d2d_memcpy_GBs_best": round(memcpy_gbs, 1),
                              "pct_of_d2d_memcpy": round(100.0 * min(cp) / min(exec_ms), 1),
                              "copy_kernel_GBs_best": round(effective_gbs(nbytes, min(ck)), 1),
                              "pct_of_copy_kernel": round(100.0 * min(ck) / min(exec_ms), 1),
                              "what": "output fill + synchronise + one event-timed call, best of 8 (reference src/cutt_bench.cpp:818-827)"},
        "bit_exact_vs_cpu_oracle": bit_exact,
        "cuttPlanMeasure": {"GBs_best": round(effective_gbs(nbytes, min(ms_m)), 1), "method": info_m.method_name,
                            "tile_order": info_m.tiledOrder, "super_tile": [info_m.superM, info_m.superK],
                            "cache_policy": info_m.cachePolicy, "grouped": info_m.tiledGrouped,
                            "plan_ms": round(plan_ms_m, 1)},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4),
                     "traffic": traffic, "traffic_source": traffic_source,
                     "kernel_ms_avg": round(avg_kernel_ms, 4), "algorithmic_bytes": 2 * nbytes},
    }
    if not args.no_cpu:
        line["cpu_baseline"] = cpu_baseline(cfg, data)
    print(json.dumps(line), flush=True)


if __name__ == "__main__":
    main()
