"""GPU parity tests: every transpose goes through the C-ABI (cuttPlan /
cuttPlanMeasure / cuttExecute / cuttDestroy) and is compared bit-exact with
the CPU oracle.  The shapes follow the reference's own test driver
(reference src/cutt_test.cpp:138-431)."""
import itertools
import sys

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def gpu():
    import torch
    assert torch.cuda.is_available(), "these tests need the MI355X"
    import gpu_util
    import cutt_amd
    cutt_amd.lib()  # fails loudly if libcutt.so is missing
    cutt_amd.set_method_override(0)
    return gpu_util


def say(msg):
    print(msg, flush=True)
    sys.stdout.flush()


@pytest.mark.parametrize("rank", [2, 3, 4, 5])
def test_all_permutations(gpu, rank):
    # reference test1: dims 2 + r*14/rank, every permutation, 8- and 4-byte elements
    dim = [2 + r * 14 // rank for r in range(rank)]
    for perm in itertools.permutations(range(rank)):
        for es in (8, 4):
            gpu.check_case(dim, list(perm), es)


@pytest.mark.parametrize("rank", [6, 7])
def test_sampled_permutations(gpu, rank):
    dim = [2 + r * 14 // rank for r in range(rank)]
    rng = np.random.default_rng(rank)
    perms = [list(p) for p in itertools.islice(itertools.permutations(range(rank)), 0, None, 97 if rank == 7 else 17)]
    perms += [[int(p) for p in rng.permutation(rank)] for _ in range(10)]
    for perm in perms:
        for es in (8, 4):
            gpu.check_case(dim, perm, es)


def test_every_candidate_small(gpu):
    # each candidate of the enumeration is executed, not only the chosen one
    import cutt_amd as cutt
    cases = [((43, 67), (1, 0)), ((40, 3, 50, 7), (2, 1, 0, 3)), ((5, 7, 11, 13, 17), (4, 2, 0, 1, 3)),
             ((31, 549, 2, 3), (3, 0, 2, 1)), ((130, 9, 70), (0, 2, 1)), ((6, 5, 4, 3, 2, 7, 8), (6, 0, 3, 2, 5, 1, 4)),
             ((3000, 2, 50), (2, 1, 0)), ((70000, 3), (1, 0)), ((3, 70000), (1, 0))]
    methods = set()
    for dim, perm in cases:
        for es in (4, 8):
            with cutt.Candidates(dim, perm, es) as c:
                n = len(c)
            for i in range(n):
                say("candidate %d/%d dim=%s perm=%s es=%d" % (i, n, dim, perm, es))
                info = gpu.check_case(dim, list(perm), es, how="candidate", candidate=i)
                methods.add(info.method_name)
    assert {"Tiled", "TiledCopy", "Packed", "PackedSplit"} <= methods


HAND_PICKED = [  # reference test3, full sizes
    ((43, 67), (1, 0)),
    ((65536 * 32, 2), (1, 0)),
    ((1305, 599, 88), (0, 2, 1)),
    ((24, 330, 64, 147), (1, 0, 2, 3)),
    ((2, 5, 9, 12), (0, 1, 2, 3)),
    ((2, 4, 6, 9, 11, 13), (0, 1, 2, 3, 4, 5)),
    ((5, 42, 75, 86, 57), (1, 3, 4, 2, 0)),
    ((5, 3, 2, 9, 14), (0, 1, 3, 2, 4)),
]


@pytest.mark.parametrize("dim,perm", HAND_PICKED)
def test_hand_picked(gpu, dim, perm):
    for es in (8, 4):
        say("hand picked dim=%s perm=%s es=%d" % (dim, perm, es))
        for how in ("plan", "measure"):
            info = gpu.check_case(list(dim), list(perm), es, how=how)
        if list(perm) == sorted(perm):
            assert info.method_name == "Trivial"


def test_forced_methods_large(gpu):
    # every method on a tensor large enough to need many workgroups
    import cutt_amd as cutt
    cases = {
        cutt.METHOD_TILED: ((1000, 30, 777), (2, 1, 0)),
        cutt.METHOD_TILEDCOPY: ((1305, 599, 30), (0, 2, 1)),
        cutt.METHOD_PACKED: ((5, 7, 11, 13, 17, 31), (4, 2, 0, 5, 1, 3)),
        cutt.METHOD_PACKEDSPLIT: ((200000, 2, 50), (2, 1, 0)),
    }
    try:
        for method, (dim, perm) in cases.items():
            cutt.set_method_override(method)
            for es in (8, 4):
                say("forced %s dim=%s es=%d" % (cutt.METHOD_NAMES[method], dim, es))
                info = gpu.check_case(list(dim), list(perm), es)
                assert info.method == method
    finally:
        cutt.set_method_override(0)


def test_wide_offset_kernels_and_sixteen_per_lane(gpu):
    # The packed kernel has a 64-bit-offset variant for tensors of 4 GB and more; CUTT_WIDE_OFFSETS=1
    # runs it on small tensors.  4-byte elements also have a 16-elements-per-lane variant.
    import os
    import cutt_amd as cutt
    cases = [((5, 7, 11, 13, 17, 31), (4, 2, 0, 5, 1, 3)), ((200000, 2, 50), (2, 1, 0)),
             ((33, 5, 42, 15, 23, 10), (4, 5, 0, 2, 1, 3)), ((129, 3, 257, 31), (2, 0, 3, 1))]
    try:
        for env in ({"CUTT_WIDE_OFFSETS": "1"}, {"CUTT_ELEMS_PER_THREAD": "16"},
                    {"CUTT_WIDE_OFFSETS": "1", "CUTT_ELEMS_PER_THREAD": "16"}):
            os.environ.update(env)
            for method in (cutt.METHOD_PACKED, cutt.METHOD_PACKEDSPLIT):
                cutt.set_method_override(method)
                for dim, perm in cases:
                    for es in (4, 8):
                        say("%s forced %s dim=%s es=%d" % (env, cutt.METHOD_NAMES[method], dim, es))
                        st = gpu.stream_handle()
                        rc, h = cutt.cuttPlan(len(dim), list(dim), list(perm), es, st)
                        if rc != cutt.CUTT_SUCCESS:
                            continue  # the forced method has no feasible candidate for this tensor
                        info = cutt.get_plan_info(h)
                        cutt.cuttDestroy(h)
                        if "CUTT_ELEMS_PER_THREAD" in env and es == 4:
                            assert info.elemsPerThread == 16
                        if es == 8:
                            assert info.elemsPerThread <= 8
                        gpu.check_case(list(dim), list(perm), es)
            for k in env:
                del os.environ[k]
    finally:
        cutt.set_method_override(0)
        os.environ.pop("CUTT_WIDE_OFFSETS", None)
        os.environ.pop("CUTT_ELEMS_PER_THREAD", None)


def test_register_table_matches_loaded_kernels(gpu):
    # the planner's occupancy estimate rests on a table of registers per lane; it must describe
    # the code object that is actually loaded
    import ctypes
    import cutt_amd
    lib = ctypes.CDLL(cutt_amd.lib_path())
    for es in (4, 8):
        for e in (1, 2, 4, 8, 16):
            if e == 16 and es == 8:
                continue
            for wide in (0, 1):
                table = lib.cuttHipPackedRegsPerLane(es, e, wide)
                loaded = lib.cuttHipPackedRegsPerLaneLoaded(es, e, wide)
                say("packed kernel es=%d E=%d wide=%d: table %d, loaded %d" % (es, e, wide, table, loaded))
                assert loaded > 0
                # same allocation granule of 8 registers = same occupancy
                assert (table + 7) // 8 == (loaded + 7) // 8, (es, e, wide, table, loaded)


def test_random_ranks_up_to_15(gpu):
    # reference test2, seeded: random shapes and permutations for ranks 2..15
    rng = np.random.default_rng(2024)
    for rank in range(2, 16):
        for _ in range(4):
            target = float(rng.uniform(3.0 ** rank, max(3.0 ** rank * 2, 3.0e6)))
            target = min(target, 2.0e7)
            dim = [2] * rank
            while float(np.prod(dim, dtype=np.float64)) < target:
                dim[int(rng.integers(0, rank))] += 1
            perm = [int(p) for p in rng.permutation(rank)]
            es = 8 if rng.random() < 0.5 else 4
            say("random rank %d dim=%s perm=%s es=%d" % (rank, dim, perm, es))
            gpu.check_case(dim, perm, es)


def test_highest_ranks(gpu):
    # Every extent is at least 2 and a tensor has fewer than 2^32 elements, so rank 31 is the highest
    # rank that exists; the per-rank tables hold 32.  Ranks 20-28 against the oracle (all extents 2,
    # a few 3), random and reversing permutations, every method the planner offers.
    import cutt_amd as cutt
    rng = np.random.default_rng(31)
    for rank in (20, 24, 26, 28):
        dim = [2] * rank
        if rank <= 24:
            for i in rng.choice(rank, size=2, replace=False):
                dim[int(i)] = 3
        for perm in ([int(p) for p in rng.permutation(rank)], list(range(rank - 1, -1, -1))):
            es = 4 if rank >= 26 else 8
            for method in (0, cutt.METHOD_TILED, cutt.METHOD_PACKED, cutt.METHOD_PACKEDSPLIT):
                cutt.set_method_override(method)
                try:
                    rc, h = cutt.cuttPlan(rank, dim, perm, es, gpu.stream_handle())
                    if rc != cutt.CUTT_SUCCESS:
                        assert method != 0
                        continue
                    cutt.cuttDestroy(h)
                    say("rank %d perm=%s es=%d method %d" % (rank, perm, es, method))
                    info = gpu.check_case(dim, perm, es)
                finally:
                    cutt.set_method_override(0)


def test_ten_streams(gpu):
    # reference test4: ten plans on ten streams executing into the same buffers
    import torch
    import cutt_amd as cutt
    dim, perm = [24, 32, 16, 36, 43, 9], [5, 1, 4, 2, 3, 0]
    vol = int(np.prod(dim))
    data = gpu.seeded(vol, 8, 4)
    d_in = gpu.to_device(data)
    d_out = torch.full_like(d_in, -1)
    torch.cuda.synchronize()
    streams = [torch.cuda.Stream() for _ in range(10)]
    handles = []
    for s in streams:
        rc, h = cutt.cuttPlan(len(dim), dim, perm, 8, s.cuda_stream)
        assert rc == cutt.CUTT_SUCCESS
        assert cutt.cuttExecute(h, d_in.data_ptr(), d_out.data_ptr()) == cutt.CUTT_SUCCESS
        handles.append(h)
    torch.cuda.synchronize()
    import oracle
    assert np.array_equal(gpu.to_host(d_out, 8), oracle.transpose_mt(dim, perm, data, 8))
    assert len(set(handles)) == 10
    for h in handles:
        assert cutt.cuttDestroy(h) == cutt.CUTT_SUCCESS


def test_error_codes(gpu):
    # reference src/cutt.cpp:59-82, 193, 287-306
    import torch
    import cutt_amd as cutt
    st = gpu.stream_handle()
    bad = [((4, 4), (0, 0), 4), ((4, 1), (1, 0), 4), ((4, 4), (1, 0), 2), ((4,), (0,), 4), ((4, 4), (1, 2), 8),
           ((4, 4), (-1, 0), 8)]
    for dim, perm, es in bad:
        rc, _ = cutt.cuttPlan(len(dim), dim, perm, es, st)
        assert rc == cutt.CUTT_INVALID_PARAMETER
    a = torch.zeros(16, dtype=torch.int64, device="cuda")
    b = torch.zeros(16, dtype=torch.int64, device="cuda")
    rc, _ = cutt.cuttPlanMeasure(2, (4, 4), (1, 0), 8, st, a.data_ptr(), a.data_ptr())
    assert rc == cutt.CUTT_INVALID_PARAMETER
    rc, h = cutt.cuttPlan(2, (4, 4), (1, 0), 8, st)
    assert rc == cutt.CUTT_SUCCESS
    assert cutt.cuttExecute(h, a.data_ptr(), a.data_ptr()) == cutt.CUTT_INVALID_PARAMETER
    assert cutt.cuttExecute(h, a.data_ptr(), b.data_ptr()) == cutt.CUTT_SUCCESS
    torch.cuda.synchronize()
    assert cutt.cuttDestroy(h) == cutt.CUTT_SUCCESS
    assert cutt.cuttDestroy(h) == cutt.CUTT_INVALID_PLAN
    assert cutt.cuttExecute(h, a.data_ptr(), b.data_ptr()) == cutt.CUTT_INVALID_PLAN
    assert cutt.cuttExecute(0xFFFFFFF0, a.data_ptr(), b.data_ptr()) == cutt.CUTT_INVALID_PLAN


def test_special_bit_patterns(gpu):
    # NaNs, infinities, denormals and -0.0 move unchanged (elements are opaque words)
    words = np.array([0x7FC00001, 0xFFC12345, 0x00000001, 0x80000000, 0x7F800000, 0xFF800000,
                      0x7FA00000, 0x00000000], dtype=np.uint32)
    data = np.tile(words, 33 * 65 // 8 + 1)[: 33 * 65]
    gpu.check_case([33, 65], [1, 0], 4, data=data)
    data8 = (data.astype(np.uint64) << np.uint64(32)) | np.uint64(0x7FF00000)
    gpu.check_case([33, 65], [1, 0], 8, data=data8)


def test_plans_from_several_threads(gpu):
    # the handle table is shared; creating, executing and destroying plans from several host
    # threads at once must neither mix handles up nor corrupt results
    import threading
    import torch
    import cutt_amd as cutt
    import oracle
    shapes = [((31, 17, 45), (2, 0, 1), 8), ((64, 33, 20), (1, 2, 0), 4), ((5, 7, 11, 13), (3, 1, 0, 2), 8),
              ((129, 257), (1, 0), 4), ((8, 9, 10, 11), (2, 3, 0, 1), 4), ((300, 40, 7), (2, 1, 0), 8)]
    errors = []

    def worker(k):
        try:
            dim, perm, es = shapes[k % len(shapes)]
            vol = int(np.prod(dim))
            data = gpu.seeded(vol, es, seed=100 + k)
            want = oracle.transpose(list(dim), list(perm), data)
            stream = torch.cuda.Stream()
            with torch.cuda.stream(stream):
                d_in = gpu.to_device(data)
                d_out = torch.full_like(d_in, -1)
            stream.synchronize()
            for _ in range(20):
                rc, h = cutt.cuttPlan(len(dim), list(dim), list(perm), es, stream.cuda_stream)
                assert rc == cutt.CUTT_SUCCESS
                assert cutt.cuttExecute(h, d_in.data_ptr(), d_out.data_ptr()) == cutt.CUTT_SUCCESS
                stream.synchronize()
                assert cutt.cuttDestroy(h) == cutt.CUTT_SUCCESS
                assert cutt.cuttExecute(h, d_in.data_ptr(), d_out.data_ptr()) == cutt.CUTT_INVALID_PLAN
            got = gpu.to_host(d_out, es)
            assert np.array_equal(got, want), "thread %d: wrong bytes" % k
        except Exception as e:  # collected and re-raised in the main thread
            errors.append((k, repr(e)))

    threads = [threading.Thread(target=worker, args=(k,)) for k in range(8)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors, errors


def test_execute_under_graph_capture(gpu):
    # cuttExecute only launches a kernel (or a device-to-device copy) on the plan's stream, so it
    # can be captured into a HIP graph; every replay must transpose what the input holds then
    import torch
    import cutt_amd as cutt
    import oracle
    for dim, perm, es in (((129, 3, 257, 31), (2, 0, 3, 1), 8), ((64, 96, 50), (1, 2, 0), 4), ((40, 50, 60), (0, 1, 2), 8)):
        vol = int(np.prod(dim))
        stream = torch.cuda.Stream()
        with torch.cuda.stream(stream):
            d_in = gpu.to_device(gpu.seeded(vol, es, seed=1))
            d_out = torch.full_like(d_in, -1)
            rc, h = cutt.cuttPlan(len(dim), list(dim), list(perm), es, stream.cuda_stream)
            assert rc == cutt.CUTT_SUCCESS
            # first launch outside the capture: the runtime loads the library's code object then
            assert cutt.cuttExecute(h, d_in.data_ptr(), d_out.data_ptr()) == cutt.CUTT_SUCCESS
        stream.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            assert cutt.cuttExecute(h, d_in.data_ptr(), d_out.data_ptr()) == cutt.CUTT_SUCCESS
        for seed in (2, 3, 4):
            data = gpu.seeded(vol, es, seed=seed)
            d_in.copy_(gpu.to_device(data))
            d_out.fill_(-1)
            torch.cuda.synchronize()
            graph.replay()
            torch.cuda.synchronize()
            say("graph replay dim=%s es=%d seed=%d" % (dim, es, seed))
            assert np.array_equal(gpu.to_host(d_out, es), oracle.transpose(list(dim), list(perm), data))
        del graph
        assert cutt.cuttDestroy(h) == cutt.CUTT_SUCCESS


def test_identity_of_2_to_31_elements_is_a_copy(gpu):
    # the fused extent no longer fits an int, so the ranks stay apart; the plan is still Trivial
    import torch
    import cutt_amd as cutt
    st = gpu.stream_handle()
    n = 65536 * 32768
    a = torch.empty(n, dtype=torch.int32, device="cuda")
    a.random_()
    b = torch.zeros_like(a)
    rc, h = cutt.cuttPlan(2, (65536, 32768), (0, 1), 4, st)
    assert rc == cutt.CUTT_SUCCESS
    assert cutt.get_plan_info(h).method_name == "Trivial"
    assert cutt.cuttExecute(h, a.data_ptr(), b.data_ptr()) == cutt.CUTT_SUCCESS
    torch.cuda.synchronize()
    assert torch.equal(a, b)
    assert cutt.cuttDestroy(h) == cutt.CUTT_SUCCESS


def test_trivial_copy_sizes_alignments_and_cache_policies(gpu):
    # The Trivial method is a kernel of the library (16 bytes per lane), not the runtime's copy:
    # byte counts that are not multiples of 16, buffers that start off the 16-byte grid (those go
    # to the runtime's copy), each cache policy (chosen by size), and the words after the copied
    # range must stay untouched.
    import torch
    import cutt_amd as cutt
    st = gpu.stream_handle()
    cases = [((3, 3), 4), ((3, 5, 7), 4), ((2, 2), 4), ((2, 2), 8), ((3, 5, 7), 8), ((1023, 5), 4),
             ((1025, 1023), 4), ((4099, 4001), 8),            # 131 MB: ordinary accesses
             ((8193, 8191), 8),                               # 537 MB: streaming loads
             ((16385, 8191), 8)]                              # 1.07 GB: streaming loads and stores
    policies = set()
    for dim, es in cases:
        n = int(np.prod(dim))
        words = n * es // 4
        perm = tuple(range(len(dim)))
        rc, h = cutt.cuttPlan(len(dim), dim, perm, es, st)
        assert rc == cutt.CUTT_SUCCESS
        info = cutt.get_plan_info(h)
        assert info.method_name == "Trivial"
        policies.add(info.cachePolicy)
        for shift_in, shift_out in ((0, 0), (1, 0), (0, 2), (3, 3)):   # in 4-byte words
            if es == 8 and (shift_in % 2 or shift_out % 2):
                continue
            say("trivial dim=%s es=%d shifts=%d,%d policy=%d" % (dim, es, shift_in, shift_out, info.cachePolicy))
            a = torch.empty(words + 8, dtype=torch.int32, device="cuda")
            a.random_()
            b = torch.full((words + 8,), -1, dtype=torch.int32, device="cuda")
            src, dst = a[shift_in:shift_in + words], b[shift_out:shift_out + words]
            assert cutt.cuttExecute(h, src.data_ptr(), dst.data_ptr()) == cutt.CUTT_SUCCESS
            torch.cuda.synchronize()
            assert torch.equal(src, dst)
            assert bool((b[:shift_out] == -1).all()) and bool((b[shift_out + words:] == -1).all())
            del a, b
        assert cutt.cuttDestroy(h) == cutt.CUTT_SUCCESS
    assert policies == {0, 1, 3}


def test_planning_the_same_tensor_again_reuses_the_decision(gpu, monkeypatch):
    # cuttPlan keeps its last decisions: the second plan for a tensor is the same plan, made without
    # the enumeration and the cost model; both plans own their tables (destroying one leaves the
    # other working); another method override or CUTT_PLAN_CACHE=0 plans from scratch.
    import torch
    import cutt_amd as cutt
    import oracle
    dim, perm, es = (30, 3, 20, 9, 24, 29), (5, 2, 0, 4, 1, 3), 4
    vol = int(np.prod(dim))
    st = gpu.stream_handle()
    data = gpu.seeded(vol, es, seed=11)
    want = oracle.transpose_mt(list(dim), list(perm), data, 8)
    d_in = gpu.to_device(data)
    d_out = torch.full_like(d_in, -1)

    def plan():
        rc, h = cutt.cuttPlan(len(dim), dim, perm, es, st)
        assert rc == cutt.CUTT_SUCCESS
        d = cutt.get_plan_info(h).as_dict()
        return h, d, d.pop("planMs")

    def runs_right(h):
        d_out.fill_(-1)
        gpu.run_plan(h, d_in, d_out)
        return np.array_equal(gpu.to_host(d_out, es), want)

    cutt.clear_plan_cache()
    h1, info1, ms1 = plan()
    h2, info2, ms2 = plan()
    say("plan ms: first %.3f, again %.3f (%s, %d candidates)" % (ms1, ms2, info1["method_name"], info1["numCandidates"]))
    assert info1 == info2
    assert ms2 < 0.5 * ms1
    assert cutt.cuttDestroy(h1) == cutt.CUTT_SUCCESS
    assert runs_right(h2)
    assert cutt.cuttDestroy(h2) == cutt.CUTT_SUCCESS

    # a method the unrestricted planner did not choose
    other = cutt.METHOD_PACKED if info1["method_name"] == "Tiled" else cutt.METHOD_TILED
    cutt.set_method_override(other)
    try:
        h3, info3, _ = plan()
        assert info3["method"] == other and runs_right(h3)
        assert cutt.cuttDestroy(h3) == cutt.CUTT_SUCCESS
    finally:
        cutt.set_method_override(0)

    monkeypatch.setenv("CUTT_PLAN_CACHE", "0")
    h4, info4, ms4 = plan()
    assert info4 == info1 and ms4 > 2 * ms2 and runs_right(h4)
    assert cutt.cuttDestroy(h4) == cutt.CUTT_SUCCESS
    monkeypatch.delenv("CUTT_PLAN_CACHE")

    cutt.clear_plan_cache()
    h5, info5, ms5 = plan()
    assert info5 == info1 and ms5 > 2 * ms2
    assert cutt.cuttDestroy(h5) == cutt.CUTT_SUCCESS


def test_tiled_with_four_rows_per_lane_in_flight(gpu, monkeypatch):
    # The Tiled kernel's second instance (a lane requests its 16 tile rows four at a time): forced
    # on shapes with full, edge and thin tiles, both widths; then chosen by the planner itself on a
    # large tensor of 4-byte elements whose rows start off the 128-byte grid.
    import cutt_amd as cutt
    cases = [((43, 67), (1, 0)), ((64, 64), (1, 0)), ((65, 127, 3), (1, 0, 2)), ((130, 9, 70), (2, 1, 0)),
             ((1000, 30, 777), (2, 1, 0)), ((17, 5, 300), (2, 1, 0)), ((300, 5, 17), (2, 1, 0)),
             ((129, 3, 257, 31), (2, 1, 0, 3))]
    monkeypatch.setenv("CUTT_TILED_GROUPED", "1")
    cutt.set_method_override(cutt.METHOD_TILED)
    try:
        for dim, perm in cases:
            for es in (4, 8):
                say("grouped tiled dim=%s perm=%s es=%d" % (dim, perm, es))
                info = gpu.check_case(list(dim), list(perm), es)
                assert info.method_name == "Tiled" and info.tiledGrouped == 1
    finally:
        cutt.set_method_override(0)
    monkeypatch.delenv("CUTT_TILED_GROUPED")
    for es, want in ((4, 1), (8, 0)):
        say("planner's own choice, es=%d" % es)
        info = gpu.check_case([4457, 44570], [1, 0], es)
        assert info.method_name == "Tiled" and info.tiledGrouped == want


def test_tiled_with_line_aligned_stores(gpu, monkeypatch):
    # The Tiled kernel's instance in which every tile row stores its own window of 64 elements that
    # starts on a 128-byte line: forced on shapes whose output runs are shorter than a line, shorter
    # than a tile, a little longer than a tile, with uniform and with rotating misalignment, both
    # widths; the last tile along Mk may lie wholly beyond some rows' ends.
    import torch
    import cutt_amd as cutt
    cases = [((43, 67), (1, 0)), ((64, 64), (1, 0)), ((65, 127, 3), (1, 0, 2)), ((130, 9, 70), (2, 1, 0)),
             ((1000, 30, 777), (2, 1, 0)), ((17, 5, 300), (2, 1, 0)), ((300, 5, 17), (2, 1, 0)),
             ((129, 3, 257, 31), (2, 1, 0, 3)), ((200, 3), (1, 0)), ((70, 40), (1, 0)), ((96, 2, 66), (2, 1, 0)),
             ((64, 32, 96), (2, 1, 0)), ((33, 7, 5, 95), (3, 1, 2, 0))]
    monkeypatch.setenv("CUTT_TILED_ALIGNED", "1")
    cutt.set_method_override(cutt.METHOD_TILED)
    try:
        for dim, perm in cases:
            for es in (4, 8):
                say("aligned-store tiled dim=%s perm=%s es=%d" % (dim, perm, es))
                info = gpu.check_case(list(dim), list(perm), es)
                assert info.method_name == "Tiled"
        # an output buffer that itself starts off the line grid
        dim, perm, es = [130, 9, 70], [2, 1, 0], 4
        vol = int(np.prod(dim))
        data = gpu.seeded(vol, es, seed=5)
        d_in = gpu.to_device(data)
        big = torch.full((vol + 64,), -1, dtype=d_in.dtype, device="cuda")
        import oracle
        for shift in (1, 7, 32, 33):
            d_out = big[shift:shift + vol]
            rc, h = cutt.cuttPlan(len(dim), dim, perm, es, gpu.stream_handle())
            assert rc == cutt.CUTT_SUCCESS
            big.fill_(-1)
            gpu.run_plan(h, d_in, d_out)
            cutt.cuttDestroy(h)
            assert np.array_equal(gpu.to_host(d_out, es), oracle.transpose(dim, perm, data))
            assert bool((big[:shift] == -1).all()) and bool((big[shift + vol:] == -1).all())
    finally:
        cutt.set_method_override(0)


def test_measuring_planner_on_a_tensor_with_millions_of_tiny_tiles(gpu):
    # 50 million 2 x 2 tiles would need a grid beyond the dispatch limit: no such candidate may
    # be timed (it would "win" with a truncated grid)
    info = gpu.check_case([2, 7, 2, 14, 17141, 3], [2, 1, 5, 3, 4, 0], 4, how="measure")
    assert info.numBlocks * info.numThreads < 2 ** 32
    info = gpu.check_case([2, 7, 2, 14, 171412, 3], [2, 1, 5, 3, 4, 0], 4, how="measure")
    assert info.numBlocks * info.numThreads < 2 ** 32


def test_every_candidate_of_random_midsize_tensors(gpu):
    # Seeded random tensors of 0.3-2 M elements, ranks 3-7: every candidate of the enumeration runs
    # on the GPU (all elements-per-lane, cache-policy and offset-width instances the planner can
    # produce at this size) and must give the oracle's bytes.
    import cutt_amd as cutt
    import oracle
    rng = np.random.default_rng(77)
    done, executed = 0, 0
    methods = set()
    while done < 40:
        rank = int(rng.integers(3, 8))
        f = rng.uniform(1, 10, size=rank)
        vol = rng.uniform(3e5, 2e6)
        dim = [int(d) for d in np.maximum(2, np.round(f * (vol / np.prod(f)) ** (1.0 / rank)))]
        perm = [int(p) for p in rng.permutation(rank)]
        if perm == sorted(perm):
            continue
        es = 4 if done % 2 else 8
        v = int(np.prod(dim))
        data = gpu.seeded(v, es, seed=done)
        expect = oracle.transpose_mt(dim, perm, data, 8)
        with cutt.Candidates(dim, perm, es) as c:
            n = len(c)
        say("random midsize %d: dim=%s perm=%s es=%d, %d candidates" % (done, dim, perm, es, n))
        for i in range(n):
            info = gpu.check_case(dim, perm, es, data=data, how="candidate", candidate=i, expect=expect)
            methods.add(info.method_name)
            executed += 1
        done += 1
    say("executed %d candidates" % executed)
    assert {"Tiled", "Packed", "PackedSplit"} <= methods


def test_work_item_orders_of_the_packed_kernel(gpu):
    """The three ways of handing work items to workgroups (a workgroup walks neighbouring slabs,
    keeps its slabs and walks Mbar positions, or takes every B-th item of its XCD's chunk) forced on
    every Packed / PackedSplit candidate of tensors with even and uneven slabs."""
    import os
    import cutt_amd as cutt
    import oracle
    cases = [((179, 13, 5, 179, 8), (3, 4, 1, 2, 0)), ((64, 96, 40, 50), (2, 0, 3, 1)), ((31, 549, 2, 3, 9), (3, 0, 2, 4, 1)),
             ((1000, 7, 300), (2, 1, 0)), ((6, 5, 4, 3, 2, 7, 8, 9), (6, 0, 7, 3, 2, 5, 1, 4))]
    saved = os.environ.get("CUTT_ITEM_ORDER")
    seen = {0: 0, 1: 0, 2: 0}
    try:
        for dim, perm in cases:
            for es in (4, 8):
                data = gpu.seeded(int(np.prod(dim)), es, seed=len(dim))
                expect = oracle.transpose_mt(list(dim), list(perm), data, 8)
                for order in (0, 1, 2):
                    os.environ["CUTT_ITEM_ORDER"] = str(order)
                    with cutt.Candidates(dim, perm, es) as c:
                        idx = [i for i in range(len(c)) if c.info(i).method_name in ("Packed", "PackedSplit")]
                    say("item order %d dim=%s perm=%s es=%d: %d packed candidates" % (order, dim, perm, es, len(idx)))
                    for i in idx:
                        info = gpu.check_case(list(dim), list(perm), es, data=data, how="candidate", candidate=i, expect=expect)
                        assert info.itemOrder == order or (order == 1 and info.itemOrder == 0)  # order 1 needs several Mbar positions
                        seen[info.itemOrder] += 1
    finally:
        if saved is None:
            os.environ.pop("CUTT_ITEM_ORDER", None)
        else:
            os.environ["CUTT_ITEM_ORDER"] = saved
    assert min(seen.values()) > 20


def test_tile_orders_and_patch_shapes_of_the_tiled_kernels(gpu, monkeypatch):
    """Every numbering of the tiled kernels' workgroups (orders 0-6) with several super-tile shapes, on shapes
    with edge tiles, several Mbar ranks and a leading rank that stays (TiledCopy), both widths."""
    import cutt_amd as cutt
    import oracle
    cases = [((130, 9, 70), (2, 1, 0)), ((200, 3, 5, 333), (3, 1, 2, 0)), ((1000, 30, 777), (2, 1, 0)), ((64, 64), (1, 0)),
             ((257, 129, 6), (1, 0, 2)), ((150, 7, 300), (0, 2, 1)), ((512, 12, 512, 3), (2, 1, 0, 3))]
    shapes = [(1, 1), (2, 2), (3, 5), (8, 4096), (4, 1), (1, 4)]
    seen = set()
    for dim, perm in cases:
        for es in (4, 8):
            data = gpu.seeded(int(np.prod(dim)), es, seed=len(dim) + es)
            expect = oracle.transpose_mt(list(dim), list(perm), data, 8)
            for order in range(7):
                for sm, sk in (shapes if order >= 3 else shapes[:1]):
                    monkeypatch.setenv("CUTT_TILED_ORDER", str(order))
                    monkeypatch.setenv("CUTT_SUPER_M", str(sm))
                    monkeypatch.setenv("CUTT_SUPER_K", str(sk))
                    with cutt.Candidates(dim, perm, es) as c:
                        idx = [i for i in range(len(c)) if c.info(i).method_name in ("Tiled", "TiledCopy")]
                    assert idx, (dim, perm)
                    for i in idx:
                        info = gpu.check_case(list(dim), list(perm), es, data=data, how="candidate", candidate=i, expect=expect)
                        assert info.tiledOrder == order
                        seen.add((info.method_name, order))
        say("tile orders dim=%s perm=%s done" % (dim, perm))
    assert {("Tiled", o) for o in range(7)} <= seen and {("TiledCopy", o) for o in range(7)} <= seen


def test_tiled_over_fused_rank_sets(gpu):
    """Tiled candidates whose tile axes run over two to four fused ranks (the reference's README.md:197-199 lists
    them as future work): every candidate of shapes with short or ragged leading ranks on either side, both
    widths, against the oracle; and the device's count of the address stream against the host model's."""
    import cutt_amd as cutt
    cases = [((36, 50, 1000, 11), (2, 0, 3, 1)), ((7, 9, 11, 700, 5), (3, 1, 0, 4, 2)), ((700, 9, 36, 5, 11), (2, 3, 0, 4, 1)),
             ((6, 11, 50, 7, 13), (4, 3, 2, 1, 0)), ((3, 5, 7, 40, 9, 11), (5, 4, 3, 1, 0, 2)), ((166, 3, 500, 41), (2, 0, 3, 1)),
             ((100, 2, 3, 2, 90, 2, 3, 2), (4, 5, 6, 7, 3, 2, 1, 0))]
    sets = set()
    st = gpu.stream_handle()
    for dim, perm in cases:
        for es in (4, 8):
            data = gpu.seeded(int(np.prod(dim)), es, seed=es + len(dim))
            with cutt.Candidates(dim, perm, es) as c:
                idx = [i for i in range(len(c)) if c.info(i).method_name == "Tiled"]
            for i in idx:
                say("fused Tiled candidate %d dim=%s perm=%s es=%d" % (i, dim, perm, es))
                info = gpu.check_case(list(dim), list(perm), es, data=data, how="candidate", candidate=i)
                sets.add((info.numMm, info.numMk))
                if info.numMm > 1 or info.numMk > 1:
                    rc, h = cutt.cuttPlanFromCandidate(len(dim), list(dim), list(perm), es, st, i)
                    assert rc == cutt.CUTT_SUCCESS
                    dev, mod = cutt.count_address_stream(h, 0)
                    d, m = dev.as_dict(), mod.as_dict()
                    for k in ("rdInstr", "wrInstr", "rdLines", "wrLines", "rdSectors", "wrSectors", "wrPartialLines"):
                        assert d[k] == m[k], (dim, perm, es, k, d[k], m[k])
                    cutt.cuttDestroy(h)
    assert {(2, 1), (1, 2), (2, 2), (3, 1), (4, 1)} <= sets, sets


def test_free_tile_numbering(gpu, monkeypatch):
    """Tile order 7 (the workgroup index as a mixed-radix number whose digits are dealt out to the two tile
    coordinates and the Mbar position) on shapes with edge tiles, for Tiled and TiledCopy, both widths."""
    import cutt_amd as cutt
    import oracle
    cases = [((200, 6, 300, 3), (2, 1, 0, 3)), ((70, 130), (1, 0)), ((650, 3, 5, 70), (3, 1, 2, 0)), ((150, 7, 300), (0, 2, 1)),
             ((512, 12, 512, 3), (2, 1, 0, 3))]
    seen_lanes = 0
    for dim, perm in cases:
        for es in (4, 8):
            data = gpu.seeded(int(np.prod(dim)), es, seed=3 + es)
            expect = oracle.transpose_mt(list(dim), list(perm), data, 8)
            # both decoders of the kernels: digit by digit, and one digit per lane (which the library falls back from
            # where an Mbar digit runs over two ranks or the digits overshoot the Mbar extent)
            for lanes in ("0", "1"):
                monkeypatch.setenv("CUTT_DIGIT_LANES", lanes)
                for digits in ["m2,k8,b0,m0,k0", "b4,k2,m0,b0,k0", "k0,m0,b0", "m3,k3,b5,m3,k3,b0,m0,k0", "b0", "m2@2,b2@2,m2@1,k0,b2@1,b0,m0",
                               "m2,k8,b2,b3,m0,k0,b0", "b3,k2,m0,b2,k0,b0"]:
                    monkeypatch.setenv("CUTT_TILE_DIGITS", digits)
                    with cutt.Candidates(dim, perm, es) as c:
                        idx = [i for i in range(len(c)) if c.info(i).method_name in ("Tiled", "TiledCopy")]
                        one_per_lane = sum(int(c.data(i, 9)[0]) for i in idx)
                    assert idx
                    seen_lanes += one_per_lane
                    for i in idx:
                        info = gpu.check_case(list(dim), list(perm), es, data=data, how="candidate", candidate=i, expect=expect)
                        assert info.tiledOrder == 7
        say("tile digits dim=%s perm=%s done" % (dim, perm))
    assert seen_lanes >= 20   # the second decoder did run


def test_free_item_numbering(gpu, monkeypatch):
    """The packed kernel's work items numbered by digits (the item number as a mixed-radix number whose digits are
    dealt out to the slabs of the two cut ranks and the Mbar position): every candidate a digit text applies to,
    against the oracle, both widths."""
    import cutt_amd as cutt
    import oracle
    dim, perm = (48, 20, 36, 12), (2, 0, 3, 1)
    for es in (4, 8):
        data = gpu.seeded(int(np.prod(dim)), es, seed=11 + es)
        expect = oracle.transpose_mt(list(dim), list(perm), data, 8)
        ran = 0
        for digits in ["b2,m0,k0,b0", "b0,k0,m0", "k2,b0,m2,k0,m0", "m0,b3,k0,b0"]:
            monkeypatch.setenv("CUTT_ITEM_DIGITS", digits)
            with cutt.Candidates(dim, perm, es) as c:
                idx = [i for i in range(len(c)) if c.info(i).method_name in ("Packed", "PackedSplit") and c.info(i).tileDigits]
            for i in idx:
                info = gpu.check_case(list(dim), list(perm), es, data=data, how="candidate", candidate=i, expect=expect)
                assert info.tileDigits, (digits, i)
                ran += 1
        say("item digits es=%d: %d candidates" % (es, ran))
        assert ran >= 8


def test_address_bit_numberings_at_full_size(gpu):
    """The numberings the planner derives from address bits, at the sizes where it applies them (beyond the
    memory-side cache): packed candidates whose bit-11 digit is moved to the top, and Tiled candidates over fused
    rank sets and with two tiles along an axis numbered by addressBitOrder; against torch's permute on the device."""
    import torch
    import cutt_amd as cutt
    import sweep_runner
    cases = [((2, 4096, 256, 64), (0, 3, 1, 2), 4, ("Packed", "PackedSplit")),
             ((128, 256, 8, 128, 8), (2, 3, 0, 1, 4), 4, ("Packed", "PackedSplit")),
             ((1024, 1024, 128), (2, 1, 0), 8, ("Tiled",)),
             ((32, 32, 512, 256), (3, 2, 1, 0), 8, ("Tiled",)),
             ((131072, 8, 4, 32), (3, 2, 1, 0), 8, ("Tiled",))]
    st = gpu.stream_handle()
    for dim, perm, es, methods in cases:
        dim, perm = list(dim), list(perm)
        vol = int(np.prod(dim, dtype=np.int64))
        d_in = sweep_runner.index_pattern(vol, es)
        want = sweep_runner.expected_on_device(d_in, dim, perm)
        with cutt.Candidates(dim, perm, es) as c:
            idx = [i for i in range(len(c)) if c.info(i).method_name in methods and c.info(i).tileDigits]
            best = c.best
        assert idx, (dim, perm)
        idx = sorted(idx, key=lambda i: i != best)[:6]
        for i in idx:
            d_out = torch.full_like(d_in, -1)
            rc, h = cutt.cuttPlanFromCandidate(len(dim), dim, perm, es, st, i)
            assert rc == cutt.CUTT_SUCCESS
            info = cutt.get_plan_info(h)
            say("dim=%s perm=%s es=%d candidate %d %s digits %s" % (dim, perm, es, i, info.method_name, info.tileDigits.decode()))
            assert info.tileDigits
            assert cutt.cuttExecute(h, d_in.data_ptr(), d_out.data_ptr()) == cutt.CUTT_SUCCESS
            torch.cuda.synchronize()
            assert torch.equal(d_out, want), (dim, perm, i)
            cutt.cuttDestroy(h)
        del d_in, want
