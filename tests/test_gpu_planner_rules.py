"""The planner's measured rules, each checked on seeded tensors of its class that it was not found on: the plan
with the rule must not be slower than the plan without it (the rule switched off through its environment knob),
timed in turn in one process.  A rule that stops paying - after a kernel change, on other silicon - shows here."""
import os
import sys

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def say(msg):
    print(msg, flush=True)
    sys.stdout.flush()


def timed_pair(cfg, env_off, reps=4, launches=3):
    """GB/s of cuttPlan's plan as it is and with the variables of env_off set, timed in turn; both outputs checked
    on the device against torch's permute of the index pattern."""
    import torch
    import cutt_amd as cutt
    import sweep_runner
    dim, perm, es = list(cfg["dim"]), list(cfg["perm"]), cfg["es"]
    vol = int(np.prod(dim, dtype=np.int64))
    st = torch.cuda.current_stream().cuda_stream
    d_in = sweep_runner.index_pattern(vol, es)
    d_out = torch.empty_like(d_in)
    want = sweep_runner.expected_on_device(d_in, dim, perm)
    saved = {k: os.environ.get(k) for k in list(env_off) + ["CUTT_PLAN_CACHE"]}
    os.environ["CUTT_PLAN_CACHE"] = "0"
    handles = {}
    try:
        rc, handles["on"] = cutt.cuttPlan(len(dim), dim, perm, es, st)
        assert rc == cutt.CUTT_SUCCESS, (rc, cfg)
        os.environ.update(env_off)
        rc, handles["off"] = cutt.cuttPlan(len(dim), dim, perm, es, st)
        assert rc == cutt.CUTT_SUCCESS, (rc, cfg, env_off)
    finally:
        for k, v in saved.items():
            if v is None:
                os.environ.pop(k, None)
            else:
                os.environ[k] = v
    infos = {k: cutt.get_plan_info(h) for k, h in handles.items()}
    best = {k: float("inf") for k in handles}
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    for _ in range(reps):
        for k, h in handles.items():
            d_out.fill_(-1)
            assert cutt.cuttExecute(h, d_in.data_ptr(), d_out.data_ptr()) == cutt.CUTT_SUCCESS
            torch.cuda.synchronize()
            assert torch.equal(d_out, want), (cfg, k)
            e0.record()
            for _ in range(launches):
                assert cutt.cuttExecute(h, d_in.data_ptr(), d_out.data_ptr()) == cutt.CUTT_SUCCESS
            e1.record()
            torch.cuda.synchronize()
            best[k] = min(best[k], e0.elapsed_time(e1) / launches)
    for h in handles.values():
        cutt.cuttDestroy(h)
    gb = 2.0 * vol * es / 1e6
    return gb / best["on"], gb / best["off"], infos["on"], infos["off"]


# The floors of these checks leave room for the timing noise of a fresh machine: a single plan's ratio moves by
# 2-3 % from run to run (the lowest of eight by up to 5 %), a mean over eight by about 1 %.
def run_rule(name, cases, env_off, applies, mean_floor, min_floor, need):
    import torch
    assert torch.cuda.is_available(), "this test needs the MI355X"
    import cutt_amd
    cutt_amd.lib()
    cutt_amd.set_method_override(0)
    ratios = []
    for cfg in cases:
        on, off, i_on, i_off = timed_pair(cfg, env_off)
        used = applies(i_on, i_off)
        say("%s dim=%s perm=%s es=%d: with %s %.0f GB/s, without %s %.0f GB/s, ratio %.3f%s" %
            (name, cfg["dim"], cfg["perm"], cfg["es"], i_on.method_name, on, i_off.method_name, off, on / off,
             "" if used else "  (rule not used: not counted)"))
        if used:
            ratios.append(on / off)
    assert len(ratios) >= need, (name, len(ratios))
    ratios = np.array(ratios)
    say("%s: %d plans, with / without: mean %.3f min %.3f max %.3f" % (name, len(ratios), ratios.mean(), ratios.min(), ratios.max()))
    assert ratios.mean() >= mean_floor and ratios.min() >= min_floor, (name, ratios)


def pow2_batched(seed, count):
    rng = np.random.default_rng(seed)
    out = []
    while len(out) < count:
        a, b = int(rng.integers(8, 13)), int(rng.integers(8, 13))
        es = 8 if len(out) % 2 == 0 else 4
        j = (27 if es == 4 else 26) - a - b
        if j < 1 or (2 ** b) // 64 >= 128:
            continue
        last = int(rng.choice([3, 5, 6]))
        out.append(dict(dim=(2 ** a, 2 ** j, 2 ** b, last), perm=(2, 1, 0, 3), es=es))
    return out


def test_workgroups_numbered_by_address_bits():
    # batched transposes on power-of-two addresses (other extents than the tensors the rule was derived on: last
    # rank 5 and 6, both widths); found: +8 % in the mean over 35 + 36 such tensors
    run_rule("address bits (Tiled)", pow2_batched(2027, 10), {"CUTT_ADDRESS_BITS": "0"},
             lambda on, off: on.method_name == "Tiled" and on.tiledOrder == 7, 1.02, 0.90, 6)


def test_packed_items_with_address_bit_11_moving():
    # seeded tensors with power-of-two extents whose plan is a packed one with its bit-11 digit moved
    # (found: +6 ... +13 % on four of five such plans, -3 % on one; on 52 other seeded plans, these twelve among
    # them: +4.7 % in the mean, -7 ... +26 %, over the 43 whose moved digit is the written bit 11, +2 %,
    # -15 ... +19 %, over the 9 where it is the read one.  This dozen holds two of the three plans that lose
    # 6-15 % and reads 0.99 in the mean, hence the bound below 1)
    import torch  # noqa: F401  (before the library is loaded: both must share one HIP runtime)
    import cutt_amd as cutt
    rng = np.random.default_rng(515)
    cases = []
    tries = 0
    while len(cases) < 12 and tries < 8000:
        tries += 1
        rank = int(rng.integers(3, 7))
        es = 8 if tries % 2 == 0 else 4
        tot = 27 if es == 8 else 28
        cuts = np.sort(rng.choice(np.arange(1, tot), size=rank - 1, replace=False))
        dim = tuple(int(2 ** e) for e in np.diff(np.concatenate(([0], cuts, [tot]))))
        perm = tuple(int(p) for p in rng.permutation(rank))
        if perm == tuple(range(rank)):
            continue
        with cutt.Candidates(dim, perm, es) as c:
            info = c.info(c.best)
            if info.method_name in ("Packed", "PackedSplit") and info.tileDigits:
                cases.append(dict(dim=dim, perm=perm, es=es))
    assert len(cases) == 12, tries
    run_rule("address bit 11 (packed)", cases, {"CUTT_ADDRESS_BITS": "0"},
             lambda on, off: bool(on.tileDigits) and on.method_name == off.method_name, 0.96, 0.78, 8)


def test_run_length_term_of_the_model_for_runs_on_the_line_grid(monkeypatch):
    # seeded tensors with power-of-two extents (every run on the 128-byte grid) whose plan changes with the model's
    # term for the shorter of a packed candidate's two run lengths (found: the plan changed on 41 of 182 such
    # tensors, +3.6 % in the mean over those, -15 ... +25 %; four 4-byte matrices +12 ... +28 %)
    import torch  # noqa: F401  (before the library is loaded: both must share one HIP runtime)
    import cutt_amd as cutt
    rng = np.random.default_rng(90210)
    cases = []
    tries = 0

    def geometry(dim, perm, es):
        with cutt.Candidates(dim, perm, es) as c:
            i = c.info(c.best)
            return i.method, i.volMmk, i.numSplit, i.numSplit2, i.numMm, i.numMk

    while len(cases) < 14 and tries < 4000:
        tries += 1
        rank = int(rng.integers(2, 7))
        es = 8 if tries % 2 == 0 else 4
        tot = int(rng.integers(26, 29)) if es == 4 else int(rng.integers(25, 28))
        if rank >= tot:
            continue
        cuts = np.sort(rng.choice(np.arange(1, tot), size=rank - 1, replace=False))
        dim = tuple(int(2 ** e) for e in np.diff(np.concatenate(([0], cuts, [tot]))))
        perm = tuple(int(p) for p in rng.permutation(rank))
        if perm == tuple(range(rank)):
            continue
        with_term = geometry(dim, perm, es)
        monkeypatch.setenv("CUTT_MODEL_RUN_LENGTH", "0")
        without = geometry(dim, perm, es)
        monkeypatch.delenv("CUTT_MODEL_RUN_LENGTH")
        if with_term != without:
            cases.append(dict(dim=dim, perm=perm, es=es))
    assert len(cases) == 14, tries
    run_rule("run lengths on the line grid (model)", cases, {"CUTT_MODEL_RUN_LENGTH": "0"},
             lambda on, off: True, 0.99, 0.82, 10)


def test_tiles_over_fused_rank_sets():
    # random tensors whose leading ranks are short on one side (found: +13 ... +21 % on three sweep tensors)
    import baseline_configs as bc
    rng = np.random.default_rng(99)
    cases = []
    while len(cases) < 18:
        rank = int(rng.integers(4, 7))
        rest = bc.random_dims(rng, rank - 1, target=2.0e8 / 24, tol=0.2)
        dim = [int(rng.integers(8, 40))] + [int(d) for d in rest]
        perm = [int(p) for p in rng.permutation(rank)]
        if perm[0] == 0 or perm == list(range(rank)):
            continue
        cases.append(dict(dim=tuple(dim), perm=tuple(perm), es=8 if len(cases) % 2 == 0 else 4))
    run_rule("tiles over fused rank sets", cases, {"CUTT_TILED_FUSE": "0"},
             lambda on, off: on.method_name == "Tiled" and (on.numMm > 1 or on.numMk > 1), 1.02, 0.90, 3)


def test_strips_sixteen_wide_for_rows_32_kb_apart():
    # 4-byte tensors whose input rows are a multiple of 32 KB apart (found: +8 ... +15 % on forty such tensors)
    rng = np.random.default_rng(8)
    cases = []
    while len(cases) < 6:
        n = int(rng.integers(1, 4))
        rows = int(rng.integers(6500, 12000))
        cases.append(dict(dim=(8192 * n, rows // n), perm=(1, 0), es=4))
    run_rule("16-wide strips", cases, {"CUTT_SUPER_M": "8"},
             lambda on, off: on.method_name == "Tiled" and off.method_name == "Tiled" and on.superM == 16, 1.03, 0.95, 4)


def test_rows_in_groups_for_unaligned_four_byte_rows():
    # 4-byte three-rank reversals off the line grid, 1.1-3.5 cache sizes per buffer (found: +5 % median on 164 plans)
    rng = np.random.default_rng(31)
    cases = []
    while len(cases) < 8:
        a, b = int(rng.integers(300, 900)), int(rng.integers(300, 900))
        c = int(1.5e8 / (a * b))
        if a % 32 == 0 or c % 32 == 0 or c < 100:
            continue
        cases.append(dict(dim=(a, b, c), perm=(2, 1, 0), es=4))
    run_rule("rows in groups", cases, {"CUTT_TILED_GROUPED": "0"},
             lambda on, off: on.method_name == "Tiled" and off.method_name == "Tiled" and on.tiledGrouped == 1 and off.tiledGrouped == 0,
             1.0, 0.93, 4)


def test_patches_for_eight_byte_rows_on_the_line_grid():
    # 8-byte tensors whose rows start on 128-byte lines, many tiles along both axes, an Mbar rank between Mm and Mk
    # (found: +2.5 % in the mean over 14 random such tensors, -1.7 ... +9 %; on 27 tensors it was not found on +1 %,
    # -7 ... +9 %, which is why the bound is that it does not lose); strips of 8 tiles through all of Mk are what the
    # rule replaces
    rng = np.random.default_rng(77)
    cases = []
    while len(cases) < 10:
        # (multiples of 64: no tile axis over fused ranks competes, the plan is the one-rank-per-side Tiled plan)
        a, b = 64 * int(rng.integers(10, 30)), 64 * int(rng.integers(18, 40))
        if (a & (a - 1)) == 0 or (b & (b - 1)) == 0:
            continue
        if len(cases) % 2 == 0:
            c = int(1.6e8 / (a * b))
            dim, perm = (a, c, b), (2, 1, 0)
        else:
            c = int(rng.integers(3, 12))
            dim, perm = (a, c, b, int(1.6e8 / (a * b * c))), (2, 1, 0, 3)
        if min(dim) < 3:
            continue
        cases.append(dict(dim=dim, perm=perm, es=8))
    run_rule("patches", cases, {"CUTT_SUPER_M": "8", "CUTT_SUPER_K": "4096"},
             lambda on, off: on.method_name == "Tiled" and off.method_name == "Tiled" and on.tiledOrder == 5 and on.superK < off.superK,
             0.985, 0.91, 5)


def test_one_strip_for_a_rank_of_nine_to_fourteen_tiles():
    # a leading rank of 9-14 tiles off the line grid is walked as one strip (found: +2.8 % in the mean over 13 tensors)
    rng = np.random.default_rng(404)
    cases = []
    while len(cases) < 18:
        a = int(rng.integers(9 * 64 - 40, 14 * 64))
        b = int(rng.integers(200, 1500))
        c = int(1.5e8 / (a * b))
        if a % 16 == 0 or c < 64:
            continue
        perm = [(2, 1, 0), (1, 0, 2), (1, 2, 0)][len(cases) % 3]
        cases.append(dict(dim=(a, b, c), perm=perm, es=8 if len(cases) % 2 == 0 else 4))
    # (46 such plans: +2 % in the mean, single ones -7 ... +16 %)
    run_rule("one strip", cases, {"CUTT_SUPER_M": "8"},
             lambda on, off: on.method_name == "Tiled" and off.method_name == "Tiled" and on.superM > 8 and on.numMm == 1,
             0.995, 0.88, 8)


def test_thin_second_tile_lets_the_tiles_along_mk_run_fastest():
    # two tiles along Mm of which the second is thin, at most 64 tiles along Mk (found: 10-25 % faster in order 2)
    rng = np.random.default_rng(12)
    cases = []
    while len(cases) < 8:
        es = 8 if len(cases) % 2 == 0 else 4
        a = 64 + int(rng.integers(3, 24 if es == 8 else 40))
        b = int(rng.integers(3 * 64, 60 * 64))
        c = int(1.2e8 / (a * b))
        if c < 8:
            continue
        # (the ranks that lead the two sides are neighbours, so no tile axis over fused ranks replaces the thin tile)
        cases.append(dict(dim=(a, b, c), perm=(1, 0, 2), es=es))
    run_rule("thin second tile", cases, {"CUTT_TILED_ORDER": "5"},
             lambda on, off: on.method_name == "Tiled" and off.method_name == "Tiled" and on.tiledOrder == 2,
             1.0, 0.93, 3)


def test_output_rows_front_to_back_for_matrices_on_the_line_grid():
    # matrices and batches of separate matrices with extents that are multiples of 64, 17-700 tiles along Mk and 16
    # and more along Mm: the tiles along Mk run fastest instead of strips (found: +4 % in the mean over 90 such
    # plans of three seeded sets, most between -2 and +9 %)
    rng = np.random.default_rng(2718)
    cases = []
    while len(cases) < 16:
        es = 4 if len(cases) % 2 == 0 else 8
        batch = 1 if len(cases) % 4 < 2 else int(rng.integers(2, 7))
        total = 2.0 ** rng.uniform(26.2, 28.2) * 4 / es / batch
        n = 64 * int(rng.integers(17, 500))
        m = int(total / n) // 64 * 64
        row = m * es
        if m < 1024 or row % 4096 == 0 or not (1024 <= row % 16384 <= 16384 - 1024):
            continue
        cases.append(dict(dim=(m, n) if batch == 1 else (m, n, batch), perm=(1, 0) if batch == 1 else (1, 0, 2), es=es))
    plain = [c for c in cases if len(c["dim"]) == 2]
    batched = [c for c in cases if len(c["dim"]) == 3]
    used = lambda on, off: on.method_name == "Tiled" and off.method_name == "Tiled" and on.tiledOrder == 2 and off.tiledOrder != 2
    run_rule("output rows front to back (matrices)", plain, {"CUTT_TILED_ORDER": "3"}, used, 1.01, 0.93, 5)
    run_rule("output rows front to back (batches)", batched, {"CUTT_TILED_ORDER": "5"}, used, 1.01, 0.93, 5)


def test_whole_mm_axis_at_a_stretch_for_fused_mm_sets_on_the_line_grid():
    # a fused Mm axis of which one rank follows Mk in the output, every row on the 128-byte grid on both sides: all
    # tiles along Mm run fastest (order 1) instead of strips of 8 (found: +3.2 % in the mean over 50 seeded plans of
    # two sets, -1.8 % at worst)
    rng = np.random.default_rng(1618)
    cases = []
    while len(cases) < 12:
        es = 4 if len(cases) % 2 == 0 else 8
        a = int(rng.choice([2, 4, 6, 8, 12, 16, 24, 32]))
        b = int(rng.integers(2, 40)) * (32 // int(np.gcd(a, 32)))
        if a * b < 128 or a * b > 8192:
            continue
        c = int(rng.integers(2, 10))
        k = int(2.0 ** rng.uniform(26.3, 27.5) * 4 / es / (a * b * c)) // 32 * 32
        if k < 512:
            continue
        kind = len(cases) % 3
        if kind == 0:
            dim, perm = (a, b, k, c), (2, 1, 3, 0)
        elif kind == 1:
            dim, perm = (a, b, c, k), (3, 1, 2, 0)
        else:
            dim, perm = (a, b, k), (2, 1, 0)
        cases.append(dict(dim=dim, perm=perm, es=es))
    run_rule("whole Mm axis at a stretch", cases, {"CUTT_TILED_ORDER": "3"},
             lambda on, off: on.method_name == "Tiled" and off.method_name == "Tiled" and on.numMm > 1 and on.tiledOrder == 1,
             0.99, 0.95, 5)


def test_work_items_per_workgroup_and_their_order():
    # packed plans: the planner's items per workgroup (two for 8-byte blocks of 10 KB and more, else four) against
    # four always, and the order in which a workgroup takes its items (its own slabs at several Mbar positions
    # when slabs of two sizes alternate) against neighbouring slabs always
    import baseline_configs as bc
    rng = np.random.default_rng(2718)
    cases = []
    while len(cases) < 14:
        rank = int(rng.integers(4, 8))
        dim = bc.random_dims(rng, rank, target=1.6e8, tol=0.1)
        perm = [int(p) for p in rng.permutation(rank)]
        if perm == list(range(rank)):
            continue
        cases.append(dict(dim=tuple(dim), perm=tuple(perm), es=8 if len(cases) % 2 == 0 else 4))
    packed = ("Packed", "PackedSplit")
    run_rule("items per workgroup", cases, {"CUTT_MAX_ITEMS": "4"},
             lambda on, off: on.method_name in packed and off.method_name == on.method_name and on.itemsPerBlock != off.itemsPerBlock,
             0.995, 0.94, 3)
    run_rule("work-item order", cases, {"CUTT_ITEM_ORDER": "0"},
             lambda on, off: on.method_name in packed and off.method_name == on.method_name and on.itemOrder != 0,
             0.99, 0.93, 2)


def test_cache_policy_of_the_global_accesses():
    # the policy the planner derives from size and address stream against each of the three pinned, on tensors
    # from inside the memory-side cache to four times its size: not more than 3 % behind the best of the three in
    # the mean
    import baseline_configs as bc
    import torch
    import cutt_amd
    assert torch.cuda.is_available(), "this test needs the MI355X"
    cutt_amd.lib()
    cutt_amd.set_method_override(0)
    rng = np.random.default_rng(1618)
    behind = []
    for k in range(12):
        rank = int(rng.integers(2, 6))
        es = 8 if k % 2 == 0 else 4
        target = [1.2e7, 3.0e7, 6.0e7, 1.2e8, 2.4e8, 4.0e8][k // 2] * (8 // es) / 2
        dim = bc.random_dims(rng, rank, target=target, tol=0.1)
        perm = [int(p) for p in rng.permutation(rank)]
        if perm == list(range(rank)):
            perm = perm[::-1]
        cfg = dict(dim=tuple(dim), perm=tuple(perm), es=es)
        rates = {}
        for pol in ("0", "1", "3"):
            on, off, i_on, i_off = timed_pair(cfg, {"CUTT_CACHE_POLICY": pol})
            rates[pol] = off
            rates["planner"] = max(rates.get("planner", 0.0), on)
        best = max(rates[p] for p in ("0", "1", "3"))
        say("cache policy dim=%s perm=%s es=%d (%.0f MB per buffer): planner (policy %d) %.0f GB/s; pinned 0 / 1 / 3: %.0f / %.0f / %.0f" %
            (cfg["dim"], cfg["perm"], es, np.prod(dim) * es / 1e6, i_on.cachePolicy, rates["planner"], rates["0"], rates["1"], rates["3"]))
        behind.append(rates["planner"] / best)
    behind = np.array(behind)
    say("cache policy: planner / best pinned: mean %.3f min %.3f" % (behind.mean(), behind.min()))
    assert behind.mean() >= 0.97 and behind.min() >= 0.88, behind


def test_order_of_the_mbar_ranks():
    # for the model's three best candidates cuttPlan also estimates the other orders in which consecutive work
    # items walk the Mbar ranks and keeps the cheapest; against the default order pinned (found: the same block
    # shape 430 us against 521 us walked the other way)
    import baseline_configs as bc
    rng = np.random.default_rng(4711)
    cases = []
    while len(cases) < 70:
        rank = int(rng.integers(4, 8))
        dim = bc.random_dims(rng, rank, target=1.6e8, tol=0.1)
        perm = [int(p) for p in rng.permutation(rank)]
        if perm == list(range(rank)):
            continue
        cases.append(dict(dim=tuple(dim), perm=tuple(perm), es=8 if len(cases) % 2 == 0 else 4))
    run_rule("Mbar order", cases, {"CUTT_MBAR_ORDER": "2"},
             lambda on, off: abs(on.usPredicted - off.usPredicted) > 1e-6 * off.usPredicted or on.method_name != off.method_name,
             0.97, 0.90, 3)   # (13 changed plans of 150 random tensors: +1.9 % in the mean, -1 ... +9 %)


def test_strips_per_mbar_position_for_fused_mm_sets():
    # a tile axis over fused ranks of which one follows Mk in the output: all strips along Mm pass before the Mbar
    # position moves on (found: 772-862 us against 1015-1257 us on six tensors of the reference's suites)
    import cutt_amd as cutt
    import baseline_configs as bc
    rng = np.random.default_rng(31337)
    cases = []
    tries = 0
    while len(cases) < 6 and tries < 3000:
        tries += 1
        rank = int(rng.integers(4, 7))
        rest = bc.random_dims(rng, rank - 1, target=1.6e8 / 20, tol=0.2)
        dim = tuple([int(rng.integers(6, 36))] + [int(d) for d in rest])
        perm = tuple(int(p) for p in rng.permutation(rank))
        if perm[0] == 0 or perm == tuple(range(rank)):
            continue
        es = 8 if tries % 2 == 0 else 4
        with cutt.Candidates(dim, perm, es) as c:
            info = c.info(c.best)
            if info.method_name == "Tiled" and info.numMm > 1 and info.tiledOrder == 3 and info.volMbar > 1:
                cases.append(dict(dim=dim, perm=perm, es=es))
    assert len(cases) == 6, tries
    run_rule("strips per Mbar position", cases, {"CUTT_TILED_ORDER": "5"},
             lambda on, off: on.method_name == "Tiled" and off.method_name == "Tiled" and on.tiledOrder == 3 and off.tiledOrder == 5,
             1.0, 0.93, 3)
