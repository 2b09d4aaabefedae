"""Host planner: rank fusing, candidate enumeration and index tables (no GPU).

Every candidate's address stream is replayed with numpy (plan_emulator.py) and
compared with the CPU oracle, so table or geometry mistakes show up here
before any kernel runs.
"""
import itertools

import numpy as np
import pytest

from plan_emulator import emulate
from test_oracle import REDUCE_CASES


@pytest.mark.parametrize("dim,perm,rdim,rperm", REDUCE_CASES)
def test_reduce_ranks_hand_cases(cutt, dim, perm, rdim, rperm):
    assert cutt.reduce_ranks(dim, perm) == (rdim, rperm)


def test_reduce_ranks_matches_oracle(cutt, oracle_mod):
    rng = np.random.default_rng(1)
    for _ in range(300):
        rank = int(rng.integers(2, 16))
        dim = [int(d) for d in rng.integers(2, 10, size=rank)]
        perm = [int(p) for p in rng.permutation(rank)]
        if rng.random() < 0.5:  # make fusable runs likely
            perm = sorted(perm[: rank // 2]) + perm[rank // 2:]
        assert cutt.reduce_ranks(dim, perm) == oracle_mod.reduce_ranks(dim, perm)


def check_all_candidates(cutt, oracle_mod, dim, perm, es, lds=0, need=None):
    dtype = np.uint32 if es == 4 else np.uint64
    vol = int(np.prod(dim))
    data = (np.arange(vol, dtype=np.uint64) * 2654435761 % (2 ** 31)).astype(dtype)
    expect = oracle_mod.transpose(dim, perm, data)
    seen = set()
    with cutt.Candidates(dim, perm, es, lds) as c:
        assert len(c) >= 1
        assert 0 <= c.best < len(c)
        for i in range(len(c)):
            info = c.info(i)
            seen.add(info.method_name)
            out, count = emulate(c, i, data)
            assert count.min() == 1 and count.max() == 1, (dim, perm, info.method_name, "write coverage")
            assert np.array_equal(out, expect), (dim, perm, es, info.as_dict())
    if need:
        assert need in seen, (need, seen)
    return seen


@pytest.mark.parametrize("rank", [2, 3, 4, 5])
def test_all_permutations_small(cutt, oracle_mod, rank):
    # shapes of the reference's test1 (src/cutt_test.cpp:138-158): dim[r] = 2 + r*14/rank
    dim = [2 + r * 14 // rank for r in range(rank)]
    for perm in itertools.permutations(range(rank)):
        for es in (4, 8):
            check_all_candidates(cutt, oracle_mod, dim, perm, es)


@pytest.mark.parametrize("rank", [6, 7])
def test_sampled_permutations_rank67(cutt, oracle_mod, rank):
    dim = [2 + r * 14 // rank for r in range(rank)]
    rng = np.random.default_rng(rank)
    for _ in range(6):
        perm = [int(p) for p in rng.permutation(rank)]
        check_all_candidates(cutt, oracle_mod, dim, perm, 8 if rng.random() < 0.5 else 4)


def test_small_lds_forces_split(cutt, oracle_mod):
    # With 2-4 KB of LDS even small tensors need PackedSplit, including uneven slabs.
    rng = np.random.default_rng(2)
    seen = set()
    for _ in range(40):
        rank = int(rng.integers(2, 6))
        dim = [int(d) for d in rng.integers(2, 24, size=rank)]
        perm = [int(p) for p in rng.permutation(rank)]
        es = 4 if rng.random() < 0.5 else 8
        seen |= check_all_candidates(cutt, oracle_mod, dim, perm, es, lds=int(rng.choice([1024, 2048, 4096])))
    assert "PackedSplit" in seen and "Packed" in seen and "Tiled" in seen and "TiledCopy" in seen


HAND_PICKED = [  # reference src/cutt_test.cpp:245-366 (test3), shrunk where the volume is large
    ((43, 67), (1, 0), "Tiled"),
    ((4099, 2), (1, 0), "Tiled"),
    ((131, 59, 8), (0, 2, 1), "TiledCopy"),
    ((24, 33, 8, 7), (1, 0, 2, 3), "Tiled"),
    ((5, 12, 15, 16, 7), (1, 3, 4, 2, 0), "Packed"),
    ((5, 3, 2, 9, 14), (0, 1, 3, 2, 4), "TiledCopy"),
    ((24, 8, 4, 6, 7, 3), (5, 1, 4, 2, 3, 0), "Packed"),
]


@pytest.mark.parametrize("dim,perm,need", HAND_PICKED)
def test_hand_picked(cutt, oracle_mod, dim, perm, need):
    for es in (4, 8):
        check_all_candidates(cutt, oracle_mod, dim, perm, es, need=need)


def test_identity_gives_trivial(cutt):
    for dim in [(2, 5, 9, 12), (2, 4, 6, 9, 11, 13)]:
        with cutt.Candidates(dim, range(len(dim)), 8) as c:
            assert len(c) == 1 and c.info(0).method_name == "Trivial"


def test_two_to_the_31_elements_and_more(cutt):
    # Beyond the reference's int volumes: up to 2^32 - 1 elements are planned.  A fused extent must
    # still fit an int, so the ranks of such an identity stay apart and it is still a plain copy.
    assert cutt.reduce_ranks((46341, 46341), (0, 1)) == ([46341, 46341], [0, 1])
    assert cutt.reduce_ranks((4, 46341, 46341), (1, 2, 0)) == ([4, 46341, 46341], [1, 2, 0])
    with cutt.Candidates((65536, 32768), (0, 1), 4) as c:
        assert len(c) == 1 and c.info(0).method_name == "Trivial"
    infos, best = method_set(cutt, (1291, 1290, 1290), (2, 0, 1), 4)
    names = {i.method_name for i in infos}
    assert "Tiled" in names and "PackedSplit" in names
    for i in infos:
        assert 0 < i.volMbar < 2 ** 31 and i.numBlocks < 2 ** 31
    # every Mbar position must stay below 2^31 for the kernels' division: a candidate whose
    # staged block is tiny is dropped, the others remain
    infos, best = method_set(cutt, (2, 2, 32768, 32767), (1, 0, 3, 2), 8)
    assert infos and all(i.volMbar < 2 ** 31 for i in infos)


def test_no_grid_beyond_the_dispatch_limit(cutt):
    # workgroups x lanes of a launch must fit a 32-bit count (the runtime truncates a larger grid
    # without an error): a Tiled candidate with tens of millions of 2 x 2 tiles is not offered, and
    # packed candidates take more work items per workgroup instead
    for dim, perm, es in [((2, 7, 2, 14, 171412, 3), (2, 1, 5, 3, 4, 0), 4), ((2, 3, 2, 2, 4000000, 2), (2, 1, 0, 5, 4, 3), 8),
                          ((3, 2, 16000000, 2), (1, 0, 3, 2), 4)]:
        infos, best = method_set(cutt, dim, perm, es)
        assert infos
        for i in infos:
            assert i.numBlocks * i.numThreads < 2 ** 32, (dim, perm, i.as_dict())


def test_invalid_problems_rejected(cutt):
    for dim, perm, es in [((4, 4), (0, 0), 4), ((4, 1), (1, 0), 4), ((4, 4), (1, 0), 2), ((4,), (0,), 4),
                          ((4, 4), (1, 2), 8), ((65536, 65536), (1, 0), 4)]:
        with pytest.raises(ValueError):
            cutt.Candidates(dim, perm, es)


def method_set(cutt, dim, perm, es):
    with cutt.Candidates(dim, perm, es) as c:
        infos = [c.info(i) for i in range(len(c))]
        return infos, infos[c.best]


def test_baseline_configs_have_their_method(cutt):
    # C1/C2: LDS-tiled kernel; C3: Packed; C4: PackedSplit must at least be available.
    infos, best = method_set(cutt, (8192, 8192), (1, 0), 4)
    assert any(i.method_name == "Tiled" for i in infos)
    infos, best = method_set(cutt, (1024, 64, 1024, 3), (2, 1, 0, 3), 8)
    t = [i for i in infos if i.method_name == "Tiled"]
    assert len(t) == 1 and t[0].volMm == 1024 and t[0].volMk == 1024 and t[0].volMbar == 192
    infos, best = method_set(cutt, (5, 7, 11, 13, 17, 1093), (4, 2, 0, 5, 1, 3), 4)
    p = [i for i in infos if i.method_name == "Packed" and i.volMmk == 6545]
    assert p and p[0].volMmkInCont == 385 and p[0].volMmkOutCont == 935 and p[0].volMbar == 14209
    infos, best = method_set(cutt, (200000, 2, 500), (2, 1, 0), 8)
    assert any(i.method_name == "PackedSplit" for i in infos)
    assert any(i.method_name == "Tiled" and i.volMm == 200000 and i.volMk == 500 for i in infos)


def test_plans_are_deterministic(cutt):
    a = method_set(cutt, (31, 549, 2, 3), (3, 0, 2, 1), 8)
    b = method_set(cutt, (31, 549, 2, 3), (3, 0, 2, 1), 8)
    assert [i.as_dict() for i in a[0]] == [i.as_dict() for i in b[0]]


def test_plans_do_not_depend_on_the_number_of_planner_threads(cutt, monkeypatch):
    # The candidates are estimated on several host threads; each estimate is a pure function of
    # its candidate, so the list and the pick are those of the single-threaded planner.
    cases = [((30, 3, 20, 9, 24, 29, 15), (5, 2, 6, 4, 0, 1, 3), 4),
             ((25, 20, 4, 30, 8, 13, 40), (0, 2, 1, 5, 6, 3, 4), 8),
             ((1024, 64, 1024, 3), (2, 1, 0, 3), 8)]
    for dim, perm, es in cases:
        got = []
        for threads in ("1", "3", "8"):
            monkeypatch.setenv("CUTT_PLAN_THREADS", threads)
            infos, best = method_set(cutt, dim, perm, es)
            got.append(([i.as_dict() for i in infos], best.as_dict()))
        assert got[0] == got[1] == got[2]


def test_rows_in_groups_only_for_large_unaligned_tensors_of_4_byte_elements(cutt):
    def tiled(dim, perm, es):
        infos, best = method_set(cutt, dim, perm, es)
        t = [i for i in infos if i.method_name == "Tiled" and i.numMm == 1 and i.numMk == 1]  # one rank per side
        assert len(t) == 1
        return t[0].tiledGrouped
    assert tiled((4457, 44570), (1, 0), 4) == 1          # rows of 17828 bytes, 795 MB
    assert tiled((1535, 157, 895), (2, 1, 0), 4) == 1
    assert tiled((4457, 44570), (1, 0), 8) == 0          # 8-byte elements
    assert tiled((8192, 8192), (1, 0), 4) == 0           # aligned rows
    assert tiled((1536, 157, 896), (2, 1, 0), 4) == 0    # aligned rows
    assert tiled((445, 4457), (1, 0), 4) == 0            # fits the memory-side cache
    assert tiled((31, 97, 101, 659), (3, 1, 2, 0), 4) == 0   # thin tiles: 2 requested lines per line of data


def test_super_tile_shapes_of_the_tiled_plan(cutt):
    def tiled(dim, perm, es):
        infos, best = method_set(cutt, dim, perm, es)
        t = [i for i in infos if i.method_name == "Tiled" and i.numMm == 1 and i.numMk == 1]
        assert len(t) == 1
        return t[0].tiledOrder, t[0].superM, t[0].superK
    # strips of 8 tiles through all of Mk, every strip for all Mbar positions in turn
    assert tiled((4457, 44570), (1, 0), 4) == (3, 8, 697)
    assert tiled((1535, 157, 895), (2, 1, 0), 4) == (5, 8, 14)
    # 8-byte rows on the 128-byte grid: patches; two wide with an Mbar rank between Mm and Mk
    assert tiled((1024, 48, 1024, 4), (2, 1, 0, 3), 8) == (5, 2, 8)
    # ... and with power-of-two strides throughout (C2) the numbering by address bits (order 7)
    assert tiled((1024, 64, 1024, 3), (2, 1, 0, 3), 8) == (7, 1, 1)
    assert tiled((2048, 1024, 95), (1, 0, 2), 8) == (5, 8, 16)      # a batch of separate matrices: strips
    assert tiled((4096, 12, 3936), (2, 1, 0), 8) == (5, 8, 8)       # input rows a multiple of 32 KB
    assert tiled((850, 64, 1024, 3), (2, 1, 0, 3), 4) == (5, 14, 16)    # 4-byte: one strip for a rank of 14 tiles
    assert tiled((1000, 64, 1024, 3), (2, 1, 0, 3), 4) == (5, 8, 16)    # ... two for 16
    assert tiled((1024, 64, 1024, 3), (2, 1, 0, 3), 4) == (7, 1, 1)
    # 4-byte input rows a multiple of 32 KB apart: strips 16 wide, beyond the memory-side cache only
    assert tiled((8192, 8192), (1, 0), 4) == (3, 16, 128)
    assert tiled((16384, 100, 77), (2, 1, 0), 4) == (5, 16, 2)
    assert tiled((8192, 2048), (1, 0), 4) == (3, 8, 32)
    assert tiled((4096, 16384), (1, 0), 4) == (3, 8, 256)
    assert tiled((8192, 8192), (1, 0), 8) == (3, 8, 128)
    # matrices with all rows on the line grid: the tiles along Mk run fastest (order 2) with 17-700 tiles there ...
    assert tiled((45440, 4416), (1, 0), 4)[0] == 2
    assert tiled((10112, 11712, 2), (1, 0, 2), 8)[0] == 2
    assert tiled((45440, 1024), (1, 0), 8)[0] == 3        # ... 16 tiles along Mk: strips
    assert tiled((2816, 51200), (1, 0), 4)[0] == 3        # 800 tiles
    assert tiled((45441, 4416), (1, 0), 4)[0] == 3        # rows off the line grid
    assert tiled((20480, 3392), (1, 0), 8)[0] == 3        # input rows a multiple of 4 KB apart
    assert tiled((8256, 16896), (1, 0), 4)[0] == 3        # ... and within 1 KB of a multiple of 16 KB
    assert tiled((4416, 25856), (1, 0), 4)[0] == 2
    assert tiled((4416, 8, 12928), (2, 1, 0), 4)[0] == 5     # an Mbar rank between Mm and Mk: not this rule
    assert tiled((2240, 2752), (1, 0), 8)[0] == 3         # inside the memory-side cache


def test_every_tile_order_visits_every_tile_once(cutt, oracle_mod, monkeypatch):
    # orders 0-6 of the tiled kernels with several super-tile shapes, replayed on the CPU
    import plan_emulator as pe
    for dim, perm in [((130, 9, 70), (2, 1, 0)), ((200, 3, 5, 33), (3, 1, 2, 0)), ((150, 7, 300), (0, 2, 1)), ((257, 129, 6), (1, 0, 2))]:
        for es in (4, 8):
            data = np.arange(int(np.prod(dim)), dtype=np.uint32 if es == 4 else np.uint64)
            expect = oracle_mod.transpose(list(dim), list(perm), data)
            for order in range(7):
                for sm, sk in ((1, 1), (2, 2), (3, 5), (8, 4096)):
                    monkeypatch.setenv("CUTT_TILED_ORDER", str(order))
                    monkeypatch.setenv("CUTT_SUPER_M", str(sm))
                    monkeypatch.setenv("CUTT_SUPER_K", str(sk))
                    with cutt.Candidates(list(dim), list(perm), es) as c:
                        tiled = [i for i in range(len(c)) if c.info(i).method_name in ("Tiled", "TiledCopy")]
                        assert tiled
                        for i in tiled:
                            assert c.info(i).tiledOrder == order
                            out, count = pe.emulate(c, i, data)
                            assert np.array_equal(out, expect) and (count == 1).all(), (dim, perm, es, order, sm, sk)


def test_random_shapes_every_candidate(cutt, oracle_mod):
    # Seeded random problems of ranks 2-8 with extents that give several tiles, uneven slabs and
    # fused ranks; every candidate of every problem is replayed on the CPU and compared with the
    # oracle, with the device's LDS size and with 8 / 16 KB (which turns Packed plans into splits).
    rng = np.random.default_rng(2024)
    seen = set()
    done = 0
    while done < 250:
        rank = int(rng.integers(2, 9))
        dim = [int(d) for d in np.maximum(2, rng.integers(2, 200, size=rank) // rng.integers(1, 20, size=rank))]
        vol = int(np.prod(dim))
        if vol < 200 or vol > 150000:
            continue
        perm = [int(p) for p in rng.permutation(rank)]
        if rng.random() < 0.3:  # ranks that stay adjacent and fuse
            perm = sorted(perm[: rank // 2]) + perm[rank // 2:]
        if perm == sorted(perm):
            continue
        es = 4 if rng.random() < 0.5 else 8
        lds = int(rng.choice([0, 0, 8192, 16384]))
        seen |= check_all_candidates(cutt, oracle_mod, dim, perm, es, lds=lds)
        done += 1
    assert {"Tiled", "TiledCopy", "Packed", "PackedSplit"} <= seen


def test_tiled_over_fused_rank_sets(cutt, oracle_mod):
    # Mm = the first ranks of the input, Mk = the first ranks of the output, each a contiguous run of
    # its side (the reference's README.md:197-199 lists this as future work).  Every such candidate is
    # replayed against the oracle; the candidate lists must hold tiles over two and three fused ranks.
    sets = set()
    for dim, perm in [((36, 5, 70, 9), (2, 3, 0, 1)),        # Mm = {0, 1}: 180 elements
                      ((7, 9, 11, 70), (3, 1, 0, 2)),         # Mm = {0, 1, 2}: 693
                      ((70, 9, 36, 5), (2, 3, 0, 1)),         # Mk = {2, 3}: 180
                      ((6, 11, 5, 7, 13), (4, 3, 2, 1, 0)),   # both sides: Mm = {0, 1}, Mk = {4, 3}
                      ((3, 5, 7, 4, 9, 11), (5, 4, 3, 1, 0, 2)),
                      ((166, 3, 50, 4), (2, 0, 3, 1))]:       # Mm stops at rank 0: rank 1 is not next to it in Mk's way
        for es in (4, 8):
            check_all_candidates(cutt, oracle_mod, dim, perm, es, need="Tiled")
            with cutt.Candidates(dim, perm, es) as c:
                for i in range(len(c)):
                    info = c.info(i)
                    if info.method_name == "Tiled":
                        sets.add((info.numMm, info.numMk))
                        # the two sets never share a rank
                        assert info.volMm * info.volMk * info.volMbar == int(np.prod(dim))
    assert (2, 1) in sets and (1, 2) in sets and (2, 2) in sets and (3, 1) in sets, sets


def test_fused_tiled_sets_only_where_tiles_would_be_ragged(cutt):
    # a leading rank that is a whole number of tiles is not extended
    infos, best = method_set(cutt, (1024, 64, 1024, 3), (2, 1, 0, 3), 8)
    assert [(i.numMm, i.numMk) for i in infos if i.method_name == "Tiled"] == [(1, 1)]
    infos, best = method_set(cutt, (36, 50, 1000, 111), (2, 0, 3, 1), 8)
    assert {(i.numMm, i.numMk) for i in infos if i.method_name == "Tiled"} >= {(1, 1), (2, 1)}


def test_free_tile_numbering(cutt, oracle_mod, monkeypatch):
    # tile order 7: the workgroup index as a mixed-radix number whose digits are dealt out to the tile
    # along Mm, the tile along Mk and the Mbar position; every tile must be visited exactly once
    cutt.set_method_override(4)  # Tiled only
    try:
        for digits in ["m2,k8,b0,m0,k0", "b4,k2,m0,b0,k0", "k0,m0,b0", "m3,k3,b5,m3,k3,b0,m0,k0", "b0", "m2@2,b2@2,m2@1,k0,b2@1,b0,m0"]:
            monkeypatch.setenv("CUTT_TILE_DIGITS", digits)
            for dim, perm in [((200, 6, 300, 3), (2, 1, 0, 3)), ((70, 130), (1, 0)), ((650, 3, 5, 70), (3, 1, 2, 0))]:
                with cutt.Candidates(dim, perm, 8) as c:
                    orders = [c.info(i).tiledOrder for i in range(len(c)) if c.info(i).method_name == "Tiled"]
                    assert orders and all(o == 7 for o in orders), (digits, dim, orders)
                check_all_candidates(cutt, oracle_mod, dim, perm, 8, need="Tiled")
    finally:
        cutt.set_method_override(0)


def test_digits_one_per_lane_decode_like_digit_by_digit(cutt, monkeypatch):
    """Tile order 7 has two decoders in the kernels: digit by digit, and - where every Mbar digit stays inside one
    Mbar rank - one digit per lane, whose contributions (tile coordinates, offsets of the Mbar position) add up.
    The table the second one reads must give, for every workgroup index, what the first one gives."""
    monkeypatch.setenv("CUTT_DIGIT_LANES", "1")
    cutt.set_method_override(4)
    try:
        cases = [((256, 6, 4, 320), (3, 1, 2, 0), "m2,b2,k0,b3,b4,m0"), ((256, 6, 4, 320), (3, 1, 2, 0), "b6@1,k0,m0,b4@6"),
                 ((128, 8, 192), (2, 1, 0), "k3,b2@4,m0,b4@1"), ((200, 6, 300, 3), (2, 1, 0, 3), "m2,k8,b6,b3,m0,k0"),
                 ((200, 6, 300, 3), (2, 1, 0, 3), "m2,k8,b0,m0,k0")]   # the last one: an Mbar digit over two ranks, no lanes
        with_lanes = 0
        for dim, perm, text in cases:
            monkeypatch.setenv("CUTT_TILE_DIGITS", text)
            with cutt.Candidates(dim, perm, 8) as c:
                i = [k for k in range(len(c)) if c.info(k).method_name == "Tiled" and c.info(k).numMm == 1 and c.info(k).numMk == 1][0]
                assert c.info(i).tiledOrder == 7
                digits = c.data(i, 8).reshape(-1, 3)
                lanes = c.data(i, 9)
                mbar = c.data(i, 0).reshape(-1, 3)
                if text.endswith("b0,m0,k0"):
                    assert lanes[0] == 0
                    continue
                assert lanes[0] == 1 and lanes[1] == int(np.prod(digits[:, 1]))
                with_lanes += 1
                table = lanes[2:].reshape(-1, 5)
                vol_mbar = int(np.prod(mbar[:, 0])) if len(mbar) else 1
                for l in range(int(lanes[1])):
                    rest, coord = l, [0, 0, 0]
                    for which, radix, weight in digits:
                        rest, v = divmod(rest, int(radix))
                        coord[which] += v * int(weight)
                    assert coord[2] < vol_mbar
                    off_in = off_out = 0
                    m = coord[2]
                    for e, si, so in mbar:
                        m, idx = divmod(m, int(e))
                        off_in += idx * int(si)
                        off_out += idx * int(so)
                    got, below = [0, 0, 0, 0], 1
                    for radix, step_m, step_k, si, so in table:
                        v = (l // below) % int(radix)
                        below *= int(radix)
                        got = [got[0] + v * int(step_m), got[1] + v * int(step_k), got[2] + v * int(si), got[3] + v * int(so)]
                    assert got == [coord[0], coord[1], off_in, off_out], (text, l)
        assert with_lanes == 4
    finally:
        cutt.set_method_override(0)


def test_free_item_numbering(cutt, oracle_mod, monkeypatch):
    # the packed kernel's work items numbered by digits: the item number as a mixed-radix number whose digits are
    # dealt out to the slab of the first cut rank (m), of the second (k) and the Mbar position (b).  A text applies
    # to the candidates whose slabs are of one size and whose extents its radices multiply to; the others keep
    # their numbering.  Every element exactly once.
    dim, perm = (24, 10, 18, 6), (2, 0, 3, 1)
    for digits in ["b2,b3,m0,k0,b0", "m0,k0,b0", "b0,k0,m0", "b3@2,m0,b2@1,k0,b0", "k2,b0,m2,k0,m0"]:
        monkeypatch.setenv("CUTT_ITEM_DIGITS", digits)
        with cutt.Candidates(dim, perm, 4, lds_per_block=2048) as c:
            numbered = [i for i in range(len(c)) if c.info(i).method_name in ("Packed", "PackedSplit") and c.info(i).tileDigits]
            assert len(numbered) >= 2, (digits, len(numbered))
            for i in numbered:   # the launch arguments hold one table entry per digit and no slab counts
                sc = c.data(i, 2)
                assert sc[8] == 1 and sc[13] == 1 and sc[1] == c.info(i).volMbar * c.info(i).numSplit * c.info(i).numSplit2
                d = c.data(i, 8)
                assert len(c.data(i, 0)) == len(d)
        check_all_candidates(cutt, oracle_mod, dim, perm, 4, need="PackedSplit", lds=2048)
    # radices that do not multiply to a coordinate's extent, digits of one weight, a digit across two Mbar ranks: ignored
    for digits in ["b7,m0,k0,b0", "b2@1,b3@1,m0,k0", "b4,b0,m0,k0"]:
        monkeypatch.setenv("CUTT_ITEM_DIGITS", digits)
        with cutt.Candidates(dim, perm, 4, lds_per_block=2048) as c:
            assert all(not c.info(i).tileDigits for i in range(len(c)) if c.info(i).volMbar in (6, 10)), digits


def test_packed_items_keep_address_bit_11_moving(cutt, monkeypatch):
    """Packed plans on power-of-two addresses: a binary digit of the item number that moves the read or the written
    address by 2 KB (bit 11) and would sit between the digits the resident workgroups differ in and the three
    slowest ones is taken out of its rank and made the slowest digit."""
    dim, perm, es = (2, 4096, 256, 64), (0, 3, 1, 2), 4
    def packed(c):
        return [i for i in range(len(c)) if c.info(i).method_name in ("Packed", "PackedSplit")]
    with cutt.Candidates(dim, perm, es) as c:
        moved = [i for i in packed(c) if c.info(i).tileDigits]
        assert moved
        for i in moved:
            info = c.info(i)
            d = c.data(i, 8).reshape(-1, 3)          # coordinate, radix, weight
            assert d[-1][1] == 2                      # the slowest digit is a binary one ...
            # ... and per coordinate the radices still multiply to the extent
            ext = [info.numSplit, info.numSplit2, info.volMbar]
            for w in range(3):
                assert int(np.prod(d[d[:, 0] == w][:, 1])) == ext[w], (i, d)
            sc = c.data(i, 2)
            assert sc[8] == 1 and sc[13] == 1 and sc[1] == ext[0] * ext[1] * ext[2]
        i = [k for k in moved if c.info(k).numSplit == 256 and c.info(k).numSplit2 == 128][0]
        # slabs of the second cut rank are 32 elements = 128 bytes apart on the read side: its digit 8 moves bit 11
        assert c.info(i).tileDigits.decode() == "m256@1,k8@1,k8@16,k2@8"
    # tensors inside the memory-side cache, extents that are no powers of two, the rule switched off: default numbering
    for d2, p2 in [((2, 512, 64, 64), (0, 3, 1, 2)), ((2, 4095, 256, 64), (0, 3, 1, 2))]:
        with cutt.Candidates(d2, p2, es) as c:
            assert not [i for i in packed(c) if c.info(i).tileDigits], d2
    monkeypatch.setenv("CUTT_ADDRESS_BITS", "0")
    with cutt.Candidates(dim, perm, es) as c:
        assert not [i for i in packed(c) if c.info(i).tileDigits]


def test_numbering_by_address_bits(cutt, monkeypatch):
    """Batched transposes on power-of-two addresses: the digits of the workgroup number that move address bit 11
    (on either side) are the three slowest (split over the XCDs), tile digits that move 1 KB / 4 KB and digits
    that move 128 KB come right below them, the 2 x 2 patch and the Mbar digits are fastest."""
    def digits(dim, perm, es):
        with cutt.Candidates(dim, perm, es) as c:
            t = [i for i in range(len(c)) if c.info(i).method_name == "Tiled" and c.info(i).numMm == 1 and c.info(i).numMk == 1]
            assert len(t) == 1
            d = c.data(t[0], 8)
            return c.info(t[0]).tiledOrder, ["%s%d@%d" % ("mkb"[d[3 * k]], d[3 * k + 1], d[3 * k + 2]) for k in range(len(d) // 3)]
    order, dg = digits((1024, 64, 1024, 3), (2, 1, 0, 3), 8)
    # tile digit 4 (the third binary digit) moves 2 KB = address bit 11 in rows of 8-byte elements
    assert order == 7 and sorted(dg[-3:]) == ["k2@4", "m2@2", "m2@4"], dg
    assert dg[:2] == ["m2@1", "k2@1"] and dg[2:6] == ["b2@1", "b2@2", "b2@4", "b2@8"], dg
    assert dg[-4] == "b3@64", dg                        # the odd factor of the Mbar extent right below the top
    assert set(dg[7:11]) == {"b2@16", "k2@2", "m2@8", "k2@8"}, dg   # 128 KB, 1 KB, 4 KB, 4 KB
    order, dg = digits((2048, 64, 1024, 3), (2, 1, 0, 3), 4)
    # 4-byte elements: a tile row is 256 bytes, so the fourth binary digit moves address bit 11
    assert order == 7 and {"m2@8", "k2@8"} <= set(dg[-3:]), dg
    # not of this class: a batch of separate matrices, extents that are no powers of two, 128 tiles along Mk,
    # a tensor inside the memory-side cache, a plain 2-D transpose
    for dim, perm, es in [((1024, 1024, 192), (1, 0, 2), 8), ((1024, 48, 1024, 4), (2, 1, 0, 3), 8), ((256, 32, 8192, 3), (2, 1, 0, 3), 8),
                          ((256, 16, 256, 3), (2, 1, 0, 3), 8), ((8192, 8192), (1, 0), 4)]:
        assert digits(dim, perm, es)[0] != 7, (dim, perm)
    monkeypatch.setenv("CUTT_ADDRESS_BITS", "0")
    assert digits((1024, 64, 1024, 3), (2, 1, 0, 3), 8)[0] == 5
