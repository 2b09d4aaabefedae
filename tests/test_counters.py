"""Known-answer tests of the cost model's counters (counterpart of the reference's test5,
src/cutt_test.cpp:410-431 -> testCounters, src/cuttGpuModel.cpp:901-1348).

The expected values are the reference's own golden tables (tests/golden/counter_goldens.json, made
by tests/golden/make_counter_goldens.py).  They pin the counter definitions for the reference's
widths (32 lanes; 128-byte transactions, 32-byte sectors); the model uses the same functions with
the gfx950 widths, for which closed forms and brute force are checked below.
"""
import ctypes
import json
import os

import numpy as np
import pytest

HERE = os.path.dirname(os.path.abspath(__file__))


@pytest.fixture(scope="module")
def gold():
    return json.load(open(os.path.join(HERE, "golden", "counter_goldens.json")))


@pytest.fixture(scope="module")
def lib(cutt):
    return cutt.lib()


def ints(v):
    return (ctypes.c_int * len(v))(*[int(x) for x in v])


def seg_counts(lib, positions, acc_width, cache_width):
    n = len(positions)
    tran = lib.cuttModelGlTransactionsSeg(ints([p // acc_width for p in positions]), n)
    full, part = ctypes.c_int(), ctypes.c_int()
    lib.cuttModelCacheLinesSeg(ints([p // cache_width for p in positions]), n, cache_width,
                               ctypes.byref(full), ctypes.byref(part))
    return [tran, full.value, part.value]


def cont_counts(lib, pos, n, acc_width, cache_width):
    tran = lib.cuttModelGlTransactionsCont(pos, n, acc_width)
    full, part = ctypes.c_int(), ctypes.c_int()
    lib.cuttModelCacheLinesCont(pos, n, cache_width, ctypes.byref(full), ctypes.byref(part))
    return [tran, full.value, part.value]


@pytest.mark.parametrize("key,acc,cache", [("arrayResultsDouble", 16, 4), ("arrayResultsFloat", 32, 8)])
def test_scattered_access_goldens(lib, gold, key, acc, cache):
    for i, row in enumerate(gold["posData"]):
        positions = [p for p in row if p != -1]
        assert seg_counts(lib, positions, acc, cache) == gold[key][3 * i:3 * i + 3], (i, positions)


@pytest.mark.parametrize("key,acc,cache", [("contResultsDouble", 16, 4), ("contResultsFloat", 32, 8)])
def test_contiguous_access_goldens(lib, gold, key, acc, cache):
    i = 0
    for pos in range(acc):
        for n in range(33):
            want = gold[key][3 * i:3 * i + 3]
            assert cont_counts(lib, pos, n, acc, cache) == want, (pos, n)
            # the scattered-access counters must agree with the closed form on contiguous input
            assert seg_counts(lib, list(range(pos, pos + n)), acc, cache) == want, (pos, n)
            i += 1


def test_contiguous_equals_scattered_for_gfx950_widths(lib):
    # 64 lanes; 128-byte lines of 4- and 8-byte elements (32 / 16 per line), 32-byte sectors (8 / 4)
    for acc, cache in ((32, 8), (16, 4), (32, 32), (16, 16)):
        for pos in range(0, 2 * acc, 3):
            for n in range(0, 65):
                assert cont_counts(lib, pos, n, acc, cache) == seg_counts(lib, list(range(pos, pos + n)), acc, cache)


def test_counters_brute_force(lib):
    rng = np.random.default_rng(0)
    for _ in range(200):
        n = int(rng.integers(1, 65))
        positions = sorted(set(int(p) for p in rng.integers(0, 400, size=n)))
        acc, cache = (16, 4) if rng.random() < 0.5 else (32, 8)
        tran = len(set(p // acc for p in positions))
        lines = {}
        for p in positions:
            lines.setdefault(p // cache, 0)
            lines[p // cache] += 1
        full = sum(1 for v in lines.values() if v == cache)
        part = len(lines) - full
        assert seg_counts(lib, positions, acc, cache) == [tran, full, part]


def sh_transactions(lib, wave, banks, nthread, vol, msh):
    flat = [x for t in msh for x in t]
    out = (ctypes.c_int * 4)()
    lib.cuttModelShTransactions(wave, banks, nthread, vol, ints(flat), len(msh), out)
    return list(out)


def sh_reference(wave, banks, nthread, vol, msh):
    """Brute force: conflict degree of every wavefront-sized request."""
    ld = st = req = 0
    for b0 in range(0, vol, nthread):
        for w0 in range(b0, min(vol, b0 + nthread), wave):
            cnt = {}
            for j in range(w0, min(w0 + wave, vol)):
                pos = sum(((j // c) % d) * ct for c, d, ct in msh)
                cnt[pos % banks] = cnt.get(pos % banks, 0) + 1
            ld += max(cnt.values())
            st += 1
            req += 1
    return [ld, st, req, req]


def test_shared_memory_transactions_on_reference_tables(lib, gold):
    # the reference's 31 recorded (numthread, volMmk, Msh table) cases, src/cuttGpuModel.cpp:1080-1100
    data = gold["shTestData"]
    triples = [data[3 * i:3 * i + 3] for i in range(len(data) // 3)]
    i = cases = 0
    while i < len(triples):
        nthread, vol, nmsh = triples[i]
        msh = triples[i + 1:i + 1 + nmsh]
        i += 1 + nmsh
        for wave, banks in ((32, 32), (64, 64), (64, 32)):
            assert sh_transactions(lib, wave, banks, nthread, vol, msh) == sh_reference(wave, banks, nthread, vol, msh)
        cases += 1
    assert cases == 31 and i == len(triples)
