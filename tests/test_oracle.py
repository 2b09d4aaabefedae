"""Pins the CPU oracle (oracle/transpose_oracle.c) against independent facts.

The oracle's own formula is never retyped here: every expected value comes
from numpy's transpose (an independent library routine), from a result worked
by hand, or from an invariant of permutations.
"""
import itertools

import numpy as np
import pytest


def np_transpose(dim, perm, data):
    """dim[0] fastest == Fortran order; output dimension j is input dimension perm[j]."""
    a = data.reshape(tuple(dim), order="F")
    return np.ascontiguousarray(np.transpose(a, perm).ravel(order="F"))


def test_readme_shape_example(oracle_mod):
    # reference README.md:95-97: dims (31,549,2,3), permutation (3,0,2,1) -> (3,31,2,549)
    dim, perm = (31, 549, 2, 3), (3, 0, 2, 1)
    data = np.arange(np.prod(dim), dtype=np.int64)
    out = oracle_mod.transpose(dim, perm, data)
    o = out.reshape((3, 31, 2, 549), order="F")
    a = data.reshape(dim, order="F")
    # output index (i3, i0, i2, i1) holds input (i0, i1, i2, i3)
    for (i0, i1, i2, i3) in [(0, 0, 0, 0), (30, 548, 1, 2), (7, 100, 1, 0), (1, 2, 0, 1)]:
        assert o[i3, i0, i2, i1] == a[i0, i1, i2, i3]


def test_hand_worked_2x3(oracle_mod):
    # input 2x3 (dim0=2 fastest): memory [a00 a10 a01 a11 a02 a12] = [0 1 2 3 4 5]
    # transposed 3x2 (dim0=3 fastest): [a00 a01 a02 a10 a11 a12] = [0 2 4 1 3 5]
    out = oracle_mod.transpose((2, 3), (1, 0), np.arange(6, dtype=np.int32))
    assert out.tolist() == [0, 2, 4, 1, 3, 5]


def test_hand_worked_2x3x4(oracle_mod):
    # perm (2,0,1): output dims (4,2,3); out[k + 4*i + 8*j] = in[i + 2*j + 6*k]
    data = np.arange(24, dtype=np.int64) * 10
    out = oracle_mod.transpose((2, 3, 4), (2, 0, 1), data)
    expect = np.empty(24, dtype=np.int64)
    for i in range(2):
        for j in range(3):
            for k in range(4):
                expect[k + 4 * i + 8 * j] = data[i + 2 * j + 6 * k]
    assert np.array_equal(out, expect)


@pytest.mark.parametrize("rank", [2, 3, 4, 5])
def test_against_numpy_all_permutations(oracle_mod, rank):
    dim = [3, 4, 2, 5, 3][:rank]
    rng = np.random.default_rng(rank)
    for dtype in (np.uint32, np.uint64):
        data = rng.integers(0, 2 ** 32, size=int(np.prod(dim)), dtype=np.uint64).astype(dtype)
        for perm in itertools.permutations(range(rank)):
            assert np.array_equal(oracle_mod.transpose(dim, perm, data), np_transpose(dim, perm, data))


def test_against_numpy_random_shapes(oracle_mod):
    rng = np.random.default_rng(7)
    for _ in range(40):
        rank = int(rng.integers(2, 8))
        dim = [int(d) for d in rng.integers(2, 9, size=rank)]
        perm = [int(p) for p in rng.permutation(rank)]
        data = rng.integers(0, 2 ** 63, size=int(np.prod(dim)), dtype=np.uint64)
        assert np.array_equal(oracle_mod.transpose(dim, perm, data), np_transpose(dim, perm, data))


def test_identity_is_copy_and_inverse_roundtrip(oracle_mod):
    rng = np.random.default_rng(3)
    dim = (5, 3, 7, 2, 4)
    data = rng.integers(0, 2 ** 32, size=int(np.prod(dim)), dtype=np.uint32)
    assert np.array_equal(oracle_mod.transpose(dim, range(5), data), data)
    for _ in range(10):
        perm = [int(p) for p in rng.permutation(5)]
        out = oracle_mod.transpose(dim, perm, data)
        odim = [dim[p] for p in perm]
        inv = [perm.index(r) for r in range(5)]
        assert np.array_equal(oracle_mod.transpose(odim, inv, out), data)
        # a transpose is a permutation of the multiset of values
        assert np.array_equal(np.sort(out), np.sort(data))


def test_rank2_is_matrix_transpose(oracle_mod):
    rng = np.random.default_rng(5)
    data = rng.integers(0, 2 ** 63, size=43 * 67, dtype=np.uint64)
    out = oracle_mod.transpose((43, 67), (1, 0), data)
    m = data.reshape(67, 43)  # row-major view: 67 rows of 43 (dim0 fastest)
    assert np.array_equal(out.reshape(43, 67), m.T)


def test_bit_patterns_survive(oracle_mod):
    # NaN payloads, denormals, negative zero: the oracle moves bytes, not numbers
    words = np.array([0x7FC00001, 0xFFC12345, 0x00000001, 0x80000000, 0x7F800000, 0x3F800000], dtype=np.uint32)
    out = oracle_mod.transpose((2, 3), (1, 0), words.view(np.float32))
    assert out.view(np.uint32).tolist() == [int(words[i]) for i in (0, 2, 4, 1, 3, 5)]


@pytest.mark.parametrize("nthreads", [1, 3, 8])
def test_multithreaded_equals_single(oracle_mod, nthreads):
    rng = np.random.default_rng(11)
    cases = [((43, 67), (1, 0)), ((70, 3, 50), (2, 1, 0)), ((33, 5, 9, 40), (3, 1, 0, 2)),
             ((6, 50, 7), (0, 2, 1)), ((5, 7, 11, 3, 4), (4, 2, 0, 3, 1)), ((130, 2), (1, 0))]
    for dim, perm in cases:
        for dtype in (np.uint32, np.uint64):
            data = rng.integers(0, 2 ** 32, size=int(np.prod(dim)), dtype=np.uint64).astype(dtype)
            assert np.array_equal(oracle_mod.transpose_mt(dim, perm, data, nthreads),
                                  oracle_mod.transpose(dim, perm, data))


# reduceRanks: cases that can be derived by hand from reference src/cutt_test.cpp:245-366
REDUCE_CASES = [
    ((43, 67), (1, 0), [43, 67], [1, 0]),
    ((1305, 599, 88), (0, 2, 1), [1305, 599, 88], [0, 2, 1]),
    ((24, 330, 64, 147), (1, 0, 2, 3), [24, 330, 64 * 147], [1, 0, 2]),
    ((2, 5, 9, 12), (0, 1, 2, 3), [2 * 5 * 9 * 12], [0]),
    ((2, 4, 6, 9, 11, 13), (0, 1, 2, 3, 4, 5), [2 * 4 * 6 * 9 * 11 * 13], [0]),
    ((5, 42, 75, 86, 57), (1, 3, 4, 2, 0), [5, 42, 75, 86 * 57], [1, 3, 2, 0]),
    ((5, 3, 2, 9, 14), (0, 1, 3, 2, 4), [15, 2, 9, 14], [0, 2, 1, 3]),
]


@pytest.mark.parametrize("dim,perm,rdim,rperm", REDUCE_CASES)
def test_reduce_ranks_hand_cases(oracle_mod, dim, perm, rdim, rperm):
    assert oracle_mod.reduce_ranks(dim, perm) == (rdim, rperm)


def test_reduce_ranks_keeps_the_bytes(oracle_mod):
    rng = np.random.default_rng(13)
    for _ in range(60):
        rank = int(rng.integers(2, 7))
        dim = [int(d) for d in rng.integers(2, 6, size=rank)]
        perm = [int(p) for p in rng.permutation(rank)]
        rdim, rperm = oracle_mod.reduce_ranks(dim, perm)
        assert int(np.prod(rdim)) == int(np.prod(dim))
        assert sorted(rperm) == list(range(len(rdim)))
        # no two adjacent output ranks of the fused problem are consecutive input ranks
        assert all(rperm[i] != rperm[i - 1] + 1 for i in range(1, len(rperm)))
        data = rng.integers(0, 2 ** 63, size=int(np.prod(dim)), dtype=np.uint64)
        assert np.array_equal(np_transpose(rdim, rperm, data), np_transpose(dim, perm, data))


def test_pattern_check_agrees_with_transpose(oracle_mod):
    rng = np.random.default_rng(17)
    for es, dtype in ((4, np.uint32), (8, np.uint64)):
        for _ in range(10):
            rank = int(rng.integers(2, 6))
            dim = [int(d) for d in rng.integers(2, 8, size=rank)]
            perm = [int(p) for p in rng.permutation(rank)]
            vol = int(np.prod(dim))
            words = oracle_mod.fill_pattern(vol * es // 4)
            assert words[:4].tolist() == [0, 1, 2, 3]
            out = np_transpose(dim, perm, words.view(dtype))
            assert oracle_mod.check_pattern(dim, perm, es, out) == -1
            if any(p != i for i, p in enumerate(perm)):
                bad = out.copy()
                bad[vol // 2] ^= 1
                assert oracle_mod.check_pattern(dim, perm, es, bad) == vol // 2
