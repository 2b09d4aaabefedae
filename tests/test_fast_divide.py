"""The multiply-high divisions the kernels use to decode work items and Mbar positions.

The library derives (mul, shift, add) on the host; the kernels evaluate
(mulhi32(n, mul) + n*add) >> shift.  Here the constants are checked against
integer division for every divisor class that can break such a scheme
(1, 2, powers of two and their neighbours, primes, divisors near 2^31) at the
numerators where a wrong rounding shows first (multiples of d and their
predecessors, the largest 31-bit number).
"""
import ctypes
import random

import pytest

import cutt_amd


class Divisor(ctypes.Structure):
    _fields_ = [("mul", ctypes.c_uint32), ("shift", ctypes.c_uint32), ("add", ctypes.c_uint32)]


class MbarDim(ctypes.Structure):
    _fields_ = [(n, ctypes.c_uint32) for n in ("extent", "strideIn", "strideOut", "belowMul", "extentMul", "ctl")]


class Mbar(ctypes.Structure):
    _fields_ = [("n", ctypes.c_int), ("d", MbarDim * 32)]


@pytest.fixture(scope="module")
def lib():
    l = ctypes.CDLL(cutt_amd.lib_path())
    l.cuttHipMakeDivisor.restype = Divisor
    l.cuttHipMakeDivisor.argtypes = [ctypes.c_uint32]
    l.cuttHipDivide.restype = ctypes.c_uint32
    l.cuttHipDivide.argtypes = [ctypes.c_uint32, Divisor]
    l.cuttHipFinishMbar.restype = ctypes.c_int
    l.cuttHipFinishMbar.argtypes = [ctypes.POINTER(Mbar)]
    return l


def device_formula(n, mul, shift, add):
    """What the kernel computes, in 32-bit arithmetic."""
    hi = (n * mul) >> 32
    return ((hi + n * add) & 0xFFFFFFFF) >> shift


def numerators(d, rng):
    top = 2**31 - 1
    ns = {0, 1, d - 1, d, d + 1, top, top - 1, top // 2}
    for k in (1, 2, 3, 7, top // d, top // d - 1, rng.randrange(1, max(2, top // d))):
        if k >= 1:
            ns.update({k * d - 1, k * d, k * d + 1})
    ns.update(rng.randrange(0, top + 1) for _ in range(40))
    return [n for n in ns if 0 <= n <= top]


def test_divisor_constants_are_exact(lib):
    rng = random.Random(11)
    ds = {1, 2, 3, 5, 6, 7, 10, 11, 12, 13, 96, 641, 65537, 2**31 - 1, 2**31 - 2, 2**30 + 1, 2**30 - 1, 1000003}
    for k in range(1, 31):
        ds.update({2**k - 1, 2**k, 2**k + 1})
    ds.update(rng.randrange(1, 2**31) for _ in range(300))
    ds.update(rng.randrange(1, 5000) for _ in range(300))
    for d in sorted(x for x in ds if 1 <= x < 2**31):
        dv = lib.cuttHipMakeDivisor(d)
        assert dv.mul < 2**32 and dv.shift < 32 and dv.add in (0, 1)
        for n in numerators(d, rng):
            want = n // d
            assert device_formula(n, dv.mul, dv.shift, dv.add) == want, (n, d)
            assert lib.cuttHipDivide(n, dv) == want, (n, d)


def test_small_divisors_exhaustive_over_a_range(lib):
    for d in range(1, 70):
        dv = lib.cuttHipMakeDivisor(d)
        for n in list(range(0, 5000)) + list(range(2**31 - 5000, 2**31)):
            assert device_formula(n, dv.mul, dv.shift, dv.add) == n // d


def test_mbar_table_decodes_like_nested_loops(lib):
    rng = random.Random(5)
    for case in range(200):
        n = rng.randrange(0, 33)
        mb = Mbar()
        mb.n = n
        vol = 1
        for k in range(n):
            e = rng.choice([2, 3, 4, 5, 7, 16, 33, 100, 1093])
            if vol * e >= 2**31:
                e = 1
            mb.d[k].extent = e
            mb.d[k].strideIn = rng.randrange(0, 2**20)
            mb.d[k].strideOut = rng.randrange(0, 2**20)
            vol *= e
        assert lib.cuttHipFinishMbar(ctypes.byref(mb)) == 0
        for m in [0, vol - 1, vol // 2] + [rng.randrange(0, vol) for _ in range(20)]:
            # nested loops: rank 0 of the table runs fastest
            rest, want_in, want_out = m, 0, 0
            for k in range(n):
                e = mb.d[k].extent
                want_in += (rest % e) * mb.d[k].strideIn
                want_out += (rest % e) * mb.d[k].strideOut
                rest //= e
            # what the lanes compute: lane k takes (m / below) % extent with the table's constants
            got_in = got_out = 0
            for k in range(32):
                d = mb.d[k]
                q = device_formula(m, d.belowMul, d.ctl & 0xFF, (d.ctl >> 16) & 1)
                q2 = device_formula(q, d.extentMul, (d.ctl >> 8) & 0xFF, (d.ctl >> 17) & 1)
                idx = q - q2 * d.extent
                if k < n:
                    got_in += idx * d.strideIn
                    got_out += idx * d.strideOut
                else:
                    assert idx == 0
            assert (got_in, got_out) == (want_in, want_out), (case, m)


def test_mbar_table_rejects_oversized_products(lib):
    mb = Mbar()
    mb.n = 2
    mb.d[0].extent = 2**16
    mb.d[1].extent = 2**15
    assert lib.cuttHipFinishMbar(ctypes.byref(mb)) != 0
    mb.d[1].extent = 2**15 - 1
    assert lib.cuttHipFinishMbar(ctypes.byref(mb)) == 0
    mb.d[1].extent = 0
    assert lib.cuttHipFinishMbar(ctypes.byref(mb)) != 0
