"""CPU oracle for the transpose path: TEST INFRASTRUCTURE ONLY.

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import
this package; the shipped library (cutt_amd) never does.  It wraps the C
restatement in transpose_oracle.c (see that file's header for the reference
lines it follows and for how each function is pinned).
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle.so")
_lib = None


def build():
    """Compile liboracle.so with the committed Makefile."""
    subprocess.check_call(["make", "-s", "-C", _HERE, "liboracle.so"])


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        l = ctypes.CDLL(_LIB_PATH)
        ip = ctypes.POINTER(ctypes.c_int)
        l.oracle_transpose.argtypes = [ctypes.c_int, ip, ip, ctypes.c_size_t, ctypes.c_void_p, ctypes.c_void_p]
        l.oracle_transpose.restype = ctypes.c_int
        l.oracle_transpose_mt.argtypes = [ctypes.c_int, ip, ip, ctypes.c_size_t, ctypes.c_void_p,
                                          ctypes.c_void_p, ctypes.c_int]
        l.oracle_transpose_mt.restype = ctypes.c_int
        l.oracle_reduce_ranks.argtypes = [ctypes.c_int, ip, ip, ip, ip]
        l.oracle_reduce_ranks.restype = ctypes.c_int
        l.oracle_fill_pattern.argtypes = [ctypes.c_void_p, ctypes.c_size_t]
        l.oracle_fill_pattern.restype = None
        l.oracle_check_pattern.argtypes = [ctypes.c_int, ip, ip, ctypes.c_size_t, ctypes.c_void_p]
        l.oracle_check_pattern.restype = ctypes.c_int64
        _lib = l
    return _lib


def _ints(v):
    return (ctypes.c_int * len(v))(*[int(x) for x in v])


def _check(dim, perm, data):
    if sorted(perm) != list(range(len(dim))):
        raise ValueError("perm is not a permutation")
    vol = int(np.prod([int(d) for d in dim], dtype=object))
    if data.ndim != 1 or data.size != vol:
        raise ValueError("data must be a flat array of prod(dim) elements")
    if not data.flags.c_contiguous:
        raise ValueError("data must be contiguous")


def transpose(dim, perm, data):
    """Index-loop transpose of a flat array (dim[0] fastest); returns a new flat array."""
    data = np.ascontiguousarray(data)
    _check(dim, perm, data)
    out = np.empty_like(data)
    rc = lib().oracle_transpose(len(dim), _ints(dim), _ints(perm), data.itemsize,
                                data.ctypes.data, out.ctypes.data)
    if rc != 0:
        raise RuntimeError("oracle_transpose failed: %d" % rc)
    return out


def transpose_mt(dim, perm, data, nthreads, out=None):
    """Multithreaded CPU transpose (the reported CPU baseline)."""
    data = np.ascontiguousarray(data)
    _check(dim, perm, data)
    if out is None:
        out = np.empty_like(data)
    rc = lib().oracle_transpose_mt(len(dim), _ints(dim), _ints(perm), data.itemsize,
                                   data.ctypes.data, out.ctypes.data, int(nthreads))
    if rc != 0:
        raise RuntimeError("oracle_transpose_mt failed: %d" % rc)
    return out


def reduce_ranks(dim, perm):
    n = len(dim)
    rd = (ctypes.c_int * n)()
    rp = (ctypes.c_int * n)()
    k = lib().oracle_reduce_ranks(n, _ints(dim), _ints(perm), rd, rp)
    return list(rd[:k]), list(rp[:k])


def fill_pattern(nwords):
    """uint32 array with words[i] = i (the reference tester's input pattern)."""
    a = np.empty(nwords, dtype=np.uint32)
    lib().oracle_fill_pattern(a.ctypes.data, nwords)
    return a


def check_pattern(dim, perm, elem_size, out):
    """-1 if `out` is the transpose of the pattern input, else the first bad output position."""
    out = np.ascontiguousarray(out)
    return int(lib().oracle_check_pattern(len(dim), _ints(dim), _ints(perm), elem_size, out.ctypes.data))
