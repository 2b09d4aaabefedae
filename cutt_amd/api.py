"""ctypes binding of libcutt.so: the four plan functions of include/cutt.h and
the hooks of include/cutt_ext.h, with the same names and argument order.

Device buffers are passed as integer addresses (e.g. ``tensor.data_ptr()``),
streams as integer ``hipStream_t`` values (e.g.
``torch.cuda.current_stream().cuda_stream``).  There is no CPU fallback: if
the library is missing the import of :func:`lib` fails.
"""
import ctypes
import os

import numpy as np

CUTT_SUCCESS = 0
CUTT_INVALID_PLAN = 1
CUTT_INVALID_PARAMETER = 2
CUTT_INVALID_DEVICE = 3
CUTT_INTERNAL_ERROR = 4
CUTT_UNDEFINED_ERROR = 5
_RESULT_NAMES = ["CUTT_SUCCESS", "CUTT_INVALID_PLAN", "CUTT_INVALID_PARAMETER", "CUTT_INVALID_DEVICE",
                 "CUTT_INTERNAL_ERROR", "CUTT_UNDEFINED_ERROR"]

METHOD_TRIVIAL, METHOD_PACKED, METHOD_PACKEDSPLIT, METHOD_TILED, METHOD_TILEDCOPY = 1, 2, 3, 4, 5
METHOD_NAMES = {0: "Unknown", 1: "Trivial", 2: "Packed", 3: "PackedSplit", 4: "Tiled", 5: "TiledCopy"}


class CuttError(RuntimeError):
    def __init__(self, code, what):
        name = _RESULT_NAMES[code] if 0 <= code < len(_RESULT_NAMES) else str(code)
        super().__init__("%s returned %s" % (what, name))
        self.code = code


class PlanInfo(ctypes.Structure):
    """Mirror of struct cuttPlanInfo (include/cutt_ext.h)."""
    _fields_ = [
        ("method", ctypes.c_int), ("fromReduced", ctypes.c_int), ("rank", ctypes.c_int),
        ("numMm", ctypes.c_int), ("numMk", ctypes.c_int),
        ("splitRank", ctypes.c_int), ("splitDim", ctypes.c_int), ("numSplit", ctypes.c_int),
        ("splitRank2", ctypes.c_int), ("splitDim2", ctypes.c_int), ("numSplit2", ctypes.c_int),
        ("volMm", ctypes.c_longlong), ("volMk", ctypes.c_longlong), ("volMmk", ctypes.c_longlong),
        ("volMbar", ctypes.c_longlong), ("volMmkInCont", ctypes.c_longlong),
        ("volMmkOutCont", ctypes.c_longlong), ("volMmkUnsplit", ctypes.c_longlong),
        ("numBlocks", ctypes.c_longlong), ("numThreads", ctypes.c_int), ("itemsPerBlock", ctypes.c_int),
        ("tiledOrder", ctypes.c_int), ("ldsBytes", ctypes.c_ulonglong),
        ("usPredicted", ctypes.c_double),
        ("rdLines", ctypes.c_double), ("wrLines", ctypes.c_double), ("rdInstr", ctypes.c_double),
        ("wrInstr", ctypes.c_double), ("wrPartialLines", ctypes.c_double), ("rdSectors", ctypes.c_double),
        ("wrSectors", ctypes.c_double), ("ldsCycles", ctypes.c_double), ("blocksPerCU", ctypes.c_double),
        ("usMeasured", ctypes.c_double),
        ("numCandidates", ctypes.c_int), ("planMs", ctypes.c_double),
        ("cachePolicy", ctypes.c_int), ("elemsPerThread", ctypes.c_int),
        ("rdEdgeDist", ctypes.c_double), ("wrEdgeDist", ctypes.c_double),
        ("tiledGrouped", ctypes.c_int), ("superM", ctypes.c_int), ("superK", ctypes.c_int),
        ("tiledAligned", ctypes.c_int), ("itemOrder", ctypes.c_int),
        ("numPieces", ctypes.c_int), ("numShapes", ctypes.c_int), ("wideOffsets", ctypes.c_int),
        ("tileDigits", ctypes.c_char * 192),
    ]

    @property
    def method_name(self):
        return METHOD_NAMES.get(self.method, "?")

    def as_dict(self):
        d = {name: getattr(self, name) for name, _ in self._fields_}
        d["tileDigits"] = self.tileDigits.decode()
        d["method_name"] = self.method_name
        return d


class StreamCounts(ctypes.Structure):
    """Mirror of struct cuttStreamCounts (include/cutt_ext.h)."""
    _fields_ = [(n, ctypes.c_double) for n in ("rdInstr", "wrInstr", "rdInstrIdle", "wrInstrIdle", "rdLines", "wrLines",
                                               "rdSectors", "wrSectors", "wrPartialLines", "ldsCycles")] + \
               [("ldsMaxDegree", ctypes.c_int)]

    def as_dict(self):
        return {name: getattr(self, name) for name, _ in self._fields_}


_HERE = os.path.dirname(os.path.abspath(__file__))
_lib = None


def lib_path():
    """The in-tree build; CUTT_AMD_LIB names another build of the same library (experiments)."""
    return os.environ.get("CUTT_AMD_LIB") or os.path.join(_HERE, "libcutt.so")


def lib():
    """Load libcutt.so (built in-tree by cutt_amd.build.build())."""
    global _lib
    if _lib is not None:
        return _lib
    path = lib_path()
    if not os.path.exists(path):
        raise ImportError("%s not found: build it with `python -c 'import cutt_amd; cutt_amd.build()'`" % path)
    l = ctypes.CDLL(path)
    ip = ctypes.POINTER(ctypes.c_int)
    hp = ctypes.POINTER(ctypes.c_uint)
    vp = ctypes.c_void_p
    l.cuttPlan.argtypes = [hp, ctypes.c_int, ip, ip, ctypes.c_size_t, vp]
    l.cuttPlan.restype = ctypes.c_int
    l.cuttPlanMeasure.argtypes = [hp, ctypes.c_int, ip, ip, ctypes.c_size_t, vp, vp, vp]
    l.cuttPlanMeasure.restype = ctypes.c_int
    l.cuttPlanFromCandidate.argtypes = [hp, ctypes.c_int, ip, ip, ctypes.c_size_t, vp, ctypes.c_int]
    l.cuttPlanFromCandidate.restype = ctypes.c_int
    l.cuttExecute.argtypes = [ctypes.c_uint, vp, vp]
    l.cuttExecute.restype = ctypes.c_int
    l.cuttExecuteNoAlloc.argtypes = [ctypes.c_int, ip, ip, ctypes.c_size_t, vp, vp, vp]
    l.cuttExecuteNoAlloc.restype = ctypes.c_int
    l.cuttDestroy.argtypes = [ctypes.c_uint]
    l.cuttDestroy.restype = ctypes.c_int
    l.cuttGetPlanInfo.argtypes = [ctypes.c_uint, ctypes.POINTER(PlanInfo)]
    l.cuttGetPlanInfo.restype = ctypes.c_int
    l.cuttCountAddressStream.argtypes = [ctypes.c_uint, ctypes.c_int, ctypes.POINTER(StreamCounts),
                                         ctypes.POINTER(StreamCounts)]
    l.cuttCountAddressStream.restype = ctypes.c_int
    l.cuttDeviceCallCounts.argtypes = [ctypes.POINTER(ctypes.c_ulonglong), ctypes.POINTER(ctypes.c_ulonglong)]
    l.cuttDeviceCallCounts.restype = None
    l.cuttSetMethodOverride.argtypes = [ctypes.c_int]
    l.cuttSetMethodOverride.restype = None
    l.cuttGetMethodOverride.argtypes = []
    l.cuttGetMethodOverride.restype = ctypes.c_int
    l.cuttClearPlanCache.argtypes = []
    l.cuttClearPlanCache.restype = None
    l.cuttGetLastMeasurement.argtypes = [ctypes.POINTER(PlanInfo), ctypes.c_int]
    l.cuttGetLastMeasurement.restype = ctypes.c_int
    l.cuttReduceRanks.argtypes = [ctypes.c_int, ip, ip, ip, ip]
    l.cuttReduceRanks.restype = ctypes.c_int
    l.cuttCandidatesCreate.argtypes = [ctypes.c_int, ip, ip, ctypes.c_size_t]
    l.cuttCandidatesCreate.restype = vp
    l.cuttCandidatesCreateEx.argtypes = [ctypes.c_int, ip, ip, ctypes.c_size_t, ctypes.c_size_t]
    l.cuttCandidatesCreateEx.restype = vp
    llp = ctypes.POINTER(ctypes.c_longlong)
    l.cuttCandidatesCreateStrided.argtypes = [ctypes.c_int, ip, ip, ctypes.c_size_t, llp, llp, ctypes.c_size_t]
    l.cuttCandidatesCreateStrided.restype = vp
    l.cuttSlabDecomposition.argtypes = [ctypes.c_int, ip, ip, ctypes.c_size_t, ctypes.c_longlong, llp, ctypes.c_longlong]
    l.cuttSlabDecomposition.restype = ctypes.c_longlong
    l.cuttCandidatesFree.argtypes = [vp]
    l.cuttCandidatesFree.restype = None
    l.cuttCandidatesCount.argtypes = [vp]
    l.cuttCandidatesCount.restype = ctypes.c_int
    l.cuttCandidatesBest.argtypes = [vp]
    l.cuttCandidatesBest.restype = ctypes.c_int
    l.cuttCandidatesInfo.argtypes = [vp, ctypes.c_int, ctypes.POINTER(PlanInfo)]
    l.cuttCandidatesInfo.restype = ctypes.c_int
    l.cuttCandidatesData.argtypes = [vp, ctypes.c_int, ctypes.c_int, ctypes.c_int,
                                     ctypes.POINTER(ctypes.c_longlong), ctypes.c_longlong]
    l.cuttCandidatesData.restype = ctypes.c_longlong
    l.cuttModelGlTransactionsSeg.argtypes = [ip, ctypes.c_int]
    l.cuttModelGlTransactionsSeg.restype = ctypes.c_int
    l.cuttModelGlTransactionsCont.argtypes = [ctypes.c_int] * 3
    l.cuttModelGlTransactionsCont.restype = ctypes.c_int
    l.cuttModelCacheLinesSeg.argtypes = [ip, ctypes.c_int, ctypes.c_int, ip, ip]
    l.cuttModelCacheLinesSeg.restype = None
    l.cuttModelCacheLinesCont.argtypes = [ctypes.c_int] * 3 + [ip, ip]
    l.cuttModelCacheLinesCont.restype = None
    l.cuttModelShTransactions.argtypes = [ctypes.c_int] * 4 + [ip, ctypes.c_int, ip]
    l.cuttModelShTransactions.restype = None
    _lib = l
    return l


def _ints(v):
    return (ctypes.c_int * len(v))(*[int(x) for x in v])


def _ptr(p):
    return ctypes.c_void_p(int(p) if p else 0)


def cuttPlan(rank, dim, permutation, sizeofType, stream=0):
    """cuttPlan: returns (result code, handle)."""
    h = ctypes.c_uint(0xFFFFFFFF)
    rc = lib().cuttPlan(ctypes.byref(h), int(rank), _ints(dim), _ints(permutation), int(sizeofType), _ptr(stream))
    return rc, h.value


def cuttPlanMeasure(rank, dim, permutation, sizeofType, stream, idata, odata):
    """cuttPlanMeasure: returns (result code, handle).  Destroys the contents of odata."""
    h = ctypes.c_uint(0xFFFFFFFF)
    rc = lib().cuttPlanMeasure(ctypes.byref(h), int(rank), _ints(dim), _ints(permutation), int(sizeofType),
                               _ptr(stream), _ptr(idata), _ptr(odata))
    return rc, h.value


def cuttPlanFromCandidate(rank, dim, permutation, sizeofType, stream, index):
    """Plan built from candidate `index` of the enumeration: returns (result code, handle)."""
    h = ctypes.c_uint(0xFFFFFFFF)
    rc = lib().cuttPlanFromCandidate(ctypes.byref(h), int(rank), _ints(dim), _ints(permutation),
                                     int(sizeofType), _ptr(stream), int(index))
    return rc, h.value


def cuttExecute(handle, idata, odata):
    return lib().cuttExecute(ctypes.c_uint(handle), _ptr(idata), _ptr(odata))


def cuttExecuteNoAlloc(rank, dim, permutation, sizeofType, stream, idata, odata):
    """Plan and execute in one call that allocates nothing on the device: returns the result code."""
    return lib().cuttExecuteNoAlloc(int(rank), _ints(dim), _ints(permutation), int(sizeofType), _ptr(stream),
                                    _ptr(idata), _ptr(odata))


def cuttDestroy(handle):
    return lib().cuttDestroy(ctypes.c_uint(handle))


def get_plan_info(handle):
    info = PlanInfo()
    rc = lib().cuttGetPlanInfo(ctypes.c_uint(handle), ctypes.byref(info))
    if rc != CUTT_SUCCESS:
        raise CuttError(rc, "cuttGetPlanInfo")
    return info


def count_address_stream(handle, num_samples=0):
    """(counts on the device, counts by the host model) for the plan's address stream."""
    dev, mod = StreamCounts(), StreamCounts()
    rc = lib().cuttCountAddressStream(ctypes.c_uint(handle), int(num_samples), ctypes.byref(dev), ctypes.byref(mod))
    if rc != CUTT_SUCCESS:
        raise CuttError(rc, "cuttCountAddressStream")
    return dev, mod


def set_method_override(method):
    lib().cuttSetMethodOverride(int(method))


def device_call_counts():
    """(device allocations, table uploads) the library has made in this process so far."""
    a, u = ctypes.c_ulonglong(0), ctypes.c_ulonglong(0)
    lib().cuttDeviceCallCounts(ctypes.byref(a), ctypes.byref(u))
    return a.value, u.value


def clear_plan_cache():
    lib().cuttClearPlanCache()


def get_last_measurement():
    n = lib().cuttGetLastMeasurement(None, 0)
    arr = (PlanInfo * max(n, 1))()
    lib().cuttGetLastMeasurement(arr, n)
    return [arr[i] for i in range(n)]


def reduce_ranks(dim, permutation):
    n = len(dim)
    rd = (ctypes.c_int * n)()
    rp = (ctypes.c_int * n)()
    k = lib().cuttReduceRanks(n, _ints(dim), _ints(permutation), rd, rp)
    if k < 0:
        raise ValueError("cuttReduceRanks failed")
    return list(rd[:k]), list(rp[:k])


def slab_decomposition(dim, permutation, sizeofType, span_limit=0):
    """How the library cuts a tensor into pieces one launch can address: (shapes, pieces) with
    shapes = [dict(dim, perm, stride_in, stride_out)] and pieces = [(shape, base_in, base_out)];
    None if it cannot be cut."""
    n = lib().cuttSlabDecomposition(len(dim), _ints(dim), _ints(permutation), int(sizeofType), int(span_limit), None, 0)
    if n < 0:
        return None
    buf = (ctypes.c_longlong * n)()
    lib().cuttSlabDecomposition(len(dim), _ints(dim), _ints(permutation), int(sizeofType), int(span_limit), buf, n)
    v = [int(x) for x in buf]
    num_shapes, num_pieces = v[0], v[1]
    pos = 2
    shapes = []
    for _ in range(num_shapes):
        r = v[pos]
        pos += 1
        f = [v[pos + i * r: pos + (i + 1) * r] for i in range(4)]
        pos += 4 * r
        shapes.append(dict(dim=f[0], perm=f[1], stride_in=f[2], stride_out=f[3]))
    pieces = [tuple(v[pos + 3 * i: pos + 3 * i + 3]) for i in range(num_pieces)]
    return shapes, pieces


class Candidates:
    """The planner's candidate list for a problem, built for MI355X properties without a GPU."""

    def __init__(self, dim, permutation, sizeofType, lds_per_block=0, stride_in=None, stride_out=None):
        if stride_in is None:
            self._l = lib().cuttCandidatesCreateEx(len(dim), _ints(dim), _ints(permutation), int(sizeofType),
                                                   int(lds_per_block))
        else:  # one piece of a larger tensor, with that tensor's element strides
            lls = lambda v: (ctypes.c_longlong * len(v))(*[int(x) for x in v])
            self._l = lib().cuttCandidatesCreateStrided(len(dim), _ints(dim), _ints(permutation), int(sizeofType),
                                                        lls(stride_in), lls(stride_out), int(lds_per_block))
        if not self._l:
            raise ValueError("invalid transpose problem")

    def close(self):
        if self._l:
            lib().cuttCandidatesFree(self._l)
            self._l = None

    def __enter__(self):
        return self

    def __exit__(self, *a):
        self.close()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def __len__(self):
        return lib().cuttCandidatesCount(self._l)

    @property
    def best(self):
        return lib().cuttCandidatesBest(self._l)

    def info(self, i):
        info = PlanInfo()
        if lib().cuttCandidatesInfo(self._l, i, ctypes.byref(info)) != 0:
            raise IndexError(i)
        return info

    def data(self, i, what, cls=0):
        n = lib().cuttCandidatesData(self._l, i, what, cls, None, 0)
        if n < 0:
            raise ValueError("no such data: candidate %d what %d" % (i, what))
        buf = (ctypes.c_longlong * max(n, 1))()
        lib().cuttCandidatesData(self._l, i, what, cls, buf, n)
        return np.frombuffer(buf, dtype=np.int64, count=n).copy()
