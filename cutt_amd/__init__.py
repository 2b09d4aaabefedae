"""cutt_amd - MI355X-native tensor transpose library with cuTT's plan API.

The product is the C-ABI shared library ``libcutt.so`` (built from ``csrc/``;
headers in ``include/``).  This package is a thin ctypes binding over it that
keeps the names and argument order of the C functions, for tests and
benchmarks written in Python.
"""
from .api import (  # noqa: F401
    CUTT_SUCCESS, CUTT_INVALID_PLAN, CUTT_INVALID_PARAMETER, CUTT_INVALID_DEVICE,
    CUTT_INTERNAL_ERROR, CUTT_UNDEFINED_ERROR,
    METHOD_NAMES, METHOD_TRIVIAL, METHOD_PACKED, METHOD_PACKEDSPLIT, METHOD_TILED, METHOD_TILEDCOPY,
    CuttError, PlanInfo, StreamCounts, lib, lib_path,
    cuttPlan, cuttPlanMeasure, cuttPlanFromCandidate, cuttExecute, cuttExecuteNoAlloc, cuttDestroy,
    get_plan_info, count_address_stream, set_method_override, clear_plan_cache, device_call_counts, get_last_measurement, reduce_ranks, Candidates, slab_decomposition,
)
from .build import build  # noqa: F401
