"""ctypes binding of libdci_hip.so (the C-ABI in include/dci_hip.h and include/dci_hip_debug.h).

The library is the product: there is no fallback.  Importing this module
without a built library raises; build it with `python -m dciknn_cuda_amd.build`.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libdci_hip.so")

NUM_COUNTERS = 4
CTR_VISITED, CTR_CANDIDATES, CTR_PROBES, CTR_STEPS = range(4)
OPT_TRAVERSAL = 0
OPT_DENSE_MIN_PROMOTIONS = 1
OPT_FORGET_HINTS = 2
OPT_APPEND = 3
APPEND_AUTO, APPEND_SORT, APPEND_MERGE = 0, 1, 2
TRAVERSAL_AUTO, TRAVERSAL_STEP, TRAVERSAL_BATCH, TRAVERSAL_DENSE = 0, 1, 2, 3
NOALLOC_SCRATCH_BYTES = 32 << 20
NUM_TIMERS = 7
T_PROJECT, T_SEGSORT, T_QPROJECT, T_TRAVERSE, T_MERGE, T_BATCH, T_DENSE = range(7)

# name -> (restype, argtypes); one line per declaration in include/dci_hip.h and include/dci_hip_debug.h
_c = ctypes
SIGNATURES = {
    "dcih_last_error": (_c.c_char_p, []),
    "dcih_abi_version": (_c.c_int, []),
    "dcih_create": (_c.c_int, [_c.c_int, _c.c_int, _c.c_int, _c.c_int, _c.c_uint64,
                               _c.POINTER(_c.c_void_p)]),
    "dcih_get_directions": (_c.c_int, [_c.c_void_p, _c.c_void_p]),
    "dcih_set_directions": (_c.c_int, [_c.c_void_p, _c.c_void_p]),
    "dcih_add": (_c.c_int, [_c.c_void_p, _c.c_int, _c.c_int64, _c.c_void_p, _c.c_int,
                            _c.c_int, _c.c_void_p]),
    "dcih_append": (_c.c_int, [_c.c_void_p, _c.c_int, _c.c_int64, _c.c_void_p, _c.c_int,
                               _c.c_int, _c.c_void_p]),
    "dcih_query": (_c.c_int, [_c.c_void_p, _c.c_int, _c.c_int, _c.c_void_p, _c.c_int,
                              _c.c_int, _c.c_int, _c.c_int, _c.c_int, _c.c_int,
                              _c.c_void_p, _c.c_void_p, _c.c_void_p, _c.c_void_p]),
    "dcih_query_noalloc": (_c.c_int, [_c.c_void_p, _c.c_int, _c.c_int, _c.c_void_p, _c.c_int,
                                      _c.c_int, _c.c_int, _c.c_int, _c.c_int, _c.c_int,
                                      _c.c_void_p, _c.c_void_p, _c.c_void_p, _c.c_void_p]),
    "dcih_debug_launch_map": (_c.c_int64, [_c.c_int, _c.c_int, _c.c_int, _c.c_int64,
                                           _c.POINTER(_c.c_int), _c.POINTER(_c.c_int),
                                           _c.POINTER(_c.c_int)]),
    "dcih_get_index": (_c.c_int, [_c.c_void_p, _c.c_void_p, _c.c_void_p]),
    "dcih_set_option": (_c.c_int, [_c.c_void_p, _c.c_int, _c.c_int]),
    "dcih_phase_profile": (_c.c_int, [_c.c_void_p, _c.c_void_p]),
    "dcih_debug_positions": (_c.c_int, [_c.c_void_p, _c.c_void_p, _c.c_void_p, _c.c_void_p]),
    "dcih_profile": (_c.c_int, [_c.c_void_p, _c.c_int]),
    "dcih_last_timings": (_c.c_int, [_c.c_void_p, _c.c_void_p]),
    "dcih_num_points": (_c.c_int64, [_c.c_void_p]),
    "dcih_clear": (_c.c_int, [_c.c_void_p]),
    "dcih_reset": (_c.c_int, [_c.c_void_p]),
    "dcih_free": (_c.c_int, [_c.c_void_p]),
    "dcih_project": (_c.c_int, [_c.c_void_p, _c.c_int, _c.c_void_p, _c.c_int64, _c.c_int,
                                _c.c_void_p, _c.c_void_p]),
    "dcih_segsort": (_c.c_int, [_c.c_void_p, _c.c_int, _c.c_int64, _c.c_int, _c.c_void_p,
                                _c.c_void_p, _c.c_void_p]),
}

_lib = None


class DCIError(RuntimeError):
    """A libdci_hip.so call returned a negative status."""

    def __init__(self, code, message):
        super().__init__("libdci_hip: %s (status %d)" % (message, code))
        self.code = code


def lib():
    """The loaded library with every entry point typed."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(
                "%s is missing: build it with `python -m dciknn_cuda_amd.build`" % LIB_PATH)
        handle = ctypes.CDLL(LIB_PATH)
        for name, (restype, argtypes) in SIGNATURES.items():
            fn = getattr(handle, name)
            fn.restype = restype
            fn.argtypes = argtypes
        _lib = handle
    return _lib


def check(status):
    if status < 0:
        raise DCIError(status, lib().dcih_last_error().decode("utf-8", "replace"))
    return status
