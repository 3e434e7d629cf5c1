"""ctypes view of the C ABI in ``include/optimi_hip.h`` (``liboptimi_hip.so``).

For callers that hold raw device pointers rather than torch tensors, and for the parity
tests, which call the library through this boundary.  Signatures are declared once, in
``PROTOTYPES``, in the order of the header.
"""

from __future__ import annotations

import ctypes as C
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "liboptimi_hip.so")

F32, BF16, F16 = 0, 1, 2
KAHAN, UPDATE, DECOUPLE_WD, ADAM_WD, DECOUPLE_LR, DAMPENING, RECTIFY, LOOKAHEAD, RESIDENT = 1, 2, 4, 8, 16, 32, 64, 128, 256
PROBE_SCRAMBLE = 512

_p, _pp, _i, _i64, _u32, _d = C.c_void_p, C.POINTER(C.c_void_p), C.c_int, C.c_int64, C.c_uint32, C.c_double
_i64p = C.POINTER(C.c_int64)
_ip = C.POINTER(C.c_int)

PROTOTYPES = {
    "optimi_hip_error_string": (C.c_char_p, [_i]),
    "optimi_hip_version": (_i, []),
    "optimi_hip_chunk_elems": (_i64, [_i]),
    "optimi_hip_group_create": (_i, [_pp]),
    "optimi_hip_group_destroy": (_i, [_p]),
    "optimi_hip_adam_multi": (_i, [_p, _i, _pp, _pp, _pp, _pp, _pp, _i64p, _i, _d, _d, _d, _d, _d, _d, _u32, _p]),
    "optimi_hip_lion_multi": (_i, [_p, _i, _pp, _pp, _pp, _pp, _i64p, _i, _d, _d, _d, _d, _u32, _p]),
    "optimi_hip_stableadamw_multi": (_i, [_p, _i, _pp, _pp, _pp, _pp, _pp, _i64p, _i, _d, _d, _d, _d, _d, _d, _d, _u32, _p]),
    "optimi_hip_adan_multi": (_i, [_p, _i, _pp, _pp, _pp, _pp, _pp, _pp, _pp, _i64p, _i, _d, _d, _d, _d, _d, _d, _d, _d, _u32, _p]),
    "optimi_hip_sgd_multi": (_i, [_p, _i, _pp, _pp, _pp, _pp, _i64p, _i, _d, _d, _d, _u32, _p]),
    "optimi_hip_radam_multi": (_i, [_p, _i, _pp, _pp, _pp, _pp, _pp, _i64p, _i, _d, _d, _d, _d, _d, _d, _d, _u32, _p]),
    "optimi_hip_ranger_multi": (_i, [_p, _i, _pp, _pp, _pp, _pp, _pp, _pp, _i64p, _i, _d, _d, _d, _d, _d, _d, _d, _d, _u32, _p]),
    "optimi_hip_adam_multi_mixed": (_i, [_p, _i, _pp, _pp, _pp, _pp, _pp, _i64p, _ip, _d, _d, _d, _d, _d, _d, _u32, _p]),
    "optimi_hip_lion_multi_mixed": (_i, [_p, _i, _pp, _pp, _pp, _pp, _i64p, _ip, _d, _d, _d, _d, _u32, _p]),
    "optimi_hip_stableadamw_multi_mixed": (_i, [_p, _i, _pp, _pp, _pp, _pp, _pp, _i64p, _ip, _d, _d, _d, _d, _d, _d, _d, _u32, _p]),
    "optimi_hip_adan_multi_mixed": (_i, [_p, _i, _pp, _pp, _pp, _pp, _pp, _pp, _pp, _i64p, _ip, _d, _d, _d, _d, _d, _d, _d, _d, _u32, _p]),
    "optimi_hip_sgd_multi_mixed": (_i, [_p, _i, _pp, _pp, _pp, _pp, _i64p, _ip, _d, _d, _d, _u32, _p]),
    "optimi_hip_radam_multi_mixed": (_i, [_p, _i, _pp, _pp, _pp, _pp, _pp, _i64p, _ip, _d, _d, _d, _d, _d, _d, _d, _u32, _p]),
    "optimi_hip_ranger_multi_mixed": (_i, [_p, _i, _pp, _pp, _pp, _pp, _pp, _pp, _i64p, _ip, _d, _d, _d, _d, _d, _d, _d, _d, _u32, _p]),
    "optimi_hip_adam_single": (_i, [_p, _p, _p, _p, _p, _i64, _i, _d, _d, _d, _d, _d, _d, _u32, _p]),
    "optimi_hip_lion_single": (_i, [_p, _p, _p, _p, _i64, _i, _d, _d, _d, _d, _u32, _p]),
    "optimi_hip_stableadamw_single": (_i, [_p, _p, _p, _p, _p, _p, _i64, _i, _d, _d, _d, _d, _d, _d, _d, _u32, _p]),
    "optimi_hip_stableadamw_single_noalloc": (_i, [_p, _p, _p, _p, _p, _i64, _i, _d, _d, _d, _d, _d, _d, _d, _u32, _p]),
    "optimi_hip_adan_single": (_i, [_p, _p, _p, _p, _p, _p, _p, _i64, _i, _d, _d, _d, _d, _d, _d, _d, _d, _u32, _p]),
    "optimi_hip_sgd_single": (_i, [_p, _p, _p, _p, _i64, _i, _d, _d, _d, _u32, _p]),
    "optimi_hip_radam_single": (_i, [_p, _p, _p, _p, _p, _i64, _i, _d, _d, _d, _d, _d, _d, _d, _u32, _p]),
    "optimi_hip_ranger_single": (_i, [_p, _p, _p, _p, _p, _p, _i64, _i, _d, _d, _d, _d, _d, _d, _d, _d, _u32, _p]),
    "optimi_hip_copy_probe": (_i, [_p, _p, _i64, _p]),
    "optimi_hip_stream_probe": (_i, [_p, _i, _pp, _i64p, _i, _i, _i, _u32, _p]),
    "optimi_hip_launch_count": (_i64, []),
    "optimi_hip_resident_bytes": (_i64, []),
    "optimi_hip_upload_count": (_i64, []),
    "optimi_hip_resident_launch_count": (_i64, []),
    "optimi_hip_launch_limit": (_i64, [_i64]),
}

_lib = None


def lib() -> C.CDLL:
    """Loads the library (no HIP call is made until a function that needs the device runs)."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(f"{LIB_PATH} is not built; run `python -m optimi_amd.build`")
        L = C.CDLL(LIB_PATH)
        for name, (res, args) in PROTOTYPES.items():
            fn = getattr(L, name)
            fn.restype = res
            fn.argtypes = args
        _lib = L
    return _lib


class OptimiHipError(RuntimeError):
    def __init__(self, status: int, what: str):
        self.status = status
        super().__init__(f"{what}: {lib().optimi_hip_error_string(status).decode()} (status {status})")


def check(status: int, what: str):
    if status != 0:
        raise OptimiHipError(status, what)


def ptr_array(ptrs):
    """A C array of void* from an iterable of integer addresses (None = NULL)."""
    ptrs = list(ptrs)
    return (C.c_void_p * max(len(ptrs), 1))(*ptrs)


def ptr_table(columns):
    """A C array of pointers to C arrays of void*: ``columns[a][i]`` is the address of array ``a`` of
    tensor ``i``.  Returns the table and the inner arrays, which the caller keeps alive for the call."""
    inner = [ptr_array(col) for col in columns]
    table = (C.c_void_p * max(len(inner), 1))(*[C.cast(col, C.c_void_p).value for col in inner])
    return table, inner


def i64_array(vals):
    vals = list(vals)
    return (C.c_int64 * max(len(vals), 1))(*vals)


class Group:
    """Owns an ``optimi_group`` handle."""

    def __init__(self):
        self.handle = C.c_void_p()
        check(lib().optimi_hip_group_create(C.byref(self.handle)), "optimi_hip_group_create")

    def close(self):
        if self.handle:
            lib().optimi_hip_group_destroy(self.handle)
            self.handle = C.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass
