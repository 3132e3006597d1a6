"""The C interface of the host-side core (``csrc/hostcore.cpp``): page pools, block tables,
request lengths and the packing of a step's index arrays.  The library is compiled with the
host compiler the first time it is asked for; there is no Python version of what it does."""
from __future__ import annotations

import ctypes

import numpy as np

from ..kernels import build as kernel_build

_INT_P = ctypes.POINTER(ctypes.c_int)
_lib = None


def int_pointer(array: np.ndarray):
    """Pointer to the data of a contiguous int32 array (the array must outlive the call)."""
    return array.ctypes.data_as(_INT_P)


def as_ints(values) -> np.ndarray:
    return np.ascontiguousarray(values, dtype=np.int32)


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        core = kernel_build.load_module("hostcore")
        p, i, l = ctypes.c_void_p, ctypes.c_int, ctypes.c_long
        signatures = {
            "hc_pool_create": (p, [i]), "hc_pool_destroy": (None, [p]), "hc_pool_total": (i, [p]),
            "hc_pool_free_count": (i, [p]), "hc_pool_take": (i, [p, i, _INT_P]),
            "hc_pool_give": (i, [p, _INT_P, i]), "hc_pool_check": (i, [p, _INT_P, i]),
            "hc_create": (p, [i, _INT_P, _INT_P, _INT_P, i]), "hc_destroy": (None, [p]),
            "hc_group_pool": (p, [p, i]), "hc_slot_pool": (p, [p]), "hc_add_request": (i, [p]),
            "hc_finish": (i, [p, i]), "hc_length": (i, [p, i]), "hc_lengths": (None, [p, i, _INT_P, _INT_P]),
            "hc_reserve": (i, [p, i, _INT_P, _INT_P, _INT_P]), "hc_commit": (i, [p, i, _INT_P, _INT_P]),
            "hc_table": (i, [p, i, i, _INT_P, i]), "hc_first_live": (i, [p, i, i]), "hc_check": (i, [p]),
            "hc_pack": (l, [p, i, _INT_P, _INT_P, _INT_P, _INT_P, _INT_P, i, _INT_P, i, i, _INT_P, i, i, i, i, _INT_P,
                            _INT_P, _INT_P, l, _INT_P]),
        }
        for name, (result, arguments) in signatures.items():
            function = getattr(core, name)
            function.restype, function.argtypes = result, arguments
        _lib = core
    return _lib
