"""ctypes binding of libgrouped_mm_hip.so (C ABI declared in include/grouped_mm_hip.h).

The library is looked up next to this file only (it is built in-tree by
``python -m grouped_mm_bf16_amd.build``).  A missing library is an error at the
first launch: there is no fallback path.
"""
from __future__ import annotations

import ctypes
import os
import threading

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libgrouped_mm_hip.so")
ABI_VERSION = 3

# enum gmm_path / gmm_dtype / gmm_status of the header
PATH_AUTO, PATH_GENERIC, PATH_MFMA = 0, 1, 2
DT_BF16, DT_F16, DT_F32 = 0, 1, 2
OK = 0

_i32, _i64, _vp = ctypes.c_int32, ctypes.c_int64, ctypes.c_void_p

# name -> (restype, argtypes); must list every symbol the header declares
SIGNATURES = {
    "gmm_abi_version": (ctypes.c_int, []),
    "gmm_status_string": (ctypes.c_char_p, [ctypes.c_int]),
    "gmm_workspace_bytes": (_i64, []),
    "gmm_2d3d": (ctypes.c_int, [_vp, _vp, _vp, _vp, _i32] + [_i64] * 3 + [_i64] * 7 + [_i32, _i32, _vp, _i64, _vp]),
    "gmm_2d3d_gather": (ctypes.c_int, [_vp] * 5 + [_i32] + [_i64] * 4 + [_i64] * 7 + [_i32, _i32, _vp, _i64, _vp]),
    "gmm_2d3d_swiglu": (ctypes.c_int, [_vp] * 5 + [_i32] + [_i64] * 4 + [_i64] * 7 + [_i32, _vp]),
    "gmm_3d3d": (ctypes.c_int, [_vp, _vp, _vp, _i32] + [_i64] * 3 + [_i64] * 9 + [_i32, _i32, _vp, _i64, _vp]),
    "gmm_2d2d": (ctypes.c_int, [_vp, _vp, _vp, _vp, _i32] + [_i64] * 3 + [_i64] * 7 + [_i32, _i32, _vp, _i64, _vp]),
    "gmm_3d2d": (ctypes.c_int, [_vp, _vp, _vp, _vp, _i32] + [_i64] * 3 + [_i64] * 7 + [_i32, _i32, _vp, _i64, _vp]),
    "gmm_moe_route_workspace_bytes": (_i64, [_i64, _i64, _i64]),
    "gmm_moe_route": (ctypes.c_int, [_vp, _i64, _i32, _i64, _i64, _i64, _i32] + [_vp] * 5 + [_vp, _i64, _vp]),
    "gmm_moe_route_noalloc": (ctypes.c_int, [_vp, _i64, _i32, _i64, _i64, _i64, _i32] + [_vp] * 5 + [_vp]),
    "gmm_moe_activation": (ctypes.c_int, [_vp, _vp, _i64, _i64, _i64, _i64, _i32, _i32, _vp]),
    "gmm_moe_combine": (ctypes.c_int, [_vp] * 4 + [_i64] * 6 + [_i32, _vp]),
    "gmm_set_path": (ctypes.c_int, [ctypes.c_int]),
    "gmm_last_path": (ctypes.c_int, []),
    "gmm_set_mfma_config": (ctypes.c_int, [ctypes.c_int]),
    "gmm_last_mfma_config": (ctypes.c_int, []),
    "gmm_set_xcd_remap": (ctypes.c_int, [ctypes.c_int]),
    "gmm_host_tile_list": (_i64, [_vp, _i32, _i32, _i32, _i32, _i32, _i32, _i32, _i32, _i32, _i32, _vp, _i64]),
    "gmm_host_tile_list2": (_i64, [_vp] + [_i32] * 11 + [_vp, _i64]),
    "gmm_host_tile_list3": (_i64, [_vp] + [_i32] * 13 + [_vp, _i64]),
    "gmm_set_tile_heights": (ctypes.c_int, [ctypes.c_int, ctypes.c_int]),
    "gmm_set_tail_split": (ctypes.c_int, [ctypes.c_int]),
    "gmm_set_group_major": (ctypes.c_int, [ctypes.c_int]),
}

_lock = threading.Lock()
_lib = None


def load() -> ctypes.CDLL:
    """Load the shared library once; raise if it is absent or of another ABI version."""
    global _lib
    if _lib is not None:
        return _lib
    with _lock:
        if _lib is not None:
            return _lib
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing: build it with `python -m grouped_mm_bf16_amd.build` "
                "(grouped_mm has no fallback path)"
            )
        lib = ctypes.CDLL(LIB_PATH)
        for name, (restype, argtypes) in SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype = restype
            fn.argtypes = argtypes
        got = lib.gmm_abi_version()
        if got != ABI_VERSION:
            raise RuntimeError(f"{LIB_PATH} has ABI version {got}, this package needs {ABI_VERSION}")
        _lib = lib
    return _lib


def check(status: int, what: str) -> None:
    if status != OK:
        msg = load().gmm_status_string(status).decode()
        raise RuntimeError(f"{what}: {msg} (status {status})")
