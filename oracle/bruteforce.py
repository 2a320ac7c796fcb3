"""ctypes front-end of oracle_bruteforce.c: TEST INFRASTRUCTURE ONLY.

Loads oracle/_build/liboracle_bruteforce.so (built by oracle/Makefile) and runs
the element-ownership fp64 triple loops on dense CPU tensors.
"""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np
import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "_build", "liboracle_bruteforce.so")
_lib = None


def build() -> str:
    subprocess.run(["make", "-s", "-C", _HERE], check=True)
    return _SO


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        _lib = ctypes.CDLL(_SO)
        _lib.oracle_upper_bound.restype = ctypes.c_int
        _lib.oracle_f32_to_bf16_bits.restype = ctypes.c_uint16
        _lib.oracle_f32_to_bf16_bits.argtypes = [ctypes.c_float]
    return _lib


def _f32(t: torch.Tensor) -> np.ndarray:
    return np.ascontiguousarray(t.detach().cpu().to(torch.float32).contiguous().numpy())


def _i32(t) -> np.ndarray:
    return np.ascontiguousarray(torch.as_tensor(t).detach().cpu().to(torch.int32).numpy())


def _p(a: np.ndarray):
    return a.ctypes.data_as(ctypes.c_void_p)


def upper_bound(offs, idx: int) -> int:
    o = _i32(offs)
    return int(lib().oracle_upper_bound(_p(o), ctypes.c_int(o.size), ctypes.c_int(idx)))


def f32_to_bf16_bits(x: float) -> int:
    return int(lib().oracle_f32_to_bf16_bits(ctypes.c_float(x)))


def grouped_mm_f64(a: torch.Tensor, b: torch.Tensor, offs=None, fill=float("nan")) -> torch.Tensor:
    """fp64 result of the four variants; unowned elements keep `fill`."""
    L = lib()
    an, bn = _f32(a), _f32(b)
    a2, b2 = a.dim() == 2, b.dim() == 2
    c = ctypes.c_int
    if not a2 and not b2:
        G, M, K = an.shape
        N = bn.shape[2]
        out = np.full((G, M, N), fill, dtype=np.float64)
        L.oracle_3d3d(_p(an), _p(bn), _p(out), c(G), c(M), c(N), c(K))
    elif a2 and b2:
        o = _i32(offs)
        M, Kt = an.shape
        N = bn.shape[1]
        out = np.full((o.size, M, N), fill, dtype=np.float64)
        L.oracle_2d2d(_p(an), _p(bn), _p(out), _p(o), c(o.size), c(M), c(N), c(Kt))
    elif a2:
        o = _i32(offs)
        Mt, K = an.shape
        N = bn.shape[2]
        out = np.full((Mt, N), fill, dtype=np.float64)
        L.oracle_2d3d(_p(an), _p(bn), _p(out), _p(o), c(o.size), c(Mt), c(N), c(K))
    else:
        o = _i32(offs)
        G, M, K = an.shape
        Nt = bn.shape[1]
        out = np.full((M, Nt), fill, dtype=np.float64)
        L.oracle_3d2d(_p(an), _p(bn), _p(out), _p(o), c(o.size), c(M), c(Nt), c(K))
    return torch.from_numpy(out)
