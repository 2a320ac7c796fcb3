"""The C ABI library: it loads, exports every symbol the header declares, and its
host-only entry points behave (no GPU work here)."""
import ctypes
import os
import re

import pytest

from grouped_mm_bf16_amd import _lib

ROOT = os.path.abspath(os.path.join(os.path.dirname(__file__), ".."))
HEADER = os.path.join(ROOT, "include", "grouped_mm_hip.h")


def declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(gmm_[a-z0-9_]+)\s*\(", text)))


def test_library_exists_and_loads():
    assert os.path.exists(_lib.LIB_PATH), "build with: python -m grouped_mm_bf16_amd.build"
    lib = _lib.load()
    assert lib.gmm_abi_version() == _lib.ABI_VERSION == 3


def test_every_declared_symbol_is_exported_and_bound():
    names = declared_functions()
    assert {"gmm_2d3d", "gmm_3d3d", "gmm_2d2d", "gmm_3d2d", "gmm_abi_version"} <= set(names)
    raw = ctypes.CDLL(_lib.LIB_PATH)
    for n in names:
        assert hasattr(raw, n), f"{n} declared in the header but not exported"
    assert sorted(_lib.SIGNATURES) == names, "ctypes table and header disagree"


def test_header_has_no_torch_or_cxx_types():
    text = open(HEADER).read()
    assert 'extern "C"' in text
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)  # declarations only, not the prose
    for word in ("torch", "at::", "std::", "Tensor"):
        assert word not in text


def test_status_strings():
    lib = _lib.load()
    assert lib.gmm_status_string(0) == b"ok"
    for s in (1, 2, 3):
        assert len(lib.gmm_status_string(s)) > 5
    with pytest.raises(RuntimeError, match="status 1"):
        _lib.check(1, "x")


def test_path_switch_round_trips():
    lib = _lib.load()
    prev = lib.gmm_set_path(_lib.PATH_GENERIC)
    assert lib.gmm_set_path(prev) == _lib.PATH_GENERIC
    assert lib.gmm_set_path(99) == -1
    prev = lib.gmm_set_xcd_remap(0)
    assert lib.gmm_set_xcd_remap(prev) == 0


def test_missing_library_is_a_loud_error(monkeypatch, tmp_path):
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", str(tmp_path / "nope.so"))
    with pytest.raises(RuntimeError, match="no fallback"):
        _lib.load()


def test_route_workspace_size_is_host_arithmetic():
    """gmm_moe_route_workspace_bytes needs no GPU: one int32 row of `experts` counters per sort workgroup of
    at most 1024 slots, at most 256 workgroups; -1 for sizes the routing does not take."""
    lib = _lib.load()
    f = lib.gmm_moe_route_workspace_bytes
    assert f(5000, 128, 8) == 40 * 128 * 4            # 40000 slots -> 40 workgroups
    assert f(8192, 8, 2) == 16 * 8 * 4
    assert f(1, 1, 1) == 4 and f(0, 8, 2) == 0
    assert f(10 ** 7, 1023, 1) == 256 * 1023 * 4      # capped at 256 workgroups
    assert f(-1, 8, 2) == -1 and f(8, 0, 1) == -1 and f(8, 1024, 1) == -1 and f(8, 8, 0) == -1
    assert f(2 ** 30, 8, 2) == -1                     # tokens * top_k must stay below 2^31
