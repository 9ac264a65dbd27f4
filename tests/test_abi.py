"""The C-ABI library loads without a GPU and exports every symbol include/moye_hip.h declares;
struct layouts seen from ctypes match the header; the Julia glue binds only declared symbols."""
import ctypes
import os
import re
import subprocess

import pytest

import moye_hip
from moye_hip import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "moye_hip.h")


def declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(moye_[a-z0-9_]+)\s*\(", text)))


def test_library_loads_and_reports_version():
    assert moye_hip.version().startswith("moye_hip")


def test_every_declared_symbol_is_exported():
    names = declared_functions()
    assert len(names) >= 45
    out = subprocess.run(["nm", "-D", "--defined-only", _lib.LIB_PATH], capture_output=True, text=True, check=True).stdout
    exported = set(re.findall(r" T (moye_[a-z0-9_]+)", out))
    missing = [n for n in names if n not in exported]
    assert not missing, "declared in moye_hip.h but not exported: %s" % missing
    extra = sorted(exported - set(names))
    assert not extra, "exported but not declared: %s" % extra
    lib = _lib.lib()
    for n in names:
        assert getattr(lib, n) is not None


def test_struct_sizes_match_header():
    # moye_tensor: ptr(8) + 4 int32 + 2 x 8 x int64; moye_tiled_mma: 13 int32; moye_tiled_copy: 9 int32
    assert ctypes.sizeof(_lib.Tensor) == 8 + 16 + 2 * 8 * 8
    assert ctypes.sizeof(_lib.TiledMMA) == 13 * 4
    assert ctypes.sizeof(_lib.TiledCopy) == 9 * 4
    assert _lib.Tensor.shape.offset == 24 and _lib.Tensor.stride.offset == 24 + 64


def test_host_entry_points_work_without_gpu():
    buf = ctypes.create_string_buffer(256)
    lib = _lib.lib()
    lib.moye_layout_coalesce.argtypes = [ctypes.c_char_p, ctypes.c_char_p, ctypes.c_size_t]
    assert lib.moye_layout_coalesce(b"(_2,(_1,_6)):(_1,(_6,_2))", buf, 256) == 0
    assert buf.value == b"_12:_1"
    assert lib.moye_layout_coalesce(b"(_2,(_1,_6)):(_1,(_6,_2))", buf, 3) == _lib.ERR_BUFFER
    assert lib.moye_layout_coalesce(None, buf, 256) == _lib.ERR_ARG
    assert b"null argument" in lib.moye_last_error()


def test_julia_glue_binds_declared_symbols_only():
    path = os.path.join(ROOT, "moye.jl_amd", "julia", "MoYeHIP.jl")
    if not os.path.exists(path):
        pytest.skip("Julia glue not written yet")
    text = open(path).read()
    used = set(re.findall(r":(moye_[a-z0-9_]+)", text))
    assert used, "no ccall found"
    assert used <= set(declared_functions()), sorted(used - set(declared_functions()))
