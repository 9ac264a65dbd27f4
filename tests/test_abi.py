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


def _julia_blocks(text):
    """A rough reading of Julia source, enough for the two mistakes that would stop `include` before anything runs:
    returns (orphans, depth): docstrings that are not directly followed by something to document, and the balance
    of block openers against `end`."""
    lines = text.split("\n")
    orphans, depth, i = [], 0, 0
    opener = re.compile(r"^\s*(function|struct|mutable struct|module|macro|if|for|while|let|begin|quote|try|do)\b|"
                        r"\b(begin|do|quote)\s*$|=\s*(begin|let|quote)\b|\b(function)\s*\(")
    definition = re.compile(r"^\s*(function|struct|mutable struct|macro|const|module|abstract type|@\w+|[\w.!]+(\{.*\})?\(.*\)\s*(where\b.*)?=|[\w.!]+\s*=)")
    while i < len(lines):
        line = lines[i]
        stripped = line.strip()
        doc_end = None
        if stripped.startswith('"""'):
            j = i if stripped.count('"""') >= 2 and len(stripped) > 3 else i + 1
            while j < len(lines) and '"""' not in lines[j] and j != i:
                j += 1
            doc_end = j
        elif re.match(r'^"([^"\\]|\\.)*"\s*$', stripped) and not line.startswith(" "):
            doc_end = i
        if doc_end is not None:
            nxt = lines[doc_end + 1] if doc_end + 1 < len(lines) else ""
            if not definition.match(nxt):
                orphans.append((i + 1, nxt.strip()[:60]))
            i = doc_end + 1
            continue
        code = re.sub(r'"([^"\\]|\\.)*"', '""', line.split("#")[0])
        if not re.search(r"\bend\b", code) or not re.match(r"^\s*(if|for|while|function|struct|try|let|begin|quote|macro|module)\b.*\bend\s*$", code):
            if opener.search(code):
                depth += 1
            if re.match(r"^\s*end\b", code) or re.search(r"\bend\s*$", code) and not opener.search(code):
                depth -= 1
        i += 1
    return orphans, depth


def test_julia_glue_has_no_orphan_docstrings_and_balanced_blocks():
    """Julia refuses to load a file in which a docstring is followed by another string literal or a blank line
    ("cannot document the following expression"), and one with an unmatched `end`.  No Julia runtime exists here, so
    the two are checked textually; the scanner is itself checked on small samples."""
    good = 'module M\n"""\n    f(x)\n\ndoc\n"""\nfunction f(x)\n    x\nend\n"one-line doc"\ng(x) = x\nend\n'
    assert _julia_blocks(good) == ([], 0)
    bad = 'module M\n"""\ndoc of f\n"""\n"doc of g"\ng(x) = x\nfunction f(x)\n    x\nend\nend\n'
    orphans, depth = _julia_blocks(bad)
    assert len(orphans) == 1 and orphans[0][0] == 2 and depth == 0
    assert _julia_blocks('function f(x)\n    if x\n        1\n    end\n')[1] == 1
    path = os.path.join(ROOT, "moye.jl_amd", "julia", "MoYeHIP.jl")
    orphans, depth = _julia_blocks(open(path).read())
    assert not orphans, orphans
    assert depth == 0
