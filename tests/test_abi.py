"""The C ABI: libvtdge.so loads and exports exactly what include/vtdge.h declares.  No GPU needed.

Only argument validation is exercised here (it happens before any HIP call); compute calls live in the
`gpu` tests.
"""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "vtdge.h")


def _declared():
    """name -> number of parameters, parsed from the header."""
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    out = {}
    for m in re.finditer(r"(?:int|const char \*)\s*(vtdge_\w+)\s*\(([^;]*?)\)\s*;", text, flags=re.S):
        args = m.group(2).strip()
        out[m.group(1)] = 0 if args == "void" else len(args.split(","))
    return out


@pytest.fixture(scope="module")
def lib():
    from vtpack_amd import _lib
    if not os.path.exists(_lib.LIB_PATH):
        _lib.build()
    return _lib.load()


def test_header_symbols_are_exported(lib):
    decl = _declared()
    assert len(decl) >= 11
    for name in decl:
        assert hasattr(lib, name), f"{name} declared in include/vtdge.h but not exported by libvtdge.so"


def test_binding_covers_header():
    from vtpack_amd import _lib
    decl = _declared()
    assert set(_lib.EXPORTS) == set(decl)
    for name, argtypes in _lib.SIGNATURES.items():
        assert len(argtypes) == decl[name], f"{name}: binding has {len(argtypes)} args, header {decl[name]}"


def test_version_and_error_string(lib):
    assert lib.vtdge_version() >= 100
    assert isinstance(lib.vtdge_last_error(), bytes)


def test_argument_validation_returns_codes(lib):
    # NULL operands -> VTDGE_ERR_ARG, no exception, message set
    rc = lib.vtdge_linear(None, 0, None, None, None, 0, None, 0, None, 16, 16, 16, 0, 0, None)
    assert rc == -1 and b"NULL" in lib.vtdge_last_error()
    buf = ctypes.create_string_buffer(4096)
    p = ctypes.cast(buf, ctypes.c_void_p)
    # unknown dtype
    assert lib.vtdge_linear(p, 16, p, None, None, 0, p, 16, None, 16, 16, 16, 0, 7, None) == -1
    # K not a multiple of 16 bytes -> unsupported
    assert lib.vtdge_linear(p, 6, p, None, None, 0, p, 16, None, 16, 16, 6, 0, 0, None) == -2
    # head_dim outside the built family
    rc = lib.vtdge_sparse_attention(p, 48, 48, p, p, 48, 48, 48, p, p, 48, 48, 1, 1, 48, 4, 4, 1.0, 0, None)
    assert rc == -2 and b"head_dim" in lib.vtdge_last_error()
    # token grid not divisible by the region size
    assert lib.vtdge_router(p, p, p, None, p, 1, 6, 8, 16, 1, 4, 3, 0, None) == -1
    # too many splits
    assert lib.vtdge_index_to_patch(p, p, 1, 1, 1, 9, 4, 1, None, 0, p, p, None) == -2
    # channels not a multiple of the 16-byte vector
    assert lib.vtdge_compress(p, p, None, 4, p, None, None, None, 0.0, 1, 17, 6, 4, 1, 0, None) == -2
    # zero rows is a valid no-op that touches no GPU
    assert lib.vtdge_layernorm(p, p, p, p, None, 0, 16, 1e-6, 0, None) == 0
