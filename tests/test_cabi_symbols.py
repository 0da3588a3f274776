"""The C-ABI library loads and exports every function include/astrai_w8a8.h declares
(no compute calls: this runs without a GPU)."""

import ctypes
import os
import re

from astrai_amd.extension import _cabi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared():
    text = open(os.path.join(ROOT, "include", "astrai_w8a8.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(astrai_w8a8_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_the_expected_entry_points():
    names = _declared()
    assert names == sorted(_cabi.PROTOTYPES), (names, sorted(_cabi.PROTOTYPES))


def test_library_loads_and_exports_every_declared_symbol():
    assert os.path.exists(_cabi.LIB_PATH), "build with `make -C astrai_amd/csrc`"
    lib = ctypes.CDLL(_cabi.LIB_PATH)
    for name in _declared():
        assert hasattr(lib, name), name
    lib.astrai_w8a8_abi_version.restype = ctypes.c_int
    assert lib.astrai_w8a8_abi_version() == _cabi.ABI_VERSION
    lib.astrai_w8a8_last_error.restype = ctypes.c_char_p
    assert lib.astrai_w8a8_last_error() == b""


def test_argument_validation_needs_no_gpu():
    lib = _cabi.load()
    assert lib is not None, _cabi.load_error()
    # null pointers are rejected before anything touches the device
    rc = lib.astrai_w8a8_gemm_int8_ptpc(None, None, None, None, None, None, 4, 4, 64, 0, None)
    assert rc == 1
    assert b"null" in lib.astrai_w8a8_last_error()
    rc = lib.astrai_w8a8_quantize_bf16_fp8(16, 16, 16, None, 8, 7, None)
    assert rc == 1 and b"fmt" in lib.astrai_w8a8_last_error()
    rc = lib.astrai_w8a8_gemv_int8_ptpc(16, 16, 16, 16, None, 16, 129, 4, 256, 0, None)
    assert rc == 2 and b"M <= 128" in lib.astrai_w8a8_last_error()
    rc = lib.astrai_w8a8_gemm_fp8_block128(16, 16, 16, 16, None, 16, 4, 4, 100, None)
    assert rc == 2 and b"128" in lib.astrai_w8a8_last_error()
    rc = lib.astrai_w8a8_gemm_fp8_pt(16, 16, 16, 16, None, None, 16, 4, 4, 64, 0, 1, None)
    assert rc == 1 and b"out_scale" in lib.astrai_w8a8_last_error()
    rc = lib.astrai_w8a8_gemm_fp8_pt(8, 16, 16, 16, None, None, 16, 4, 4, 64, 0, 0, None)
    assert rc == 1 and b"aligned" in lib.astrai_w8a8_last_error()
