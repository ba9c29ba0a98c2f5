"""The C ABI: the library loads without a GPU, exports every symbol the header declares,
and rejects bad arguments before touching the device."""

import ctypes
import os
import re

import pytest

from keras_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def header_symbols():
    text = open(os.path.join(ROOT, "include", "k3q.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(k3q_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    lib = _lib.load()
    names = header_symbols()
    assert len(names) >= 10
    for name in names:
        assert hasattr(lib, name), f"{name} is declared in include/k3q.h but not exported"
    # and the ctypes table binds exactly the declared set
    assert sorted(_lib.SIGNATURES) == names
    # test hooks live under another prefix and stay out of the ABI header
    text = open(os.path.join(ROOT, "include", "k3q.h")).read()
    for name in _lib.TEST_SIGNATURES:
        assert name.startswith("k3qt_") and hasattr(lib, name) and name not in text


def test_version_and_error_strings():
    lib = _lib.load()
    assert lib.k3q_version() >= 100
    for code in range(0, -8, -1):
        assert lib.k3q_error_string(code)
    assert b"unknown" in lib.k3q_error_string(-99)


def test_argument_validation_without_device():
    lib = _lib.load()
    null = ctypes.c_void_p(0)
    one = ctypes.c_void_p(16)  # never dereferenced: the calls below must be rejected first
    assert lib.k3q_pack_int4(null, -1, 2, 2, null, null) == -2
    assert lib.k3q_pack_int4(null, 2, 2, 2, null, null) == -1
    assert lib.k3q_pack_int4(null, 0, 2, 2, null, null) == 0  # empty tensor: nothing to do
    assert lib.k3q_unpack_int4(one, 1, 2, 1, 5, 1, one, null) == -2  # orig_len > 2 * packed_len
    assert lib.k3q_absmax_quantize(one, 7, 1, 8, 8, 1e-7, -127.0, 127.0, one, one, null) == -4
    assert lib.k3q_absmax_quantize(one, 0, 1, 8, 4, 1e-7, -127.0, 127.0, one, one, null) == -2
    assert lib.k3q_absmax_quantize(one, 0, 1, 8, 8, 1e-7, -200.0, 127.0, one, one, null) == -7
    assert lib.k3q_absmax_quantize(null, 0, 1, 8, 8, 1e-7, -127.0, 127.0, one, one, null) == -1
    assert lib.k3q_absmax_quantize(one, 0, 0, 8, 8, 1e-7, -127.0, 127.0, one, one, null) == 0
    assert lib.k3q_gemm_i8(one, one, 0, 4, 4, 4, null, null, null, 5, 0, one, null, null, 0, null) == -4
    assert lib.k3q_gemm_i8(one, one, 3, 4, 4, 4, null, null, null, 0, 0, one, null, null, 0, null) == -2
    assert lib.k3q_gemm_i8(one, one, 0, 4, 4, 4, null, null, null, 0, 0, null, null, null, 0, null) == -1
    assert lib.k3q_gemm_i8_addend(one, one, 4, 16, 8, null, null, one, 5, 0, one, null, 0, null) == -4
    assert lib.k3q_gemm_i8_addend(one, one, 4, 16, 8, null, null, null, 0, 0, one, null, 0, null) == -1
    assert lib.k3q_gemm_i8_addend(one, one, 4, 12, 8, null, null, one, 0, 0, one, null, 0, null) == -2  # N % 16
    assert lib.k3q_gemm_i8_addend(one, one, 65, 16, 8, null, null, one, 0, 0, one, null, 0, null) == -2
    assert lib.k3q_gemm_i8_addend(one, one, 0, 16, 8, null, null, null, 0, 0, one, null, 0, null) == 0
    assert lib.k3q_gemv_w4(one, 0, 1, 0, 8, one, one, null, -1, null, one, null, 0, null) == -2
    assert lib.k3q_gemv_w4(one, 9, 1, 16, 8, one, one, null, -1, null, one, null, 0, null) == -4
    assert lib.k3q_gemv_w4(one, 0, 1, 16, 8, one, one, null, 128, null, one, null, 0, null) == -1  # zero missing
    assert lib.k3q_gemv_w4_workspace_bytes(1, 8192, 8192) >= 8192 * 4
    assert lib.k3q_gemv_w4_fused(one, 0, 1, 0, 8, one, one, null, -1, null, one, null, 0, null, 0, null) == -2
    assert lib.k3q_gemv_w4_counters_bytes(8192) == 64 * 4 and lib.k3q_gemv_w4_counters_bytes(0) == 0
    assert lib.k3q_gemv_w4_addend(one, 0, 65, 16, 8, one, one, null, -1, one, one, null, 0, null, 0, null) == -2
    assert lib.k3q_gemv_w4_addend(one, 0, 4, 16, 8, one, one, null, -1, null, one, null, 0, null, 0, null) == -1
    assert lib.k3q_gemv_w4_addend(one, 0, 0, 16, 8, one, one, null, -1, null, one, null, 0, null, 0, null) == 0
    assert lib.k3q_gemm_w4_kmajor(one, 0, 64, 128, 64, one, one, null, -1, null, one, one, 1 << 20, null) == -4  # bf16 only
    assert lib.k3q_gemm_w4_kmajor(one, 1, 64, 100, 64, one, one, null, -1, null, one, one, 1 << 20, null) == -2  # K % 128
    assert lib.k3q_gemm_w4_kmajor(one, 1, 64, 128, 64, one, one, null, 128, null, one, one, 1 << 20, null) == -1  # zero missing
    assert lib.k3q_gemm_w4_kmajor(one, 1, 64, 128, 64, one, one, null, -1, null, one, null, 0, null) == -5
    assert lib.k3q_gemm_w4_kmajor_workspace_bytes(64, 4096, 4096, 128) > 0
    assert lib.k3q_gemm_w4_kmajor_workspace_bytes(8, 4096, 4096, 128) == 0
    assert lib.k3q_gemv_w4_multi(one, 1, 1, 64, -1, one, -1, null, 0, null, 0, null) == -2
    assert lib.k3q_gemv_w4_multi(one, 1, 1, 64, 2, null, -1, null, 0, null, 0, null) == -1
    assert lib.k3q_gemv_w4_multi(one, 1, 1, 64, 0, null, -1, null, 0, null, 0, null) == 0
    assert lib.k3q_gemv_w4_multi(one, 1, 1, 64, 17, one, -1, null, 0, null, 0, null) == -2
    assert lib.k3q_gemm_wbf16(one, 1, one, 3, 4, 8, 64, null, one, null, 0, null) == -2  # bf16 x takes parts == 1
    assert lib.k3q_gemm_wbf16(one, 0, one, 1, 4, 8, 64, null, one, null, 0, null) == -2  # f32 x takes parts 2 | 3
    assert lib.k3q_gemm_wbf16(one, 5, one, 1, 4, 8, 64, null, one, null, 0, null) == -4
    assert lib.k3q_gemm_wbf16(one, 1, null, 1, 4, 8, 64, null, one, null, 0, null) == -1
    assert lib.k3q_gemm_wbf16(one, 1, one, 1, 0, 8, 64, null, one, null, 0, null) == 0
    assert lib.k3q_gemm_wbf16_workspace_bytes(4, 256, 512, 3) >= 4 * 3 * 512 * 2
    assert lib.k3q_gemm_wbf16_workspace_bytes(4, 256, 512, 4) == 0
    assert lib.k3q_gemm_i8_workspace_bytes(4096, 256, 128) == 256 * 128  # room for the [N,K] copy
    assert lib.k3q_gemm_i8_workspace_bytes(1, 8192, 8192) >= 8192 * 4  # decode size: split-K partials
    assert lib.k3q_gemm_i8_workspace_bytes(16, 0, 128) == 0


def test_error_codes_become_python_exceptions():
    with pytest.raises(ValueError):
        _lib.check(-2, "x")
    with pytest.raises(TypeError):
        _lib.check(-4, "x")
    with pytest.raises(RuntimeError):
        _lib.check(-6, "x")
    _lib.check(0, "x")
