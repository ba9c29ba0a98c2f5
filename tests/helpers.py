"""Shared helpers for the parity tests."""

import ctypes
import os

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
ORACLE_SO = os.path.join(ROOT, "oracle", "libk3q_oracle.so")

# tolerances stated by the task: float outputs within 1e-3 (bf16: 1e-2) max relative error
RTOL = {torch.float32: 1e-3, torch.bfloat16: 1e-2}


def max_rel_err(got, want):
    """max |got - want| / max |want|  (relative to the largest reference magnitude)."""
    got = got.detach().double().cpu()
    want = want.detach().double().cpu()
    denom = want.abs().max().clamp_min(1e-30)
    return ((got - want).abs().max() / denom).item()


def max_elem_rel_err(got, want, floor_frac=1e-2):
    """element-wise |got - want| / max(|want|, floor) with floor = floor_frac * rms(want)."""
    got = got.detach().double().cpu()
    want = want.detach().double().cpu()
    floor = floor_frac * want.pow(2).mean().sqrt().clamp_min(1e-30)
    return ((got - want).abs() / want.abs().clamp_min(floor)).max().item()


def assert_close(got, want, dtype, what=""):
    tol = RTOL[dtype]
    e = max_rel_err(got, want)
    assert e <= tol, f"{what}: max relative error {e:.3e} > {tol:.0e}"
    return e


_oracle = None


def c_oracle():
    """The C restatement (oracle/k3q_oracle.c), built by oracle/Makefile."""
    global _oracle
    if _oracle is None:
        if not os.path.exists(ORACLE_SO):
            import subprocess

            subprocess.check_call(["make", "-C", os.path.join(ROOT, "oracle")])
        lib = ctypes.CDLL(ORACLE_SO)
        i64, vp, ci, cf = ctypes.c_int64, ctypes.c_void_p, ctypes.c_int, ctypes.c_float
        lib.k3q_oracle_absmax_quantize.argtypes = [vp, ci, i64, i64, cf, cf, cf, vp, vp]
        lib.k3q_oracle_pack_int4.argtypes = [vp, i64, i64, i64, vp]
        lib.k3q_oracle_unpack_int4.argtypes = [vp, i64, i64, i64, i64, ci, vp]
        lib.k3q_oracle_gemm_i8.argtypes = [vp, vp, i64, i64, i64, vp]
        lib.k3q_oracle_descale.argtypes = [vp, i64, i64, ci, vp, vp, vp, vp]
        lib.k3q_oracle_w4_matmul_f64.argtypes = [vp, i64, i64, i64, vp, vp, vp, i64, vp, vp]
        for f in ("absmax_quantize", "pack_int4", "unpack_int4", "gemm_i8", "descale",
                  "w4_matmul_f64"):
            getattr(lib, "k3q_oracle_" + f).restype = None
        _oracle = lib
    return _oracle


def c_gemm_i8(a, b):
    """int8 [M,K] x int8 [K,N] -> int32 [M,N] on the CPU (C oracle, OpenMP)."""
    a = a.contiguous()
    b = b.contiguous()
    M, K = a.shape
    N = b.shape[1]
    c = torch.empty((M, N), dtype=torch.int32)
    c_oracle().k3q_oracle_gemm_i8(a.data_ptr(), b.data_ptr(), M, N, K, c.data_ptr())
    return c


def c_w4_matmul_f64(x, w_packed, scale, zero, block_size, bias, N):
    """Exact-ish (float64) value of the int4 weight-only matmul."""
    x = x.float().contiguous()
    M, K = x.shape
    wp = w_packed.contiguous()
    sc = scale.float().contiguous()
    zp = zero.contiguous() if zero is not None else None
    bs = bias.float().contiguous() if bias is not None else None
    y = torch.empty((M, N), dtype=torch.float64)
    c_oracle().k3q_oracle_w4_matmul_f64(
        x.data_ptr(), M, K, N, wp.data_ptr(), sc.data_ptr(),
        zp.data_ptr() if zp is not None else None,
        block_size if block_size and block_size > 0 else -1,
        bs.data_ptr() if bs is not None else None, y.data_ptr())
    return y
