"""ctypes binding of libk3q.so (the C ABI declared in include/k3q.h).

The library is the product: there is no CPU or eager-torch fallback.  If the
shared object is missing, or a tensor is not on a HIP device, the call raises.
"""

import ctypes
import os

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libk3q.so")

K3Q_F32 = 0
K3Q_BF16 = 1
K3Q_I32 = 2
K3Q_I64 = 3

_ERRORS = {
    -1: ValueError,
    -2: ValueError,
    -3: ValueError,
    -4: TypeError,
    -5: ValueError,
    -6: RuntimeError,
    -7: ValueError,
}

_i64 = ctypes.c_int64
_int = ctypes.c_int
_f32 = ctypes.c_float
_ptr = ctypes.c_void_p

# name -> (restype, argtypes); must list every symbol include/k3q.h declares
SIGNATURES = {
    "k3q_version": (_int, []),
    "k3q_error_string": (ctypes.c_char_p, [_int]),
    "k3q_absmax_quantize": (
        _int,
        [_ptr, _int, _i64, _i64, _i64, _f32, _f32, _f32, _ptr, _ptr, _ptr],
    ),
    "k3q_weight_absmax_quantize": (
        _int, [_ptr, _int, _i64, _i64, _i64, _f32, _f32, _f32, _ptr, _ptr, _ptr, _ptr]),
    "k3q_weight_quantize_grouped": (
        _int, [_ptr, _int, _i64, _i64, _i64, _f32, _f32, _f32, _ptr, _ptr, _ptr, _ptr]),
    "k3q_pack_int4": (_int, [_ptr, _i64, _i64, _i64, _ptr, _ptr]),
    "k3q_unpack_int4": (_int, [_ptr, _i64, _i64, _i64, _i64, _int, _ptr, _ptr]),
    "k3q_gemm_i8_workspace_bytes": (_i64, [_i64, _i64, _i64]),
    "k3q_prepack_kernel_i8": (_int, [_ptr, _i64, _i64, _ptr, _ptr]),
    "k3q_gemm_i8": (
        _int,
        [_ptr, _ptr, _int, _i64, _i64, _i64, _ptr, _ptr, _ptr, _int, _int, _ptr, _ptr, _ptr,
         _i64, _ptr],
    ),
    "k3q_gemm_i8_addend": (
        _int,
        [_ptr, _ptr, _i64, _i64, _i64, _ptr, _ptr, _ptr, _int, _int, _ptr, _ptr, _i64, _ptr],
    ),
    "k3q_gemm_w8_workspace_bytes": (_i64, [_i64, _i64, _i64]),
    "k3q_gemm_w8": (
        _int,
        [_ptr, _int, _ptr, _int, _i64, _i64, _i64, _ptr, _ptr, _ptr, _ptr, _i64, _ptr],
    ),
    "k3q_gemm_wbf16_workspace_bytes": (_i64, [_i64, _i64, _i64, _int]),
    "k3q_gemm_wbf16": (
        _int,
        [_ptr, _int, _ptr, _int, _i64, _i64, _i64, _ptr, _ptr, _ptr, _i64, _ptr],
    ),
    "k3q_gemv_w4_nk": (
        _int,
        [_ptr, _int, _i64, _i64, _i64, _ptr, _ptr, _int, _ptr, _i64, _ptr, _ptr],
    ),
    "k3q_embedding_lookup": (
        _int,
        [_ptr, _int, _i64, _ptr, _i64, _i64, _int, _ptr, _int, _ptr, _i64, _int, _ptr, _ptr, _ptr],
    ),
    "k3q_gemv_w4_workspace_bytes": (_i64, [_i64, _i64, _i64]),
    "k3q_gemv_w4": (
        _int,
        [_ptr, _int, _i64, _i64, _i64, _ptr, _ptr, _ptr, _i64, _ptr, _ptr, _ptr, _i64, _ptr],
    ),
    "k3q_gemv_w4_counters_bytes": (_i64, [_i64]),
    "k3q_gemv_w4_fused": (
        _int,
        [_ptr, _int, _i64, _i64, _i64, _ptr, _ptr, _ptr, _i64, _ptr, _ptr, _ptr, _i64, _ptr, _i64,
         _ptr],
    ),
    "k3q_gemv_w4_addend": (
        _int,
        [_ptr, _int, _i64, _i64, _i64, _ptr, _ptr, _ptr, _i64, _ptr, _ptr, _ptr, _i64, _ptr, _i64,
         _ptr],
    ),
    "k3q_gemv_w4_static_max_bytes": (_i64, []),
    "k3q_gemv_w4_static": (
        _int,
        [_ptr, _int, _i64, _i64, _i64, _ptr, _ptr, _ptr, _i64, _ptr, _ptr, _ptr],
    ),
    "k3q_w4s_shadow_bytes": (_i64, [_i64, _i64]),
    "k3q_w4s_params_bytes": (_i64, [_i64, _i64, _i64]),
    "k3q_w4s_pack": (_int, [_ptr, _i64, _i64, _ptr, _ptr]),
    "k3q_w4s_pack_params": (_int, [_ptr, _int, _ptr, _i64, _i64, _i64, _ptr, _ptr]),
    "k3q_gemv_w4s_supported": (_int, [_i64, _i64, _i64, _i64]),
    "k3q_gemv_w4s": (
        _int,
        [_ptr, _int, _i64, _i64, _i64, _ptr, _ptr, _ptr, _i64, _ptr, _i64, _ptr, _ptr],
    ),
    "k3q_gemv_w4s_multi": (_int, [_ptr, _int, _i64, _i64, _int, _ptr, _i64, _ptr]),
    "k3q_gemv_w4s_pre": (_int, [_ptr, _int, _i64, _i64, _ptr, _int, _ptr, _i64, _int, _ptr]),
    "k3q_w4_kmajor_pack": (_int, [_ptr, _i64, _i64, _ptr, _ptr]),
    "k3q_w8s_shadow_bytes": (_i64, [_i64, _i64]),
    "k3q_w8s_pack": (_int, [_ptr, _i64, _i64, _ptr, _ptr]),
    "k3q_dense_i8_w8s_supported": (_int, [_i64, _i64, _i64]),
    "k3q_dense_i8_w8s": (
        _int,
        [_ptr, _int, _i64, _i64, _i64, _ptr, _ptr, _ptr, _i64, _f32, _f32, _f32, _ptr, _ptr],
    ),
    "k3q_gemm_i8_w8s": (_int, [_ptr, _ptr, _int, _i64, _i64, _i64, _ptr, _ptr, _ptr, _i64, _ptr, _ptr]),
    "k3q_dense_i8_w8s_multi": (
        _int, [_ptr, _int, _ptr, _ptr, _i64, _i64, _int, _ptr, _f32, _f32, _f32, _ptr]),
    "k3q_dense_i8_w8s_pre": (
        _int, [_ptr, _int, _i64, _i64, _ptr, _int, _ptr, _f32, _f32, _f32, _int, _ptr]),
    "k3q_input_op_quantize": (
        _int, [_ptr, _int, _i64, _i64, _ptr, _f32, _f32, _f32, _ptr, _ptr, _ptr, _ptr]),
    "k3q_rmsnorm": (_int, [_ptr, _ptr, _int, _i64, _i64, _i64, _f32, _ptr, _i64, _ptr]),
    "k3q_silu_mul": (_int, [_ptr, _ptr, _int, _i64, _i64, _i64, _i64, _ptr, _i64, _ptr]),
    "k3q_decode_attention": (
        _int,
        [_ptr, _ptr, _ptr, _int, _i64, _i64, _i64, _i64, _ptr, _ptr, _ptr, _ptr, _ptr, _ptr, _ptr, _ptr],
    ),
    "k3q_gemm_w4_kmajor_workspace_bytes": (_i64, [_i64, _i64, _i64, _i64]),
    "k3q_gemm_w4_kmajor": (
        _int,
        [_ptr, _int, _i64, _i64, _i64, _ptr, _ptr, _ptr, _i64, _ptr, _ptr, _ptr, _i64, _ptr],
    ),
    "k3q_gemm_w4_strip": (
        _int,
        [_ptr, _int, _i64, _i64, _i64, _ptr, _ptr, _ptr, _i64, _ptr, _ptr, _ptr, _i64, _ptr],
    ),
    "k3q_gemv_w4_multi": (
        _int,
        [_ptr, _int, _i64, _i64, _int, _ptr, _i64, _ptr, _i64, _ptr, _i64, _ptr],
    ),
}

# test hooks (keras_amd/csrc/k3q_testing.h): exported by the library, not part of the C ABI
TEST_SIGNATURES = {
    "k3qt_gemv_w4_plan": (
        _int,
        [_ptr, _int, _i64, _i64, _i64, _ptr, _ptr, _ptr, _i64, _ptr, _ptr, _ptr, _i64, _ptr, _i64,
         _ptr, _ptr],
    ),
}


class GemvW4Problem(ctypes.Structure):
    """`k3q_gemv_w4_problem` of include/k3q.h."""

    _fields_ = [("N", ctypes.c_int64), ("w_packed", ctypes.c_void_p), ("scale", ctypes.c_void_p),
                ("zero", ctypes.c_void_p), ("bias", ctypes.c_void_p), ("y", ctypes.c_void_p)]


class GemvW4sProblem(ctypes.Structure):
    """`k3q_gemv_w4s_problem` of include/k3q.h."""

    _fields_ = [("N", ctypes.c_int64), ("shadow", ctypes.c_void_p), ("scale", ctypes.c_void_p),
                ("gparams", ctypes.c_void_p), ("bias", ctypes.c_void_p), ("y", ctypes.c_void_p)]


class InputOp(ctypes.Structure):
    """`k3q_input_op` of include/k3q.h."""

    _fields_ = [("kind", ctypes.c_int), ("epsilon", ctypes.c_float), ("operand", ctypes.c_void_p)]


K3Q_INPUT_RMS_NORM = 1
K3Q_INPUT_SILU_GATE = 2


class W8sProblem(ctypes.Structure):
    """`k3q_w8s_problem` of include/k3q.h."""

    _fields_ = [("N", ctypes.c_int64), ("shadow", ctypes.c_void_p), ("kernel_scale", ctypes.c_void_p),
                ("bias", ctypes.c_void_p), ("y", ctypes.c_void_p)]


_lib = None


def load():
    """Load libk3q.so once; raise if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            f"{LIB_PATH} is missing: build it with `python -m keras_amd.csrc.build` "
            "(the quantized path has no fallback implementation)"
        )
    lib = ctypes.CDLL(LIB_PATH)
    for name, (res, args) in list(SIGNATURES.items()) + list(TEST_SIGNATURES.items()):
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


def check(code, what):
    if code == 0:
        return
    text = load().k3q_error_string(code).decode()
    raise _ERRORS.get(code, RuntimeError)(f"{what}: {text} (k3q code {code})")


def dtype_code(dtype):
    if dtype == torch.float32:
        return K3Q_F32
    if dtype == torch.bfloat16:
        return K3Q_BF16
    raise TypeError(
        f"the k3q kernels take float32 or bfloat16 tensors, got {dtype}"
    )


def require_device(*tensors):
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise RuntimeError(
                "k3q kernels run on a HIP device only; got a tensor on "
                f"'{t.device}' (there is no CPU fallback)"
            )


def stream_ptr(device=None):
    return ctypes.c_void_p(torch.cuda.current_stream(device).cuda_stream)


def ptr(t):
    return ctypes.c_void_p(t.data_ptr()) if t is not None else ctypes.c_void_p(0)
