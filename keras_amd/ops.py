"""Tensor-level entry points of the quantized forward (thin wrappers over the C ABI).

These are the calls a `_int8_call` / `_int4_call` makes: they take and return
torch tensors that live on the HIP device, run on torch's current stream and
allocate only outputs (plus one cached, zero-initialised scratch buffer per
device and stream for the split-K kernels).
"""

import ctypes
import threading

import torch

from keras_amd import _lib

_workspaces = {}
_scratch_lock = threading.Lock()


def _workspace(device, nbytes):
    """Scratch for split-K partial sums and the per-call [N, K] weight copy.

    One buffer per (device, stream, host thread): the calls one thread makes on one stream are
    ordered, so they can share it; calls on different streams may overlap, and two threads on
    one stream may interleave the launches of a two-kernel call, so neither shares.
    """
    stream = torch.cuda.current_stream(device)
    key = (device.index, stream.cuda_stream, threading.get_ident())
    with _scratch_lock:
        ws = _workspaces.get(key)
        if ws is None or ws.numel() < nbytes:
            # A captured HIP graph keeps the address of the buffer its kernels were recorded with:
            # an outgrown buffer is retired, never freed (sizes at least double, so the retired
            # ones together stay below the live one).
            if ws is not None:
                _retired.append(ws)
            size = max(int(nbytes), 1 << 20, 2 * (ws.numel() if ws is not None else 0))
            ws = torch.zeros(size, dtype=torch.uint8, device=device)
            _workspaces[key] = ws
    return ws


_retired = []


_counters = {}


def _arrival_counters(device, nbytes):
    """Arrival counters of the single-launch K split: zero between calls, one set per
    (device, stream, host thread), like the workspace they go with."""
    stream = torch.cuda.current_stream(device)
    key = (device.index, stream.cuda_stream, threading.get_ident())
    with _scratch_lock:
        c = _counters.get(key)
        if c is None or c.numel() < nbytes:
            if c is not None:
                _retired.append(c)  # a captured graph may still count in it
            c = torch.zeros(max(int(nbytes), 1 << 16), dtype=torch.uint8, device=device)
            _counters[key] = c
    return c


INT4_ADDEND_MAX_ROWS = 64


def _check_bias_size(bias, M, N):
    """A bias is N values, or M x N (a row per row of the input: an addend).  Checked before
    anything is launched: the kernels read bias[0 .. N) or [0 .. M * N) unconditionally."""
    if bias is not None and bias.numel() != N and bias.numel() != M * N:
        raise ValueError(f"bias holds {bias.numel()} values; the output is [{M}, {N}]: "
                         f"expected {N} (one row) or {M * N} (a row per input row)")


def int4_matmul(x, kernel_packed, kernel_scale, orig_output_dim, kernel_zero=None,
                block_size=None, bias=None, plan=None, single_launch=True, addend=None):
    """`x[..., K] . W4[K, N]` for a Dense int4 kernel as the layer stores it.

    kernel_packed: int8 [K, ceil(N/2)] (two nibbles per byte along N).
    kernel_scale:  [N] (per-channel, `block_size` None or -1) or [G, N].
    kernel_zero:   int8 [G, N] for grouped quantisation.
    Scales and bias must already be in x.dtype (the layer reads its float
    variables in the compute dtype).  Returns x.dtype [..., N].
    Reference: keras/src/layers/core/dense.py:988-1095.
    """
    _lib.require_device(x, kernel_packed, kernel_scale, kernel_zero, bias)
    code = _lib.dtype_code(x.dtype)
    K = kernel_packed.shape[0]
    N = int(orig_output_dim)
    if x.shape[-1] != K:
        raise ValueError(
            f"last axis of the input ({x.shape[-1]}) does not match the kernel's input dim ({K})"
        )
    if kernel_packed.dtype != torch.int8 or kernel_packed.shape[1] != (N + 1) // 2:
        raise ValueError("kernel must be int8 of shape [input_dim, ceil(units / 2)]")
    grouped = block_size is not None and block_size > 0
    if kernel_scale.dtype != x.dtype or (bias is not None and bias.dtype != x.dtype):
        raise TypeError("kernel_scale and bias must be read in the input's dtype")
    lead = x.shape[:-1]
    x2 = x.reshape(-1, K)
    if not x2.is_contiguous():
        x2 = x2.contiguous()
    M = x2.shape[0]
    _check_bias_size(bias, M, N)
    kp = kernel_packed if kernel_packed.is_contiguous() else kernel_packed.contiguous()
    ks = kernel_scale if kernel_scale.is_contiguous() else kernel_scale.contiguous()
    kz = None
    if grouped:
        if kernel_zero is None:
            raise ValueError("grouped int4 needs kernel_zero")
        kz = kernel_zero if kernel_zero.is_contiguous() else kernel_zero.contiguous()
    y = torch.empty((M, N), dtype=x.dtype, device=x.device)
    lib = _lib.load()
    nbytes = lib.k3q_gemv_w4_workspace_bytes(M, K, N)
    if plan is not None:
        # an overridden plan may split K into many more workgroups than the built-in one
        nbytes = max(nbytes, (K // 16 + 1) * min(M, 16) * N * 4)
    ws = _workspace(x.device, nbytes)
    args = [
        _lib.ptr(x2), code, M, K, N, _lib.ptr(kp), _lib.ptr(ks), _lib.ptr(kz),
        int(block_size) if grouped else -1, _lib.ptr(bias), _lib.ptr(y),
        _lib.ptr(ws), ws.numel(),
    ]
    cnt = _arrival_counters(x.device, lib.k3q_gemv_w4_counters_bytes(N)) if single_launch else None
    args += [_lib.ptr(cnt), cnt.numel() if single_launch else 0]
    if addend is None and bias is not None and M > 1 and bias.numel() == M * N:
        addend, bias = bias, None  # a bias with a row per row of x is an addend
    if addend is not None:
        # [M, N] rows added to the rounded product the way a bias is (a residual), decode sizes
        if bias is not None or plan is not None or M > INT4_ADDEND_MAX_ROWS:
            raise ValueError("addend: at most %d rows, no bias, no plan" % INT4_ADDEND_MAX_ROWS)
        _lib.require_device(addend)
        if addend.dtype != x.dtype or addend.numel() != M * N:
            raise ValueError("addend must hold M x N values of the input's dtype")
        ad = addend.reshape(M, N)
        args[9] = _lib.ptr(ad if ad.is_contiguous() else ad.contiguous())
        rc = lib.k3q_gemv_w4_addend(*args, _lib.stream_ptr(x.device))
    elif plan is None:
        rc = lib.k3q_gemv_w4_fused(*args, _lib.stream_ptr(x.device))
    else:
        arr = (ctypes.c_int * 4)(*[int(v) for v in plan[:4]])
        rc = lib.k3qt_gemv_w4_plan(*args, arr, _lib.stream_ptr(x.device))
    _lib.check(rc, "k3q_gemv_w4")
    return y.reshape(*lead, N)


def int4_matmul_multi(x, kernels, block_size=None):
    """`[x . W_i for W_i in kernels]` for int4 Dense kernels that share the input `x[..., K]`:
    one launch when the calls are decode-sized and the kernels' launch plans agree (kernels of
    one shape do), otherwise one launch each; the same bits as `int4_matmul` either way.

    kernels: dicts with `kernel_packed` int8 [K, ceil(N/2)], `kernel_scale` ([N] or [G, N], in
    x.dtype), `units` (N), and optionally `kernel_zero` int8 [G, N] (grouped) and `bias` [N].
    Reference: each is keras/src/layers/core/dense.py:988-1095; calling several layers on one
    input in one launch has no counterpart there.
    """
    grouped = block_size is not None and block_size > 0
    code = _lib.dtype_code(x.dtype)
    K = x.shape[-1]
    lead = x.shape[:-1]
    x2 = x.reshape(-1, K)
    if not x2.is_contiguous():
        x2 = x2.contiguous()
    M = x2.shape[0]
    lib = _lib.load()
    problems = (_lib.GemvW4Problem * len(kernels))()
    outs, keep = [], []
    ws_bytes = cnt_bytes = 0
    for i, k in enumerate(kernels):
        kp, ks = k["kernel_packed"], k["kernel_scale"]
        kz, bias = k.get("kernel_zero"), k.get("bias")
        N = int(k["units"])
        _lib.require_device(x, kp, ks, kz, bias)
        if kp.dtype != torch.int8 or kp.shape[0] != K or kp.shape[1] != (N + 1) // 2:
            raise ValueError("kernel must be int8 of shape [input_dim, ceil(units / 2)]")
        if ks.dtype != x.dtype or (bias is not None and bias.dtype != x.dtype):
            raise TypeError("kernel_scale and bias must be read in the input's dtype")
        if grouped and kz is None:
            raise ValueError("grouped int4 needs kernel_zero")
        if bias is not None and bias.numel() != N:
            raise ValueError(f"bias holds {bias.numel()} values, the layer has {N} units")
        kp = kp if kp.is_contiguous() else kp.contiguous()
        ks = ks if ks.is_contiguous() else ks.contiguous()
        if kz is not None and not kz.is_contiguous():
            kz = kz.contiguous()
        y = torch.empty((M, N), dtype=x.dtype, device=x.device)
        keep.append((kp, ks, kz, bias))
        outs.append(y)
        problems[i] = _lib.GemvW4Problem(
            N, kp.data_ptr(), ks.data_ptr(), kz.data_ptr() if grouped else None,
            bias.data_ptr() if bias is not None else None, y.data_ptr())
        ws_bytes += (lib.k3q_gemv_w4_workspace_bytes(M, K, N) + 255) // 256 * 256
        cnt_bytes += lib.k3q_gemv_w4_counters_bytes(N)
    ws = _workspace(x.device, ws_bytes)
    cnt = _arrival_counters(x.device, cnt_bytes)
    rc = lib.k3q_gemv_w4_multi(_lib.ptr(x2), code, M, K, len(kernels), ctypes.byref(problems),
                               int(block_size) if grouped else -1, _lib.ptr(ws), ws.numel(),
                               _lib.ptr(cnt), cnt.numel(), _lib.stream_ptr(x.device))
    _lib.check(rc, "k3q_gemv_w4_multi")
    return [y.reshape(*lead, y.shape[1]) for y in outs]


STRIP_MAX_ROWS = 16


def int4_strip_supported(M, K, N, block_size=None):
    """Whether `int4_matmul_strip` takes M bfloat16 rows against a [K, N] int4 kernel."""
    bs = int(block_size) if block_size is not None and block_size > 0 else -1
    return bool(_lib.load().k3q_gemv_w4s_supported(int(M), int(K), int(N), bs))


def int4_strip_copy(kernel_packed, units):
    """The strip-linear copy of an int4 kernel that `int4_matmul_strip` streams (layout:
    include/k3q.h, k3q_gemv_w4s).  Made once per layer from the stored `[K, ceil(N/2)]` kernel
    by a device kernel; the same number of bytes as the kernel (an odd strip count is padded)."""
    _lib.require_device(kernel_packed)
    K, N = kernel_packed.shape[0], int(units)
    if kernel_packed.dtype != torch.int8 or kernel_packed.shape[1] != (N + 1) // 2:
        raise ValueError("kernel must be int8 of shape [input_dim, ceil(units / 2)]")
    lib = _lib.load()
    nbytes = lib.k3q_w4s_shadow_bytes(K, N)
    if nbytes <= 0:
        raise ValueError("the strip-linear copy needs K % 128 == 0")
    kp = kernel_packed if kernel_packed.is_contiguous() else kernel_packed.contiguous()
    out = torch.empty(nbytes, dtype=torch.uint8, device=kp.device)
    _lib.check(lib.k3q_w4s_pack(_lib.ptr(kp), K, N, _lib.ptr(out), _lib.stream_ptr(kp.device)), "k3q_w4s_pack")
    return out


def int4_strip_params(kernel_scale, kernel_zero, K, units, block_size):
    """Scales and zero points of a grouped (block 128) int4 kernel in the order the strip kernel
    reads them: per (strip, group) four records of four bfloat16 scales and four `zero + 128` bytes."""
    _lib.require_device(kernel_scale, kernel_zero)
    lib = _lib.load()
    N = int(units)
    nbytes = lib.k3q_w4s_params_bytes(int(K), N, int(block_size))
    if nbytes <= 0:
        raise ValueError("strip parameters: groups of 128 and K % 128 == 0 only")
    sc = kernel_scale if kernel_scale.is_contiguous() else kernel_scale.contiguous()
    zp = kernel_zero if kernel_zero.is_contiguous() else kernel_zero.contiguous()
    if tuple(sc.shape) != (K // 128, N) or tuple(zp.shape) != (K // 128, N) or zp.dtype != torch.int8:
        raise ValueError("scale / zero must be [K / 128, N], zero int8")
    out = torch.empty(nbytes, dtype=torch.uint8, device=sc.device)
    rc = lib.k3q_w4s_pack_params(_lib.ptr(sc), _lib.dtype_code(sc.dtype), _lib.ptr(zp), int(K), N,
                                 int(block_size), _lib.ptr(out), _lib.stream_ptr(sc.device))
    _lib.check(rc, "k3q_w4s_pack_params")
    return out


def int4_matmul_strip(x, shadow, units, kernel_scale=None, gparams=None, block_size=None, bias=None,
                      addend=None):
    """`x[..., K] . W4[K, N]` for up to 16 bfloat16 rows from `int4_strip_copy(kernel)`: one launch,
    no scratch.  Per-channel: `kernel_scale` bfloat16 [N]; grouped (block 128): `gparams` from
    `int4_strip_params`.  `bias` [N], or `addend` [M, N] added the way a bias is.
    Reference: keras/src/layers/core/dense.py:988-1095."""
    _lib.require_device(x, shadow, kernel_scale, gparams, bias, addend)
    if x.dtype != torch.bfloat16:
        raise TypeError("the strip route computes in bfloat16")
    grouped = block_size is not None and block_size > 0
    N = int(units)
    K = x.shape[-1]
    lead = x.shape[:-1]
    x2 = x.reshape(-1, K)
    x2 = x2 if x2.is_contiguous() else x2.contiguous()
    M = x2.shape[0]
    lib = _lib.load()
    if shadow.numel() != lib.k3q_w4s_shadow_bytes(K, N):
        raise ValueError("the strip-linear copy does not belong to a [%d, %d] kernel" % (K, N))
    stride = 0
    b = bias
    if addend is not None:
        if bias is not None:
            raise ValueError("addend and bias exclude each other")
        if addend.numel() != M * N:
            raise ValueError(f"addend holds {addend.numel()} values; the output is [{M}, {N}]")
        b = addend.reshape(M, N)
        b = b if b.is_contiguous() else b.contiguous()
        stride = N
    elif bias is not None and bias.numel() != N:
        raise ValueError(f"bias holds {bias.numel()} values, the layer has {N} units")
    if b is not None and b.dtype != torch.bfloat16:
        raise TypeError("bias must be read in the input's dtype")
    if grouped:
        if gparams is None or gparams.numel() != lib.k3q_w4s_params_bytes(K, N, int(block_size)):
            raise ValueError("grouped int4 needs the strip parameters of this kernel")
    elif kernel_scale is None or kernel_scale.dtype != torch.bfloat16 or kernel_scale.numel() != N:
        raise ValueError("per-channel int4 needs bfloat16 scales [N]")
    y = torch.empty((M, N), dtype=x.dtype, device=x.device)
    rc = lib.k3q_gemv_w4s(_lib.ptr(x2), _lib.K3Q_BF16, M, K, N, _lib.ptr(shadow),
                          None if grouped else _lib.ptr(kernel_scale), _lib.ptr(gparams) if grouped else None,
                          int(block_size) if grouped else -1, _lib.ptr(b), stride, _lib.ptr(y),
                          _lib.stream_ptr(x.device))
    _lib.check(rc, "k3q_gemv_w4s")
    return y.reshape(*lead, N)


def int4_matmul_strip_multi(x, kernels, block_size=None, input_op=None, bias_rows=False):
    """`[op(x) . W_i]` for kernels that share `x[..., K]` (up to 16 bfloat16 rows): one launch for those
    whose launch plans agree.  kernels: dicts with `shadow`, `units`, `kernel_scale` (per-channel)
    or `gparams` (grouped), and optionally `bias` [N] (bias_rows: [M, N], a row per row of x).
    input_op: None, `("rms_norm", gain, epsilon)` or `("silu_gate", gate)`, applied to the rows inside
    the kernel (`int4_strip_input_op_supported`), with the bits of `rmsnorm` / `silu_mul`."""
    grouped = block_size is not None and block_size > 0
    K = x.shape[-1]
    lead = x.shape[:-1]
    x2 = x.reshape(-1, K)
    x2 = x2 if x2.is_contiguous() else x2.contiguous()
    M = x2.shape[0]
    lib = _lib.load()
    problems = (_lib.GemvW4sProblem * len(kernels))()
    outs = []
    for i, k in enumerate(kernels):
        N = int(k["units"])
        bias = k.get("bias")
        _lib.require_device(x, k["shadow"], k.get("kernel_scale"), k.get("gparams"), bias)
        want = M * N if bias_rows else N
        if bias is not None and (bias.numel() != want or bias.dtype != torch.bfloat16 or not bias.is_contiguous()):
            raise ValueError(f"bias must hold {want} bfloat16 values, contiguous")
        if k["shadow"].numel() != lib.k3q_w4s_shadow_bytes(K, N):
            raise ValueError("the strip-linear copy does not belong to a [%d, %d] kernel" % (K, N))
        y = torch.empty((M, N), dtype=x.dtype, device=x.device)
        outs.append(y)
        problems[i] = _lib.GemvW4sProblem(
            N, k["shadow"].data_ptr(), None if grouped else k["kernel_scale"].data_ptr(),
            k["gparams"].data_ptr() if grouped else None,
            bias.data_ptr() if bias is not None else None, y.data_ptr())
    if input_op is None and not bias_rows:
        rc = lib.k3q_gemv_w4s_multi(_lib.ptr(x2), _lib.K3Q_BF16, M, K, len(kernels), ctypes.byref(problems),
                                    int(block_size) if grouped else -1, _lib.stream_ptr(x.device))
        _lib.check(rc, "k3q_gemv_w4s_multi")
    else:
        pre, keep = _input_op_struct(input_op, M, K, x.device)
        rc = lib.k3q_gemv_w4s_pre(_lib.ptr(x2), _lib.K3Q_BF16, M, K, ctypes.byref(pre) if pre is not None else None,
                                  len(kernels), ctypes.byref(problems), int(block_size) if grouped else -1,
                                  1 if bias_rows else 0, _lib.stream_ptr(x.device))
        _lib.check(rc, "k3q_gemv_w4s_pre")
        del keep
    return [y.reshape(*lead, y.shape[1]) for y in outs]


# rows up to which the gate silu(g) * u is recomputed by every workgroup of a decode matmul (an exp
# and a reciprocal per value: beyond, the separate launch is cheaper)
STRIP_SILU_MAX_ROWS = 2


def _input_op_struct(input_op, M, K, device):
    """`k3q_input_op` for `("rms_norm", gain, epsilon)` / `("silu_gate", gate)`; also returns the
    tensors that must stay alive across the call."""
    if input_op is None:
        return None, None
    kind = input_op[0]
    if kind == "rms_norm":
        gain, eps = input_op[1], float(input_op[2])
        _lib.require_device(gain)
        if gain.dtype != torch.bfloat16 or gain.numel() != K:
            raise ValueError(f"the gain must hold {K} bfloat16 values")
        gain = gain if gain.is_contiguous() else gain.contiguous()
        return _lib.InputOp(_lib.K3Q_INPUT_RMS_NORM, eps, gain.data_ptr()), gain
    if kind == "silu_gate":
        gate = input_op[1]
        _lib.require_device(gate)
        if gate.dtype != torch.bfloat16 or gate.numel() != M * K:
            raise ValueError(f"the gate must hold {M} x {K} bfloat16 values")
        gate = gate.reshape(M, K)
        gate = gate if gate.is_contiguous() else gate.contiguous()
        return _lib.InputOp(_lib.K3Q_INPUT_SILU_GATE, 0.0, gate.data_ptr()), gate
    raise ValueError(f"unknown input operation {kind!r}")


def apply_input_op(input_op, x):
    """The operation as a launch of its own: `rmsnorm(x, gain, eps)` or `silu_mul(gate, x)`."""
    if input_op is None:
        return x
    if input_op[0] == "rms_norm":
        gain, eps = input_op[1], float(input_op[2])
        if rmsnorm_supported(x, gain):
            return rmsnorm(x, gain, eps)
        return torch.nn.functional.rms_norm(x, (x.shape[-1],), gain, eps)
    if input_op[0] == "silu_gate":
        gate = input_op[1].reshape(x.shape)
        if silu_mul_supported(gate, x):
            return silu_mul(gate, x)
        return torch.nn.functional.silu(gate) * x
    raise ValueError(f"unknown input operation {input_op[0]!r}")


# rows up to which the normalisation is repeated by every workgroup (about ten float operations per
# value: measured at 8 rows of 4096, 4.9 us more in the projections' launch against 4.3 us for the
# launch saved; at one row 0.6 us)
STRIP_RMS_MAX_ROWS = 4


def input_op_quantize_supported(input_op, x2):
    """Whether `input_op_quantize` takes these rows: bfloat16 on the device, dense, rows of whole
    16-byte pieces up to 16384 values."""
    K = x2.shape[-1]
    return (input_op is not None and input_op[0] in ("rms_norm", "silu_gate") and x2.is_cuda
            and x2.dtype == torch.bfloat16 and x2.dim() == 2 and x2.is_contiguous() and K % 8 == 0 and 0 < K <= 16384
            and x2.shape[0] > 0)


def input_op_quantize(input_op, x2, epsilon=1e-7, value_range=(-127, 127)):
    """`h = op(x2)` and `q, scale = abs_max_quantize(h, axis=-1)` in one launch, the bits of the
    separate kernels (`apply_input_op`, `quantizers.abs_max_quantize`).  x2 `[M, K]` bfloat16; returns
    `(h, q, scale)` with scale `[M, 1]` bfloat16."""
    _lib.require_device(x2)
    M, K = (int(d) for d in x2.shape)
    pre, keep = _input_op_struct(input_op, M, K, x2.device)
    h = torch.empty_like(x2)
    q = torch.empty((M, K), dtype=torch.int8, device=x2.device)
    s = torch.empty((M,), dtype=torch.bfloat16, device=x2.device)
    rc = _lib.load().k3q_input_op_quantize(_lib.ptr(x2), _lib.K3Q_BF16, M, K, ctypes.byref(pre), float(epsilon),
                                           float(value_range[0]), float(value_range[1]), _lib.ptr(h), _lib.ptr(q),
                                           _lib.ptr(s), _lib.stream_ptr(x2.device))
    _lib.check(rc, "k3q_input_op_quantize")
    del keep
    return h, q, s.reshape(M, 1)


def _input_op_rows_ok(input_op, M, K):
    if input_op[0] == "rms_norm":
        return K % 512 == 0 and K <= 65536 and M <= STRIP_RMS_MAX_ROWS
    return input_op[0] == "silu_gate" and M <= STRIP_SILU_MAX_ROWS


def int4_strip_input_op_supported(input_op, M, K, N, block_size=None):
    """Whether `int4_matmul_strip_multi` folds this operation into its launch for these sizes: x whole
    in a workgroup's LDS (not staged in halves), whole blocks of 512 for the normalisation, few rows
    for the gate."""
    bs = int(block_size) if block_size is not None and block_size > 0 else -1
    return (_input_op_rows_ok(input_op, M, K) and M * K <= 65536
            and bool(_lib.load().k3q_gemv_w4s_supported(M, K, N, bs)))


def int8_strip_input_op_supported(input_op, M, K, N, value_range=(-127, 127)):
    """The same for `int8_dense_strip_multi`: sizes at which the kernel quantises the rows itself."""
    return (_input_op_rows_ok(input_op, M, K) and int8_strip_quantises_inside(M, K, value_range)
            and bool(_lib.load().k3q_dense_i8_w8s_supported(M, K, N)))


def int4_kmajor_copy(kernel_packed, units):
    """The K-contiguous copy `int4_matmul_kmajor` reads: int32 [N, K/8], eight consecutive k of
    a column per dword, even k in the low half-word's nibbles, odd k in the high half-word's
    (include/k3q.h, k3q_gemm_w4_kmajor).  Made once per layer from the stored
    `[K, ceil(N/2)]` kernel; K % 8 == 0."""
    _lib.require_device(kernel_packed)
    lib = _lib.load()
    K, N = int(kernel_packed.shape[0]), int(units)
    if kernel_packed.dtype != torch.int8 or kernel_packed.dim() != 2 or kernel_packed.shape[1] != (N + 1) // 2:
        raise ValueError(f"expected the stored int8 kernel [K, ceil({N}/2)], got {tuple(kernel_packed.shape)}")
    if K % 8:
        raise ValueError("the K-contiguous copy needs K % 8 == 0")
    src = kernel_packed if kernel_packed.is_contiguous() else kernel_packed.contiguous()
    out = torch.empty((N, K // 8), dtype=torch.int32, device=src.device)
    _lib.check(lib.k3q_w4_kmajor_pack(_lib.ptr(src), K, N, _lib.ptr(out), _lib.stream_ptr(src.device)),
               "k3q_w4_kmajor_pack")
    return out


def int4_kmajor_supported(M, K, N, block_size=None):
    lib = _lib.load()
    bs = int(block_size) if block_size is not None and block_size > 0 else -1
    return lib.k3q_gemm_w4_kmajor_workspace_bytes(M, K, N, bs) > 0


def int4_matmul_kmajor(x, kernel_kmajor, kernel_scale, kernel_zero=None, block_size=None, bias=None):
    """`x[..., K] . W4` for 17 ... 512 bfloat16 rows from `int4_kmajor_copy(kernel)`; the kernel
    is read once, as int4.  Reference: keras/src/layers/core/dense.py:988-1095."""
    _lib.require_device(x, kernel_kmajor, kernel_scale, kernel_zero, bias)
    if x.dtype != torch.bfloat16 or kernel_scale.dtype != torch.bfloat16:
        raise TypeError("the K-contiguous route computes in bfloat16")
    grouped = block_size is not None and block_size > 0
    N, K8 = kernel_kmajor.shape
    K = K8 * 8
    if x.shape[-1] != K:
        raise ValueError(f"last axis of the input ({x.shape[-1]}) does not match the kernel's input dim ({K})")
    lead = x.shape[:-1]
    x2 = x.reshape(-1, K)
    x2 = x2 if x2.is_contiguous() else x2.contiguous()
    M = x2.shape[0]
    if bias is not None and bias.numel() != N:
        raise ValueError(f"bias holds {bias.numel()} values, the layer has {N} units")
    y = torch.empty((M, N), dtype=x.dtype, device=x.device)
    lib = _lib.load()
    bs = int(block_size) if grouped else -1
    nbytes = lib.k3q_gemm_w4_kmajor_workspace_bytes(M, K, N, bs)
    if nbytes <= 0:
        raise ValueError(f"the K-contiguous route does not take M={M}, K={K}, N={N}, block_size={block_size}")
    ws = _workspace(x.device, nbytes)
    ks = kernel_scale if kernel_scale.is_contiguous() else kernel_scale.contiguous()
    rc = lib.k3q_gemm_w4_kmajor(_lib.ptr(x2), _lib.dtype_code(x.dtype), M, K, N, _lib.ptr(kernel_kmajor),
                                _lib.ptr(ks), _lib.ptr(kernel_zero) if grouped else None, bs,
                                _lib.ptr(bias), _lib.ptr(y), _lib.ptr(ws), ws.numel(),
                                _lib.stream_ptr(x.device))
    _lib.check(rc, "k3q_gemm_w4_kmajor")
    return y.reshape(*lead, N)


def int4_tiles_strip_supported(M, K, N, block_size=None):
    """Whether `int4_matmul_tiles_strip` takes M bfloat16 rows against a [K, N] kernel's strip copy."""
    grouped = block_size is not None and block_size > 0
    return (int4_kmajor_supported(M, K, N, block_size) and (not grouped or block_size % 128 == 0)
            and _lib.load().k3q_w4s_shadow_bytes(int(K), int(N)) > 0)


def int4_matmul_tiles_strip(x, shadow, units, kernel_scale, kernel_zero=None, block_size=None, bias=None):
    """`x[..., K] . W4` for 17 ... 512 bfloat16 rows on the int4 tile kernel, reading the SAME
    strip-linear copy (`int4_strip_copy`) that the decode kernel streams: a layer then keeps one derived
    copy of its kernel for every row count up to 512.  kernel_scale `[N]` or `[G, N]` and
    kernel_zero `[G, N]` as stored (bfloat16 scales).  Reference: keras/src/layers/core/dense.py:988-1095."""
    _lib.require_device(x, shadow, kernel_scale, kernel_zero, bias)
    if x.dtype != torch.bfloat16 or kernel_scale.dtype != torch.bfloat16:
        raise TypeError("the int4 tile route computes in bfloat16")
    grouped = block_size is not None and block_size > 0
    N, K = int(units), x.shape[-1]
    lib = _lib.load()
    if shadow.numel() != lib.k3q_w4s_shadow_bytes(K, N):
        raise ValueError("the strip-linear copy does not belong to a [%d, %d] kernel" % (K, N))
    lead = x.shape[:-1]
    x2 = x.reshape(-1, K)
    x2 = x2 if x2.is_contiguous() else x2.contiguous()
    M = x2.shape[0]
    if bias is not None and bias.numel() != N:
        raise ValueError(f"bias holds {bias.numel()} values, the layer has {N} units")
    bs = int(block_size) if grouped else -1
    nbytes = lib.k3q_gemm_w4_kmajor_workspace_bytes(M, K, N, bs)
    if nbytes <= 0 or not int4_tiles_strip_supported(M, K, N, block_size):
        raise ValueError(f"the int4 tile route does not take M={M}, K={K}, N={N}, block_size={block_size}")
    y = torch.empty((M, N), dtype=x.dtype, device=x.device)
    ws = _workspace(x.device, nbytes)
    ks = kernel_scale if kernel_scale.is_contiguous() else kernel_scale.contiguous()
    rc = lib.k3q_gemm_w4_strip(_lib.ptr(x2), _lib.dtype_code(x.dtype), M, K, N, _lib.ptr(shadow),
                               _lib.ptr(ks), _lib.ptr(kernel_zero) if grouped else None, bs,
                               _lib.ptr(bias), _lib.ptr(y), _lib.ptr(ws), ws.numel(),
                               _lib.stream_ptr(x.device))
    _lib.check(rc, "k3q_gemm_w4_strip")
    return y.reshape(*lead, N)


GEMM_EXACT_EPILOGUE = 1
# up to this many rows the int8 matmul streams the [K, N] kernel in place; above, the prepacked
# copy on 128-row MFMA tiles (K split over workgroups while the tiles are few) is faster
# (K = N = 4096, 17..64 rows: 11-13 us against 26-63 us in 16-row passes)
SKINNY_MAX_ROWS = 8


def prepack_int8_kernel(kernel):
    """[K, N] int8 kernel -> the [N, K] shadow copy the MFMA GEMM consumes.

    Made once per layer (the layer's own variable keeps its [K, N] layout).
    """
    _lib.require_device(kernel)
    if kernel.dtype != torch.int8 or kernel.dim() != 2:
        raise TypeError("kernel must be a 2-D int8 tensor")
    k = kernel if kernel.is_contiguous() else kernel.contiguous()
    K, N = k.shape
    out = torch.empty((N, K), dtype=torch.int8, device=k.device)
    rc = _lib.load().k3q_prepack_kernel_i8(_lib.ptr(k), K, N, _lib.ptr(out),
                                           _lib.stream_ptr(k.device))
    _lib.check(rc, "k3q_prepack_kernel_i8")
    return out


def int8_matmul(a, kernel, a_scale=None, kernel_scale=None, bias=None, out_dtype=None,
                prepacked=None, exact_epilogue=False, want_acc=False, want_y=True, strip=None,
                kernel_shape=None):
    """`a[M, K] int8 . kernel[K, N] int8` with the de-scale epilogue fused.

    Returns y (out_dtype [M, N]); with want_acc also the int32 accumulators.
    `prepacked` is the cached result of `prepack_int8_kernel(kernel)`; without it
    the [N, K] copy is rebuilt in scratch memory on every call.  `strip` is the cached
    `int8_strip_copy(kernel)` of the decode kernel: with K % 128 == 0 the tile kernel reads
    that copy instead (the same bits), so a layer need not keep a prepacked one beside it.
    `kernel` may be None when `strip` serves the call (more than 8 rows, K % 128 == 0) and
    `kernel_shape = (K, N)` is given.
    Reference: keras/src/layers/core/dense.py:961-983.
    """
    _lib.require_device(a, kernel, a_scale, kernel_scale, bias, prepacked, strip)
    if a.dtype != torch.int8 or (kernel is not None and kernel.dtype != torch.int8):
        raise TypeError("int8_matmul takes int8 operands")
    M, K = a.shape
    if kernel is None:
        if strip is None or kernel_shape is None or kernel_shape[0] != K or K % 128 or M <= SKINNY_MAX_ROWS:
            raise ValueError("without the stored kernel the call needs its strip-linear copy, kernel_shape, "
                             "K % 128 == 0 and more than %d rows" % SKINNY_MAX_ROWS)
        N = int(kernel_shape[1])
    else:
        if kernel.shape[0] != K:
            raise ValueError(f"inner dimensions differ: {a.shape} x {kernel.shape}")
        N = kernel.shape[1]
    if out_dtype is None:
        out_dtype = a_scale.dtype if a_scale is not None else torch.float32
    code = _lib.dtype_code(out_dtype)
    for t in (a_scale, kernel_scale, bias):
        if t is not None and t.dtype != out_dtype:
            raise TypeError("scales and bias must be read in the output dtype")
    a = a if a.is_contiguous() else a.contiguous()
    sa = a_scale.reshape(-1).contiguous() if a_scale is not None else None
    sb = kernel_scale.reshape(-1).contiguous() if kernel_scale is not None else None
    _check_bias_size(bias, M, N)
    y = torch.empty((M, N), dtype=out_dtype, device=a.device) if want_y else None
    acc = torch.empty((M, N), dtype=torch.int32, device=a.device) if want_acc else None
    lib = _lib.load()
    skinny = M <= SKINNY_MAX_ROWS and N % 16 == 0 and K % 8 == 0
    nbytes = lib.k3q_gemm_i8_workspace_bytes(M, N, K)
    if strip is not None and not skinny and K % 128 == 0:
        if strip.numel() != lib.k3q_w8s_shadow_bytes(K, N):
            raise ValueError("the strip-linear copy does not belong to a [%d, %d] kernel" % (K, N))
        b, layout = strip, 2
        nbytes = max(0, nbytes - (N * K + 15) // 16 * 16)  # (room for the partials of a K split only)
    elif prepacked is not None and not skinny:
        # no per-call [N,K] copy: only the part of the scratch beyond it (partial sums of a
        # K split, taken for few-tile problems) is of use; a K that is not a multiple of 128
        # keeps all of it (both operands are zero-padded into it)
        b, layout = prepacked, 1
        if K % 128 == 0:
            nbytes = max(0, nbytes - (N * K + 15) // 16 * 16)
    else:
        b = kernel if kernel.is_contiguous() else kernel.contiguous()
        layout = 0
    ws = _workspace(a.device, nbytes) if nbytes > 0 else None
    ws_bytes = nbytes if ws is not None else 0
    if bias is not None and M > 1 and bias.numel() == M * N:
        # a bias with a row per row of a: an addend (a residual), decode sizes only
        if not skinny or want_acc or not want_y:
            raise ValueError("a per-row addend takes at most %d rows, N %% 16 == 0, K %% 8 == 0 "
                             "and returns y only" % SKINNY_MAX_ROWS)
        ad = bias.reshape(M, N)
        rc = lib.k3q_gemm_i8_addend(
            _lib.ptr(a), _lib.ptr(b), M, N, K, _lib.ptr(sa), _lib.ptr(sb),
            _lib.ptr(ad if ad.is_contiguous() else ad.contiguous()), code,
            GEMM_EXACT_EPILOGUE if exact_epilogue else 0, _lib.ptr(y), _lib.ptr(ws), ws_bytes,
            _lib.stream_ptr(a.device))
        _lib.check(rc, "k3q_gemm_i8_addend")
        return y
    rc = lib.k3q_gemm_i8(
        _lib.ptr(a), _lib.ptr(b), layout, M, N, K, _lib.ptr(sa), _lib.ptr(sb), _lib.ptr(bias),
        code, GEMM_EXACT_EPILOGUE if exact_epilogue else 0, _lib.ptr(y), _lib.ptr(acc),
        _lib.ptr(ws), ws_bytes, _lib.stream_ptr(a.device),
    )
    _lib.check(rc, "k3q_gemm_i8")
    if want_acc and want_y:
        return y, acc
    return acc if want_acc else y


GEMM_ROUND_ACC_BF16 = 2


def int8_matmul_nk(a, kernel_nk, a_scale=None, kernel_scale=None, out_dtype=None,
                   exact_epilogue=False, want_acc=False, round_acc_bf16=False):
    """`a[M, K] int8 . kernel_nk[N, K]^T` with the de-scale fused: the kernel is given
    with K contiguous, which is how a tied int8 embedding table `[vocab, dim]` serves as
    the LM head (keras/src/layers/core/reversible_embedding.py:272-296).  Nothing is
    transposed or copied; decode-sized M runs the bandwidth-bound kernel, larger M the
    MFMA GEMM.  round_acc_bf16 (float32 output): the accumulator is cast to bfloat16
    before the division, as a bfloat16-compute layer with float32 scales does.
    """
    _lib.require_device(a, kernel_nk, a_scale, kernel_scale)
    if a.dtype != torch.int8 or kernel_nk.dtype != torch.int8:
        raise TypeError("int8_matmul_nk takes int8 operands")
    M, K = a.shape
    if kernel_nk.dim() != 2 or kernel_nk.shape[1] != K:
        raise ValueError(f"inner dimensions differ: {tuple(a.shape)} x {tuple(kernel_nk.shape)}^T")
    N = kernel_nk.shape[0]
    if out_dtype is None:
        out_dtype = a_scale.dtype if a_scale is not None else torch.float32
    code = _lib.dtype_code(out_dtype)
    for t in (a_scale, kernel_scale):
        if t is not None and t.dtype != out_dtype:
            raise TypeError("scales must be read in the output dtype")
    a = a if a.is_contiguous() else a.contiguous()
    b = kernel_nk if kernel_nk.is_contiguous() else kernel_nk.contiguous()
    sa = a_scale.reshape(-1).contiguous() if a_scale is not None else None
    sb = kernel_scale.reshape(-1).contiguous() if kernel_scale is not None else None
    y = torch.empty((M, N), dtype=out_dtype, device=a.device)
    acc = torch.empty((M, N), dtype=torch.int32, device=a.device) if want_acc else None
    lib = _lib.load()
    ws, ws_bytes = None, 0
    if M <= 64 or K % 128 != 0:
        # the decode kernels may split K and then need room for int32 partials; a K that is not
        # a multiple of 128 has both operands zero-padded into scratch
        ws = _workspace(a.device, lib.k3q_gemm_i8_workspace_bytes(M, N, K))
        ws_bytes = ws.numel()
    rc = lib.k3q_gemm_i8(
        _lib.ptr(a), _lib.ptr(b), 1, M, N, K, _lib.ptr(sa), _lib.ptr(sb), None, code,
        (GEMM_EXACT_EPILOGUE if exact_epilogue else 0)
        | (GEMM_ROUND_ACC_BF16 if round_acc_bf16 else 0),
        _lib.ptr(y), _lib.ptr(acc), _lib.ptr(ws), ws_bytes, _lib.stream_ptr(a.device),
    )
    _lib.check(rc, "k3q_gemm_i8")
    return (y, acc) if want_acc else y


def embedding_lookup(ids, table, scale, dim, bits=8, zero=None, block_size=None,
                     out_dtype=None, check_ids=True):
    """Rows `ids` of a quantized embedding table, de-quantised.

    table: int8 [vocab, dim] (bits=8) or packed int4 [vocab, ceil(dim/2)] (bits=4).
    scale: [vocab], or [vocab, groups] with `zero` int8 of the same shape for grouped int4.
    out_dtype: the dtype the reference's chain ends in, i.e. the promotion of the compute
    dtype and the scale dtype; bfloat16 only with bfloat16 scales.
    check_ids: raise IndexError for ids outside [-vocab, vocab) as the reference does
    (reads a flag back from the device, i.e. synchronises); without it such ids give rows of
    zeros.  Reference: keras/src/layers/core/embedding.py:521-582.
    """
    _lib.require_device(ids, table, scale, zero)
    if ids.dtype not in (torch.int32, torch.int64):
        ids = ids.to(torch.int32)
    ids = ids if ids.is_contiguous() else ids.contiguous()
    if table.dtype != torch.int8 or table.dim() != 2:
        raise TypeError("the embedding table must be a 2-D int8 tensor")
    vocab = table.shape[0]
    want_cols = dim if bits == 8 else (dim + 1) // 2
    if table.shape[1] != want_cols:
        raise ValueError(f"table has {table.shape[1]} columns, expected {want_cols}")
    grouped = block_size is not None and block_size > 0
    if out_dtype is None:
        out_dtype = scale.dtype
    if out_dtype == torch.bfloat16 and scale.dtype != torch.bfloat16:
        raise TypeError("float32 scales promote the result to float32")
    table = table if table.is_contiguous() else table.contiguous()
    scale = scale if scale.is_contiguous() else scale.contiguous()
    if grouped:
        if zero is None:
            raise ValueError("grouped int4 needs the zero points")
        zero = zero if zero.is_contiguous() else zero.contiguous()
    count = ids.numel()
    out = torch.empty((count, dim), dtype=out_dtype, device=table.device)
    flag = torch.zeros(1, dtype=torch.int32, device=table.device) if check_ids else None
    rc = _lib.load().k3q_embedding_lookup(
        _lib.ptr(ids), _lib.K3Q_I64 if ids.dtype == torch.int64 else _lib.K3Q_I32, count,
        _lib.ptr(table), vocab, int(dim), int(bits), _lib.ptr(scale), _lib.dtype_code(scale.dtype),
        _lib.ptr(zero) if grouped else None, int(block_size) if grouped else -1,
        _lib.dtype_code(out_dtype), _lib.ptr(out), _lib.ptr(flag), _lib.stream_ptr(table.device),
    )
    _lib.check(rc, "k3q_embedding_lookup")
    if check_ids and int(flag.item()) != 0:
        raise IndexError("index out of range in self")
    return out.reshape(*ids.shape, dim)


def int4_matmul_nk(x, table_packed, scale, zero=None, block_size=None):
    """`x[..., K] . W4[N, K]^T` for an int4 kernel stored K-contiguous: int8
    [N, ceil(K/2)], low nibble = even k -- a tied int4 embedding table used as the LM head
    (keras/src/layers/core/reversible_embedding.py:298-381, no activation quantizer).
    scale: [N] (per row) or [N, G] with `zero` int8 [N, G] (grouped along K).
    Returns [..., N] in bfloat16 when x and scale are bfloat16, float32 otherwise.
    """
    _lib.require_device(x, table_packed, scale, zero)
    xcode = _lib.dtype_code(x.dtype)
    scode = _lib.dtype_code(scale.dtype)
    K = x.shape[-1]
    if table_packed.dtype != torch.int8 or table_packed.dim() != 2 or table_packed.shape[1] != (K + 1) // 2:
        raise ValueError("table must be int8 of shape [N, ceil(K / 2)]")
    N = table_packed.shape[0]
    grouped = block_size is not None and block_size > 0
    lead = x.shape[:-1]
    x2 = x.reshape(-1, K)
    x2 = x2 if x2.is_contiguous() else x2.contiguous()
    tp = table_packed if table_packed.is_contiguous() else table_packed.contiguous()
    sc = scale if scale.is_contiguous() else scale.contiguous()
    zp = None
    if grouped:
        if zero is None:
            raise ValueError("grouped int4 needs the zero points")
        zp = zero if zero.is_contiguous() else zero.contiguous()
    out_dtype = torch.bfloat16 if (x.dtype == torch.bfloat16 and scale.dtype == torch.bfloat16) else torch.float32
    y = torch.empty((x2.shape[0], N), dtype=out_dtype, device=x.device)
    rc = _lib.load().k3q_gemv_w4_nk(
        _lib.ptr(x2), xcode, x2.shape[0], K, N, _lib.ptr(tp), _lib.ptr(sc), scode, _lib.ptr(zp),
        int(block_size) if grouped else -1, _lib.ptr(y), _lib.stream_ptr(x.device),
    )
    _lib.check(rc, "k3q_gemv_w4_nk")
    return y.reshape(*lead, N)


def int8_weight_only_matmul(x, kernel, kernel_scale, bias=None, prepacked=None):
    """`x[..., K] (float) . kernel[K, N] (int8)` with the per-channel de-scale:
    `y = T(T(x . W) / kernel_scale) + bias` -- a Dense int8 layer without an activation
    quantizer (keras/src/layers/core/dense.py:961-983).  Scale and bias in x.dtype."""
    _lib.require_device(x, kernel, kernel_scale, bias, prepacked)
    code = _lib.dtype_code(x.dtype)
    if kernel is None:  # only the [N, K] form is at hand (a tied embedding table)
        N, K = prepacked.shape
    else:
        K, N = kernel.shape
    if x.shape[-1] != K:
        raise ValueError(f"last axis of the input ({x.shape[-1]}) does not match the kernel ({K})")
    if kernel_scale.dtype != x.dtype or (bias is not None and bias.dtype != x.dtype):
        raise TypeError("kernel_scale and bias must be read in the input's dtype")
    lead = x.shape[:-1]
    x2 = x.reshape(-1, K)
    x2 = x2 if x2.is_contiguous() else x2.contiguous()
    M = x2.shape[0]
    if bias is not None and bias.numel() != N:
        raise ValueError(f"bias holds {bias.numel()} values, the layer has {N} units")
    if prepacked is not None:
        b, layout = prepacked, 1
    else:
        b, layout = (kernel if kernel.is_contiguous() else kernel.contiguous()), 0
    lib = _lib.load()
    ws = _workspace(x.device, lib.k3q_gemm_w8_workspace_bytes(M, N, K))
    y = torch.empty((M, N), dtype=x.dtype, device=x.device)
    rc = lib.k3q_gemm_w8(_lib.ptr(x2), code, _lib.ptr(b), layout, M, N, K,
                         _lib.ptr(kernel_scale.reshape(-1).contiguous()), _lib.ptr(bias), _lib.ptr(y),
                         _lib.ptr(ws), ws.numel(), _lib.stream_ptr(x.device))
    _lib.check(rc, "k3q_gemm_w8")
    return y.reshape(*lead, N)


def split_f32_kernel(w_nk):
    """float32 [N, K] kernel -> bfloat16 [N, 3K] = [wh | wh | wl], w = wh + wl to 2^-17: the
    operand `float_matmul_nk` takes for float32 inputs.  Made once per layer."""
    wh = w_nk.to(torch.bfloat16)
    wl = (w_nk - wh.to(torch.float32)).to(torch.bfloat16)
    return torch.cat([wh, wh, wl], dim=1).contiguous()


def float_matmul_nk(x, wt, parts=1, bias=None):
    """`x[M, K] . w[N, K]^T` in x.dtype against a de-quantised kernel kept as bfloat16.

    x bfloat16: wt = w [N, K], parts 1.  x float32: wt = `split_f32_kernel(w)` [N, 3K], parts 3.
    Reference: the `ops.einsum(self.equation, inputs, float_kernel)` of
    keras/src/layers/core/einsum_dense.py:1186 and :1236 for kernels the fused int4 kernel
    cannot consume in place.
    """
    _lib.require_device(x, wt, bias)
    if wt.dtype != torch.bfloat16 or wt.dim() != 2 or not wt.is_contiguous():
        raise TypeError("the kernel must be a contiguous 2-D bfloat16 tensor")
    if x.dim() != 2:
        raise ValueError("x must be [M, K]")
    want_parts = 1 if x.dtype == torch.bfloat16 else 3
    if parts not in (want_parts, 2 if want_parts == 3 else want_parts):
        raise ValueError(f"parts={parts} does not fit inputs of {x.dtype}")
    M, K = x.shape
    if wt.shape[1] != parts * K:
        raise ValueError(f"kernel row length {wt.shape[1]} is not parts * K = {parts * K}")
    if bias is not None and bias.dtype != x.dtype:
        raise TypeError("bias must be read in the input's dtype")
    N = wt.shape[0]
    x = x if x.is_contiguous() else x.contiguous()
    y = torch.empty((M, N), dtype=x.dtype, device=x.device)
    lib = _lib.load()
    ws = _workspace(x.device, lib.k3q_gemm_wbf16_workspace_bytes(M, N, K, parts))
    rc = lib.k3q_gemm_wbf16(_lib.ptr(x), _lib.dtype_code(x.dtype), _lib.ptr(wt), parts, M, N, K,
                            _lib.ptr(bias), _lib.ptr(y), _lib.ptr(ws), ws.numel(),
                            _lib.stream_ptr(x.device))
    _lib.check(rc, "k3q_gemm_wbf16")
    return y



INT8_STRIP_MAX_ROWS = 16


def int8_strip_supported(M, K, N):
    """Whether `int8_dense_strip` takes M rows against a [K, N] int8 kernel."""
    return bool(_lib.load().k3q_dense_i8_w8s_supported(int(M), int(K), int(N)))


def int8_strip_copy(kernel):
    """The strip-linear copy of a stored int8 kernel `[K, N]` that `int8_dense_strip` reads
    (include/k3q.h, k3q_w8s_pack): uint8 bytes, made once per layer."""
    _lib.require_device(kernel)
    if kernel.dtype != torch.int8 or kernel.dim() != 2:
        raise ValueError(f"expected the stored int8 kernel [K, N], got {kernel.dtype} {tuple(kernel.shape)}")
    lib = _lib.load()
    K, N = (int(d) for d in kernel.shape)
    nbytes = lib.k3q_w8s_shadow_bytes(K, N)
    if nbytes <= 0:
        raise ValueError(f"no strip-linear copy for a [{K}, {N}] kernel (K % 64 != 0)")
    src = kernel if kernel.is_contiguous() else kernel.contiguous()
    out = torch.empty(nbytes, dtype=torch.uint8, device=src.device)
    _lib.check(lib.k3q_w8s_pack(_lib.ptr(src), K, N, _lib.ptr(out), _lib.stream_ptr(src.device)), "k3q_w8s_pack")
    return out


# rows and values of x up to which every workgroup of `int8_dense_strip` quantises the rows itself;
# beyond, one quantizer launch and the kernel's pre-quantised form are faster (measured at
# K = N = 8192: 4 rows 17.5 us against 18.9, 8 rows 19.9 against 19.5; 8 rows of 4096: 9.7 against 9.3)
INT8_STRIP_FUSED_MAX_ROWS = 4
INT8_STRIP_FUSED_QUANTIZER_MAX = 32768


def int8_strip_quantises_inside(M, K, value_range):
    """Whether the strip kernel quantises these rows itself (otherwise a quantizer launch comes first).
    Its quantizer clips before it rounds, which is exact only between integer ends of the range."""
    lo, hi = float(value_range[0]), float(value_range[1])
    return (M <= INT8_STRIP_FUSED_MAX_ROWS and M * K <= INT8_STRIP_FUSED_QUANTIZER_MAX and lo == round(lo) and hi == round(hi)
            and -128 <= lo < hi <= 127)


def int8_dense_strip(x, shadow, units, kernel_scale, bias=None, epsilon=1e-7, value_range=(-127, 127),
                     quantize=None):
    """The int8 Dense forward for up to 16 bfloat16 rows: abs-max quantisation of the rows, exact
    int8 matmul against `int8_strip_copy(kernel)`, bit-exact bfloat16 de-scale, bias (N values)
    or addend (a row per row of x).  One launch for small x; for larger x the rows are
    quantised by `quantize(x2)` (default: `quantizers.abs_max_quantize` with these settings)
    first.  Same bits as `abs_max_quantize` + `int8_matmul(..., exact_epilogue=True)`.
    Reference: keras/src/layers/core/dense.py:956-972."""
    _lib.require_device(x, shadow, kernel_scale, bias)
    lib = _lib.load()
    if x.dtype != torch.bfloat16 or kernel_scale.dtype != torch.bfloat16:
        raise TypeError("the strip route computes in bfloat16")
    K, N = int(x.shape[-1]), int(units)
    lead = x.shape[:-1]
    x2 = x.reshape(-1, K)
    x2 = x2 if x2.is_contiguous() else x2.contiguous()
    M = x2.shape[0]
    if not lib.k3q_dense_i8_w8s_supported(M, K, N):
        raise ValueError(f"int8_dense_strip does not take M={M}, K={K}, N={N}")
    if shadow.dtype != torch.uint8 or shadow.numel() != lib.k3q_w8s_shadow_bytes(K, N):
        raise ValueError("shadow is not int8_strip_copy(kernel) of this [K, N]")
    if kernel_scale.numel() != N:
        raise ValueError(f"kernel_scale holds {kernel_scale.numel()} values, expected {N}")
    _check_bias_size(bias, M, N)
    if bias is not None and bias.dtype != torch.bfloat16:
        raise TypeError("bias must be bfloat16")
    stride = N if (bias is not None and M > 1 and bias.numel() == M * N) else 0
    ks = kernel_scale if kernel_scale.is_contiguous() else kernel_scale.contiguous()
    y = torch.empty((M, N), dtype=torch.bfloat16, device=x.device)
    if not int8_strip_quantises_inside(M, K, value_range):
        if quantize is None:
            from keras_amd import quantizers

            q, s = quantizers.abs_max_quantize(x2, axis=-1, value_range=value_range, epsilon=epsilon)
        else:
            q, s = quantize(x2)
        rc = lib.k3q_gemm_i8_w8s(_lib.ptr(q), _lib.ptr(s), _lib.dtype_code(s.dtype), M, K, N, _lib.ptr(shadow),
                                 _lib.ptr(ks), _lib.ptr(bias) if bias is not None else None, stride,
                                 _lib.ptr(y), _lib.stream_ptr(x.device))
        _lib.check(rc, "k3q_gemm_i8_w8s")
        return y.reshape(*lead, N)
    rc = lib.k3q_dense_i8_w8s(_lib.ptr(x2), _lib.dtype_code(x.dtype), M, K, N, _lib.ptr(shadow), _lib.ptr(ks),
                              _lib.ptr(bias) if bias is not None else None, stride, float(epsilon),
                              float(value_range[0]), float(value_range[1]), _lib.ptr(y),
                              _lib.stream_ptr(x.device))
    _lib.check(rc, "k3q_dense_i8_w8s")
    return y.reshape(*lead, N)


def int8_dense_strip_multi(x, kernels, epsilon=1e-7, value_range=(-127, 127), quantize=None, input_op=None,
                           bias_rows=False):
    """`[int8_dense_strip(op(x), k) for k in kernels]` for layers that share `x[..., K]` (up to 16
    bfloat16 rows) and quantise it alike: one launch for those whose launch plans agree, the same
    bits as the separate calls.  kernels: dicts with `shadow`, `units`, `kernel_scale` and
    optionally `bias` [N] (bias_rows: [M, N]).  input_op: as in `int4_matmul_strip_multi`
    (`int8_strip_input_op_supported`)."""
    lib = _lib.load()
    K = int(x.shape[-1])
    lead = x.shape[:-1]
    x2 = x.reshape(-1, K)
    x2 = x2 if x2.is_contiguous() else x2.contiguous()
    M = x2.shape[0]
    if x.dtype != torch.bfloat16:
        raise TypeError("the strip route computes in bfloat16")
    problems = (_lib.W8sProblem * len(kernels))()
    outs, keep = [], []
    for i, k in enumerate(kernels):
        N = int(k["units"])
        bias, ks = k.get("bias"), k["kernel_scale"]
        _lib.require_device(x, k["shadow"], ks, bias)
        if not lib.k3q_dense_i8_w8s_supported(M, K, N):
            raise ValueError(f"int8_dense_strip_multi does not take M={M}, K={K}, N={N}")
        if k["shadow"].dtype != torch.uint8 or k["shadow"].numel() != lib.k3q_w8s_shadow_bytes(K, N):
            raise ValueError("shadow is not int8_strip_copy(kernel) of this [K, N]")
        if ks.dtype != torch.bfloat16 or ks.numel() != N:
            raise ValueError(f"kernel_scale must hold {N} bfloat16 values")
        want = M * N if bias_rows else N
        if bias is not None and (bias.numel() != want or bias.dtype != torch.bfloat16 or not bias.is_contiguous()):
            raise ValueError(f"bias must hold {want} bfloat16 values, contiguous")
        ks = ks if ks.is_contiguous() else ks.contiguous()
        keep.append(ks)
        y = torch.empty((M, N), dtype=torch.bfloat16, device=x.device)
        outs.append(y)
        problems[i] = _lib.W8sProblem(N, k["shadow"].data_ptr(), ks.data_ptr(),
                                      bias.data_ptr() if bias is not None else None, y.data_ptr())
    if input_op is not None or bias_rows:
        if not int8_strip_quantises_inside(M, K, value_range):
            raise ValueError("input operations and per-row addends need rows the kernel quantises itself")
        pre, keep_op = _input_op_struct(input_op, M, K, x.device)
        rc = lib.k3q_dense_i8_w8s_pre(_lib.ptr(x2), _lib.K3Q_BF16, M, K, ctypes.byref(pre) if pre is not None else None,
                                      len(kernels), ctypes.byref(problems), float(epsilon), float(value_range[0]),
                                      float(value_range[1]), 1 if bias_rows else 0, _lib.stream_ptr(x.device))
        _lib.check(rc, "k3q_dense_i8_w8s_pre")
        del keep_op
        return [y.reshape(*lead, y.shape[1]) for y in outs]
    q = s = None
    if not int8_strip_quantises_inside(M, K, value_range):
        if quantize is None:
            from keras_amd import quantizers

            q, s = quantizers.abs_max_quantize(x2, axis=-1, value_range=value_range, epsilon=epsilon)
        else:
            q, s = quantize(x2)
        if s.dtype != torch.bfloat16:
            raise TypeError("the rows' scales must be bfloat16")
    rc = lib.k3q_dense_i8_w8s_multi(_lib.ptr(x2), _lib.K3Q_BF16, _lib.ptr(q), _lib.ptr(s), M, K, len(kernels),
                                    ctypes.byref(problems), float(epsilon), float(value_range[0]),
                                    float(value_range[1]), _lib.stream_ptr(x.device))
    _lib.check(rc, "k3q_dense_i8_w8s_multi")
    return [y.reshape(*lead, y.shape[1]) for y in outs]


def decode_attention_supported(q, cache_k):
    """bfloat16, head width 128, one new position."""
    return (q.is_cuda and q.dtype == torch.bfloat16 and q.dim() == 4 and q.shape[1] == 1
            and q.shape[-1] == 128 and cache_k.dtype == torch.bfloat16 and cache_k.shape[2] <= 32768)


def decode_attention(q, k, v, cos_table, sin_table, pos, cache_k, cache_v, oob_flag=None):
    """One decode position of causal self-attention: q, k, v `[B, 1, H, 128]` bfloat16 (as the
    projections give them), `cos_table` / `sin_table` `[max_len, 128]`, `pos` an int64 device
    tensor holding the position, the caches `[B, H, max_len, 128]` (row `pos` is written).
    Returns `[B, 1, H, 128]`.  What it replaces in a decoder step: the rotation of q and k,
    two `index_copy_` into the caches and `scaled_dot_product_attention` under a mask that
    admits keys `<= pos`.  A position outside `[0, max_len)` (where `index_copy_` raises) leaves
    the caches alone, returns zero rows and sets `oob_flag` (an int32 device tensor of one element
    that the caller reads when it synchronises anyway; without one the call checks a flag of its
    own, which costs a synchronisation)."""
    _lib.require_device(q, k, v, cos_table, sin_table, pos, cache_k, cache_v)
    lib = _lib.load()
    B, T, H, hd = q.shape
    if T != 1 or k.shape != q.shape or v.shape != q.shape:
        raise ValueError(f"decode_attention takes one position: q, k, v [B, 1, H, hd], got {tuple(q.shape)}")
    max_len = cache_k.shape[2]
    if tuple(cache_k.shape) != (B, H, max_len, hd) or cache_v.shape != cache_k.shape:
        raise ValueError(f"caches must be [B, H, max_len, hd], got {tuple(cache_k.shape)}")
    if tuple(cos_table.shape) != (max_len, hd) or tuple(sin_table.shape) != (max_len, hd):
        raise ValueError(f"rotation tables must be [max_len, hd] = [{max_len}, {hd}]")
    if pos.dtype != torch.int64 or pos.numel() != 1:
        raise ValueError("pos must be one int64 value on the device")
    for t in (q, k, v, cos_table, sin_table, cache_k, cache_v):
        if t.dtype != torch.bfloat16:
            raise TypeError("decode_attention computes in bfloat16")
    if not (cache_k.is_contiguous() and cache_v.is_contiguous()):
        raise ValueError("the caches are written in place and must be contiguous")
    q, k, v = (t if t.is_contiguous() else t.contiguous() for t in (q, k, v))
    cos_table = cos_table if cos_table.is_contiguous() else cos_table.contiguous()
    sin_table = sin_table if sin_table.is_contiguous() else sin_table.contiguous()
    out = torch.empty((B, 1, H, hd), dtype=torch.bfloat16, device=q.device)
    own_flag = oob_flag is None and not torch.cuda.is_current_stream_capturing()
    if own_flag:
        oob_flag = torch.zeros(1, dtype=torch.int32, device=q.device)
    if oob_flag is not None:
        _lib.require_device(oob_flag)
        if oob_flag.dtype != torch.int32 or oob_flag.numel() != 1:
            raise ValueError("oob_flag must be one int32 value on the device")
    rc = lib.k3q_decode_attention(_lib.ptr(q), _lib.ptr(k), _lib.ptr(v), _lib.dtype_code(q.dtype), B, H, hd,
                                  max_len, _lib.ptr(cos_table), _lib.ptr(sin_table), _lib.ptr(pos),
                                  _lib.ptr(cache_k), _lib.ptr(cache_v), _lib.ptr(out), _lib.ptr(oob_flag),
                                  _lib.stream_ptr(q.device))
    _lib.check(rc, "k3q_decode_attention")
    if own_flag and int(oob_flag.item()):
        raise IndexError(f"decode_attention: position {int(pos.item())} is outside the cache of {max_len} rows")
    return out


def _rows_view(t):
    """[rows, dim] view of a tensor whose last axis is contiguous and whose leading axes collapse
    into one stride (else a contiguous copy): (tensor, rows, dim, row stride in elements)."""
    dim = t.shape[-1]
    t2 = t.reshape(-1, dim) if t.dim() != 2 else t
    if t2.stride(-1) != 1 or (t2.shape[0] > 1 and t2.stride(0) % 8):
        t2 = t2.contiguous()
    return t2, t2.shape[0], dim, (t2.stride(0) if t2.shape[0] > 1 else dim)


def rmsnorm_supported(x, weight):
    return (x.is_cuda and x.dtype == torch.bfloat16 and weight.dtype == torch.bfloat16
            and x.shape[-1] % 8 == 0 and x.shape[-1] <= 16384 and weight.numel() == x.shape[-1])


def rmsnorm(x, weight, epsilon):
    """`rms_norm(x, weight, epsilon)` over the last axis, bfloat16, one short launch (the decoder
    harness's normalisation between the quantized layers)."""
    _lib.require_device(x, weight)
    lib = _lib.load()
    x2, rows, dim, xs = _rows_view(x)
    w = weight if weight.is_contiguous() else weight.contiguous()
    y = torch.empty((rows, dim), dtype=x.dtype, device=x.device)
    rc = lib.k3q_rmsnorm(_lib.ptr(x2), _lib.ptr(w), _lib.dtype_code(x.dtype), rows, dim, xs, float(epsilon),
                         _lib.ptr(y), dim, _lib.stream_ptr(x.device))
    _lib.check(rc, "k3q_rmsnorm")
    return y.reshape(x.shape)


def silu_mul_supported(gate, up):
    return (gate.is_cuda and gate.dtype == torch.bfloat16 and up.dtype == torch.bfloat16
            and gate.shape == up.shape and gate.shape[-1] % 8 == 0)


def silu_mul(gate, up):
    """`silu(gate) * up`, bfloat16, one launch; the operands may be column slices of a wider
    tensor (rows given by a stride)."""
    _lib.require_device(gate, up)
    lib = _lib.load()
    g2, rows, dim, gs = _rows_view(gate)
    u2, _, _, us = _rows_view(up)
    y = torch.empty((rows, dim), dtype=gate.dtype, device=gate.device)
    rc = lib.k3q_silu_mul(_lib.ptr(g2), _lib.ptr(u2), _lib.dtype_code(gate.dtype), rows, dim, gs, us,
                          _lib.ptr(y), dim, _lib.stream_ptr(gate.device))
    _lib.check(rc, "k3q_silu_mul")
    return y.reshape(gate.shape)
