"""`keras.quantizers` primitives of the int8 / int4 path on MI355X.

Same names, arguments, return values and error text as the reference
(keras/src/quantizers/quantizers.py); the tensor paths run as HIP kernels
through the k3q C ABI.

  abs_max_quantize                          quantizers.py:70-120
  AbsMaxQuantizer                           quantizers.py:307-373
  abs_max_quantize_grouped_with_zero_point  quantizers.py:123-234
  pack_int4 / unpack_int4                   quantizers.py:623-900
  dequantize_with_sz_map                    quantizers.py:1631-1668

`to_numpy=True` keeps the reference's meaning for host tensors and arrays: the
arithmetic is done with numpy on the host (the reference does this on purpose,
to keep the float kernel off the device while a model is being converted) and
the results are moved to the device of the input.  A float32 / bfloat16 tensor
that already lives on a HIP device is quantised where it is, by kernels that
repeat numpy's float32 operations one by one (k3q_weight_quantize.hip): the same
integers, scales and zero points, bit for bit, without the trip to the host.
"""

import math

import numpy as np
import torch

from keras_amd import _lib

EPSILON = 1e-7  # keras/src/backend/config.py:10


def _standardize_axis(axis, rank):
    if isinstance(axis, int):
        axis = (axis,)
    axis = tuple(a + rank if a < 0 else a for a in axis)
    for a in axis:
        if a < 0 or a >= rank:
            raise ValueError(f"axis {a} is out of bounds for a rank-{rank} tensor")
    return tuple(sorted(set(axis)))


def _to_host_array(x):
    if isinstance(x, torch.Tensor):
        t = x.detach()
        if t.dtype == torch.bfloat16:
            t = t.float()
        return t.cpu().numpy()
    return np.asarray(x)


def _check_int8_range(value_range, dtype):
    if dtype == "int8" and (value_range[0] < -128 or value_range[1] > 127):
        raise ValueError(
            "Quantizer with output_dtype='int8' requires value_range to be "
            f"within the interval [-128, 127]. Received: value_range={value_range}"
        )


def abs_max_quantize(
    inputs,
    axis,
    value_range=(-127, 127),
    dtype="int8",
    epsilon=EPSILON,
    to_numpy=False,
):
    """Abs-max quantisation; returns `(quantized int8, scale)`.

    The scale has the input's dtype and the reduced axes kept with length 1.
    Tensor path: one fused HIP kernel over the rows formed by the reduced axes
    (they are moved to the back when they are not trailing already).
    """
    if dtype != "int8":
        raise NotImplementedError(
            f"abs_max_quantize on this path produces int8 only, got dtype={dtype}"
        )
    if to_numpy and _on_device(inputs) and len(_standardize_axis(axis, inputs.dim())) > 0:
        return _abs_max_quantize_numpy_bits(inputs, axis, value_range, epsilon)
    if to_numpy:
        # reference: quantizers.py:95-109
        device = inputs.device if isinstance(inputs, torch.Tensor) else None
        original_dtype = inputs.dtype if isinstance(inputs, torch.Tensor) else None
        arr = _to_host_array(inputs)
        ax = _standardize_axis(axis, arr.ndim)
        scale = np.divide(
            value_range[1],
            np.add(np.max(np.abs(arr), axis=ax, keepdims=True), epsilon),
        )
        out = np.multiply(arr, scale)
        out = np.clip(np.round(out), value_range[0], value_range[1]).astype(dtype)
        q = torch.from_numpy(out)
        s = torch.from_numpy(np.asarray(scale))
        if original_dtype is not None:
            s = s.to(original_dtype)
        if device is not None:
            q, s = q.to(device), s.to(device)
        return q, s

    x = inputs
    if not isinstance(x, torch.Tensor):
        raise TypeError("abs_max_quantize(to_numpy=False) takes a torch tensor")
    _lib.require_device(x)
    _check_int8_range(value_range, dtype)
    code = _lib.dtype_code(x.dtype)
    rank = x.dim()
    ax = _standardize_axis(axis, rank)
    kept = [i for i in range(rank) if i not in ax]
    trailing = ax == tuple(range(rank - len(ax), rank))
    xr = x if trailing else x.permute(kept + list(ax))
    cols = 1
    for a in ax:
        cols *= x.shape[a]
    rows = x.numel() // cols if cols else 0
    if cols == 0:
        raise ValueError("Cannot compute the max of an empty tensor.")
    x2 = xr.reshape(rows, cols)
    if x2.stride(-1) != 1:
        x2 = x2.contiguous()
    q2 = torch.empty((rows, cols), dtype=torch.int8, device=x.device)
    s1 = torch.empty((rows,), dtype=x.dtype, device=x.device)
    lib = _lib.load()
    rc = lib.k3q_absmax_quantize(
        _lib.ptr(x2), code, rows, cols, x2.stride(0) if rows > 1 else cols,
        float(epsilon), float(value_range[0]), float(value_range[1]),
        _lib.ptr(q2), _lib.ptr(s1), _lib.stream_ptr(x.device),
    )
    _lib.check(rc, "k3q_absmax_quantize")
    scale_shape = [1 if i in ax else x.shape[i] for i in range(rank)]
    if trailing:
        q = q2.reshape(x.shape)
    else:
        perm = kept + list(ax)
        inv = [perm.index(i) for i in range(rank)]
        q = q2.reshape([x.shape[i] for i in perm]).permute(inv)
    return q, s1.reshape(scale_shape)


def _on_device(x):
    return isinstance(x, torch.Tensor) and x.is_cuda and x.dtype in (torch.float32, torch.bfloat16)


def _abs_max_quantize_numpy_bits(x, axis, value_range, epsilon):
    """The `to_numpy=True` result (quantizers.py:95-109: float32 numpy arithmetic, scale cast back
    to the input's dtype) for a tensor that lives on the device, computed there."""
    _check_int8_range(value_range, "int8")
    rank = x.dim()
    ax = _standardize_axis(axis, rank)
    scale_shape = [1 if i in ax else x.shape[i] for i in range(rank)]
    if x.numel() == 0:
        raise ValueError("Cannot compute the max of an empty tensor.")
    if ax[-1] == rank - 1 and ax == tuple(range(ax[0], rank)):
        # trailing axes: the row kernel in float32 is the same operation sequence
        q, s = abs_max_quantize(x.float() if x.dtype != torch.float32 else x, ax, value_range, "int8",
                                epsilon, to_numpy=False)
        return q, s.to(x.dtype)
    run = ax == tuple(range(ax[0], ax[-1] + 1))
    if run:
        src, perm = x.contiguous(), None
    else:
        # reduced axes that are not neighbours: bring them together in front of the trailing kept axes
        kept = [i for i in range(rank) if i not in ax]
        head = [i for i in kept if i < ax[0]]
        perm = head + list(ax) + [i for i in kept if i > ax[0]]
        src = x.permute(perm).contiguous()
    shape = list(src.shape)
    a0 = ax[0] if run else len([i for i in range(rank) if i not in ax and i < ax[0]])
    outer = int(np.prod(shape[:a0], dtype=np.int64)) if a0 else 1
    R = int(np.prod(shape[a0:a0 + len(ax)], dtype=np.int64))
    inner = int(np.prod(shape[a0 + len(ax):], dtype=np.int64))
    q = torch.empty(shape, dtype=torch.int8, device=x.device)
    s = torch.empty((outer * inner,), dtype=x.dtype, device=x.device)
    ws = torch.empty((outer * inner,), dtype=torch.int32, device=x.device)
    rc = _lib.load().k3q_weight_absmax_quantize(
        _lib.ptr(src), _lib.dtype_code(x.dtype), outer, R, inner, float(epsilon),
        float(value_range[0]), float(value_range[1]), _lib.ptr(q), _lib.ptr(s), _lib.ptr(ws),
        _lib.stream_ptr(x.device))
    _lib.check(rc, "k3q_weight_absmax_quantize")
    if perm is not None:
        inv = [perm.index(i) for i in range(rank)]
        q = q.permute(inv)
        kept_shape = [shape[i] for i in range(len(shape)) if not (a0 <= i < a0 + len(ax))]
        kept_axes = [p_ for i, p_ in enumerate(perm) if not (a0 <= i < a0 + len(ax))]
        s = s.reshape(kept_shape).permute(sorted(range(len(kept_axes)), key=kept_axes.__getitem__))
    return q, s.reshape(scale_shape)


class Quantizer:
    """keras/src/quantizers/quantizers.py:19-66."""

    def __init__(self, output_dtype="int8"):
        self.output_dtype = output_dtype

    def __call__(self, x):
        return x

    @classmethod
    def from_config(cls, config):
        return cls(**config)

    def get_config(self):
        raise NotImplementedError(f"{self} does not implement get_config()")


class AbsMaxQuantizer(Quantizer):
    """keras/src/quantizers/quantizers.py:307-373."""

    def __init__(self, axis=None, value_range=(-127, 127), epsilon=EPSILON,
                 output_dtype="int8"):
        Quantizer.__init__(self, output_dtype=output_dtype)
        if axis is not None:
            if isinstance(axis, int):
                axis = (axis,)
            self.axis = tuple(axis)
        else:
            self.axis = None
        self.value_range = value_range
        self.epsilon = epsilon
        if output_dtype == "int8":
            if value_range[0] < -128 or value_range[1] > 127:
                raise ValueError(
                    f"Quantizer with output_dtype='int8' requires value_range "
                    f"to be within the interval [-128, 127]. Received: "
                    f"value_range={value_range}"
                )

    def __call__(self, x, axis=None, to_numpy=False):
        if axis is None:
            axis = self.axis
        if axis is None:
            axis = -1
        return abs_max_quantize(
            x, axis, self.value_range, self.output_dtype, self.epsilon, to_numpy
        )

    def get_config(self):
        config = {
            "value_range": self.value_range,
            "epsilon": self.epsilon,
            "output_dtype": self.output_dtype,
        }
        if self.axis is not None:
            config["axis"] = self.axis
        return config


def abs_max_quantize_grouped_with_zero_point(
    inputs, block_size, value_range=(-8, 7), dtype="int8", epsilon=EPSILON,
    to_numpy=True,
):
    """Grouped asymmetric quantisation of a `[input_dim, output_dim]` kernel.

    The numpy variant, the one `Dense.quantize` / `EinsumDense.quantize` call
    (quantizers.py:179-234): on the host for host inputs, on the device -- the same
    float32 operations, the same bits -- for a float32 / bfloat16 tensor that lives
    there.  Returns `(q int8 [K,N], scale [G,N], zero int8 [G,N])` on the device of
    `inputs`.
    """
    if not to_numpy:
        raise NotImplementedError(
            "only the numpy variant (to_numpy=True) is on the inference path: the tensor variant "
            "(quantizers.py:237-306) goes through the GPTQ parameter search, which the layers never call"
        )
    if _on_device(inputs):
        if inputs.dim() != 2:
            raise ValueError(f"expected a [input_dim, output_dim] kernel, got shape {tuple(inputs.shape)}")
        if dtype != "int8":
            raise NotImplementedError(f"the grouped quantizer produces int8 storage only, got dtype={dtype}")
        _check_int8_range(value_range, dtype)
        x = inputs.contiguous()
        K, N = x.shape
        G = math.ceil(K / block_size)
        q = torch.empty((K, N), dtype=torch.int8, device=x.device)
        st = torch.empty((G, N), dtype=x.dtype, device=x.device)
        zt = torch.empty((G, N), dtype=torch.int8, device=x.device)
        rc = _lib.load().k3q_weight_quantize_grouped(
            _lib.ptr(x), _lib.dtype_code(x.dtype), K, N, int(block_size), float(epsilon),
            float(value_range[0]), float(value_range[1]), _lib.ptr(q), _lib.ptr(st), _lib.ptr(zt),
            _lib.stream_ptr(x.device))
        _lib.check(rc, "k3q_weight_quantize_grouped")
        return q, st, zt
    device = inputs.device if isinstance(inputs, torch.Tensor) else None
    original_dtype = inputs.dtype if isinstance(inputs, torch.Tensor) else None
    arr = _to_host_array(inputs)
    input_dim, output_dim = arr.shape
    n_groups = math.ceil(input_dim / block_size)
    qmin, qmax = value_range
    padded_dim = n_groups * block_size
    if padded_dim > input_dim:
        pad = np.zeros((padded_dim - input_dim, output_dim), dtype=arr.dtype)
        arr = np.concatenate([arr, pad], axis=0)
    grouped = arr.reshape(n_groups, block_size, output_dim)
    lo = np.min(grouped, axis=1, keepdims=True)
    hi = np.max(grouped, axis=1, keepdims=True)
    scale = np.divide(np.subtract(hi, lo) + epsilon, qmax - qmin)
    zero = np.clip(np.round(np.divide(-lo, scale)) + qmin, qmin, qmax)
    q = np.clip(np.round(np.divide(grouped, scale)) + zero, qmin, qmax).astype(dtype)
    q = q.reshape(padded_dim, output_dim)[:input_dim, :]
    scale = np.squeeze(scale, axis=1)
    zero = np.squeeze(zero, axis=1).astype("int8")
    qt = torch.from_numpy(np.ascontiguousarray(q))
    st = torch.from_numpy(scale)
    zt = torch.from_numpy(zero)
    if original_dtype is not None:
        st = st.to(original_dtype)
    if device is not None:
        qt, st, zt = qt.to(device), st.to(device), zt.to(device)
    return qt, st, zt


def _packing_dtype(dtype):
    if dtype not in ("int8", "uint8"):
        raise ValueError(
            f"Expected dtype to be 'int8' or 'uint8', but got '{dtype}'."
        )
    return torch.int8 if dtype == "int8" else torch.uint8


def _dtype_name(t):
    return str(t.dtype).replace("torch.", "")


def _as_outer_len_inner(shape, axis):
    outer = 1
    for d in shape[:axis]:
        outer *= d
    inner = 1
    for d in shape[axis + 1:]:
        inner *= d
    return outer, shape[axis], inner


def pack_int4(arr, axis=0, dtype="int8"):
    """Pack int4 values (held in int8 / uint8) two per byte along `axis`.

    Returns `(packed, packed_shape, orig_len)`; low nibble = even index, an odd
    length is padded with one zero slice (quantizers.py:700-750).
    """
    tdt = _packing_dtype(dtype)
    if not isinstance(arr, torch.Tensor):
        arr = torch.as_tensor(np.asarray(arr))
    if arr.dtype != tdt:
        raise TypeError(
            f"Expected {dtype} tensor for packing, got {_dtype_name(arr)}."
        )
    _lib.require_device(arr)
    rank = arr.dim()
    if axis < 0:
        axis += rank
    src = arr.contiguous()
    outer, n, inner = _as_outer_len_inner(tuple(src.shape), axis)
    packed_shape = list(src.shape)
    packed_shape[axis] = (n + 1) // 2
    out = torch.empty(packed_shape, dtype=tdt, device=arr.device)
    rc = _lib.load().k3q_pack_int4(
        _lib.ptr(src), outer, n, inner, _lib.ptr(out), _lib.stream_ptr(arr.device)
    )
    _lib.check(rc, "k3q_pack_int4")
    return out, tuple(packed_shape), n


def unpack_int4(packed, orig_len, axis=0, dtype="int8"):
    """Inverse of `pack_int4` (quantizers.py:830-900): int8 storage holding two
    nibbles per byte -> one value per byte, `(v ^ 8) - 8` sign fix for "int8",
    trimmed to `orig_len` along `axis`."""
    tdt = _packing_dtype(dtype)
    if not isinstance(packed, torch.Tensor):
        packed = torch.as_tensor(np.asarray(packed))
    if packed.dtype not in (torch.int8, torch.uint8):
        raise TypeError(
            f"Expected int8 or uint8 tensor for unpacking, got {packed.dtype}"
        )
    _lib.require_device(packed)
    rank = packed.dim()
    if axis < 0:
        axis += rank
    src = packed.contiguous()
    outer, plen, inner = _as_outer_len_inner(tuple(src.shape), axis)
    orig_len = int(orig_len)
    if orig_len > 2 * plen:
        orig_len = 2 * plen  # slicing past the end keeps what is there
    out_shape = list(src.shape)
    out_shape[axis] = orig_len
    out = torch.empty(out_shape, dtype=tdt, device=packed.device)
    rc = _lib.load().k3q_unpack_int4(
        _lib.ptr(src), outer, plen, inner, orig_len, 1 if dtype == "int8" else 0,
        _lib.ptr(out), _lib.stream_ptr(packed.device),
    )
    _lib.check(rc, "k3q_unpack_int4")
    return out


def dequantize_with_sz_map(weights_matrix, scale, zero, g_idx, group_axis=-1):
    """`(w - zero[g]) * scale[g]` with groups looked up through `g_idx`
    (quantizers.py:1631-1668).  Not on the forward path of this build (the int4
    GEMV folds scale and zero point in-kernel); kept for callers that want the
    float kernel, e.g. the `kernel` property of a layer.  Plain torch indexing
    on whatever device the operands live on."""
    groups = g_idx.to(torch.int32).long()
    s = torch.index_select(scale, group_axis % scale.dim(), groups)
    z = torch.index_select(zero, group_axis % zero.dim(), groups).to(s.dtype)
    return torch.multiply(torch.subtract(weights_matrix, z), s)
