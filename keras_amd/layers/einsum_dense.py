"""`EinsumDense` with the int8 / int4 quantized forward on MI355X.

Mirrors the quantization-related surface of `keras.layers.EinsumDense`
(keras/src/layers/core/einsum_dense.py): equation analysis, variable names and
shapes (`_kernel`, `kernel_scale` in the reference's broadcast layout,
`kernel_zero`, `g_idx`), `quantize`, `_int8_call`, `_int4_call`.

The quantized einsum is lowered to the 2-D kernels: every equation whose labels
split into free (input and output), contracted (input and kernel) and kept
(kernel and output) sets is a GEMM of the input viewed as [free, contracted]
with the kernel viewed as [contracted, kept]; the views are free of copies for
the usual projection equations (`btd,dnh->btnh`, `btnh,nhd->btd`, `ab,bc->ac`).
"""

import math
import string

import torch

from keras_amd import dtype_policies, ops as kops, quantizers
from keras_amd.layers.dense import (_ACTIVATIONS, activation_name, glorot_uniform, int8_strip_route,
                                    lora_initializer,
                                    serialize_quantization_config)
from keras_amd.layers.layer import Layer, as_tensor, require_default_g_idx, to_torch_dtype
from keras_amd.layers.together import quantize_rows
from keras_amd.quantization_config import QuantizationConfig, get_block_size_for_layer


def _canonical_specs(equation, input_rank):
    """(input, kernel, output) label strings with `...` replaced by fresh labels.

    Accepts `X,Y->Z`, `...X,Y->...Z` and `X...,Y->Z...`
    (keras/src/layers/core/einsum_dense.py:1728-1757, :1932-1993).
    """
    eq = equation.replace(" ", "")
    bad = ValueError(
        f"Invalid einsum equation '{equation}'. Equations must be in the "
        "form [X],[Y]->[Z], ...[X],[Y]->...[Z], or [X]...,[Y]->[Z]...."
    )
    if eq.count("->") != 1 or eq.count(",") != 1:
        raise bad
    lhs, out = eq.split("->")
    a, b = lhs.split(",")
    if "." in b:
        raise bad
    if "..." not in a and "..." not in out:
        if not (a.isalpha() and b.isalpha() and out.isalpha()):
            raise bad
        return a, b, out, 0, False
    left = a.startswith("...") and out.startswith("...")
    right = a.endswith("...") and out.endswith("...")
    if left == right:
        raise bad
    core_in = a[3:] if left else a[:-3]
    core_out = out[3:] if left else out[:-3]
    if not (core_in.isalpha() and b.isalpha() and core_out.isalpha()):
        raise bad
    if right and len(core_in) < 2:
        raise bad
    n = input_rank - len(core_in)
    spare = sorted(set(string.ascii_letters) - set(core_in) - set(b) - set(core_out))
    pad = "".join(spare[:n])
    if left:
        return pad + core_in, b, pad + core_out, n, True
    return core_in + pad, b, core_out + pad, n, False


def analyze_einsum_shapes(equation, bias_axes, input_shape, output_shape):
    """Kernel shape, bias shape and full output shape of an EinsumDense
    (keras/src/layers/core/einsum_dense.py:1700-1899)."""
    i_spec, k_spec, o_spec, elided, left = _canonical_specs(equation, len(input_shape))
    out_dims = [output_shape] if isinstance(output_shape, int) else list(output_shape)
    out_dims.insert(0, input_shape[0])
    if elided > 0 and left:
        for i in range(1, elided):
            out_dims.insert(1, input_shape[i])
    elif elided > 0:
        for i in range(len(input_shape) - elided, len(input_shape)):
            out_dims.append(input_shape[i])
    size_in = {c: input_shape[i] for i, c in enumerate(i_spec)}
    size_out = {c: out_dims[i] for i, c in enumerate(o_spec)}
    for c in i_spec:
        if c in size_out and size_out[c] is not None and size_out[c] != size_in[c]:
            raise ValueError(
                "Input shape and output shape do not match at shared "
                f"dimension '{c}'. Input shape is {size_in[c]}, "
                f"and output shape is {size_out[c]}."
            )
    for c in o_spec:
        if c not in i_spec and c not in k_spec:
            raise ValueError(
                f"Dimension '{c}' was specified in the output '{o_spec}' but has no "
                f"corresponding dim in the input spec '{i_spec}' or weight spec '{k_spec}'"
            )
    kernel_shape = []
    for c in k_spec:
        if c in size_out:
            kernel_shape.append(size_out[c])
        elif c in size_in:
            kernel_shape.append(size_in[c])
        else:
            raise ValueError(
                f"Weight dimension '{c}' did not have a match in either "
                f"the input spec '{i_spec}' or the output spec '{o_spec}'. "
                "For this layer, the weight must be fully specified."
            )
    bias_shape = None
    if bias_axes is not None:
        # labels of the user's output spec only (the padded ones never carry a bias)
        user_o = o_spec[elided:] if left else (o_spec[:-elided] if elided else o_spec)
        for c in bias_axes:
            if c not in user_o:
                raise ValueError(
                    f"Bias dimension '{c}' was requested, but is not part "
                    f"of the output spec '{user_o}'"
                )
        first = min(user_o.find(c) for c in bias_axes)
        bias_shape = [size_out[c] if c in bias_axes else 1 for c in user_o[first:]]
        if not left:
            bias_shape += [1] * elided
    return tuple(kernel_shape), (None if bias_shape is None else tuple(bias_shape)), tuple(out_dims)


def analyze_quantization_info(equation, input_rank):
    """Axes bookkeeping for per-axis quantisation of an einsum
    (keras/src/layers/core/einsum_dense.py:1902-2062).

    For the input and for the kernel: the axes the quantizer reduces, and the
    transpose / expand_dims / squeeze that turn a keepdims scale into a tensor
    that broadcasts against the einsum output.  The reference shares one scratch
    variable between its label scans and both fix-up loops; when an operand has
    more reduced axes than the output has axes missing from it, the surplus axes
    are squeezed and inserted at the last position that variable held.  That
    behaviour decides stored `kernel_scale` shapes, so it is kept.
    """
    i_spec, k_spec, o_spec, _, _ = _canonical_specs(equation, input_rank)
    parts = {}
    for name, spec in (("input", i_spec), ("kernel", k_spec)):
        parts[name] = {
            "reduced": [ax for ax, c in enumerate(spec) if c not in o_spec],
            "expand": [ax for ax, c in enumerate(o_spec) if c not in spec],
            "transpose": [spec.index(c) for c in o_spec if c in spec],
            "squeeze": [],
        }
    position = o_spec.find(k_spec[-1])
    for name in ("input", "kernel"):
        part = parts[name]
        for ax in part["reduced"]:
            if part["expand"]:
                position = part["expand"].pop(0)
            else:
                part["squeeze"].append(ax)
            part["transpose"].insert(position, ax)
    parts["specs"] = (i_spec, k_spec, o_spec)
    parts["custom_gradient_equation"] = f"{o_spec},{k_spec}->{i_spec}"
    return parts


def _adjust_scale(scale, part):
    """transpose, expand_dims, squeeze (einsum_dense.py:1650-1680)."""
    if part["transpose"]:
        scale = scale.permute(part["transpose"])
    for ax in sorted(part["expand"]):
        scale = scale.unsqueeze(ax)
    for ax in sorted(part["squeeze"], reverse=True):
        if scale.shape[ax] == 1:
            scale = scale.squeeze(ax)
    return scale


class _GemmView:
    """How an einsum `X,Y->Z` maps onto `[M, K] x [K, N]`."""

    def __init__(self, i_spec, k_spec, o_spec):
        si, sk, so = set(i_spec), set(k_spec), set(o_spec)
        if si & sk & so:
            raise NotImplementedError(
                f"labels {sorted(si & sk & so)} appear in the input, the kernel and the output: "
                "batched-kernel einsums are not lowered to the quantized GEMM"
            )
        if (si - sk - so) or (sk - si - so):
            raise NotImplementedError("einsums that sum a label out of one operand alone are not supported")
        self.contracted = [c for c in k_spec if c in si]        # kernel order
        self.kept = [c for c in o_spec if c in sk]              # output order
        self.free = [c for c in i_spec if c in so]              # input order
        self.in_perm = [i_spec.index(c) for c in self.free + self.contracted]
        self.k_perm = [k_spec.index(c) for c in self.contracted + self.kept]
        gemm_out = self.free + self.kept
        self.out_perm = [gemm_out.index(c) for c in o_spec]
        self.in_is_view = self.in_perm == list(range(len(i_spec)))
        self.k_is_view = self.k_perm == list(range(len(k_spec)))
        self.out_is_view = self.out_perm == list(range(len(o_spec)))
        # int4 stores reshape(kernel, [prod(reduced), prod(kept)]) row-major: that is the
        # [K, N] matrix only when the kernel is already laid out [contracted..., kept...]
        # with the kept labels in kernel order equal to their output order
        self.k_plain = self.k_is_view


class _BatchedView:
    """An einsum `X,Y->Z` that `_GemmView` does not take, as a stack of `[M, K] x [K, N]`
    products: labels that the input, the kernel and the output share count the products,
    a label the input alone carries is summed by giving the kernel a copy per value, and an
    einsum without a shared summed label has K = 1."""

    def __init__(self, i_spec, k_spec, o_spec):
        si, sk, so = set(i_spec), set(k_spec), set(o_spec)
        if sk - si - so:
            # (unreachable through build(): a kernel label that neither the input nor the output
            # carries has no size, and `analyze_einsum_shapes` raises ValueError for it, as the
            # reference does, keras/src/layers/core/einsum_dense.py:1854-1866)
            raise NotImplementedError(
                f"labels {sorted(sk - si - so)} are summed out of the kernel alone: the layer cannot be built")
        self.i_spec, self.k_spec, self.o_spec = i_spec, k_spec, o_spec
        self.batch = [c for c in i_spec if c in sk and c in so]
        self.free = [c for c in i_spec if c in so and c not in sk]
        self.kept = [c for c in k_spec if c in so and c not in si]
        self.contracted = [c for c in i_spec if c in sk and c not in so]
        self.input_only = [c for c in i_spec if c not in sk and c not in so]
        # the quantizer reduces the labels the output lacks; the rows it sees keep the others in
        # input order, so that its scales reshape into the keepdims shape the reference adjusts
        self.rows = [c for c in i_spec if c in so]
        self.reduced = [c for c in i_spec if c not in so]


class EinsumDense(Layer):
    def __init__(self, equation, output_shape, activation=None, bias_axes=None,
                 kernel_initializer=None, bias_initializer="zeros", dtype=None, name=None,
                 device=None, quantization_config=None, lora_rank=None, lora_alpha=None):
        super().__init__(dtype=dtype, name=name, device=device)
        self.lora_rank = lora_rank
        self.lora_alpha = lora_alpha if lora_alpha is not None else lora_rank
        self.quantization_config = quantization_config  # einsum_dense.py __init__ / build
        self.equation = equation
        self.partial_output_shape = (output_shape,) if isinstance(output_shape, int) else tuple(output_shape)
        self.bias_axes = bias_axes
        self.activation = activation if callable(activation) else _ACTIVATIONS[activation]
        self.kernel_initializer = kernel_initializer or glorot_uniform
        self.bias_initializer = bias_initializer
        self.lora_enabled = False
        self.exact_epilogue = None
        self._cache = {}

    # ---- build ---------------------------------------------------------------
    def build(self, input_shape):
        self._build_input_shape = tuple(input_shape)
        kernel_shape, bias_shape, full_output_shape = analyze_einsum_shapes(
            self.equation, self.bias_axes, tuple(input_shape), self.partial_output_shape
        )
        self.full_output_shape = full_output_shape
        self.input_rank = len(input_shape)
        self.original_kernel_shape = kernel_shape
        if self.quantization_mode is not None:
            self.quantized_build(kernel_shape, mode=self.quantization_mode,
                                 config=self.quantization_config)
        if self.quantization_mode not in ("int8", "int4"):
            self._kernel = self.add_weight(
                name="kernel", shape=kernel_shape, initializer=self.kernel_initializer, trainable=True
            )
        if bias_shape is not None:
            self.bias = self.add_weight(
                name="bias", shape=bias_shape, initializer=self.bias_initializer, trainable=True
            )
        else:
            self.bias = None
        self.built = True
        if self.lora_rank:
            self.enable_lora(self.lora_rank, lora_alpha=self.lora_alpha)  # einsum_dense.py:234-235

    @property
    def kernel(self):
        if not self.built:
            raise AttributeError("You must build the layer before accessing `kernel`.")
        kernel = as_tensor(self._kernel)
        if self.quantization_mode == "int4":
            kernel = quantizers.unpack_int4(kernel, self._int4_unpacked_column_size, axis=-1)
            kernel = kernel.reshape(self.original_kernel_shape)
        if self.lora_enabled:  # einsum_dense.py:298-306
            delta = (self.lora_alpha / self.lora_rank) * torch.matmul(
                as_tensor(self.lora_kernel_a), as_tensor(self.lora_kernel_b))
            kernel = torch.add(kernel, delta).to(to_torch_dtype(self.compute_dtype))
        return kernel

    def enable_lora(self, rank, lora_alpha=None, a_initializer="he_uniform", b_initializer="zeros"):
        """keras/src/layers/core/einsum_dense.py:327-385: float32 `lora_kernel_a` of the kernel's
        shape with its last axis replaced by `rank`, `lora_kernel_b` [rank, last axis]."""
        if not self.built:
            raise ValueError("Cannot enable lora on a layer that isn't yet built.")
        if self.lora_enabled:
            raise ValueError("lora is already enabled. This can only be done once per layer.")
        if self.quantization_mode == "int4":
            shape = tuple(self.original_kernel_shape)
        else:
            shape = tuple(self._kernel.shape)
        self.lora_kernel_a = self.add_weight(name="lora_kernel_a", shape=shape[:-1] + (rank,), dtype="float32",
                                             initializer=lora_initializer(a_initializer), trainable=True)
        self.lora_kernel_b = self.add_weight(name="lora_kernel_b", shape=(rank, shape[-1]), dtype="float32",
                                             initializer=lora_initializer(b_initializer), trainable=True)
        self.lora_enabled = True
        self.lora_rank = rank
        self.lora_alpha = lora_alpha if lora_alpha is not None else rank

    def _quantized_call_with_lora(self, quantized_call, inputs):
        """einsum_dense.py:1109-1118, :1251-1261: de-scaled quantized product, + low-rank term, cast,
        + bias, activation (the kernels run without their fused bias here)."""
        bias, activation = self.bias, self.activation
        self.bias, self.activation, self.lora_enabled = None, None, False
        try:
            x = quantized_call(inputs)
        finally:
            self.bias, self.activation, self.lora_enabled = bias, activation, True
        lora_x = torch.einsum(self.equation, inputs, self.read(self.lora_kernel_a))
        lora_x = torch.matmul(lora_x, self.read(self.lora_kernel_b))
        x = torch.add(x, (self.lora_alpha / self.lora_rank) * lora_x).to(to_torch_dtype(self.compute_dtype))
        if bias is not None:
            x = torch.add(x, self.read(bias))
        if activation is not None:
            x = activation(x)
        return x

    def _get_kernel_with_merged_lora(self):
        """`(kernel, kernel_scale, kernel_zero)` as saved
        (keras/src/layers/core/einsum_dense.py:1493-1623): with LoRA enabled, de-quantise (int8: the
        kernel over its scale taken back through the expand / squeeze / transpose bookkeeping;
        int4: as Dense on the flat matrix, reshaped), add `(alpha / rank) * a . b`, quantise again as
        `quantize()` does."""
        mode = self.quantization_mode
        if mode is None:
            return self.kernel, None, None
        kernel_zero = as_tensor(self.kernel_zero) if hasattr(self, "kernel_zero") else None
        if not self.lora_enabled:
            return as_tensor(self._kernel), as_tensor(self.kernel_scale), kernel_zero
        cd = to_torch_dtype(self.compute_dtype)
        if mode == "int4":
            unpacked = quantizers.unpack_int4(as_tensor(self._kernel), self._int4_unpacked_column_size, axis=-1)
            block_size = self._int4_block_size
            grouped = block_size is not None and block_size != -1
            if grouped:
                kernel_fp = quantizers.dequantize_with_sz_map(
                    unpacked, as_tensor(self.kernel_scale), kernel_zero, as_tensor(self.g_idx), group_axis=0)
            else:
                kernel_fp = torch.divide(unpacked.to(cd), as_tensor(self.kernel_scale))
            kernel_fp = kernel_fp.reshape(self.original_kernel_shape)
        elif mode == "int8":
            part = self._quant_info["kernel"]
            scale = as_tensor(self.kernel_scale)
            for ax in sorted(part["squeeze"]):
                scale = scale.unsqueeze(ax)
            for ax in sorted(part["expand"], reverse=True):
                scale = scale.squeeze(ax)
            if part["transpose"]:
                perm = part["transpose"]
                scale = scale.permute(sorted(range(len(perm)), key=perm.__getitem__))
            kernel_fp = torch.divide(as_tensor(self._kernel), scale)
        else:
            raise self._quantization_mode_error(mode)
        update = (self.lora_alpha / self.lora_rank) * torch.matmul(
            as_tensor(self.lora_kernel_a), as_tensor(self.lora_kernel_b))
        merged = torch.add(kernel_fp, update)
        if mode == "int4":
            flat = merged.reshape(self._int4_rows, self._int4_unpacked_column_size)
            if grouped:
                q, new_scale, kernel_zero = quantizers.abs_max_quantize_grouped_with_zero_point(
                    flat, block_size=block_size, to_numpy=True)
            else:
                q, new_scale = quantizers.abs_max_quantize(flat, axis=0, value_range=(-8, 7), dtype="int8",
                                                           to_numpy=True)
                new_scale = torch.squeeze(new_scale, dim=0)
                kernel_zero = None
            new_kernel, _, _ = quantizers.pack_int4(q.to(self.device), axis=-1)
        else:
            new_kernel, new_scale = quantizers.abs_max_quantize(
                merged, axis=tuple(self._kernel_reduced_axes), to_numpy=True)
            new_scale = _adjust_scale(new_scale, self._quant_info["kernel"]).contiguous()
            kernel_zero = None
        return new_kernel, new_scale, kernel_zero

    def call(self, inputs, training=None):
        if self.lora_enabled:
            x = torch.einsum(self.equation, inputs, self.kernel)
            if self.bias is not None:
                x = torch.add(x, self.read(self.bias))
            return self.activation(x) if self.activation is not None else x
        x = torch.einsum(self.equation, inputs, self.read(self._kernel))
        if self.bias is not None:
            x = torch.add(x, self.read(self.bias))
        if self.activation is not None:
            x = self.activation(x)
        return x

    # ---- quantized variables -----------------------------------------------------
    def _set_quantization_info(self):
        if hasattr(self, "_quant_info"):
            return
        info = analyze_quantization_info(self.equation, self.input_rank)
        self._quant_info = info
        self._input_reduced_axes = info["input"]["reduced"]
        self._kernel_reduced_axes = info["kernel"]["reduced"]
        self._custom_gradient_equation = info["custom_gradient_equation"]
        self._gemm = None
        self._batched = None
        try:
            self._gemm = _GemmView(*info["specs"])
        except NotImplementedError as e:
            self._gemm_error = e
            try:
                self._batched = _BatchedView(*info["specs"])
            except NotImplementedError as e2:
                self._gemm_error = e2

    def quantized_build(self, kernel_shape, mode, config=None):
        if mode == "int8":
            self._int8_build(kernel_shape, config)
        elif mode == "int4":
            self._int4_build(kernel_shape, config)
        else:
            raise self._quantization_mode_error(mode)
        self._is_quantized = True

    def _get_kernel_scale_shape(self, kernel_shape):
        """Per-channel scale shape: the kernel shape with reduced axes set to 1, taken
        through the kernel's transpose / expand / squeeze (einsum_dense.py:1478-1491)."""
        probe = torch.empty(
            [1 if ax in self._kernel_reduced_axes else d for ax, d in enumerate(kernel_shape)],
            device="meta",
        )
        return tuple(_adjust_scale(probe, self._quant_info["kernel"]).shape)

    def _int8_build(self, kernel_shape, config=None):
        self._set_quantization_info()
        self.inputs_quantizer = QuantizationConfig.activation_quantizer_or_default(
            config, quantizers.AbsMaxQuantizer()
        )
        self.quantization_axis = tuple(self._input_reduced_axes)
        self._kernel = self.add_weight(name="kernel", shape=kernel_shape, dtype="int8")
        self.kernel_scale = self.add_weight(
            name="kernel_scale", shape=self._get_kernel_scale_shape(kernel_shape), initializer="ones"
        )

    def _flat_dims(self, kernel_shape):
        rows = cols = 1
        for ax, d in enumerate(kernel_shape):
            if ax in self._kernel_reduced_axes:
                rows *= d
            else:
                cols *= d
        return rows, cols

    def _int4_build(self, kernel_shape, config=None):
        self._set_quantization_info()
        self.inputs_quantizer = QuantizationConfig.activation_quantizer_or_default(config, None)
        self.quantization_axis = tuple(self._input_reduced_axes)
        self.original_kernel_shape = tuple(kernel_shape)
        rows, cols = self._flat_dims(kernel_shape)
        block_size = get_block_size_for_layer(self, config)
        use_grouped = block_size is not None and block_size != -1
        self._int4_block_size = block_size if use_grouped else None
        self._int4_unpacked_column_size = cols
        self._int4_rows = rows
        self._kernel = self.add_weight(name="kernel", shape=(rows, (cols + 1) // 2), dtype="int8")
        scale_shape = (math.ceil(rows / block_size), cols) if use_grouped else (cols,)
        self.kernel_scale = self.add_weight(name="kernel_scale", shape=scale_shape, initializer="ones")
        if use_grouped:
            self.kernel_zero = self.add_weight(name="kernel_zero", shape=scale_shape, dtype="int8")
            self.g_idx = self.add_weight(
                name="g_idx", shape=(rows,), dtype="float32",
                initializer=lambda shape, dtype: torch.floor_divide(
                    torch.arange(rows, dtype=dtype), block_size),
            )

    # ---- quantize ---------------------------------------------------------------------
    def _quantize(self, mode, config, type_check=True):
        if type_check and type(self) is not EinsumDense:
            raise self._not_implemented_error(self.quantize)
        self.quantization_config = config
        kernel_shape = self._kernel.shape
        self._set_quantization_info()
        kernel_zero = None
        if mode == "int8":
            weight_quantizer = QuantizationConfig.weight_quantizer_or_default(
                config, quantizers.AbsMaxQuantizer(axis=self._kernel_reduced_axes)
            )
            kernel_value, kernel_scale = weight_quantizer(as_tensor(self._kernel), to_numpy=True)
            kernel_scale = _adjust_scale(kernel_scale, self._quant_info["kernel"]).contiguous()
        elif mode == "int4":
            block_size = get_block_size_for_layer(self, config)
            use_grouped = block_size is not None and block_size != -1
            rows, cols = self._flat_dims(kernel_shape)
            flat = as_tensor(self._kernel).reshape(rows, cols)
            if not use_grouped:
                q4, kernel_scale = quantizers.abs_max_quantize(
                    flat, axis=0, value_range=(-8, 7), dtype="int8", to_numpy=True
                )
                kernel_scale = torch.squeeze(kernel_scale, dim=0)
            else:
                q4, kernel_scale, kernel_zero = quantizers.abs_max_quantize_grouped_with_zero_point(
                    flat, block_size=block_size, to_numpy=True
                )
            kernel_value, _, _ = quantizers.pack_int4(q4.to(self.device), axis=-1)
        else:
            raise self._quantization_mode_error(mode)
        self._variables = [v for v in self._variables if v is not self._kernel]
        del self._kernel
        self.quantized_build(kernel_shape, mode, config)
        self._kernel.assign(kernel_value)
        self.kernel_scale.assign(kernel_scale)
        if kernel_zero is not None:
            self.kernel_zero.assign(kernel_zero)
        if self.dtype_policy.quantization_mode is None:
            policy_name = mode
            if mode == "int4":
                block_size = get_block_size_for_layer(self, config)
                policy_name = f"int4/{-1 if block_size is None else block_size}"
            self._dtype_policy = dtype_policies.get(f"{policy_name}_from_{self.dtype_policy.name}")
        self._cache.clear()

    # ---- helpers ---------------------------------------------------------------------------
    def _cached(self, key, var, make):
        if var is None:
            return None
        hit = self._cache.get(key)
        if hit is not None and hit[0] == var.version and hit[1] is var:
            return hit[2]
        value = make(as_tensor(var))
        if (hit is not None and isinstance(hit[2], torch.Tensor) and isinstance(value, torch.Tensor)
                and hit[2].shape == value.shape and hit[2].dtype == value.dtype and hit[2].device == value.device):
            # a rebuilt copy keeps its address: a captured HIP graph that holds the old copy's address
            # goes on reading live memory (the new values) instead of memory that was freed
            hit[2].copy_(value)
            value = hit[2]
        self._cache[key] = (var.version, var, value)
        return value

    def _gemm_view(self):
        if self._gemm is None:
            raise self._gemm_error
        return self._gemm

    def _strip_operands(self, rows, input_dim, units, grouped, block_size):
        """As Dense._strip_operands: the operands of the strip-linear decode route, or None."""
        cd = to_torch_dtype(self.compute_dtype)
        if not (0 < rows <= kops.STRIP_MAX_ROWS and cd == torch.bfloat16
                and kops.int4_strip_supported(rows, input_dim, units, block_size if grouped else None)):
            return None
        spec = dict(units=units,
                    shadow=self._cached("w4s", self._kernel, lambda t: kops.int4_strip_copy(t, units)))
        if grouped:
            scale, zero = self.kernel_scale, self.kernel_zero
            stamp = (id(scale), scale.version, id(zero), zero.version)
            hit = self._cache.get("w4s_params")
            if hit is None or hit[0] != stamp:
                value = kops.int4_strip_params(as_tensor(scale), as_tensor(zero), input_dim, units, block_size)
                hit = self._cache["w4s_params"] = (stamp, None, value)
            spec["gparams"] = hit[2]
        else:
            spec["kernel_scale"] = self._cached("kernel_scale", self.kernel_scale,
                                                lambda t: t.to(cd).reshape(-1).contiguous())
        return spec

    def _input_rows(self, inputs, gv):
        x = inputs if gv.in_is_view else inputs.permute(gv.in_perm)
        k = 1
        for d in x.shape[len(gv.free):]:
            k *= d
        free_shape = tuple(x.shape[:len(gv.free)])
        return x.reshape(-1, k), free_shape

    def _finish(self, y2, free_shape, gv, fused_bias):
        kept_shape = tuple(self.full_output_shape_of(c) for c in gv.kept)
        y = y2.reshape(*free_shape, *kept_shape)
        if not gv.out_is_view:
            y = y.permute(gv.out_perm)
        if self.bias is not None and not fused_bias:
            y = torch.add(y, self.read(self.bias))
        if self.activation is not None:
            y = self.activation(y)
        return y

    def full_output_shape_of(self, label):
        k_spec = self._quant_info["specs"][1]
        return self.original_kernel_shape[k_spec.index(label)]

    def _fusable_bias(self, gv, n):
        """The bias as an [N] vector when it spans exactly the kept (kernel) axes, which
        are then the trailing output axes; otherwise None and the bias is added after."""
        o_spec = self._quant_info["specs"][2]
        trailing = list(o_spec[len(o_spec) - len(gv.kept):]) == gv.kept
        if self.bias is None:
            # (a row lent by `call_add` for a one-row call stands in for the bias)
            return (getattr(self, "_row_bias", None) if trailing else None), True
        kept_shape = tuple(self.full_output_shape_of(c) for c in gv.kept)
        if trailing and self.bias.shape == kept_shape:
            cd = to_torch_dtype(self.compute_dtype)
            return self._cached("bias", self.bias, lambda t: t.to(cd).reshape(-1).contiguous()), True
        return None, False

    def _row_bias_ok(self):
        if self.bias is not None or self.activation is not None or not self.built:
            return False
        if getattr(self, "_gemm", None) is None:
            return False
        gv = self._gemm_view()
        o_spec = self._quant_info["specs"][2]
        return list(o_spec[len(o_spec) - len(gv.kept):]) == gv.kept

    def _rows_of(self, inputs):
        return self._input_rows(inputs, self._gemm_view())[0].shape[0]

    # ---- quantized forward -----------------------------------------------------------------
    def _int8_call(self, inputs, training=None):
        """keras/src/layers/core/einsum_dense.py:1030-1118 as quantise-rows + int8 GEMM."""
        if self.lora_enabled:
            return self._quantized_call_with_lora(self._int8_call, inputs)
        if self._gemm is None and self._batched is not None:
            return self._int8_call_batched(inputs)
        gv = self._gemm_view()
        x2, free_shape = self._input_rows(inputs, gv)
        cd = to_torch_dtype(self.compute_dtype)

        def kernel_matrix(t):
            k2 = t if gv.k_is_view else t.permute(gv.k_perm)
            return k2.reshape(x2.shape[1], -1).contiguous()

        k2 = self._cached("kernel2d", self._kernel, kernel_matrix)
        n = k2.shape[1]
        bias, fused = self._fusable_bias(gv, n)
        if not self.inputs_quantizer:
            # Weight-only (einsum_dense.py:1085-1101).  The torch backend divides every weight
            # by its scale first and contracts in float; here the contraction runs on the
            # exact int8 values and the scale divides the result -- the same quantity without
            # the per-weight rounding.
            y2 = kops.int8_weight_only_matmul(
                x2, k2,
                self._cached("kernel_scale", self.kernel_scale,
                             lambda t: t.to(cd).reshape(-1).contiguous()),
                bias=bias,
                prepacked=self._cached("prepacked", self._kernel, lambda t: kops.prepack_int8_kernel(kernel_matrix(t))))
            return self._finish(y2, free_shape, gv, fused)
        exact = self.exact_epilogue
        if exact is None:
            exact = True
        if exact and int8_strip_route(self.inputs_quantizer, x2, n):
            # decode sizes, as Dense: one launch from the strip-linear copy of the [K, N] matrix
            y2 = kops.int8_dense_strip(
                x2, self._cached("w8s", self._kernel, lambda t: kops.int8_strip_copy(kernel_matrix(t))), n,
                self._cached("kernel_scale", self.kernel_scale, lambda t: t.to(cd).reshape(-1).contiguous()),
                bias=bias, epsilon=self.inputs_quantizer.epsilon,
                value_range=self.inputs_quantizer.value_range,
                quantize=lambda rows: quantize_rows(self.inputs_quantizer, rows))
            return self._finish(y2, free_shape, gv, fused)
        q, scale = quantize_rows(self.inputs_quantizer, x2)
        y2 = kops.int8_matmul(
            q, k2, a_scale=scale,
            kernel_scale=self._cached("kernel_scale", self.kernel_scale,
                                      lambda t: t.to(cd).reshape(-1).contiguous()),
            bias=bias, out_dtype=cd, exact_epilogue=exact,
            # the tile GEMM's operand: the decode kernel's strip-linear copy where it can take it
            # (one derived copy per layer), else the [N, K] copy
            **(dict(strip=self._cached("w8s", self._kernel, lambda t: kops.int8_strip_copy(kernel_matrix(t))))
               if x2.shape[1] % 128 == 0 else
               dict(prepacked=self._cached("prepacked", self._kernel,
                                           lambda t: kops.prepack_int8_kernel(kernel_matrix(t))))),
        )
        return self._finish(y2, free_shape, gv, fused)

    def _int8_call_batched(self, inputs):
        """keras/src/layers/core/einsum_dense.py:1030-1118 for equations with labels shared by
        input, kernel and output, without a summed label, or with one the input alone carries
        (e.g. "abcde,afce->acdbf", "a,b->ab", "ab,ab->a", einsum_dense_test.py:598-629).

        The integer einsum runs as one exact int8 GEMM per value of the shared labels (raw int32
        accumulators); the de-scale is then the reference's own broadcast, `acc / (inputs_scale *
        kernel_scale)` with both scales in the shapes its transpose / expand / squeeze
        bookkeeping gives them, so results (and result shapes) are the reference's for every
        equation it accepts."""
        bv = self._batched
        cd = to_torch_dtype(self.compute_dtype)
        if not self.inputs_quantizer:
            # weight-only (einsum_dense.py:1085-1101): every weight divided by its scale, float einsum
            ks = as_tensor(self.kernel_scale).to(cd)
            part = self._quant_info["kernel"]
            for ax in sorted(part["squeeze"]):
                ks = ks.unsqueeze(ax)
            for ax in sorted(part["expand"], reverse=True):
                ks = ks.squeeze(ax)
            if part["transpose"]:
                perm = part["transpose"]
                ks = ks.permute(sorted(range(len(perm)), key=perm.__getitem__))
            y = torch.einsum(self.equation, inputs.to(cd), torch.divide(as_tensor(self._kernel).to(cd), ks))
        else:
            size = dict(zip(bv.i_spec, inputs.shape))
            size.update(zip(bv.k_spec, self._kernel.shape))
            prod = lambda labels: math.prod(size[c] for c in labels)
            # quantise over the labels the output lacks: rows in input order, those labels last
            x2 = inputs.permute([bv.i_spec.index(c) for c in bv.rows + bv.reduced]).reshape(
                prod(bv.rows), prod(bv.reduced))
            q2, scale = quantize_rows(self.inputs_quantizer, x2.contiguous())
            s_in = scale.reshape([1 if c in bv.reduced else size[c] for c in bv.i_spec])
            s_adj = _adjust_scale(s_in, self._quant_info["input"])
            # [batch, M, K] rows against [batch, K, N] kernels
            q_labels = bv.rows + bv.reduced
            q = q2.reshape([size[c] for c in q_labels])
            order = bv.batch + bv.free + bv.contracted + bv.input_only
            q3 = q.permute([q_labels.index(c) for c in order]).reshape(
                prod(bv.batch), prod(bv.free), prod(bv.contracted + bv.input_only)).contiguous()

            def kernel_stack(t):
                k = t.permute([bv.k_spec.index(c) for c in bv.batch + bv.contracted + bv.kept])
                k = k.reshape(prod(bv.batch), prod(bv.contracted), 1, prod(bv.kept))
                k = k.expand(-1, -1, prod(bv.input_only), -1)  # a copy per value of an input-only label
                return k.reshape(prod(bv.batch), -1, prod(bv.kept)).contiguous()

            shape_key = tuple(size[c] for c in bv.input_only)
            hit = self._cache.get("kernel_stack")
            if hit is None or hit[0] != (self._kernel.version, shape_key) or hit[1] is not self._kernel:
                hit = self._cache["kernel_stack"] = ((self._kernel.version, shape_key), self._kernel,
                                                     kernel_stack(as_tensor(self._kernel)))
            k3 = hit[2]
            acc = torch.stack([kops.int8_matmul(q3[b], k3[b], want_acc=True, want_y=False)
                               for b in range(q3.shape[0])])
            acc = acc.reshape([size[c] for c in bv.batch + bv.free + bv.kept])
            have = bv.batch + bv.free + bv.kept
            acc = acc.permute([have.index(c) for c in bv.o_spec])
            y = torch.divide(acc.to(cd), torch.multiply(s_adj, as_tensor(self.kernel_scale).to(cd)))
        if self.bias is not None:
            y = torch.add(y, self.read(self.bias))
        if self.activation is not None:
            y = self.activation(y)
        return y

    def _int4_call_batched(self, inputs):
        """keras/src/layers/core/einsum_dense.py:1120-1261 for the equations `_int8_call_batched`
        takes: the kernel is de-quantised once (kept until a variable changes), reshaped to its own
        shape and contracted in the compute dtype, as the reference does on every call."""
        cd = to_torch_dtype(self.compute_dtype)
        block_size = self._int4_block_size
        grouped = block_size is not None and block_size > 0
        variables = [self._kernel, self.kernel_scale] + ([self.kernel_zero, self.g_idx] if grouped else [])
        stamp = tuple((id(v), v.version) for v in variables) + (cd,)
        hit = self._cache.get("int4_float_kernel")
        if hit is None or hit[0] != stamp:
            unpacked = quantizers.unpack_int4(as_tensor(self._kernel), self._int4_unpacked_column_size, axis=-1)
            scale = as_tensor(self.kernel_scale).to(cd)
            if grouped:
                fk = quantizers.dequantize_with_sz_map(
                    unpacked, scale, as_tensor(self.kernel_zero), as_tensor(self.g_idx), group_axis=0).to(cd)
            else:
                fk = torch.divide(unpacked.to(cd), scale)
            hit = self._cache["int4_float_kernel"] = (stamp, fk.reshape(self.original_kernel_shape))
        if self.inputs_quantizer and not grouped:
            # einsum_dense.py:1163-1184 (a grouped kernel never reads the quantizer, :1188-1261): rows
            # quantised over the labels the output lacks, cast back to the compute dtype, contracted
            # against the float kernel, divided by the input scale in the shape the reference's
            # transpose / expand / squeeze bookkeeping gives it
            bv = self._batched
            size = dict(zip(bv.i_spec, inputs.shape))
            prod = lambda labels: math.prod(size[c] for c in labels)
            q_labels = bv.rows + bv.reduced
            x2 = inputs.to(cd).permute([bv.i_spec.index(c) for c in q_labels]).reshape(prod(bv.rows), prod(bv.reduced))
            q2, scale = quantize_rows(self.inputs_quantizer, x2.contiguous())
            s_in = scale.reshape([1 if c in bv.reduced else size[c] for c in bv.i_spec])
            q = q2.reshape([size[c] for c in q_labels]).permute([q_labels.index(c) for c in bv.i_spec])
            y = torch.einsum(self.equation, q.to(cd), hit[1])
            y = torch.divide(y, _adjust_scale(s_in, self._quant_info["input"]))
        else:
            y = torch.einsum(self.equation, inputs.to(cd), hit[1])
        if self.bias is not None:
            y = torch.add(y, self.read(self.bias))
        if self.activation is not None:
            y = self.activation(y)
        return y

    def _int4_call(self, inputs, training=None):
        """keras/src/layers/core/einsum_dense.py:1120-1261, weight-only."""
        if self.lora_enabled:
            return self._quantized_call_with_lora(self._int4_call, inputs)
        if self._gemm is None and self._batched is not None:
            return self._int4_call_batched(inputs)
        gv = self._gemm_view()
        x2, free_shape = self._input_rows(inputs, gv)
        cd = to_torch_dtype(self.compute_dtype)
        block_size = self._int4_block_size
        grouped = block_size is not None and block_size > 0
        if not gv.k_plain:
            return self._int4_call_dequantized(x2, free_shape, gv, cd, grouped)
        bias, fused = self._fusable_bias(gv, self._int4_unpacked_column_size)
        if grouped:
            require_default_g_idx(self, block_size)  # (the de-quantised route above reads g_idx)
        # (a grouped kernel ignores an activation quantizer, as the reference's sub-channel branch
        # does: einsum_dense.py:1188-1261 never reads it)
        if self.inputs_quantizer and not grouped:
            # Activation-quantized, per-channel (einsum_dense.py:1163-1187).  The torch
            # backend contracts the quantised rows, cast back to float, with the kernel
            # divided by its scale weight by weight; here the contraction is the exact int32
            # one and both scales divide the result -- the same quantity without the
            # per-weight rounding.
            q, scale = quantize_rows(self.inputs_quantizer, x2)
            unpacked = quantizers.unpack_int4(
                as_tensor(self._kernel), self._int4_unpacked_column_size, axis=-1)
            y2 = kops.int8_matmul(
                q, unpacked, a_scale=scale,
                kernel_scale=self._cached("kernel_scale", self.kernel_scale,
                                          lambda t: t.to(cd).reshape(-1).contiguous()),
                bias=bias, out_dtype=cd, exact_epilogue=True)
            return self._finish(y2, free_shape, gv, fused)
        from keras_amd.layers.dense import kmajor_rows

        units = self._int4_unpacked_column_size
        strip = (self._strip_operands(x2.shape[0], x2.shape[1], units, grouped, block_size)
                 if x2.dtype == torch.bfloat16 else None)
        if strip is not None:
            # decode sizes: the strip-linear copy of the kernel (one launch, no scratch)
            per_row = bias is not None and x2.shape[0] > 1 and bias.numel() == x2.shape[0] * units
            y2 = kops.int4_matmul_strip(
                x2, strip["shadow"], units, kernel_scale=strip.get("kernel_scale"),
                gparams=strip.get("gparams"), block_size=block_size if grouped else None,
                bias=None if per_row else bias, addend=bias if per_row else None)
            return self._finish(y2, free_shape, gv, fused)
        if (x2.dtype == torch.bfloat16 and kmajor_rows(x2.shape[0], units, x2.shape[1])
                and kops.int4_kmajor_supported(x2.shape[0], x2.shape[1], units,
                                               block_size if grouped else None)):
            # as Dense: the int4 tile kernel, from the strip-linear copy the decode kernel streams
            # where it takes the shape, else from a K-contiguous copy; the kernel is read once as int4
            scale_cd = self._cached("kernel_scale", self.kernel_scale, lambda t: t.to(cd).contiguous())
            if kops.int4_tiles_strip_supported(x2.shape[0], x2.shape[1], units, block_size if grouped else None):
                y2 = kops.int4_matmul_tiles_strip(
                    x2, self._cached("w4s", self._kernel, lambda t: kops.int4_strip_copy(t, units)), units,
                    scale_cd, kernel_zero=as_tensor(self.kernel_zero) if grouped else None,
                    block_size=block_size if grouped else None, bias=bias)
            else:
                y2 = kops.int4_matmul_kmajor(
                    x2, self._cached("kmajor", self._kernel, lambda t: kops.int4_kmajor_copy(t, units)),
                    scale_cd, kernel_zero=as_tensor(self.kernel_zero) if grouped else None,
                    block_size=block_size if grouped else None, bias=bias)
            return self._finish(y2, free_shape, gv, fused)
        y2 = kops.int4_matmul(
            x2, as_tensor(self._kernel),
            self._cached("kernel_scale", self.kernel_scale, lambda t: t.to(cd).contiguous()),
            units,
            kernel_zero=as_tensor(self.kernel_zero) if grouped else None,
            block_size=block_size if grouped else None,
            bias=bias,
        )
        return self._finish(y2, free_shape, gv, fused)

    def _int8_together_spec(self, inputs):
        """As Dense._int8_together_spec, for GEMM-shaped equations."""
        if (not self.built or self.quantization_mode != "int8" or self.lora_enabled
                or self.exact_epilogue is False or getattr(self, "_gemm", None) is None):
            return None
        gv = self._gemm_view()
        x2, free_shape = self._input_rows(inputs, gv)
        cd = to_torch_dtype(self.compute_dtype)

        def kernel_matrix(t):
            k2 = t if gv.k_is_view else t.permute(gv.k_perm)
            return k2.reshape(x2.shape[1], -1).contiguous()

        n = 1
        for c in gv.kept:
            n *= self.full_output_shape_of(c)
        if not int8_strip_route(self.inputs_quantizer, x2, n):
            return None
        bias, fused = self._fusable_bias(gv, n)
        if bias is not None and bias.numel() != n:
            return None
        q = self.inputs_quantizer
        return dict(x2=x2, settings=(float(q.epsilon), tuple(float(v) for v in q.value_range)), quantizer=q,
                    kernel=dict(shadow=self._cached("w8s", self._kernel,
                                                    lambda t: kops.int8_strip_copy(kernel_matrix(t))),
                                units=n, bias=bias,
                                kernel_scale=self._cached("kernel_scale", self.kernel_scale,
                                                          lambda t: t.to(cd).reshape(-1).contiguous())),
                    finish=lambda y2: self._finish(y2, free_shape, gv, fused))

    def _int4_together_spec(self, inputs):
        """As Dense._int4_together_spec, for equations whose input rows and stored kernel are
        the GEMM's operands as they lie (e.g. "btd,dnh->btnh")."""
        if (not self.built or self.quantization_mode != "int4" or self.inputs_quantizer
                or self.lora_enabled or getattr(self, "_gemm", None) is None):
            return None
        gv = self._gemm_view()
        if not (gv.k_plain and gv.in_is_view):
            return None
        cd = to_torch_dtype(self.compute_dtype)
        block_size = self._int4_block_size
        grouped = block_size is not None and block_size > 0
        if grouped:
            require_default_g_idx(self, block_size)
        x2, free_shape = self._input_rows(inputs, gv)
        bias, fused = self._fusable_bias(gv, self._int4_unpacked_column_size)
        strip = (self._strip_operands(x2.shape[0], x2.shape[1], self._int4_unpacked_column_size, grouped,
                                      block_size) if x2.dtype == torch.bfloat16 else None)
        if strip is not None:
            strip["bias"] = bias
        return dict(
            x2=x2, block_size=block_size if grouped else None, strip=strip,
            kernel=dict(kernel_packed=as_tensor(self._kernel),
                        kernel_scale=self._cached("kernel_scale", self.kernel_scale,
                                                  lambda t: t.to(cd).contiguous()),
                        units=self._int4_unpacked_column_size,
                        kernel_zero=as_tensor(self.kernel_zero) if grouped else None, bias=bias),
            finish=lambda y2: self._finish(y2, free_shape, gv, fused))

    def _int4_dequantized_kernel(self, gv, cd, grouped):
        """The float kernel of einsum_dense.py:1143-1150 / :1213-1222 (unpack, divide by the
        scale | dequantize_with_sz_map, cast, reshape to the kernel's own shape), then laid
        out as the [N, K] operand of the float GEMM.  Kept until a variable changes."""
        variables = [self._kernel, self.kernel_scale]
        if grouped:
            variables += [self.kernel_zero, self.g_idx]
        stamp = tuple((id(v), v.version) for v in variables) + (cd,)
        hit = self._cache.get("int4_dequantized")
        if hit is not None and hit[0] == stamp:
            return hit[1], hit[2]
        unpacked = quantizers.unpack_int4(
            as_tensor(self._kernel), self._int4_unpacked_column_size, axis=-1)
        scale = as_tensor(self.kernel_scale).to(cd)
        if grouped:
            fk = quantizers.dequantize_with_sz_map(
                unpacked, scale, as_tensor(self.kernel_zero), as_tensor(self.g_idx), group_axis=0
            ).to(cd)
        else:
            fk = torch.divide(unpacked.to(cd), scale)
        fk = fk.reshape(self.original_kernel_shape).permute(gv.k_perm)
        k = 1
        for c in gv.contracted:
            k *= self.full_output_shape_of(c)
        w_nk = fk.reshape(k, -1).t().contiguous()
        if cd == torch.bfloat16:
            wt, parts = w_nk, 1
        else:
            wt, parts = kops.split_f32_kernel(w_nk.to(torch.float32)), 3
        self._cache["int4_dequantized"] = (stamp, wt, parts)
        return wt, parts

    def _int4_call_dequantized(self, x2, free_shape, gv, cd, grouped):
        """int4 kernels stored as a row-major reshape of a kernel whose contracted axes are not
        leading (e.g. "btd,ndh->btnh"): a stored column then mixes output columns and rows of
        K, so its scale cannot be taken out of the sum.  The reference's order is the only
        one: de-quantise, reshape, contract in the compute dtype."""
        if x2.dtype not in (torch.bfloat16, torch.float32):
            raise TypeError(f"int4 EinsumDense computes in bfloat16 or float32, got {x2.dtype}")
        wt, parts = self._int4_dequantized_kernel(gv, cd, grouped)
        if self.inputs_quantizer and not grouped:
            # einsum_dense.py:1163-1184: quantised rows, cast back to float, against the float
            # kernel; then the division by the input scale, then the bias
            q, scale = quantize_rows(self.inputs_quantizer, x2)
            y2 = kops.float_matmul_nk(q.to(cd), wt, parts)
            y2 = torch.divide(y2, scale.to(cd))
            return self._finish(y2, free_shape, gv, False)
        bias, fused = self._fusable_bias(gv, wt.shape[0])
        y2 = kops.float_matmul_nk(x2.to(cd), wt, parts, bias=bias)
        return self._finish(y2, free_shape, gv, fused)

    # ---- serialization -------------------------------------------------------------------------
    def get_config(self):
        config = {
            "name": self.name,
            "output_shape": list(self.partial_output_shape),
            "equation": self.equation,
            "activation": activation_name(self.activation),
            "bias_axes": self.bias_axes,
            "dtype": self.dtype_policy.name,
            "quantization_config": serialize_quantization_config(self.quantization_config),
        }
        if self.lora_rank:
            config["lora_rank"] = self.lora_rank
            config["lora_alpha"] = self.lora_alpha
        return config

    @property
    def variable_serialization_spec(self):
        """einsum_dense.py:560-610, the modes built here."""
        return {
            None: ["kernel", "bias"],
            "int8": ["kernel", "bias", "kernel_scale"],
            "int4": ["kernel", "bias", "kernel_scale", "kernel_zero", "g_idx"],
        }

    def save_own_variables(self, store):
        if not self.built:
            return
        mode = self.quantization_mode
        kernel_value, merged_scale, merged_zero = self._get_kernel_with_merged_lora()
        idx = 0
        for name in self.variable_serialization_spec[mode]:
            if name == "kernel":
                value = kernel_value
            elif name == "bias" and self.bias is None:
                continue
            elif name == "kernel_zero" and mode == "int4":
                if merged_zero is None:
                    continue
                value = merged_zero
            elif name == "g_idx" and not hasattr(self, name):
                continue
            elif name == "kernel_scale" and mode in ("int4", "int8"):
                value = merged_scale
            else:
                value = getattr(self, name)
            store[str(idx)] = as_tensor(value)
            idx += 1

    def load_own_variables(self, store):
        if not self.built:
            return
        idx = 0
        for name in self.variable_serialization_spec[self.quantization_mode]:
            if name == "kernel":
                target = self._kernel
            elif name == "bias" and self.bias is None:
                continue
            elif name in ("kernel_zero", "g_idx") and not hasattr(self, name):
                continue
            else:
                target = getattr(self, name)
            target.assign(store[str(idx)])
            idx += 1
        if self.lora_enabled:  # einsum_dense.py:497-499: the saved kernel holds the update
            self.lora_kernel_a.assign(torch.zeros_like(as_tensor(self.lora_kernel_a)))
            self.lora_kernel_b.assign(torch.zeros_like(as_tensor(self.lora_kernel_b)))
        self._cache.clear()
