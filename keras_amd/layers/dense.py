"""`Dense` with the int8 / int4 quantized forward on MI355X.

Mirrors the quantization-related surface of `keras.layers.Dense`
(keras/src/layers/core/dense.py): variable names, shapes and dtypes
(`_kernel`, `kernel_scale`, `kernel_zero`, `g_idx`, `bias`), `quantize(mode,
config)`, the dtype-policy names it leaves behind, the positional
`save_own_variables` / `load_own_variables` order, and `_int8_call` /
`_int4_call`.  The two call methods run the k3q HIP kernels; the float `call`
is a plain torch matmul and exists so that a float layer can be built,
compared against and converted.
"""

import math

import torch

from keras_amd import dtype_policies, ops as kops, quantizers
from keras_amd.layers.layer import Layer, as_tensor, require_default_g_idx, to_torch_dtype
from keras_amd.layers.together import quantize_rows
from keras_amd.quantization_config import QuantizationConfig, get_block_size_for_layer

_ACTIVATIONS = {
    None: None,
    "linear": None,
    "relu": torch.relu,
    "gelu": torch.nn.functional.gelu,
    "silu": torch.nn.functional.silu,
    "swish": torch.nn.functional.silu,
    "sigmoid": torch.sigmoid,
    "tanh": torch.tanh,
}

# `exact_epilogue` of a layer: None / True reproduce the reference's rounding chain bit for
# bit (the default: it costs under 2 % of a prefill-sized matmul); False rounds once at the end.


def activation_name(fn):
    for name, f in _ACTIVATIONS.items():
        if f is fn:
            return name
    raise ValueError(f"activation {fn} has no serializable name")


def serialize_quantization_config(config):
    if config is None:
        return None
    return {"class_name": type(config).__name__, "config": config.get_config()}


def glorot_uniform(shape, dtype, generator=None):
    """U(-L, L), L = sqrt(6 / (fan_in + fan_out))
    (keras/src/initializers/random_initializers.py:292-318)."""
    fan_in, fan_out = shape[0], shape[-1]
    if len(shape) > 2:
        receptive = 1
        for d in shape[:-2]:
            receptive *= d
        fan_in, fan_out = shape[-2] * receptive, shape[-1] * receptive
    limit = math.sqrt(6.0 / (fan_in + fan_out))
    return ((torch.rand(shape, generator=generator) * 2.0 - 1.0) * limit).to(dtype)


def he_uniform(shape, dtype, generator=None):
    """U(-L, L), L = sqrt(6 / fan_in) (keras/src/initializers/random_initializers.py, `HeUniform`)."""
    fan_in = shape[0]
    if len(shape) > 2:
        receptive = 1
        for d in shape[:-2]:
            receptive *= d
        fan_in = shape[-2] * receptive
    limit = math.sqrt(6.0 / max(fan_in, 1))
    return ((torch.rand(shape, generator=generator) * 2.0 - 1.0) * limit).to(dtype)


LORA_INITIALIZERS = {"he_uniform": he_uniform, "zeros": "zeros", "ones": "ones"}


def lora_initializer(spec):
    if callable(spec):
        return spec
    if spec not in LORA_INITIALIZERS:
        raise ValueError(f"Unknown initializer: {spec}")
    return LORA_INITIALIZERS[spec]


# rows for which the int4 forward reads the K-contiguous copy of the kernel (measured against
# the 32-row passes below it and the de-quantise + GEMM route above it, groups of 128, us:
# K=4096, N=14336: 17 rows 22 against 27, 32 rows 23 against 31, 64 rows 26 against 60, 128 rows
# 38 against 65, 256 rows 58 against 81, 512 rows 98 against 98; K=N=4096: 17 rows 14.5 against
# 13.4, 32 rows 16 against 17, 64 rows 19 against 32, 128 rows 24 against 30, 512 rows 40
# against 45; K=14336, N=4096: 17 rows 29 against 27, 512 rows 96 against 102)
KMAJOR_MIN_ROWS, KMAJOR_MAX_ROWS = 33, 512
# from 17 rows on kernels at least this wide or this large (17 rows, groups of 128, us:
# K=5120, N=13824: 26 against 36; K=13824, N=5120: 29 against 37; K=11008, N=4096: 25 against
# 27; K=8192, N=28672: 59 against 129; K=N=5120: 18 against 18.5 and K=N=4096: 14.5 against
# 13.4, both left on the decode kernel)
KMAJOR_MIN_ROWS_WIDE, KMAJOR_WIDE_UNITS, KMAJOR_LARGE_WEIGHTS = 17, 8192, 40 << 20


def kmajor_rows(rows, units, input_dim=0):
    """Whether `rows` bfloat16 rows into `units` outputs take the K-contiguous int4 route."""
    wide = units >= KMAJOR_WIDE_UNITS or units * input_dim >= KMAJOR_LARGE_WEIGHTS
    low = KMAJOR_MIN_ROWS_WIDE if wide else KMAJOR_MIN_ROWS
    return low <= rows <= KMAJOR_MAX_ROWS


def int8_strip_route(quantizer, x2, units):
    """Whether an int8 call of these rows goes to `ops.int8_dense_strip`: bfloat16 rows on the
    device, few enough, a plain abs-max quantizer (whatever its range and epsilon), a shape the
    kernel takes."""
    return (type(quantizer) is quantizers.AbsMaxQuantizer and quantizer.output_dtype == "int8"
            and x2.is_cuda and x2.dtype == torch.bfloat16 and 0 < x2.shape[0] <= kops.INT8_STRIP_MAX_ROWS
            and kops.int8_strip_supported(x2.shape[0], x2.shape[1], units))


class Dense(Layer):
    def __init__(self, units, activation=None, use_bias=True, kernel_initializer=None,
                 bias_initializer="zeros", dtype=None, name=None, device=None,
                 quantization_config=None, lora_rank=None, lora_alpha=None):
        super().__init__(dtype=dtype, name=name, device=device)
        self.quantization_config = quantization_config  # dense.py:98-130
        self.lora_rank = lora_rank
        self.lora_alpha = lora_alpha if lora_alpha is not None else lora_rank
        if not isinstance(units, int) or units <= 0:
            raise ValueError(
                f"Received an invalid value for `units`, expected a positive integer. Received: units={units}"
            )
        self.units = units
        self.activation = activation if callable(activation) else _ACTIVATIONS[activation]
        self.use_bias = use_bias
        self.kernel_initializer = kernel_initializer or glorot_uniform
        self.bias_initializer = bias_initializer
        self.lora_enabled = False
        self.exact_epilogue = None
        self._cache = {}

    # ---- build --------------------------------------------------------------
    def build(self, input_shape):
        self._build_input_shape = tuple(input_shape)
        kernel_shape = (input_shape[-1], self.units)
        if self.quantization_mode:
            self.quantized_build(kernel_shape, mode=self.quantization_mode,
                                 config=self.quantization_config)
        if self.quantization_mode not in ("int8", "int4"):
            self._kernel = self.add_weight(
                name="kernel", shape=kernel_shape, initializer=self.kernel_initializer, trainable=True
            )
        if self.use_bias:
            self.bias = self.add_weight(
                name="bias", shape=(self.units,), initializer=self.bias_initializer, trainable=True
            )
        else:
            self.bias = None
        self.built = True
        if self.lora_rank:
            self.enable_lora(self.lora_rank)  # (dense.py:160-161: the alpha is not passed on)

    @property
    def kernel(self):
        """The kernel as a consumer sees it: the int4 kernel comes back unpacked to
        `[input_dim, units]` int8; with LoRA enabled the low-rank update is added and the sum
        cast to the compute dtype (keras/src/layers/core/dense.py:163-236)."""
        if not self.built:
            raise AttributeError("You must build the layer before accessing `kernel`.")
        kernel = as_tensor(self._kernel)
        if self.quantization_mode == "int4":
            kernel = quantizers.unpack_int4(kernel, self._orig_output_dim, axis=-1)
        if self.lora_enabled:
            delta = (self.lora_alpha / self.lora_rank) * torch.matmul(
                as_tensor(self.lora_kernel_a), as_tensor(self.lora_kernel_b))
            kernel = torch.add(kernel, delta).to(to_torch_dtype(self.compute_dtype))
        return kernel

    def enable_lora(self, rank, lora_alpha=None, a_initializer="he_uniform", b_initializer="zeros"):
        """keras/src/layers/core/dense.py:251-312: float32 `lora_kernel_a` [input_dim, rank] and
        `lora_kernel_b` [rank, units]; the forward adds (alpha / rank) * (x . a) . b."""
        if not self.built:
            raise ValueError("Cannot enable lora on a layer that isn't yet built.")
        if self.lora_enabled:
            raise ValueError("lora is already enabled. This can only be done once per layer.")
        if self.quantization_mode == "int4" and hasattr(self, "_orig_input_dim"):
            input_dim = self._orig_input_dim
        else:
            input_dim = self._kernel.shape[0]
        self.lora_kernel_a = self.add_weight(name="lora_kernel_a", shape=(input_dim, rank), dtype="float32",
                                             initializer=lora_initializer(a_initializer), trainable=True)
        self.lora_kernel_b = self.add_weight(name="lora_kernel_b", shape=(rank, self.units), dtype="float32",
                                             initializer=lora_initializer(b_initializer), trainable=True)
        self.lora_enabled = True
        self.lora_rank = rank
        self.lora_alpha = lora_alpha if lora_alpha is not None else rank

    def _quantized_call_with_lora(self, quantized_call, inputs):
        """The reference's order with LoRA enabled (dense.py:972-986, :1085-1095): the de-scaled
        quantized product first, then the low-rank term, the cast, the bias, the activation --
        so the kernels run without their fused bias here."""
        bias, activation = self.bias, self.activation
        self.bias, self.activation, self.lora_enabled = None, None, False
        try:
            x = quantized_call(inputs)
        finally:
            self.bias, self.activation, self.lora_enabled = bias, activation, True
        x = torch.add(x, self._lora_term(inputs)).to(to_torch_dtype(self.compute_dtype))
        if bias is not None:
            x = torch.add(x, self.read(bias))
        if activation is not None:
            x = activation(x)
        return x

    def _lora_term(self, inputs):
        """(alpha / rank) * (inputs . a) . b as the quantized calls add it (dense.py:977-980,
        :1086-1089): two small float matmuls in the compute dtype."""
        lora_x = torch.matmul(inputs, self.read(self.lora_kernel_a))
        lora_x = torch.matmul(lora_x, self.read(self.lora_kernel_b))
        return (self.lora_alpha / self.lora_rank) * lora_x

    def call(self, inputs, training=None):
        if self.lora_enabled:
            x = torch.matmul(inputs, self.kernel)
            if self.bias is not None:
                x = torch.add(x, self.read(self.bias))
            return self.activation(x) if self.activation is not None else x
        x = torch.matmul(inputs, self.read(self._kernel))
        if self.bias is not None:
            x = torch.add(x, self.read(self.bias))
        if self.activation is not None:
            x = self.activation(x)
        return x

    # ---- quantized variables --------------------------------------------------
    def quantized_build(self, kernel_shape, mode, config=None):
        if mode == "int8":
            self._int8_build(kernel_shape, config)
        elif mode == "int4":
            self._int4_build(kernel_shape, config)
        else:
            raise self._quantization_mode_error(mode)
        self._is_quantized = True

    def _int8_build(self, kernel_shape, config=None):
        self.inputs_quantizer = QuantizationConfig.activation_quantizer_or_default(
            config, quantizers.AbsMaxQuantizer()
        )
        self._kernel = self.add_weight(name="kernel", shape=kernel_shape, dtype="int8")
        self.kernel_scale = self.add_weight(name="kernel_scale", shape=(self.units,), initializer="ones")

    def _int4_build(self, kernel_shape, config=None):
        self.inputs_quantizer = QuantizationConfig.activation_quantizer_or_default(config, None)
        input_dim, output_dim = kernel_shape
        packed_cols = (output_dim + 1) // 2
        self._kernel = self.add_weight(name="kernel", shape=(input_dim, packed_cols), dtype="int8")
        block_size = get_block_size_for_layer(self, config)
        self._int4_block_size = block_size
        if block_size is None or block_size == -1:
            scale_shape = (self.units,)
        else:
            scale_shape = (math.ceil(input_dim / block_size), self.units)
        self.kernel_scale = self.add_weight(name="kernel_scale", shape=scale_shape, initializer="ones")
        if block_size is not None and block_size > 0:
            self.kernel_zero = self.add_weight(name="kernel_zero", shape=scale_shape, dtype="int8")
            # float32 on purpose, as in the reference (dense.py:868-889)
            self.g_idx = self.add_weight(
                name="g_idx", shape=(input_dim,), dtype="float32",
                initializer=lambda shape, dtype: torch.floor_divide(
                    torch.arange(input_dim, dtype=dtype), block_size),
            )
        self._orig_input_dim = input_dim
        self._orig_output_dim = output_dim

    # ---- quantize (one-time, host side) --------------------------------------
    def _quantize(self, mode, config, type_check=True):
        if type_check and type(self) is not Dense:
            raise self._not_implemented_error(self.quantize)
        self.quantization_config = config
        kernel_shape = self._kernel.shape
        if mode == "int8":
            weight_quantizer = QuantizationConfig.weight_quantizer_or_default(
                config, quantizers.AbsMaxQuantizer(axis=0)
            )
            kernel_value, kernel_scale = weight_quantizer(as_tensor(self._kernel), to_numpy=True)
            kernel_scale = torch.squeeze(kernel_scale, dim=0)
            self._drop_float_kernel()
            self.quantized_build(kernel_shape, mode, config)
            self._kernel.assign(kernel_value)
            self.kernel_scale.assign(kernel_scale)
        elif mode == "int4":
            block_size = get_block_size_for_layer(self, config)
            kernel_zero = None
            if block_size is None or block_size == -1:
                weight_quantizer = QuantizationConfig.weight_quantizer_or_default(
                    config,
                    quantizers.AbsMaxQuantizer(axis=0, value_range=(-8, 7), output_dtype="int8"),
                )
                kernel_value_int4, kernel_scale = weight_quantizer(as_tensor(self._kernel), to_numpy=True)
                kernel_scale = torch.squeeze(kernel_scale, dim=0)
            else:
                kernel_value_int4, kernel_scale, kernel_zero = (
                    quantizers.abs_max_quantize_grouped_with_zero_point(
                        as_tensor(self._kernel), block_size=block_size, to_numpy=True
                    )
                )
            packed, _, _ = quantizers.pack_int4(kernel_value_int4.to(self.device), axis=-1)
            self._drop_float_kernel()
            self.quantized_build(kernel_shape, mode, config)
            self._kernel.assign(packed)
            self.kernel_scale.assign(kernel_scale)
            if kernel_zero is not None:
                self.kernel_zero.assign(kernel_zero)
        else:
            raise self._quantization_mode_error(mode)

        if self.dtype_policy.quantization_mode is None:
            policy_name = mode
            if mode == "int4":
                block_size = get_block_size_for_layer(self, config)
                policy_name = f"int4/{-1 if block_size is None else block_size}"
            self._dtype_policy = dtype_policies.get(f"{policy_name}_from_{self.dtype_policy.name}")
        self._cache.clear()

    def _drop_float_kernel(self):
        self._variables = [v for v in self._variables if v is not self._kernel]
        del self._kernel

    # ---- cached derived operands ------------------------------------------------
    def _cached(self, key, var, make):
        """Value derived from a variable, rebuilt when the variable is assigned."""
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

    def _read_cached(self, key, var):
        cd = to_torch_dtype(self.compute_dtype)
        return self._cached(key, var, lambda t: t.to(cd).contiguous())

    def _strip_operands(self, rows, input_dim, units, grouped, block_size):
        """The operands of the strip-linear decode route (`ops.int4_matmul_strip`) when it takes
        `rows` bfloat16 rows of this layer, else None: the copy of the kernel it streams and, for
        grouped kernels, the re-ordered scales / zero points -- made on first use, kept while the
        variables they come from do not change."""
        if not (0 < rows <= kops.STRIP_MAX_ROWS and to_torch_dtype(self.compute_dtype) == torch.bfloat16
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
            spec["kernel_scale"] = self._read_cached("kernel_scale", self.kernel_scale)
        return spec

    def _tile_operand(self, input_dim):
        """The derived copy of the int8 kernel that the tile GEMM reads, as a keyword of
        `ops.int8_matmul`: the decode kernel's strip-linear copy where the tile kernel can take it
        (one derived copy per layer; same bits and speed as from a [N, K] copy), else the [N, K] copy."""
        if input_dim % 128 == 0:
            return dict(strip=self._cached("w8s", self._kernel, kops.int8_strip_copy))
        return dict(prepacked=self._cached("prepacked", self._kernel, kops.prepack_int8_kernel))

    # ---- quantized forward --------------------------------------------------------
    def _int8_call(self, inputs, training=None):
        """keras/src/layers/core/dense.py:938-986: quantise rows, int8 GEMM, de-scale, bias."""
        if self.lora_enabled:
            return self._quantized_call_with_lora(self._int8_call, inputs)
        if not self.inputs_quantizer:
            # weight-only: float activations against the int8 kernel, then the de-scale
            y = kops.int8_weight_only_matmul(
                inputs, as_tensor(self._kernel),
                self._read_cached("kernel_scale", self.kernel_scale),
                bias=self._call_bias(),
                prepacked=self._cached("prepacked", self._kernel, kops.prepack_int8_kernel),
            )
            if self.activation is not None:
                y = self.activation(y)
            return y
        lead = inputs.shape[:-1]
        x2 = inputs.reshape(-1, inputs.shape[-1])
        M, N = x2.shape[0], self.units
        exact = self.exact_epilogue
        if exact is None:
            exact = True
        if exact and int8_strip_route(self.inputs_quantizer, x2, N):
            # decode sizes: quantizer, matmul and de-scale in one launch, from the strip-linear copy
            y = kops.int8_dense_strip(
                x2, self._cached("w8s", self._kernel, kops.int8_strip_copy), N,
                self._read_cached("kernel_scale", self.kernel_scale), bias=self._call_bias(),
                epsilon=self.inputs_quantizer.epsilon, value_range=self.inputs_quantizer.value_range,
                quantize=lambda rows: quantize_rows(self.inputs_quantizer, rows))
            y = y.reshape(*lead, N)
            if self.activation is not None:
                y = self.activation(y)
            return y
        q, scale = quantize_rows(self.inputs_quantizer, x2)
        y = kops.int8_matmul(
            q, as_tensor(self._kernel), a_scale=scale,
            kernel_scale=self._read_cached("kernel_scale", self.kernel_scale),
            bias=self._call_bias(),
            out_dtype=to_torch_dtype(self.compute_dtype),
            exact_epilogue=exact, **self._tile_operand(x2.shape[1]),
        )
        y = y.reshape(*lead, N)
        if self.activation is not None:
            y = self.activation(y)
        return y

    def _int4_call(self, inputs, training=None):
        """keras/src/layers/core/dense.py:988-1095, weight-only: the packed kernel is
        consumed in place (no unpack, no de-quantised copy)."""
        if self.lora_enabled:
            return self._quantized_call_with_lora(self._int4_call, inputs)
        block_size = getattr(self, "_int4_block_size", None)
        grouped = block_size is not None and block_size > 0
        # (a grouped kernel ignores an activation quantizer, as the reference's sub-channel branch
        # does: dense.py:1040-1084 never reads it)
        if self.inputs_quantizer and not grouped:
            # activation-quantized, per-channel (dense.py:1023-1031): int8 rows against the
            # nibbles unpacked to int8 in scratch, exact int32 accumulation, one de-scale
            lead = inputs.shape[:-1]
            x2 = inputs.reshape(-1, inputs.shape[-1])
            q, scale = quantize_rows(self.inputs_quantizer, x2)
            units = self._orig_output_dim
            operand = {}
            if x2.shape[1] % 128 == 0 and x2.shape[0] > kops.SKINNY_MAX_ROWS:
                # the tile GEMM reads a strip-linear int8 copy of the unpacked kernel, made once and kept
                # while the kernel does not change (one byte per weight beside the stored half byte: this
                # configuration, which the reference does not default to, holds 3x the stored bytes)
                # instead of unpacking the whole kernel into scratch on every call
                unpacked = None
                operand = dict(strip=self._cached(
                    "w8s_unpacked", self._kernel,
                    lambda t: kops.int8_strip_copy(quantizers.unpack_int4(t, units, axis=-1))))
            else:
                unpacked = quantizers.unpack_int4(as_tensor(self._kernel), units, axis=-1)
            y = kops.int8_matmul(
                q, unpacked, a_scale=scale,
                kernel_scale=self._read_cached("kernel_scale", self.kernel_scale),
                bias=self._call_bias(),
                out_dtype=to_torch_dtype(self.compute_dtype), exact_epilogue=True, kernel_shape=(x2.shape[1], units),
                **operand,
            )
            y = y.reshape(*lead, self._orig_output_dim)
            if self.activation is not None:
                y = self.activation(y)
            return y
        if grouped:
            require_default_g_idx(self, block_size)
        rows = inputs.numel() // inputs.shape[-1] if inputs.shape[-1] else 0
        strip = (self._strip_operands(rows, inputs.shape[-1], self._orig_output_dim, grouped, block_size)
                 if inputs.dtype == torch.bfloat16 else None)
        if strip is not None:
            # decode sizes: the strip-linear copy of the kernel, streamed once, all of K inside a
            # workgroup (one launch, no scratch)
            bias = self._call_bias()
            per_row = bias is not None and rows > 1 and bias.numel() == rows * self._orig_output_dim
            y = kops.int4_matmul_strip(
                inputs, strip["shadow"], self._orig_output_dim, kernel_scale=strip.get("kernel_scale"),
                gparams=strip.get("gparams"), block_size=block_size if grouped else None,
                bias=None if per_row else bias, addend=bias if per_row else None)
        elif (inputs.dtype == torch.bfloat16 and kmajor_rows(rows, self._orig_output_dim, inputs.shape[-1])
                and kops.int4_kmajor_supported(rows, inputs.shape[-1], self._orig_output_dim,
                                               block_size if grouped else None)):
            # a few dozen to a hundred-odd rows: from the K-contiguous copy of the kernel (made
            # on first use, kept while the kernel does not change), read once as int4
            units = self._orig_output_dim
            if kops.int4_tiles_strip_supported(rows, inputs.shape[-1], units, block_size if grouped else None):
                # ... from the SAME strip-linear copy the decode kernel streams: one derived copy per layer
                y = kops.int4_matmul_tiles_strip(
                    inputs, self._cached("w4s", self._kernel, lambda t: kops.int4_strip_copy(t, units)), units,
                    self._read_cached("kernel_scale", self.kernel_scale),
                    kernel_zero=as_tensor(self.kernel_zero) if grouped else None,
                    block_size=block_size if grouped else None, bias=self._call_bias())
            else:
                y = kops.int4_matmul_kmajor(
                    inputs, self._cached("kmajor", self._kernel, lambda t: kops.int4_kmajor_copy(t, units)),
                    self._read_cached("kernel_scale", self.kernel_scale),
                    kernel_zero=as_tensor(self.kernel_zero) if grouped else None,
                    block_size=block_size if grouped else None,
                    bias=self._call_bias(),
                )
        else:
            y = kops.int4_matmul(
                inputs, as_tensor(self._kernel),
                self._read_cached("kernel_scale", self.kernel_scale), self._orig_output_dim,
                kernel_zero=as_tensor(self.kernel_zero) if grouped else None,
                block_size=block_size if grouped else None,
                bias=self._call_bias(),
            )
        if self.activation is not None:
            y = self.activation(y)
        return y

    def _call_bias(self):
        """The bias of this call: the layer's own, or -- for a layer without one -- the rows
        that `call_add` lends for the duration of a call (one row: a bias; a row per row of the
        input: the int4 decode kernel's addend)."""
        if self.bias is None:
            return getattr(self, "_row_bias", None)
        return self._read_cached("bias", self.bias)

    def _row_bias_ok(self):
        return self.bias is None and self.activation is None

    def _rows_of(self, inputs):
        return inputs.numel() // inputs.shape[-1]

    def _int8_together_spec(self, inputs):
        """What `call_together` needs to run this layer's int8 forward in a launch shared with other
        layers (decode sizes, the strip-linear copy): rows, quantizer settings, operands, and the
        step from the [M, N] result to the layer's output.  None when the layer's forward is
        anything else."""
        if (not self.built or self.quantization_mode != "int8" or self.lora_enabled
                or self.exact_epilogue is False):
            return None
        x2 = inputs.reshape(-1, inputs.shape[-1])
        if not int8_strip_route(self.inputs_quantizer, x2, self.units):
            return None
        bias = self._call_bias()
        if bias is not None and bias.numel() != self.units:
            return None
        lead = inputs.shape[:-1]

        def finish(y2):
            y = y2.reshape(*lead, self.units)
            return self.activation(y) if self.activation is not None else y

        q = self.inputs_quantizer
        return dict(x2=x2, settings=(float(q.epsilon), tuple(float(v) for v in q.value_range)), quantizer=q,
                    kernel=dict(shadow=self._cached("w8s", self._kernel, kops.int8_strip_copy), units=self.units,
                                kernel_scale=self._read_cached("kernel_scale", self.kernel_scale), bias=bias),
                    finish=finish)

    def _int4_together_spec(self, inputs):
        """What `call_together` needs to run this layer's weight-only int4 forward in a launch
        shared with other layers: the [M, K] rows, the kernel's operands and the step that
        turns the [M, N] result into the layer's output.  None when the layer's forward is
        anything else."""
        if (not self.built or self.quantization_mode != "int4" or self.inputs_quantizer
                or self.lora_enabled):
            return None
        block_size = getattr(self, "_int4_block_size", None)
        grouped = block_size is not None and block_size > 0
        if grouped:
            require_default_g_idx(self, block_size)
        lead = inputs.shape[:-1]

        def finish(y2):
            y = y2.reshape(*lead, self._orig_output_dim)
            return self.activation(y) if self.activation is not None else y

        x2 = inputs.reshape(-1, inputs.shape[-1])
        strip = (self._strip_operands(x2.shape[0], x2.shape[1], self._orig_output_dim, grouped, block_size)
                 if x2.dtype == torch.bfloat16 else None)
        if strip is not None:
            strip["bias"] = self._call_bias()
        return dict(
            x2=x2, block_size=block_size if grouped else None, strip=strip,
            kernel=dict(kernel_packed=as_tensor(self._kernel),
                        kernel_scale=self._read_cached("kernel_scale", self.kernel_scale),
                        units=self._orig_output_dim,
                        kernel_zero=as_tensor(self.kernel_zero) if grouped else None,
                        bias=self._call_bias()),
            finish=finish)

    # ---- serialization ---------------------------------------------------------------
    @property
    def variable_serialization_spec(self):
        """Order of variables in a store, per mode (dense.py:486-541)."""
        return {
            None: ["kernel", "bias"],
            "int8": ["kernel", "bias", "kernel_scale"],
            "int4": ["kernel", "bias", "kernel_scale", "kernel_zero", "g_idx"],
        }

    def _get_kernel_with_merged_lora(self):
        """`(kernel, kernel_scale, kernel_zero)` as they are saved
        (keras/src/layers/core/dense.py:1301-1427): without LoRA the variables themselves; with
        it the kernel is de-quantised (int8: `cast(q, compute) / scale`; int4: unpack, then
        divide or `dequantize_with_sz_map`), `(alpha / rank) * a . b` is added in float, and the sum
        is quantised again the way `quantize()` does it (host numpy path), giving new scales
        (and zero points)."""
        mode = self.quantization_mode
        if mode is None:
            return self.kernel, None, None
        kernel_value = as_tensor(self._kernel)
        kernel_scale = as_tensor(self.kernel_scale)
        kernel_zero = as_tensor(self.kernel_zero) if hasattr(self, "kernel_zero") else None
        if not self.lora_enabled:
            return kernel_value, kernel_scale, kernel_zero
        cd = to_torch_dtype(self.compute_dtype)
        block_size = getattr(self, "_int4_block_size", None)
        grouped = block_size is not None and block_size != -1
        if mode == "int4":
            unpacked = quantizers.unpack_int4(kernel_value, self._orig_output_dim, axis=-1)
            if grouped:
                float_kernel = quantizers.dequantize_with_sz_map(
                    unpacked, kernel_scale, kernel_zero, as_tensor(self.g_idx), group_axis=0).to(cd)
            else:
                float_kernel = torch.divide(unpacked.to(cd), kernel_scale)
            quant_range = (-8, 7)
        elif mode == "int8":
            float_kernel = torch.divide(kernel_value.to(cd), kernel_scale)
            quant_range = (-127, 127)
        else:
            raise self._quantization_mode_error(mode)
        delta = (self.lora_alpha / self.lora_rank) * torch.matmul(
            as_tensor(self.lora_kernel_a), as_tensor(self.lora_kernel_b))
        merged = torch.add(float_kernel, delta)
        if mode == "int4" and grouped:
            requantized, kernel_scale, kernel_zero = quantizers.abs_max_quantize_grouped_with_zero_point(
                merged, block_size=block_size, to_numpy=True)
        else:
            requantized, kernel_scale = quantizers.abs_max_quantize(
                merged, axis=0, value_range=quant_range, dtype="int8", to_numpy=True)
            kernel_scale = torch.squeeze(kernel_scale, dim=0)
            kernel_zero = None
        if mode == "int4":
            kernel_value, _, _ = quantizers.pack_int4(requantized.to(self.device), axis=-1)
        else:
            kernel_value = requantized
        return kernel_value, kernel_scale, kernel_zero

    def save_own_variables(self, store):
        """Write variables under "0", "1", ... in spec order, skipping absent ones; a LoRA update
        is merged into what is written (dense.py:314-378)."""
        if not self.built:
            return
        mode = self.quantization_mode
        if mode not in self.variable_serialization_spec:
            raise self._quantization_mode_error(mode)
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
        mode = self.quantization_mode
        if mode not in self.variable_serialization_spec:
            raise self._quantization_mode_error(mode)
        idx = 0
        for name in self.variable_serialization_spec[mode]:
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
        if self.lora_enabled:
            # what was saved has the update merged in (dense.py:428-430)
            self.lora_kernel_a.assign(torch.zeros_like(as_tensor(self.lora_kernel_a)))
            self.lora_kernel_b.assign(torch.zeros_like(as_tensor(self.lora_kernel_b)))
        self._cache.clear()

    def get_config(self):
        config = {
            "name": self.name,
            "units": self.units,
            "activation": activation_name(self.activation),
            "use_bias": self.use_bias,
            "dtype": self.dtype_policy.name,
            "quantization_config": serialize_quantization_config(self.quantization_config),
        }
        if self.lora_rank:
            config["lora_rank"] = self.lora_rank
            config["lora_alpha"] = self.lora_alpha
        return config
