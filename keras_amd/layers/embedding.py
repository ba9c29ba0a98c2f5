"""`Embedding` and `ReversibleEmbedding` with the int8 / int4 quantized forward on MI355X.

Mirrors the quantization-related surface of `keras.layers.Embedding`
(keras/src/layers/core/embedding.py) and `keras.layers.ReversibleEmbedding`
(keras/src/layers/core/reversible_embedding.py): variable names, shapes and dtypes
(`_embeddings` int8 `[vocab, dim]` or packed int4 `[vocab, ceil(dim/2)]`,
`embeddings_scale`, `embeddings_zero`, `g_idx`, and the `reverse_*` twins of an untied
layer), `quantize(mode, config)`, the dtype-policy names it leaves behind and the
positional store order.  The lookup runs `k3q_embedding_lookup`; the int8 reverse
projection (the LM head) runs the int8 GEMM / decode kernels with the tied table read in
place as an `[N, K]` operand.

Both layers set `autocast = False` in the reference (embedding.py:132): their float
variables are read in their own dtype, and torch's type promotion decides the output dtype
(a float32 scale under a bfloat16 compute dtype gives float32 outputs).
"""

import math

import torch

from keras_amd import dtype_policies, ops as kops, quantizers
from keras_amd.layers.dense import int8_strip_route
from keras_amd.layers.layer import Layer, as_tensor, require_default_g_idx, to_torch_dtype
from keras_amd.quantization_config import (
    Int4QuantizationConfig,
    QuantizationConfig,
    get_block_size_for_layer,
)


def uniform_initializer(shape, dtype, generator=None):
    """keras "uniform": U(-0.05, 0.05) (keras/src/initializers/random_initializers.py:118-170)."""
    return ((torch.rand(shape, generator=generator) * 2.0 - 1.0) * 0.05).to(dtype)


def _promote(a, b):
    return a if a == b else torch.float32


class Embedding(Layer):
    def __init__(self, input_dim, output_dim, embeddings_initializer=None, mask_zero=False,
                 dtype=None, name=None, device=None, quantization_config=None, lora_rank=None,
                 lora_alpha=None):
        if not isinstance(input_dim, int) or isinstance(input_dim, bool) or input_dim <= 0:
            raise ValueError(
                "`input_dim` must be a positive integer. "
                f"Received: input_dim={input_dim} (of type {type(input_dim).__name__})."
            )
        if not isinstance(output_dim, int) or isinstance(output_dim, bool) or output_dim <= 0:
            raise ValueError(
                "`output_dim` must be a positive integer. "
                f"Received: output_dim={output_dim} (of type {type(output_dim).__name__})."
            )
        super().__init__(dtype=dtype, name=name, device=device)
        self.input_dim = input_dim
        self.output_dim = output_dim
        self.embeddings_initializer = embeddings_initializer or uniform_initializer
        self.mask_zero = mask_zero
        self.autocast = False
        self.lora_enabled = False
        self.lora_rank = lora_rank
        self.lora_alpha = lora_alpha if lora_alpha is not None else lora_rank
        self.quantization_config = quantization_config
        # raise IndexError for ids outside the table as the reference does; costs one
        # device -> host read per call, switch off in a serving loop
        self.check_ids = True

    # ---- build --------------------------------------------------------------
    def build(self, input_shape=None):
        if self.built:
            return
        embeddings_shape = (self.input_dim, self.output_dim)
        if self.quantization_mode:
            self.quantized_build(embeddings_shape, mode=self.quantization_mode,
                                 config=self.quantization_config)
        if self.quantization_mode not in ("int8", "int4"):
            self._embeddings = self.add_weight(
                name="embeddings", shape=embeddings_shape,
                initializer=self.embeddings_initializer, trainable=True,
            )
        self.built = True
        if self.lora_rank:
            self.enable_lora(self.lora_rank)  # embedding.py:166-167

    @property
    def embeddings(self):
        """The table as a consumer sees it: int4 comes back unpacked to int8
        `[vocab, dim]`; with LoRA enabled the low-rank update is added (embedding.py:169-191)."""
        if not self.built:
            raise AttributeError("You must build the layer before accessing `embeddings`.")
        embeddings = as_tensor(self._embeddings)
        if self.quantization_mode == "int4":
            embeddings = quantizers.unpack_int4(embeddings, self._orig_output_dim, axis=-1)
        if self.lora_enabled:
            embeddings = torch.add(embeddings, self._lora_delta())
        return embeddings

    def enable_lora(self, rank, lora_alpha=None, a_initializer="he_uniform", b_initializer="zeros"):
        """embedding.py:214-261: float32 `lora_embeddings_a` [input_dim, rank] and
        `lora_embeddings_b` [rank, output_dim]; a lookup adds (alpha / rank) * a[ids] . b."""
        from keras_amd.layers.dense import lora_initializer

        if not self.built:
            raise ValueError("Cannot enable lora on a layer that isn't yet built.")
        if self.lora_enabled:
            raise ValueError("lora is already enabled. This can only be done once per layer.")
        self.lora_embeddings_a = self.add_weight(name="lora_embeddings_a", shape=(self.input_dim, rank),
                                                 dtype="float32", initializer=lora_initializer(a_initializer),
                                                 trainable=True)
        self.lora_embeddings_b = self.add_weight(name="lora_embeddings_b", shape=(rank, self.output_dim),
                                                 dtype="float32", initializer=lora_initializer(b_initializer),
                                                 trainable=True)
        self.lora_enabled = True
        self.lora_rank = rank
        self.lora_alpha = lora_alpha if lora_alpha is not None else rank

    def _lora_delta(self):
        return (self.lora_alpha / self.lora_rank) * torch.matmul(
            as_tensor(self.lora_embeddings_a), as_tensor(self.lora_embeddings_b))

    def _add_lora_rows(self, outputs, inputs):
        """embedding.py:533-540 / :575-582: the rows of `a` at the ids times `b`, scaled, added to the
        de-quantised rows, the sum cast to the compute dtype (the layer does not autocast, so
        the update is float32)."""
        idx = inputs.long()
        idx = torch.where(idx < 0, idx + self.input_dim, idx)
        lora = torch.matmul(torch.nn.functional.embedding(idx, as_tensor(self.lora_embeddings_a)),
                            as_tensor(self.lora_embeddings_b))
        out = torch.add(outputs, (self.lora_alpha / self.lora_rank) * lora)
        return out.to(to_torch_dtype(self.compute_dtype))

    def _get_embeddings_with_merged_lora(self):
        """`(embeddings, embeddings_scale, embeddings_zero)` as saved (embedding.py:683-818): with LoRA
        enabled the table is de-quantised, `(alpha / rank) * a . b` added, and the sum quantised again
        the way `quantize()` does it."""
        mode = self.quantization_mode
        if mode is None:
            return self.embeddings, None, None
        value = as_tensor(self._embeddings)
        scale = as_tensor(self.embeddings_scale)
        zero = as_tensor(self.embeddings_zero) if hasattr(self, "embeddings_zero") else None
        if not self.lora_enabled:
            return value, scale, zero
        cd = to_torch_dtype(self.compute_dtype)
        block_size = getattr(self, "_int4_block_size", None)
        grouped = block_size is not None and block_size != -1
        if mode == "int4":
            unpacked = quantizers.unpack_int4(value, self._orig_output_dim, axis=-1)
            if grouped:
                table = quantizers.dequantize_with_sz_map(unpacked.to(cd), scale, zero, as_tensor(self.g_idx),
                                                          group_axis=-1)
            else:
                table = torch.divide(unpacked.to(cd), torch.unsqueeze(scale, -1))
            quant_range = (-8, 7)
        elif mode == "int8":
            table = torch.divide(value.to(cd), torch.unsqueeze(scale, -1))
            quant_range = (-127, 127)
        else:
            raise self._quantization_mode_error(mode)
        merged = torch.add(table, self._lora_delta())
        if mode == "int4" and grouped:
            value_t, scale_t, zero_t = quantizers.abs_max_quantize_grouped_with_zero_point(
                torch.transpose(merged, 0, 1), block_size=block_size, value_range=quant_range, dtype="int8",
                to_numpy=True)
            requantized = torch.transpose(value_t, 0, 1).contiguous()
            scale = torch.transpose(scale_t, 0, 1).contiguous()
            zero = torch.transpose(zero_t, 0, 1).contiguous()
        else:
            requantized, scale = quantizers.abs_max_quantize(merged, axis=-1, value_range=quant_range,
                                                            dtype="int8", to_numpy=True)
            scale = torch.squeeze(scale, dim=-1)
            zero = None
        if mode == "int4":
            value, _, _ = quantizers.pack_int4(requantized.to(self.device), axis=-1)
        else:
            value = requantized
        return value, scale, zero

    def __call__(self, inputs, training=None, **kwargs):
        # ids are not cast to the compute dtype (layer.py:883-901 only touches floats)
        if not isinstance(inputs, torch.Tensor):
            inputs = torch.as_tensor(inputs)
        if not self.built:
            self.build(tuple(inputs.shape))
        if inputs.device != self.device:
            inputs = inputs.to(self.device)
        if self.quantization_mode is not None:
            return self.quantized_call(inputs, **kwargs)
        return self.call(inputs, **kwargs)

    def call(self, inputs):
        if inputs.dtype not in (torch.int32, torch.int64):
            inputs = inputs.to(torch.int32)
        idx = inputs.long()
        idx = torch.where(idx < 0, idx + self.input_dim, idx)
        out = torch.nn.functional.embedding(idx, self.embeddings if self.lora_enabled else as_tensor(self._embeddings))
        return out.to(to_torch_dtype(self.compute_dtype))

    def compute_mask(self, inputs, mask=None):
        if not self.mask_zero:
            return None
        return torch.not_equal(inputs, 0)

    def compute_output_shape(self, input_shape):
        return (*input_shape, self.output_dim)

    # ---- quantized variables --------------------------------------------------
    @property
    def variable_serialization_spec(self):
        """embedding.py:409-428."""
        return {
            None: ["embeddings"],
            "int8": ["embeddings", "embeddings_scale"],
            "int4": ["embeddings", "embeddings_scale", "embeddings_zero", "g_idx"],
        }

    def quantized_build(self, embeddings_shape, mode, config=None):
        if mode == "int8":
            self._int8_build(embeddings_shape, config)
        elif mode == "int4":
            self._int4_build(embeddings_shape, config)
        else:
            raise self._quantization_mode_error(mode)
        self._is_quantized = True

    def _int8_build(self, embeddings_shape, config=None):
        self._embeddings = self.add_weight(name="embeddings", shape=embeddings_shape, dtype="int8")
        # one scale per vocabulary row: the reduction runs over output_dim (embedding.py:447-455)
        self.embeddings_scale = self.add_weight(
            name="embeddings_scale", shape=(self.input_dim,), initializer="ones"
        )

    def _int4_build(self, embeddings_shape, config=None):
        input_dim, output_dim = embeddings_shape
        packed_cols = (output_dim + 1) // 2
        self._embeddings = self.add_weight(
            name="embeddings", shape=(input_dim, packed_cols), dtype="int8"
        )
        block_size = get_block_size_for_layer(self, config)
        self._int4_block_size = block_size
        if block_size is None or block_size == -1:
            scale_shape = (self.input_dim,)
        else:
            scale_shape = (self.input_dim, math.ceil(output_dim / block_size))
        self.embeddings_scale = self.add_weight(
            name="embeddings_scale", shape=scale_shape, initializer="ones"
        )
        if block_size is not None and block_size > 0:
            self.embeddings_zero = self.add_weight(
                name="embeddings_zero", shape=scale_shape, dtype="int8"
            )
            # float32 on purpose, as in the reference (embedding.py:500-516)
            self.g_idx = self.add_weight(
                name="g_idx", shape=(output_dim,), dtype="float32",
                initializer=lambda shape, dtype: torch.floor_divide(
                    torch.arange(output_dim, dtype=dtype), block_size),
            )
        self._orig_output_dim = output_dim

    # ---- quantized forward -------------------------------------------------------
    def _lookup_dtype(self):
        return _promote(to_torch_dtype(self.compute_dtype), as_tensor(self.embeddings_scale).dtype)

    def _int8_call(self, inputs, training=None):
        """embedding.py:521-541: gather rows and scales, cast, divide -- one kernel."""
        out = kops.embedding_lookup(
            inputs, as_tensor(self._embeddings), as_tensor(self.embeddings_scale),
            self.output_dim, bits=8, out_dtype=self._lookup_dtype(), check_ids=self.check_ids,
        )
        return self._add_lora_rows(out, inputs) if self.lora_enabled else out

    def _int4_call(self, inputs, training=None):
        """embedding.py:542-582: the packed rows are gathered and de-quantised in one kernel;
        the table is never unpacked in memory."""
        block_size = getattr(self, "_int4_block_size", None)
        grouped = block_size is not None and block_size > 0
        if grouped:
            require_default_g_idx(self, block_size)
        out = kops.embedding_lookup(
            inputs, as_tensor(self._embeddings), as_tensor(self.embeddings_scale),
            self._orig_output_dim, bits=4,
            zero=as_tensor(self.embeddings_zero) if grouped else None,
            block_size=block_size if grouped else None,
            out_dtype=self._lookup_dtype(), check_ids=self.check_ids,
        )
        return self._add_lora_rows(out, inputs) if self.lora_enabled else out

    # ---- quantize (one-time, host side) ---------------------------------------------
    def _drop(self, attr):
        var = getattr(self, attr)
        self._variables = [v for v in self._variables if v is not var]
        delattr(self, attr)

    def _quantize_table(self, mode, config, block_size):
        """Quantised forward table: (value int8 [V, D] or packed, scale, zero | None)."""
        table = as_tensor(self._embeddings)
        if mode == "int8":
            wq = QuantizationConfig.weight_quantizer_or_default(
                config, quantizers.AbsMaxQuantizer(axis=-1))
            value, scale = wq(table, to_numpy=True)
            return value, torch.squeeze(scale, dim=-1), None
        use_grouped = block_size is not None and block_size != -1
        zero = None
        if not use_grouped:
            wq = QuantizationConfig.weight_quantizer_or_default(
                config, quantizers.AbsMaxQuantizer(axis=-1, value_range=(-8, 7), output_dtype="int8"))
            value, scale = wq(table, to_numpy=True)
            scale = torch.squeeze(scale, dim=-1)
        else:
            # grouped along output_dim: quantise the transpose, transpose back
            value_t, scale_t, zero_t = quantizers.abs_max_quantize_grouped_with_zero_point(
                torch.transpose(table, 0, 1), block_size=block_size, value_range=(-8, 7),
                dtype="int8", to_numpy=True,
            )
            value = torch.transpose(value_t, 0, 1).contiguous()
            scale = torch.transpose(scale_t, 0, 1).contiguous()
            zero = torch.transpose(zero_t, 0, 1).contiguous()
        packed, _, _ = quantizers.pack_int4(value.to(self.device), axis=-1)
        return packed, scale, zero

    def _set_quantized_policy(self, mode, config):
        if self.dtype_policy.quantization_mode is None:
            policy_name = mode
            if mode == "int4":
                block_size = get_block_size_for_layer(self, config)
                policy_name = f"int4/{-1 if block_size is None else block_size}"
            self._dtype_policy = dtype_policies.get(f"{policy_name}_from_{self.dtype_policy.name}")

    def _quantize(self, mode, config, type_check=True):
        """embedding.py:584-684."""
        if type_check and type(self) is not Embedding:
            raise self._not_implemented_error(self.quantize)
        if mode not in ("int8", "int4"):
            raise self._quantization_mode_error(mode)
        self.quantization_config = config
        embeddings_shape = (self.input_dim, self.output_dim)
        block_size = get_block_size_for_layer(self, config) if mode == "int4" else None
        value, scale, zero = self._quantize_table(mode, config, block_size)
        self._drop("_embeddings")
        self.quantized_build(embeddings_shape, mode, config)
        self._embeddings.assign(value)
        self.embeddings_scale.assign(scale)
        if zero is not None:
            self.embeddings_zero.assign(zero)
        self._set_quantized_policy(mode, config)

    def _quantization_mode_error(self, mode):
        return NotImplementedError(
            "Invalid quantization mode. Expected one of ('int8', 'int4'). "
            f"Received: quantization_mode={mode}"
        )

    # ---- serialization ----------------------------------------------------------------
    def _spec_entries(self):
        """(name, variable) in store order, skipping entries this configuration lacks
        (embedding.py:276-372)."""
        mode = self.quantization_mode
        if mode not in self.variable_serialization_spec:
            raise self._quantization_mode_error(mode)
        out = []
        for name in self.variable_serialization_spec[mode]:
            attr = "_embeddings" if name == "embeddings" else name
            if not hasattr(self, attr):
                continue
            out.append((name, getattr(self, attr)))
        return out

    def save_own_variables(self, store):
        """Store order of `_spec_entries`; a LoRA update is merged into the table, the scales and
        the zero points that are written (embedding.py:263-309)."""
        if not self.built:
            return
        merged = {}
        if self.lora_enabled:
            value, scale, zero = self._get_embeddings_with_merged_lora()
            merged = {"embeddings": value, "embeddings_scale": scale, "embeddings_zero": zero}
        for idx, (name, var) in enumerate(self._spec_entries()):
            value = merged.get(name)
            store[str(idx)] = as_tensor(var) if value is None else value

    def load_own_variables(self, store):
        if not self.built:
            return
        for idx, (name, var) in enumerate(self._spec_entries()):
            value = store[str(idx)]
            if name == "g_idx" and isinstance(value, torch.Tensor):
                value = value.to(as_tensor(var).dtype)
            var.assign(value)
        if self.lora_enabled:  # embedding.py:355-361: what was saved holds the update
            self.lora_embeddings_a.assign(torch.zeros_like(as_tensor(self.lora_embeddings_a)))
            self.lora_embeddings_b.assign(torch.zeros_like(as_tensor(self.lora_embeddings_b)))

    def get_config(self):
        config = {
            "name": self.name,
            "input_dim": self.input_dim,
            "output_dim": self.output_dim,
            "mask_zero": self.mask_zero,
            "dtype": self.dtype_policy.name,
            "quantization_config": (
                None if self.quantization_config is None else {
                    "class_name": type(self.quantization_config).__name__,
                    "config": self.quantization_config.get_config(),
                }
            ),
        }
        if self.lora_rank:
            config["lora_rank"] = self.lora_rank
            config["lora_alpha"] = self.lora_alpha
        return config


class ReversibleEmbedding(Embedding):
    """`Embedding` that can also project back to the vocabulary (`reverse=True`), i.e. the
    LM head (reversible_embedding.py:16-541)."""

    def __init__(self, input_dim, output_dim, tie_weights=True, embeddings_initializer=None,
                 mask_zero=False, reverse_dtype=None, logit_soft_cap=None, **kwargs):
        super().__init__(input_dim, output_dim, embeddings_initializer=embeddings_initializer,
                         mask_zero=mask_zero, **kwargs)
        self.tie_weights = tie_weights
        self.reverse_dtype = reverse_dtype
        self.logit_soft_cap = logit_soft_cap
        self.exact_epilogue = None
        self._cache = {}

    def build(self, input_shape=None):
        if self.built:
            return
        super().build(input_shape)
        if not self.tie_weights and self.quantization_mode not in ("int8", "int4"):
            self.reverse_embeddings = self.add_weight(
                name="reverse_embeddings", shape=(self.output_dim, self.input_dim),
                initializer=self.embeddings_initializer, trainable=True,
            )

    def __call__(self, inputs, reverse=False, training=None):
        if not reverse:
            return super().__call__(inputs)
        if not isinstance(inputs, torch.Tensor):
            inputs = torch.as_tensor(inputs)
        if not self.built:
            self.build()
        if inputs.device != self.device:
            inputs = inputs.to(self.device)
        cd = to_torch_dtype(self.compute_dtype)
        if inputs.dtype.is_floating_point and inputs.dtype != cd:
            inputs = inputs.to(cd)
        if self.quantization_mode is not None:
            return self.quantized_call(inputs, reverse=True)
        return self.call(inputs, reverse=True)

    def call(self, inputs, reverse=False):
        if not reverse:
            return super().call(inputs)
        if self.tie_weights:
            kernel = torch.transpose(as_tensor(self._embeddings), 0, 1)
        else:
            kernel = as_tensor(self.reverse_embeddings)
        if self.reverse_dtype is not None:
            rd = to_torch_dtype(self.reverse_dtype)
            inputs, kernel = inputs.to(rd), kernel.to(rd)
        rt = _promote(inputs.dtype, kernel.dtype)
        logits = torch.matmul(inputs.to(rt), kernel.to(rt))
        return self._soft_cap(logits)

    def _soft_cap(self, logits):
        if self.logit_soft_cap is None:
            return logits
        cap = self.logit_soft_cap
        return torch.multiply(torch.tanh(torch.divide(logits, cap)), cap)

    def compute_mask(self, inputs, mask=None):
        return None

    def compute_output_shape(self, input_shape, reverse=False):
        output_shape = list(input_shape)
        if reverse:
            output_shape[-1] = self.input_dim
        else:
            output_shape += [self.output_dim]
        return output_shape

    # ---- quantized variables ------------------------------------------------------
    @property
    def variable_serialization_spec(self):
        """reversible_embedding.py:176-189."""
        spec = {k: list(v) for k, v in super().variable_serialization_spec.items()}
        if not self.tie_weights:
            for mode, names in spec.items():
                names.append("reverse_embeddings")
                if mode in ("int4", "int8"):
                    names.append("reverse_embeddings_scale")
                if mode == "int4":
                    names.append("reverse_embeddings_zero")
        return spec

    def _int8_build(self, embeddings_shape, config=None):
        super()._int8_build(embeddings_shape, config)
        self.inputs_quantizer = QuantizationConfig.activation_quantizer_or_default(
            config, quantizers.AbsMaxQuantizer(axis=-1))
        if not self.tie_weights:
            self.reverse_embeddings = self.add_weight(
                name="reverse_embeddings", shape=(self.output_dim, self.input_dim), dtype="int8")
            self.reverse_embeddings_scale = self.add_weight(
                name="reverse_embeddings_scale", shape=(self.input_dim,), initializer="ones")

    def _int4_build(self, embeddings_shape, config=None):
        super()._int4_build(embeddings_shape, config)
        self.inputs_quantizer = QuantizationConfig.activation_quantizer_or_default(
            config, quantizers.AbsMaxQuantizer(axis=-1))
        if not self.tie_weights:
            packed_rows = (self.output_dim + 1) // 2
            self.reverse_embeddings = self.add_weight(
                name="reverse_embeddings", shape=(packed_rows, self.input_dim), dtype="int8")
            block_size = get_block_size_for_layer(self, config)
            if block_size is None or block_size == -1:
                reverse_scale_shape = (self.input_dim,)
            else:
                reverse_scale_shape = (math.ceil(self.output_dim / block_size), self.input_dim)
            self.reverse_embeddings_scale = self.add_weight(
                name="reverse_embeddings_scale", shape=reverse_scale_shape, initializer="ones")
            if block_size is not None and block_size != -1:
                # variable dtype (not int8), as in the reference (reversible_embedding.py:262-269)
                self.reverse_embeddings_zero = self.add_weight(
                    name="reverse_embeddings_zero", shape=reverse_scale_shape)

    # ---- quantized forward -----------------------------------------------------------
    def _cached(self, key, var, make):
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

    def _int8_call(self, inputs, reverse=False, training=None):
        """reversible_embedding.py:272-296.  Tied weights: the `[vocab, dim]` int8 table IS
        the `[N, K]` operand of the GEMM; nothing is transposed."""
        if not reverse:
            return super()._int8_call(inputs)
        cd = to_torch_dtype(self.compute_dtype)
        lead = inputs.shape[:-1]
        x2 = inputs.reshape(-1, inputs.shape[-1])
        if not self.inputs_quantizer:
            # weight-only: float rows against the int8 kernel, then the de-scale
            scale_var = self.embeddings_scale if self.tie_weights else self.reverse_embeddings_scale
            scale = as_tensor(scale_var)
            if scale.dtype != cd:
                raise NotImplementedError(
                    "The weight-only int8 reverse projection needs its scales in the compute "
                    f"dtype (got {scale.dtype} scales under {cd} compute)."
                )
            if self.tie_weights:
                logits = kops.int8_weight_only_matmul(x2, None, scale,
                                                      prepacked=as_tensor(self._embeddings))
            else:
                logits = kops.int8_weight_only_matmul(
                    x2, as_tensor(self.reverse_embeddings), scale,
                    prepacked=self._cached("prepacked", self.reverse_embeddings,
                                           kops.prepack_int8_kernel))
            return self._soft_cap(logits.reshape(*lead, self.input_dim))
        scale_var = self.embeddings_scale if self.tie_weights else self.reverse_embeddings_scale
        out_dtype = _promote(cd, as_tensor(scale_var).dtype)
        M, N = x2.shape[0], self.input_dim
        exact = self.exact_epilogue
        if exact is None:
            exact = True
        if (self.tie_weights and exact and out_dtype == torch.bfloat16
                and int8_strip_route(self.inputs_quantizer, x2, N)):
            # decode sizes: the table's strip-linear copy as the [dim, vocab] kernel of the projection
            # (made once, as many bytes as the table): quantizer, exact int8 matmul and de-scale in
            # one launch, the bits of the route below
            logits = kops.int8_dense_strip(
                x2, self._cached("w8s", self._embeddings, lambda t: kops.int8_strip_copy(t.t().contiguous())), N,
                as_tensor(scale_var), epsilon=self.inputs_quantizer.epsilon,
                value_range=self.inputs_quantizer.value_range,
                quantize=lambda rows: self.inputs_quantizer(rows, axis=-1))
            return self._soft_cap(logits.reshape(*lead, N))
        q, in_scale = self.inputs_quantizer(x2, axis=-1)
        in_scale = in_scale.to(out_dtype)  # widening an existing value is exact
        round_acc = cd == torch.bfloat16 and out_dtype == torch.float32
        if self.tie_weights:
            logits = kops.int8_matmul_nk(
                q, as_tensor(self._embeddings), a_scale=in_scale,
                kernel_scale=as_tensor(scale_var), out_dtype=out_dtype,
                exact_epilogue=exact, round_acc_bf16=round_acc,
            )
        else:
            if round_acc:
                raise NotImplementedError(
                    "Untied int8 reverse projection with bfloat16 compute and float32 scales "
                    "is not on the fused path yet."
                )
            logits = kops.int8_matmul(
                q, as_tensor(self.reverse_embeddings), a_scale=in_scale,
                kernel_scale=as_tensor(scale_var), out_dtype=out_dtype,
                prepacked=self._cached("prepacked", self.reverse_embeddings,
                                       kops.prepack_int8_kernel),
                exact_epilogue=exact,
            )
        return self._soft_cap(logits.reshape(*lead, N))

    def _tied_strip_operands(self, x2, scale, grouped, block_size):
        """Operands of `ops.int4_matmul_strip` for the tied int4 table used as the LM head, or None
        when that route does not take these rows: the table (packed along its last axis, K of the
        projection) unpacked, transposed and packed again the way a Dense kernel `[dim, vocab]` is,
        then copied in strip-linear order; grouped scales / zero points transposed to `[groups, vocab]`.
        Made on first use, kept while the variables do not change."""
        K, N = self._orig_output_dim, self.input_dim
        if not (x2.is_cuda and x2.dtype == torch.bfloat16 and scale.dtype == torch.bfloat16
                and 0 < x2.shape[0] <= kops.STRIP_MAX_ROWS and x2.shape[1] == K
                and kops.int4_strip_supported(x2.shape[0], K, N, block_size if grouped else None)):
            return None

        def relay(table):
            dense = quantizers.unpack_int4(table, K, axis=-1).t().contiguous()  # [dim, vocab] int8
            return kops.int4_strip_copy(quantizers.pack_int4(dense, axis=-1)[0], N)

        spec = dict(shadow=self._cached("w4s", self._embeddings, relay))
        if grouped:
            sv, zv = self.embeddings_scale, self.embeddings_zero
            stamp = (id(sv), sv.version, id(zv), zv.version)
            hit = self._cache.get("w4s_params")
            if hit is None or hit[0] != stamp:
                value = kops.int4_strip_params(as_tensor(sv).t().contiguous(),
                                               as_tensor(zv).to(torch.int8).t().contiguous(), K, N, block_size)
                hit = self._cache["w4s_params"] = (stamp, None, value)
            spec["gparams"] = hit[2]
        else:
            spec["kernel_scale"] = scale if scale.is_contiguous() else scale.contiguous()
        return spec

    def _int4_call(self, inputs, reverse=False, training=None):
        """reversible_embedding.py:298-381.

        Tied weights: the packed `[vocab, ceil(dim/2)]` table is the K-contiguous int4 kernel
        of the projection and is read in place; at decode sizes (`_tied_strip_operands`) a
        strip-linear copy of it is streamed by the Dense decode kernel instead.  Untied weights: `reverse_embeddings` is
        packed along its first axis (two k per byte); it is re-packed once, on the device,
        into the Dense layout (two columns per byte, same size) and cached, after which the
        call is a Dense int4 call.  With an activation quantizer (a layer built from a policy
        without a config): per-row scales go through the exact int8 GEMM on the table unpacked
        once to int8; grouped scales multiply the quantised rows, as float values, with the
        de-quantised kernel and divide by the input scale afterwards, as the reference does."""
        if not reverse:
            return super()._int4_call(inputs)
        cd = to_torch_dtype(self.compute_dtype)
        block_size = getattr(self, "_int4_block_size", None)
        grouped = block_size is not None and block_size > 0
        if grouped:
            require_default_g_idx(self, block_size)
        lead = inputs.shape[:-1]
        x2 = inputs.reshape(-1, inputs.shape[-1])
        in_scale = None
        if self.inputs_quantizer:
            x2, in_scale = self.inputs_quantizer(x2, axis=-1)
        if self.tie_weights:
            scale = as_tensor(self.embeddings_scale)
            if in_scale is not None and not grouped:
                # int8 rows x int4 table: exact int32 accumulation, one de-scale
                out_dtype = _promote(cd, scale.dtype)
                table8 = self._cached(
                    "unpacked", self._embeddings,
                    lambda t: quantizers.unpack_int4(t, self._orig_output_dim, axis=-1))
                logits = kops.int8_matmul_nk(
                    x2, table8, a_scale=in_scale.to(out_dtype), kernel_scale=scale,
                    out_dtype=out_dtype, exact_epilogue=True,
                    round_acc_bf16=(cd == torch.bfloat16 and out_dtype == torch.float32))
            elif in_scale is None and (strip := self._tied_strip_operands(x2, scale, grouped, block_size)):
                # decode sizes: the table re-laid once as the [dim, vocab] int4 kernel of the
                # projection in strip-linear order (as many bytes as the table), streamed by the
                # Dense decode kernel
                logits = kops.int4_matmul_strip(x2, strip["shadow"], self.input_dim, block_size=block_size if grouped else None,
                                                kernel_scale=strip.get("kernel_scale"), gparams=strip.get("gparams"))
            else:
                logits = kops.int4_matmul_nk(
                    x2 if in_scale is None else x2.to(cd), as_tensor(self._embeddings), scale,
                    zero=as_tensor(self.embeddings_zero) if grouped else None,
                    block_size=block_size if grouped else None)
                if in_scale is not None:
                    logits = torch.divide(logits, in_scale)
        else:
            # the variable is read without autocast (float32 under a mixed policy): torch then
            # promotes the whole de-scale / de-quantisation to that dtype
            scale = as_tensor(self.reverse_embeddings_scale)
            out_dtype = _promote(cd, scale.dtype)
            if in_scale is not None and not grouped:
                # int8 rows x int4 kernel: exact int32 accumulation, one de-scale
                table8 = self._cached(
                    "reverse_unpacked_nk", self.reverse_embeddings,
                    lambda t: quantizers.unpack_int4(t, self.output_dim, axis=0).t().contiguous())
                logits = kops.int8_matmul_nk(
                    x2, table8, a_scale=in_scale.to(out_dtype), kernel_scale=scale,
                    out_dtype=out_dtype, exact_epilogue=True,
                    round_acc_bf16=(cd == torch.bfloat16 and out_dtype == torch.float32))
            else:
                relaid = self._cached(
                    "relaid", self.reverse_embeddings,
                    lambda t: quantizers.pack_int4(
                        quantizers.unpack_int4(t, self.output_dim, axis=0), axis=-1)[0])
                if grouped:
                    # x . ((w - zero) * scale) in the promoted dtype (the quantised rows are
                    # small integers: their cast is exact), then the input scale
                    zero = self._cached("zero_i8", self.reverse_embeddings_zero,
                                        lambda t: t.to(torch.int8).contiguous())
                    logits = kops.int4_matmul(x2.to(out_dtype), relaid, scale, self.input_dim,
                                              kernel_zero=zero, block_size=block_size)
                    if in_scale is not None:
                        logits = torch.divide(logits, in_scale)
                elif out_dtype == cd:
                    logits = kops.int4_matmul(x2, relaid, scale, self.input_dim)
                else:
                    # T(x . w) in the compute dtype, divided by the float32 scale afterwards
                    ones = self._cached("ones_cd", self.reverse_embeddings_scale,
                                        lambda t: torch.ones_like(t, dtype=cd))
                    logits = kops.int4_matmul(x2, relaid, ones, self.input_dim)
                    logits = torch.divide(logits.to(out_dtype), scale)
        return self._soft_cap(logits.reshape(*lead, self.input_dim))

    # ---- quantize -----------------------------------------------------------------------
    def _quantize(self, mode, config, type_check=True):
        """reversible_embedding.py:383-541."""
        if type_check and type(self) is not ReversibleEmbedding:
            raise self._not_implemented_error(self.quantize)
        if mode not in ("int8", "int4"):
            raise self._quantization_mode_error(mode)
        self.quantization_config = config
        embeddings_shape = (self.input_dim, self.output_dim)
        # the reference reads the block size from the config object only here (:439-444)
        block_size = None
        if mode == "int4" and isinstance(config, Int4QuantizationConfig):
            block_size = config.block_size
        use_grouped = block_size is not None and block_size != -1
        value, scale, zero = self._quantize_table(mode, config, block_size)
        self._drop("_embeddings")
        rev = None
        if not self.tie_weights:
            rtable = as_tensor(self.reverse_embeddings)
            if mode == "int8":
                wq = QuantizationConfig.weight_quantizer_or_default(
                    config, quantizers.AbsMaxQuantizer(axis=0))
                rvalue, rscale = wq(rtable, to_numpy=True)
                rev = (rvalue, torch.squeeze(rscale, dim=0), None)
            else:
                if not use_grouped:
                    wq = QuantizationConfig.weight_quantizer_or_default(
                        config,
                        quantizers.AbsMaxQuantizer(axis=0, value_range=(-8, 7), output_dtype="int8"))
                    rvalue, rscale = wq(rtable, to_numpy=True)
                    rscale, rzero = torch.squeeze(rscale, dim=0), None
                else:
                    rvalue, rscale, rzero = quantizers.abs_max_quantize_grouped_with_zero_point(
                        rtable, block_size=block_size, value_range=(-8, 7), dtype="int8",
                        to_numpy=True)
                rpacked, _, _ = quantizers.pack_int4(rvalue.to(self.device), axis=0)
                rev = (rpacked, rscale, rzero)
            self._drop("reverse_embeddings")
        self.quantized_build(embeddings_shape, mode, config)
        self._embeddings.assign(value)
        self.embeddings_scale.assign(scale)
        if zero is not None:
            self.embeddings_zero.assign(zero)
        if rev is not None:
            self.reverse_embeddings.assign(rev[0])
            self.reverse_embeddings_scale.assign(rev[1])
            if rev[2] is not None:
                self.reverse_embeddings_zero.assign(rev[2])
        self._set_quantized_policy(mode, config)
        self._cache.clear()

    def get_config(self):
        config = super().get_config()
        config.update({
            "tie_weights": self.tie_weights,
            "reverse_dtype": self.reverse_dtype,
            "logit_soft_cap": self.logit_soft_cap,
        })
        return config
