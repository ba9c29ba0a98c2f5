"""Quantization configs of the int8 / int4 path.

Reference: keras/src/quantizers/quantization_config.py:7-198 (config classes)
and :256-390 (`validate_and_resolve_config`, `get_block_size_for_layer`).
Modes other than "int8" and "int4" are training or calibration schemes that
this build does not cover; they are rejected with the reference's wording
where one exists.
"""

from keras_amd.dtype_policies import QUANTIZATION_MODES, Int4DTypePolicy
from keras_amd.quantizers import AbsMaxQuantizer


class QuantizationConfig:
    def __init__(self, weight_quantizer=None, activation_quantizer=None):
        self.weight_quantizer = weight_quantizer
        self.activation_quantizer = activation_quantizer

    @property
    def mode(self):
        raise NotImplementedError(
            "Subclasses must implement this property. Do not instantiate "
            "QuantizationConfig directly."
        )

    def get_config(self):
        def ser(q):
            if q is None:
                return None
            return {"class_name": type(q).__name__, "config": q.get_config()}

        return {
            "weight_quantizer": ser(self.weight_quantizer),
            "activation_quantizer": ser(self.activation_quantizer),
        }

    @staticmethod
    def _deserialize_quantizer(spec):
        if spec is None:
            return None
        if spec["class_name"] != "AbsMaxQuantizer":
            raise ValueError(f"Unknown quantizer class: {spec['class_name']}")
        cfg = dict(spec["config"])
        for key in ("value_range", "axis"):
            if key in cfg and cfg[key] is not None:
                cfg[key] = tuple(cfg[key])
        return AbsMaxQuantizer(**cfg)

    @classmethod
    def from_config(cls, config):
        return cls(
            weight_quantizer=cls._deserialize_quantizer(config.get("weight_quantizer")),
            activation_quantizer=cls._deserialize_quantizer(config.get("activation_quantizer")),
        )

    @staticmethod
    def weight_quantizer_or_default(config, default):
        if config is not None and config.weight_quantizer is not None:
            return config.weight_quantizer
        return default

    @staticmethod
    def activation_quantizer_or_default(config, default):
        if config is not None:
            return config.activation_quantizer
        return default


class Int8QuantizationConfig(QuantizationConfig):
    """W8A8 dynamic: int8 weights, per-row dynamic int8 activations."""

    def __init__(self, weight_quantizer=None, activation_quantizer="default"):
        if activation_quantizer == "default":
            activation_quantizer = AbsMaxQuantizer()
        super().__init__(weight_quantizer, activation_quantizer)
        if self.weight_quantizer is not None:
            if self.weight_quantizer.output_dtype != "int8":
                raise ValueError(
                    "Int8QuantizationConfig requires a weight_quantizer "
                    "with output_dtype='int8'. Received: "
                    f"output_dtype={self.weight_quantizer.output_dtype}"
                )

    @property
    def mode(self):
        return "int8"


class Int4QuantizationConfig(QuantizationConfig):
    """W4A16 weight-only; grouped (block_size 128) unless block_size is None / -1."""

    def __init__(self, weight_quantizer=None, activation_quantizer="default", block_size=128):
        if activation_quantizer == "default":
            activation_quantizer = None
        super().__init__(weight_quantizer, activation_quantizer)
        if block_size is not None and block_size != -1 and block_size <= 0:
            raise ValueError(
                f"block_size must be None, -1, or a positive integer. "
                f"Received: block_size={block_size}"
            )
        self.block_size = block_size
        is_sub_channel = block_size is not None and block_size > 0
        has_custom_quantizer = (
            self.weight_quantizer is not None or self.activation_quantizer is not None
        )
        if is_sub_channel and has_custom_quantizer:
            raise ValueError(
                "Int4 sub-channel quantization (block_size > 0) does not "
                "support custom quantizers. Either set block_size to None "
                "or -1 for per-channel quantization, or remove the custom "
                f"quantizer arguments. Received: block_size={block_size}"
            )
        if self.weight_quantizer is not None:
            if self.weight_quantizer.value_range != (-8, 7):
                raise ValueError(
                    "Int4QuantizationConfig requires a weight_quantizer "
                    "with value_range=(-8, 7). Received: "
                    f"value_range={self.weight_quantizer.value_range}"
                )
            if self.weight_quantizer.output_dtype != "int8":
                raise ValueError(
                    "Int4QuantizationConfig requires a weight_quantizer "
                    "with output_dtype='int8'. Received: "
                    f"output_dtype={self.weight_quantizer.output_dtype}"
                )

    @property
    def mode(self):
        return "int4"

    def get_config(self):
        config = super().get_config()
        config["block_size"] = self.block_size
        return config

    @classmethod
    def from_config(cls, config):
        return cls(
            weight_quantizer=cls._deserialize_quantizer(config.get("weight_quantizer")),
            activation_quantizer=cls._deserialize_quantizer(config.get("activation_quantizer")),
            block_size=config.get("block_size", None),
        )


def _validate_mode(mode):
    if mode is not None and mode not in QUANTIZATION_MODES:
        raise ValueError(
            "Invalid quantization mode. "
            f"Expected one of {QUANTIZATION_MODES}. Received: mode={mode}"
        )


def validate_and_resolve_config(mode, config):
    """`quantize(mode, config)` arguments -> one config object (reference :256-341)."""
    if isinstance(config, str):
        mode = config
        config = None
    _validate_mode(mode)
    if config is None:
        if mode == "int8":
            config = Int8QuantizationConfig()
        elif mode == "int4":
            config = Int4QuantizationConfig()
        elif mode == "gptq":
            raise ValueError(
                "For GPTQ, you must pass a `GPTQConfig` object in the `config` argument."
            )
        elif mode == "awq":
            raise ValueError(
                "For AWQ, you must pass an `AWQConfig` object in the `config` argument."
            )
        elif mode in ("float8", "ternary"):
            raise NotImplementedError(
                f"Quantization mode '{mode}' is outside the int8 / int4 inference path "
                "implemented here."
            )
        else:
            raise ValueError("You must provide either `mode` or `config` to `quantize`.")
    elif not isinstance(config, QuantizationConfig):
        raise ValueError(
            "Argument `config` must be an instance of `QuantizationConfig`. "
            f"Received: config={config} (of type {type(config)})"
        )
    if mode is not None and config.mode != mode:
        raise ValueError(
            f"Contradictory arguments: mode='{mode}' but config.mode='{config.mode}'"
        )
    _validate_mode(config.mode)
    return config


def get_block_size_for_layer(layer, config):
    """Group size for int4: from the config when one is given, else from the layer's
    `Int4DTypePolicy`; None means per-channel (reference :352-390)."""
    if config and isinstance(config, Int4QuantizationConfig):
        return config.block_size
    if isinstance(layer.dtype_policy, Int4DTypePolicy):
        block_size = layer.dtype_policy.block_size
        return None if block_size == -1 else block_size
    return None
