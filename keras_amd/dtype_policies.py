"""Dtype-policy names of the quantized path.

Only the naming contract of the reference is kept: `"float32"`, `"bfloat16"`,
`"mixed_bfloat16"`, `"int8_from_<source>"`, `"int4/<block_size>_from_<source>"`
(keras/src/dtype_policies/dtype_policy.py:215-256, :291-370, :606-638).
"""

import torch

QUANTIZATION_MODES = ("int8", "float8", "int4", "ternary", "gptq", "awq")

_DTYPES = {"float32": torch.float32, "bfloat16": torch.bfloat16, "float16": torch.float16}


class DTypePolicy:
    """`name` -> (compute dtype, variable dtype); "mixed_X" computes in X and
    keeps variables in float32."""

    def __init__(self, name="float32"):
        if not isinstance(name, str):
            raise TypeError(f"'name' must be a string, such as 'mixed_bfloat16'. Received: name={name}")
        self._name = name
        if name.startswith("mixed_"):
            compute, variable = name[len("mixed_"):], "float32"
        else:
            compute = variable = name
        if compute not in _DTYPES:
            raise ValueError(f"Cannot convert '{name}' to a mixed precision DTypePolicy.")
        self._compute_dtype = compute
        self._variable_dtype = variable

    @property
    def name(self):
        return self._name

    @property
    def compute_dtype(self):
        return self._compute_dtype

    @property
    def variable_dtype(self):
        return self._variable_dtype

    @property
    def quantization_mode(self):
        return None

    def __eq__(self, other):
        return type(self) is type(other) and self.name == other.name

    def __repr__(self):
        return f'<{type(self).__name__} "{self._name}">'


class QuantizedDTypePolicy(DTypePolicy):
    def __init__(self, mode, source_name=None):
        source_name = source_name or "float32"
        if mode not in QUANTIZATION_MODES:
            raise ValueError(
                "Invalid quantization mode. "
                f"Expected one of {QUANTIZATION_MODES}. Received: mode={mode}"
            )
        super().__init__(source_name)
        self._source_name = source_name
        self._quantization_mode = mode
        self._name = f"{mode}_from_{source_name}"

    @property
    def quantization_mode(self):
        return self._quantization_mode

    def __eq__(self, other):
        return (
            isinstance(other, QuantizedDTypePolicy)
            and self._quantization_mode == other._quantization_mode
            and self._source_name == other._source_name
            and getattr(self, "block_size", None) == getattr(other, "block_size", None)
        )


class Int4DTypePolicy(QuantizedDTypePolicy):
    """`"int4/<block_size>"`; -1 (or the legacy literal "None") means per-channel."""

    def __init__(self, mode, source_name=None):
        parts = mode.split("/")
        expected_format = "'int4/<block_size>'"
        if len(parts) != 2 or parts[0] != "int4":
            raise ValueError(
                "Invalid mode for Int4DTypePolicy. Expected format "
                f"{expected_format}, but got '{mode}'."
            )
        if parts[1] == "None":
            block_size = -1
        else:
            try:
                block_size = int(parts[1])
            except ValueError:
                raise ValueError(
                    "Invalid mode for Int4DTypePolicy. <block_size> must be "
                    f"an integer. Expected format {expected_format}, but got '{mode}'."
                )
        if block_size < -1 or block_size == 0:
            raise ValueError(
                "Invalid block_size in mode. Supported values are "
                "-1 (per-channel) or a positive integer (sub-channel), "
                f"but got {block_size} from '{mode}'."
            )
        super().__init__(mode="int4", source_name=source_name)
        self._name = f"int4/{block_size}_from_{self._source_name}"
        self.block_size = block_size


def get(identifier):
    """Policy object from a policy or a name such as "int4/128_from_mixed_bfloat16"."""
    if identifier is None:
        return DTypePolicy("float32")
    if isinstance(identifier, DTypePolicy):
        return identifier
    if isinstance(identifier, torch.dtype):
        identifier = str(identifier).replace("torch.", "")
    if not isinstance(identifier, str):
        raise ValueError(f"Cannot interpret `dtype` argument. Received: {identifier}")
    if identifier.startswith(QUANTIZATION_MODES):
        if "_from_" not in identifier:
            raise ValueError(
                "Cannot convert `policy` into a valid pair (`mode`, `source_name`) "
                f"to instantiate `QuantizedDTypePolicy`. Received: policy={identifier}"
            )
        mode, source = identifier.split("_from_", 1)
        if mode.startswith("int4/"):
            return Int4DTypePolicy(mode, source)
        return QuantizedDTypePolicy(mode, source)
    return DTypePolicy(identifier)
