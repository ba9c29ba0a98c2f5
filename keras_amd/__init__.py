"""MI355X-native quantized inference path of Keras 3 `Dense` / `EinsumDense`.

    keras_amd.quantizers   abs_max_quantize, AbsMaxQuantizer, pack_int4, unpack_int4, ...
    keras_amd.layers       Dense, EinsumDense with quantize("int8" | "int4")
    keras_amd.ops          tensor-level entry points over the C ABI (libk3q.so)
    keras_amd.saving       `.weights.h5` / `.keras` files of quantized models (no h5py)
"""

from keras_amd import dtype_policies, layers, ops, quantization_config, quantizers, saving  # noqa: F401
from keras_amd.quantization_config import (  # noqa: F401
    Int4QuantizationConfig,
    Int8QuantizationConfig,
    QuantizationConfig,
)

__version__ = "0.1.0"
