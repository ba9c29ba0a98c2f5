"""MI355X-native quantized inference path of Keras 3 `Dense` / `EinsumDense`."""

from keras_amd import quantizers  # noqa: F401

__version__ = "0.1.0"
