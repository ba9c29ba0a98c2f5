from keras_amd.layers.dense import Dense
from keras_amd.layers.einsum_dense import EinsumDense

__all__ = ["Dense", "EinsumDense"]
