from keras_amd.layers.dense import Dense
from keras_amd.layers.einsum_dense import EinsumDense
from keras_amd.layers.embedding import Embedding, ReversibleEmbedding

__all__ = ["Dense", "EinsumDense", "Embedding", "ReversibleEmbedding"]
