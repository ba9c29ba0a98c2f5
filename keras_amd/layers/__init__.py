from keras_amd.layers.dense import Dense
from keras_amd.layers.einsum_dense import EinsumDense
from keras_amd.layers.embedding import Embedding, ReversibleEmbedding
from keras_amd.layers.together import call_add, call_together

__all__ = ["Dense", "EinsumDense", "Embedding", "ReversibleEmbedding", "call_add", "call_together"]
