"""CPU: host logic of the Embedding / ReversibleEmbedding mirrors -- variables, shapes, policy
names, store order, argument checks.  Nothing here launches a kernel."""

import pytest
import torch

from keras_amd.layers import Embedding, ReversibleEmbedding
from keras_amd.quantization_config import Int4QuantizationConfig
from oracle import keras_cpu_path as ref


def test_constructor_checks():
    for bad in (0, -3, 2.5, True):
        with pytest.raises(ValueError, match="`input_dim` must be a positive integer"):
            Embedding(bad, 4, device="cpu")
        with pytest.raises(ValueError, match="`output_dim` must be a positive integer"):
            Embedding(4, bad, device="cpu")
    layer = Embedding(5, 4, device="cpu")
    with pytest.raises(AttributeError, match="build the layer"):
        layer.embeddings
    with pytest.raises(ValueError, match="isn't yet built"):
        layer.quantize("int8")


def test_float_call_and_int8_conversion_on_host():
    layer = Embedding(10, 16, device="cpu", mask_zero=True)
    layer.build()
    ids = torch.tensor([[1, 0, -1]])
    out = layer(ids)
    t = layer._embeddings.value
    assert torch.equal(out[0, 2], t[9]) and tuple(out.shape) == (1, 3, 16)
    assert torch.equal(layer.compute_mask(ids), torch.tensor([[True, False, True]]))
    assert layer.compute_output_shape((2, 7)) == (2, 7, 16)
    table = t.clone()
    layer.quantize("int8")
    q, s = ref.embedding_quantize_int8(table)
    assert layer.dtype_policy.name == "int8_from_float32" and layer.quantization_mode == "int8"
    assert torch.equal(layer._embeddings.value, q) and torch.equal(layer.embeddings_scale.value, s)
    assert layer._embeddings.shape == (10, 16) and layer.embeddings_scale.shape == (10,)
    assert [v.name.split("/")[-1] for v in layer._variables] == ["embeddings", "embeddings_scale"]
    with pytest.raises(ValueError, match="already quantized"):
        layer.quantize("int8")
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        layer(ids)
    store = {}
    layer.save_own_variables(store)
    assert sorted(store) == ["0", "1"] and store["0"].dtype == torch.int8
    clone = Embedding(10, 16, dtype="int8_from_float32", device="cpu")
    clone.build()
    clone.load_own_variables(store)
    assert torch.equal(clone._embeddings.value, q)
    with pytest.raises(ValueError, match="shape"):
        clone._embeddings.assign(torch.zeros(3, 3, dtype=torch.int8))


@pytest.mark.parametrize("policy,scale_shape,grouped", [
    ("int4/128_from_float32", (100, 2), True), ("int4/64_from_bfloat16", (100, 4), True),
    ("int4/-1_from_float32", (100,), False),
])
def test_int4_layer_built_from_policy(policy, scale_shape, grouped):
    layer = Embedding(100, 256, dtype=policy, device="cpu")
    layer.build()
    assert layer._embeddings.shape == (100, 128) and layer._embeddings.dtype == "int8"
    assert layer.embeddings_scale.shape == scale_shape
    assert hasattr(layer, "embeddings_zero") == grouped and hasattr(layer, "g_idx") == grouped
    if grouped:
        bs = layer._int4_block_size
        assert layer.embeddings_zero.dtype == "int8" and layer.g_idx.dtype == "float32"
        assert torch.equal(layer.g_idx.value, torch.floor_divide(torch.arange(256.0), bs))
        assert list(layer.variable_serialization_spec["int4"]) == [
            "embeddings", "embeddings_scale", "embeddings_zero", "g_idx"]
    store = {}
    layer.save_own_variables(store)
    assert len(store) == (4 if grouped else 2)


def test_odd_output_dim_packs_to_ceil():
    layer = Embedding(7, 33, dtype="int4/-1_from_float32", device="cpu")
    layer.build()
    assert layer._embeddings.shape == (7, 17) and layer._orig_output_dim == 33


def test_subclass_is_not_quantized_by_the_parent():
    class Sub(Embedding):
        pass

    sub = Sub(4, 4, device="cpu")
    sub.build()
    with pytest.raises(NotImplementedError, match="does not have a `quantize` method"):
        sub.quantize("int8")
    with pytest.raises(ValueError):
        Embedding(4, 4, device="cpu").quantize("gptq")


def test_reversible_embedding_variables():
    tied = ReversibleEmbedding(50, 32, device="cpu")
    tied.build()
    assert not hasattr(tied, "reverse_embeddings")
    x = torch.randn(3, 32)
    assert torch.allclose(tied(x, reverse=True), x @ tied._embeddings.value.T)
    assert tied.compute_output_shape((2, 5, 32), reverse=True) == [2, 5, 50]
    assert tied.compute_output_shape((2, 5)) == [2, 5, 32]
    capped = ReversibleEmbedding(50, 32, device="cpu", logit_soft_cap=2.0)
    capped.build()
    assert capped(x, reverse=True).abs().max() <= 2.0
    untied = ReversibleEmbedding(50, 32, tie_weights=False, device="cpu")
    untied.build()
    assert untied.reverse_embeddings.shape == (32, 50)
    rt, ft = untied.reverse_embeddings.value.clone(), untied._embeddings.value.clone()
    untied.quantize("int8")
    assert untied.reverse_embeddings.dtype == "int8" and untied.reverse_embeddings_scale.shape == (50,)
    rq, rs = ref.dense_quantize_int8(rt)  # abs-max over axis 0, as for a Dense kernel
    assert torch.equal(untied.reverse_embeddings.value, rq)
    assert torch.equal(untied.reverse_embeddings_scale.value, rs)
    assert torch.equal(untied._embeddings.value, ref.embedding_quantize_int8(ft)[0])
    assert untied.variable_serialization_spec["int8"] == [
        "embeddings", "embeddings_scale", "reverse_embeddings", "reverse_embeddings_scale"]
    assert untied.inputs_quantizer is not None
    store = {}
    untied.save_own_variables(store)
    assert len(store) == 4
    # built from a policy: the reference gives such a layer the default activation quantizer
    pol = ReversibleEmbedding(50, 32, tie_weights=False, dtype="int4/16_from_float32", device="cpu")
    pol.build()
    assert pol.inputs_quantizer is not None
    assert pol.reverse_embeddings.shape == (16, 50) and pol.reverse_embeddings_scale.shape == (2, 50)
    assert pol.reverse_embeddings_zero.dtype == "float32"  # variable dtype, not int8, as in the reference
    cfg = ReversibleEmbedding(50, 32, dtype="int4/16_from_float32", device="cpu",
                              quantization_config=Int4QuantizationConfig(block_size=16))
    cfg.build()
    assert cfg.inputs_quantizer is None
