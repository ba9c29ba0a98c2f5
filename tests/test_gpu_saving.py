"""GPU: a model quantized on the device, saved in the reference's formats and loaded again
computes the same outputs bit for bit."""

import pytest
import torch

import keras_amd as ka
from keras_amd import saving
from keras_amd.models import Model

pytestmark = pytest.mark.gpu


class Stack(Model):
    def __init__(self, dtype="mixed_bfloat16", layer_dtype=None, **kwargs):
        super().__init__(dtype=dtype, **kwargs)
        # a saved model re-creates its layers under the (quantized) policy they were saved with
        kw = dict(dtype=layer_dtype or dtype, device=self.device)
        if layer_dtype and layer_dtype.startswith("int4"):
            # what quantize("int4") resolved to; without it a policy-built ReversibleEmbedding
            # takes the default activation quantizer (reversible_embedding.py:229-233)
            kw["quantization_config"] = ka.Int4QuantizationConfig()
        self.embed = ka.layers.ReversibleEmbedding(512, 256, tie_weights=True, **kw)
        self.proj = ka.layers.EinsumDense("abc,cde->abde", output_shape=(None, 4, 64), bias_axes="e", **kw)
        self.ffn = [ka.layers.Dense(512, activation="relu", **kw), ka.layers.Dense(256, **kw)]
        self.embed.build()
        self.proj.build((2, 8, 256))
        self.ffn[0].build((2, 8, 256))
        self.ffn[1].build((2, 8, 512))

    def get_config(self):
        return {"name": self.name, "dtype": self.dtype_policy.name,
                "layer_dtype": self.ffn[0].dtype_policy.name}

    def forward(self, ids):
        x = self.embed(ids)
        p = self.proj(x)
        x = self.ffn[1](self.ffn[0](p.reshape(*p.shape[:2], -1)))
        return x, self.embed(x, reverse=True)


@pytest.mark.parametrize("mode", ["int8", "int4"])
@pytest.mark.parametrize("dtype", ["mixed_bfloat16", "float32"])
def test_quantize_save_load_same_outputs(dev, tmp_path, mode, dtype):
    torch.manual_seed(0)
    model = Stack(dtype=dtype, device=dev, name="stack")
    report = model.quantize(mode)
    assert report.num_quantized == 4
    ids = torch.randint(0, 512, (2, 8), device=dev)
    want_x, want_logits = model.forward(ids)

    path = tmp_path / "stack.keras"
    model.save(path)
    loaded = saving.load_model(path, custom_objects={"Stack": Stack}, device=dev)
    assert isinstance(loaded, Stack) and loaded.name == "stack"
    assert loaded.dtype_policy.name == model.dtype_policy.name
    for a, b in zip(model._flatten_layers(), loaded._flatten_layers()):
        assert type(a) is type(b) and a.dtype_policy.name == b.dtype_policy.name
        assert b.quantization_mode == mode
        # creation order differs (converted after build vs built under the policy): by name
        va, vb = {v.name: v for v in a._variables}, {v.name: v for v in b._variables}
        assert va.keys() == vb.keys()
        for name in va:
            assert va[name].dtype == vb[name].dtype and torch.equal(va[name].value, vb[name].value), name
    got_x, got_logits = loaded.forward(ids)
    assert torch.equal(got_x, want_x) and torch.equal(got_logits, want_logits)

    # weights-only file into a model converted separately
    wpath = tmp_path / "stack.weights.h5"
    model.save_weights(wpath)
    other = Stack(dtype=dtype, device=dev, name="other")
    other.quantize(mode)
    other.load_weights(wpath)
    again_x, again_logits = other.forward(ids)
    assert torch.equal(again_x, want_x) and torch.equal(again_logits, want_logits)
