"""CPU: the `Model.quantize` walk (keras/src/models/model.py:454-699) on stand-in layers --
what is visited, what is skipped and why, which exceptions propagate, what the report says."""

import warnings

import pytest

from keras_amd.layers.layer import Layer
from keras_amd.models import Model, QuantizationReport, should_quantize_layer


class Quantizable(Layer):
    def __init__(self, name):
        super().__init__(name=name, device="cpu")
        self.built = True
        self.calls = []

    def _quantize(self, mode, config, type_check=True):
        self.calls.append((mode, type(config).__name__, type_check))
        self._is_quantized = True
        self._dtype_policy = __import__("keras_amd").dtype_policies.get(
            f"{'int4/128' if mode == 'int4' else mode}_from_float32")


class Plain(Layer):  # no quantized form: Layer._quantize raises NotImplementedError
    def __init__(self, name):
        super().__init__(name=name, device="cpu")
        self.built = True


class Broken(Quantizable):
    def _quantize(self, mode, config, type_check=True):
        raise RuntimeError("real bug")


class Inner(Model):
    def __init__(self):
        super().__init__(name="inner", device="cpu")
        self.deep = Quantizable("deep_dense")


class Net(Model):
    def __init__(self, broken=False):
        super().__init__(name="net", device="cpu")
        self.a = Quantizable("attn_query")
        self.norm = Plain("norm")
        self.stack = [Quantizable("ffn_up"), {"x": Quantizable("ffn_down")}]
        self.inner = Inner()
        self.shared = self.a  # the same layer reachable twice is visited once
        if broken:
            self.bad = Broken("bad")


def run(model, *args, **kwargs):
    with warnings.catch_warnings(record=True) as w:
        warnings.simplefilter("always")
        report = model.quantize(*args, **kwargs)
    return report, [str(x.message) for x in w]


def test_walk_order_and_skips():
    net = Net()
    names = [l.name for l in net._flatten_layers()]
    assert names == ["attn_query", "norm", "ffn_up", "ffn_down", "inner", "deep_dense"]
    report, warned = run(net, "int8")
    assert [p for p, _, _ in report.quantized] == ["attn_query", "ffn_up", "ffn_down", "deep_dense"]
    assert all(m == "int8" and s == "int8_from_float32" for _, m, s in report.quantized)
    assert report.skipped == [("norm", QuantizationReport.SKIP_NO_SUPPORT)]  # nested model: not listed
    assert net.a.calls == [("int8", "Int8QuantizationConfig", True)]
    assert len(warned) == 1 and "1 layer(s) were skipped because they do not support quantization" in warned[0]
    assert "Quantized 4 layer(s) in mode 'int8'" in warned[0]
    assert net._quantization_report is report
    again, _ = run(net, "int8")
    assert again.num_quantized == 0
    assert len(again.skipped_by_reason(QuantizationReport.SKIP_ALREADY_QUANTIZED)) == 4
    assert "Quantization report (mode='int8')" in report.render()


@pytest.mark.parametrize("filters,expected", [
    ("ffn", ["ffn_up", "ffn_down"]),
    (["query$", "^deep"], ["attn_query", "deep_dense"]),
    (lambda l: l.name.endswith("down"), ["ffn_down"]),
])
def test_filters(filters, expected):
    net = Net()
    report, _ = run(net, "int4", filters=filters)
    assert [p for p, _, _ in report.quantized] == expected
    assert all(s == "int4/128_from_float32" for _, _, s in report.quantized)
    filtered = report.skipped_by_reason(QuantizationReport.SKIP_FILTERED)
    assert "norm" in filtered and len(filtered) == 5 - len(expected)
    assert should_quantize_layer(net.a, None) and should_quantize_layer(net.a, 42)


def test_errors_propagate_and_arguments_are_checked():
    with pytest.raises(RuntimeError, match="real bug"):
        Net(broken=True).quantize("int8")
    net = Net()
    with pytest.raises(ValueError, match="filters"):
        net.quantize("int8", filters=3)
    with pytest.raises(ValueError, match="Unrecognized keyword arguments"):
        net.quantize("int8", nope=True)
    with pytest.raises(ValueError):
        net.quantize("int3")
    report, _ = run(net, "int8", type_check=False)
    assert net.a.calls == [("int8", "Int8QuantizationConfig", False)]
    assert report.summary_warning() is not None
    clean = Model(name="empty", device="cpu")
    r, warned = run(clean, "int8")
    assert r.num_quantized == 0 and r.summary_warning() is None and warned == []
