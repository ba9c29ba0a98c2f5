"""Host-side logic that needs no GPU: configs, policy names, variable layout, store order,
error behaviour and the einsum bookkeeping (product against oracle)."""

import pytest
import torch

import keras_amd as ka
from keras_amd import dtype_policies
from keras_amd.layers import Dense, EinsumDense
from keras_amd.layers import einsum_dense as ked
from keras_amd.quantization_config import validate_and_resolve_config
from oracle import keras_cpu_path as ref


@pytest.fixture
def host_pack(monkeypatch):
    """`pack_int4` is a device kernel; on a GPU-less host the oracle stands in so that the
    rest of `quantize("int4")` (pure host logic) can be exercised."""
    monkeypatch.setattr(ka.quantizers, "pack_int4",
                        lambda arr, axis=0, dtype="int8": ref.pack_int4(arr.cpu(), axis, dtype))


def test_config_resolution():
    c = validate_and_resolve_config("int8", None)
    assert c.mode == "int8" and c.activation_quantizer is not None
    c = validate_and_resolve_config("int4", None)
    assert c.mode == "int4" and c.block_size == 128 and c.activation_quantizer is None
    assert validate_and_resolve_config(None, "int8").mode == "int8"  # string shortcut
    with pytest.raises(ValueError, match="Contradictory"):
        validate_and_resolve_config("int8", ka.Int4QuantizationConfig())
    with pytest.raises(ValueError, match="Invalid quantization mode"):
        validate_and_resolve_config("int5", None)
    with pytest.raises(ValueError, match="must provide either"):
        validate_and_resolve_config(None, None)
    with pytest.raises(ValueError, match="GPTQConfig"):
        validate_and_resolve_config("gptq", None)
    with pytest.raises(ValueError, match="instance of"):
        validate_and_resolve_config("int8", object())


def test_int4_config_validation():
    with pytest.raises(ValueError, match="block_size must be"):
        ka.Int4QuantizationConfig(block_size=0)
    with pytest.raises(ValueError, match="does not support custom quantizers"):
        ka.Int4QuantizationConfig(weight_quantizer=ka.quantizers.AbsMaxQuantizer(axis=0, value_range=(-8, 7)))
    with pytest.raises(ValueError, match="value_range=\\(-8, 7\\)"):
        ka.Int4QuantizationConfig(weight_quantizer=ka.quantizers.AbsMaxQuantizer(axis=0), block_size=None)
    cfg = ka.Int4QuantizationConfig(block_size=64)
    again = ka.Int4QuantizationConfig.from_config(cfg.get_config())
    assert again.block_size == 64
    legacy = ka.Int4QuantizationConfig.from_config({})  # saved before block_size existed
    assert legacy.block_size is None
    with pytest.raises(ValueError, match="within the interval"):
        ka.quantizers.AbsMaxQuantizer(value_range=(-200, 127))
    q = ka.quantizers.AbsMaxQuantizer(axis=-1, value_range=(-8, 7))
    assert q.get_config() == {"value_range": (-8, 7), "epsilon": 1e-7, "output_dtype": "int8", "axis": (-1,)}


def test_dtype_policy_names():
    p = dtype_policies.get("int8_from_mixed_bfloat16")
    assert (p.quantization_mode, p.compute_dtype, p.variable_dtype) == ("int8", "bfloat16", "float32")
    p = dtype_policies.get("int4/128_from_float32")
    assert p.quantization_mode == "int4" and p.block_size == 128 and p.name == "int4/128_from_float32"
    assert dtype_policies.get("int4/None_from_float32").name == "int4/-1_from_float32"  # legacy spelling
    for bad in ("int4/0_from_float32", "int4/x_from_float32", "int4/-2_from_float32"):
        with pytest.raises(ValueError):
            dtype_policies.get(bad)
    with pytest.raises(ValueError):
        dtype_policies.get("int8")


@pytest.mark.parametrize("policy", ["float32", "mixed_bfloat16", "bfloat16"])
def test_dense_int8_quantize_layout(policy):
    layer = Dense(16, dtype=policy, device="cpu")
    layer.build((None, 8))
    kernel = layer._kernel.value.clone()
    layer.quantize("int8")
    assert layer.dtype_policy.name == f"int8_from_{policy}"
    assert layer.quantization_mode == "int8"
    assert layer._kernel.dtype == "int8" and layer._kernel.shape == (8, 16)
    assert layer.kernel_scale.shape == (16,) and layer.kernel_scale.dtype == layer.variable_dtype
    qk, ks = ref.dense_quantize_int8(kernel)
    assert torch.equal(layer._kernel.value, qk) and torch.equal(layer.kernel_scale.value.float(), ks.float())
    store = {}
    layer.save_own_variables(store)
    assert [tuple(store[k].shape) for k in sorted(store)] == [(8, 16), (16,), (16,)]  # kernel, bias, scale
    with pytest.raises(ValueError, match="already quantized"):
        layer.quantize("int8")


@pytest.mark.parametrize("block_size,name", [(128, "int4/128"), (64, "int4/64"), (None, "int4/-1"), (-1, "int4/-1")])
def test_dense_int4_quantize_layout(host_pack, block_size, name):
    layer = Dense(15, use_bias=False, device="cpu")  # odd units: packed width is ceil(15 / 2)
    layer.build((None, 300))
    kernel = layer._kernel.value.clone()
    layer.quantize("int4", config=ka.Int4QuantizationConfig(block_size=block_size))
    assert layer.dtype_policy.name == f"{name}_from_float32"
    assert layer._kernel.shape == (300, 8) and layer._kernel.dtype == "int8"
    assert layer._orig_input_dim == 300 and layer._orig_output_dim == 15
    qk = ref.dense_quantize_int4(kernel, block_size)
    assert torch.equal(layer._kernel.value, qk["kernel"])
    assert torch.equal(layer.kernel_scale.value, qk["kernel_scale"])
    store = {}
    layer.save_own_variables(store)
    if block_size in (None, -1):
        assert layer.kernel_scale.shape == (15,) and not hasattr(layer, "kernel_zero")
        assert list(store) == ["0", "1"]  # kernel, kernel_scale (no bias, no zero, no g_idx)
    else:
        groups = -(-300 // block_size)
        assert layer.kernel_scale.shape == (groups, 15) and layer.kernel_zero.shape == (groups, 15)
        assert layer.kernel_zero.dtype == "int8" and layer.g_idx.dtype == "float32"
        assert torch.equal(layer.g_idx.value, torch.arange(300).float() // block_size)
        assert list(store) == ["0", "1", "2", "3"]
        assert store["2"].dtype == torch.int8 and store["3"].dtype == torch.float32


def test_bare_int4_is_grouped_128(host_pack):
    layer = Dense(16, device="cpu")
    layer.build((None, 256))
    layer.quantize("int4")
    assert layer.dtype_policy.name == "int4/128_from_float32" and layer._int4_block_size == 128


def test_build_from_quantized_policy_and_reload(host_pack):
    src = Dense(16, device="cpu")
    src.build((None, 256))
    src.quantize("int4")
    store = {}
    src.save_own_variables(store)
    dst = Dense(16, dtype="int4/128_from_float32", device="cpu")
    dst.build((None, 256))
    assert dst._kernel.shape == (256, 8) and dst.kernel_zero.shape == (2, 16)
    dst.load_own_variables(store)
    for name in ("_kernel", "kernel_scale", "kernel_zero", "g_idx", "bias"):
        assert torch.equal(getattr(dst, name).value, getattr(src, name).value)
    with pytest.raises(ValueError, match="must match"):
        dst._kernel.assign(torch.zeros(3, 3, dtype=torch.int8))


def test_quantize_errors():
    layer = Dense(4, device="cpu")
    with pytest.raises(ValueError, match="isn't yet built"):
        layer.quantize("int8")
    layer.build((None, 4))
    f16 = Dense(4, dtype="float16", device="cpu")
    f16.build((None, 4))
    with pytest.raises(ValueError, match="float16"):
        f16.quantize("int8")

    class Sub(Dense):
        pass

    sub = Sub(4, device="cpu")
    sub.build((None, 4))
    with pytest.raises(NotImplementedError):
        sub.quantize("int8")


def test_no_silent_cpu_path():
    layer = Dense(4, device="cpu")
    layer.build((None, 8))
    layer.quantize("int8")
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        layer(torch.randn(2, 8))
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        ka.quantizers.abs_max_quantize(torch.randn(2, 8), axis=-1)
    with pytest.raises(RuntimeError):
        ka.quantizers.pack_int4(torch.zeros(2, 2, dtype=torch.int8))
    with pytest.raises(RuntimeError):
        ka.quantizers.unpack_int4(torch.zeros(2, 2, dtype=torch.int8), 4)


EQS = [("btd,dnh->btnh", 3), ("btnh,nhd->btd", 4), ("ab,bcd->acd", 2), ("btd,ndh->btnh", 3),
       ("abcde,afce->acdbf", 5), ("a,b->ab", 1), ("ab,ab->a", 2), ("...b,bc->...c", 3),
       ("ab...,bc->ac...", 4), ("abc,cd->abd", 3), ("abc,cde->abde", 3), ("bnh,nhd->bd", 3)]


@pytest.mark.parametrize("equation,rank", EQS)
def test_einsum_bookkeeping_matches_oracle(equation, rank):
    mine = ked.analyze_quantization_info(equation, rank)
    theirs = ref.einsum_quantization_info(equation, rank)
    for part in ("input", "kernel"):
        assert mine[part] == theirs[part]
    assert mine["custom_gradient_equation"] == theirs["custom_gradient_equation"]


@pytest.mark.parametrize("equation,out,inp,kshape,bias_axes,bshape", [
    ("ab,bcd->acd", (8, 32), (None, 3), (3, 8, 32), "d", (32,)),
    ("btd,dnh->btnh", (None, 32, 128), (8, 512, 4096), (4096, 32, 128), "nh", (32, 128)),
    ("btnh,nhd->btd", (None, 4096), (8, 512, 32, 128), (32, 128, 4096), "d", (4096,)),
    ("abcde,afce->acdbf", (2, 4, 8, 16), (1, 8, 2, 4, 32), (1, 16, 2, 32), "d", (4, 1, 1)),
    ("...b,bc->...c", (5,), (2, 3, 7), (7, 5), "c", (5,)),
    ("ab,bc->ac", 64, (None, 256), (256, 64), None, None),
])
def test_einsum_shapes(equation, out, inp, kshape, bias_axes, bshape):
    k, b, full = ked.analyze_einsum_shapes(equation, bias_axes, inp, out)
    assert k == kshape and b == bshape


def test_einsum_dense_scale_shapes(host_pack):
    cases = [("btd,dnh->btnh", (None, 4, 8), (2, 3, 16), (1, 1, 4, 8)),
             ("btnh,nhd->btd", (None, 16), (2, 3, 4, 8), (1, 1, 16)),
             ("ab,bcd->acd", (8, 32), (None, 3), (1, 8, 32))]
    for eq, out, inp, want in cases:
        layer = EinsumDense(eq, out, device="cpu")
        layer.build(inp)
        layer.quantize("int8")
        assert layer.kernel_scale.shape == want and layer.dtype_policy.name == "int8_from_float32"
    # int4: flattened [rows, cols] kernel, (n_groups, cols) scales (einsum_dense_test.py:1599-1640)
    for block_size, scale_shape in [(64, (4, 64)), (128, (2, 64)), (None, (64,)), (-1, (64,))]:
        layer = EinsumDense("ab,bc->ac", 64, bias_axes="c", device="cpu")
        layer.build((None, 256))
        layer.quantize("int4", config=ka.Int4QuantizationConfig(block_size=block_size))
        assert layer._kernel.shape == (256, 32) and layer.kernel_scale.shape == scale_shape
        assert layer._int4_block_size == (None if block_size in (None, -1) else block_size)
    layer = EinsumDense("bnh,nhd->bd", 8, device="cpu")  # two reduced axes flattened into rows
    layer.build((None, 4, 64))
    layer.quantize("int4", config=ka.Int4QuantizationConfig(block_size=128))
    assert layer._kernel.shape == (256, 4) and layer.kernel_scale.shape == (2, 8)


def test_einsum_errors():
    with pytest.raises(ValueError, match="Invalid einsum equation"):
        EinsumDense("ab,bc,cd->ad", 4, device="cpu").build((2, 3))
    with pytest.raises(ValueError, match="Bias dimension"):
        EinsumDense("ab,bc->ac", 4, bias_axes="z", device="cpu").build((2, 3))


def test_autocast_reads_are_cached_until_the_variable_changes():
    # Layer.read under a mixed policy: the cast copy is made once, rebuilt after assign() and after
    # an in-place write to the stored tensor
    layer = Dense(8, dtype="mixed_bfloat16", device="cpu", use_bias=True)
    layer.build((None, 4))
    first = layer.read(layer.bias)
    assert first.dtype == torch.bfloat16 and layer.read(layer.bias) is first
    layer.bias.assign(torch.ones(8))
    second = layer.read(layer.bias)
    assert second is not first and second.float().sum().item() == 8
    layer.bias.value.mul_(2)
    third = layer.read(layer.bias)
    assert third is not second and third.float().sum().item() == 16
    same = Dense(8, dtype="float32", device="cpu")
    same.build((None, 4))
    assert same.read(same.bias) is same.bias.value  # nothing to cast: the stored tensor itself


def test_resident_bytes_counts_variables_once():
    layer = Dense(8, dtype="float32", device="cpu")
    layer.build((None, 4))
    assert layer.resident_bytes() == {"stored": 4 * 8 * 4 + 8 * 4, "derived": 0}
