"""GPU parity: Dense / EinsumDense quantized layers end to end against the CPU oracle."""

import pytest
import torch

import keras_amd as ka
from keras_amd import quantizers as kq
from keras_amd.layers import Dense, EinsumDense
from oracle import keras_cpu_path as ref
from tests.helpers import RTOL, max_rel_err

pytestmark = pytest.mark.gpu

TORCH = {"float32": torch.float32, "bfloat16": torch.bfloat16}


def bits(t):
    return t.view(torch.int16) if t.dtype == torch.bfloat16 else t.view(torch.int32)


def build_dense(dev, K, N, policy, seed, use_bias=True):
    g = torch.Generator().manual_seed(seed)
    layer = Dense(N, use_bias=use_bias, dtype=policy, device=dev,
                  kernel_initializer=lambda s, d: ref.glorot_uniform(s[0], s[1], generator=g).to(d),
                  bias_initializer=lambda s, d: (torch.randn(s, generator=g) * 0.02).to(d))
    layer.build((None, K))
    return layer


@pytest.mark.parametrize("policy", ["float32", "mixed_bfloat16", "bfloat16"])
@pytest.mark.parametrize("M,K,N", [(16, 4096, 4096), (5, 128, 48), (300, 256, 512), (2, 100, 30)])
def test_dense_int8_layer(dev, policy, M, K, N):
    layer = build_dense(dev, K, N, policy, seed=0)
    kernel_f = layer._kernel.value.cpu()
    bias_f = layer.bias.value.cpu()
    cd = TORCH[layer.compute_dtype]
    x = torch.randn(M, K, generator=torch.Generator().manual_seed(1))
    y_float = layer(x)
    layer.quantize("int8")
    assert layer.dtype_policy.name == f"int8_from_{policy}"
    assert layer._kernel.dtype == "int8" and layer.kernel_scale.dtype == layer.variable_dtype
    qk, ks = ref.dense_quantize_int8(kernel_f)
    assert torch.equal(layer._kernel.value.cpu(), qk)
    assert torch.equal(bits(layer.kernel_scale.value.cpu()), bits(ks))
    layer.exact_epilogue = True
    y = layer(x)
    want = ref.dense_int8_call(x.to(cd), qk, ks, bias_f, compute_dtype=cd)
    assert y.dtype == cd
    assert torch.equal(bits(y.cpu()), bits(want))
    layer.exact_epilogue = False
    assert max_rel_err(layer(x), want) <= RTOL[cd]
    # the reference's own (weak) check: dense_test.py:438-463
    mse = (y_float.float().cpu() - y.float().cpu()).pow(2).mean().item()
    mse_ref = (y_float.float().cpu() - want.float()).pow(2).mean().item()
    assert mse <= 1.25 * mse_ref + 1e-5


@pytest.mark.parametrize("policy", ["float32", "mixed_bfloat16"])
@pytest.mark.parametrize("block_size", [128, 64, None, -1])
@pytest.mark.parametrize("M,K,N", [(1, 1024, 512), (16, 512, 384), (7, 300, 64), (40, 256, 96)])
def test_dense_int4_layer(dev, policy, block_size, M, K, N):
    layer = build_dense(dev, K, N, policy, seed=2)
    kernel_f = layer._kernel.value.cpu()
    bias_f = layer.bias.value.cpu()
    cd = TORCH[layer.compute_dtype]
    x = torch.randn(M, K, generator=torch.Generator().manual_seed(3))
    y_float = layer(x)
    layer.quantize("int4", config=ka.Int4QuantizationConfig(block_size=block_size))
    per_channel = block_size is None or block_size == -1
    assert layer.dtype_policy.name == f"int4/{-1 if per_channel else block_size}_from_{policy}"
    qk = ref.dense_quantize_int4(kernel_f, block_size)
    assert torch.equal(layer._kernel.value.cpu(), qk["kernel"])
    assert torch.equal(layer.kernel_scale.value.cpu(), qk["kernel_scale"])
    assert torch.equal(layer.kernel.cpu(), qk["unpacked"])
    if per_channel:
        assert not hasattr(layer, "kernel_zero")
    else:
        assert torch.equal(layer.kernel_zero.value.cpu(), qk["kernel_zero"])
        assert torch.equal(layer.g_idx.value.cpu(), qk["g_idx"])
    y = layer(x)
    want = ref.dense_int4_call(
        x.to(cd), qk["kernel"], qk["kernel_scale"], N, kernel_zero=qk["kernel_zero"],
        g_idx=qk["g_idx"], block_size=block_size, bias=bias_f, compute_dtype=cd)
    assert y.dtype == cd and tuple(y.shape) == (M, N)
    assert max_rel_err(y, want) <= RTOL[cd]
    # quantisation noise must be the reference's, not more (its own weak test bounds the MSE
    # of an 8 -> 16 layer, dense_test.py:438-463; the bound does not carry to other sizes)
    mse = (y_float.float().cpu() - y.float().cpu()).pow(2).mean().item()
    mse_ref = (y_float.float().cpu() - want.float()).pow(2).mean().item()
    assert mse <= 1.25 * mse_ref + 1e-5


def test_dense_leading_axes_and_activation(dev):
    layer = Dense(64, activation="relu", device=dev)
    layer.build((None, None, 256))
    x = torch.randn(2, 3, 256)
    layer.quantize("int8")
    y = layer(x)
    assert tuple(y.shape) == (2, 3, 64) and (y >= 0).all()
    flat = layer(x.reshape(6, 256)).reshape(2, 3, 64)
    assert torch.equal(y, flat)


def test_variables_reload_round_trip(dev):
    a = build_dense(dev, 512, 256, "float32", seed=5)
    a.quantize("int4")
    store = {}
    a.save_own_variables(store)
    assert list(store) == ["0", "1", "2", "3", "4"]
    b = Dense(256, dtype="int4/128_from_float32", device=dev)
    b.build((None, 512))
    b.load_own_variables({k: v.cpu() for k, v in store.items()})
    x = torch.randn(3, 512)
    assert torch.equal(a(x), b(x))


EQUATIONS = [
    # equation, output_shape, input_shape  (einsum_dense_test.py:556-691 and the target attention-projection shapes, scaled)
    ("btnh,nhd->btd", (None, 8), (1, 2, 2, 4)),
    ("btd,ndh->btnh", (None, 2, 8), (1, 2, 4)),
    ("btd,df->btf", (None, 4), (1, 2, 4)),
    ("ab,bcd->acd", (8, 32), (2, 3)),
    ("btd,dnh->btnh", (None, 4, 32), (3, 5, 256)),
    ("btnh,nhd->btd", (None, 256), (3, 5, 4, 64)),
    ("...b,bc->...c", (24,), (2, 3, 128)),
]


@pytest.mark.parametrize("equation,output_shape,input_shape", EQUATIONS)
@pytest.mark.parametrize("policy", ["float32", "mixed_bfloat16"])
def test_einsum_dense_int8(dev, equation, output_shape, input_shape, policy):
    g = torch.Generator().manual_seed(1337)
    layer = EinsumDense(equation, output_shape, dtype=policy, device=dev,
                        kernel_initializer=lambda s, d: (torch.rand(s, generator=g) - 0.5).to(d))
    layer.build(input_shape)
    cd = TORCH[layer.compute_dtype]
    kernel_f = layer._kernel.value.cpu()
    x = torch.rand(input_shape, generator=g)
    y_float = layer(x)
    layer.quantize("int8")
    qk, ks, _ = ref.einsum_dense_quantize_int8(kernel_f, equation, len(input_shape))
    assert torch.equal(layer._kernel.value.cpu(), qk)
    assert tuple(layer.kernel_scale.shape) == tuple(ks.shape)
    assert torch.equal(layer.kernel_scale.value.cpu(), ks)
    layer.exact_epilogue = True
    y = layer(x)
    want = ref.einsum_dense_int8_call(x.to(cd), qk, ks, equation, compute_dtype=cd)
    assert tuple(y.shape) == tuple(want.shape)
    assert torch.equal(bits(y.cpu().contiguous()), bits(want.contiguous()))
    assert (y_float.float() - y.float()).pow(2).mean().item() < 2e-2


# equations outside the plain GEMM view: labels shared by input, kernel and output, no summed
# label, a label the input alone carries; the first three are the reference's own
# (einsum_dense_test.py:598-629: "reduce and transpose", "expand", "squeeze")
GENERAL = [
    ("abcde,afce->acdbf", (2, 4, 8, 16), (1, 8, 2, 4, 32), "d"),
    ("a,b->ab", (4,), (5,), None),
    ("ab,ab->a", (2,), (2, 4), None),
    ("ab,c->ac", (5,), (3, 4), "c"),
    ("bhqd,hdk->bhqk", (8, 16, 96), (3, 8, 16, 64), "k"),
    ("abcde,afce->acdbf", (3, 4, 40, 48), (2, 40, 3, 4, 256), None),
]


@pytest.mark.parametrize("equation,output_shape,input_shape,bias_axes", GENERAL)
@pytest.mark.parametrize("policy", ["float32", "mixed_bfloat16"])
def test_einsum_dense_int8_general_equations(dev, equation, output_shape, input_shape, bias_axes, policy):
    g = torch.Generator().manual_seed(99)
    layer = EinsumDense(equation, output_shape, bias_axes=bias_axes, dtype=policy, device=dev,
                        kernel_initializer=lambda s, d: (torch.rand(s, generator=g) - 0.5).to(d),
                        bias_initializer=lambda s, d: torch.randn(s, generator=g).to(d))
    layer.build(input_shape)
    cd = TORCH[layer.compute_dtype]
    kernel_f = layer._kernel.value.cpu()
    bias_f = layer.bias.value.cpu() if layer.bias is not None else None
    x = torch.rand(input_shape, generator=g) - 0.3
    y_float = layer(x)
    layer.quantize("int8")
    assert layer.dtype_policy.name == f"int8_from_{policy}"
    qk, ks, _ = ref.einsum_dense_quantize_int8(kernel_f, equation, len(input_shape))
    assert layer._kernel.dtype == "int8" and layer.kernel_scale.dtype == "float32"
    assert torch.equal(layer._kernel.value.cpu(), qk)
    assert tuple(layer.kernel_scale.shape) == tuple(ks.shape)
    assert torch.equal(layer.kernel_scale.value.cpu(), ks)
    y = layer(x)
    want = ref.einsum_dense_int8_call(x.to(cd), qk, ks, equation, bias=bias_f, compute_dtype=cd)
    # (the reference's scale bookkeeping gives "ab,ab->a" a [1, a] result: kept as it is)
    assert tuple(y.shape) == tuple(want.shape) and y.dtype == cd
    assert torch.equal(bits(y.cpu().contiguous()), bits(want.contiguous()))
    assert (y_float.float().cpu() - y.float().cpu()).pow(2).mean().item() < 2e-2
    # the same layer built from its quantized policy (as the reference's test does), variables loaded
    twin = EinsumDense(equation, output_shape, bias_axes=bias_axes, dtype=f"int8_from_{policy}", device=dev)
    twin.build(input_shape)
    assert twin._kernel.dtype == "int8" and twin.kernel_scale.dtype == "float32"
    store = {}
    layer.save_own_variables(store)
    twin.load_own_variables(store)
    assert torch.equal(bits(twin(x).cpu().contiguous()), bits(want.contiguous()))


@pytest.mark.parametrize("equation,output_shape,input_shape,bias_axes", GENERAL)
@pytest.mark.parametrize("block_size", [8, None])
@pytest.mark.parametrize("policy", ["float32", "mixed_bfloat16"])
def test_einsum_dense_int4_general_equations(dev, equation, output_shape, input_shape, bias_axes, block_size, policy):
    g = torch.Generator().manual_seed(98)
    layer = EinsumDense(equation, output_shape, bias_axes=bias_axes, dtype=policy, device=dev,
                        kernel_initializer=lambda s, d: (torch.rand(s, generator=g) - 0.5).to(d),
                        bias_initializer=lambda s, d: torch.randn(s, generator=g).to(d))
    layer.build(input_shape)
    cd = TORCH[layer.compute_dtype]
    kernel_f = layer._kernel.value.cpu()
    bias_f = layer.bias.value.cpu() if layer.bias is not None else None
    x = torch.rand(input_shape, generator=g) - 0.3
    layer.quantize("int4", config=ka.Int4QuantizationConfig(block_size=block_size))
    qk = ref.einsum_dense_quantize_int4(kernel_f, equation, len(input_shape), block_size)
    assert torch.equal(layer._kernel.value.cpu(), qk["kernel"])
    assert torch.equal(layer.kernel_scale.value.cpu(), qk["kernel_scale"])
    y = layer(x)
    want = ref.einsum_dense_int4_call(x.to(cd), qk, equation, bias=bias_f, compute_dtype=cd,
                                      block_size=block_size)
    assert tuple(y.shape) == tuple(want.shape) and y.dtype == cd
    # the same op sequence as the reference on the device (de-quantise, reshape, float einsum):
    # only the order of the sums inside the einsum differs
    assert max_rel_err(y, want) <= RTOL[cd]


# kernels whose contracted axis is not leading ("ndh" contracts d): the stored int4 matrix is a
# row-major reshape that mixes output columns, so these run de-quantise + float GEMM
NON_LEADING = [
    EQUATIONS[1],
    ("btd,ndh->btnh", (None, 8, 64), (2, 5, 256)),
    ("btd,ndh->btnh", (None, 4, 40), (1, 3, 72)),   # K % 64 != 0: the plain kernel
    ("ab,cb->ac", (48,), (7, 128)),
]


@pytest.mark.parametrize("equation,output_shape,input_shape", NON_LEADING)
@pytest.mark.parametrize("block_size", [128, 8, None])
@pytest.mark.parametrize("policy", ["mixed_bfloat16", "float32"])
def test_einsum_dense_int4_non_leading_contraction(dev, equation, output_shape, input_shape, block_size, policy):
    g = torch.Generator().manual_seed(77)
    layer = EinsumDense(equation, output_shape, dtype=policy, device=dev, bias_axes=None,
                        kernel_initializer=lambda s, d: (torch.rand(s, generator=g) - 0.5).to(d))
    layer.build(input_shape)
    cd = TORCH[layer.compute_dtype]
    kernel_f = layer._kernel.value.cpu()
    x = torch.rand(input_shape, generator=g) - 0.5
    y_float = layer(x)
    layer.quantize("int4", config=ka.Int4QuantizationConfig(block_size=block_size))
    qk = ref.einsum_dense_quantize_int4(kernel_f, equation, len(input_shape), block_size)
    assert torch.equal(layer._kernel.value.cpu(), qk["kernel"])
    assert torch.equal(layer.kernel_scale.value.cpu(), qk["kernel_scale"])
    y = layer(x)
    again = layer(x)  # second call: the cached de-quantised kernel
    want = ref.einsum_dense_int4_call(x.to(cd), qk, equation, compute_dtype=cd, block_size=block_size)
    assert tuple(y.shape) == tuple(want.shape) and y.dtype == cd
    assert torch.equal(y, again)
    assert max_rel_err(y, want) <= RTOL[cd]
    # the float reference evaluated exactly: the kernel is at least about as close as torch's chain
    uk = ref.unpack_int4(qk["kernel"], qk["cols"], axis=-1)
    ks = qk["kernel_scale"].to(cd)
    if block_size is None:
        fk = torch.divide(uk.to(cd), ks)
    else:
        fk = ref.dequantize_with_sz_map(uk, ks, qk["kernel_zero"], qk["g_idx"], group_axis=0).to(cd)
    exact = torch.einsum(equation, x.to(cd).double(), fk.reshape(qk["original_kernel_shape"]).double())
    assert max_rel_err(y, exact) <= max(2 * max_rel_err(want, exact), RTOL[cd] / 4)
    mse = (y_float.float().cpu() - y.float().cpu()).pow(2).mean().item()
    mse_ref = (y_float.float().cpu() - want.float()).pow(2).mean().item()
    assert mse <= 1.25 * mse_ref + 1e-5


@pytest.mark.parametrize("equation,output_shape,input_shape", NON_LEADING[:2])
@pytest.mark.parametrize("policy", ["mixed_bfloat16", "float32"])
def test_einsum_dense_int4_non_leading_activation_quantized(dev, equation, output_shape, input_shape, policy):
    g = torch.Generator().manual_seed(78)
    layer = EinsumDense(equation, output_shape, dtype=policy, device=dev, bias_axes="h",
                        kernel_initializer=lambda s, d: (torch.rand(s, generator=g) - 0.5).to(d),
                        bias_initializer=lambda s, d: (torch.rand(s, generator=g) * 0.1).to(d))
    layer.build(input_shape)
    cd = TORCH[layer.compute_dtype]
    kernel_f = layer._kernel.value.cpu()
    bias = layer.bias.value.cpu()
    x = torch.rand(input_shape, generator=g)
    config = ka.Int4QuantizationConfig(block_size=None, activation_quantizer=ka.quantizers.AbsMaxQuantizer())
    layer.quantize("int4", config=config)
    qk = ref.einsum_dense_quantize_int4(kernel_f, equation, len(input_shape), None)
    y = layer(x)
    want = ref.einsum_dense_int4_activation_quantized_call(x.to(cd), qk, equation, bias=bias, compute_dtype=cd)
    assert tuple(y.shape) == tuple(want.shape) and y.dtype == cd
    assert max_rel_err(y, want) <= RTOL[cd]


@pytest.mark.parametrize("equation,output_shape,input_shape", [EQUATIONS[0], EQUATIONS[2], EQUATIONS[4], EQUATIONS[5]])
@pytest.mark.parametrize("block_size", [128, None])
def test_einsum_dense_int4(dev, equation, output_shape, input_shape, block_size):
    g = torch.Generator().manual_seed(1337)
    layer = EinsumDense(equation, output_shape, dtype="mixed_bfloat16", device=dev,
                        kernel_initializer=lambda s, d: (torch.rand(s, generator=g) - 0.5).to(d))
    layer.build(input_shape)
    kernel_f = layer._kernel.value.cpu()
    x = torch.rand(input_shape, generator=g)
    y_float = layer(x)
    layer.quantize("int4", config=ka.Int4QuantizationConfig(block_size=block_size))
    qk = ref.einsum_dense_quantize_int4(kernel_f, equation, len(input_shape), block_size)
    assert torch.equal(layer._kernel.value.cpu(), qk["kernel"])
    assert torch.equal(layer.kernel_scale.value.cpu(), qk["kernel_scale"])
    y = layer(x)
    want = ref.einsum_dense_int4_call(x.to(torch.bfloat16), qk, equation, compute_dtype=torch.bfloat16,
                                      block_size=block_size)
    assert max_rel_err(y, want) <= RTOL[torch.bfloat16]
    mse = (y_float.float().cpu() - y.float().cpu()).pow(2).mean().item()
    mse_ref = (y_float.float().cpu() - want.float()).pow(2).mean().item()
    assert mse <= 1.25 * mse_ref + 1e-5


@pytest.mark.parametrize("t", [1, 512])
def test_config4_attention_projections(dev, t):
    # target configuration 4: d_model 4096, 32 heads x 128, batch 8, bf16
    g = torch.Generator().manual_seed(4)
    for equation, out_shape, in_shape in [
        ("btd,dnh->btnh", (None, 32, 128), (8, t, 4096)),
        ("btnh,nhd->btd", (None, 4096), (8, t, 32, 128)),
    ]:
        layer = EinsumDense(equation, out_shape, dtype="mixed_bfloat16", device=dev,
                            kernel_initializer=lambda s, d: ref.glorot_uniform(4096, 4096, shape=s, generator=g).to(d))
        layer.build(in_shape)
        kernel_f = layer._kernel.value.cpu()
        x = torch.randn(in_shape, generator=g).to(torch.bfloat16)
        layer.quantize("int8")
        layer.exact_epilogue = True
        y = layer(x)
        qk, ks, _ = ref.einsum_dense_quantize_int8(kernel_f, equation, len(in_shape))
        ts = slice(0, min(t, 16))
        want = ref.einsum_dense_int8_call(x[3:4, ts], qk, ks, equation, compute_dtype=torch.bfloat16)
        assert torch.equal(bits(y[3:4, ts].cpu().contiguous()), bits(want.contiguous()))


def test_unsupported_paths_raise(dev):
    layer = Dense(16, device=dev)
    with pytest.raises(ValueError):
        layer.quantize("int8")  # not built
    layer.build((None, 32))
    with pytest.raises(ValueError):
        layer.quantize("int5")
    layer.quantize("int8")
    with pytest.raises(ValueError):
        layer.quantize("int8")  # already quantized
    cpu_layer = Dense(16, device="cpu")
    cpu_layer.build((None, 32))
    cpu_layer.quantize("int8")
    with pytest.raises(RuntimeError):
        cpu_layer(torch.randn(2, 32))  # no CPU fallback


@pytest.mark.parametrize("mode,block_size", [("int8", None), ("int4", None), ("int4", 128)])
@pytest.mark.parametrize("policy", ["float32", "mixed_bfloat16"])
def test_dense_lora_on_quantized_layer_and_merge_on_save(dev, mode, block_size, policy):
    # keras/src/layers/core/dense.py:251-312 (enable_lora), :972-986 / :1085-1095 (the quantized
    # calls add the low-rank term before the bias), :1301-1427 (the update is merged into what is
    # saved: de-quantise, add, quantise again), :428-430 (a load zeroes the update)
    g = torch.Generator().manual_seed(23)
    M, K, N, rank, alpha = 6, 256, 192, 4, 8
    layer = build_dense(dev, K, N, policy, seed=4)
    cd = TORCH[layer.compute_dtype]
    kernel_f, bias_f = layer._kernel.value.cpu(), layer.bias.value.cpu()
    if mode == "int8":
        layer.quantize("int8")
    else:
        layer.quantize("int4", config=ka.Int4QuantizationConfig(block_size=block_size))
    with pytest.raises(ValueError):
        Dense(4, device=dev).enable_lora(2)          # not built
    layer.enable_lora(rank, lora_alpha=alpha)
    with pytest.raises(ValueError):
        layer.enable_lora(rank)                      # only once
    assert tuple(layer.lora_kernel_a.shape) == (K, rank) and tuple(layer.lora_kernel_b.shape) == (rank, N)
    assert layer.lora_kernel_a.dtype == "float32" and layer.lora_kernel_b.dtype == "float32"
    assert float(layer.lora_kernel_b.value.abs().max()) == 0.0    # b starts at zero
    a = torch.randn(K, rank, generator=g) * 0.05
    b = torch.randn(rank, N, generator=g) * 0.05
    layer.lora_kernel_a.assign(a)
    layer.lora_kernel_b.assign(b)
    x = torch.randn(M, K, generator=g)
    y = layer(x)
    # forward against the oracle: quantized product, + low-rank term, cast, + bias
    if mode == "int8":
        qk, ks = ref.dense_quantize_int8(kernel_f)
        base = ref.dense_int8_call(x.to(cd), qk, ks, None, compute_dtype=cd)
        merged = ref.dense_merged_lora_kernel("int8", qk, ks, a, b, alpha, rank, compute_dtype=cd)
    else:
        q4 = ref.dense_quantize_int4(kernel_f, block_size)
        qk, ks = q4["kernel"], q4["kernel_scale"]
        base = ref.dense_int4_call(x.to(cd), qk, ks, N, kernel_zero=q4["kernel_zero"], g_idx=q4["g_idx"],
                                   block_size=block_size, bias=None, compute_dtype=cd)
        merged = ref.dense_merged_lora_kernel("int4", qk, ks, a, b, alpha, rank, compute_dtype=cd,
                                              kernel_zero=q4["kernel_zero"], g_idx=q4["g_idx"],
                                              block_size=block_size, orig_output_dim=N)
    want = (base + ref.dense_lora_term(x, a, b, alpha, rank, compute_dtype=cd)).to(cd) + bias_f.to(cd)
    assert y.dtype == cd and max_rel_err(y, want) <= RTOL[cd]
    if mode == "int8" and cd == torch.float32:
        # the base product is bit-exact; only the two small float matmuls differ in their sums
        assert max_rel_err(y, want) <= 1e-5
    # what is saved: the merged kernel, its new scales (and zero points), bit for bit the oracle's
    store = {}
    layer.save_own_variables(store)
    names = [n for n in layer.variable_serialization_spec[mode]
             if not (n in ("kernel_zero", "g_idx") and (mode == "int8" or not block_size))]
    got = dict(zip(names, (store[str(i)] for i in range(len(names)))))
    assert len(store) == len(names)
    assert torch.equal(got["kernel"].cpu(), merged[0])
    assert torch.equal(got["kernel_scale"].cpu(), merged[1])
    if block_size:
        assert torch.equal(got["kernel_zero"].cpu(), merged[2])
    assert not torch.equal(got["kernel"].cpu(), qk)
    # a fresh quantized layer without LoRA that loads the store answers like the LoRA layer,
    # to within the quantisation of the merged kernel
    cfg = layer.get_config()
    assert cfg["lora_rank"] == rank and cfg["lora_alpha"] == alpha
    plain = Dense(N, dtype=layer.dtype_policy.name, device=dev)
    plain.build((None, K))
    plain.load_own_variables(store)
    y2 = plain(x)
    assert max_rel_err(y2, y) <= (3e-2 if mode == "int8" else 0.25)
    # loading into the LoRA layer itself zeroes the update (it is in the kernel now)
    layer.load_own_variables(store)
    assert float(layer.lora_kernel_a.value.abs().max()) == 0.0
    assert float(layer.lora_kernel_b.value.abs().max()) == 0.0
    assert torch.equal(bits(layer(x).cpu().contiguous()), bits(y2.cpu().contiguous()))


@pytest.mark.parametrize("mode,block_size", [("int8", None), ("int4", None), ("int4", 64)])
@pytest.mark.parametrize("equation,output_shape,input_shape", [
    ("btd,dnh->btnh", (None, 4, 32), (3, 5, 256)), ("btnh,nhd->btd", (None, 256), (3, 5, 4, 64))])
def test_einsum_dense_lora_on_quantized_layer_and_merge_on_save(dev, mode, block_size, equation, output_shape,
                                                                input_shape):
    # keras/src/layers/core/einsum_dense.py:327-385, :1109-1118 / :1251-1261, :1493-1623, :497-499
    g = torch.Generator().manual_seed(29)
    rank, alpha = 4, 2
    layer = EinsumDense(equation, output_shape, bias_axes=None, dtype="float32", device=dev,
                        kernel_initializer=lambda s, d: (torch.rand(s, generator=g) - 0.5).to(d))
    layer.build(input_shape)
    kernel_f = layer._kernel.value.cpu()
    kshape = tuple(kernel_f.shape)
    if mode == "int8":
        layer.quantize("int8")
        qk, ks, _ = ref.einsum_dense_quantize_int8(kernel_f, equation, len(input_shape))
    else:
        layer.quantize("int4", config=ka.Int4QuantizationConfig(block_size=block_size))
        q4 = ref.einsum_dense_quantize_int4(kernel_f, equation, len(input_shape), block_size)
    layer.enable_lora(rank, lora_alpha=alpha)
    assert tuple(layer.lora_kernel_a.shape) == kshape[:-1] + (rank,)
    assert tuple(layer.lora_kernel_b.shape) == (rank, kshape[-1])
    a = torch.randn(kshape[:-1] + (rank,), generator=g) * 0.05
    b = torch.randn(rank, kshape[-1], generator=g) * 0.05
    layer.lora_kernel_a.assign(a)
    layer.lora_kernel_b.assign(b)
    x = torch.rand(input_shape, generator=g) - 0.4
    y = layer(x)
    lora = (alpha / rank) * torch.matmul(torch.einsum(equation, x, a), b)
    if mode == "int8":
        want = ref.einsum_dense_int8_call(x, qk, ks, equation) + lora
        merged = ref.einsum_dense_merged_lora_kernel("int8", qk, ks, a, b, alpha, rank, equation, len(input_shape))
    else:
        want = ref.einsum_dense_int4_call(x, q4, equation, block_size=block_size) + lora
        merged = ref.einsum_dense_merged_lora_kernel("int4", None, None, a, b, alpha, rank, equation,
                                                     len(input_shape), qk=q4, block_size=block_size)
    assert max_rel_err(y, want) <= 1e-3
    store = {}
    layer.save_own_variables(store)
    assert torch.equal(store["0"].cpu(), merged[0])
    assert tuple(store["1"].shape) == tuple(merged[1].shape) and torch.equal(store["1"].cpu(), merged[1])
    if block_size:
        assert torch.equal(store["2"].cpu(), merged[2])
    plain = EinsumDense(equation, output_shape, dtype=layer.dtype_policy.name, device=dev)
    plain.build(input_shape)
    plain.load_own_variables(store)
    assert max_rel_err(plain(x), y) <= (3e-2 if mode == "int8" else 0.25)
    layer.load_own_variables(store)
    assert float(layer.lora_kernel_a.value.abs().max()) == 0.0 and float(layer.lora_kernel_b.value.abs().max()) == 0.0


def test_non_default_g_idx_is_rejected(dev):
    # the reference looks the group of row k up in g_idx (quantizers.py:1659-1668); the fused kernels
    # take k // block_size, so a stored map that says anything else has to raise, not compute
    for make in (lambda: Dense(64, device=dev), lambda: EinsumDense("ab,bc->ac", (64,), device=dev)):
        layer = make()
        layer.build((None, 256))
        layer.quantize("int4", config=ka.Int4QuantizationConfig(block_size=128))
        x = torch.randn(3, 256, generator=torch.Generator().manual_seed(1))
        layer(x)  # the map quantize() wrote is fine
        g = layer.g_idx.value.clone()
        layer.g_idx.assign(g.flip(0))
        with pytest.raises(ValueError, match="g_idx"):
            layer(x)
        layer.g_idx.assign(g)
        layer(x)


# ---- non-default configs: weight-only int8, activation-quantized int4 --------------------
@pytest.mark.parametrize("policy", ["float32", "mixed_bfloat16", "bfloat16"])
@pytest.mark.parametrize("M,K,N", [(16, 4096, 4096), (5, 128, 48), (300, 256, 512), (2, 100, 30),
                                   (700, 1024, 2048),
                                   # decode sizes: the streaming kernel (1..8 rows, K % 16 == 0)
                                   (1, 4096, 4096), (3, 8192, 1000), (4, 4096, 14336), (8, 1024, 7),
                                   (7, 16, 33), (1, 16384, 64), (9, 4096, 512),
                                   (300, 256, 1001), (40, 512, 30522)])
def test_dense_int8_weight_only(dev, policy, M, K, N):
    layer = build_dense(dev, K, N, policy, seed=5)
    kernel_f = layer._kernel.value.cpu()
    bias_f = layer.bias.value.cpu()
    cd = TORCH[layer.compute_dtype]
    x = torch.randn(M, K, generator=torch.Generator().manual_seed(6))
    layer.quantize("int8", config=ka.Int8QuantizationConfig(activation_quantizer=None))
    assert layer.inputs_quantizer is None
    qk, ks = ref.dense_quantize_int8(kernel_f)
    assert torch.equal(layer._kernel.value.cpu(), qk)
    y = layer(x)
    want = ref.dense_int8_call(x.to(cd), qk, ks, bias_f, compute_dtype=cd, quantize_inputs=False)
    assert y.dtype == cd and tuple(y.shape) == (M, N)
    assert max_rel_err(y, want) <= RTOL[cd]
    # and against the exact value: float64 matmul of the same operands
    exact = (x.to(cd).double() @ qk.double()) / ks.to(cd).double() + bias_f.to(cd).double()
    assert max_rel_err(y, exact) <= RTOL[cd]


@pytest.mark.parametrize("policy", ["float32", "mixed_bfloat16"])
@pytest.mark.parametrize("M,K,N", [(1, 1024, 512), (16, 512, 384), (7, 300, 64), (40, 256, 96),
                                   (300, 512, 256)])
def test_dense_int4_activation_quantized(dev, policy, M, K, N):
    layer = build_dense(dev, K, N, policy, seed=7)
    kernel_f = layer._kernel.value.cpu()
    bias_f = layer.bias.value.cpu()
    cd = TORCH[layer.compute_dtype]
    x = torch.randn(M, K, generator=torch.Generator().manual_seed(8))
    config = ka.Int4QuantizationConfig(block_size=None, activation_quantizer=ka.quantizers.AbsMaxQuantizer())
    layer.quantize("int4", config=config)
    assert layer.inputs_quantizer is not None
    qk = ref.dense_quantize_int4(kernel_f, None)
    assert torch.equal(layer._kernel.value.cpu(), qk["kernel"])
    y = layer(x)
    want, inter = ref.dense_int4_call(
        x.to(cd), qk["kernel"], qk["kernel_scale"], N, block_size=None, bias=bias_f,
        compute_dtype=cd, quantize_inputs=True, return_intermediates=True)
    assert inter["acc"].dtype == torch.int32
    # integer accumulation and the exact epilogue: bit-identical to the reference chain
    assert y.dtype == cd and torch.equal(bits(y.cpu()), bits(want))


@pytest.mark.parametrize("equation,output_shape,input_shape", EQUATIONS)
@pytest.mark.parametrize("policy", ["float32", "mixed_bfloat16"])
def test_einsum_dense_int8_weight_only(dev, equation, output_shape, input_shape, policy):
    g = torch.Generator().manual_seed(2024)
    layer = EinsumDense(equation, output_shape, dtype=policy, device=dev,
                        kernel_initializer=lambda s, d: (torch.rand(s, generator=g) - 0.5).to(d))
    layer.build(input_shape)
    cd = TORCH[layer.compute_dtype]
    kernel_f = layer._kernel.value.cpu()
    x = torch.rand(input_shape, generator=g)
    layer.quantize("int8", config=ka.Int8QuantizationConfig(activation_quantizer=None))
    assert layer.inputs_quantizer is None
    qk, ks, _ = ref.einsum_dense_quantize_int8(kernel_f, equation, len(input_shape))
    y = layer(x)
    want = ref.einsum_dense_int8_weight_only_call(x.to(cd), qk, ks, equation, compute_dtype=cd)
    assert tuple(y.shape) == tuple(want.shape) and y.dtype == cd
    # the reference rounds every de-quantised weight to the compute dtype, the kernel divides
    # once at the end: same quantity, float tolerance
    assert max_rel_err(y, want) <= RTOL[cd]


@pytest.mark.parametrize("equation,output_shape,input_shape", [EQUATIONS[0], EQUATIONS[2], EQUATIONS[4], EQUATIONS[5]])
@pytest.mark.parametrize("policy", ["float32", "mixed_bfloat16"])
def test_einsum_dense_int4_activation_quantized(dev, equation, output_shape, input_shape, policy):
    g = torch.Generator().manual_seed(2025)
    layer = EinsumDense(equation, output_shape, dtype=policy, device=dev,
                        kernel_initializer=lambda s, d: (torch.rand(s, generator=g) - 0.5).to(d))
    layer.build(input_shape)
    cd = TORCH[layer.compute_dtype]
    kernel_f = layer._kernel.value.cpu()
    x = torch.rand(input_shape, generator=g)
    config = ka.Int4QuantizationConfig(block_size=None, activation_quantizer=ka.quantizers.AbsMaxQuantizer())
    layer.quantize("int4", config=config)
    assert layer.inputs_quantizer is not None
    qk = ref.einsum_dense_quantize_int4(kernel_f, equation, len(input_shape), None)
    assert torch.equal(layer._kernel.value.cpu(), qk["kernel"])
    y = layer(x)
    want = ref.einsum_dense_int4_activation_quantized_call(x.to(cd), qk, equation, compute_dtype=cd)
    assert tuple(y.shape) == tuple(want.shape) and y.dtype == cd
    assert max_rel_err(y, want) <= RTOL[cd]


@pytest.mark.parametrize("mode,equation,output_shape,input_shape,threshold", [
    # einsum_dense_test.py:629-677, the reference's own cases and thresholds
    ("int8", "btnh,nhd->btd", (None, 8), (1, 2, 2, 4), 1e-3),
    ("int8", "btd,ndh->btnh", (None, 2, 8), (1, 2, 4), 1e-3),
    ("int8", "btd,df->btf", (None, 4), (1, 2, 4), 1e-3),
    ("int4", "btnh,nhd->btd", (None, 8), (1, 2, 2, 4), 4e-3),
    ("int4", "btd,ndh->btnh", (None, 2, 8), (1, 2, 4), 4e-3),
    ("int4", "btd,df->btf", (None, 4), (1, 2, 4), 4e-3),
])
def test_quantize_with_specific_equations(dev, mode, equation, output_shape, input_shape, threshold):
    # einsum_dense_test.py:678-697: quantize a float layer, the output stays close (MSE)
    g = torch.Generator().manual_seed(1337)
    fan = 1
    for d in input_shape[1:]:
        fan *= d

    def glorot(shape, dtype):
        limit = (6.0 / (fan + shape[-1])) ** 0.5
        return ((torch.rand(shape, generator=g) * 2 - 1) * limit).to(dtype)

    layer = EinsumDense(equation, output_shape, device=dev, kernel_initializer=glorot)
    layer.build(input_shape)
    x = torch.rand(input_shape, generator=g)
    y_float = layer(x)
    layer.quantize(mode)
    y_quantized = layer(x)
    mse = (y_float.float() - y_quantized.float()).pow(2).mean().item()
    assert mse < threshold


@pytest.mark.parametrize("rows", [1, 8, 16, 100])
@pytest.mark.parametrize("block_size", [128, None])
def test_call_together_matches_separate_calls(dev, rows, block_size):
    # attention-style projections (EinsumDense) and MLP-style ones (Dense, one with a bias and
    # an activation) on one input: call_together returns what the layers return one by one
    g = torch.Generator().manual_seed(11)
    init = lambda s, d: (torch.rand(s, generator=g) - 0.5).to(d)
    cfg = ka.Int4QuantizationConfig(block_size=block_size)
    proj = [EinsumDense("btd,dnh->btnh", (None, 4, 64), dtype="mixed_bfloat16", device=dev,
                        kernel_initializer=init) for _ in range(3)]
    x = torch.randn((1, rows, 256), generator=g)
    for layer in proj:
        layer.build((1, rows, 256))
        layer.quantize("int4", config=cfg)
    want = [layer(x) for layer in proj]
    got = ka.layers.call_together(proj, x)
    for a, b in zip(got, want):
        assert a.shape == b.shape and a.dtype == b.dtype
        assert max_rel_err(a, b) <= RTOL[torch.bfloat16] / 2  # another order of the fp32 sums
    mlp = [Dense(512, use_bias=False, dtype="mixed_bfloat16", device=dev, kernel_initializer=init),
           Dense(512, use_bias=True, activation="relu", dtype="mixed_bfloat16", device=dev,
                 kernel_initializer=init)]
    x2 = torch.randn((rows, 256), generator=g)
    for layer in mlp:
        layer.build((rows, 256))
        layer.quantize("int4", config=cfg)
    want = [layer(x2) for layer in mlp]
    got = ka.layers.call_together(mlp, x2)
    for a, b in zip(got, want):
        assert a.shape == b.shape and a.dtype == b.dtype
        assert max_rel_err(a, b) <= RTOL[torch.bfloat16] / 2
    # a layer that is not weight-only int4 sends the whole group down the one-by-one road
    other = Dense(512, dtype="mixed_bfloat16", device=dev, kernel_initializer=init)
    other.build((rows, 256))
    other.quantize("int8")
    want = [layer(x2) for layer in (mlp[0], other)]
    got = ka.layers.call_together((mlp[0], other), x2)
    for a, b in zip(got, want):
        assert torch.equal(a, b)


@pytest.mark.parametrize("rows", [1, 8, 40])
@pytest.mark.parametrize("dtype", ["mixed_bfloat16", "float32"])
def test_call_together_int8_quantises_shared_rows_once(dev, rows, dtype, monkeypatch):
    # int8 layers on one input: the rows are quantised by one call, the results are the bits
    # of the separate calls; a layer with another value range quantises for itself
    g = torch.Generator().manual_seed(12)
    init = lambda s, d: (torch.rand(s, generator=g) - 0.5).to(d)
    proj = [EinsumDense("btd,dnh->btnh", (None, 4, 64), dtype=dtype, device=dev, kernel_initializer=init)
            for _ in range(3)]
    mlp = [Dense(512, use_bias=(j == 1), dtype=dtype, device=dev, kernel_initializer=init) for j in range(2)]
    x = torch.randn((1, rows, 256), generator=g)
    for layer in proj + mlp:
        layer.build((1, rows, 256))
        layer.quantize("int8")
    calls = []
    real = kq.abs_max_quantize
    monkeypatch.setattr(kq, "abs_max_quantize", lambda *a, **k: (calls.append(1), real(*a, **k))[1])
    want = [layer(x) for layer in proj + mlp]
    assert len(calls) == 5
    del calls[:]
    got = ka.layers.call_together(proj + mlp, x)
    assert len(calls) == 1
    for a, b in zip(got, want):
        assert a.shape == b.shape and torch.equal(a, b)
    # outside call_together nothing is remembered
    del calls[:]
    proj[0](x)
    proj[1](x)
    assert len(calls) == 2
    # another quantizer configuration is not served from the shared rows
    mlp[1].inputs_quantizer = kq.AbsMaxQuantizer(axis=-1, value_range=(-100, 100))
    del calls[:]
    want = [mlp[0](x), mlp[1](x)]
    del calls[:]
    got = ka.layers.call_together(mlp, x)
    assert len(calls) == 2
    for a, b in zip(got, want):
        assert torch.equal(a, b)


@pytest.mark.parametrize("mode", ["int8", "int4"])
@pytest.mark.parametrize("dtype", ["mixed_bfloat16", "float32"])
def test_call_add_is_the_separate_add(dev, mode, dtype):
    # residual + layer(x): one row goes through the matmul's bias slot, up to 16 rows of a
    # weight-only int4 layer through the decode kernel's addend (same bits as the add after
    # it); more rows, int8 beyond one row, a layer with a bias or an activation take the plain sum
    g = torch.Generator().manual_seed(13)
    init = lambda s, d: (torch.rand(s, generator=g) - 0.5).to(d)
    cd = torch.bfloat16 if dtype == "mixed_bfloat16" else torch.float32
    out = EinsumDense("btnh,nhd->btd", (None, 256), dtype=dtype, device=dev, kernel_initializer=init)
    down = Dense(256, use_bias=False, dtype=dtype, device=dev, kernel_initializer=init)
    biased = Dense(256, use_bias=True, dtype=dtype, device=dev, kernel_initializer=init,
                   bias_initializer=init)
    out.build((1, 1, 4, 64))
    for layer in (down, biased):
        layer.build((1, 1, 512))
    for layer in (out, down, biased):
        layer.quantize(mode)
    for rows in (1, 3, 8, 16, 17, 40):
        res = torch.randn((1, rows, 256), generator=g).to(cd).to(dev)
        a = torch.randn((1, rows, 4, 64), generator=g).to(cd).to(dev)
        h = torch.randn((1, rows, 512), generator=g).to(cd).to(dev)
        for layer, x in ((out, a), (down, h), (biased, h)):
            want = res + layer(x)
            got = ka.layers.call_add(layer, x, res)
            assert got.shape == want.shape and got.dtype == want.dtype
            assert torch.equal(got, want), (rows, layer.name)
            assert getattr(layer, "_row_bias", None) is None
    # the lent row is gone afterwards: the layer alone gives its own result again
    h = torch.randn((1, 1, 512), generator=g).to(cd).to(dev)
    plain = down(h)
    ka.layers.call_add(down, h, torch.ones((1, 1, 256), dtype=cd, device=dev))
    assert torch.equal(down(h), plain)


@pytest.mark.parametrize("equation,output_shape,input_shape,bias_axes", GENERAL[:5])
@pytest.mark.parametrize("policy", ["float32", "mixed_bfloat16"])
def test_einsum_dense_int4_activation_quantized_general_equations(dev, equation, output_shape, input_shape,
                                                                  bias_axes, policy):
    # equations outside the [M, K] x [K, N] view (labels shared by all three operands, no summed
    # label, a label only the input carries) with a per-channel int4 kernel AND an activation
    # quantizer: the reference's torch branch (einsum_dense.py:1163-1184) -- rows quantised over the
    # labels the output lacks, cast back, float einsum against the de-quantised kernel, division by
    # the adjusted input scale
    g = torch.Generator().manual_seed(97)
    layer = EinsumDense(equation, output_shape, bias_axes=bias_axes, dtype=policy, device=dev,
                        kernel_initializer=lambda s, d: (torch.rand(s, generator=g) - 0.5).to(d),
                        bias_initializer=lambda s, d: torch.randn(s, generator=g).to(d))
    layer.build(input_shape)
    cd = TORCH[layer.compute_dtype]
    kernel_f = layer._kernel.value.cpu()
    bias_f = layer.bias.value.cpu() if layer.bias is not None else None
    x = torch.rand(input_shape, generator=g) - 0.3
    config = ka.Int4QuantizationConfig(block_size=None, activation_quantizer=ka.quantizers.AbsMaxQuantizer())
    layer.quantize("int4", config=config)
    assert layer.inputs_quantizer is not None
    qk = ref.einsum_dense_quantize_int4(kernel_f, equation, len(input_shape), None)
    assert torch.equal(layer._kernel.value.cpu(), qk["kernel"])
    y = layer(x)
    want = ref.einsum_dense_int4_activation_quantized_call(x.to(cd), qk, equation, bias=bias_f, compute_dtype=cd)
    assert tuple(y.shape) == tuple(want.shape) and y.dtype == cd
    assert max_rel_err(y, want) <= RTOL[cd]


@pytest.mark.parametrize("kind", ["dense", "einsum", "einsum_non_leading"])
def test_grouped_int4_ignores_an_activation_quantizer(dev, kind):
    # the reference's sub-channel branches never read `inputs_quantizer` (dense.py:1040-1084,
    # einsum_dense.py:1188-1261): a grouped int4 layer configured with one is the weight-only layer
    g = torch.Generator().manual_seed(96)
    init = lambda s, d: (torch.rand(s, generator=g) - 0.5).to(d)
    if kind == "dense":
        layer = Dense(96, dtype="mixed_bfloat16", device=dev, kernel_initializer=init, use_bias=False)
        shape, eq = (5, 256), None
    elif kind == "einsum":
        layer = EinsumDense("btd,dnh->btnh", (None, 4, 24), dtype="mixed_bfloat16", device=dev, kernel_initializer=init)
        shape, eq = (2, 3, 256), "btd,dnh->btnh"
    else:
        layer = EinsumDense("btd,ndh->btnh", (None, 4, 24), dtype="mixed_bfloat16", device=dev, kernel_initializer=init)
        shape, eq = (2, 3, 256), "btd,ndh->btnh"
    layer.build(shape)
    kernel_f = layer._kernel.value.cpu()
    x = torch.rand(shape, generator=g) - 0.5
    # (Int4QuantizationConfig refuses the combination, as the reference's does, so the quantizer is
    # attached by hand -- what a subclass or a hand-edited layer could carry)
    layer.quantize("int4", config=ka.Int4QuantizationConfig(block_size=128))
    layer.inputs_quantizer = ka.quantizers.AbsMaxQuantizer()
    y = layer(x)
    cd = torch.bfloat16
    if eq is None:
        q4 = ref.dense_quantize_int4(kernel_f, 128)
        want = ref.dense_int4_call(x.to(cd), q4["kernel"], q4["kernel_scale"], 96, kernel_zero=q4["kernel_zero"],
                                   g_idx=q4["g_idx"], block_size=128, compute_dtype=cd)
    else:
        qk = ref.einsum_dense_quantize_int4(kernel_f, eq, 3, 128)
        want = ref.einsum_dense_int4_call(x.to(cd), qk, eq, compute_dtype=cd, block_size=128)
    assert tuple(y.shape) == tuple(want.shape) and y.dtype == cd
    assert max_rel_err(y, want) <= RTOL[cd]


@pytest.mark.parametrize("mode", ["int8", "int4"])
def test_derived_copy_keeps_its_address_when_the_kernel_is_assigned(dev, mode):
    # the strip-linear copy is rebuilt in place when the kernel variable is assigned: a captured
    # graph that holds the copy's address then reads the new values, not freed memory
    layer = build_dense(dev, 4096, 4096, "mixed_bfloat16", seed=11, use_bias=False)
    other = build_dense(dev, 4096, 4096, "mixed_bfloat16", seed=12, use_bias=False)
    layer.quantize(mode)
    other.quantize(mode)
    x = torch.randn(2, 4096, generator=torch.Generator().manual_seed(13)).to(torch.bfloat16).to(dev)
    y0 = layer(x)
    key = "w8s" if mode == "int8" else "w4s"
    copy0 = layer._cache[key][2]
    address = copy0.data_ptr()
    for name in ("_kernel", "kernel_scale") + (("kernel_zero",) if mode == "int4" else ()):
        getattr(layer, name).assign(getattr(other, name).value)
    y1 = layer(x)
    assert layer._cache[key][2].data_ptr() == address
    assert torch.equal(bits(y1.cpu()), bits(other(x).cpu()))
    assert not torch.equal(bits(y1.cpu()), bits(y0.cpu()))
