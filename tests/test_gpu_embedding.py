"""GPU parity: quantized Embedding lookup, ReversibleEmbedding reverse projection and the
[N, K]-layout int8 matmul, through the C ABI, against the CPU oracle."""

import pytest
import torch

from keras_amd import ops as kops
from keras_amd.layers import Embedding, ReversibleEmbedding
from keras_amd.quantization_config import Int4QuantizationConfig
from oracle import keras_cpu_path as ref
from tests.helpers import RTOL, c_gemm_i8, max_rel_err

pytestmark = pytest.mark.gpu

TORCH = {"float32": torch.float32, "bfloat16": torch.bfloat16}


def bits(t):
    return t.view(torch.int16) if t.dtype == torch.bfloat16 else t.view(torch.int32)


def table(V, D, seed=0):
    g = torch.Generator().manual_seed(seed)
    return (torch.rand(V, D, generator=g) * 2.0 - 1.0) * 0.05


def some_ids(V, shape, seed, dtype=torch.int64):
    ids = torch.randint(-V, V, shape, generator=torch.Generator().manual_seed(seed))
    flat = ids.view(-1)
    flat[0], flat[-1] = V - 1, -V  # both ends of the valid range
    return ids.to(dtype)


# ---- k3q_embedding_lookup ----------------------------------------------------------------
@pytest.mark.parametrize("scale_dtype,out_dtype", [(torch.float32, torch.float32),
                                                   (torch.bfloat16, torch.bfloat16),
                                                   (torch.bfloat16, torch.float32)])
@pytest.mark.parametrize("V,D", [(1000, 4096), (37, 64), (50, 48), (9, 33), (5, 1)])
@pytest.mark.parametrize("ids_dtype", [torch.int32, torch.int64])
def test_lookup_int8(dev, scale_dtype, out_dtype, V, D, ids_dtype):
    q, s = ref.embedding_quantize_int8(table(V, D))
    s = s.to(scale_dtype)
    ids = some_ids(V, (3, 17), seed=1, dtype=ids_dtype)
    cd = "bfloat16" if out_dtype == torch.bfloat16 or scale_dtype == torch.bfloat16 else "float32"
    if scale_dtype == torch.bfloat16 and out_dtype == torch.float32:
        cd = "float32"  # float32 compute with a bfloat16 scale variable
    want = ref.embedding_int8_call(ids, q, s, compute_dtype=cd)
    assert want.dtype == out_dtype
    got = kops.embedding_lookup(ids.to(dev), q.to(dev), s.to(dev), D, bits=8, out_dtype=out_dtype)
    assert got.dtype == out_dtype and tuple(got.shape) == (3, 17, D)
    assert torch.equal(bits(got.cpu()), bits(want))


@pytest.mark.parametrize("scale_dtype,out_dtype", [(torch.float32, torch.float32),
                                                   (torch.bfloat16, torch.bfloat16)])
@pytest.mark.parametrize("V,D,block", [(500, 4096, 128), (500, 4096, None), (40, 256, 64),
                                       (40, 256, -1), (11, 96, 32), (11, 100, 20), (7, 33, 8),
                                       (7, 33, None), (10, 16, 4)])
def test_lookup_int4(dev, scale_dtype, out_dtype, V, D, block):
    qd = ref.embedding_quantize_int4(table(V, D, seed=2), block_size=block)
    s = qd["embeddings_scale"].to(scale_dtype)
    ids = some_ids(V, (29,), seed=3)
    cd = "bfloat16" if out_dtype == torch.bfloat16 else "float32"
    want = ref.embedding_int4_call(ids, qd["embeddings"], s, D, embeddings_zero=qd["embeddings_zero"],
                                   g_idx=qd["g_idx"], block_size=block, compute_dtype=cd)
    grouped = block is not None and block > 0
    got = kops.embedding_lookup(
        ids.to(dev), qd["embeddings"].to(dev), s.to(dev), D, bits=4,
        zero=qd["embeddings_zero"].to(dev) if grouped else None,
        block_size=block if grouped else None, out_dtype=out_dtype)
    assert torch.equal(bits(got.cpu()), bits(want))


def test_lookup_out_of_range(dev):
    q, s = ref.embedding_quantize_int8(table(10, 32))
    qd, sd = q.to(dev), s.to(dev)
    for bad in (10, -11, 1 << 40):
        ids = torch.tensor([1, bad, 2], device=dev)
        with pytest.raises(IndexError):
            kops.embedding_lookup(ids, qd, sd, 32)
        out = kops.embedding_lookup(ids, qd, sd, 32, check_ids=False)
        want = ref.embedding_int8_call(torch.tensor([1, 2]), q, s)
        assert torch.equal(out[[0, 2]].cpu(), want)
        assert torch.count_nonzero(out[1]).item() == 0
    assert kops.embedding_lookup(torch.zeros((0,), dtype=torch.int64, device=dev), qd, sd, 32).shape == (0, 32)
    with pytest.raises(RuntimeError):
        kops.embedding_lookup(torch.tensor([1]), q, s, 32)  # host tensors: no CPU path


# ---- int8 matmul with an [N, K] kernel -----------------------------------------------------
@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("M,K,N", [(1, 4096, 32000), (8, 4096, 32000), (16, 256, 1000),
                                   (5, 4096, 64), (3, 64, 7), (17, 512, 333), (64, 1024, 2048),
                                   (40, 128, 50), (300, 256, 1000), (65, 4096, 512)])
def test_int8_matmul_nk(dev, out_dtype, M, K, N):
    g = torch.Generator().manual_seed(M * 7 + N)
    a = torch.randint(-127, 128, (M, K), generator=g, dtype=torch.int8)
    b = torch.randint(-127, 128, (N, K), generator=g, dtype=torch.int8)
    sa = (torch.rand(M, generator=g) * 50 + 1).to(out_dtype)
    sb = (torch.rand(N, generator=g) * 50 + 1).to(out_dtype)
    y, acc = kops.int8_matmul_nk(a.to(dev), b.to(dev), a_scale=sa.to(dev), kernel_scale=sb.to(dev),
                                 out_dtype=out_dtype, exact_epilogue=True, want_acc=True)
    want_acc = c_gemm_i8(a, b.t().contiguous())
    assert torch.equal(acc.cpu(), want_acc)
    want = torch.divide(want_acc.to(out_dtype), torch.multiply(sa.unsqueeze(-1), sb))
    assert torch.equal(bits(y.cpu()), bits(want))


def test_int8_matmul_nk_round_acc(dev):
    g = torch.Generator().manual_seed(5)
    for M, K, N in [(4, 4096, 1000), (200, 256, 512)]:
        a = torch.randint(-127, 128, (M, K), generator=g, dtype=torch.int8)
        b = torch.randint(-127, 128, (N, K), generator=g, dtype=torch.int8)
        sa = (torch.rand(M, generator=g) * 50 + 1).to(torch.bfloat16).float()
        sb = torch.rand(N, generator=g) * 50 + 1
        y = kops.int8_matmul_nk(a.to(dev), b.to(dev), a_scale=sa.to(dev), kernel_scale=sb.to(dev),
                                out_dtype=torch.float32, exact_epilogue=True, round_acc_bf16=True)
        acc = c_gemm_i8(a, b.t().contiguous())
        want = torch.divide(acc.to(torch.bfloat16), torch.multiply(sa.unsqueeze(-1), sb))
        assert want.dtype == torch.float32
        assert torch.equal(y.cpu(), want)


# ---- layers -----------------------------------------------------------------------------------
def build_embedding(cls, dev, V, D, policy, seed, **kw):
    g = torch.Generator().manual_seed(seed)
    layer = cls(V, D, dtype=policy, device=dev,
                embeddings_initializer=lambda s, d: ((torch.rand(s, generator=g) * 2 - 1) * 0.05).to(d), **kw)
    layer.build()
    return layer


@pytest.mark.parametrize("policy", ["float32", "mixed_bfloat16", "bfloat16"])
@pytest.mark.parametrize("V,D", [(10, 16), (100, 256), (1000, 4096)])
def test_embedding_int8_layer(dev, policy, V, D):
    layer = build_embedding(Embedding, dev, V, D, policy, seed=0)
    t = layer._embeddings.value.cpu()
    ids = torch.randint(0, V - 1, (64, 3), generator=torch.Generator().manual_seed(1))
    y_float = layer(ids)
    layer.quantize("int8")
    assert layer.dtype_policy.name == f"int8_from_{policy}"
    assert layer._embeddings.dtype == "int8" and layer.embeddings_scale.dtype == layer.variable_dtype
    q, s = ref.embedding_quantize_int8(t)
    assert torch.equal(layer._embeddings.value.cpu(), q)
    assert torch.equal(bits(layer.embeddings_scale.value.cpu()), bits(s))
    y = layer(ids)
    want = ref.embedding_int8_call(ids, q, s, compute_dtype=layer.compute_dtype)
    assert y.dtype == want.dtype and torch.equal(bits(y.cpu()), bits(want))
    # embedding_test.py:364-394
    assert (y_float.float().cpu() - y.float().cpu()).pow(2).mean().item() < 1e-3
    with pytest.raises(ValueError):
        layer.quantize("int8")
    store = {}
    layer.save_own_variables(store)
    assert sorted(store) == ["0", "1"]
    clone = Embedding(V, D, dtype=layer.dtype_policy.name, device=dev)
    clone.build()
    clone.load_own_variables(store)
    assert torch.equal(bits(clone(ids).cpu()), bits(want))


@pytest.mark.parametrize("mode,block_size", [("int8", None), ("int4", None), ("int4", 64)])
@pytest.mark.parametrize("policy", ["float32", "bfloat16"])
def test_embedding_lora_on_quantized_layer_and_merge_on_save(dev, mode, block_size, policy):
    # keras/src/layers/core/embedding.py:214-261 (enable_lora), :533-540 / :575-582 (a lookup adds the
    # rows of the update), :683-818 (the update is merged into what is saved), :355-361 (zeroed on load)
    g = torch.Generator().manual_seed(31)
    V, D, rank, alpha = 200, 256, 4, 8
    layer = build_embedding(Embedding, dev, V, D, policy, seed=6)
    t = layer._embeddings.value.cpu()
    if mode == "int8":
        layer.quantize("int8")
        q, s = ref.embedding_quantize_int8(t)
        zero = g_idx = None
    else:
        layer.quantize("int4", config=Int4QuantizationConfig(block_size=block_size))
        qd = ref.embedding_quantize_int4(t, block_size=block_size)
        q, s, zero, g_idx = qd["embeddings"], qd["embeddings_scale"], qd["embeddings_zero"], qd["g_idx"]
    layer.enable_lora(rank, lora_alpha=alpha)
    with pytest.raises(ValueError):
        layer.enable_lora(rank)
    assert tuple(layer.lora_embeddings_a.shape) == (V, rank) and tuple(layer.lora_embeddings_b.shape) == (rank, D)
    a = torch.randn(V, rank, generator=g) * 0.02
    b = torch.randn(rank, D, generator=g) * 0.02
    layer.lora_embeddings_a.assign(a)
    layer.lora_embeddings_b.assign(b)
    ids = torch.randint(0, V, (5, 7), generator=g)
    y = layer(ids)
    cd = layer.compute_dtype
    if mode == "int8":
        base = ref.embedding_int8_call(ids, q, s, compute_dtype=cd)
    else:
        base = ref.embedding_int4_call(ids, q, s, D, embeddings_zero=zero, g_idx=g_idx, block_size=block_size,
                                       compute_dtype=cd)
    want = (base + (alpha / rank) * (a[ids] @ b)).to(y.dtype)
    assert y.dtype == want.dtype and (y.float().cpu() - want.float()).abs().max().item() <= 1e-2 * want.abs().max().item()
    merged = ref.embedding_merged_lora_table(mode, q, s, a, b, alpha, rank, compute_dtype=cd, embeddings_zero=zero,
                                             g_idx=g_idx, block_size=block_size, orig_output_dim=D)
    store = {}
    layer.save_own_variables(store)
    assert torch.equal(store["0"].cpu(), merged[0])
    assert torch.equal(bits(store["1"].cpu()), bits(merged[1]))
    if block_size:
        assert torch.equal(store["2"].cpu(), merged[2])
    assert not torch.equal(store["0"].cpu(), q)
    plain = Embedding(V, D, dtype=layer.dtype_policy.name, device=dev)
    plain.build()
    plain.load_own_variables(store)
    y2 = plain(ids)
    assert (y2.float().cpu() - y.float().cpu()).abs().max().item() <= (0.02 if mode == "int8" else 0.2) * y.float().abs().max().item()
    layer.load_own_variables(store)
    assert float(layer.lora_embeddings_a.value.abs().max()) == 0.0
    assert torch.equal(bits(layer(ids).cpu()), bits(y2.cpu()))
    assert layer.get_config()["lora_rank"] == rank


@pytest.mark.parametrize("policy", ["float32", "bfloat16"])
@pytest.mark.parametrize("block_size", [128, 64, 8, None, -1])
@pytest.mark.parametrize("V,D", [(10, 16), (100, 256), (300, 4096)])
def test_embedding_int4_layer(dev, policy, block_size, V, D):
    layer = build_embedding(Embedding, dev, V, D, policy, seed=2)
    t = layer._embeddings.value.cpu()
    ids = torch.randint(0, V, (4, 8), generator=torch.Generator().manual_seed(3))
    y_float = layer(ids)
    layer.quantize("int4", config=Int4QuantizationConfig(block_size=block_size))
    assert layer._int4_block_size == block_size
    bs_name = -1 if block_size is None else block_size
    assert layer.dtype_policy.name == f"int4/{bs_name}_from_{policy}"
    qd = ref.embedding_quantize_int4(t, block_size=block_size)
    assert torch.equal(layer._embeddings.value.cpu(), qd["embeddings"])
    assert torch.equal(bits(layer.embeddings_scale.value.cpu()), bits(qd["embeddings_scale"]))
    grouped = block_size is not None and block_size > 0
    if grouped:
        assert torch.equal(layer.embeddings_zero.value.cpu(), qd["embeddings_zero"])
        assert torch.equal(layer.g_idx.value.cpu(), qd["g_idx"]) and layer.g_idx.dtype == "float32"
    else:
        assert not hasattr(layer, "g_idx") and not hasattr(layer, "embeddings_zero")
    assert torch.equal(layer.embeddings.cpu(), qd["unpacked"])
    y = layer(ids)
    want = ref.embedding_int4_call(ids, qd["embeddings"], qd["embeddings_scale"], D,
                                   embeddings_zero=qd["embeddings_zero"], g_idx=qd["g_idx"],
                                   block_size=block_size, compute_dtype=layer.compute_dtype)
    assert y.dtype == want.dtype and torch.equal(bits(y.cpu()), bits(want))
    assert (y_float.float().cpu() - y.float().cpu()).pow(2).mean().item() < 1e-3
    store = {}
    layer.save_own_variables(store)
    assert len(store) == (4 if grouped else 2)


@pytest.mark.parametrize("policy", ["float32", "mixed_bfloat16", "bfloat16"])
@pytest.mark.parametrize("M,V,D", [(1, 32000, 4096), (8, 32000, 4096), (16, 1000, 256),
                                   (300, 1000, 256), (5, 77, 64)])
def test_reversible_embedding_int8_tied(dev, policy, M, V, D):
    layer = build_embedding(ReversibleEmbedding, dev, V, D, policy, seed=4)
    t = layer._embeddings.value.cpu()
    cd = TORCH[layer.compute_dtype]
    x = torch.randn(M, D, generator=torch.Generator().manual_seed(5))
    y_float = layer(x, reverse=True)
    layer.quantize("int8")
    q, s = ref.embedding_quantize_int8(t)
    assert torch.equal(layer._embeddings.value.cpu(), q)
    layer.exact_epilogue = True
    y = layer(x, reverse=True)
    want = ref.reversible_embedding_int8_reverse(x.to(cd), q, s.to(TORCH[layer.variable_dtype]),
                                                 compute_dtype=cd)
    assert y.dtype == want.dtype and tuple(y.shape) == (M, V)
    assert torch.equal(bits(y.cpu()), bits(want))
    # decode sizes of a wide bfloat16 table stream its strip-linear copy (same bits); everything
    # else reads the table in place
    assert ("w8s" in layer._cache) == (policy == "bfloat16" and M <= 16 and V == 32000)
    layer.exact_epilogue = False
    assert max_rel_err(layer(x, reverse=True), want) <= RTOL[cd]
    err = (y_float.float().cpu() - y.float().cpu()).abs().max().item()
    assert err <= 0.05 * y_float.float().abs().max().item() + 1e-3
    # the forward lookup of the same layer still works
    ids = torch.randint(0, V, (2, 5), generator=torch.Generator().manual_seed(6))
    assert torch.equal(bits(layer(ids).cpu()),
                       bits(ref.embedding_int8_call(ids, q, s, compute_dtype=layer.compute_dtype)))


@pytest.mark.parametrize("M", [4, 100])
def test_reversible_embedding_int8_untied_and_soft_cap(dev, M):
    V, D = 512, 128
    layer = build_embedding(ReversibleEmbedding, dev, V, D, "float32", seed=7, tie_weights=False,
                            logit_soft_cap=0.3)
    rt = layer.reverse_embeddings.value.cpu()
    x = torch.randn(M, D, generator=torch.Generator().manual_seed(8))
    layer.quantize("int8")
    assert layer.reverse_embeddings.dtype == "int8" and layer.reverse_embeddings.shape == (D, V)
    rq, rs = ref.dense_quantize_int8(rt)  # AbsMaxQuantizer(axis=0) on [D, V], as Dense does
    assert torch.equal(layer.reverse_embeddings.value.cpu(), rq)
    layer.exact_epilogue = True
    y = layer(x, reverse=True)
    logits = ref.dense_int8_call(x, rq, rs)
    want = torch.multiply(torch.tanh(torch.divide(logits, 0.3)), 0.3)
    assert torch.allclose(y.cpu(), want, rtol=1e-6, atol=1e-7)
    store = {}
    layer.save_own_variables(store)
    assert len(store) == 4


@pytest.mark.parametrize("x_dtype,scale_dtype", [(torch.float32, torch.float32),
                                                 (torch.bfloat16, torch.bfloat16),
                                                 (torch.bfloat16, torch.float32)])
@pytest.mark.parametrize("M,V,D,block", [(1, 4000, 4096, 128), (8, 4000, 4096, None), (3, 500, 256, 128),
                                         (11, 77, 384, 128), (2, 64, 512, 256), (4, 33, 256, -1),
                                         (5, 40, 96, 32), (2, 21, 100, 20), (3, 17, 33, None)])
def test_int4_matmul_nk(dev, x_dtype, scale_dtype, M, V, D, block):
    qd = ref.embedding_quantize_int4(table(V, D, seed=11), block_size=block)
    s = qd["embeddings_scale"].to(scale_dtype)
    x = torch.randn(M, D, generator=torch.Generator().manual_seed(12)).to(x_dtype)
    want = ref.reversible_embedding_int4_reverse(
        x, qd["embeddings"], s, D, embeddings_zero=qd["embeddings_zero"], g_idx=qd["g_idx"],
        block_size=block, compute_dtype=x_dtype)
    grouped = block is not None and block > 0
    got = kops.int4_matmul_nk(x.to(dev), qd["embeddings"].to(dev), s.to(dev),
                              zero=qd["embeddings_zero"].to(dev) if grouped else None,
                              block_size=block if grouped else None)
    assert got.dtype == want.dtype and tuple(got.shape) == (M, V)
    # float64 value of the same product: both must sit within the dtype's tolerance of it
    w = qd["unpacked"].double()
    if grouped:
        gi = qd["g_idx"].long()
        w = (w - qd["embeddings_zero"].double()[:, gi]) * s.double()[:, gi]
        exact = x.double() @ w.T
    else:
        exact = (x.double() @ w.T) / s.double()
    tol = RTOL[torch.bfloat16 if x_dtype == torch.bfloat16 else torch.float32]
    assert max_rel_err(got, exact) <= tol
    assert max_rel_err(got, want) <= tol


@pytest.mark.parametrize("M", [1, 8, 16])
@pytest.mark.parametrize("block_size", [128, None])
def test_reversible_embedding_int4_tied_decode_sizes_take_the_strip_copy(dev, M, block_size):
    """A tied table wide enough for the Dense decode kernel is re-laid once as that kernel's
    strip-linear copy; more rows, or other dtypes, keep reading the table in place."""
    V, D = 3200, 4096
    layer = build_embedding(ReversibleEmbedding, dev, V, D, "bfloat16", seed=21)
    t = layer._embeddings.value.cpu()
    layer.quantize("int4", config=Int4QuantizationConfig(block_size=block_size))
    qd = ref.embedding_quantize_int4(t.float(), block_size=block_size)
    x = torch.randn(M, D, generator=torch.Generator().manual_seed(22))
    y = layer(x, reverse=True)
    assert "w4s" in layer._cache and ("w4s_params" in layer._cache) == (block_size is not None)
    want = ref.reversible_embedding_int4_reverse(
        x.to(torch.bfloat16), qd["embeddings"], qd["embeddings_scale"].to(torch.bfloat16), D,
        embeddings_zero=qd["embeddings_zero"], g_idx=qd["g_idx"], block_size=block_size,
        compute_dtype=torch.bfloat16)
    assert y.dtype == want.dtype and tuple(y.shape) == (M, V)
    assert max_rel_err(y, want) <= RTOL[torch.bfloat16]
    # the table read in place (more rows than the decode kernel takes) agrees with it row by row
    x40 = torch.cat([x, torch.randn(40 - M, D, generator=torch.Generator().manual_seed(23))])
    y40 = layer(x40, reverse=True)
    assert max_rel_err(y40[:M], want) <= RTOL[torch.bfloat16]
    # an assignment to the table rebuilds the copy (in place: its address stays what captured graphs hold)
    before, stamp = layer._cache["w4s"][2].data_ptr(), layer._cache["w4s"][0]
    layer._embeddings.assign(layer._embeddings.value.clone())
    y2 = layer(x, reverse=True)
    assert layer._cache["w4s"][0] != stamp and layer._cache["w4s"][2].data_ptr() == before
    assert torch.equal(bits(y2.cpu()), bits(y.cpu()))


@pytest.mark.parametrize("policy", ["float32", "bfloat16", "mixed_bfloat16"])
@pytest.mark.parametrize("block_size", [128, None])
def test_reversible_embedding_int4_tied(dev, policy, block_size):
    V, D, M = 1000, 512, 6
    layer = build_embedding(ReversibleEmbedding, dev, V, D, policy, seed=13)
    t = layer._embeddings.value.cpu()
    cd = TORCH[layer.compute_dtype]
    x = torch.randn(M, D, generator=torch.Generator().manual_seed(14))
    y_float = layer(x, reverse=True)
    layer.quantize("int4", config=Int4QuantizationConfig(block_size=block_size))
    qd = ref.embedding_quantize_int4(t.float(), block_size=block_size)
    assert torch.equal(layer._embeddings.value.cpu(), qd["embeddings"])
    y = layer(x, reverse=True)
    vd = TORCH[layer.variable_dtype]
    want = ref.reversible_embedding_int4_reverse(
        x.to(cd), qd["embeddings"], qd["embeddings_scale"].to(vd), D,
        embeddings_zero=qd["embeddings_zero"], g_idx=qd["g_idx"], block_size=block_size,
        compute_dtype=cd)
    assert y.dtype == want.dtype and tuple(y.shape) == (M, V)
    assert max_rel_err(y, want) <= RTOL[cd]
    err = (y_float.float().cpu() - y.float().cpu()).abs().max().item()
    assert err <= 0.2 * y_float.float().abs().max().item() + 1e-3
    ids = torch.tensor([1, 2, 3])
    assert layer(ids).shape == (3, D)


@pytest.mark.parametrize("policy", ["float32", "bfloat16", "mixed_bfloat16"])
@pytest.mark.parametrize("block_size", [128, 32, None])
@pytest.mark.parametrize("M,V,D", [(4, 512, 256), (40, 1000, 384)])
def test_reversible_embedding_int4_untied(dev, policy, block_size, M, V, D):
    layer = build_embedding(ReversibleEmbedding, dev, V, D, policy, seed=15, tie_weights=False)
    rt = layer.reverse_embeddings.value.cpu()
    cd = TORCH[layer.compute_dtype]
    x = torch.randn(M, D, generator=torch.Generator().manual_seed(16))
    y_float = layer(x, reverse=True)
    layer.quantize("int4", config=Int4QuantizationConfig(block_size=block_size))
    assert layer.reverse_embeddings.dtype == "int8" and layer.reverse_embeddings.shape == (D // 2, V)
    assert layer.reverse_embeddings_scale.dtype == layer.variable_dtype
    qd = ref.reversible_embedding_quantize_reverse_int4(rt.float(), block_size=block_size)
    assert torch.equal(layer.reverse_embeddings.value.cpu(), qd["reverse_embeddings"])
    grouped = block_size is not None
    vd = TORCH[layer.variable_dtype]
    if grouped:
        assert layer.reverse_embeddings_zero.dtype == layer.variable_dtype
        assert torch.equal(layer.reverse_embeddings_zero.value.float().cpu(), qd["zero"].float())
    y = layer(x, reverse=True)
    want = ref.reversible_embedding_int4_reverse(
        x.to(cd), qd["reverse_embeddings"], qd["scale"].to(vd), D,
        embeddings_zero=qd["zero"].to(vd) if grouped else None,
        g_idx=layer.g_idx.value.cpu() if grouped else None, block_size=block_size,
        compute_dtype=cd, tie_weights=False)
    assert y.dtype == want.dtype and tuple(y.shape) == (M, V)
    assert max_rel_err(y, want) <= RTOL[cd]
    err = (y_float.float().cpu() - y.float().cpu()).abs().max().item()
    assert err <= 0.25 * y_float.float().abs().max().item() + 1e-3
    store = {}
    layer.save_own_variables(store)
    assert len(store) == (7 if grouped else 4)


@pytest.mark.parametrize("policy,block", [("int4/128_from_float32", 128), ("int4/-1_from_float32", None),
                                          ("int4/-1_from_bfloat16", None), ("int4/-1_from_mixed_bfloat16", None),
                                          ("int4/128_from_bfloat16", 128)])
def test_reversible_embedding_int4_policy_built_quantizes_inputs(dev, policy, block):
    # a layer built from a policy has no config: the reference gives it the default
    # activation quantizer (reversible_embedding.py:229-233)
    V, D, M = 600, 256, 5
    src = build_embedding(ReversibleEmbedding, dev, V, D, policy.split("_from_")[1], seed=17)
    src.quantize("int4", config=Int4QuantizationConfig(block_size=block))
    store = {}
    src.save_own_variables(store)
    layer = ReversibleEmbedding(V, D, dtype=policy, device=dev)
    layer.build()
    layer.load_own_variables(store)
    assert layer.inputs_quantizer is not None and src.inputs_quantizer is None
    cd = TORCH[layer.compute_dtype]
    x = torch.randn(M, D, generator=torch.Generator().manual_seed(18))
    y = layer(x, reverse=True)
    grouped = block is not None
    want = ref.reversible_embedding_int4_reverse(
        x.to(cd), store["0"].cpu(), store["1"].cpu(), D,
        embeddings_zero=store["2"].cpu() if grouped else None,
        g_idx=store["3"].cpu() if grouped else None, block_size=block, compute_dtype=cd,
        quantize_inputs=True)
    assert y.dtype == want.dtype
    if grouped:
        assert max_rel_err(y, want) <= RTOL[cd]
    else:
        assert torch.equal(bits(y.cpu()), bits(want))  # integer accumulation, exact epilogue


@pytest.mark.parametrize("policy,block", [("int4/128_from_float32", 128), ("int4/-1_from_float32", None),
                                          ("int4/-1_from_bfloat16", None), ("int4/-1_from_mixed_bfloat16", None),
                                          ("int4/128_from_bfloat16", 128), ("int4/32_from_mixed_bfloat16", 32)])
def test_reversible_embedding_int4_untied_policy_built_quantizes_inputs(dev, policy, block):
    # untied weights and the default activation quantizer of a policy-built layer: int8 rows
    # against `reverse_embeddings`; float32 scales under bfloat16 compute promote the de-scale
    V, D, M = 520, 256, 6
    src = build_embedding(ReversibleEmbedding, dev, V, D, policy.split("_from_")[1], seed=27,
                          tie_weights=False)
    src.quantize("int4", config=Int4QuantizationConfig(block_size=block))
    store = {}
    src.save_own_variables(store)
    layer = ReversibleEmbedding(V, D, tie_weights=False, dtype=policy, device=dev)
    layer.build()
    layer.load_own_variables(store)
    assert layer.inputs_quantizer is not None
    cd = TORCH[layer.compute_dtype]
    x = torch.randn(M, D, generator=torch.Generator().manual_seed(28))
    y = layer(x, reverse=True)
    grouped = block is not None
    names = [n for n, _ in layer._spec_entries()]
    get = lambda n: store[str(names.index(n))].cpu()  # noqa: E731
    want = ref.reversible_embedding_int4_reverse(
        x.to(cd), get("reverse_embeddings"), get("reverse_embeddings_scale"), D,
        embeddings_zero=get("reverse_embeddings_zero") if grouped else None,
        g_idx=get("g_idx") if grouped else None, block_size=block, compute_dtype=cd,
        tie_weights=False, quantize_inputs=True)
    assert y.dtype == want.dtype and tuple(y.shape) == (M, V)
    if grouped:
        assert max_rel_err(y, want) <= RTOL[cd]
    else:
        assert torch.equal(bits(y.cpu()), bits(want))  # integer accumulation, exact epilogue


@pytest.mark.parametrize("mode", ["int4", "int8"])
@pytest.mark.parametrize("tie_weights", [True, False])
def test_reversible_embedding_reference_property(dev, mode, tie_weights):
    # reversible_embedding_test.py:156-185: (10, 16) layer, uniform inputs, weak MSE bounds
    g = torch.Generator().manual_seed(19)
    layer = build_embedding(ReversibleEmbedding, dev, 10, 16, "float32", seed=20, tie_weights=tie_weights)
    x = torch.randint(0, 9, (64, 3), generator=g)
    x_reverse = torch.rand(64, 16, generator=g)
    y_float, y_reverse_float = layer(x), layer(x_reverse, reverse=True)
    layer.quantize(mode)
    if not tie_weights:
        assert layer.reverse_embeddings.dtype == "int8"
        assert layer.reverse_embeddings_scale.dtype == layer.variable_dtype
    mse = (y_float - layer(x)).pow(2).mean().item()
    mse_reverse = (y_reverse_float - layer(x_reverse, reverse=True)).pow(2).mean().item()
    assert mse < 1e-3 and mse_reverse < 1e-2


@pytest.mark.parametrize("policy", ["float32", "bfloat16"])
@pytest.mark.parametrize("tie_weights", [True, False])
def test_reversible_embedding_int8_weight_only(dev, policy, tie_weights):
    from keras_amd.quantization_config import Int8QuantizationConfig

    V, D, M = 640, 256, 9
    layer = build_embedding(ReversibleEmbedding, dev, V, D, policy, seed=21, tie_weights=tie_weights)
    cd = TORCH[layer.compute_dtype]
    table_f = (layer._embeddings if tie_weights else layer.reverse_embeddings).value.cpu().float()
    x = torch.randn(M, D, generator=torch.Generator().manual_seed(22))
    layer.quantize("int8", config=Int8QuantizationConfig(activation_quantizer=None))
    assert layer.inputs_quantizer is None
    y = layer(x, reverse=True)
    if tie_weights:
        q, s = ref.embedding_quantize_int8(table_f)
        kernel = q.t()
    else:
        kernel, s = ref.dense_quantize_int8(table_f)
    # reversible_embedding.py:272-296 with inputs_scale = ones: float matmul, cast, divide
    want = torch.divide(ref.matmul(x.to(cd), kernel).to(cd), torch.multiply(torch.ones(1, dtype=cd), s.to(cd)))
    assert y.dtype == cd and max_rel_err(y, want) <= RTOL[cd]
