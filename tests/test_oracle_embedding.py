"""CPU: pins for the Embedding / ReversibleEmbedding functions of the oracle.

The functions compose primitives that tests/test_oracle.py already pins (abs-max quantizer,
pack / unpack, the grouped quantizer, the int8 matmul); what is checked here is the
composition: which axis is reduced, which scale meets which row, multiply versus divide,
the nibble order along the output dim -- each against plain Python loops on small tables,
plus the reference's own property tests (embedding_test.py:364-394, :793-824, :921-941).
"""

import math

import numpy as np
import pytest
import torch

from oracle import keras_cpu_path as ref


def table(V, D, seed=0):
    g = torch.Generator().manual_seed(seed)
    return (torch.rand(V, D, generator=g) * 2.0 - 1.0) * 0.05  # keras "uniform" initializer


def test_int8_table_quantization_and_lookup_by_loops():
    V, D = 7, 12
    t = table(V, D)
    q, s = ref.embedding_quantize_int8(t)
    assert q.dtype == torch.int8 and tuple(s.shape) == (V,)
    tn = t.numpy()
    for v in range(V):
        amax = np.abs(tn[v]).max()
        sc = np.float32(127.0) / (np.float32(amax) + np.float32(1e-7))
        assert s[v].item() == pytest.approx(float(sc), rel=1e-6)
        for d in range(D):
            want = int(np.clip(np.round(np.float32(tn[v, d]) * sc), -127, 127))
            assert q[v, d].item() == want
    ids = torch.tensor([[0, 6], [3, -1]])  # -1 wraps to the last row
    out = ref.embedding_int8_call(ids, q, s)
    assert tuple(out.shape) == (2, 2, D) and out.dtype == torch.float32
    for (i, j), v in {(0, 0): 0, (0, 1): 6, (1, 0): 3, (1, 1): V - 1}.items():
        for d in range(D):
            assert out[i, j, d].item() == np.float32(q[v, d].item()) / np.float32(s[v].item())


@pytest.mark.parametrize("block_size", [None, 4, 8])
def test_int4_table_by_loops(block_size):
    V, D = 6, 16
    t = table(V, D, seed=1)
    qd = ref.embedding_quantize_int4(t, block_size=block_size)
    packed, unpacked = qd["embeddings"], qd["unpacked"]
    assert tuple(packed.shape) == (V, D // 2)
    # nibble order along the output dim: low nibble = even column
    for v in range(V):
        for j in range(D // 2):
            byte = packed[v, j].item() & 0xFF
            lo, hi = byte & 0xF, byte >> 4
            assert ((lo ^ 8) - 8) == unpacked[v, 2 * j].item()
            assert ((hi ^ 8) - 8) == unpacked[v, 2 * j + 1].item()
    ids = torch.tensor([5, 0, 2])
    out = ref.embedding_int4_call(ids, packed, qd["embeddings_scale"], D,
                                  embeddings_zero=qd["embeddings_zero"], g_idx=qd["g_idx"],
                                  block_size=block_size)
    if block_size is None:
        assert tuple(qd["embeddings_scale"].shape) == (V,)
        for r, v in enumerate(ids.tolist()):
            for d in range(D):
                want = np.float32(unpacked[v, d].item()) / np.float32(qd["embeddings_scale"][v].item())
                assert out[r, d].item() == want
    else:
        G = math.ceil(D / block_size)
        assert tuple(qd["embeddings_scale"].shape) == (V, G)
        assert tuple(qd["embeddings_zero"].shape) == (V, G) and qd["embeddings_zero"].dtype == torch.int8
        # embedding_test.py:921-941
        assert torch.equal(qd["g_idx"], torch.tensor(np.arange(D) // block_size, dtype=torch.float32))
        for r, v in enumerate(ids.tolist()):
            for d in range(D):
                gi = d // block_size
                want = (np.float32(unpacked[v, d].item()) - np.float32(qd["embeddings_zero"][v, gi].item())) \
                    * np.float32(qd["embeddings_scale"][v, gi].item())
                assert out[r, d].item() == want
        # the grouped parameters are those of the group's own min / max (asymmetric)
        tn = t.numpy()
        for v in range(V):
            for gi in range(G):
                seg = tn[v, gi * block_size:(gi + 1) * block_size]
                sc = (np.float32(seg.max()) - np.float32(seg.min()) + np.float32(1e-7)) / np.float32(15)
                assert qd["embeddings_scale"][v, gi].item() == pytest.approx(float(sc), rel=1e-6)


@pytest.mark.parametrize("mode,V,D,block", [("int8", 10, 16, None), ("int4", 10, 16, 128),
                                            ("int4", 100, 256, 64), ("int4", 100, 256, None)])
def test_reference_weak_mse_property(mode, V, D, block):
    # embedding_test.py:364-394 and :793-824: mean squared error against the float layer < 1e-3
    t = table(V, D, seed=2)
    ids = torch.randint(0, V - 1, (64, 3), generator=torch.Generator().manual_seed(3))
    y_float = t[ids]
    if mode == "int8":
        q, s = ref.embedding_quantize_int8(t)
        y = ref.embedding_int8_call(ids, q, s)
    else:
        qd = ref.embedding_quantize_int4(t, block_size=block)
        y = ref.embedding_int4_call(ids, qd["embeddings"], qd["embeddings_scale"], D,
                                    embeddings_zero=qd["embeddings_zero"], g_idx=qd["g_idx"],
                                    block_size=block)
    assert (y_float - y).pow(2).mean().item() < 1e-3


def test_lookup_dtype_promotion_without_autocast():
    # bfloat16 compute, float32 scale variable (the layer does not autocast): float32 out
    t = table(5, 8, seed=4)
    q, s = ref.embedding_quantize_int8(t)
    out = ref.embedding_int8_call(torch.tensor([1, 2]), q, s, compute_dtype="bfloat16")
    assert out.dtype == torch.float32
    assert torch.equal(out, q[[1, 2]].float() / s[[1, 2]].unsqueeze(-1))
    out_bf = ref.embedding_int8_call(torch.tensor([1, 2]), q, s.to(torch.bfloat16), compute_dtype="bfloat16")
    assert out_bf.dtype == torch.bfloat16


def test_out_of_range_ids_raise():
    t = table(5, 8)
    q, s = ref.embedding_quantize_int8(t)
    with pytest.raises(IndexError):
        ref.embedding_int8_call(torch.tensor([5]), q, s)
    with pytest.raises(IndexError):
        ref.embedding_int8_call(torch.tensor([-6]), q, s)


def test_reverse_projection_tied_int8_closed_form():
    V, D, M = 9, 32, 3
    t = table(V, D, seed=5)
    q, s = ref.embedding_quantize_int8(t)
    x = torch.randn(M, D, generator=torch.Generator().manual_seed(6))
    logits, inter = ref.reversible_embedding_int8_reverse(x, q, s, return_intermediates=True)
    assert tuple(logits.shape) == (M, V)
    xq, xs = inter["q"], inter["inputs_scale"]
    for m in range(M):
        for v in range(V):
            acc = sum(int(xq[m, d]) * int(q[v, d]) for d in range(D))
            assert inter["acc"][m, v].item() == acc
            want = np.float32(acc) / (np.float32(xs[m, 0].item()) * np.float32(s[v].item()))
            assert logits[m, v].item() == want
    # and it approximates the float projection
    want_f = x @ t.T
    assert (logits - want_f).abs().max().item() < 0.05 * want_f.abs().max().item() + 1e-3
    capped = ref.reversible_embedding_int8_reverse(x, q, s, logit_soft_cap=0.5)
    assert torch.allclose(capped, torch.tanh(logits / 0.5) * 0.5)


@pytest.mark.parametrize("block_size", [None, 8])
def test_reverse_projection_tied_int4_by_loops(block_size):
    V, D, M = 5, 16, 2
    t = table(V, D, seed=7)
    qd = ref.embedding_quantize_int4(t, block_size=block_size)
    x = torch.randn(M, D, generator=torch.Generator().manual_seed(8))
    logits = ref.reversible_embedding_int4_reverse(
        x, qd["embeddings"], qd["embeddings_scale"], D, embeddings_zero=qd["embeddings_zero"],
        g_idx=qd["g_idx"], block_size=block_size)
    assert tuple(logits.shape) == (M, V) and logits.dtype == torch.float32
    w = qd["unpacked"]
    for m in range(M):
        for v in range(V):
            if block_size is None:
                acc = sum(float(x[m, d]) * float(w[v, d]) for d in range(D))
                want = acc / float(qd["embeddings_scale"][v])
            else:
                want = sum(
                    float(x[m, d]) * (float(w[v, d]) - float(qd["embeddings_zero"][v, d // block_size]))
                    * float(qd["embeddings_scale"][v, d // block_size]) for d in range(D))
            assert logits[m, v].item() == pytest.approx(want, rel=2e-5, abs=1e-6)
    # and it approximates the float projection (int4: coarse)
    want_f = x @ t.T
    assert (logits - want_f).abs().max().item() < 0.25 * want_f.abs().max().item() + 1e-3


@pytest.mark.parametrize("block_size", [None, 8])
@pytest.mark.parametrize("quantize_inputs", [False, True])
def test_reverse_projection_untied_int4_by_loops(block_size, quantize_inputs):
    V, D, M = 5, 16, 2
    rt = table(D, V, seed=9)  # reverse_embeddings [D, V]
    qd = ref.reversible_embedding_quantize_reverse_int4(rt, block_size=block_size)
    assert tuple(qd["reverse_embeddings"].shape) == (D // 2, V)
    w = qd["unpacked"]  # [D, V]
    # packed along axis 0: low nibble = even row
    for j in range(D // 2):
        for v in range(V):
            byte = qd["reverse_embeddings"][j, v].item() & 0xFF
            assert ((byte & 0xF) ^ 8) - 8 == w[2 * j, v].item()
            assert ((byte >> 4) ^ 8) - 8 == w[2 * j + 1, v].item()
    g_idx = None if block_size is None else torch.floor_divide(torch.arange(D, dtype=torch.float32), block_size)
    zero = None if qd["zero"] is None else qd["zero"].float()
    x = torch.randn(M, D, generator=torch.Generator().manual_seed(10))
    logits = ref.reversible_embedding_int4_reverse(
        x, qd["reverse_embeddings"], qd["scale"], D, embeddings_zero=zero, g_idx=g_idx,
        block_size=block_size, tie_weights=False, quantize_inputs=quantize_inputs)
    if quantize_inputs:
        xq, xs = ref.abs_max_quantize(x, axis=-1)
        xv, xdiv = xq.float(), xs
    else:
        xv, xdiv = x, torch.ones(M, 1)
    for m in range(M):
        for v in range(V):
            if block_size is None:
                acc = sum(float(xv[m, d]) * float(w[d, v]) for d in range(D))
                want = acc / (float(xdiv[m, 0]) * float(qd["scale"][v]))
            else:
                acc = sum(float(xv[m, d]) * (float(w[d, v]) - float(zero[d // block_size, v]))
                          * float(qd["scale"][d // block_size, v]) for d in range(D))
                want = acc / float(xdiv[m, 0])
            assert logits[m, v].item() == pytest.approx(want, rel=3e-5, abs=1e-6)
    want_f = x @ rt
    assert (logits - want_f).abs().max().item() < 0.3 * want_f.abs().max().item() + 1e-3


def test_reverse_projection_tied_int4_with_input_quantizer():
    V, D, M = 6, 16, 3
    t = table(V, D, seed=11)
    x = torch.randn(M, D, generator=torch.Generator().manual_seed(12))
    qd = ref.embedding_quantize_int4(t, block_size=None)
    logits = ref.reversible_embedding_int4_reverse(x, qd["embeddings"], qd["embeddings_scale"], D,
                                                   block_size=None, quantize_inputs=True)
    xq, xs = ref.abs_max_quantize(x, axis=-1)
    for m in range(M):
        for v in range(V):
            acc = sum(int(xq[m, d]) * int(qd["unpacked"][v, d]) for d in range(D))
            import numpy as np
            want = np.float32(acc) / (np.float32(xs[m, 0].item()) * np.float32(qd["embeddings_scale"][v].item()))
            assert logits[m, v].item() == want


def test_einsum_non_default_configs_against_float64():
    # weight-only int8 and activation-quantized int4 EinsumDense (torch branch): the value is
    # einsum(x, q / scale) resp. einsum(xq, q4 / scale) / x_scale, checked in float64
    g = torch.Generator().manual_seed(21)
    for equation, kshape, xshape in [("btd,dnh->btnh", (16, 2, 4), (2, 3, 16)),
                                     ("btnh,nhd->btd", (2, 4, 8), (2, 3, 2, 4)),
                                     ("ab,bc->ac", (8, 6), (5, 8))]:
        kernel = torch.rand(kshape, generator=g) - 0.5
        x = torch.rand(xshape, generator=g)
        q8, s8, info = ref.einsum_dense_quantize_int8(kernel, equation, len(xshape))
        got = ref.einsum_dense_int8_weight_only_call(x, q8, s8, equation)
        s_full = ref._adjust_scale_for_dequant(s8, info["kernel"])
        want = torch.einsum(equation, x.double(), q8.double() / s_full.double())
        assert torch.allclose(got.double(), want, rtol=1e-5, atol=1e-6)
        assert (got - torch.einsum(equation, x, kernel)).abs().max() < 0.05
        qk = ref.einsum_dense_quantize_int4(kernel, equation, len(xshape), None)
        got4 = ref.einsum_dense_int4_activation_quantized_call(x, qk, equation)
        xq, xs = ref.abs_max_quantize(x, axis=tuple(qk["info"]["input"]["reduced"]))
        w = (qk["unpacked"].double() / qk["kernel_scale"].double()).reshape(kshape)
        want4 = torch.einsum(equation, xq.double(), w) / ref._adjust_scale(xs, qk["info"]["input"]).double()
        assert torch.allclose(got4.double(), want4, rtol=1e-5, atol=1e-6)
        assert (got4 - torch.einsum(equation, x, kernel)).abs().max() < 0.35
