"""Pins the CPU oracle: reference known-answer vectors, closed forms, brute force and the
cross-check between the torch restatement and the independent C restatement."""

import json
import math
import os

import numpy as np
import pytest
import torch

from oracle import keras_cpu_path as ref
from tests.helpers import c_gemm_i8, c_oracle, c_w4_matmul_f64

HERE = os.path.dirname(os.path.abspath(__file__))


# ---------------------------------------------------------------- pack / unpack
def test_pack_docstring_vectors():
    data = json.load(open(os.path.join(HERE, "golden", "pack_int4_docstring_vectors.json")))
    for case in data["cases"]:
        arr = torch.tensor(case["input"], dtype=torch.int8)
        packed, shape, n = ref.pack_int4(arr, axis=case["axis"])
        assert packed.tolist() == case["packed"]
        assert n == case["orig_len"] and shape == tuple(packed.shape)
        back = ref.unpack_int4(packed, n, axis=case["axis"])
        assert back.tolist() == case["input"]


def test_pack_closed_form_all_pairs():
    lo = torch.arange(-8, 8, dtype=torch.int8).repeat(16)
    hi = torch.arange(-8, 8, dtype=torch.int8).repeat_interleave(16)
    arr = torch.stack([lo, hi], dim=0)  # pack along axis 0: one byte per column
    packed, _, _ = ref.pack_int4(arr, axis=0)
    want = ((lo.to(torch.int32) & 15) | ((hi.to(torch.int32) & 15) << 4)).to(torch.uint8).view(torch.int8)
    assert torch.equal(packed[0], want)


def test_unpack_exhaustive_bytes():
    b = torch.arange(256, dtype=torch.int32).to(torch.uint8)
    got = ref.unpack_int4(b.view(torch.int8).reshape(1, 256), 2, axis=0)
    v = b.to(torch.int32)
    assert torch.equal(got[0].to(torch.int32), ((v & 15) ^ 8) - 8)
    assert torch.equal(got[1].to(torch.int32), (((v >> 4) & 15) ^ 8) - 8)
    gotu = ref.unpack_int4(b.reshape(1, 256), 2, axis=0, dtype="uint8")
    assert torch.equal(gotu[0].to(torch.int32), v & 15)
    assert torch.equal(gotu[1].to(torch.int32), (v >> 4) & 15)


SCENARIOS = [((8, 8), 0), ((8, 8), 1), ((5, 8), 0), ((8, 5), 1), ((4, 6, 8), 1), ((4, 6, 5), -1),
             ((2, 3, 4, 5), 2)]  # quantizers_test.py:157-175


@pytest.mark.parametrize("shape,axis", SCENARIOS)
@pytest.mark.parametrize("dtype", ["int8", "uint8"])
def test_pack_round_trip_scenarios(shape, axis, dtype):
    g = torch.Generator().manual_seed(0)
    if dtype == "int8":
        arr = torch.randint(-8, 8, shape, generator=g, dtype=torch.int8)
    else:
        arr = torch.randint(0, 16, shape, generator=g, dtype=torch.uint8)
    packed, pshape, n = ref.pack_int4(arr, axis=axis, dtype=dtype)
    ax = axis % len(shape)
    assert pshape[ax] == math.ceil(shape[ax] / 2) and n == shape[ax]
    assert torch.equal(ref.unpack_int4(packed, n, axis=axis, dtype=dtype), arr)
    # C restatement agrees byte for byte
    outer = int(np.prod(shape[:ax])) if ax else 1
    inner = int(np.prod(shape[ax + 1:])) if ax + 1 < len(shape) else 1
    cp = torch.empty(pshape, dtype=arr.dtype)
    c_oracle().k3q_oracle_pack_int4(arr.contiguous().data_ptr(), outer, shape[ax], inner, cp.data_ptr())
    assert torch.equal(cp, packed)
    cu = torch.empty(shape, dtype=arr.dtype)
    c_oracle().k3q_oracle_unpack_int4(cp.data_ptr(), outer, pshape[ax], inner, n,
                                      1 if dtype == "int8" else 0, cu.data_ptr())
    assert torch.equal(cu, arr)


def test_pack_errors():
    with pytest.raises(ValueError):
        ref.pack_int4(torch.zeros(2, 2, dtype=torch.int8), dtype="int16")
    with pytest.raises(TypeError):
        ref.pack_int4(torch.zeros(2, 2, dtype=torch.uint8), dtype="int8")
    with pytest.raises(TypeError):
        ref.unpack_int4(torch.zeros(2, 2, dtype=torch.int32), 4)


# ---------------------------------------------------------------- abs-max quantizer
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_abs_max_invariants(dtype):
    g = torch.Generator().manual_seed(0)
    x = (torch.randn(3, 4, 5, generator=g) * 2).to(dtype)
    q, s = ref.abs_max_quantize(x, axis=-1)
    assert q.dtype == torch.int8 and s.dtype == dtype and tuple(s.shape) == (3, 4, 1)
    assert q.min() >= -127 and q.max() <= 127
    # the arg-max element of every row maps to +-127
    idx = x.abs().float().argmax(-1, keepdim=True)
    assert (q.gather(-1, idx).abs() >= 126).all()
    deq = q.float() / s.float()
    assert (deq - x.float()).pow(2).mean().sqrt() < 0.1
    # numpy path == tensor path in float32 (quantizers_test.py:106-115)
    if dtype == torch.float32:
        qn, sn = ref.abs_max_quantize(x, axis=-1, to_numpy=True)
        assert torch.equal(qn, q) and torch.allclose(sn, s, rtol=1e-6, atol=0)


def test_abs_max_closed_form_rows():
    x = torch.zeros(4, 8)
    x[1] = torch.tensor([127.0, 0.5, 1.5, 2.5, -0.5, -1.5, 63.5, -127.0])  # scale ~ 1: ties to even
    x[2] = 2.0 ** torch.arange(-4, 4).float()
    q, s = ref.abs_max_quantize(x, axis=-1)
    assert torch.equal(q[0], torch.zeros(8, dtype=torch.int8))
    assert s[0, 0].item() == pytest.approx(127.0 / 1e-7, rel=1e-6)
    # 127 / (127 + 1e-7) rounds to exactly 1.0 in float32
    assert s[1, 0].item() == 1.0
    assert q[1].tolist() == [127, 0, 2, 2, 0, -2, 64, -127]
    assert q[2].tolist() == [round(v) for v in (x[2] * s[2, 0]).tolist()]


def test_abs_max_empty_axis_reduces_nothing():
    # keras/src/backend/torch/numpy.py:302-304: amax over axis=() returns x itself (as numpy's
    # max over an empty axis tuple does), so every element gets its own scale 127 / (|x| + eps)
    # and every element that is not tiny lands on +-127
    x = torch.tensor([[0.5, -3.0, 0.0], [1e-3, 7.25, -1.0]])
    q, s = ref.abs_max_quantize(x, axis=())
    assert tuple(s.shape) == tuple(x.shape)
    assert torch.allclose(s, 127.0 / (x.abs() + 1e-7), rtol=1e-6, atol=0)
    assert q.tolist() == [[127, -127, 0], [127, 127, -127]]
    qn, sn = ref.abs_max_quantize(x, axis=(), to_numpy=True)
    assert torch.equal(qn, q) and torch.allclose(sn, s, rtol=1e-6, atol=0)
    q2, s2 = ref.AbsMaxQuantizer()(x, axis=())
    assert torch.equal(q2, q) and torch.equal(s2, s)


@pytest.mark.parametrize("dtype_code,dtype", [(0, torch.float32), (1, torch.bfloat16)])
def test_abs_max_c_restatement_agrees(dtype_code, dtype):
    g = torch.Generator().manual_seed(1)
    x = (torch.randn(64, 1000, generator=g) * 3).to(dtype)
    x[5] = 0
    x[6, 3] = 1e-6
    q, s = ref.abs_max_quantize(x, axis=-1)
    cq = torch.empty_like(q)
    cs = torch.empty(64, dtype=dtype)
    c_oracle().k3q_oracle_absmax_quantize(x.data_ptr(), dtype_code, 64, 1000, 1e-7, -127.0, 127.0,
                                          cq.data_ptr(), cs.data_ptr())
    assert torch.equal(cs.float(), s.flatten().float())
    assert torch.equal(cq, q)


def test_bf16_epsilon_is_rounded_before_the_add():
    # torch casts the 0-dim float32 epsilon to bfloat16 before adding: distinguishes the two
    # candidate semantics on rows whose max is tiny
    bitsv = torch.arange(0x2000, 0x3800, dtype=torch.int32).to(torch.int16).view(torch.bfloat16)
    x = bitsv.reshape(-1, 1)
    _, s = ref.abs_max_quantize(x, axis=-1)
    eps_bf = torch.tensor(1e-7).to(torch.bfloat16).float()
    want = (127.0 / (x.float() + eps_bf).to(torch.bfloat16).float()).to(torch.bfloat16)
    assert torch.equal(s, want)


# ---------------------------------------------------------------- grouped quantizer
def test_grouped_quantizer_against_loops():
    g = torch.Generator().manual_seed(42)
    w = torch.randn(500, 6, generator=g)  # 500 rows / block 128: last group is zero padded
    q, s, z = ref.abs_max_quantize_grouped_with_zero_point(w, block_size=128)
    assert tuple(q.shape) == (500, 6) and tuple(s.shape) == (4, 6) and tuple(z.shape) == (4, 6)
    assert z.dtype == torch.int8 and q.min() >= -8 and q.max() <= 7
    wn = w.numpy()
    for gi in range(4):
        rows = wn[gi * 128:(gi + 1) * 128]
        if rows.shape[0] < 128:
            rows = np.concatenate([rows, np.zeros((128 - rows.shape[0], 6), np.float32)])
        for n in range(6):
            lo, hi = rows[:, n].min(), rows[:, n].max()
            sc = np.float32((hi - lo + np.float32(1e-7)) / np.float32(15))
            zp = np.clip(np.round(-lo / sc) + -8, -8, 7)
            assert s[gi, n].item() == pytest.approx(float(sc), rel=1e-6)
            assert z[gi, n].item() == int(zp)
            for r in range(min(128, 500 - gi * 128)):
                want = int(np.clip(np.round(np.float32(rows[r, n]) / sc) + zp, -8, 7))
                assert q[gi * 128 + r, n].item() == want
    # de-quantised error bound of quantizers_test.py:754-788
    g_idx = torch.floor_divide(torch.arange(500, dtype=torch.float32), 128)
    deq = ref.dequantize_with_sz_map(q, s, z, g_idx, group_axis=0)
    assert (deq - w).pow(2).mean().sqrt() < 0.15


def test_dequantize_with_sz_map_double_loop():
    g = torch.Generator().manual_seed(3)
    q = torch.randint(-8, 8, (12, 5), generator=g, dtype=torch.int8)
    s = torch.rand(3, 5, generator=g) + 0.1
    z = torch.randint(-8, 8, (3, 5), generator=g, dtype=torch.int8)
    g_idx = torch.tensor([0, 0, 0, 0, 1, 1, 1, 1, 2, 2, 2, 2], dtype=torch.float32)
    got = ref.dequantize_with_sz_map(q, s, z, g_idx, group_axis=0)
    for k in range(12):
        for n in range(5):
            gi = int(g_idx[k])
            assert got[k, n].item() == pytest.approx((q[k, n].item() - z[gi, n].item()) * s[gi, n].item(), rel=1e-6)


# ---------------------------------------------------------------- integer matmul / epilogue
def test_int8_matmul_brute_force():
    g = torch.Generator().manual_seed(0)
    a = torch.randint(-128, 128, (7, 33), generator=g, dtype=torch.int8)
    b = torch.randint(-128, 128, (33, 5), generator=g, dtype=torch.int8)
    got = ref.matmul(a, b)
    assert got.dtype == torch.int32
    want = a.numpy().astype(np.int64) @ b.numpy().astype(np.int64)
    assert np.array_equal(got.numpy().astype(np.int64), want)
    assert torch.equal(c_gemm_i8(a, b), got)
    e = ref.einsum("ab,bc->ac", a, b)
    assert torch.equal(e, got)


def test_int8_matmul_no_overflow_at_max_k():
    a = torch.full((2, 14336), 127, dtype=torch.int8)
    b = torch.full((14336, 3), -127, dtype=torch.int8)
    assert ref.matmul(a, b)[0, 0].item() == -14336 * 127 * 127
    assert c_gemm_i8(a, b)[1, 2].item() == -14336 * 127 * 127


@pytest.mark.parametrize("dtype_code,dtype", [(0, torch.float32), (1, torch.bfloat16)])
def test_dense_int8_call_matches_c_restatement(dtype_code, dtype):
    g = torch.Generator().manual_seed(5)
    x = torch.randn(9, 256, generator=g).to(dtype)
    kernel = ref.glorot_uniform(256, 40, generator=g)
    bias = torch.randn(40, generator=g) * 0.02
    qk, ks = ref.dense_quantize_int8(kernel)
    y, inter = ref.dense_int8_call(x, qk, ks, bias, compute_dtype=dtype, return_intermediates=True)
    assert torch.equal(inter["acc"], c_gemm_i8(inter["q"], qk))
    cy = torch.empty(9, 40, dtype=dtype)
    # keep the operands alive across the call: data_ptr() of a temporary dangles
    acc_c, si_c = inter["acc"].contiguous(), inter["inputs_scale"].contiguous()
    ks_c, bias_c = ks.to(dtype).contiguous(), bias.to(dtype).contiguous()
    c_oracle().k3q_oracle_descale(acc_c.data_ptr(), 9, 40, dtype_code, si_c.data_ptr(),
                                  ks_c.data_ptr(), bias_c.data_ptr(), cy.data_ptr())
    assert torch.equal(cy.float(), y.float())
    # closed form in float64 within the stated tolerance
    exact = inter["acc"].double() / (ks.double() * inter["inputs_scale"].double()) + bias.double()
    tol = 1e-3 if dtype == torch.float32 else 2e-2
    assert ((y.double() - exact).abs().max() / exact.abs().max()).item() < tol


@pytest.mark.parametrize("block_size", [None, 32])
def test_dense_int4_call_against_f64(block_size):
    g = torch.Generator().manual_seed(6)
    kernel = ref.glorot_uniform(128, 24, generator=g)
    qk = ref.dense_quantize_int4(kernel, block_size)
    x = torch.randn(5, 128, generator=g)
    y = ref.dense_int4_call(x, qk["kernel"], qk["kernel_scale"], 24, kernel_zero=qk["kernel_zero"],
                            g_idx=qk["g_idx"], block_size=block_size)
    exact = c_w4_matmul_f64(x, qk["kernel"], qk["kernel_scale"], qk["kernel_zero"], block_size, None, 24)
    assert ((y.double() - exact).abs().max() / exact.abs().max()).item() < 1e-5
    # and the weight-only result approximates the float layer
    assert (y - x @ kernel).pow(2).mean().item() < 2e-2


# ---------------------------------------------------------------- LoRA merged on save
@pytest.mark.parametrize("mode,block_size", [("int8", None), ("int4", None), ("int4", 32)])
def test_merged_lora_kernel_invariants(mode, block_size):
    g = torch.Generator().manual_seed(17)
    K, N, rank, alpha = 96, 40, 4, 8.0
    kernel = ref.glorot_uniform(K, N, generator=g)
    if mode == "int8":
        qk, ks = ref.dense_quantize_int8(kernel)
        kw = dict()
        dequant = lambda q, s, z: q.float() / s
    else:
        q4 = ref.dense_quantize_int4(kernel, block_size)
        qk, ks = q4["kernel"], q4["kernel_scale"]
        kw = dict(kernel_zero=q4["kernel_zero"], g_idx=q4["g_idx"], block_size=block_size, orig_output_dim=N)
        if block_size:
            dequant = lambda q, s, z: ref.dequantize_with_sz_map(ref.unpack_int4(q, N, axis=-1), s, z, q4["g_idx"], group_axis=0)
        else:
            dequant = lambda q, s, z: ref.unpack_int4(q, N, axis=-1).float() / s
    a = torch.randn(K, rank, generator=g) * 0.05
    zero_b = torch.zeros(rank, N)
    # a zero update: quantising the de-quantised kernel again gives the same integers (every
    # column / group of an abs-max quantised kernel holds an extreme of the range)
    q0, s0, z0 = ref.dense_merged_lora_kernel(mode, qk, ks, a, zero_b, alpha, rank, **kw)
    if not block_size:
        assert torch.equal(q0, qk)
        assert torch.allclose(s0, ks, rtol=1e-5, atol=0)
        assert z0 is None
    else:
        # (grouped: the asymmetric re-quantisation need not hit the same integers, the values must)
        assert (dequant(q0, s0, z0) - dequant(qk, ks, kw["kernel_zero"])).abs().max() <= 0.51 / s0.min()
    # a real update: the saved kernel de-quantises to (old de-quantised kernel + update) within
    # half a quantisation step of its own scales
    b = torch.randn(rank, N, generator=g) * 0.05
    q1, s1, z1 = ref.dense_merged_lora_kernel(mode, qk, ks, a, b, alpha, rank, **kw)
    target = dequant(qk, ks, kw.get("kernel_zero")) + (alpha / rank) * (a @ b)
    got = dequant(q1, s1, z1)
    step = (1.0 / s1) if s1.dim() == 1 else (1.0 / s1).repeat_interleave(block_size, dim=0)[:K]
    assert ((got - target).abs() <= 0.5001 * step + 1e-6).all()
    assert q1.dtype == torch.int8 and tuple(q1.shape) == tuple(qk.shape)
    assert not torch.equal(q1, qk)


# ---------------------------------------------------------------- EinsumDense bookkeeping
def test_einsum_info_hand_derived_rows():
    a = ref.einsum_quantization_info("btd,dnh->btnh", 3)
    assert a["input"]["reduced"] == [2] and a["kernel"]["reduced"] == [0]
    b = ref.einsum_quantization_info("btnh,nhd->btd", 4)
    assert b["input"]["reduced"] == [2, 3] and b["input"]["transpose"] == [0, 1, 3, 2]
    assert b["input"]["squeeze"] == [3] and b["kernel"]["reduced"] == [0, 1]
    k = torch.randn(4096 // 64, 4, 8)  # stand-in for [d, n, h]
    _, s, _ = ref.einsum_dense_quantize_int8(k, "btd,dnh->btnh", 3)
    assert tuple(s.shape) == (1, 1, 4, 8)
    k2 = torch.randn(4, 8, 16)
    _, s2, _ = ref.einsum_dense_quantize_int8(k2, "btnh,nhd->btd", 4)
    assert tuple(s2.shape) == (1, 1, 16)


def test_einsum_info_shared_label_and_stale_index_rows():
    # hand-derived from keras/src/layers/core/einsum_dense.py:1995-2040 for the equations of
    # einsum_dense_test.py:598-629.  "abcde,afce->acdbf": input keeps a,b,c,d (transpose to
    # a,c,d,b), e is reduced and takes the place of f (the one output label the input lacks);
    # kernel a,f,c,e: e is reduced and takes the place of d, the place of b is left to expand
    a = ref.einsum_quantization_info("abcde,afce->acdbf", 5)
    assert a["input"] == dict(reduced=[4], expand=[], transpose=[0, 2, 3, 1, 4], squeeze=[])
    assert a["kernel"] == dict(reduced=[3], expand=[3], transpose=[0, 2, 3, 1], squeeze=[])
    _, s, _ = ref.einsum_dense_quantize_int8(torch.randn(1, 16, 2, 32), "abcde,afce->acdbf", 5)
    assert tuple(s.shape) == (1, 2, 1, 1, 16)   # broadcasts against a,c,d,b,f
    # "ab,ab->a": b is reduced on both sides and the output lacks no label, so the reduced axis
    # is marked for squeezing and inserted at the stale index, output_spec.find("b") == -1, i.e.
    # before the last entry: transpose [1, 0].  A [a, 1] scale becomes [1, a]; the squeeze of
    # axis 1 (size a) is a no-op on the torch backend.  The de-scaled result is therefore [1, a].
    b = ref.einsum_quantization_info("ab,ab->a", 2)
    assert b["input"] == dict(reduced=[1], expand=[], transpose=[1, 0], squeeze=[1])
    assert b["kernel"] == dict(reduced=[1], expand=[], transpose=[1, 0], squeeze=[1])
    g = torch.Generator().manual_seed(5)
    k, x = torch.rand(3, 8, generator=g) - 0.5, torch.rand(3, 8, generator=g)
    qk, ks, _ = ref.einsum_dense_quantize_int8(k, "ab,ab->a", 2)
    assert tuple(ks.shape) == (1, 3)
    y = ref.einsum_dense_int8_call(x, qk, ks, "ab,ab->a")
    assert tuple(y.shape) == (1, 3)
    assert (y.reshape(-1) - torch.einsum("ab,ab->a", x, k)).abs().max().item() < 2e-2
    # "a,b->ab": nothing is reduced; each operand's scale is per element and gains the other's axis
    c = ref.einsum_quantization_info("a,b->ab", 1)
    assert c["input"] == dict(reduced=[], expand=[1], transpose=[0], squeeze=[])
    assert c["kernel"] == dict(reduced=[], expand=[0], transpose=[0], squeeze=[])


@pytest.mark.parametrize("equation,kshape,xshape", [
    ("btnh,nhd->btd", (2, 4, 8), (1, 2, 2, 4)), ("btd,ndh->btnh", (2, 4, 8), (1, 2, 4)),
    ("btd,df->btf", (4, 4), (1, 2, 4)), ("ab,bcd->acd", (3, 8, 32), (2, 3)),
    ("...b,bc->...c", (7, 5), (2, 3, 7)), ("abc,cd->abd", (6, 9), (2, 3, 6)),
    ("abcde,afce->acdbf", (1, 16, 2, 32), (1, 8, 2, 4, 32)), ("a,b->ab", (4,), (5,)),
    ("ab,c->ac", (5,), (3, 4)), ("bhqd,hdk->bhqk", (4, 8, 6), (2, 4, 3, 8)),
])
def test_einsum_int8_descale_approximates_float(equation, kshape, xshape):
    # the scales must broadcast against the einsum output such that the de-scaled integer
    # einsum approximates the float einsum: a wrong axis, transpose or squeeze breaks this
    g = torch.Generator().manual_seed(1337)
    kernel = torch.rand(kshape, generator=g) - 0.5
    x = torch.rand(xshape, generator=g)
    qk, ks, _ = ref.einsum_dense_quantize_int8(kernel, equation, len(xshape))
    y = ref.einsum_dense_int8_call(x, qk, ks, equation)
    want = torch.einsum(equation, x, kernel)
    assert tuple(y.shape) == tuple(want.shape)
    assert (y - want).pow(2).mean().item() < 1e-3


# ---------------------------------------------------------------- EinsumDense int4 (forward), LoRA
def _nibble(byte, high):
    """Signed value of one nibble of a stored byte, spelled out (no call into the oracle)."""
    v = ((int(byte) & 0xFF) >> (4 if high else 0)) & 15
    return v - 16 if v >= 8 else v


def _einsum_int4_kernel_by_loops(qk, block_size):
    """The float64 kernel an int4 EinsumDense de-quantises to, built weight by weight from the
    packed bytes: flat row r, flat column c sit in byte [r, c // 2] (even c in the low nibble);
    the flat matrix is the row-major reshape of the kernel (einsum_dense.py:1388-1398)."""
    rows, cols = qk["rows"], qk["cols"]
    packed = qk["kernel"].numpy()
    scale = qk["kernel_scale"].double().numpy()
    zero = None if qk["kernel_zero"] is None else qk["kernel_zero"].numpy()
    flat = np.zeros((rows, cols), np.float64)
    for r in range(rows):
        for c in range(cols):
            v = _nibble(packed[r, c // 2], c % 2 == 1)
            if block_size in (None, -1):
                flat[r, c] = v / scale[c]
            else:
                gi = r // block_size
                flat[r, c] = (v - int(zero[gi, c])) * scale[gi, c]
    out = np.zeros(qk["original_kernel_shape"], np.float64)
    for i in range(rows * cols):
        out[np.unravel_index(i, out.shape)] = flat[i // cols, i % cols]
    return out


EINSUM_INT4_CASES = [
    ("btd,dnh->btnh", (16, 3, 6), (2, 3, 16)),      # contracted axis leads: flat = true [K, N]
    ("btnh,nhd->btd", (2, 8, 10), (2, 3, 2, 8)),    # two contracted axes lead
    ("ab,bcd->acd", (16, 3, 4), (5, 16)),
    ("btd,ndh->btnh", (3, 16, 6), (2, 2, 16)),      # contracted axis in the middle: the reshape mixes
    ("abc,cd->abd", (16, 7), (2, 3, 16)),           # odd column count: half-filled last byte
]


@pytest.mark.parametrize("equation,kshape,xshape", EINSUM_INT4_CASES)
@pytest.mark.parametrize("block_size", [None, 8])
def test_einsum_dense_int4_call_by_loops(equation, kshape, xshape, block_size):
    g = torch.Generator().manual_seed(23)
    kernel = torch.rand(kshape, generator=g) - 0.5
    x = torch.randn(xshape, generator=g)
    bias_shape = torch.einsum(equation, x, kernel).shape[-1:]
    bias = torch.randn(bias_shape, generator=g) * 0.1
    qk = ref.einsum_dense_quantize_int4(kernel, equation, len(xshape), block_size)
    # rows = product of the kernel axes the output lacks, columns = the rest
    lhs, out = equation.split("->")
    kspec = lhs.split(",")[1]
    rows = int(np.prod([d for c, d in zip(kspec, kshape) if c not in out]))
    assert qk["rows"] == rows and qk["rows"] * qk["cols"] == int(np.prod(kshape))
    assert tuple(qk["kernel"].shape) == (rows, (qk["cols"] + 1) // 2)
    w64 = _einsum_int4_kernel_by_loops(qk, block_size)
    want = np.einsum(equation, x.double().numpy(), w64) + bias.double().numpy()
    y = ref.einsum_dense_int4_call(x, qk, equation, bias=bias, block_size=block_size)
    assert y.dtype == torch.float32 and tuple(y.shape) == want.shape
    assert np.abs(y.double().numpy() - want).max() / np.abs(want).max() < 1e-5
    # the de-quantised kernel is the float kernel to within half a step of the column's scale
    # (grouped: one step of the group's, the value and the zero point being rounded separately),
    # so a scale applied to the wrong axis fails here
    if block_size is None:
        bound = 0.5001 * (1.0 / qk["kernel_scale"].double().numpy())[None, :]
    else:
        bound = 1.0001 * np.repeat(qk["kernel_scale"].double().numpy(), block_size, axis=0)[:rows]
    flat_err = np.abs(w64.reshape(rows, qk["cols"]) - kernel.double().numpy().reshape(rows, qk["cols"]))
    assert (flat_err <= bound + 1e-7).all()
    # bfloat16 compute: same quantity within the bfloat16 bound
    yb = ref.einsum_dense_int4_call(x, qk, equation, bias=bias, compute_dtype="bfloat16", block_size=block_size)
    assert yb.dtype == torch.bfloat16
    assert np.abs(yb.double().numpy() - want).max() / np.abs(want).max() < 2e-2


@pytest.mark.parametrize("compute_dtype,tol", [("float32", 1e-5), ("bfloat16", 2e-2)])
def test_dense_lora_term_is_two_matmuls(compute_dtype, tol):
    g = torch.Generator().manual_seed(29)
    x = torch.randn(5, 24, generator=g)
    a = torch.randn(24, 4, generator=g) * 0.3
    b = torch.randn(4, 9, generator=g) * 0.3
    got = ref.dense_lora_term(x, a, b, alpha=8.0, rank=4, compute_dtype=compute_dtype)
    want = np.zeros((5, 9))
    xa = np.zeros((5, 4))
    for m in range(5):
        for r in range(4):
            xa[m, r] = sum(float(x[m, k]) * float(a[k, r]) for k in range(24))
    for m in range(5):
        for n in range(9):
            want[m, n] = (8.0 / 4) * sum(xa[m, r] * float(b[r, n]) for r in range(4))
    assert tuple(got.shape) == (5, 9) and got.dtype == getattr(torch, compute_dtype)
    assert np.abs(got.double().numpy() - want).max() / np.abs(want).max() < tol
    # alpha / rank is the only scaling: doubling alpha doubles the term, a zero b removes it
    twice = ref.dense_lora_term(x, a, b, alpha=16.0, rank=4, compute_dtype=compute_dtype)
    assert torch.equal(twice, 2 * got)
    assert ref.dense_lora_term(x, a, torch.zeros(4, 9), 8.0, 4, compute_dtype).abs().max().item() == 0


def _einsum_int8_dequant_by_loops(equation, q, s):
    """float64 q / scale with the stored scale indexed by hand: the stored scale broadcasts
    against the OUTPUT labels (size 1 where the kernel lacks the label), einsum_dense.py:1449-1491."""
    lhs, out = equation.split("->")
    kspec = lhs.split(",")[1]
    s = s.double().numpy()
    assert s.ndim == len(out), (s.shape, out)
    w = np.zeros(tuple(q.shape), np.float64)
    for idx in np.ndindex(*q.shape):
        pos = dict(zip(kspec, idx))
        sidx = tuple(pos[c] if (c in kspec and s.shape[i] != 1) else 0 for i, c in enumerate(out))
        w[idx] = float(q[idx]) / s[sidx]
    return w


@pytest.mark.parametrize("equation,kshape,rank_in,ab_shapes", [
    ("btd,dnh->btnh", (12, 3, 4), 3, ((12, 2), (2, 3, 4))),
    ("btnh,nhd->btd", (3, 4, 10), 4, ((3, 4, 2), (2, 10))),
    ("abcde,afce->acdbf", (1, 6, 2, 8), 5, ((1, 6, 2, 2), (2, 8))),
    ("ab,bcd->acd", (8, 3, 4), 2, ((8, 2), (2, 3, 4))),
])
def test_einsum_merged_lora_kernel_int8(equation, kshape, rank_in, ab_shapes):
    # lora_kernel_a has the kernel's shape up to its last axis + [rank], lora_kernel_b is
    # [rank, last axis] (einsum_dense.py:327-360); matmul(a, b) therefore has the kernel's shape
    g = torch.Generator().manual_seed(31)
    kernel = torch.rand(kshape, generator=g) - 0.5
    qk, ks, info = ref.einsum_dense_quantize_int8(kernel, equation, rank_in)
    rank = 2
    a = torch.randn(kshape[:-1] + (rank,), generator=g) * 0.05
    b0 = torch.zeros(rank, kshape[-1])
    q0, s0, z0 = ref.einsum_dense_merged_lora_kernel("int8", qk, ks, a, b0, 4.0, rank, equation, rank_in)
    assert z0 is None and torch.equal(q0, qk) and tuple(s0.shape) == tuple(ks.shape)
    assert torch.allclose(s0, ks, rtol=1e-5, atol=0)
    b = torch.randn(rank, kshape[-1], generator=g) * 0.05
    q1, s1, _ = ref.einsum_dense_merged_lora_kernel("int8", qk, ks, a, b, 4.0, rank, equation, rank_in)
    assert tuple(s1.shape) == tuple(ks.shape) and not torch.equal(q1, qk)
    old = _einsum_int8_dequant_by_loops(equation, qk, ks)
    new = _einsum_int8_dequant_by_loops(equation, q1, s1)
    update = (4.0 / rank) * np.matmul(a.double().numpy(), b.double().numpy())
    step = np.abs(new / np.where(q1.numpy() == 0, 1, q1.numpy()))  # |1 / scale| wherever q != 0
    step = np.where(q1.numpy() == 0, step.max(), step)
    assert (np.abs(new - (old + update)) <= 0.5001 * step + 1e-6).all()


@pytest.mark.parametrize("equation,kshape,rank_in", [
    ("btd,dnh->btnh", (16, 3, 4), 3), ("btnh,nhd->btd", (2, 8, 10), 4), ("btd,ndh->btnh", (3, 16, 4), 3),
])
@pytest.mark.parametrize("block_size", [None, 8])
def test_einsum_merged_lora_kernel_int4(equation, kshape, rank_in, block_size):
    g = torch.Generator().manual_seed(37)
    kernel = torch.rand(kshape, generator=g) - 0.5
    qk = ref.einsum_dense_quantize_int4(kernel, equation, rank_in, block_size)
    rank = 2
    a = torch.randn(kshape[:-1] + (rank,), generator=g) * 0.3
    old = _einsum_int4_kernel_by_loops(qk, block_size)
    q0, s0, z0 = ref.einsum_dense_merged_lora_kernel(
        "int4", None, None, a, torch.zeros(rank, kshape[-1]), 4.0, rank, equation, rank_in,
        qk=qk, block_size=block_size)
    assert tuple(q0.shape) == tuple(qk["kernel"].shape) and q0.dtype == torch.int8
    if block_size is None:
        assert z0 is None and torch.equal(q0, qk["kernel"])
        assert torch.allclose(s0, qk["kernel_scale"], rtol=1e-5, atol=0)
    b = torch.randn(rank, kshape[-1], generator=g) * 0.3
    q1, s1, z1 = ref.einsum_dense_merged_lora_kernel("int4", None, None, a, b, 4.0, rank, equation, rank_in,
                                                     qk=qk, block_size=block_size)
    merged = dict(qk, kernel=q1, kernel_scale=s1, kernel_zero=z1)
    new = _einsum_int4_kernel_by_loops(merged, block_size)
    update = (4.0 / rank) * np.matmul(a.double().numpy(), b.double().numpy())
    rows, cols = qk["rows"], qk["cols"]
    if block_size is None:
        bound = 0.5001 * (1.0 / s1.double().numpy())[None, :]
    else:
        bound = 1.0001 * np.repeat(s1.double().numpy(), block_size, axis=0)[:rows]
    target = (old + update).reshape(rows, cols)
    err = np.abs(new.reshape(rows, cols) - target)
    if block_size is not None:
        # the zero point is clipped to the int4 range, so a group whose values do not straddle
        # zero is not representable within a step (quantizers.py:210-222): leave those out
        grp = target.reshape(rows // block_size, block_size, cols)
        straddles = (grp.min(axis=1) <= 0) & (grp.max(axis=1) >= 0)
        assert straddles.mean() > 0.5
        err = np.where(np.repeat(straddles, block_size, axis=0), err, 0.0)
    assert (err <= bound + 1e-6).all()
    assert not torch.equal(q1, qk["kernel"])


@pytest.mark.parametrize("mode,block_size", [("int8", None), ("int4", None), ("int4", 8)])
def test_embedding_merged_lora_table(mode, block_size):
    g = torch.Generator().manual_seed(41)
    V, D, rank, alpha = 11, 24, 3, 6.0
    table = torch.randn(V, D, generator=g) * 0.2
    a = torch.randn(V, rank, generator=g) * 0.3
    if mode == "int8":
        q, s = ref.embedding_quantize_int8(table)
        zero = g_idx = None
        kw = dict()
    else:
        e = ref.embedding_quantize_int4(table, block_size)
        q, s, zero, g_idx = e["embeddings"], e["embeddings_scale"], e["embeddings_zero"], e["g_idx"]
        kw = dict(embeddings_zero=zero, g_idx=g_idx, block_size=block_size, orig_output_dim=D)

    def dequant(q, s, z):
        """float64 table by loops: row v, column d; int4 byte [v, d // 2], even d low nibble;
        per-row scale divides, grouped (groups along d) scale multiplies (embedding.py:726-752)."""
        out = np.zeros((V, D))
        for v in range(V):
            for d in range(D):
                val = int(q[v, d]) if mode == "int8" else _nibble(q[v, d // 2], d % 2 == 1)
                if block_size is None:
                    out[v, d] = val / float(s[v])
                else:
                    out[v, d] = (val - int(z[v, d // block_size])) * float(s[v, d // block_size])
        return out

    q0, s0, z0 = ref.embedding_merged_lora_table(mode, q, s, a, torch.zeros(rank, D), alpha, rank, **kw)
    assert tuple(q0.shape) == tuple(q.shape) and q0.dtype == torch.int8 and tuple(s0.shape) == tuple(s.shape)
    if block_size is None:
        assert z0 is None and torch.equal(q0, q) and torch.allclose(s0, s, rtol=1e-5, atol=0)
    else:
        assert tuple(z0.shape) == tuple(zero.shape) and z0.dtype == torch.int8
    b = torch.randn(rank, D, generator=g) * 0.3
    q1, s1, z1 = ref.embedding_merged_lora_table(mode, q, s, a, b, alpha, rank, **kw)
    target = dequant(q, s, zero) + (alpha / rank) * (a.double().numpy() @ b.double().numpy())
    got = dequant(q1, s1, z1)
    if block_size is None:
        bound = 0.5001 * (1.0 / s1.double().numpy())[:, None]
    else:
        bound = 1.0001 * np.repeat(s1.double().numpy(), block_size, axis=1)[:, :D]
    err = np.abs(got - target)
    if block_size is not None:
        grp = target.reshape(V, D // block_size, block_size)
        straddles = (grp.min(axis=2) <= 0) & (grp.max(axis=2) >= 0)
        assert straddles.mean() > 0.5
        err = np.where(np.repeat(straddles, block_size, axis=1), err, 0.0)
    assert (err <= bound + 1e-6).all()
    assert not torch.equal(q1, q)
