"""GPU parity: the strip-linear int4 decode route (k3q_w4s_pack, k3q_gemv_w4s) against the CPU
oracle, the float64 value and the route over the stored kernel."""

import pytest
import torch

from keras_amd import _lib, ops as kops
from oracle import keras_cpu_path as ref
from tests.helpers import RTOL, c_w4_matmul_f64, max_rel_err
from tests.test_gpu_int4_matmul import make_layer

pytestmark = pytest.mark.gpu


def strip_operands(dev, qk, K, N, block_size):
    grouped = block_size is not None and block_size > 0
    kernel = qk["kernel"].to(dev)
    shadow = kops.int4_strip_copy(kernel, N)
    scale = qk["kernel_scale"].to(torch.bfloat16).to(dev)
    gparams = kops.int4_strip_params(scale, qk["kernel_zero"].to(dev), K, N, block_size) if grouped else None
    return kernel, shadow, scale, gparams


def test_strip_copy_layout(dev):
    # every nibble of the copy against the layout the header states, from a kernel of known values
    K, N = 256, 48  # three strips: the copy is padded to four
    g = torch.Generator().manual_seed(0)
    q = torch.randint(-8, 8, (K, N), generator=g, dtype=torch.int8)
    packed, _, _ = ref.pack_int4(q.numpy(), axis=-1) if hasattr(ref, "pack_int4") else (None, None, None)
    from keras_amd import quantizers
    packed = quantizers.pack_int4(q.to(dev), axis=-1)[0]
    shadow = kops.int4_strip_copy(packed, N).cpu().view(torch.int32).reshape(4, K // 128, 64, 4)
    for strip in range(4):
        for unit in range(K // 128):
            for lane in (0, 5, 17, 63):
                i, gq = lane & 15, lane >> 4
                for s in range(4):
                    d = int(shadow[strip, unit, lane, s]) & 0xFFFFFFFF
                    for e in range(8):
                        k = 128 * unit + 32 * s + 8 * gq + e
                        n = 16 * strip + i
                        want = (int(q[k, n]) & 0xF) if n < N else 0
                        bit = 16 + 4 * (e >> 1) if e & 1 else 4 * (e >> 1)
                        assert (d >> bit) & 0xF == want, (strip, unit, lane, s, e)


def run_strip_case(dev, M, K, N, block_size, with_bias, seed=0):
    qk, bias = make_layer(K, N, block_size, seed, with_bias)
    g = torch.Generator().manual_seed(seed + 1)
    x = torch.randn(M, K, generator=g).to(torch.bfloat16)
    grouped = block_size is not None and block_size > 0
    dt = torch.bfloat16
    want = ref.dense_int4_call(x, qk["kernel"], qk["kernel_scale"], N, kernel_zero=qk["kernel_zero"],
                               g_idx=qk["g_idx"], block_size=block_size, bias=bias, compute_dtype=dt)
    assert kops.int4_strip_supported(M, K, N, block_size)
    kernel, shadow, scale, gparams = strip_operands(dev, qk, K, N, block_size)
    bias_t = bias.to(dt).to(dev) if bias is not None else None
    got = kops.int4_matmul_strip(x.to(dev), shadow, N, kernel_scale=None if grouped else scale,
                                 gparams=gparams, block_size=block_size, bias=bias_t)
    torch.cuda.synchronize()
    assert got.dtype == dt and tuple(got.shape) == (M, N)
    exact = c_w4_matmul_f64(x, qk["kernel"], scale.cpu(), qk["kernel_zero"], block_size,
                            bias_t.cpu() if bias is not None else None, N)
    e_ref, e_exact, e_ref_exact = max_rel_err(got, want), max_rel_err(got, exact), max_rel_err(want, exact)
    tol = RTOL[dt]
    assert e_ref <= tol, (e_ref, e_exact, e_ref_exact)  # the stated bound, unconditionally
    assert e_exact <= max(2.0 * e_ref_exact, tol / 4), (e_exact, e_ref_exact)
    other = kops.int4_matmul(x.to(dev), kernel, scale, N,
                             kernel_zero=qk["kernel_zero"].to(dev) if grouped else None,
                             block_size=block_size, bias=bias_t)
    assert max_rel_err(got, other) <= tol
    return got


@pytest.mark.parametrize("M", [1, 4, 8, 9, 16])
@pytest.mark.parametrize("block_size", [None, 128])
def test_strip_decode_config(dev, M, block_size):
    # target configuration 2: K = N = 8192 (above 8 rows x is staged in two parts)
    run_strip_case(dev, M, 8192, 8192, block_size, with_bias=False)


@pytest.mark.parametrize("M,K,N,block_size", [
    (1, 4096, 4096, 128), (3, 4096, 14336, 128), (2, 14336, 4096, 128), (1, 4096, 32000, 128),
    (8, 4096, 4096, None), (5, 4096, 3072, 128), (1, 5120, 5120, None), (7, 8192, 3088, 128),
    (1, 28672, 4096, None), (4, 5120, 13824, 128), (2, 6144, 6144, None),
    (16, 4096, 4096, 128), (12, 4096, 14336, None), (16, 8192, 4096, 128), (10, 12288, 3072, None),
    (16, 8192, 8192, None), (16, 8192, 4096, 128),
    # x staged in two unequal parts (a slice of 7 or 5 rounds of the ring)
    (8, 14336, 4096, 128), (8, 14336, 4096, None), (5, 14336, 4096, 128), (7, 14336, 3584, None),
    (9, 10240, 4096, 128), (10, 10240, 8192, None), (16, 6144, 4096, 128), (12, 8192, 8192, 128),
])
def test_strip_shapes(dev, M, K, N, block_size):
    run_strip_case(dev, M, K, N, block_size, with_bias=(M % 2 == 1), seed=M)


def test_strip_rejects_what_it_does_not_take(dev):
    for M, K, N, bs in [(17, 4096, 4096, None), (16, 14336, 4096, 128), (9, 8192, 16384, None), (1, 4096, 4096, 64),
                        (16, 4096, 32000, 128), (1, 4000, 4096, None),
                        (1, 4096, 1024, None), (1, 4096, 4104, None), (9, 14336, 4096, 128),
                        (1, 1024, 4096, None), (1, 128 * 33, 4096, None), (1, 2048, 4096, None)]:
        assert not kops.int4_strip_supported(M, K, N, bs), (M, K, N, bs)
    lib = _lib.load()
    one = torch.zeros(64, dtype=torch.uint8, device=dev)
    p, s = _lib.ptr(one), _lib.stream_ptr(dev)
    assert lib.k3q_gemv_w4s(p, 1, 17, 4096, 4096, p, p, None, -1, None, 0, p, s) == -2
    assert lib.k3q_gemv_w4s(p, 0, 1, 4096, 4096, p, p, None, -1, None, 0, p, s) == -4
    assert lib.k3q_gemv_w4s(p, 1, 1, 4096, 4096, p, None, None, -1, None, 0, p, s) == -1
    assert lib.k3q_gemv_w4s(p, 1, 1, 4096, 4096, p, p, None, -1, p, 7, p, s) == -2
    assert lib.k3q_w4s_shadow_bytes(4096, 4096) == 4096 * 4096 // 2
    assert lib.k3q_w4s_shadow_bytes(4096, 48) == 4 * 32 * 1024


def test_strip_addend_is_the_add_after(dev):
    K, N, M = 4096, 4096, 8
    for bs in (None, 128):
        qk, _ = make_layer(K, N, bs, 70, False)
        g = torch.Generator().manual_seed(71)
        x = torch.randn(M, K, generator=g).to(torch.bfloat16).to(dev)
        res = torch.randn(M, N, generator=g).to(torch.bfloat16).to(dev)
        grouped = bs is not None
        _, shadow, scale, gparams = strip_operands(dev, qk, K, N, bs)
        kw = dict(kernel_scale=None if grouped else scale, gparams=gparams, block_size=bs)
        want = res + kops.int4_matmul_strip(x, shadow, N, **kw)
        got = kops.int4_matmul_strip(x, shadow, N, addend=res, **kw)
        assert torch.equal(got.view(torch.int16), want.view(torch.int16))


@pytest.mark.parametrize("M", [1, 8])
@pytest.mark.parametrize("block_size", [None, 128])
def test_strip_multi_matches_single_calls(dev, M, block_size):
    # several kernels against one x in one launch: every workgroup computes what it computes in a
    # single call, so the bits are the single calls' bits
    K = 4096
    widths = [4096, 4096, 4096, 14336, 3072]
    x = torch.randn(M, K, generator=torch.Generator().manual_seed(M)).to(torch.bfloat16).to(dev)
    kernels, singles = [], []
    grouped = block_size is not None
    for i, N in enumerate(widths):
        qk, bias = make_layer(K, N, block_size, 60 + i, i % 2 == 0)
        _, shadow, scale, gparams = strip_operands(dev, qk, K, N, block_size)
        spec = dict(shadow=shadow, units=N, kernel_scale=None if grouped else scale, gparams=gparams,
                    bias=bias.to(torch.bfloat16).to(dev) if bias is not None else None)
        kernels.append(spec)
        singles.append(kops.int4_matmul_strip(x, shadow, N, kernel_scale=spec["kernel_scale"], gparams=gparams,
                                              block_size=block_size, bias=spec["bias"]))
    for base, end in ((0, 3), (0, 5), (3, 5)):
        got = kops.int4_matmul_strip_multi(x, kernels[base:end], block_size=block_size)
        for jdx, y in enumerate(got):
            assert torch.equal(y.view(torch.int16), singles[base + jdx].view(torch.int16)), (base, jdx)


def test_strip_repeatable(dev):
    qk, _ = make_layer(4096, 4096, 128, 3, False)
    x = torch.randn(4, 4096).to(torch.bfloat16).to(dev)
    _, shadow, scale, gparams = strip_operands(dev, qk, 4096, 4096, 128)
    first = kops.int4_matmul_strip(x, shadow, 4096, gparams=gparams, block_size=128)
    for _ in range(5):
        assert torch.equal(first, kops.int4_matmul_strip(x, shadow, 4096, gparams=gparams, block_size=128))
