"""GPU parity: int8 GEMM + de-scale epilogue (k3q_gemm_i8) against the CPU oracle."""

import pytest
import torch

from keras_amd import ops as kops
from keras_amd import quantizers as kq
from oracle import keras_cpu_path as ref
from tests.helpers import RTOL, c_gemm_i8, max_rel_err

pytestmark = pytest.mark.gpu


def make_case(M, K, N, dtype, seed, with_bias=True):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(M, K, generator=g).to(dtype)
    kernel = ref.glorot_uniform(K, N, generator=g)
    bias = (torch.randn(N, generator=g) * 0.02) if with_bias else None
    qkernel, kscale = ref.dense_quantize_int8(kernel)
    return x, qkernel, kscale, bias


def run_dense_int8(dev, M, K, N, dtype, prepack, exact, seed=0, with_bias=True, row_gain=None):
    x, qk, ks, bias = make_case(M, K, N, dtype, seed, with_bias)
    if row_gain is not None:
        x = (x.float() * row_gain[:, None]).to(dtype)
    want, inter = ref.dense_int8_call(x, qk, ks, bias, compute_dtype=dtype, return_intermediates=True)
    q, s = kq.abs_max_quantize(x.to(dev), axis=-1)
    assert torch.equal(q.cpu(), inter["q"])
    qk_d = qk.to(dev)
    # prepack: True = the [N, K] copy, "strip" = the decode kernel's strip-linear copy as the tiles'
    # operand (K % 128 == 0; other shapes fall back to the stored kernel), False = the stored kernel
    pre = kops.prepack_int8_kernel(qk_d) if prepack is True else None
    strip = kops.int8_strip_copy(qk_d) if prepack == "strip" and K % 64 == 0 else None
    y, acc = kops.int8_matmul(
        q, qk_d, a_scale=s, kernel_scale=ks.to(dtype).to(dev),
        bias=bias.to(dtype).to(dev) if bias is not None else None, out_dtype=dtype,
        prepacked=pre, strip=strip, exact_epilogue=exact, want_acc=True)
    torch.cuda.synchronize()
    assert torch.equal(acc.cpu(), inter["acc"]), "int32 accumulators differ from the reference"
    if exact:
        # same op chain, same rounding points: bit-identical
        assert torch.equal(y.cpu().view(torch.int16 if dtype == torch.bfloat16 else torch.int32),
                           want.view(torch.int16 if dtype == torch.bfloat16 else torch.int32))
    else:
        # the opt-in fast epilogue rounds once where the reference's chain rounds four times:
        # in bfloat16 the two can sit two ulps (2^-7 each) apart on the largest outputs
        e = max_rel_err(y, want)
        assert e <= RTOL[dtype] * (2 if dtype == torch.bfloat16 else 1), e
    return y


SHAPES = [
    (1, 128, 4), (3, 128, 12), (16, 4096, 4096), (17, 256, 260), (64, 512, 1000),
    (255, 384, 256), (256, 1024, 512), (300, 640, 772), (513, 256, 1028),
    # N % 4 != 0 (a vocabulary of 50257 or 30522): the tiles store those rows element-wise
    (300, 256, 1001), (129, 384, 50257), (64, 128, 30522), (200, 512, 3), (1000, 128, 130),
    # K % 128 != 0: operands zero-padded into scratch, then the tiles (model widths 1600, 960;
    # odd and unaligned K; with a K split; N % 4 != 0 as well)
    (5, 100, 30), (8, 8, 16), (33, 64, 7), (2, 200, 64), (300, 1600, 640), (64, 960, 1280),
    (130, 6400, 1600), (77, 333, 129), (40, 72, 264), (1100, 200, 1001),
]


@pytest.mark.parametrize("M,K,N", SHAPES)
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("prepack", [True, False, "strip"])
def test_dense_int8_exact_epilogue(dev, M, K, N, dtype, prepack):
    run_dense_int8(dev, M, K, N, dtype, prepack, exact=True)


@pytest.mark.parametrize("M,K,N", [(16, 4096, 4096), (300, 640, 772), (512, 4096, 4096)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_dense_int8_fast_epilogue(dev, M, K, N, dtype):
    run_dense_int8(dev, M, K, N, dtype, prepack=True, exact=False)


@pytest.mark.parametrize("M,K,N", [(300, 640, 772), (16, 512, 256), (513, 256, 1028)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_dense_int8_wide_range_scales(dev, M, K, N, dtype):
    # rows of x spread over 60 decades: input scales from 1e-28 to 1e32, so the de-scale
    # divides by very small and very large numbers (the bfloat16 epilogue switches from the
    # reciprocal to the IEEE division per tile) and some outputs are tiny
    gains = torch.tensor([1e-30, 1e-12, 1e-3, 1.0, 1e5, 1e12, 1e30])
    row_gain = gains[torch.arange(M) % len(gains)]
    run_dense_int8(dev, M, K, N, dtype, prepack=True, exact=True, row_gain=row_gain)
    # one well-scaled block of rows next to the rest: tiles of both kinds in one call
    row_gain = torch.ones(M)
    row_gain[M // 2:] = gains[torch.arange(M - M // 2) % len(gains)]
    run_dense_int8(dev, M, K, N, dtype, prepack=True, exact=True, row_gain=row_gain, seed=3)


# few tiles and a long K: the tile kernel splits K over workgroups and a second kernel sums
# the int32 partials and applies the epilogue; the result must not change by a bit
@pytest.mark.parametrize("M,K,N", [(128, 4096, 4096), (130, 8192, 1028), (256, 14336, 512),
                                   (384, 8192, 2048), (200, 4096, 260)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_dense_int8_split_k(dev, M, K, N, dtype):
    run_dense_int8(dev, M, K, N, dtype, prepack=True, exact=True)
    run_dense_int8(dev, M, K, N, dtype, prepack="strip", exact=True, seed=4)
    run_dense_int8(dev, M, K, N, dtype, prepack=False, exact=True, seed=5, with_bias=False)
    run_dense_int8(dev, M, K, N, dtype, prepack=True, exact=False, seed=6)


def test_config1_dense_4096(dev):
    # target configuration 1: Dense(4096) on [16, 4096] float32 inputs, bias, seed 0
    run_dense_int8(dev, 16, 4096, 4096, torch.float32, prepack=True, exact=True, seed=0)


def test_gemm_extreme_values(dev):
    # +-127 everywhere: |acc| = K * 127 * 127 must not overflow or saturate
    K = 14336
    a = torch.full((130, K), 127, dtype=torch.int8)
    a[::2] = -127
    b = torch.full((K, 260), -127, dtype=torch.int8)
    acc = kops.int8_matmul(a.to(dev), b.to(dev), want_acc=True, want_y=False,
                           prepacked=kops.prepack_int8_kernel(b.to(dev)))
    want = torch.matmul(a.to(torch.int32), b.to(torch.int32))
    assert torch.equal(acc.cpu(), want)
    assert want.abs().max().item() == K * 127 * 127


@pytest.mark.parametrize("M,K,N", [(4096, 8192, 8192), (2048, 4096, 4096), (512, 8192, 28672),
                                   (8192, 8192, 8192), (2048, 8192, 28672), (8192, 8192, 28672),
                                   (8192, 4096, 4096)])
def test_gemm_full_size_accumulators(dev, M, K, N):
    # full target sizes: sampled rows against the CPU oracle (bit-exact) plus two
    # size-independent integer identities over the whole output
    g = torch.Generator().manual_seed(7)
    a = torch.randint(-127, 128, (M, K), generator=g, dtype=torch.int8)
    b = torch.randint(-127, 128, (K, N), generator=g, dtype=torch.int8)
    a_d, b_d = a.to(dev), b.to(dev)
    acc = kops.int8_matmul(a_d, b_d, want_acc=True, want_y=False,
                           prepacked=kops.prepack_int8_kernel(b_d))
    rows = torch.randint(0, M, (24,), generator=g)
    want_rows = c_gemm_i8(a[rows], b)
    assert torch.equal(acc[rows.to(dev)].cpu(), want_rows)
    # sum over rows of acc == (column sums of a) . b ; sum over columns == a . (row sums of b)
    colsum_a = a.to(torch.int64).sum(0)
    rowsum_b = b.to(torch.int64).sum(1)
    assert torch.equal(acc.to(torch.int64).sum(0).cpu(), colsum_a @ b.to(torch.int64))
    assert torch.equal(acc.to(torch.int64).sum(1).cpu(), a.to(torch.int64) @ rowsum_b)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_dense_int8_full_size_rows_bit_exact(dev, dtype):
    # the benchmark configuration end to end (quantize + GEMM + de-scale + bias); every row of
    # the layer is independent of the others, so sampled rows are checked against the oracle
    # run on those rows alone, bit for bit
    M, K, N = 4096, 8192, 8192
    g = torch.Generator().manual_seed(11)
    x = torch.randn(M, K, generator=g).to(dtype)
    kernel = ref.glorot_uniform(K, N, generator=g)
    bias = torch.randn(N, generator=g) * 0.02
    qk, ks = ref.dense_quantize_int8(kernel)
    q, s = kq.abs_max_quantize(x.to(dev), axis=-1)
    qk_d = qk.to(dev)
    y = kops.int8_matmul(q, qk_d, a_scale=s, kernel_scale=ks.to(dtype).to(dev),
                         bias=bias.to(dtype).to(dev), out_dtype=dtype,
                         prepacked=kops.prepack_int8_kernel(qk_d), exact_epilogue=True)
    rows = torch.cat([torch.tensor([0, 255, 256, M - 1]), torch.randint(0, M, (28,), generator=g)])
    want = ref.dense_int8_call(x[rows], qk, ks, bias, compute_dtype=dtype)
    bits = torch.int16 if dtype == torch.bfloat16 else torch.int32
    assert torch.equal(y[rows.to(dev)].cpu().view(bits), want.view(bits))


def test_prepack_is_transpose(dev):
    g = torch.Generator().manual_seed(1)
    for K, N in [(128, 64), (100, 37), (4096, 4096), (65, 129)]:
        b = torch.randint(-128, 128, (K, N), generator=g, dtype=torch.int8)
        assert torch.equal(kops.prepack_int8_kernel(b.to(dev)).cpu(), b.t().contiguous())


DECODE_SHAPES = [(1, 4096, 4096), (8, 4096, 4096), (16, 4096, 4096), (3, 64, 48), (17, 512, 1040),
                 (33, 256, 512), (64, 1024, 2048), (5, 8, 16), (12, 14336, 4096), (2, 4096, 14336)]


@pytest.mark.parametrize("M,K,N", DECODE_SHAPES)
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_dense_int8_decode_sizes(dev, M, K, N, dtype):
    # M <= 64 without a prepacked kernel: the bandwidth-bound kernel that reads [K, N] in place
    y = run_dense_int8(dev, M, K, N, dtype, prepack=False, exact=True, seed=M + K)
    # and the layer-level route (prepacked given, still routed by M) agrees bit for bit
    y2 = run_dense_int8(dev, M, K, N, dtype, prepack=True, exact=True, seed=M + K)
    assert torch.equal(y, y2)


@pytest.mark.parametrize("M,K,N", [(2, 4096, 4096), (8, 4096, 4096), (8, 14336, 4096), (5, 64, 48),
                                   (3, 512, 1040), (8, 8, 16)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_int8_addend_is_the_add_after(dev, M, K, N, dtype):
    # an [M, N] addend (a residual) in the decode kernel's epilogue, where a bias would be
    # added: the bits of `addend + int8_matmul(...)`, with and without a K split
    x, qk, ks, _ = make_case(M, K, N, dtype, seed=M + N, with_bias=False)
    res = torch.randn(M, N, generator=torch.Generator().manual_seed(5)).to(dtype).to(dev)
    q, s = kq.abs_max_quantize(x.to(dev), axis=-1)
    args = dict(a_scale=s, kernel_scale=ks.to(dtype).to(dev), out_dtype=dtype, exact_epilogue=True)
    want = res + kops.int8_matmul(q, qk.to(dev), **args)
    keep = res.clone()
    got = kops.int8_matmul(q, qk.to(dev), bias=res, **args)
    bits = torch.int16 if dtype == torch.bfloat16 else torch.int32
    assert torch.equal(got.view(bits), want.view(bits))
    assert torch.equal(res, keep)
    with pytest.raises(ValueError):
        kops.int8_matmul(q, qk.to(dev), bias=res, want_acc=True, **args)
