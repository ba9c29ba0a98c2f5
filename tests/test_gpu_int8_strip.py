"""GPU: the one-launch int8 Dense forward for decode sizes (quantizer + exact int8 matmul +
bit-exact bfloat16 de-scale from the strip-linear copy of the kernel) against the oracle and
against the two-launch route it replaces."""

import pytest
import torch

from keras_amd import ops as kops, quantizers as kq
from oracle import keras_cpu_path as ref

pytestmark = pytest.mark.gpu

bits = lambda t: t.contiguous().view(torch.int16)


@pytest.mark.parametrize("K,N", [(64, 16), (128, 48), (256, 40), (1024, 3072)])
def test_strip_copy_layout(dev, K, N):
    # [strip = n/16][unit = k/64][lane][16 bytes]: lane i + 16 g holds column 16 strip + i, bytes
    # k = 64 unit + 16 g + (0..15); strips padded to even with zeros
    g = torch.Generator().manual_seed(K + N)
    w = torch.randint(-128, 128, (K, N), generator=g, dtype=torch.int8)
    got = kops.int8_strip_copy(w.to(dev)).cpu().view(torch.int8)
    strips = ((N + 15) // 16 + 1) // 2 * 2
    assert got.numel() == strips * (K // 64) * 1024
    got = got.reshape(strips, K // 64, 4, 16, 16)  # strip, unit, g, i, byte
    want = torch.zeros(strips * 16, K, dtype=torch.int8)
    want[:N] = w.t()
    want = want.reshape(strips, 16, K // 64, 4, 16).permute(0, 2, 3, 1, 4)
    assert torch.equal(got, want)


def run_case(dev, M, K, N, with_bias, addend=False, epsilon=1e-7, value_range=(-127, 127), seed=0):
    g = torch.Generator().manual_seed(seed + M + K + N)
    x = (torch.randn(M, K, generator=g) * 3).to(torch.bfloat16)
    if M > 1:
        x[1] = 0  # an all-zero row: scale 127 / eps
    kernel = ref.glorot_uniform(K, N, generator=g)
    qk, ks = ref.dense_quantize_int8(kernel)
    bias = None
    if addend:
        bias = torch.randn(M, N, generator=g).to(torch.bfloat16)
    elif with_bias:
        bias = (torch.randn(N, generator=g) * 0.1).to(torch.bfloat16)
    qk_d, ks_d = qk.to(dev), ks.to(torch.bfloat16).to(dev)
    assert kops.int8_strip_supported(M, K, N)
    shadow = kops.int8_strip_copy(qk_d)
    y = kops.int8_dense_strip(x.to(dev), shadow, N, ks_d, bias=bias.to(dev) if bias is not None else None,
                              epsilon=epsilon, value_range=value_range)
    assert y.dtype == torch.bfloat16 and tuple(y.shape) == (M, N)
    # the two-launch route: quantizer kernel, then the GEMM family with the bit-exact epilogue
    q, s = kq.abs_max_quantize(x.to(dev), axis=-1, value_range=value_range, epsilon=epsilon)
    late = addend and M > 8  # (the two-launch route takes a row of addends per row up to 8 rows)
    two = kops.int8_matmul(q, qk_d, a_scale=s, kernel_scale=ks_d,
                           bias=bias.to(dev) if bias is not None and not late else None,
                           out_dtype=torch.bfloat16, exact_epilogue=True)
    if late:
        two = two + bias.to(dev)
    assert torch.equal(bits(y), bits(two))
    if epsilon == 1e-7 and value_range == (-127, 127):
        if addend:
            want = ref.dense_int8_call(x, qk, ks, None, compute_dtype=torch.bfloat16) + bias
        else:
            want = ref.dense_int8_call(x, qk, ks, bias.float() if bias is not None else None,
                                       compute_dtype=torch.bfloat16)
        assert torch.equal(bits(y.cpu()), bits(want))


@pytest.mark.parametrize("M", [1, 2, 4, 8, 9, 16])
@pytest.mark.parametrize("K,N", [(4096, 4096), (4096, 14336), (14336, 4096), (8192, 8192), (4096, 32000),
                                 (1024, 3072), (2048, 5120), (1536, 3088)])
@pytest.mark.parametrize("fused", [True, False])
def test_dense_int8_strip_bit_exact(dev, M, K, N, fused, monkeypatch):
    # both forms of the kernel at every shape: the rows quantised inside every workgroup, and
    # quantised by the quantizer kernel first
    monkeypatch.setattr(kops, "INT8_STRIP_FUSED_QUANTIZER_MAX", 1 << 30 if fused else 0)
    monkeypatch.setattr(kops, "INT8_STRIP_FUSED_MAX_ROWS", 16)
    if not kops.int8_strip_supported(M, K, N):
        # too many rows of this width for LDS: the two-launch route keeps those
        assert M * K > 114688
        return
    run_case(dev, M, K, N, with_bias=(M % 2 == 0))


@pytest.mark.parametrize("M", [2, 8, 16])
def test_dense_int8_strip_addend_and_settings(dev, M):
    run_case(dev, M, 4096, 4096, with_bias=False, addend=True)
    run_case(dev, M, 4096, 4096, with_bias=True, epsilon=1e-3, value_range=(-100, 90), seed=5)


def test_dense_int8_strip_repeatable_and_graph(dev):
    g = torch.Generator().manual_seed(3)
    M, K, N = 4, 4096, 14336
    x = torch.randn(M, K, generator=g).to(torch.bfloat16).to(dev)
    w = torch.randint(-127, 128, (K, N), generator=g, dtype=torch.int8).to(dev)
    ks = (torch.rand(N, generator=g) * 50 + 50).to(torch.bfloat16).to(dev)
    shadow = kops.int8_strip_copy(w)
    first = kops.int8_dense_strip(x, shadow, N, ks)
    for _ in range(20):
        assert torch.equal(bits(kops.int8_dense_strip(x, shadow, N, ks)), bits(first))
    side = torch.cuda.Stream()
    out = torch.empty_like(first)
    with torch.cuda.stream(side):
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            out.copy_(kops.int8_dense_strip(x, shadow, N, ks))
    torch.cuda.synchronize()
    for _ in range(3):
        out.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(bits(out), bits(first))


@pytest.mark.parametrize("M", [1, 8])
@pytest.mark.parametrize("fused", [True, False])
def test_dense_int8_strip_multi_matches_single_calls(dev, M, fused, monkeypatch):
    # several kernels against one x in one launch: every workgroup computes what it computes in a
    # single call (integer sums), so the bits are the single calls' bits -- also where the shared
    # launch makes workgroups take turns that a problem alone would not need
    monkeypatch.setattr(kops, "INT8_STRIP_FUSED_QUANTIZER_MAX", 1 << 30 if fused else 0)
    monkeypatch.setattr(kops, "INT8_STRIP_FUSED_MAX_ROWS", 16)
    K = 4096
    widths = [4096, 4096, 4096, 14336, 3072]
    g = torch.Generator().manual_seed(40 + M)
    x = (torch.randn(M, K, generator=g) * 2).to(torch.bfloat16).to(dev)
    kernels, singles = [], []
    for i, N in enumerate(widths):
        w = torch.randint(-127, 128, (K, N), generator=g, dtype=torch.int8).to(dev)
        ks = (torch.rand(N, generator=g) * 50 + 50).to(torch.bfloat16).to(dev)
        bias = (torch.randn(N, generator=g) * 0.1).to(torch.bfloat16).to(dev) if i % 2 == 0 else None
        spec = dict(shadow=kops.int8_strip_copy(w), units=N, kernel_scale=ks, bias=bias)
        kernels.append(spec)
        singles.append(kops.int8_dense_strip(x, spec["shadow"], N, ks, bias=bias))
    for base, end in ((0, 3), (0, 5), (3, 5)):
        got = kops.int8_dense_strip_multi(x, kernels[base:end])
        for j, y in enumerate(got):
            assert torch.equal(bits(y), bits(singles[base + j])), (base, j)


@pytest.mark.parametrize("rows", [1, 8])
def test_call_together_int8_layers_at_decode_widths(dev, rows):
    # Dense and EinsumDense int8 layers on one input go through one launch and give the bits of
    # the separate calls (which are the oracle's, tested above)
    import keras_amd as ka
    from keras_amd.layers import Dense, EinsumDense

    g = torch.Generator().manual_seed(77)
    init = lambda s, d: (torch.rand(s, generator=g) - 0.5).to(d)
    proj = [EinsumDense("btd,dnh->btnh", (None, 32, 128), dtype="bfloat16", device=dev, kernel_initializer=init)
            for _ in range(3)]
    x = torch.randn((rows, 1, 4096), generator=g).to(torch.bfloat16).to(dev)
    for layer in proj:
        layer.build((None, 1, 4096))
        layer.quantize("int8")
    want = [layer(x) for layer in proj]
    got = ka.layers.call_together(proj, x)
    for a, b in zip(got, want):
        assert a.shape == b.shape and torch.equal(bits(a), bits(b))
    mlp = [Dense(14336, use_bias=False, dtype="bfloat16", device=dev, kernel_initializer=init),
           Dense(14336, use_bias=True, activation="relu", dtype="bfloat16", device=dev, kernel_initializer=init)]
    x2 = x.reshape(rows, 4096)
    for layer in mlp:
        layer.build((None, 4096))
        layer.quantize("int8")
    want = [layer(x2) for layer in mlp]
    got = ka.layers.call_together(mlp, x2)
    for a, b in zip(got, want):
        assert a.shape == b.shape and torch.equal(bits(a), bits(b))


def test_dense_int8_strip_rejects(dev):
    for M, K, N in [(17, 4096, 4096), (1, 4096, 1024), (1, 4000, 4096), (1, 4096, 4100), (16, 14336, 4096),
                    (1, 512, 4096)]:
        assert not kops.int8_strip_supported(M, K, N)
    x = torch.zeros(1, 4096, dtype=torch.bfloat16, device=dev)
    w = torch.zeros(4096, 4096, dtype=torch.int8, device=dev)
    ks = torch.ones(4096, dtype=torch.bfloat16, device=dev)
    shadow = kops.int8_strip_copy(w)
    with pytest.raises(ValueError):
        kops.int8_dense_strip(x, shadow[:-16], 4096, ks)
    with pytest.raises(ValueError):
        kops.int8_dense_strip(x, shadow, 4096, ks, bias=torch.zeros(5, dtype=torch.bfloat16, device=dev))
    with pytest.raises(TypeError):
        kops.int8_dense_strip(x.float(), shadow, 4096, ks)
    with pytest.raises(ValueError):
        kops.int8_dense_strip(torch.zeros(17, 4096, dtype=torch.bfloat16, device=dev), shadow, 4096, ks)


def test_dense_int8_strip_fractional_range(dev):
    """Between non-integer ends clip-then-round is not round-then-clip: the in-kernel quantizer refuses
    such a range, and the op quantises the rows with the quantizer kernel first (same bits as the
    oracle either way)."""
    import ctypes

    from keras_amd import _lib

    run_case(dev, 2, 4096, 4096, with_bias=True, value_range=(-100.5, 90.25), seed=9)
    lib = _lib.load()
    x = torch.zeros(1, 4096, dtype=torch.bfloat16, device=dev)
    ks = torch.ones(4096, dtype=torch.bfloat16, device=dev)
    shadow = kops.int8_strip_copy(torch.zeros(4096, 4096, dtype=torch.int8, device=dev))
    y = torch.empty(1, 4096, dtype=torch.bfloat16, device=dev)
    rc = lib.k3q_dense_i8_w8s(_lib.ptr(x), _lib.K3Q_BF16, 1, 4096, 4096, _lib.ptr(shadow), _lib.ptr(ks), None, 0,
                              1e-7, -100.5, 90.25, _lib.ptr(y), _lib.stream_ptr(dev))
    assert rc == -7
    torch.cuda.synchronize()
