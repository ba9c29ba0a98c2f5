"""Decode matmuls with an operation on their input folded in (k3q_gemv_w4s_pre,
k3q_dense_i8_w8s_pre): the normalisation or the gate is applied to the rows inside the kernel and
must give the bits of the separate launch (k3q_rmsnorm / k3q_silu_mul) followed by the plain matmul."""
import pytest
import torch

import keras_amd as ka
from keras_amd import ops as kops
from keras_amd.layers import Dense, call_add, call_together

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def dev():
    if not torch.cuda.is_available():
        pytest.skip("needs a HIP device")
    return torch.device("cuda:0")


def bits(t):
    return t.contiguous().view(torch.int16)


def int4_kernels(dev, K, Ns, grouped, g):
    out = []
    for N in Ns:
        packed = torch.randint(-128, 128, (K, N // 2), generator=g, dtype=torch.int8).to(dev)
        k = dict(units=N, shadow=kops.int4_strip_copy(packed, N))
        if grouped:
            scale = (torch.rand(K // 128, N, generator=g) * 0.01 + 0.001).to(torch.bfloat16).to(dev)
            zero = torch.randint(-8, 8, (K // 128, N), generator=g, dtype=torch.int8).to(dev)
            k["gparams"] = kops.int4_strip_params(scale, zero, K, N, 128)
        else:
            k["kernel_scale"] = (torch.rand(N, generator=g) + 0.5).to(torch.bfloat16).to(dev)
        out.append(k)
    return out


@pytest.mark.parametrize("grouped", [False, True])
@pytest.mark.parametrize("M,K,Ns", [(1, 4096, (4096, 4096, 4096)), (8, 4096, (14336, 14336)), (3, 8192, (8192,)),
                                    (16, 4096, (4096,)), (1, 14336, (4096,)), (2, 4608, (3072, 4096))])
def test_int4_rms_norm_inside(dev, M, K, Ns, grouped, monkeypatch):
    monkeypatch.setattr(kops, "STRIP_RMS_MAX_ROWS", 16)  # (the kernel takes any decode size; the op layer is choosier)
    g = torch.Generator().manual_seed(M + K + len(Ns))
    x = (torch.randn(M, K, generator=g) * 2).to(torch.bfloat16).to(dev)
    gain = (torch.rand(K, generator=g) + 0.5).to(torch.bfloat16).to(dev)
    kernels = int4_kernels(dev, K, Ns, grouped, g)
    bs = 128 if grouped else None
    op = ("rms_norm", gain, 1e-6)
    assert all(kops.int4_strip_input_op_supported(op, M, K, N, bs) for N in Ns)
    got = kops.int4_matmul_strip_multi(x, kernels, block_size=bs, input_op=op)
    want = kops.int4_matmul_strip_multi(kops.rmsnorm(x, gain, 1e-6), kernels, block_size=bs)
    for a, b in zip(got, want):
        assert torch.equal(bits(a), bits(b))


@pytest.mark.parametrize("grouped", [False, True])
@pytest.mark.parametrize("M,K,N", [(1, 14336, 4096), (2, 14336, 4096), (1, 4096, 4096), (2, 8192, 8192)])
def test_int4_silu_gate_inside_with_residual(dev, M, K, N, grouped):
    g = torch.Generator().manual_seed(M * 3 + K + N)
    up = (torch.randn(M, K, generator=g) * 2).to(torch.bfloat16).to(dev)
    gate = (torch.randn(M, K, generator=g) * 2).to(torch.bfloat16).to(dev)
    res = torch.randn(M, N, generator=g).to(torch.bfloat16).to(dev)
    (kernel,) = int4_kernels(dev, K, (N,), grouped, g)
    bs = 128 if grouped else None
    op = ("silu_gate", gate)
    assert kops.int4_strip_input_op_supported(op, M, K, N, bs)
    (got,) = kops.int4_matmul_strip_multi(up, [dict(kernel, bias=res)], block_size=bs, input_op=op, bias_rows=True)
    want = kops.int4_matmul_strip(kops.silu_mul(gate, up), kernel["shadow"], N,
                                  kernel_scale=kernel.get("kernel_scale"), gparams=kernel.get("gparams"),
                                  block_size=bs, addend=res)
    assert torch.equal(bits(got), bits(want))
    assert not kops.int4_strip_input_op_supported(op, 8, K, N, bs)  # too many rows for the gate


def int8_kernels(dev, K, Ns, g):
    out = []
    for N in Ns:
        w = torch.randint(-127, 128, (K, N), generator=g, dtype=torch.int8).to(dev)
        out.append(dict(units=N, shadow=kops.int8_strip_copy(w),
                        kernel_scale=(torch.rand(N, generator=g) * 50 + 50).to(torch.bfloat16).to(dev)))
    return out


@pytest.mark.parametrize("M,K,Ns", [(1, 4096, (4096, 4096, 4096)), (4, 4096, (14336, 14336)), (2, 8192, (8192,)),
                                    (1, 14336, (4096,)), (2, 1024, (3072,))])
def test_int8_rms_norm_inside(dev, M, K, Ns):
    g = torch.Generator().manual_seed(M + K + len(Ns) + 1)
    x = (torch.randn(M, K, generator=g) * 2).to(torch.bfloat16).to(dev)
    gain = (torch.rand(K, generator=g) + 0.5).to(torch.bfloat16).to(dev)
    kernels = int8_kernels(dev, K, Ns, g)
    op = ("rms_norm", gain, 1e-6)
    assert all(kops.int8_strip_input_op_supported(op, M, K, N) for N in Ns)
    got = kops.int8_dense_strip_multi(x, kernels, input_op=op)
    want = kops.int8_dense_strip_multi(kops.rmsnorm(x, gain, 1e-6), kernels)
    for a, b in zip(got, want):
        assert torch.equal(bits(a), bits(b))


@pytest.mark.parametrize("M,K,N", [(1, 14336, 4096), (2, 14336, 4096), (1, 4096, 4096)])
def test_int8_silu_gate_inside_with_residual(dev, M, K, N):
    g = torch.Generator().manual_seed(M * 5 + K + N)
    up = (torch.randn(M, K, generator=g) * 2).to(torch.bfloat16).to(dev)
    gate = (torch.randn(M, K, generator=g) * 2).to(torch.bfloat16).to(dev)
    res = torch.randn(M, N, generator=g).to(torch.bfloat16).to(dev)
    (kernel,) = int8_kernels(dev, K, (N,), g)
    op = ("silu_gate", gate)
    assert kops.int8_strip_input_op_supported(op, M, K, N)
    (got,) = kops.int8_dense_strip_multi(up, [dict(kernel, bias=res)], input_op=op, bias_rows=True)
    want = kops.int8_dense_strip(kops.silu_mul(gate, up), kernel["shadow"], N, kernel["kernel_scale"], bias=res)
    assert torch.equal(bits(got), bits(want))


def test_input_op_rejects(dev):
    g = torch.Generator().manual_seed(0)
    x = torch.zeros(1, 4096, dtype=torch.bfloat16, device=dev)
    kernels = int4_kernels(dev, 4096, (4096,), False, g)
    with pytest.raises(ValueError):
        kops.int4_matmul_strip_multi(x, kernels, input_op=("rms_norm", torch.ones(100, dtype=torch.bfloat16, device=dev), 1e-6))
    with pytest.raises(ValueError):
        kops.int4_matmul_strip_multi(x, kernels, input_op=("silu_gate", torch.ones(2, 4096, dtype=torch.bfloat16, device=dev)))
    with pytest.raises(ValueError):
        kops.int4_matmul_strip_multi(x, kernels, input_op=("tanh", x))
    # a K that is not whole blocks of 512: the normalisation stays a launch of its own
    assert not kops.int4_strip_input_op_supported(("rms_norm", None, 1e-6), 1, 4352, 4096)


@pytest.mark.parametrize("mode", ["int4", "int8"])
@pytest.mark.parametrize("rows", [1, 2, 8])
def test_layers_with_input_ops_match_separate_launches(dev, mode, rows):
    """call_together / call_add with an input operation: the same bits as the operation's own launch
    followed by the plain calls, whichever route the sizes take."""
    g = torch.Generator().manual_seed(rows)
    init = lambda shape, dtype: (torch.randn(shape, generator=g) * 0.02).to(dtype)
    proj = [Dense(4096, use_bias=False, dtype="bfloat16", device=dev, kernel_initializer=init) for _ in range(2)]
    down = Dense(4096, use_bias=False, dtype="bfloat16", device=dev, kernel_initializer=init)
    for layer in proj + [down]:
        layer.build((None, 4096))
        layer.quantize(mode)
    x = (torch.randn(rows, 1, 4096, generator=g) * 2).to(torch.bfloat16).to(dev)
    gain = (torch.rand(4096, generator=g) + 0.5).to(torch.bfloat16).to(dev)
    op = ("rms_norm", gain, 1e-6)
    got = call_together(proj, x, input_op=op)
    want = call_together(proj, kops.rmsnorm(x, gain, 1e-6))
    for a, b in zip(got, want):
        assert a.shape == b.shape and torch.equal(bits(a), bits(b))
    gate, up = want
    res = torch.randn(rows, 1, 4096, generator=g).to(torch.bfloat16).to(dev)
    got = call_add(down, up, res, input_op=("silu_gate", gate))
    want = call_add(down, kops.silu_mul(gate, up), res)
    assert got.shape == want.shape and torch.equal(bits(got), bits(want))


@pytest.mark.parametrize("value_range", [(-127, 127), (-100.5, 90.25)])
@pytest.mark.parametrize("rows,dim,kind", [(8, 4096, "rms_norm"), (1, 4096, "rms_norm"), (1024, 4096, "rms_norm"),
                                           (5, 14336, "silu_gate"), (8, 14336, "rms_norm"), (3, 136, "rms_norm"),
                                           (16, 16384, "silu_gate")])
def test_input_op_quantize_matches_the_two_launches(dev, rows, dim, kind, value_range):
    """k3q_input_op_quantize: h, q and scale carry the bits of k3q_rmsnorm / k3q_silu_mul followed by
    k3q_absmax_quantize."""
    from keras_amd import quantizers as kq

    g = torch.Generator().manual_seed(rows + dim)
    x = (torch.randn(rows, dim, generator=g) * 2).to(torch.bfloat16).to(dev)
    if rows > 2:
        x[1] = 0  # an all-zero row: scale = range / eps
    if kind == "rms_norm":
        op = ("rms_norm", (torch.rand(dim, generator=g) + 0.5).to(torch.bfloat16).to(dev), 1e-6)
    else:
        op = ("silu_gate", (torch.randn(rows, dim, generator=g) * 2).to(torch.bfloat16).to(dev))
    assert kops.input_op_quantize_supported(op, x)
    h, q, s = kops.input_op_quantize(op, x, epsilon=1e-7, value_range=value_range)
    want_h = kops.apply_input_op(op, x)
    want_q, want_s = kq.abs_max_quantize(want_h, axis=-1, value_range=value_range, epsilon=1e-7)
    assert torch.equal(bits(h), bits(want_h))
    assert s.shape == want_s.shape and torch.equal(bits(s), bits(want_s))
    assert torch.equal(q, want_q)
