"""GPU parity: the weight quantizers of `quantize()` run on the device for kernels that live there
(k3q_weight_absmax_quantize, k3q_weight_quantize_grouped) and must return the bits of the
reference's numpy float32 path (keras/src/quantizers/quantizers.py:95-109, :182-234), which the
oracle restates with numpy itself."""

import pytest
import torch

from keras_amd import quantizers as kq
from oracle import keras_cpu_path as ref

pytestmark = pytest.mark.gpu


def bits(t):
    t = t.contiguous()
    return t.view(torch.int16) if t.dtype == torch.bfloat16 else t.view(torch.int32)


def kernel_like(shape, seed, dtype=torch.float32):
    g = torch.Generator().manual_seed(seed)
    w = (torch.rand(shape, generator=g) * 2 - 1) * 0.05
    w.view(-1)[::97] = 0.0                      # exact zeros
    w.view(-1)[5::131] *= 40.0                  # outliers that set a column's scale
    return w.to(dtype)


ABSMAX_CASES = [
    # shape, axis
    ((64, 48), 0), ((257, 1001), 0), ((1, 7), 0), ((300, 3), 0), ((4096, 4096), 0),
    ((96, 4, 8), 0), ((4, 8, 96), (0, 1)), ((3, 64, 6), 1), ((2, 5, 7, 4), (1, 2)),
    ((5, 6, 7), (0, 2)), ((2, 3, 4, 5), (0, 2)),        # reduced axes that are not neighbours
    ((33, 130), -1), ((6, 5, 16), (1, 2)), ((4, 9), (0, 1)),
]


@pytest.mark.parametrize("shape,axis", ABSMAX_CASES)
@pytest.mark.parametrize("value_range", [(-127, 127), (-8, 7)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_device_absmax_weight_quantizer_has_numpy_bits(dev, shape, axis, value_range, dtype):
    w = kernel_like(shape, sum(shape), dtype)
    if len(shape) == 2:
        w[:, 0] = 0  # an all-zero column: scale = hi / epsilon
    want_q, want_s = ref.abs_max_quantize(w, axis, value_range=value_range, to_numpy=True)
    q, s = kq.abs_max_quantize(w.to(dev), axis, value_range=value_range, to_numpy=True)
    assert q.is_cuda and q.dtype == torch.int8 and s.dtype == dtype
    assert tuple(q.shape) == tuple(shape) and tuple(s.shape) == tuple(want_s.shape)
    assert torch.equal(q.cpu(), want_q)
    assert torch.equal(bits(s.cpu()), bits(want_s))
    # and the host route of the same call (a CPU tensor in, numpy arithmetic) still agrees
    qh, sh = kq.abs_max_quantize(w, axis, value_range=value_range, to_numpy=True)
    assert torch.equal(qh, want_q) and torch.equal(bits(sh), bits(want_s))


GROUPED_CASES = [
    # K, N, block
    (512, 256, 128), (500, 6, 128), (96, 40, 32), (128, 1001, 128), (1, 4, 128), (130, 8, 64),
    (4096, 4096, 128), (64, 12, 7),
]


@pytest.mark.parametrize("K,N,block", GROUPED_CASES)
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_device_grouped_weight_quantizer_has_numpy_bits(dev, K, N, block, dtype):
    w = kernel_like((K, N), K + N + block, dtype)
    if K >= 2 * block:
        w[:block, 0] = 0.0         # a group of zeros: scale = epsilon / 15, everything at the zero point
        w[block:2 * block, 1] = w[block:2 * block, 1].abs() + 0.01   # a group that does not straddle zero
    want_q, want_s, want_z = ref.abs_max_quantize_grouped_with_zero_point(w, block)
    q, s, z = kq.abs_max_quantize_grouped_with_zero_point(w.to(dev), block, to_numpy=True)
    assert q.is_cuda and s.dtype == dtype and z.dtype == torch.int8
    assert torch.equal(q.cpu(), want_q)
    assert torch.equal(bits(s.cpu()), bits(want_s))
    assert torch.equal(z.cpu(), want_z)
    qh, sh, zh = kq.abs_max_quantize_grouped_with_zero_point(w, block, to_numpy=True)
    assert torch.equal(qh, want_q) and torch.equal(bits(sh), bits(want_s)) and torch.equal(zh, want_z)


def test_device_grouped_weight_quantizer_at_rounding_boundaries(dev):
    # The device kernel takes rint(x / scale) from x * (1 / scale) unless that product lies next to a
    # half-integer, where it divides.  Every weight here sits on such a boundary or within a few
    # float32 steps of one -- (m + 1/2) * scale for the levels m of its group, moved by -4 ... +4
    # ulps -- with scales and minima that differ from column to column, so both the test for
    # "next to" and the division behind it decide the integers.  Bit for bit against the numpy path.
    import numpy as np

    block, N, G = 128, 1024, 4
    rng = np.random.default_rng(5)
    span = rng.uniform(0.01, 3.0, size=N).astype(np.float32)         # max - min of a group, per column
    lo = np.where(np.arange(N) % 3 == 0, 0.0, -rng.uniform(0.0, 1.0, size=N) * span).astype(np.float32)
    hi = (lo + span).astype(np.float32)
    scale = ((hi - lo) + np.float32(1e-7)) / np.float32(15.0)         # the scale numpy will find
    m_lo = np.ceil(lo.astype(np.float64) / scale)                     # half-integers m + 1/2 inside (lo, hi)
    m_hi = np.floor(hi.astype(np.float64) / scale) - 1
    w = np.empty((G * block, N), dtype=np.float32)
    for row in range(G * block):
        r = row % block
        if r == 0:
            w[row] = lo
        elif r == 1:
            w[row] = hi
        else:
            m = m_lo + (row * 5) % np.maximum(m_hi - m_lo + 1, 1)
            x = ((m + 0.5) * scale.astype(np.float64)).astype(np.float32)
            steps = (row * 7) % 9 - 4
            for _ in range(abs(steps)):
                x = np.nextafter(x, np.float32(np.inf if steps > 0 else -np.inf))
            w[row] = np.minimum(np.maximum(x, lo), hi)
    w = torch.from_numpy(w)
    want_q, want_s, want_z = ref.abs_max_quantize_grouped_with_zero_point(w, block)
    assert torch.equal(bits(want_s), bits(torch.from_numpy(np.tile(scale, (G, 1)))))  # the scales aimed at
    q, s, z = kq.abs_max_quantize_grouped_with_zero_point(w.to(dev), block, to_numpy=True)
    assert torch.equal(bits(s.cpu()), bits(want_s)) and torch.equal(z.cpu(), want_z)
    assert torch.equal(q.cpu(), want_q)
    # the case is what it claims to be: most quotients are within 1e-5 of a half-integer
    r = w.double().reshape(G, block, N) / want_s.double()[:, None, :]
    near = ((r - r.floor() - 0.5).abs() < 1e-5).double().mean().item()
    assert near > 0.5, near


def test_device_weight_quantizers_at_llama_kernel_size(dev):
    # 4096 x 14336 (the gate / up projection of config 5): both quantizers against the oracle
    w = kernel_like((4096, 14336), 7)
    wd = w.to(dev)
    q8, s8 = ref.dense_quantize_int8(w)
    got_q, got_s = kq.abs_max_quantize(wd, axis=0, to_numpy=True)
    assert torch.equal(got_q.cpu(), q8) and torch.equal(bits(got_s.reshape(-1).cpu()), bits(s8))
    q4 = ref.dense_quantize_int4(w, 128)
    gq, gs, gz = kq.abs_max_quantize_grouped_with_zero_point(wd, 128, to_numpy=True)
    packed, _, _ = kq.pack_int4(gq, axis=-1)
    assert torch.equal(packed.cpu(), q4["kernel"])
    assert torch.equal(bits(gs.cpu()), bits(q4["kernel_scale"])) and torch.equal(gz.cpu(), q4["kernel_zero"])
    qc = ref.dense_quantize_int4(w, None)
    cq, cs = kq.abs_max_quantize(wd, axis=0, value_range=(-8, 7), to_numpy=True)
    packed, _, _ = kq.pack_int4(cq, axis=-1)
    assert torch.equal(packed.cpu(), qc["kernel"]) and torch.equal(bits(cs.reshape(-1).cpu()), bits(qc["kernel_scale"]))


def test_device_weight_quantizer_errors(dev):
    w = torch.zeros(4, 4, device=dev)
    with pytest.raises(ValueError):
        kq.abs_max_quantize(w, 0, value_range=(-200, 127), to_numpy=True)
    with pytest.raises(ValueError):
        kq.abs_max_quantize_grouped_with_zero_point(torch.zeros(2, 3, 4, device=dev), 2, to_numpy=True)
    with pytest.raises(NotImplementedError):
        kq.abs_max_quantize_grouped_with_zero_point(w, 2, to_numpy=False)
    with pytest.raises(ValueError):
        kq.abs_max_quantize(torch.zeros(0, 4, device=dev), 0, to_numpy=True)
