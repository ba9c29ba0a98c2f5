"""GPU parity: pack/unpack and the abs-max quantizer against the CPU oracle (bit-exact)."""

import numpy as np
import pytest
import torch

from keras_amd import quantizers as kq
from oracle import keras_cpu_path as ref

pytestmark = pytest.mark.gpu

PACK_SCENARIOS = [
    # (shape, axis) -- the seven scenarios of quantizers_test.py:157-175 plus large ones
    ((8, 8), 0), ((8, 8), 1), ((5, 8), 0), ((8, 5), 1), ((4, 6, 8), 1), ((4, 6, 5), -1),
    ((2, 3, 4, 5), 2), ((3, 2), 0), ((1, 1), 0), ((64, 256), -1), ((64, 256), 0),
    ((127, 384), 0), ((33, 48), 1), ((16, 32, 64), 1), ((256, 8192), -1), ((1024, 4096), 0),
]


@pytest.mark.parametrize("shape,axis", PACK_SCENARIOS)
@pytest.mark.parametrize("dtype", ["int8", "uint8"])
def test_pack_unpack_matches_oracle(dev, shape, axis, dtype):
    g = torch.Generator().manual_seed(hash((shape, axis)) % 1000)
    if dtype == "int8":
        arr = torch.randint(-8, 8, shape, generator=g, dtype=torch.int8)
    else:
        arr = torch.randint(0, 16, shape, generator=g, dtype=torch.uint8)
    p_ref, shape_ref, n_ref = ref.pack_int4(arr, axis=axis, dtype=dtype)
    p_gpu, shape_gpu, n_gpu = kq.pack_int4(arr.to(dev), axis=axis, dtype=dtype)
    assert shape_gpu == shape_ref and n_gpu == n_ref
    assert torch.equal(p_gpu.cpu(), p_ref)
    u_ref = ref.unpack_int4(p_ref, n_ref, axis=axis, dtype=dtype)
    u_gpu = kq.unpack_int4(p_gpu, n_gpu, axis=axis, dtype=dtype)
    assert u_gpu.dtype == u_ref.dtype
    assert torch.equal(u_gpu.cpu(), u_ref)
    assert torch.equal(u_gpu.cpu(), arr)


@pytest.mark.parametrize("axis", [-1, 0])
def test_pack_unpack_config2_kernel_size(dev, axis):
    # the 8192 x 8192 kernel of configuration 2, packed along the last axis (the layers' layout)
    # and along axis 0 (K-packed, what the configuration's wording describes), int8 storage
    g = torch.Generator().manual_seed(8192 + axis)
    arr = torch.randint(-8, 8, (8192, 8192), generator=g, dtype=torch.int8)
    p_ref, shape_ref, n_ref = ref.pack_int4(arr, axis=axis)
    p_gpu, shape_gpu, n_gpu = kq.pack_int4(arr.to(dev), axis=axis)
    assert shape_gpu == shape_ref == ((8192, 4096) if axis == -1 else (4096, 8192)) and n_gpu == n_ref == 8192
    assert torch.equal(p_gpu.cpu(), p_ref)
    u_gpu = kq.unpack_int4(p_gpu, n_gpu, axis=axis)
    assert torch.equal(u_gpu.cpu(), arr)
    assert torch.equal(ref.unpack_int4(p_ref, n_ref, axis=axis), arr)


def test_unpack_all_bytes(dev):
    b = torch.arange(256, dtype=torch.int32).to(torch.uint8).view(torch.int8).reshape(16, 16)
    for axis in (0, 1):
        for dtype in ("int8", "uint8"):
            want = ref.unpack_int4(b, 32, axis=axis, dtype=dtype)
            got = kq.unpack_int4(b.to(dev), 32, axis=axis, dtype=dtype)
            assert torch.equal(got.cpu(), want)


def test_pack_garbage_high_bits(dev):
    # values outside [-8, 7]: only the low nibble may survive, as in the reference
    g = torch.Generator().manual_seed(3)
    arr = torch.randint(-128, 128, (64, 64), generator=g, dtype=torch.int8)
    for axis in (0, 1):
        want, _, _ = ref.pack_int4(arr, axis=axis)
        got, _, _ = kq.pack_int4(arr.to(dev), axis=axis)
        assert torch.equal(got.cpu(), want)


def test_pack_errors(dev):
    with pytest.raises(ValueError):
        kq.pack_int4(torch.zeros(2, 2, dtype=torch.int8, device=dev), dtype="int16")
    with pytest.raises(TypeError):
        kq.pack_int4(torch.zeros(2, 2, dtype=torch.uint8, device=dev), dtype="int8")
    with pytest.raises(TypeError):
        kq.unpack_int4(torch.zeros(2, 2, dtype=torch.int32, device=dev), 4)


QUANT_SHAPES = [(1, 8), (3, 4, 5), (16, 4096), (7, 333), (4, 8192), (33, 1024), (2, 14336),
                (5, 20000), (300, 512), (2, 65536), (2, 3, 100000)]


@pytest.mark.parametrize("shape", QUANT_SHAPES)
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_abs_max_quantize_last_axis(dev, shape, dtype):
    g = torch.Generator().manual_seed(sum(shape))
    x = (torch.randn(shape, generator=g) * 3.0).to(dtype)
    q_ref, s_ref = ref.abs_max_quantize(x, axis=-1)
    q, s = kq.abs_max_quantize(x.to(dev), axis=-1)
    assert q.dtype == torch.int8 and s.dtype == dtype
    assert tuple(s.shape) == tuple(s_ref.shape)
    assert torch.equal(s.cpu().view(torch.int16 if dtype == torch.bfloat16 else torch.int32),
                       s_ref.view(torch.int16 if dtype == torch.bfloat16 else torch.int32))
    assert torch.equal(q.cpu(), q_ref)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_abs_max_quantize_row_lengths_around_the_kernel_forms(dev, dtype):
    """Row lengths on both sides of every switch between the quantizer's forms (a wave or a
    workgroup per row, 1 ... 8 groups of 16 values per thread, rows that fill every thread or not),
    with few and many rows and a zero row."""
    g = torch.Generator().manual_seed(7)
    bits = torch.int16 if dtype == torch.bfloat16 else torch.int32
    for groups in (1, 63, 64, 65, 127, 128, 129, 255, 256, 257, 511, 512, 513, 1023, 1024, 1025, 2047, 2048, 2049):
        cols = 16 * groups
        for rows in (1, 5, 1024 if cols <= 2064 else 9):
            x = (torch.randn(rows, cols, generator=g) * (0.01 if groups % 2 else 30.0)).to(dtype)
            if rows > 2:
                x[1] = 0
            q_ref, s_ref = ref.abs_max_quantize(x, axis=-1)
            q, s = kq.abs_max_quantize(x.to(dev), axis=-1)
            assert torch.equal(q.cpu(), q_ref), (rows, cols)
            assert torch.equal(s.cpu().view(bits), s_ref.view(bits)), (rows, cols)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_abs_max_quantize_special_rows(dev, dtype):
    x = torch.zeros(6, 64)
    x[1, 3] = 1e-6
    x[2] = torch.linspace(-2, 2, 64)
    x[3] = 2.0 ** torch.arange(-32, 32).float()
    x[4, :] = 0.5
    x[4, 0] = 127.0  # scale == 1 -> the 0.5 entries are exact ties
    x[5, :] = 1.5
    x[5, 0] = -127.0
    x = x.to(dtype)
    q_ref, s_ref = ref.abs_max_quantize(x, axis=-1)
    q, s = kq.abs_max_quantize(x.to(dev), axis=-1)
    assert torch.equal(q.cpu(), q_ref)
    assert torch.equal(s.cpu().float(), s_ref.float())


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_abs_max_quantize_axes_and_ranges(dev, dtype):
    g = torch.Generator().manual_seed(11)
    x = torch.randn(4, 6, 8, 16, generator=g).to(dtype)
    for axis in [(2, 3), (3,), (1,), (0, 2), -2]:
        q_ref, s_ref = ref.abs_max_quantize(x, axis=axis)
        q, s = kq.abs_max_quantize(x.to(dev), axis=axis)
        assert tuple(s.shape) == tuple(s_ref.shape)
        assert torch.equal(q.cpu(), q_ref), axis
        assert torch.equal(s.cpu().float(), s_ref.float()), axis
    q_ref, s_ref = ref.abs_max_quantize(x, axis=-1, value_range=(-8, 7))
    q, s = kq.abs_max_quantize(x.to(dev), axis=-1, value_range=(-8, 7))
    assert torch.equal(q.cpu(), q_ref)
    q_ref, s_ref = ref.abs_max_quantize(x, axis=-1, epsilon=1e-3)
    q, s = kq.abs_max_quantize(x.to(dev), axis=-1, epsilon=1e-3)
    assert torch.equal(q.cpu(), q_ref)
    assert torch.equal(s.cpu().float(), s_ref.float())


def test_quantizer_noncontiguous_rows(dev):
    g = torch.Generator().manual_seed(5)
    x = torch.randn(32, 512, generator=g)
    xs = x[:, :256]
    q_ref, s_ref = ref.abs_max_quantize(xs, axis=-1)
    q, s = kq.abs_max_quantize(x.to(dev)[:, :256], axis=-1)
    assert torch.equal(q.cpu(), q_ref)
    assert torch.equal(s.cpu(), s_ref)
