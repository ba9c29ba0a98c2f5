"""The decode-sized int4 matmul for callers that cannot allocate (k3q_gemv_w4_static): its
partial sums and arrival counters live in a device array inside the library.  Checked through
the C ABI against k3q_gemv_w4_fused (caller's workspace): same kernels, same order, same bits."""

import pytest
import torch

from keras_amd import _lib
from oracle import keras_cpu_path as ref

pytestmark = pytest.mark.gpu


def _operands(dev, M, K, N, block_size, dtype, seed):
    g = torch.Generator().manual_seed(seed)
    kernel = ref.glorot_uniform(K, N, generator=g)
    qk = ref.dense_quantize_int4(kernel, block_size)
    grouped = block_size is not None
    x = torch.randn(M, K, generator=g).to(dtype).to(dev)
    bias = (torch.randn(N, generator=g) * 0.02).to(dtype).to(dev)
    return dict(x=x, w=qk["kernel"].to(dev), scale=qk["kernel_scale"].to(dtype).to(dev),
                zero=qk["kernel_zero"].to(dev) if grouped else None, bias=bias)


def _both(dev, M, K, N, block_size, dtype, seed):
    lib = _lib.load()
    op = _operands(dev, M, K, N, block_size, dtype, seed)
    grouped = block_size is not None
    s = _lib.stream_ptr(dev)
    head = [_lib.ptr(op["x"]), _lib.dtype_code(dtype), M, K, N, _lib.ptr(op["w"]), _lib.ptr(op["scale"]),
            _lib.ptr(op["zero"]), block_size if grouped else -1, _lib.ptr(op["bias"])]
    ws = torch.empty(max(lib.k3q_gemv_w4_workspace_bytes(M, K, N), 16), dtype=torch.uint8, device=dev)
    counters = torch.zeros(max(lib.k3q_gemv_w4_counters_bytes(N), 4), dtype=torch.uint8, device=dev)
    want = torch.empty((M, N), dtype=dtype, device=dev)
    got = torch.full((M, N), float("nan"), dtype=dtype, device=dev)
    assert lib.k3q_gemv_w4_fused(*head, _lib.ptr(want), _lib.ptr(ws), ws.numel(), _lib.ptr(counters),
                                 counters.numel(), s) == 0
    assert lib.k3q_gemv_w4_static(*head, _lib.ptr(got), s) == 0
    torch.cuda.synchronize()
    bits = torch.int16 if dtype == torch.bfloat16 else torch.int32
    assert torch.equal(got.view(bits), want.view(bits)), (M, K, N, block_size, dtype)


def test_static_scratch_matches_workspace_call_twice_second_smaller(dev):
    # two calls in a row on the same device array, the second with a smaller input
    _both(dev, 8, 8192, 8192, 128, torch.bfloat16, 1)
    _both(dev, 3, 2048, 1024, None, torch.bfloat16, 2)


@pytest.mark.parametrize("M,K,N,block_size,dtype", [
    (1, 8192, 8192, None, torch.bfloat16), (16, 4096, 14336, 128, torch.bfloat16),
    (4, 14336, 4096, 128, torch.float32), (2, 100, 30, 50, torch.bfloat16),
    (1, 4096, 32000, 128, torch.bfloat16),
])
def test_static_scratch_shapes(dev, M, K, N, block_size, dtype):
    _both(dev, M, K, N, block_size, dtype, 3)
    _both(dev, M, K, N, block_size, dtype, 4)  # again: the counters were left at zero


def test_static_scratch_rejects_what_does_not_fit(dev):
    lib = _lib.load()
    one = torch.zeros(64, dtype=torch.uint8, device=dev)
    p = _lib.ptr(one)
    s = _lib.stream_ptr(dev)
    assert lib.k3q_gemv_w4_static_max_bytes() == 16 << 20
    # more rows than a decode step, and a K split whose partials exceed the array
    assert lib.k3q_gemv_w4_static(p, 1, 17, 64, 64, p, p, None, -1, None, p, s) == -2
    big_n = 1 << 22
    assert lib.k3q_gemv_w4_static(p, 1, 16, 1 << 15, big_n, p, p, None, -1, None, p, s) == -5
    assert lib.k3q_gemv_w4_static(p, 9, 1, 64, 64, p, p, None, -1, None, p, s) == -4
    assert lib.k3q_gemv_w4_static(None, 1, 1, 64, 64, p, p, None, -1, None, p, s) == -1
