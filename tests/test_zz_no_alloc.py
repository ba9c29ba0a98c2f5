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


def _call_fused(lib, dev, op, M, K, N, block_size, dtype, out, ws, counters):
    head = [_lib.ptr(op["x"]), _lib.dtype_code(dtype), M, K, N, _lib.ptr(op["w"]), _lib.ptr(op["scale"]),
            _lib.ptr(op["zero"]), block_size if block_size else -1, _lib.ptr(op["bias"])]
    assert lib.k3q_gemv_w4_fused(*head, _lib.ptr(out), _lib.ptr(ws), ws.numel(), _lib.ptr(counters),
                                 counters.numel(), _lib.stream_ptr(dev)) == 0


def test_first_call_on_the_device_under_graph_capture(dev):
    # This test comes first in the file and no other file calls the entry point, so the call
    # below is the first one of the process on this device: the symbol look-up happens while the
    # stream is capturing.  The graph is replayed with changed rows, with eager work between the
    # replays, and every replay is compared bit for bit with the workspace call run eagerly.
    lib = _lib.load()
    M, K, N, bs, dt = 4, 8192, 8192, 128, torch.bfloat16   # K split over workgroups: partials + counters in use
    op = _operands(dev, M, K, N, bs, dt, 11)
    assert lib.k3q_gemv_w4_workspace_bytes(M, K, N) > 0
    ws = torch.empty(lib.k3q_gemv_w4_workspace_bytes(M, K, N), dtype=torch.uint8, device=dev)
    counters = torch.zeros(lib.k3q_gemv_w4_counters_bytes(N), dtype=torch.uint8, device=dev)
    want = torch.empty((M, N), dtype=dt, device=dev)
    got = torch.full((M, N), float("nan"), dtype=dt, device=dev)
    head = [_lib.ptr(op["x"]), _lib.dtype_code(dt), M, K, N, _lib.ptr(op["w"]), _lib.ptr(op["scale"]),
            _lib.ptr(op["zero"]), bs, _lib.ptr(op["bias"])]
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        assert lib.k3q_gemv_w4_static(*head, _lib.ptr(got), _lib.stream_ptr(dev)) == 0
    torch.cuda.synchronize()
    g = torch.Generator().manual_seed(12)
    for replay in range(3):
        op["x"].copy_(torch.randn(M, K, generator=g).to(dt))
        _call_fused(lib, dev, op, M, K, N, bs, dt, want, ws, counters)   # eager work between replays
        got.fill_(float("nan"))
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(got.view(torch.int16), want.view(torch.int16)), replay
    # and eagerly afterwards, on the same array
    _both(dev, M, K, N, bs, dt, 13)


def test_static_scratch_allocates_no_device_memory(dev):
    # free device memory as the driver reports it is the same before and after calls of several
    # shapes (K split with partials, no split, float32 rows, the widest supported shape); the
    # operands are made first and torch's allocator is not asked for anything in between
    lib = _lib.load()
    cases = [(8, 8192, 8192, 128, torch.bfloat16), (1, 4096, 4096, None, torch.bfloat16),
             (4, 14336, 4096, 128, torch.float32), (16, 4096, 14336, 128, torch.bfloat16),
             (2, 100, 30, 50, torch.bfloat16)]
    prepared = []
    for i, (M, K, N, bs, dt) in enumerate(cases):
        op = _operands(dev, M, K, N, bs, dt, 20 + i)
        prepared.append((op, torch.empty((M, N), dtype=dt, device=dev)))
    s = _lib.stream_ptr(dev)
    torch.cuda.synchronize()
    free_before, _ = torch.cuda.mem_get_info(dev)
    reserved_before = torch.cuda.memory_reserved(dev)
    for (M, K, N, bs, dt), (op, out) in zip(cases, prepared):
        head = [_lib.ptr(op["x"]), _lib.dtype_code(dt), M, K, N, _lib.ptr(op["w"]), _lib.ptr(op["scale"]),
                _lib.ptr(op["zero"]), bs if bs else -1, _lib.ptr(op["bias"])]
        for _ in range(3):
            assert lib.k3q_gemv_w4_static(*head, _lib.ptr(out), s) == 0
    torch.cuda.synchronize()
    free_after, _ = torch.cuda.mem_get_info(dev)
    assert free_after == free_before, (free_before, free_after)
    assert torch.cuda.memory_reserved(dev) == reserved_before


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
