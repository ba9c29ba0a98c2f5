"""GPU parity on seeded random shapes: every route boundary (decode kernels, row passes,
tile GEMM with and without a K split, the de-quantise route, plain fallbacks) gets crossed
by shapes nobody picked by hand."""

import random

import pytest
import torch

from tests.test_gpu_int4_matmul import run_case as run_int4, run_kmajor_case
from tests.test_gpu_int8_matmul import run_dense_int8

pytestmark = pytest.mark.gpu


def shapes(seed, count, max_m, max_kn):
    rng = random.Random(seed)
    out = []
    for _ in range(count):
        m = rng.choice([1, 2, 7, 8, 9, 16, 17, 31, 33, 47, 48, 64, 65, 80, 127, 128, 129, 200, 256,
                        rng.randint(1, max_m)])
        k_unit, n_unit = rng.choice([1, 2, 8, 16, 64, 128]), rng.choice([1, 2, 4, 8, 16, 64, 256])
        k = k_unit * rng.randint(1, max(1, max_kn // k_unit))
        n = n_unit * rng.randint(1, max(1, max_kn // n_unit))
        out.append((m, k, n))
    return out


@pytest.mark.parametrize("M,K,N", shapes(1, 80, 400, 2048))
def test_int8_random_shapes(dev, M, K, N):
    rng = random.Random(M * 1000003 + K * 1009 + N)
    dtype = rng.choice([torch.float32, torch.bfloat16])
    run_dense_int8(dev, M, K, N, dtype, prepack=rng.random() < 0.6, exact=True,
                   seed=rng.randint(0, 99), with_bias=rng.random() < 0.5)


@pytest.mark.parametrize("M,K,N", shapes(2, 80, 300, 2048))
def test_int4_random_shapes(dev, M, K, N):
    rng = random.Random(M * 1000003 + K * 1009 + N)
    dtype = rng.choice([torch.float32, torch.bfloat16])
    block = rng.choice([None, -1, 16, 32, 64, 128])
    run_int4(dev, M, K, N, block, dtype, with_bias=rng.random() < 0.5, seed=rng.randint(0, 99))


def kmajor_shapes(seed, count):
    # what the K-contiguous int4 route takes: 17 ... 512 rows, K % 128 == 0, N % 32 == 0, groups
    # of a multiple of 64 that divide K (or per-channel); every tile shape and group length
    rng = random.Random(seed)
    out = []
    for _ in range(count):
        m = rng.choice([17, 32, 33, 63, 64, 65, 127, 128, 129, 255, 256, 257, 511, 512, rng.randint(17, 512)])
        k = 128 * rng.randint(1, 40)
        n = 32 * rng.choice([1, 2, 3, 4, 7, 8, 9, 16, 33, 64, rng.randint(1, 150)])
        blocks = [None] + [b for b in (64, 128, 192, 256, 320, 512, 640) if k % b == 0]
        out.append((m, k, n, rng.choice(blocks)))
    return out


@pytest.mark.parametrize("M,K,N,block_size", kmajor_shapes(3, 60))
def test_int4_kmajor_random_shapes(dev, M, K, N, block_size):
    rng = random.Random(M * 1000003 + K * 1009 + N)
    run_kmajor_case(dev, M, K, N, block_size, with_bias=rng.random() < 0.5, seed=rng.randint(0, 99))
