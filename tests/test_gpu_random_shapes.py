"""GPU parity on seeded random shapes: every route boundary (decode kernels, row passes,
tile GEMM with and without a K split, the de-quantise route, plain fallbacks) gets crossed
by shapes nobody picked by hand."""

import random

import pytest
import torch

from tests.test_gpu_int4_matmul import run_case as run_int4
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
