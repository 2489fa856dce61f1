"""Seeded sweeps of random shapes against the CPU oracle for the operators whose kernels are chosen
by shape: matrix products (all transpose forms; tile family, split-K, ragged tiles and a ragged
last k-step), batched products, and max / average pooling (window, padding and stride drawn at
random; max pooling bit-exact including tie order, through both symbol families)."""
import numpy as np
import pytest

from oracle import ops as O
from util import assert_close

pytestmark = pytest.mark.gpu


def _dims(rng, hi):
    pool = [1, 2, 3, 4, 5, 7, 8, 15, 16, 17, 31, 32, 33, 63, 64, 65, 100, 127, 128, 129, 200, 255, 256, 257, 300, 513]
    return int(rng.choice([d for d in pool if d <= hi]))


def _matmul_cases(seed, count):
    rng = np.random.RandomState(seed)
    out = []
    for _ in range(count):
        M, N = _dims(rng, 513), _dims(rng, 513)
        K = int(rng.choice([1, 3, 4, 15, 16, 17, 20, 32, 48, 63, 64, 100, 256, 1000, 4099]))
        out.append((M, N, K, bool(rng.randint(2)), bool(rng.randint(2))))
    return out


@pytest.mark.parametrize("M,N,K,tA,tB", _matmul_cases(7, 200))
def test_random_matmul(M, N, K, tA, tB):
    from tsplit_amd import gpu_links, ndarray
    ctx = ndarray.gpu(0)
    rng = np.random.RandomState((M * 131 + N * 17 + K) % (2 ** 31))
    A = rng.normal(size=(K, M) if tA else (M, K)).astype(np.float32)
    B = rng.normal(size=(N, K) if tB else (K, N)).astype(np.float32)
    C = ndarray.empty((M, N), ctx)
    gpu_links.matrix_multiply(ndarray.array(A, ctx), tA, ndarray.array(B, ctx), tB, C)
    err = assert_close(C.asnumpy(), O.matmul(A, tA, B, tB), 2e-3, f"matmul {M}x{N}x{K} tA={tA} tB={tB}")
    assert err < 1e-4


def _batched_cases(seed, count):
    rng = np.random.RandomState(seed)
    out = []
    for _ in range(count):
        lead = tuple(int(v) for v in rng.randint(1, 5, size=rng.randint(1, 3)))
        out.append((lead, _dims(rng, 300), _dims(rng, 300), int(rng.choice([1, 5, 16, 17, 33, 64, 100, 130])),
                    bool(rng.randint(2)), bool(rng.randint(2))))
    return out


@pytest.mark.parametrize("lead,M,N,K,tA,tB", _batched_cases(11, 80))
def test_random_batched_matmul(lead, M, N, K, tA, tB):
    from tsplit_amd import gpu_links, ndarray
    ctx = ndarray.gpu(0)
    rng = np.random.RandomState((M * 131 + N * 17 + K + len(lead)) % (2 ** 31))
    A = rng.normal(size=lead + ((K, M) if tA else (M, K))).astype(np.float32)
    B = rng.normal(size=lead + ((N, K) if tB else (K, N))).astype(np.float32)
    C = ndarray.empty(lead + (M, N), ctx)
    gpu_links.batch_matrix_multiply(ndarray.array(A, ctx), tA, ndarray.array(B, ctx), tB, C)
    err = assert_close(C.asnumpy(), O.batch_matmul(A, tA, B, tB), 2e-3, f"batched {lead} {M}x{N}x{K} tA={tA} tB={tB}")
    assert err < 1e-4


def _pool_cases(seed, count):
    rng = np.random.RandomState(seed)
    out = []
    while len(out) < count:
        kH = int(rng.choice([1, 2, 3, 4, 5]))
        kW = kH if rng.rand() < 0.7 else int(rng.choice([1, 2, 3, 4, 5]))
        stride = int(rng.choice([1, 2, 2, 3]))
        pad = int(rng.randint(0, min(kH, kW) // 2 + 1))          # padding stays below the window
        H, W = int(rng.randint(1, 40)), int(rng.randint(1, 40))
        if H + 2 * pad < kH or W + 2 * pad < kW:
            continue
        out.append(((int(rng.choice([1, 2, 3])), int(rng.choice([1, 3, 16, 33])), H, W), kH, kW, pad, stride))
    return out


@pytest.mark.parametrize("shape,kH,kW,pad,stride", _pool_cases(3, 150))
def test_random_pooling(shape, kH, kW, pad, stride):
    from tsplit_amd import gpu_links as L, ndarray
    ctx = ndarray.gpu(0)
    rng = np.random.RandomState((shape[2] * 41 + shape[3] * 7 + kH * 3 + kW + stride) % (2 ** 31))
    ties = rng.rand() < 0.4
    x = (rng.randint(0, 3, size=shape) if ties else rng.normal(size=shape)).astype(np.float32)
    ref = O.max_pool(x, kH, kW, pad, stride)
    dy = rng.normal(size=ref.shape).astype(np.float32)
    gx, gdy = ndarray.array(x, ctx), ndarray.array(dy, ctx)
    y, dx = ndarray.empty(ref.shape, ctx), ndarray.empty(shape, ctx)
    ref_dx = O.max_pool_grad(x, dy, kH, kW, pad, stride, dtype=np.float32)
    L.max_pooling2d(gx, kH, kW, y, pad, stride)
    L.max_pooling2d_gradient(gx, gdy, kH, kW, dx, pad, stride)
    np.testing.assert_array_equal(y.asnumpy(), ref)
    np.testing.assert_array_equal(dx.asnumpy(), ref_dx)
    L.CuDNN_max_pooling2d(gx, kH, kW, y, pad, stride)
    L.CuDNN_max_pooling2d_gradient(y, gdy, gx, kH, kW, dx, pad, stride)
    np.testing.assert_array_equal(y.asnumpy(), ref)
    np.testing.assert_array_equal(dx.asnumpy(), ref_dx)
    # average pooling on the same geometry
    L.average_pooling2d(gx, kH, kW, y, pad, stride)
    L.average_pooling2d_gradient(gdy, kH, kW, dx, pad, stride)
    assert_close(y.asnumpy(), O.avg_pool(x, kH, kW, pad, stride), 1e-4, "avg_pool")
    assert_close(dx.asnumpy(), O.avg_pool_grad(dy, shape, kH, kW, pad, stride), 1e-4, "avg_pool_grad")
