"""GPU parity of DLGpuMatrixMultiply (fp32 MFMA tile engine) against the CPU oracle.
Tolerance: 2e-3 max relative error (measured errors are ~1e-6: fp32 MFMA accumulates in fp32)."""
import numpy as np
import pytest

from oracle import ops as O
from util import assert_close

pytestmark = pytest.mark.gpu
TOL = 2e-3

CASES = [
    # M, N, K
    (128, 256, 784), (128, 256, 256), (128, 10, 256),          # MLP forward
    (784, 256, 128), (256, 10, 128), (128, 256, 10),           # MLP backward shapes
    (64, 1000, 4096), (64, 4096, 4096),                        # VGG classifier (skinny, split-K)
    (1, 1, 1), (3, 5, 7), (65, 129, 17), (130, 250, 33), (200, 64, 300), (64, 300, 5000),
    # large and ragged: many tiles, split-free; a long reduction on skinny tiles
    (8192, 512, 512), (2000, 1030, 1040), (64, 4096, 8192),
]


@pytest.mark.parametrize("M,N,K", CASES)
@pytest.mark.parametrize("tA,tB", [(False, False), (False, True), (True, False), (True, True)])
def test_matmul(M, N, K, tA, tB, rng):
    from tsplit_amd import gpu_links, ndarray
    ctx = ndarray.gpu(0)
    A = rng.normal(size=(K, M) if tA else (M, K)).astype(np.float32)
    B = rng.normal(size=(N, K) if tB else (K, N)).astype(np.float32)
    C = ndarray.empty((M, N), ctx)
    gpu_links.matrix_multiply(ndarray.array(A, ctx), tA, ndarray.array(B, ctx), tB, C)
    err = assert_close(C.asnumpy(), O.matmul(A, tA, B, tB), TOL, f"matmul {M}x{N}x{K} tA={tA} tB={tB}")
    assert err < 1e-4      # fp32 accumulation: far inside the stated tolerance


def test_matmul_identity_and_linearity(rng):
    """Size-independent properties at the VGG FC1 shape: A @ I = A; (A @ (B1 + B2)) = A@B1 + A@B2."""
    from tsplit_amd import gpu_links, ndarray
    ctx = ndarray.gpu(0)
    M, K, N = 64, 25088, 4096
    A = rng.normal(size=(M, K)).astype(np.float32)
    # one-hot columns: picks columns of A exactly
    sel = rng.randint(0, K, N)
    B = np.zeros((K, N), np.float32)
    B[sel, np.arange(N)] = 1.0
    C = ndarray.empty((M, N), ctx)
    gA = ndarray.array(A, ctx)
    gpu_links.matrix_multiply(gA, False, ndarray.array(B, ctx), False, C)
    np.testing.assert_array_equal(C.asnumpy(), A[:, sel])
    B1 = rng.normal(size=(K, N)).astype(np.float32) * 0.01
    C1, C2, C12 = ndarray.empty((M, N), ctx), ndarray.empty((M, N), ctx), ndarray.empty((M, N), ctx)
    gpu_links.matrix_multiply(gA, False, ndarray.array(B1, ctx), False, C1)
    gpu_links.matrix_multiply(gA, False, ndarray.array(B, ctx), False, C2)
    gpu_links.matrix_multiply(gA, False, ndarray.array(B1 + B, ctx), False, C12)
    assert_close(C12.asnumpy(), C1.asnumpy().astype(np.float64) + C2.asnumpy(), 1e-4, "linearity")


def test_matmul_shape_mismatch():
    from tsplit_amd import gpu_links, ndarray
    ctx = ndarray.gpu(0)
    with pytest.raises(RuntimeError):
        gpu_links.matrix_multiply(ndarray.empty((4, 5), ctx), False, ndarray.empty((6, 3), ctx), False,
                                  ndarray.empty((4, 3), ctx))
