"""CPU checks that pin the oracle's sparse products and dropout.

Sparse: scipy's CSR products (the reference's own CPU path) against dense float64 products and
against a literal walk of the CSR arrays, all four transpose combinations, empty rows included.
Dropout: the generator against the published Philox-4x32-10 known-answer vectors (Random123
kat_vectors), then the arithmetic: survivors scaled by 1/(1-p), the rest exactly zero, the
same mask on every call, the gradient gated by the forward mask, the dropped fraction within
five standard deviations of p.  Which elements cuDNN would drop is not checkable here."""
import numpy as np
import pytest
import scipy.sparse

from oracle import loops as LP
from oracle import ops as O

def _load_kat():
    import json
    import os
    with open(os.path.join(os.path.dirname(__file__), "golden", "philox4x32_10_kat.json")) as f:
        doc = json.load(f)
    h = lambda words: tuple(int(w, 16) for w in words)
    return [(h(v["counter"]), h(v["key"]), h(v["output"])) for v in doc["vectors"]]


PHILOX_KAT = _load_kat()


@pytest.mark.parametrize("ctr,key,expect", PHILOX_KAT)
def test_philox_known_answers(ctr, key, expect):
    out = O.philox4x32_10(*ctr, *key)
    assert tuple(int(v) for v in out) == expect


def test_philox_vectorised_equals_scalar():
    idx = np.array([0, 1, 2, 77, 2**32 - 1], dtype=np.uint64)
    vec = O.philox4x32_10(idx, idx * 0 + 5, idx * 0, idx * 0, 11, 22)
    for n, i in enumerate(idx):
        one = O.philox4x32_10(int(i), 5, 0, 0, 11, 22)
        assert [int(w[n]) for w in vec] == [int(w) for w in one]


@pytest.mark.parametrize("p", [0.0, 0.1, 0.3, 0.5, 0.9, 1.0])
def test_dropout_arithmetic_and_fraction(p, rng):
    n = 200003
    x = rng.normal(size=n).astype(np.float32) + 3.0     # no zeros among the inputs
    y, keep = O.dropout(x, p, dtype=np.float32)
    assert keep.dtype == bool and keep.shape == x.shape
    if p < 1.0:
        scale = np.float32(1) / (np.float32(1) - np.float32(p))
        assert np.array_equal(y[keep], x[keep] * scale)
    assert np.all(y[~keep] == 0)
    dropped = 1.0 - keep.mean()
    assert abs(dropped - p) <= 5 * np.sqrt(max(p * (1 - p), 1e-12) / n) + 1e-9
    y2, keep2 = O.dropout(x, p, dtype=np.float32)
    assert np.array_equal(keep, keep2) and np.array_equal(y, y2)          # re-seeded on every call
    dy = rng.normal(size=n).astype(np.float32)
    dx = O.dropout_grad(dy, p, keep, dtype=np.float32)
    assert np.all(dx[~keep] == 0)
    if p < 1.0:
        assert np.array_equal(dx[keep], dy[keep] * scale)


def test_dropout_mask_is_a_prefix_property():
    """Element i depends on i alone: a shorter tensor sees the first bits of a longer one."""
    a, b = O.dropout_mask(1000, 0.4), O.dropout_mask(37, 0.4)
    assert np.array_equal(a[:37], b)
    # a lower drop probability keeps every element a higher one keeps
    assert np.all(O.dropout_mask(5000, 0.2)[O.dropout_mask(5000, 0.6)])


def _random_csr(rng, nrow, ncol, density, empty_rows=()):
    m = scipy.sparse.random(nrow, ncol, density=density, format="csr", dtype=np.float32,
                            random_state=rng, data_rvs=lambda k: rng.normal(size=k).astype(np.float32))
    m = m.tolil()
    for r in empty_rows:
        m[r, :] = 0
    m = m.tocsr()
    m.eliminate_zeros()
    m.sort_indices()
    return m


@pytest.mark.parametrize("trans", [False, True])
def test_csrmv_against_dense_and_loops(trans, rng):
    m = _random_csr(rng, 13, 9, 0.3, empty_rows=(0, 5))
    x = rng.normal(size=13 if trans else 9).astype(np.float32)
    got = O.csrmv(m.data, m.indptr, m.indices, 13, 9, trans, x)
    dense = m.toarray().astype(np.float64)
    want = (dense.T if trans else dense) @ x.astype(np.float64)
    assert np.allclose(got, want, rtol=1e-12, atol=1e-12)
    assert np.allclose(got, LP.csrmv_loops(m.data, m.indptr, m.indices, 13, 9, trans, x), rtol=1e-12, atol=1e-12)


@pytest.mark.parametrize("transA", [False, True])
@pytest.mark.parametrize("transB", [False, True])
def test_csrmm_against_dense_and_loops(transA, transB, rng):
    nrow, ncol, n = 11, 7, 5
    m = _random_csr(rng, nrow, ncol, 0.35, empty_rows=(3,))
    inner = nrow if transA else ncol
    B = rng.normal(size=(n, inner) if transB else (inner, n)).astype(np.float32)
    got = O.csrmm(m.data, m.indptr, m.indices, nrow, ncol, transA, B, transB)
    dense = m.toarray().astype(np.float64)
    want = (dense.T if transA else dense) @ (B.T if transB else B).astype(np.float64)
    assert got.shape == want.shape
    assert np.allclose(got, want, rtol=1e-12, atol=1e-12)
    assert np.allclose(got, LP.csrmm_loops(m.data, m.indptr, m.indices, nrow, ncol, transA, B, transB),
                       rtol=1e-12, atol=1e-12)


def test_csr_identity_and_permutation():
    """Closed forms: the identity returns its operand; a permutation matrix permutes rows."""
    n = 6
    eye = scipy.sparse.identity(n, dtype=np.float32, format="csr")
    B = np.arange(n * 3, dtype=np.float32).reshape(n, 3)
    assert np.array_equal(O.csrmm(eye.data, eye.indptr, eye.indices, n, n, False, B, False), B)
    perm = np.array([2, 0, 5, 1, 4, 3])
    P = scipy.sparse.csr_matrix((np.ones(n, np.float32), (np.arange(n), perm)), shape=(n, n))
    assert np.array_equal(O.csrmm(P.data, P.indptr, P.indices, n, n, False, B, False), B[perm])
    assert np.array_equal(O.csrmv(P.data, P.indptr, P.indices, n, n, True, B[:, 0])[perm], B[:, 0])
