"""StridedBatchGemm forward (ops/includes/strided_batch_gemm.h:45-57): the numpy restatement is
pinned against what cuBLAS's column-major definition fixes -- a brute-force triple loop on a tiny
case for all four transposition pairs, and the two configurations the layers use read as the
row-major products they stand for (scores = alpha Q K^T, context = P V)."""
import numpy as np
import pytest

from oracle import layer_ops as lo


def _colmajor(flat, rows, cols):
    """Matrix whose column-major storage is ``flat`` (leading dimension = rows)."""
    return np.asarray(flat, np.float64).reshape(cols, rows).T


@pytest.mark.parametrize("op_a", [0, 1])
@pytest.mark.parametrize("op_b", [0, 1])
def test_against_the_column_major_definition(rng, op_a, op_b):
    bsz, m, n, k = 3, 4, 5, 6
    alpha, beta = 0.75, -0.5
    a = rng.standard_normal((bsz, m * k)).astype(np.float32)
    b = rng.standard_normal((bsz, n * k)).astype(np.float32)
    c = rng.standard_normal((bsz, m * n)).astype(np.float32)
    got = lo.strided_batch_gemm(a, b, m, n, k, alpha, beta, op_a, op_b, c)
    assert got.shape == (bsz, n, m) and got.dtype == np.float32
    for i in range(bsz):
        # cuBLAS: A is k x m (lda = k) when transposed, m x k (lda = m) when not; same for B
        am = _colmajor(a[i], k, m).T if op_a else _colmajor(a[i], m, k)
        bm = _colmajor(b[i], n, k).T if op_b else _colmajor(b[i], k, n)
        want = np.zeros((m, n))
        for r in range(m):
            for s in range(n):
                for t in range(k):
                    want[r, s] += am[r, t] * bm[t, s]
        want = alpha * want + beta * _colmajor(c[i], m, n)
        # the result array is the column-major storage of C: element (r, s) at [s, r]
        np.testing.assert_allclose(got[i].T, want, rtol=1e-5, atol=1e-5)


def test_layer_configurations_are_scores_and_context(rng):
    bh, from_len, to_len, hd = 6, 5, 7, 8
    q = rng.standard_normal((bh, from_len, hd)).astype(np.float16)
    k = rng.standard_normal((bh, to_len, hd)).astype(np.float16)
    v = rng.standard_normal((bh, to_len, hd)).astype(np.float16)
    alpha = 1.0 / np.sqrt(hd)
    # transformer_encoder_layer.cpp:34-37, :121-123: Config(alpha, 0, T, N), m = to, n = from, k = hd,
    # A = k, B = q
    sc = lo.strided_batch_gemm(k, q, to_len, from_len, hd, alpha, 0.0, 1, 0)
    want = alpha * np.einsum("bid,bjd->bij", q.astype(np.float64), k.astype(np.float64))
    assert sc.shape == (bh, from_len, to_len) and sc.dtype == np.float16
    np.testing.assert_allclose(sc.astype(np.float64), want, atol=2e-3)
    # :38-42, :139-141: Config(1, 0, N, N), m = hd, n = from, k = to, A = v, B = probabilities
    p = rng.random((bh, from_len, to_len)).astype(np.float16)
    ctx = lo.strided_batch_gemm(v, p, hd, from_len, to_len, 1.0, 0.0, 0, 0)
    want = np.einsum("bij,bjd->bid", p.astype(np.float64), v.astype(np.float64))
    assert ctx.shape == (bh, from_len, hd)
    np.testing.assert_allclose(ctx.astype(np.float64), want, atol=4e-3)
