"""GPU parity of the int8 MFMA GEMM through the C ABI.

int32 accumulators are bit-exact against the oracle's integer triple loop (small
shapes) and against an exact float64 BLAS product (large shapes: |acc| <= K*127^2
< 2^53, so the float64 product of integer matrices is exact).  int8 outputs follow
clamp(floor(acc*alpha + 0.5), -127, 127) bit-exactly given exact accumulators.
"""
import numpy as np
import pytest
import torch

from helpers import DEV, to_dev, to_np

pytestmark = pytest.mark.gpu

SMALL = [(1, 1, 16), (3, 5, 16), (32, 32, 32), (33, 31, 48), (64, 16, 128), (130, 70, 144),
         (257, 129, 272), (300, 513, 400), (128, 256, 1024)]
LARGE = [(4096, 2304, 768), (4096, 768, 768), (4096, 3072, 768), (4096, 768, 3072),
         (512, 1536, 512), (512, 2048, 512), (4096, 4096, 1024), (4096, 1024, 4096),
         (1000, 30522 // 6, 128), (64, 1000, 1024)]


def _k():
    from lightseq_amd import kernels
    return kernels


def _exact_i32(a, w):
    return np.rint(a.astype(np.float64) @ w.astype(np.float64).T).astype(np.int64)


@pytest.mark.parametrize("M,N,K", SMALL)
def test_gemm_i32_small_vs_oracle(oracle, rng, M, N, K):
    a = rng.integers(-127, 128, size=(M, K), dtype=np.int8)
    w = rng.integers(-127, 128, size=(N, K), dtype=np.int8)
    want = oracle.gemm_i8_i32(a, w)
    np.testing.assert_array_equal(want, _exact_i32(a, w))  # the oracle itself, against BLAS
    c = torch.full((M, N), 7, dtype=torch.int32, device=DEV)
    _k().gemm_i8_i32o(to_dev(a), to_dev(w), c, M, N, K)
    np.testing.assert_array_equal(to_np(c), want)


@pytest.mark.parametrize("M,N,K", SMALL)
def test_gemm_i8_small_vs_oracle(oracle, rng, M, N, K):
    a = rng.integers(-127, 128, size=(M, K), dtype=np.int8)
    w = rng.integers(-127, 128, size=(N, K), dtype=np.int8)
    alpha = 3.0 / (np.sqrt(K) * 127)
    want = oracle.gemm_i8_i8(a, w, alpha)
    c = torch.full((M, N), 7, dtype=torch.int8, device=DEV)
    _k().gemm_i8_i8o(to_dev(a), to_dev(w), c, M, N, K, alpha)
    np.testing.assert_array_equal(to_np(c), want)


@pytest.mark.parametrize("M,N,K", LARGE)
def test_gemm_large_exact(rng, M, N, K):
    a = rng.integers(-127, 128, size=(M, K), dtype=np.int8)
    w = rng.integers(-127, 128, size=(N, K), dtype=np.int8)
    ref = _exact_i32(a, w)
    c = torch.zeros((M, N), dtype=torch.int32, device=DEV)
    _k().gemm_i8_i32o(to_dev(a), to_dev(w), c, M, N, K)
    np.testing.assert_array_equal(to_np(c).astype(np.int64), ref)
    alpha = np.float32(4.0 * 0.08 / (6.0 * 127))
    f = ref.astype(np.float32) * alpha  # |acc| < 2^24 for K <= 1024; larger K: same float cast as the kernel
    want8 = np.clip(np.floor(f + np.float32(0.5)), -127, 127).astype(np.int8)
    c8 = torch.zeros((M, N), dtype=torch.int8, device=DEV)
    _k().gemm_i8_i8o(to_dev(a), to_dev(w), c8, M, N, K, float(alpha))
    np.testing.assert_array_equal(to_np(c8), want8)


def test_gemm_extreme_values(rng):
    """All-(-127) x all-(-127) at K=4096 reaches the largest accumulator of the path."""
    M, N, K = 64, 64, 4096
    a = np.full((M, K), -127, np.int8)
    w = np.full((N, K), -127, np.int8)
    c = torch.zeros((M, N), dtype=torch.int32, device=DEV)
    _k().gemm_i8_i32o(to_dev(a), to_dev(w), c, M, N, K)
    assert np.all(to_np(c) == K * 127 * 127)


def test_gemm_linearity(rng):
    """Size-independent property at full size: (A1 + A2) W^T == A1 W^T + A2 W^T."""
    M, N, K = 4096, 3072, 768
    a1 = rng.integers(-60, 61, size=(M, K), dtype=np.int8)
    a2 = rng.integers(-60, 61, size=(M, K), dtype=np.int8)
    w = rng.integers(-127, 128, size=(N, K), dtype=np.int8)
    wd = to_dev(w)
    outs = []
    for a in (a1, a2, (a1 + a2).astype(np.int8)):
        c = torch.zeros((M, N), dtype=torch.int32, device=DEV)
        _k().gemm_i8_i32o(to_dev(a), wd, c, M, N, K)
        outs.append(c)
    assert torch.equal(outs[0] + outs[1], outs[2])


def test_gemm_rejects_bad_k():
    from lightseq_amd.lib import LSHError
    a = torch.zeros((4, 8), dtype=torch.int8, device=DEV)
    c = torch.zeros((4, 4), dtype=torch.int32, device=DEV)
    with pytest.raises(LSHError):
        _k().gemm_i8_i32o(a, a, c, 4, 4, 8)
