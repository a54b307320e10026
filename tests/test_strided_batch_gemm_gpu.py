"""GPU parity of lsh_strided_batch_gemm_f16 / _f32 (StridedBatchGemm<T>::Forward) against the
numpy restatement: float32 accumulation on both sides, so fp32 results agree to summation
order and fp16 results to one rounding of the output."""
import numpy as np
import pytest
import torch

from helpers import DEV, to_dev, to_np, torch_dtype

pytestmark = pytest.mark.gpu


def _lo():
    from oracle import layer_ops
    return layer_ops


def _ops():
    from lightseq_amd import ops
    return ops


@pytest.mark.parametrize("dtype", [np.float16, np.float32])
@pytest.mark.parametrize("op_a,op_b", [(1, 0), (0, 0), (0, 1), (1, 1)])
@pytest.mark.parametrize("bsz,m,n,k", [(24, 40, 33, 64), (5, 64, 128, 200), (3, 7, 1, 5)])
def test_strided_batch_gemm(rng, dtype, op_a, op_b, bsz, m, n, k):
    a = rng.standard_normal((bsz, m * k)).astype(dtype)
    b = rng.standard_normal((bsz, n * k)).astype(dtype)
    alpha = 1.0 / np.sqrt(k)
    want = _lo().strided_batch_gemm(a, b, m, n, k, alpha, 0.0, op_a, op_b)
    out = torch.zeros(bsz, n, m, dtype=torch_dtype(dtype), device=DEV)
    _ops().strided_batch_gemm(bsz, m, n, k, alpha, 0.0, op_a, op_b, to_dev(a), to_dev(b), out)
    tol = 2e-3 if dtype == np.float16 else 1e-5
    np.testing.assert_allclose(to_np(out).astype(np.float64), want.astype(np.float64), atol=tol,
                               rtol=tol)
    # beta: accumulate onto the previous output
    want2 = _lo().strided_batch_gemm(a, b, m, n, k, alpha, 0.5, op_a, op_b, to_np(out))
    _ops().strided_batch_gemm(bsz, m, n, k, alpha, 0.5, op_a, op_b, to_dev(a), to_dev(b), out)
    np.testing.assert_allclose(to_np(out).astype(np.float64), want2.astype(np.float64),
                               atol=2 * tol, rtol=2 * tol)


def test_scores_softmax_context_chain_equals_the_fused_attention(rng):
    """The operator chain of the reference layer (StridedBatchGemm, launch_attn_softmax,
    StridedBatchGemm, launch_transform4d_0213) against the fused kernel the layers here run."""
    batch, heads, seq, hd = 2, 4, 72, 64
    q, k, v = (rng.standard_normal((batch * heads, seq, hd)).astype(np.float16) for _ in range(3))
    pad = np.zeros((batch, seq), np.float32)
    pad[1, 50:] = -1e8
    with np.errstate(over="ignore"):
        pad = pad.astype(np.float16)
    ops = _ops()
    sc = torch.zeros(batch, heads, seq, seq, dtype=torch.float16, device=DEV)
    ops.strided_batch_gemm(batch * heads, seq, seq, hd, 1.0 / np.sqrt(hd), 0.0, 1, 0, to_dev(k),
                           to_dev(q), sc)
    ops.launch_attn_softmax(sc, to_dev(pad), batch, heads, seq, seq, False)
    ctx = torch.zeros(batch * heads, seq, hd, dtype=torch.float16, device=DEV)
    ops.strided_batch_gemm(batch * heads, hd, seq, seq, 1.0, 0.0, 0, 0, to_dev(v), sc, ctx)
    merged = torch.zeros(batch, seq, heads * hd, dtype=torch.float16, device=DEV)
    ops.launch_transform4d_0213(merged, ctx, batch, seq, heads * hd, heads, 1)
    fused = torch.zeros_like(merged)
    ops.layer_attention(to_dev(q), to_dev(k), to_dev(v), to_dev(pad), fused, batch, seq, heads, hd)
    np.testing.assert_allclose(to_np(merged).astype(np.float64), to_np(fused).astype(np.float64),
                               atol=3e-3)


def test_strided_batch_gemm_argument_errors():
    from lightseq_amd import lib
    t = torch.zeros(64, dtype=torch.half, device=DEV)
    with pytest.raises(lib.LSHError, match="op must be"):
        _ops().strided_batch_gemm(1, 4, 4, 4, 1.0, 0.0, 2, 0, t, t, t)
    with pytest.raises(lib.LSHError, match="bad arguments"):
        _ops().strided_batch_gemm(1, 0, 4, 4, 1.0, 0.0, 0, 0, t, t, t)
