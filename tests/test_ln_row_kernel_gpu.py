"""GPU parity of the workgroup-per-row layer-norm kernel (lsh_layer_norm_row_kernel(1)), through
the same C-ABI launchers and to the same bars as the default kernel: int8 codes within +-1 on
<= 0.1 % of the elements, fp16 / fp32 residuals within the tolerance of each test.
"""
import numpy as np
import pytest
import torch

import test_kernels_gpu as tk
from conftest import assert_codes_close
from helpers import DEV, to_dev, to_np

pytestmark = pytest.mark.gpu


@pytest.fixture
def row_kernel():
    from lightseq_amd import kernels
    prev = kernels.layer_norm_row_kernel(True)
    yield kernels
    kernels.layer_norm_row_kernel(prev)


def test_switch_returns_previous_setting():
    from lightseq_amd import kernels
    first = kernels.layer_norm_row_kernel(True)
    assert kernels.layer_norm_row_kernel(False) is True
    assert kernels.layer_norm_row_kernel(first) is False


@pytest.mark.parametrize("dtype", tk.DTYPES)
@pytest.mark.parametrize("post_ln", [False, True])
@pytest.mark.parametrize("shape", tk.LN_SHAPES)
def test_norm_layer_resual_i8O(oracle, rng, row_kernel, dtype, post_ln, shape):
    tk.test_norm_layer_resual_i8O(oracle, rng, dtype, post_ln, shape)


@pytest.mark.parametrize("dtype", tk.DTYPES)
@pytest.mark.parametrize("acc_dtype", [np.int8, np.int32])
@pytest.mark.parametrize("post_ln,colsum", [(False, False), (True, False), (True, True)])
@pytest.mark.parametrize("shape", tk.LN_SHAPES)
def test_residual_bias_ln_i8O(oracle, rng, row_kernel, dtype, acc_dtype, post_ln, colsum, shape):
    tk.test_residual_bias_ln_i8O(oracle, rng, dtype, acc_dtype, post_ln, colsum, shape)


@pytest.mark.parametrize("dtype", tk.DTYPES)
def test_residual_bias_ln_null_residual_bias(oracle, rng, row_kernel, dtype):
    tk.test_residual_bias_ln_null_residual_bias(oracle, rng, dtype)


@pytest.mark.parametrize("dtype", tk.DTYPES)
@pytest.mark.parametrize("colsum", [False, True])
@pytest.mark.parametrize("shape", tk.LN_SHAPES)
def test_residual_bias_ln_i32I(oracle, rng, row_kernel, dtype, colsum, shape):
    tk.test_residual_bias_ln_i32I(oracle, rng, dtype, colsum, shape)


@pytest.mark.parametrize("tokens,hidden,nparts", [(16, 1024, 8), (5, 768, 3), (64, 1024, 2), (3, 256, 4)])
def test_accumulator_planes(oracle, rng, row_kernel, tokens, hidden, nparts):
    """The planes are summed exactly: the result equals the launch on their integer sum."""
    planes = rng.integers(-60000, 60000, size=(nparts, tokens, hidden), dtype=np.int32)
    total = planes.sum(0, dtype=np.int64).astype(np.int32)
    res = (rng.standard_normal((tokens, hidden))).astype(np.float16)
    g = (1 + 0.1 * rng.standard_normal(hidden)).astype(np.float16)
    b = (0.1 * rng.standard_normal(hidden)).astype(np.float16)
    rb = (0.1 * rng.standard_normal(hidden)).astype(np.float16)
    ds, qs = 1e-5, 127 / 4.0
    want_q, want_res = oracle.residual_bias_ln_i8O(total, g, b, rb, res, ds, qs, False, None)
    outs = []
    for inp, n in ((planes, nparts), (total[None], 1)):
        resd = to_dev(res)
        out = torch.zeros((tokens, hidden), dtype=torch.int8, device=DEV)
        row_kernel.ker_residual_bias_ln_planes_i32I_i8O(to_dev(inp), n, tokens * hidden, to_dev(g), to_dev(b),
                                                        to_dev(rb), out, resd, tokens, hidden, ds, qs)
        outs.append((to_np(out), to_np(resd)))
    np.testing.assert_array_equal(outs[0][0], outs[1][0])
    np.testing.assert_array_equal(outs[0][1].view(np.uint16), outs[1][1].view(np.uint16))
    assert_codes_close(outs[0][0], want_q)
    np.testing.assert_allclose(outs[0][1].astype(np.float32), want_res.astype(np.float32), atol=8e-3, rtol=0)


def test_row_result_does_not_depend_on_the_other_rows(rng, row_kernel):
    """A row launched alone gives the bits it gives inside a larger launch."""
    tokens, hidden = 37, 1024
    acc = rng.integers(-127, 128, size=(tokens, hidden), dtype=np.int8)
    res = rng.standard_normal((tokens, hidden)).astype(np.float16)
    g = (1 + 0.1 * rng.standard_normal(hidden)).astype(np.float16)
    b = (0.1 * rng.standard_normal(hidden)).astype(np.float16)
    rb = (0.1 * rng.standard_normal(hidden)).astype(np.float16)

    def run(rows):
        resd = to_dev(res[rows])
        out = torch.zeros((len(rows), hidden), dtype=torch.int8, device=DEV)
        row_kernel.ker_residual_bias_ln_i8I_i8O_launcher(to_dev(acc[rows]), to_dev(g), to_dev(b), to_dev(rb),
                                                         out, resd, len(rows), hidden, 2.0 / 127, 127 / 4.0,
                                                         1024)
        return to_np(out), to_np(resd)

    all_q, all_r = run(np.arange(tokens))
    for r in (0, 17, 36):
        q, rr = run(np.array([r]))
        np.testing.assert_array_equal(q[0], all_q[r])
        np.testing.assert_array_equal(rr[0].view(np.uint16), all_r[r].view(np.uint16))
