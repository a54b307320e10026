"""GPU parity: every fused HIP kernel of the encoder path against the CPU oracle,
called through the C ABI, on seeded inputs.

Bars: int8 outputs within +-1 code on <= 0.1 % of elements; fp16/fp32 outputs
within the absolute tolerance written in each test.
"""
import numpy as np
import pytest
import torch

from conftest import assert_codes_close
from helpers import DEV, to_dev, to_np

pytestmark = pytest.mark.gpu

DTYPES = [np.float16, np.float32]
# (tokens, hidden): vector path (hidden % 256 == 0), ragged vector path, scalar fallback
LN_SHAPES = [(37, 768), (64, 512), (5, 1024), (9, 200), (3, 2048), (4, 77)]


def _k():
    from lightseq_amd import kernels
    return kernels


def _randT(rng, shape, dtype, scale=1.0):
    return (rng.standard_normal(shape) * scale).astype(dtype)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("n", [0, 1, 7, 8 * 1000 + 3, 512 * 768])
def test_quantize_tensor(oracle, rng, dtype, n):
    x = _randT(rng, (n,), dtype, 2.0)
    qs = 127 / 4.0
    want = oracle.quantize_tensor(x, qs)
    out = torch.zeros(max(n, 1), dtype=torch.int8, device=DEV)
    xd = to_dev(x) if n else torch.zeros(1, dtype=torch.float16 if dtype == np.float16 else torch.float32, device=DEV)
    _k().launch_quantize_tensor(xd, out, 1, n, qs)
    np.testing.assert_array_equal(to_np(out)[:n], want)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("n", [1, 5, 4 * 999 + 2, 256 * 768])
def test_dequantize_tensor(oracle, rng, dtype, n):
    x = rng.integers(-2**24, 2**24, size=n, dtype=np.int32)
    ds = 4.0 * 0.08 / (127 * 127)
    want = oracle.dequantize_tensor(x, ds, dtype)
    out = torch.zeros(n, dtype=torch.float16 if dtype == np.float16 else torch.float32, device=DEV)
    _k().launch_dequantize_tensor(to_dev(x), out, 1, n, ds)
    got = to_np(out)
    # one rounding of an exactly representable product order: allow 1 ulp of T
    np.testing.assert_allclose(got.astype(np.float64), want.astype(np.float64), rtol=2e-3 if dtype == np.float16 else 2e-7, atol=1e-7)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("post_ln", [False, True])
@pytest.mark.parametrize("shape", LN_SHAPES)
def test_norm_layer_resual_i8O(oracle, rng, dtype, post_ln, shape):
    tokens, hidden = shape
    x = _randT(rng, shape, dtype, 1.5)
    g = (1 + 0.1 * rng.standard_normal(hidden)).astype(dtype)
    b = _randT(rng, (hidden,), dtype, 0.1)
    rb = _randT(rng, (hidden,), dtype, 0.1)
    qs = 127 / 4.0
    want_q, want_res = oracle.norm_layer_resual_i8O(x, g, b, rb, qs, post_ln)
    xd = to_dev(x)
    out = torch.zeros(shape, dtype=torch.int8, device=DEV)
    _k().ker_norm_layer_resual_i8O_launcher(tokens, hidden, xd, out, to_dev(g), to_dev(b), to_dev(rb),
                                            1024, qs, post_ln)
    assert_codes_close(to_np(out), want_q)
    np.testing.assert_allclose(to_np(xd).astype(np.float32), want_res.astype(np.float32),
                               atol=4e-3 if dtype == np.float16 else 2e-5, rtol=0)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("acc_dtype", [np.int8, np.int32])
@pytest.mark.parametrize("post_ln,colsum", [(False, False), (True, False), (True, True)])
@pytest.mark.parametrize("shape", LN_SHAPES)
def test_residual_bias_ln_i8O(oracle, rng, dtype, acc_dtype, post_ln, colsum, shape):
    tokens, hidden = shape
    if acc_dtype == np.int8:
        acc = rng.integers(-127, 128, size=shape, dtype=np.int8)
        ds = 2.0 / 127
    else:
        acc = rng.integers(-200000, 200000, size=shape, dtype=np.int32)
        ds = 1e-5
    res = _randT(rng, shape, dtype, 1.0)
    g = (1 + 0.1 * rng.standard_normal(hidden)).astype(dtype)
    b = _randT(rng, (hidden,), dtype, 0.1)
    rb = _randT(rng, (hidden,), dtype, 0.1)
    cs = _randT(rng, (hidden,), dtype, 0.2) if colsum else None
    qs = 127 / 4.0
    want_q, want_res = oracle.residual_bias_ln_i8O(acc, g, b, rb, res, ds, qs, post_ln, cs)
    resd = to_dev(res)
    out = torch.zeros(shape, dtype=torch.int8, device=DEV)
    fn = (_k().ker_residual_bias_ln_i8I_i8O_launcher if acc_dtype == np.int8
          else _k().ker_residual_bias_ln_i32I_i8O_launcher)
    fn(to_dev(acc), to_dev(g), to_dev(b), to_dev(rb), out, resd, tokens, hidden, ds, qs, 1024,
       post_ln, False, False, None if cs is None else to_dev(cs))
    assert_codes_close(to_np(out), want_q)
    np.testing.assert_allclose(to_np(resd).astype(np.float32), want_res.astype(np.float32),
                               atol=8e-3 if dtype == np.float16 else 2e-5, rtol=0)


@pytest.mark.parametrize("dtype", DTYPES)
def test_residual_bias_ln_null_residual_bias(oracle, rng, dtype):
    shape = (17, 768)
    acc = rng.integers(-127, 128, size=shape, dtype=np.int8)
    res = _randT(rng, shape, dtype)
    g = np.ones(768, dtype)
    b = np.zeros(768, dtype)
    want_q, want_res = oracle.residual_bias_ln_i8O(acc, g, b, None, res, 0.01, 30.0, True, None)
    resd = to_dev(res)
    out = torch.zeros(shape, dtype=torch.int8, device=DEV)
    _k().ker_residual_bias_ln_i8I_i8O_launcher(to_dev(acc), to_dev(g), to_dev(b), None, out, resd, 17,
                                               768, 0.01, 30.0, 1024, True)
    assert_codes_close(to_np(out), want_q)
    np.testing.assert_allclose(to_np(resd).astype(np.float32), want_res.astype(np.float32), atol=8e-3)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("colsum", [False, True])
@pytest.mark.parametrize("shape", LN_SHAPES)
def test_residual_bias_ln_i32I(oracle, rng, dtype, colsum, shape):
    tokens, hidden = shape
    acc = rng.integers(-200000, 200000, size=shape, dtype=np.int32)
    res = _randT(rng, shape, dtype, 1.0)
    g = (1 + 0.1 * rng.standard_normal(hidden)).astype(dtype)
    b = _randT(rng, (hidden,), dtype, 0.1)
    cs = _randT(rng, (hidden,), dtype, 0.2) if colsum else None
    want = oracle.residual_bias_ln_i32I(acc, g, b, res, 1e-5, cs)
    resd = to_dev(res)  # in place, as the reference calls it
    _k().ker_residual_bias_ln_i32I_launcher(to_dev(acc), to_dev(g), to_dev(b), resd, resd, tokens,
                                            hidden, 1e-5, 1024, False,
                                            None if cs is None else to_dev(cs))
    np.testing.assert_allclose(to_np(resd).astype(np.float32), want.astype(np.float32),
                               atol=4e-3 if dtype == np.float16 else 2e-5, rtol=0)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("shape", [(33, 3072), (7, 2048), (5, 100), (1, 16)])
def test_bias_gelu(oracle, rng, dtype, shape):
    tokens, feat = shape
    x = rng.integers(-127, 128, size=shape, dtype=np.int8)
    bias = _randT(rng, (feat,), dtype, 0.3)
    ds, qs = 2.2 / 127, 127 / 2.2
    want = oracle.bias_gelu_i8I_i8O(x, bias, ds, qs)
    out = torch.zeros(shape, dtype=torch.int8, device=DEV)
    _k().ker_bias_gelu_i8I_i8O_launcher(tokens, to_dev(x), out, to_dev(bias), feat, ds, qs)
    assert_codes_close(to_np(out), want)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("shape", [(4096, 3072), (1024, 64), (1500, 192), (5000, 1088), (2049, 320), (3000, 1280), (16500, 256), (20000, 64), (16384, 3072), (40001, 128), (20011, 1024), (16500, 512)])
def test_bias_gelu_tabulated_equals_evaluated(oracle, rng, dtype, shape):
    """With 1024 rows or more the kernel looks the codes up in per-column tables built in LDS:
    the same bytes as evaluating every element (all 256 input codes occur, -128 included), in
    place as well, and within the oracle's tolerance."""
    tokens, feat = shape
    x = rng.integers(-128, 128, size=shape, dtype=np.int8)
    bias = _randT(rng, (feat,), dtype, 0.3)
    ds, qs = 2.2 / 127, 127 / 2.2
    xd, bd = to_dev(x), to_dev(bias)
    tab = torch.zeros(shape, dtype=torch.int8, device=DEV)
    ev = torch.zeros(shape, dtype=torch.int8, device=DEV)
    k = _k()
    k.ker_bias_gelu_i8I_i8O_launcher(tokens, xd, tab, bd, feat, ds, qs)
    prev = k.bias_act_lut_kernel(False)
    try:
        k.ker_bias_gelu_i8I_i8O_launcher(tokens, xd, ev, bd, feat, ds, qs)
    finally:
        k.bias_act_lut_kernel(prev)
    assert prev is True
    assert torch.equal(tab, ev)
    inplace = xd.clone()
    k.ker_bias_gelu_i8I_i8O_launcher(tokens, inplace, inplace, bd, feat, ds, qs)
    assert torch.equal(inplace, ev)
    valid = x != -128  # the oracle's domain is the symmetric code range
    assert_codes_close(to_np(tab)[valid], oracle.bias_gelu_i8I_i8O(np.where(valid, x, 0).astype(np.int8), bias, ds, qs)[valid])


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("narrow", [False, True])
@pytest.mark.parametrize("shape", [(33, 2048), (5, 100)])
def test_bias_relu(oracle, rng, dtype, narrow, shape):
    tokens, feat = shape
    x = rng.integers(-127, 128, size=shape, dtype=np.int8)
    bias = _randT(rng, (feat,), dtype, 0.3)
    clip = 2.0
    ds, qs = 2.2 / 127, 127 / clip
    want = oracle.bias_relu_i8I_i8O(x, bias, ds, qs, clip, narrow)
    out = torch.zeros(shape, dtype=torch.int8, device=DEV)
    _k().ker_bias_relu_i8I_i8O_launcher(tokens, to_dev(x), out, to_dev(bias), feat, ds, qs, clip,
                                        False, False, narrow)
    assert_codes_close(to_np(out), want)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("B,S,h,d", [(3, 17, 12, 64), (2, 5, 4, 6), (1, 128, 8, 64), (3, 128, 12, 64), (2, 50, 8, 32),
                                     (2, 100, 3, 128), (5, 33, 6, 64), (2, 300, 4, 64)])
def test_arrange_encself_qkv(oracle, rng, dtype, B, S, h, d):
    H = h * d
    ori = rng.integers(-127, 128, size=(B * S, 3 * H), dtype=np.int8)
    bias = _randT(rng, (3 * H,), dtype, 0.3)
    ds = 2.2 / 127
    want = oracle.arrange_encself_qkv_i8I(ori, bias, B, S, h, ds)
    out = torch.zeros((3, B, h, S, d), dtype=torch.float16 if dtype == np.float16 else torch.float32,
                      device=DEV)
    _k().ker_arrange_encself_qkv_i8I_launcher(B * S, H, to_dev(ori), to_dev(bias), out, B * S * H, S, d,
                                              h, 1024, ds)
    np.testing.assert_allclose(to_np(out).astype(np.float32), want.astype(np.float32),
                               atol=2e-3 if dtype == np.float16 else 1e-6, rtol=0)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("B,S,h,d", [(2, 19, 16, 64), (2, 5, 4, 6)])
def test_arrange_encself_qkv_i8O(oracle, rng, dtype, B, S, h, d):
    H = h * d
    ori = rng.integers(-127, 128, size=(B * S, 3 * H), dtype=np.int8)
    bias = _randT(rng, (3 * H,), dtype, 0.3)
    ds, qs = 2.2 / 127, 127 / 2.5
    wq, wk, wv, wdv = oracle.arrange_encself_qkv_i8I_i8O(ori, bias, B, S, h, ds, qs)
    tdt = torch.float16 if dtype == np.float16 else torch.float32
    q, k, v = (torch.zeros((B, h, S, d), dtype=torch.int8, device=DEV) for _ in range(3))
    dv = torch.zeros((B, h, S, d), dtype=tdt, device=DEV)
    _k().ker_arrange_encself_qkv_i8I_i8O_launcher(B * S, H, to_dev(ori), to_dev(bias), q, k, v, dv, S, d,
                                                  h, 1024, ds, qs)
    assert_codes_close(to_np(q), wq)
    assert_codes_close(to_np(k), wk)
    assert_codes_close(to_np(v), wv)
    # d_v is the dequantised v; where codes agree it must match to 1 ulp of T
    same = to_np(v) == wv
    np.testing.assert_allclose(to_np(dv).astype(np.float32)[same], wdv.astype(np.float32)[same],
                               atol=2e-3 if dtype == np.float16 else 1e-6, rtol=0)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("B,S,h,d", [(3, 17, 12, 64), (2, 5, 4, 6)])
def test_arrange_atten_output(oracle, rng, dtype, B, S, h, d):
    x = _randT(rng, (B, h, S, d), dtype, 0.3)
    qs = 127 / 1.0
    want = oracle.arrange_atten_output_i8O(x, qs)
    out = torch.zeros((B * S, h * d), dtype=torch.int8, device=DEV)
    _k().ker_arrange_atten_output_i8O_launcher(B * S, h * d, to_dev(x), out, S, d, h, 1024, qs)
    np.testing.assert_array_equal(to_np(out), want)


def _pad_mask(rng, B, S):
    lens = rng.integers(max(1, S // 4), S + 1, size=B)
    lens[0] = S
    return (np.arange(S)[None, :] >= lens[:, None]).astype(np.int32)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("B,S,h", [(3, 128, 4), (2, 33, 3), (1, 300, 2), (2, 1, 2)])
def test_correlation_softmax_encself(oracle, rng, dtype, B, S, h):
    c = _randT(rng, (B, h, S, S), dtype, 2.0)
    mask = _pad_mask(rng, B, S)
    want = oracle.correlation_softmax_encself(c, mask)
    cd = to_dev(c)
    _k().ker_correlation_softmax_encself_launcher(B, S, h, cd, to_dev(mask))
    np.testing.assert_allclose(to_np(cd).astype(np.float32), want.astype(np.float32),
                               atol=1e-3 if dtype == np.float16 else 1e-6, rtol=0)
    # textbook property: valid rows sum to one over valid keys, padded rows are zero
    got = to_np(cd).astype(np.float64)
    for b in range(B):
        valid = mask[b] == 0
        np.testing.assert_allclose(got[b][:, valid, :].sum(-1), 1.0, atol=5e-3)
        assert np.all(got[b][:, ~valid, :] == 0) and np.all(got[b][:, :, ~valid] == 0)


@pytest.mark.parametrize("B,S,h,d", [(2, 128, 3, 64), (3, 50, 2, 64), (1, 200, 2, 64), (2, 64, 4, 32),
                                     (1, 7, 1, 64)])
def test_encself_attention_fused(oracle, rng, B, S, h, d):
    """Fused attention == the reference's 4-step sequence (scores GEMM -> softmax ->
    context GEMM -> arrange+quant) as the oracle restates it."""
    q = _randT(rng, (B, h, S, d), np.float16, 0.6)
    k = _randT(rng, (B, h, S, d), np.float16, 0.6)
    v = _randT(rng, (B, h, S, d), np.float16, 0.6)
    mask = _pad_mask(rng, B, S)
    scores = oracle.attn_scores(q, k, np.sqrt(1.0 / d))
    probs = oracle.correlation_softmax_encself(scores, mask)
    want_ctx = oracle.attn_context(probs, v)
    qs = 127 / 0.5
    want_q = oracle.arrange_atten_output_i8O(want_ctx, qs)
    ctx = torch.zeros((B, h, S, d), dtype=torch.float16, device=DEV)
    ctx_q = torch.zeros((B * S, h * d), dtype=torch.int8, device=DEV)
    _k().encself_attention(to_dev(q), to_dev(k), to_dev(v), to_dev(mask), ctx, ctx_q, qs, B, S, h, d)
    got = to_np(ctx).astype(np.float32)
    np.testing.assert_allclose(got, want_ctx.astype(np.float32), atol=2e-3, rtol=0)
    # the int8 output quantises the fused kernel's own fp16 context
    np.testing.assert_array_equal(to_np(ctx_q), oracle.arrange_atten_output_i8O(to_np(ctx), qs))
    assert_codes_close(to_np(ctx_q), want_q, max_frac=5e-3)
    # padded queries give exact zeros
    for b in range(B):
        assert np.all(got[b][:, mask[b] == 1, :] == 0)


@pytest.mark.parametrize("B,S,h", [(2, 128, 4), (3, 50, 6), (8, 128, 12), (1, 7, 4), (16, 96, 4),
                                   (5, 128, 16)])
def test_qkv_projection_and_attention_in_one_kernel(rng, B, S, h):
    """lsh_qkv_attention_i8 == the int8-output QKV GEMM followed by the attention on its codes,
    byte for byte (the chain of quant_bert_encoder.cc.cu:305-347)."""
    d = 64
    H = h * d
    x = rng.integers(-127, 128, size=(B * S, H), dtype=np.int8)
    w = rng.integers(-127, 128, size=(3 * H, H), dtype=np.int8)
    bias = _randT(rng, (3 * H,), np.float16, 0.3)
    mask = _pad_mask(rng, B, S)
    # accumulators of K = H random products spread ~ 127^2 sqrt(H) / 3: alpha brings them to codes
    alpha = 127.0 / (3.0 * 127 * 127 * np.sqrt(H) / 3.0)
    ds, qs = 1.4 / 127, 127 / 0.9
    xd, wd, bd, md = to_dev(x), to_dev(w), to_dev(bias), to_dev(mask)
    codes = torch.zeros((B * S, 3 * H), dtype=torch.int8, device=DEV)
    _k().gemm_i8_i8o(xd, wd, codes, B * S, 3 * H, H, alpha)
    assert 20 < float(codes.float().abs().mean()) < 100          # the codes use their range
    want = torch.full((B * S, H), 7, dtype=torch.int8, device=DEV)
    _k().encself_attention_i8qkv(codes, bd, ds, md, None, want, qs, B, S, h, d)
    got = torch.full((B * S, H), 9, dtype=torch.int8, device=DEV)
    _k().qkv_attention_i8(xd, wd, bd, md, got, alpha, ds, qs, B, S, h, d)
    np.testing.assert_array_equal(to_np(got), to_np(want))
    assert to_np(got).any()


@pytest.mark.parametrize("B,S,h,lens", [(4, 128, 4, [128, 97, 33, 1]), (3, 50, 4, [50, 17, 32]),
                                        (8, 128, 12, [128, 64, 65, 96, 32, 31, 100, 5])])
def test_qkv_projection_and_attention_against_the_oracle(oracle, rng, B, S, h, lens):
    """lsh_qkv_attention_i8 against the oracle's chain (int8 GEMM -> arrange + dequantise ->
    scores -> masked soft-max -> context -> merge + quantise; transformerKernels.cc.cu:1119-1172
    for the mask) on right-padded sequences of ragged lengths: valid rows to the int8 bar, rows
    of padded queries exactly zero."""
    d = 64
    H = h * d
    x = rng.integers(-127, 128, size=(B * S, H), dtype=np.int8)
    w = rng.integers(-127, 128, size=(3 * H, H), dtype=np.int8)
    bias = _randT(rng, (3 * H,), np.float16, 0.3)
    mask = (np.arange(S)[None, :] >= np.asarray(lens)[:, None]).astype(np.int32)
    alpha = 127.0 / (127 * 127 * np.sqrt(H) / 3.0)
    ds, qs = 1.4 / 127, 127 / 0.9
    codes = oracle.gemm_i8_i8(x, w, alpha)
    qkv = oracle.arrange_encself_qkv_i8I(codes, bias, B, S, h, ds)
    probs = oracle.correlation_softmax_encself(oracle.attn_scores(qkv[0], qkv[1], np.sqrt(1.0 / d)), mask)
    want = oracle.arrange_atten_output_i8O(oracle.attn_context(probs, qkv[2]), qs)
    got = torch.full((B * S, H), 9, dtype=torch.int8, device=DEV)
    _k().qkv_attention_i8(to_dev(x), to_dev(w), to_dev(bias), to_dev(mask), got, alpha, ds, qs, B, S, h, d)
    got = to_np(got)
    valid = (mask == 0).reshape(-1)
    assert_codes_close(got[valid], want[valid], max_frac=5e-3, what="context codes")
    assert np.abs(got[valid]).mean() > 5
    assert not got[~valid].any(), "rows of padded queries must be zero"


@pytest.mark.parametrize("B,S,h,lens", [(32, 128, 12, None), (8, 128, 4, [128, 1, 32, 33, 64, 65, 96, 97]),
                                        (16, 100, 4, None), (5, 128, 4, [0, 128, 77, 31, 100]),
                                        (24, 40, 8, None), (3, 128, 2 * 2, [128, 128, 128])])
def test_planned_qkv_attention_leaves_the_same_bytes(oracle, rng, B, S, h, lens):
    """With a plan (pairs dealt longest sequence first, blocks of nothing but padding left out)
    the launch gives the bytes of the unplanned one everywhere -- rows of padded queries are
    zero on both -- for right-padded sequences of every block count, a sequence of padding only,
    and a mask with padding in the middle; and the oracle's chain on the valid rows."""
    d = 64
    H = h * d
    x = rng.integers(-127, 128, size=(B * S, H), dtype=np.int8)
    w = rng.integers(-127, 128, size=(3 * H, H), dtype=np.int8)
    bias = _randT(rng, (3 * H,), np.float16, 0.3)
    if lens is None:
        lens = rng.integers(max(1, S // 4), S + 1, size=B)
    lens = np.minimum(np.asarray(lens), S)
    mask = (np.arange(S)[None, :] >= lens[:, None]).astype(np.int32)
    if B >= 8:
        mask[3, 5:9] = 1      # padding inside a sequence: masked keys, zeroed queries, blocks kept
    alpha = 127.0 / (127 * 127 * np.sqrt(H) / 3.0)
    ds, qs = 1.4 / 127, 127 / 0.9
    xd, wd, bd, md = to_dev(x), to_dev(w), to_dev(bias), to_dev(mask)
    want = torch.full((B * S, H), 7, dtype=torch.int8, device=DEV)
    _k().qkv_attention_i8(xd, wd, bd, md, want, alpha, ds, qs, B, S, h, d)
    plan = _k().qkv_attention_plan(md, B, S, h)
    got = torch.full((B * S, H), 9, dtype=torch.int8, device=DEV)
    _k().qkv_attention_planned_i8(xd, wd, bd, md, plan, got, alpha, ds, qs, B, S, h, d)
    np.testing.assert_array_equal(to_np(got), to_np(want))
    # the plan is a permutation of the (sequence, head) pairs with the right block counts
    p = to_np(plan)
    pairs = sorted((int(v) & 0xffff, (int(v) >> 16) & 0xfff) for v in p)
    assert pairs == [(b, hh) for b in range(B) for hh in range(h)]
    eff = np.array([0 if not (mask[b] == 0).any() else int(np.nonzero(mask[b] == 0)[0][-1]) + 1 for b in range(B)])
    for v in p:
        assert (int(v) >> 28) & 7 == (eff[int(v) & 0xffff] + 31) // 32
    # against the oracle on the rows of valid queries
    codes = oracle.gemm_i8_i8(x, w, alpha)
    qkv = oracle.arrange_encself_qkv_i8I(codes, bias, B, S, h, ds)
    probs = oracle.correlation_softmax_encself(oracle.attn_scores(qkv[0], qkv[1], np.sqrt(1.0 / d)), mask)
    ref = oracle.arrange_atten_output_i8O(oracle.attn_context(probs, qkv[2]), qs)
    valid = (mask == 0).reshape(-1)
    if valid.any():
        assert_codes_close(to_np(got)[valid], ref[valid], max_frac=5e-3, what="context codes")
    assert not to_np(got)[~valid].any()


def test_qkv_projection_and_attention_in_one_kernel_rejects_other_shapes(rng):
    import lightseq_amd.lib as L
    for B, S, h, d in [(2, 128, 4, 32), (2, 129, 4, 64), (2, 64, 2, 64), (2, 64, 3, 64)]:
        H = h * d
        x = torch.zeros((B * S, H), dtype=torch.int8, device=DEV)
        w = torch.zeros((3 * H, H), dtype=torch.int8, device=DEV)
        bias = torch.zeros((3 * H,), dtype=torch.float16, device=DEV)
        mask = torch.zeros((B, S), dtype=torch.int32, device=DEV)
        out = torch.zeros((B * S, H), dtype=torch.int8, device=DEV)
        with pytest.raises(L.LSHError) as e:
            _k().qkv_attention_i8(x, w, bias, mask, out, 1e-3, 0.01, 100.0, B, S, h, d)
        assert e.value.code == L.LSH_ERR_UNSUPPORTED


@pytest.mark.parametrize("B,S,h,d", [(2, 128, 3, 64), (3, 50, 2, 64), (1, 200, 2, 64), (2, 64, 4, 32),
                                     (1, 7, 1, 64), (2, 130, 2, 128)])
def test_encself_attention_from_int8_qkv(oracle, rng, B, S, h, d):
    """Attention fed by the int8 QKV product == ker_arrange_encself_qkv_i8I followed by the
    fused attention on its fp16 q, k, v, bit for bit; and the oracle's sequence to the
    usual bar."""
    H = h * d
    codes = rng.integers(-127, 128, size=(B * S, 3 * H), dtype=np.int8)
    bias = _randT(rng, (3 * H,), np.float16, 0.3)
    mask = _pad_mask(rng, B, S)
    ds, qs = 1.4 / 127, 127 / 0.9
    # two-kernel route
    arr = torch.zeros((3, B, h, S, d), dtype=torch.float16, device=DEV)
    _k().ker_arrange_encself_qkv_i8I_launcher(B * S, H, to_dev(codes), to_dev(bias), arr, B * S * H, S,
                                              d, h, 1024, ds)
    ctx0 = torch.zeros((B, h, S, d), dtype=torch.float16, device=DEV)
    ctxq0 = torch.zeros((B * S, H), dtype=torch.int8, device=DEV)
    _k().encself_attention(arr[0], arr[1], arr[2], to_dev(mask), ctx0, ctxq0, qs, B, S, h, d)
    # one-kernel route
    ctx1 = torch.full((B, h, S, d), 7.0, dtype=torch.float16, device=DEV)
    ctxq1 = torch.full((B * S, H), 7, dtype=torch.int8, device=DEV)
    _k().encself_attention_i8qkv(to_dev(codes), to_dev(bias), ds, to_dev(mask), ctx1, ctxq1, qs, B, S,
                                 h, d)
    np.testing.assert_array_equal(to_np(ctx1).view(np.uint16), to_np(ctx0).view(np.uint16))
    np.testing.assert_array_equal(to_np(ctxq1), to_np(ctxq0))
    # against the restatement of the reference's sequence
    q, k, v = oracle.arrange_encself_qkv_i8I(codes, bias, B, S, h, ds)
    probs = oracle.correlation_softmax_encself(oracle.attn_scores(q, k, np.sqrt(1.0 / d)), mask)
    want_ctx = oracle.attn_context(probs, v)
    np.testing.assert_allclose(to_np(ctx1).astype(np.float32), want_ctx.astype(np.float32), atol=3e-3,
                               rtol=0)
    assert_codes_close(to_np(ctxq1), oracle.arrange_atten_output_i8O(want_ctx, qs), max_frac=5e-3)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("scaled", [False, True])
def test_enc_emb(oracle, rng, dtype, scaled):
    V, H, B, S, pad = 97, 256, 3, 11, 0
    table = rng.integers(-127, 128, size=(V, H), dtype=np.int8)
    pos = _randT(rng, (S + 3, H), dtype, 0.02)
    tokens = rng.integers(1, V, size=(B, S), dtype=np.int32)
    tokens[1, 7:] = pad
    tokens[2, 3:] = pad
    ds = 0.08 / 127
    want, want_mask = oracle.enc_emb_i8I(table, pos, tokens, pad, ds, scaled)
    out = torch.zeros((B, S, H), dtype=torch.float16 if dtype == np.float16 else torch.float32, device=DEV)
    mask = torch.full((B, S), -1, dtype=torch.int32, device=DEV)
    _k().launch_enc_emb_i8I(to_dev(table), to_dev(pos), to_dev(tokens), out, mask, pad, B, S, H, None,
                            None, 0, ds, scaled)
    np.testing.assert_array_equal(to_np(mask), want_mask)
    np.testing.assert_allclose(to_np(out).astype(np.float32), want.astype(np.float32),
                               atol=1e-3 if dtype == np.float16 else 1e-6, rtol=0)


@pytest.mark.parametrize("dtype", DTYPES)
def test_scaled_colsum(oracle, rng, dtype):
    rows, cols = 300, 130
    w = _randT(rng, (rows, cols), dtype, 0.02)
    want = oracle.scaled_colsum(w, 1.5)
    out = torch.zeros(cols, dtype=torch.float16 if dtype == np.float16 else torch.float32, device=DEV)
    _k().launch_scaled_colsum(to_dev(w), out, rows, cols, 1.5)
    np.testing.assert_allclose(to_np(out).astype(np.float32), want.astype(np.float32),
                               atol=2e-3 if dtype == np.float16 else 1e-5, rtol=0)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("layout", [0, 1])
def test_quantize_weight(oracle, rng, dtype, layout):
    rows, cols = 130, 75
    w = _randT(rng, (rows, cols), dtype, 0.02)
    qs = 127 / 0.08
    want = oracle.quantize_tensor(w, qs)
    if layout == 1:
        want = np.ascontiguousarray(want.T)
    out = torch.zeros(want.shape, dtype=torch.int8, device=DEV)
    _k().quantize_weight(torch.from_numpy(w), out, rows, cols, qs, layout)
    np.testing.assert_array_equal(to_np(out), want)


def test_col32_and_bad_arguments_fail_loudly(rng):
    from lightseq_amd.lib import LSHError, LSH_ERR_UNSUPPORTED, LSH_ERR_INVALID
    x = torch.zeros(64, dtype=torch.float16, device=DEV)
    o = torch.zeros(64, dtype=torch.int8, device=DEV)
    with pytest.raises(LSHError) as e:
        _k().launch_quantize_tensor(x, o, 1, 64, 1.0, out_col32=True)
    assert e.value.code == LSH_ERR_UNSUPPORTED
    with pytest.raises(LSHError) as e:
        _k().launch_enc_emb_i8I(o, x, torch.zeros(4, dtype=torch.int32, device=DEV), x,
                                torch.zeros(4, dtype=torch.int32, device=DEV), 0, 1, 4, 12, None, None, 0,
                                1.0, False)
    assert e.value.code == LSH_ERR_INVALID and "hidden_dim % 8" in str(e.value)
    with pytest.raises(ValueError):
        _k().launch_quantize_tensor(x.cpu(), o, 1, 64, 1.0)
