"""Pins the CPU oracle (no GPU needed).

Every check here is independent of the oracle's own formulas: library routines in
float64 (torch layer_norm / softmax / tanh-GELU / fake_quantize, numpy BLAS and
transposes), exhaustive or hand-computed known answers, algebraic identities and
the closed-form baselines the reference's own tests use
(tests/util.py:64-90 quantize/dequantize, tests/test_ls_layers.py:1669-1710
quant-linear closed form, lightseq/csrc/tests/x86/test_kernel.py:51-86 u8-shift
int8 GEMM with row compensation, tests/quant_test.py:22-98 tie rule).
"""
import numpy as np
import pytest
import torch

from conftest import assert_codes_close

F16, F32 = np.float16, np.float32


# --------------------------------------------------------------------------- #
# binary16 conversions
# --------------------------------------------------------------------------- #
def test_h2f_exhaustive(oracle):
    bits = np.arange(65536, dtype=np.uint16)
    want = bits.view(np.float16).astype(np.float32)
    got = np.array([oracle.h2f(int(b)) for b in bits], dtype=np.float32)
    nan = np.isnan(want)
    assert np.array_equal(np.isnan(got), nan)
    assert np.array_equal(got[~nan].view(np.uint32), want[~nan].view(np.uint32))


def test_f2h_round_to_nearest_even(oracle, rng):
    xs = np.concatenate([
        rng.standard_normal(20000).astype(F32) * 3,
        (rng.standard_normal(5000) * 1e-6).astype(F32),          # subnormal halves
        (rng.standard_normal(2000) * 3e4).astype(F32),           # near overflow
        np.array([0.0, -0.0, 65504, 65519.99, 65520, 1e6, -1e6, 2**-24, 2**-25, 2**-25 * 1.0001,
                  1 + 2**-11, 1 + 3 * 2**-11, 1 + 2**-11 + 2**-20, np.inf, -np.inf], dtype=F32)])
    with np.errstate(over="ignore"):
        want = xs.astype(np.float16).view(np.uint16)
    got = np.array([oracle.f2h(float(x)) for x in xs], dtype=np.uint16)
    np.testing.assert_array_equal(got, want)
    # every half value survives a round trip
    for b in range(0, 65536, 7):
        if not np.isnan(np.uint16(b).view(np.float16)):
            assert oracle.f2h(oracle.h2f(b)) == b


# --------------------------------------------------------------------------- #
# quantisers
# --------------------------------------------------------------------------- #
def test_float2int8_known_answers_and_ties(oracle):
    # quant_scale = 1: code = floor(x + 0.5), ties go up (toward +inf), clamp to +-127
    for x, q in [(0.0, 0), (0.49, 0), (0.5, 1), (1.5, 2), (2.5, 3), (-0.5, 0), (-1.5, -1),
                 (-2.5, -2), (-0.51, -1), (126.5, 127), (127.4, 127), (500.0, 127), (-127.5, -127),
                 (-128.0, -127), (-1e9, -127), (1e9, 127)]:
        assert oracle.float2int8(x, 1.0) == q, (x, q)
    # exact binary scales: x * qs is exact, so the answer is arithmetic, not float luck
    assert oracle.float2int8(0.3125, 8.0) == 3      # 2.5 -> 3
    assert oracle.float2int8(-0.3125, 8.0) == -2    # -2.5 -> -2
    assert oracle.float2int8(3.0, 0.25) == 1        # 0.75 -> 1


def test_float2int8_properties(oracle, rng):
    clip = 4.0
    qs = 127 / clip
    x = np.sort((rng.standard_normal(20000) * 2.5).astype(F32))
    q = oracle.quantize_tensor(x, qs)
    assert np.all(np.diff(q.astype(int)) >= 0)                       # monotone
    assert q.min() == -127 and q.max() == 127                        # symmetric saturation
    deq = q.astype(F32) * F32(clip / 127)
    inside = np.abs(x) <= clip
    assert np.all(np.abs(deq[inside] - x[inside]) <= clip / 127 / 2 * 1.0001)  # half a step
    np.testing.assert_array_equal(oracle.quantize_tensor(deq, qs), q)  # idempotent
    # away from ties it agrees with torch's own per-tensor fake quantiser (round-half-even
    # differs from floor(x+0.5) only on exact ties)
    n = rng.integers(-140, 141, size=5000)
    frac = rng.uniform(-0.4, 0.4, size=5000)
    xs = ((n + frac) * (clip / 127)).astype(F32)
    tq = torch.fake_quantize_per_tensor_affine(torch.from_numpy(xs), clip / 127, 0, -127, 127)
    want = np.rint(tq.numpy().astype(np.float64) / (clip / 127)).astype(np.int8)
    np.testing.assert_array_equal(oracle.quantize_tensor(xs, qs), want)


def test_float2int8_matches_reference_test_quantiser(oracle, rng):
    """tests/util.py:70-77 of the reference: floor(x / (cmax/127) + 0.5) clamped; it
    divides where the inference kernels multiply, so compare away from ties."""
    clip = 2.0
    n = rng.integers(-127, 128, size=4000)
    frac = rng.uniform(-0.45, 0.45, size=4000)
    x = ((n + frac) * (clip / 127)).astype(F32)
    want = np.clip(np.floor(x.astype(np.float64) / (clip / 127) + 0.5), -127, 127).astype(np.int8)
    np.testing.assert_array_equal(oracle.quantize_tensor(x, 127 / clip), want)


def test_posfloat2int8_unsigned_identity(oracle, rng):
    """[0, clip] maps onto [-127, 127]; x ~= (q + 127) * clip / 254 (Appendix-A identity
    behind the ReLU column-sum trick)."""
    clip = 1.65
    qs = 127 / clip
    assert oracle.posfloat2int8(0.0, qs, clip) == -127
    assert oracle.posfloat2int8(clip, qs, clip) == 127
    assert oracle.posfloat2int8(10 * clip, qs, clip) == 127
    x = rng.uniform(0, clip, size=5000).astype(F32)
    q = np.array([oracle.posfloat2int8(float(v), qs, clip) for v in x], dtype=np.int32)
    back = (q + 127) * (clip / 254)
    assert np.abs(back - x).max() <= clip / 254 / 2 * 1.001
    assert np.all(np.diff(q[np.argsort(x)]) >= 0)


def test_requant_acc_known_answers(oracle):
    # alpha a power of two: acc * alpha is exact in float
    for acc, alpha, q in [(100, 0.125, 13), (-100, 0.125, -12), (99, 0.125, 12), (4, 0.125, 1),
                          (3, 0.125, 0), (-4, 0.125, 0), (-5, 0.125, -1), (2000, 0.125, 127),
                          (-2000, 0.125, -127), (0, 0.5, 0), (2**24 + 2, 2**-20, 16)]:
        assert oracle.requant_acc(acc, alpha) == q, (acc, alpha, q)


def test_quantize_dequantize_tensor(oracle, rng):
    for dt in (F16, F32):
        x = (rng.standard_normal((7, 33)) * 2).astype(dt)
        q = oracle.quantize_tensor(x, 31.75)
        want = np.clip(np.floor(x.astype(np.float64) * 31.75 + 0.5), -127, 127)
        # the float product can only differ from the exact one on a tie: none in random data
        np.testing.assert_array_equal(q, want.astype(np.int8))
        acc = rng.integers(-2**20, 2**20, size=(5, 9), dtype=np.int32)
        d = oracle.dequantize_tensor(acc, 1.25e-4, dt)
        np.testing.assert_allclose(d.astype(np.float64), acc * 1.25e-4, rtol=1e-3 if dt == F16 else 1e-6)


# --------------------------------------------------------------------------- #
# LayerNorm family vs torch.nn.functional.layer_norm in float64
# --------------------------------------------------------------------------- #
def _ln64(x, g, b, eps=1e-12):
    t = torch.nn.functional.layer_norm(torch.from_numpy(x.astype(np.float64)), (x.shape[-1],),
                                       torch.from_numpy(g.astype(np.float64)),
                                       torch.from_numpy(b.astype(np.float64)), eps)
    return t.numpy()


def _q64(x, qs):
    return np.clip(np.floor(x * qs + 0.5), -127, 127).astype(np.int8)


@pytest.mark.parametrize("dt", [F16, F32])
@pytest.mark.parametrize("post_ln", [False, True])
def test_norm_layer_resual_vs_torch(oracle, rng, dt, post_ln):
    x = (rng.standard_normal((11, 96)) * 1.3 + 0.2).astype(dt)
    g = (1 + 0.2 * rng.standard_normal(96)).astype(dt)
    b = (0.1 * rng.standard_normal(96)).astype(dt)
    rb = (0.1 * rng.standard_normal(96)).astype(dt)
    q, res = oracle.norm_layer_resual_i8O(x, g, b, rb, 127 / 4.0, post_ln)
    ln = _ln64(x, g, b)
    assert_codes_close(q, _q64(ln, 127 / 4.0), max_frac=2e-3)
    want_res = (ln if post_ln else x.astype(np.float64)) + rb.astype(np.float64)
    np.testing.assert_allclose(res.astype(np.float64), want_res, atol=4e-3 if dt == F16 else 1e-5)


@pytest.mark.parametrize("dt", [F16, F32])
@pytest.mark.parametrize("acc_dt", [np.int8, np.int32])
@pytest.mark.parametrize("post_ln,use_colsum", [(False, False), (True, False), (True, True)])
def test_residual_bias_ln_vs_torch(oracle, rng, dt, acc_dt, post_ln, use_colsum):
    H = 80
    acc = (rng.integers(-127, 128, size=(9, H)).astype(np.int8) if acc_dt == np.int8
           else rng.integers(-300000, 300000, size=(9, H), dtype=np.int32))
    ds = 2.0 / 127 if acc_dt == np.int8 else 7e-6
    res = rng.standard_normal((9, H)).astype(dt)
    g = (1 + 0.2 * rng.standard_normal(H)).astype(dt)
    b = (0.1 * rng.standard_normal(H)).astype(dt)
    rb = (0.1 * rng.standard_normal(H)).astype(dt)
    cs = (0.3 * rng.standard_normal(H)).astype(dt) if use_colsum else None
    q, new_res = oracle.residual_bias_ln_i8O(acc, g, b, rb, res, ds, 127 / 4.0, post_ln, cs)
    r = acc.astype(np.float64) * np.float64(F32(ds)) + res.astype(np.float64)
    if cs is not None:
        r = r + cs.astype(np.float64)
    ln = _ln64(r, g, b)
    assert_codes_close(q, _q64(ln, 127 / 4.0), max_frac=3e-3)
    want_res = (ln if post_ln else r) + rb.astype(np.float64)
    np.testing.assert_allclose(new_res.astype(np.float64), want_res, atol=8e-3 if dt == F16 else 1e-5)
    # the float-output variant is the same LayerNorm without the quantiser
    if acc_dt == np.int32:
        out = oracle.residual_bias_ln_i32I(acc, g, b, res, ds, cs)
        np.testing.assert_allclose(out.astype(np.float64), ln, atol=4e-3 if dt == F16 else 1e-5)


def test_layer_norm_invariants(oracle, rng):
    """Shift/scale invariance of LayerNorm and its epsilon: a constant row maps to the
    bias exactly (variance 0, rstd = 1e6 multiplies an exact zero)."""
    H = 64
    g = np.ones(H, F32)
    b = (0.1 * rng.standard_normal(H)).astype(F32)
    x = np.full((1, H), 3.25, F32)
    q, res = oracle.norm_layer_resual_i8O(x, g, b, np.zeros(H, F32), 50.0, True)
    np.testing.assert_array_equal(res[0], b)
    y = rng.standard_normal((4, H)).astype(F32)
    q1, _ = oracle.norm_layer_resual_i8O(y, g, b, b, 30.0, True)
    q2, _ = oracle.norm_layer_resual_i8O(y * 4 + 10, g, b, b, 30.0, True)
    assert_codes_close(q1, q2, max_frac=5e-3)


# --------------------------------------------------------------------------- #
# bias + activation
# --------------------------------------------------------------------------- #
@pytest.mark.parametrize("dt", [F16, F32])
def test_bias_gelu_vs_torch_tanh_gelu(oracle, rng, dt):
    x = rng.integers(-127, 128, size=(13, 64), dtype=np.int8)
    bias = (0.3 * rng.standard_normal(64)).astype(dt)
    ds, qs = 2.2 / 127, 127 / 2.2
    got = oracle.bias_gelu_i8I_i8O(x, bias, ds, qs)
    pre = x.astype(np.float64) * np.float64(F32(ds)) + bias.astype(np.float64)
    act = torch.nn.functional.gelu(torch.from_numpy(pre), approximate="tanh").numpy()
    assert_codes_close(got, _q64(act, np.float64(F32(qs))), max_frac=2e-3)


@pytest.mark.parametrize("narrow", [False, True])
def test_bias_relu(oracle, rng, narrow):
    x = rng.integers(-127, 128, size=(13, 64), dtype=np.int8)
    bias = (0.3 * rng.standard_normal(64)).astype(F16)
    clip = 1.65
    ds, qs = 2.2 / 127, 127 / clip
    got = oracle.bias_relu_i8I_i8O(x, bias, ds, qs, clip, narrow)
    pre = np.maximum(x.astype(np.float64) * np.float64(F32(ds)) + bias.astype(np.float64), 0)
    if narrow:
        want = np.clip(np.floor(pre * 2 * np.float64(F32(qs)) - np.float64(F32(qs)) * clip + 0.5), -127, 127)
    else:
        want = np.clip(np.floor(pre * np.float64(F32(qs)) + 0.5), -127, 127)
    assert_codes_close(got, want.astype(np.int8), max_frac=2e-3)
    if narrow:  # zero activations sit at the bottom code
        assert np.all(got[pre == 0] == -127)


def test_relu_colsum_identity(oracle, rng):
    """The ReLU offset trick: with unsigned codes u = q + 127, x ~= u * c / 254, so
    x @ W == (c/254) * (q @ W) + (c/2) * colsum(W) * (127/127).  Checks that
    acc * dequant/2 + scaled_colsum reproduces the float product
    (model/quant_bert_encoder.cc.cu:156-175, 476-483)."""
    I, H, c7, c3 = 96, 24, 1.65, 0.08
    x = rng.uniform(0, c7, size=(5, I)).astype(F32)
    wq = rng.integers(-127, 128, size=(H, I), dtype=np.int8)            # [N, K] codes
    w_float = (wq.astype(F32) * F32(c3 / 127)).T                        # [I, H] dequantised
    q = np.array([[oracle.posfloat2int8(float(v), 127 / c7, c7) for v in row] for row in x], np.int8)
    acc = oracle.gemm_i8_i32(q, wq)
    colsum = oracle.scaled_colsum(w_float, c7 / 2)
    got = acc * (c3 * c7 / (2 * 127 * 127)) + colsum
    want = ((q.astype(np.float64) + 127) * c7 / 254) @ w_float.astype(np.float64)
    np.testing.assert_allclose(got, want, atol=1e-4)
    np.testing.assert_allclose(want, x.astype(np.float64) @ w_float, atol=c7 / 254 / 2 * np.abs(w_float).sum(0).max())


# --------------------------------------------------------------------------- #
# permutations, embedding, colsum
# --------------------------------------------------------------------------- #
@pytest.mark.parametrize("dt", [F16, F32])
def test_arrange_qkv_is_a_transpose(oracle, rng, dt):
    B, S, h, d = 2, 5, 3, 4
    H = h * d
    ori = rng.integers(-127, 128, size=(B * S, 3 * H), dtype=np.int8)
    bias = (0.3 * rng.standard_normal(3 * H)).astype(dt)
    ds = 2.2 / 127
    got = oracle.arrange_encself_qkv_i8I(ori, bias, B, S, h, ds)
    val = (ori.astype(F32) * F32(ds)).astype(dt).astype(np.float64) + bias.astype(np.float64)
    want = val.reshape(B, S, 3, h, d).transpose(2, 0, 3, 1, 4)
    np.testing.assert_allclose(got.astype(np.float64), want, atol=2e-3 if dt == F16 else 1e-6)
    # zero bias and unit scale: a pure permutation of the codes
    z = oracle.arrange_encself_qkv_i8I(ori, np.zeros(3 * H, F32), B, S, h, 1.0)
    np.testing.assert_array_equal(z, ori.reshape(B, S, 3, h, d).transpose(2, 0, 3, 1, 4).astype(F32))
    q8, k8, v8, dv = oracle.arrange_encself_qkv_i8I_i8O(ori, np.zeros(3 * H, F32), B, S, h, 1.0, 1.0)
    np.testing.assert_array_equal(np.stack([q8, k8, v8]), z.astype(np.int8))
    np.testing.assert_array_equal(dv, v8.astype(F32))


def test_arrange_atten_output_inverts_head_split(oracle, rng):
    B, S, h, d = 2, 7, 3, 4
    x = rng.integers(-100, 101, size=(B, h, S, d)).astype(F32)
    got = oracle.arrange_atten_output_i8O(x, 1.0)
    np.testing.assert_array_equal(got, x.transpose(0, 2, 1, 3).reshape(B * S, h * d).astype(np.int8))


@pytest.mark.parametrize("dt", [F16, F32])
@pytest.mark.parametrize("scaled", [False, True])
def test_enc_emb(oracle, rng, dt, scaled):
    V, H, B, S, pad = 31, 16, 2, 6, 3
    table = rng.integers(-127, 128, size=(V, H), dtype=np.int8)
    pos = (0.02 * rng.standard_normal((S, H))).astype(dt)
    tok = rng.integers(0, V, size=(B, S), dtype=np.int32)
    tok[0, 4:] = pad
    ds = 0.08 / 127
    out, mask = oracle.enc_emb_i8I(table, pos, tok, pad, ds, scaled)
    np.testing.assert_array_equal(mask, (tok == pad).astype(np.int32))
    scale = np.float64(F32(ds)) * (np.sqrt(H) if scaled else 1.0)
    want = table[tok].astype(np.float64) * scale + pos[None].astype(np.float64)
    want[tok == pad] = 0
    np.testing.assert_allclose(out.astype(np.float64), want, atol=1e-3 if dt == F16 else 1e-6)


def test_scaled_colsum(oracle, rng):
    w = (0.02 * rng.standard_normal((50, 12))).astype(F16)
    got = oracle.scaled_colsum(w, 0.8)
    np.testing.assert_allclose(got.astype(np.float64), w.astype(np.float64).sum(0) * 0.8, atol=1e-3)


# --------------------------------------------------------------------------- #
# attention core
# --------------------------------------------------------------------------- #
def _mask(rng, B, S):
    lens = rng.integers(1, S + 1, size=B)
    lens[0] = S
    return (np.arange(S)[None] >= lens[:, None]).astype(np.int32)


@pytest.mark.parametrize("dt", [F16, F32])
def test_softmax_vs_torch(oracle, rng, dt):
    B, h, S = 3, 2, 9
    c = (2 * rng.standard_normal((B, h, S, S))).astype(dt)
    mask = _mask(rng, B, S)
    got = oracle.correlation_softmax_encself(c, mask).astype(np.float64)
    t = torch.from_numpy(c.astype(np.float64)).masked_fill(torch.from_numpy(mask[:, None, None, :] == 1), -np.inf)
    want = torch.softmax(t, -1).numpy()
    want[np.broadcast_to(mask[:, None, :, None] == 1, want.shape)] = 0  # padded queries: zero rows
    np.testing.assert_allclose(got, want, atol=1e-3 if dt == F16 else 1e-6)


def test_softmax_special_rows(oracle):
    S = 5
    c = np.zeros((1, 1, S, S), F32)
    c[0, 0, 0] = [1, 2, 3, 4, 5]
    mask = np.array([[0, 1, 1, 1, 1]], np.int32)  # only key 0 valid -> one-hot
    got = oracle.correlation_softmax_encself(c, mask)
    np.testing.assert_array_equal(got[0, 0, 0], [1, 0, 0, 0, 0])
    np.testing.assert_array_equal(got[0, 0, 1:], 0)
    mask0 = np.zeros((1, S), np.int32)
    flat = oracle.correlation_softmax_encself(np.full((1, 1, S, S), 7.0, F32), mask0)
    np.testing.assert_allclose(flat, 1.0 / S, rtol=1e-6)


def test_attention_gemms_vs_numpy(oracle, rng):
    B, h, S, d = 2, 3, 7, 8
    q = (0.6 * rng.standard_normal((B, h, S, d))).astype(F16)
    k = (0.6 * rng.standard_normal((B, h, S, d))).astype(F16)
    v = (0.6 * rng.standard_normal((B, h, S, d))).astype(F16)
    alpha = np.sqrt(1.0 / d)
    sc = oracle.attn_scores(q, k, alpha)
    a16 = np.float64(F16(alpha))
    want = np.einsum("bhid,bhjd->bhij", q.astype(np.float64), k.astype(np.float64)) * a16
    np.testing.assert_allclose(sc.astype(np.float64), want, atol=2e-3)
    p = np.abs(rng.standard_normal((B, h, S, S))).astype(F16)
    ctx = oracle.attn_context(p, v)
    want = np.einsum("bhij,bhjd->bhid", p.astype(np.float64), v.astype(np.float64))
    np.testing.assert_allclose(ctx.astype(np.float64), want, atol=4e-3)


# --------------------------------------------------------------------------- #
# int8 GEMM
# --------------------------------------------------------------------------- #
@pytest.mark.parametrize("M,N,K", [(1, 1, 1), (3, 5, 7), (17, 9, 64), (40, 33, 300)])
def test_gemm_i32_exact_two_ways(oracle, rng, M, N, K):
    a = rng.integers(-127, 128, size=(M, K), dtype=np.int8)
    w = rng.integers(-127, 128, size=(N, K), dtype=np.int8)
    got = oracle.gemm_i8_i32(a, w)
    # (1) exact float64 BLAS product of integer matrices
    np.testing.assert_array_equal(got, np.rint(a.astype(np.float64) @ w.astype(np.float64).T).astype(np.int32))
    # (2) the x86 test idiom of the reference: shift A to uint8 and compensate with the
    # row sums of W (lightseq/csrc/tests/x86/test_kernel.py:51-86)
    a_u8 = (a.astype(np.int64) + 128)
    comp = -128 * w.astype(np.int64).sum(1)
    np.testing.assert_array_equal(got, a_u8 @ w.astype(np.int64).T + comp[None, :])


def test_gemm_extremes(oracle):
    K = 4096
    a = np.full((2, K), -127, np.int8)
    w = np.full((3, K), 127, np.int8)
    assert np.all(oracle.gemm_i8_i32(a, w) == -K * 127 * 127)
    assert np.all(oracle.gemm_i8_i8(a, w, 1.0) == -127)
    assert np.all(oracle.gemm_i8_i8(a, -w, 1.0) == 127)


def test_quant_linear_closed_form(oracle, rng):
    """The reference's own quant-linear baseline (tests/test_ls_layers.py:1669-1710):
    deq(q(x)) @ deq(q(W))^T, then quantise the output with its clip.  The integer GEMM
    with alpha = c_w c_in / (c_out 127) must give the same codes."""
    M, N, K = 12, 20, 64
    c_in, c_w, c_out = 4.0, 0.08, 2.2
    x = rng.standard_normal((M, K)).astype(F32)
    w = (0.02 * rng.standard_normal((N, K))).astype(F32)
    xq = oracle.quantize_tensor(x, 127 / c_in)
    wq = oracle.quantize_tensor(w, 127 / c_w)
    got = oracle.gemm_i8_i8(xq, wq, c_w * c_in / (c_out * 127))
    real = (xq.astype(np.float64) * c_in / 127) @ (wq.astype(np.float64) * c_w / 127).T
    want = np.clip(np.floor(real / (c_out / 127) + 0.5), -127, 127).astype(np.int8)
    assert_codes_close(got, want, max_frac=5e-3)


# --------------------------------------------------------------------------- #
# whole layer: integer path vs a float64 fake-quant model of the same layer
# --------------------------------------------------------------------------- #
def _fake_quant_layer_f64(w, ids, cfg):
    """Independent float64 model of one post-LN GELU layer with fake quantisation at
    the sites the engine quantises (Appendix-B dataflow), written with matmuls on
    dequantised values -- no integer arithmetic, no shared code with the oracle."""
    H, h = cfg["hidden"], cfg["head_num"]
    d = H // h
    c = w["clip_max"].astype(np.float64)
    B, S = ids.shape

    def fq(x, clip):
        return np.clip(np.floor(x * (127 / clip) + 0.5), -127, 127) * (clip / 127)

    def ln(x, g, b):
        return _ln64(x, g.astype(np.float64), b.astype(np.float64))

    def deq_w(wq, clip):
        return wq.astype(np.float64) * clip / 127

    emb = w["tok_emb_q"][ids].astype(np.float64) * (np.float64(w["emb_clip_max"]) / 127) \
        + w["pos_emb"][None, :S].astype(np.float64)
    x = emb.reshape(B * S, H)
    l1 = ln(x, w["ln1_scale"][0], w["ln1_bias"][0])
    q0 = fq(l1, c[4])
    x = l1 + w["b_out"][0].astype(np.float64)
    qkv = fq(q0 @ deq_w(w["w_qkv"][0], c[0]).T, c[8]) + w["b_qkv"][0].astype(np.float64)
    qkv = qkv.reshape(B, S, 3, h, d).transpose(2, 0, 3, 1, 4)
    sc = np.einsum("bhid,bhjd->bhij", qkv[0], qkv[1]) / np.sqrt(d)
    p = torch.softmax(torch.from_numpy(sc), -1).numpy()
    ctx = np.einsum("bhij,bhjd->bhid", p, qkv[2]).transpose(0, 2, 1, 3).reshape(B * S, H)
    o = fq(fq(ctx, c[5]) @ deq_w(w["w_out"][0], c[1]).T, c[9])
    r = o + x
    l2 = ln(r, w["ln2_scale"][0], w["ln2_bias"][0])
    x = l2 + w["b_ffn2"][0].astype(np.float64)
    f = fq(fq(l2, c[6]) @ deq_w(w["w_ffn1"][0], c[2]).T, c[10]) + w["b_ffn1"][0].astype(np.float64)
    a = fq(torch.nn.functional.gelu(torch.from_numpy(f), approximate="tanh").numpy(), c[7])
    r2 = a @ deq_w(w["w_ffn2"][0], c[3]).T + x
    return ln(r2, w["final_ln_scale"], w["final_ln_bias"]).reshape(B, S, H)


def test_encoder_layer_vs_float_fake_quant_model(oracle):
    from lightseq_amd import synthetic
    from oracle.model_io import oracle_weights_from_message
    cfg = synthetic.bert_config("tiny")
    cfg.update(n_layer=1)
    msg = synthetic.make_quant_bert(cfg, seed=4)
    ids, _ = synthetic.make_token_ids(cfg, 3, 24, seed=1, min_len=24)  # no padding
    w = oracle_weights_from_message(msg, cfg)
    got, mask, _ = oracle.quant_bert_encoder(w, ids)
    assert mask.sum() == 0
    want = _fake_quant_layer_f64(w, ids, cfg)
    diff = np.abs(got.astype(np.float64) - want)
    # fp16 storage of the residual stream / attention and rare code flips: a few 1e-3
    assert diff.mean() < 4e-3 and np.quantile(diff, 0.999) < 3e-2, (diff.mean(), diff.max())


def test_encoder_rejects_bad_shapes(oracle):
    from lightseq_amd import synthetic
    from oracle.model_io import oracle_weights_from_message
    cfg = synthetic.bert_config("tiny")
    msg = synthetic.make_quant_bert(cfg, seed=0)
    w = oracle_weights_from_message(msg, cfg)
    with pytest.raises(RuntimeError):
        oracle.quant_bert_encoder(w, np.ones((1, cfg["max_step"] + 1), np.int32))
