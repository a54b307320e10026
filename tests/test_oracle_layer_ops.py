"""Pins the numpy restatements of the csrc operator/layer path (oracle/layer_ops.py) and of
the pure-PyTorch quantisation-aware layer (oracle/qat.py) with checks that do not restate
them: torch / scipy library routines, the test-side formulas of the reference
(tests/util.py:64-90, tests/test_ls_layers.py:1699-1707), closed forms, and the agreement of
the two independently written restatements with each other."""
import numpy as np
import pytest
import torch
from scipy.special import softmax

from oracle import layer_ops as lo
from oracle import oracle, qat

F32 = np.float32


# ---- scalar quantisers -------------------------------------------------------------------
def test_quantize_matches_torch_and_the_inference_quantiser(rng):
    x = (rng.standard_normal(20000) * 3).astype(F32)
    cmax = F32(4.0)
    q, mask = lo.quantize(x, cmax)
    # torch's per-tensor fake quantiser rounds half to even: compare away from ties
    frac = np.abs(x / (cmax / 127) - np.round(x / (cmax / 127)))
    safe = np.abs(frac - 0.5) > 1e-3
    tq = torch.fake_quantize_per_tensor_affine(torch.from_numpy(x), float(cmax / 127), 0, -127, 127)
    np.testing.assert_array_equal(q[safe], np.round(tq.numpy()[safe] / (cmax / 127)).astype(np.int8))
    # the inference-side quantiser multiplies by 127/clip instead of dividing by clip/127
    qa = oracle.quantize_tensor(x, F32(127) / cmax)
    assert (q != qa).mean() < 1e-4 and np.abs(q.astype(int) - qa).max() <= 1
    # and the quantisation-aware restatement agrees code for code
    np.testing.assert_array_equal(q, qat.tensor_quant(x, cmax)[0].astype(np.int8))
    # mask bits of the reference's test helper (tests/util.py:64-68)
    np.testing.assert_array_equal(mask, (x <= -cmax) * 4 + (x >= cmax) * 2)


def test_quantize_ties_saturation_idempotence():
    cmax = F32(127.0)  # scale 1: codes are the values
    x = np.array([0.5, 1.5, -0.5, -1.5, 126.5, 127.5, 300, -300, -126.5], F32)
    q, _ = lo.quantize(x, cmax)
    np.testing.assert_array_equal(q, [1, 2, 0, -1, 127, 127, 127, -127, -126])
    y = lo.dequantize(q, cmax)
    np.testing.assert_array_equal(lo.quantize(y, cmax)[0], q)
    assert lo.dequantize(np.int8(-128), cmax) == -127.0  # clamped to the clip


def test_fake_quantize_forms(rng):
    x = (rng.standard_normal(5000) * 2).astype(F32)
    cmax = F32(3.0)
    fq, _ = lo.fake_quantize(x, cmax)
    np.testing.assert_allclose(fq, lo.dequantize(lo.quantize(x, cmax)[0], cmax), rtol=1e-6)
    np.testing.assert_allclose(fq, qat.fake_tensor_quant(x, cmax), rtol=1e-6)
    # unsigned form: 255 levels over [0, clip], written independently in float64
    pos = np.abs(x)
    uq, mask = lo.fake_quantize(pos, cmax, 2, symmetry=False)
    step = 3.0 / 254
    want = np.clip(np.floor(pos.astype(np.float64) / step + 0.5), 0, 254) * step
    np.testing.assert_allclose(uq, want, atol=1e-6)
    np.testing.assert_allclose(uq, qat.fake_tensor_quant(pos, cmax, unsigned=True), atol=1e-6)
    assert set(np.unique(mask)) <= {0, 2}
    assert np.abs(uq - pos)[pos < cmax].max() <= step / 2 + 1e-6


def test_alpha_closed_form():
    assert lo.igemm_alpha([4.0, 0.5, 8.0]) == F32(4.0 * 0.5 / (8.0 * 127))


# ---- row kernels ----------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", [np.float16, np.float32])
def test_layer_norm(rng, dtype):
    rows, hidden = 12, 64
    x = (rng.standard_normal((rows, hidden)) * 2 + 0.3).astype(dtype)
    g = (1 + 0.1 * rng.standard_normal(hidden)).astype(dtype)
    b = (0.1 * rng.standard_normal(hidden)).astype(dtype)
    out, var, mean = lo.launch_layer_norm(x, g, b)
    want = torch.nn.functional.layer_norm(torch.from_numpy(x.astype(np.float64)), (hidden,),
                                          torch.from_numpy(g.astype(np.float64)),
                                          torch.from_numpy(b.astype(np.float64)), eps=1e-8).numpy()
    tol = 4e-3 if dtype == np.float16 else 1e-5
    np.testing.assert_allclose(out.astype(np.float64), want, atol=tol)
    np.testing.assert_allclose(mean.astype(np.float64), x.astype(np.float64).mean(-1), atol=tol)
    np.testing.assert_allclose(var.astype(np.float64), x.astype(np.float64).var(-1) + 1e-8,
                               rtol=2e-3 if dtype == np.float16 else 1e-4)
    q, mask, _, _ = lo.launch_layer_norm_i8(x, g, b, np.array([2.0], dtype))
    wq = np.clip(np.floor(want / (2.0 / 127) + 0.5), -127, 127)
    assert np.abs(q - wq).max() <= 1 and (q != wq).mean() < 5e-3
    assert ((mask == 2) == (q == 127)).mean() > 0.99


@pytest.mark.parametrize("dtype", [np.float16, np.float32])
def test_attn_softmax(rng, dtype):
    b, h, fl, tl = 2, 3, 7, 7
    x = rng.standard_normal((b, h, fl, tl)).astype(dtype) * 3
    pad = np.zeros((b, tl), dtype)
    pad[1, 5:] = -1e8  # -inf in fp16
    with np.errstate(over="ignore"):
        pad = pad.astype(dtype)
    got = lo.launch_attn_softmax(x, pad)
    ref = x.astype(np.float64) + np.where(np.isinf(pad.astype(np.float64)) | (pad < -1e7), -np.inf,
                                          0.0)[:, None, None, :]
    want = softmax(ref, axis=-1)
    np.testing.assert_allclose(got.astype(np.float64), want, atol=1e-3 if dtype == np.float16 else 1e-6)
    assert (got[1, :, :, 5:] == 0).all()
    causal = lo.launch_attn_softmax(x, None, mask_future=True)
    ref = np.where(np.triu(np.ones((fl, tl), bool), 1)[None, None], -np.inf, x.astype(np.float64))
    np.testing.assert_allclose(causal.astype(np.float64), softmax(ref, axis=-1),
                               atol=1e-3 if dtype == np.float16 else 1e-6)


# ---- permutations ----------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", [np.float16, np.float32])
def test_quant_bias_add_transform_20314(rng, dtype):
    b, s, h, d = 2, 5, 3, 8
    q = rng.integers(-127, 128, size=(b, s, 3, h, d), dtype=np.int8)
    bias = (rng.standard_normal((3, h, d)) * 0.5).astype(dtype)
    cmax = F32(6.0)
    out = lo.launch_quant_bias_add_transform_20314(q, bias, cmax, b, s, 3, h, d)
    assert out.shape == (3, b, h, s, d) and out.dtype == dtype
    want = np.einsum("bsthd->tbhsd", q.astype(np.float64) * (6.0 / 127) + bias.astype(np.float64)[None, None])
    np.testing.assert_allclose(out.astype(np.float64), want, atol=8e-3 if dtype == np.float16 else 1e-5)
    # cache clip: every value lands on the grid of the second quantiser
    fq = lo.launch_quant_bias_add_transform_20314(q, bias, cmax, b, s, 3, h, d, out_clip_max=F32(4.0))
    grid = fq.astype(np.float64) / (4.0 / 127)
    assert np.abs(grid - np.round(grid)).max() < (0.05 if dtype == np.float16 else 1e-4)
    assert np.abs(fq.astype(np.float64)).max() <= 4.0 + 1e-2


def test_transform4d_0213_roundtrip(rng):
    b, s, h, d = 2, 5, 3, 8
    x = rng.standard_normal((1, b, h, s, d)).astype(np.float16)
    y = lo.launch_transform4d_0213(x, b, s, h * d, h, 1)
    np.testing.assert_array_equal(y.reshape(b, s, h, d), np.swapaxes(x[0], 1, 2))
    x3 = rng.standard_normal((3, b, h, s, d)).astype(np.float32)
    y3 = lo.launch_transform4d_0213(x3, b, s, h * d, h, 3)
    np.testing.assert_array_equal(y3, np.einsum("tbhsd->bsthd", x3))
    q, _ = lo.launch_quant_transform4d_0213(x3, F32(2.0), b, s, h * d, h, 3)
    np.testing.assert_array_equal(q, lo.quantize(np.einsum("tbhsd->bsthd", x3), F32(2.0))[0])


# ---- epilogues ----------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", [np.float16, np.float32])
@pytest.mark.parametrize("act", ["relu", "gelu"])
def test_bias_act_epilogues(rng, dtype, act):
    rows, dim = 9, 32
    q = rng.integers(-127, 128, size=(rows, dim), dtype=np.int8)
    bias = (rng.standard_normal(dim) * 0.3).astype(dtype)
    c_prev, c_next = F32(5.0), F32(3.0)
    x = torch.from_numpy(q.astype(np.float64) * (5.0 / 127) + bias.astype(np.float64)[None])
    want = (torch.relu(x) if act == "relu" else torch.nn.functional.gelu(x, approximate="tanh")).numpy()
    qo, _ = lo.launch_ls_quant_dropout_act_bias(q, bias, c_prev, c_next, act)
    wq = np.clip(np.floor(want / (3.0 / 127) + 0.5), -127, 127)
    tol_frac = 0.04 if dtype == np.float16 else 2e-3
    assert np.abs(qo - wq).max() <= 1 and (qo != wq).mean() < tol_frac
    fo, _ = lo.launch_ls_fakequant_dropout_act_bias(q, bias, c_prev, c_next, act,
                                                    symmetry=(act != "relu"))
    assert fo.dtype == dtype
    step = 3.0 / (254 if act == "relu" else 127)
    np.testing.assert_allclose(fo.astype(np.float64), np.clip(want, -3.0, 3.0),
                               atol=step / 2 + (6e-3 if dtype == np.float16 else 1e-5))


@pytest.mark.parametrize("dtype", [np.float16, np.float32])
def test_residual_epilogues(rng, dtype):
    rows, dim = 6, 16
    q = rng.integers(-127, 128, size=(rows, dim), dtype=np.int8)
    bias = (rng.standard_normal(dim) * 0.3).astype(dtype)
    res = rng.standard_normal((rows, dim)).astype(dtype)
    got = lo.launch_ls_quant_dropout_res_bias(q, F32(5.0), bias, res)
    want = q.astype(np.float64) * (5.0 / 127) + bias.astype(np.float64)[None] + res.astype(np.float64)
    np.testing.assert_allclose(got.astype(np.float64), want, atol=1e-2 if dtype == np.float16 else 1e-5)
    vals = rng.standard_normal((rows, dim)).astype(dtype)
    got = lo.launch_ls_dropout_res_bias(vals, bias, res)
    want = vals.astype(np.float64) + bias.astype(np.float64)[None] + res.astype(np.float64)
    np.testing.assert_allclose(got.astype(np.float64), want, atol=6e-3 if dtype == np.float16 else 1e-5)


def test_quant_linear_matches_reference_test_formula(rng):
    """tests/test_ls_layers.py:1699-1707: dequantize(quantize(.)) on input, weight and output
    around a float linear; equal to the int8 GEMM with alpha up to the rounding of the output
    quantiser."""
    tok, fin, fout = 12, 32, 24
    x = rng.standard_normal((tok, fin)).astype(np.float16)
    w = (rng.standard_normal((fout, fin)) * 0.2).astype(np.float16)
    cm = np.array([3.0, 0.6, 6.0], np.float16)
    got = lo.quant_linear_forward(x, w, cm)
    fx = lo.dequantize(lo.quantize(x, 3.0)[0], 3.0).astype(np.float64)
    fw = lo.dequantize(lo.quantize(w, cm[1])[0], cm[1]).astype(np.float64)
    out = fx @ fw.T
    want = lo.dequantize(lo.quantize(out.astype(F32), 6.0)[0], 6.0)
    d = np.abs(got.astype(np.float64) - want)
    assert d.max() <= 6.0 / 127 + 1e-3 and (d > 1e-3).mean() < 0.01
    np.testing.assert_allclose(qat.quant_linear(x, w, None, 3.0, F32(cm[1]), 6.0), want, atol=6.0 / 127 + 1e-3)


# ---- the quantisation-aware layer -----------------------------------------------------------------
def _layer_params(rng, hs, ims, w_std=0.02):
    p = {"qkv_w": rng.standard_normal((3 * hs, hs)) * w_std, "qkv_b": rng.standard_normal(3 * hs) * 0.02,
         "out_w": rng.standard_normal((hs, hs)) * w_std, "out_b": rng.standard_normal(hs) * 0.02,
         "ln1_w": 1 + 0.05 * rng.standard_normal(hs), "ln1_b": 0.02 * rng.standard_normal(hs),
         "fc1_w": rng.standard_normal((ims, hs)) * w_std, "fc1_b": rng.standard_normal(ims) * 0.02,
         "fc2_w": rng.standard_normal((hs, ims)) * w_std, "fc2_b": rng.standard_normal(hs) * 0.02,
         "ln2_w": 1 + 0.05 * rng.standard_normal(hs), "ln2_b": 0.02 * rng.standard_normal(hs)}
    return {k: v.astype(F32) for k, v in p.items()}


@pytest.mark.parametrize("pre_ln", [False, True])
@pytest.mark.parametrize("act", ["relu", "gelu"])
def test_qat_layer_without_quant_is_torch_encoder_layer(rng, pre_ln, act):
    """With the quantisers off the module is a plain encoder layer: torch's own
    ``nn.TransformerEncoderLayer`` must give the same numbers."""
    b, s, hs, nh, ims = 3, 10, 32, 4, 64
    p = _layer_params(rng, hs, ims, 0.1)
    x = rng.standard_normal((b, s, hs)).astype(F32)
    pad = np.zeros((b, s), bool)
    pad[1, 7:] = True
    pad[2, 4:] = True
    import collections
    got = qat.encoder_layer(x, p, collections.defaultdict(float), nh, pre_ln, act, pad, quant=False)
    ref = torch.nn.TransformerEncoderLayer(hs, nh, ims, dropout=0.0, activation=act,
                                           batch_first=True, norm_first=pre_ln).double().eval()
    t = lambda k: torch.from_numpy(p[k].astype(np.float64))
    with torch.no_grad():
        ref.self_attn.in_proj_weight.copy_(t("qkv_w"))
        ref.self_attn.in_proj_bias.copy_(t("qkv_b"))
        ref.self_attn.out_proj.weight.copy_(t("out_w"))
        ref.self_attn.out_proj.bias.copy_(t("out_b"))
        ref.norm1.weight.copy_(t("ln1_w")); ref.norm1.bias.copy_(t("ln1_b"))
        ref.linear1.weight.copy_(t("fc1_w")); ref.linear1.bias.copy_(t("fc1_b"))
        ref.linear2.weight.copy_(t("fc2_w")); ref.linear2.bias.copy_(t("fc2_b"))
        ref.norm2.weight.copy_(t("ln2_w")); ref.norm2.bias.copy_(t("ln2_b"))
        torch.backends.mha.set_fastpath_enabled(False)
        want = ref(torch.from_numpy(x.astype(np.float64)),
                   src_key_padding_mask=torch.from_numpy(pad)).numpy()
    np.testing.assert_allclose(got, want, atol=2e-5)


def config0(rng, pre_ln=False, act="relu", batch=8, seq=64, hs=512, nh=8, ims=2048):
    """The single-layer case: activations ~ N(0,1), weights ~ N(0, 0.02) with clip 4 sigma,
    activation clips at 4 sigma of the tensors they quantise (measured on the float layer)."""
    p = _layer_params(rng, hs, ims, 0.02)
    x = rng.standard_normal((batch, seq, hs)).astype(F32)
    xt = x.transpose(1, 0, 2)
    ln = lambda v, a, c: qat.layer_norm(v, p[a], p[c])
    h0 = ln(xt, "ln1_w", "ln1_b") if pre_ln else xt
    qkv = h0 @ p["qkv_w"].T
    amax = {"qkv_in": 4 * h0.std(), "qkv_w": 0.08, "qkv_out": 4 * qkv.std()}
    hd = hs // nh
    q, k, v = np.split(qkv + p["qkv_b"], 3, -1)
    hsplit = lambda z: z.reshape(seq, batch * nh, hd).transpose(1, 0, 2)
    pr = softmax(hsplit(q * hd ** -0.5) @ hsplit(k).transpose(0, 2, 1), axis=-1)
    ctx = (pr @ hsplit(v)).transpose(1, 0, 2).reshape(seq, batch, hs)
    ao = ctx @ p["out_w"].T
    amax.update({"out_in": 4 * ctx.std(), "out_w": 0.08, "out_out": 4 * ao.std()})
    h1 = xt + ao + p["out_b"]
    if not pre_ln:
        h1 = ln(h1, "ln1_w", "ln1_b")
    f_in = ln(h1, "ln2_w", "ln2_b") if pre_ln else h1
    f1 = f_in @ p["fc1_w"].T
    a1 = qat.activation(f1 + p["fc1_b"], act)
    f2 = a1 @ p["fc2_w"].T
    amax.update({"fc1_in": 4 * f_in.std(), "fc1_w": 0.08, "fc1_out": 4 * f1.std(),
                 "fc2_in": max(4 * a1.std(), 1e-3), "fc2_w": 0.08, "fc2_out": 4 * f2.std()})
    amax = {k: float(np.float16(v)) for k, v in amax.items()}
    return p, x, amax


def pack_para(p, amax, dtype=np.float16):
    """The flat blob of the csrc layer from the named parameters (cache clip = 16)."""
    order = ["qkv_w", "qkv_b", "out_w", "out_b", "ln1_w", "ln1_b", "fc1_w", "fc1_b", "fc2_w",
             "fc2_b", "ln2_w", "ln2_b"]
    clips = [amax[k] for k in ("qkv_in", "qkv_w", "qkv_out", "out_in", "out_w", "out_out",
                               "fc1_in", "fc1_w", "fc1_out", "fc2_in", "fc2_w")] + [16.0]
    return np.concatenate([p[k].reshape(-1) for k in order] + [np.array(clips)]).astype(dtype)


@pytest.mark.parametrize("pre_ln,act", [(False, "relu"), (True, "gelu")])
def test_layer_restatement_agrees_with_the_quantisation_aware_layer(pre_ln, act):
    """Two restatements written from different reference files (the csrc kernels in fp16 and
    the PyTorch module in float) describe the same quantised layer: outputs agree to the
    fp16 / requantisation noise, far below the 2e-2 bar of the layer parity."""
    rng = np.random.default_rng(0)
    p, x, amax = config0(rng, pre_ln, act, batch=2, seq=16, hs=128, nh=4, ims=256)
    want = qat.encoder_layer(x, p, amax, 4, pre_ln, act, None, fc2_output_quant=False)
    para = pack_para(p, amax)
    mask = np.zeros((2, 16), np.float16)
    got = lo.encoder_layer_forward(para, x.astype(np.float16), mask, 4, 256, pre_ln, act)
    d = np.abs(got.astype(np.float64) - want)
    assert d.max() < 2e-2 and d.mean() < 3e-3, (d.max(), d.mean())
    # the output quantiser of fc2 (absent from the int8 kernels) costs at most half its step
    # before the residual add and layer norm
    with_q = qat.encoder_layer(x, p, amax, 4, pre_ln, act, None, fc2_output_quant=True)
    assert np.abs(with_q - want).max() < 0.2
