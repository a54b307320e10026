"""CPU restatement (numpy) of the reference's csrc operator/layer forward path in quantised
mode: the ``launch_*`` kernels of ``lightseq/csrc/kernels/cuda`` and the forward of
``TransformerEncoderLayer<T>`` / ``TransformerDecoderLayer<T>`` / ``QuantLinearLayer<T>``
built from them.

TEST INFRASTRUCTURE ONLY: imported by ``tests/`` -- never by the shipped package.

Arrays typed ``T`` are ``numpy.float16`` or ``numpy.float32``.  Arithmetic is float32 with a
rounding to ``T`` wherever the reference stores or computes in ``T`` (its fp16 kernels use
half2 adds and multiplies at a few points; those are restated with float16 arithmetic, which
numpy rounds to nearest even like the hardware).  Dropout ratios are 0 (inference).

Parity unpinned: the reference builds these kernels with ``--use_fast_math``
(training/ops/pytorch/builder/transformer_builder.py:52-62), so its divisions, ``tanhf``,
``__expf`` and ``rsqrtf`` are approximations defined by no source file; this restatement
uses IEEE float32 division and libm functions.  The int8-output GEMM epilogue is
``clamp(floor(acc * alpha + 0.5), -127, 127)`` as everywhere in this repository (cuBLASLt's
rounding is unspecified).
"""
import numpy as np

F32 = np.float32
Q = F32(127.0)  # kernels.h:20 kQuantRangeI8
LN_EPSILON = F32(1e-8)  # normalize_kernels.cu:12
SOFTMAX_EPSILON = F32(1e-8)  # softmax_kernels.cu:11
REDUCE_FLOAT_INF_NEG = F32(-100000000.0)  # block_reduce.h:13


def _f(x):
    return np.asarray(x).astype(F32)


def clip_mask_bits(x, clip_max, start_bit, symmetry=True):
    """kernels.h:425-435 get_clip_mask."""
    x = _f(x)
    m = np.zeros(x.shape, np.uint8)
    hi = x >= clip_max
    m[hi] = 1 << (start_bit - 1)
    if symmetry:
        m[(~hi) & (x <= -clip_max)] = 1 << start_bit
    return m


def quantize(x, clip_max, start_bit=2):
    """kernels.h:463-471: returns (int8 codes, clip-mask bits)."""
    x = _f(x)
    cm = F32(clip_max)
    scale = cm / Q
    q = np.floor(x / scale + F32(0.5))
    q = np.minimum(np.maximum(q, -Q), Q)
    return q.astype(np.int8), clip_mask_bits(x, cm, start_bit)


def fake_quantize(x, clip_max, start_bit=2, symmetry=True):
    """kernels.h:473-488: returns (float32 values, clip-mask bits)."""
    x = _f(x)
    cm = F32(clip_max)
    scale = cm / Q
    if not symmetry:
        scale = scale / F32(2)
    i8f = x / scale
    if not symmetry:
        i8f = i8f - Q
    i8 = np.minimum(np.maximum(np.floor(i8f + F32(0.5)), -Q), Q)
    out = i8 * scale if symmetry else (i8 + Q) * scale
    return out.astype(F32), clip_mask_bits(x, cm, start_bit, symmetry)


def dequantize(q, clip_max):
    """kernels.h:497-501."""
    cm = F32(clip_max)
    res = np.asarray(q).astype(F32) * (cm / Q)
    return np.minimum(np.maximum(res, -cm), cm)


def igemm_alpha(clip_max3):
    """quantize_kernels.cu:74-79: alpha = cmax_in * cmax_w / (cmax_out * 127)."""
    c = _f(clip_max3)
    return F32(c[0] * c[1] / (c[2] * Q))


def launch_quantize(f, clip_max, start_bit=2, want_alpha=False):
    """quantize_kernels.cu:41-149 (flat) and :600-758 (2-D, row-major): quantises ``f`` with
    clip_max[0]; alpha (if asked) comes from clip_max[0..2]."""
    cm = _f(clip_max)
    q, mask = quantize(_f(f), cm[0], start_bit)
    return (q, mask, igemm_alpha(cm)) if want_alpha else (q, mask)


def launch_fake_quantize(x, clip_max, start_bit=2, symmetry=True):
    """quantize_kernels.cu:151-273."""
    cm = _f(clip_max)
    out, mask = fake_quantize(_f(x), cm[0], start_bit, symmetry)
    return out.astype(np.asarray(x).dtype), mask


def launch_dequantize(q, clip_max, dtype):
    """quantize_kernels.cu:275-348."""
    return dequantize(q, _f(clip_max)[0]).astype(dtype)


def _ln_stats(x):
    """normalize_kernels.cu:40-69: mean and E[x^2] - mean^2 + 1e-8 per row, float32."""
    x64 = x.astype(np.float64)
    h = x.shape[-1]
    mean = (x64.sum(-1) / h).astype(F32)
    var = ((x64 * x64).sum(-1) / h).astype(F32) - mean * mean + LN_EPSILON
    return mean, var


def launch_layer_norm(inp, gamma, beta):
    """normalize_kernels.cu:40-180: returns (ln_res T, vars T, means T)."""
    dt = np.asarray(inp).dtype
    x = _f(inp)
    mean, var = _ln_stats(x)
    rstd = (F32(1) / np.sqrt(var.astype(np.float64))).astype(F32)
    out = (x - mean[:, None]) * rstd[:, None] * _f(gamma)[None] + _f(beta)[None]
    return out.astype(dt), var.astype(dt), mean.astype(dt)


def launch_layer_norm_i8(inp, gamma, beta, clip_max_out):
    """normalize_kernels.cu:204-380: returns (codes, clip mask, vars T, means T)."""
    dt = np.asarray(inp).dtype
    x = _f(inp)
    mean, var = _ln_stats(x)
    rstd = (F32(1) / np.sqrt(var.astype(np.float64))).astype(F32)
    out = (x - mean[:, None]) * rstd[:, None] * _f(gamma)[None] + _f(beta)[None]
    q, mask = quantize(out, _f(clip_max_out).reshape(-1)[0], 2)
    return q, mask, var.astype(dt), mean.astype(dt)


def launch_attn_softmax(vals, attn_mask, mask_future=False):
    """softmax_kernels.cu:35-279: vals T [B, h, from, to], attn_mask T [B, to] additive or
    None; exp(x - max) / (sum + 1e-8), math in float32, result cast to T."""
    dt = np.asarray(vals).dtype
    x = _f(vals).copy()
    b, h, fl, tl = x.shape
    if attn_mask is not None:
        with np.errstate(invalid="ignore", over="ignore"):
            x = x + _f(attn_mask)[:, None, None, :]
    if mask_future:
        fut = np.triu(np.ones((fl, tl), bool), 1)
        x = np.where(fut[None, None], REDUCE_FLOAT_INF_NEG, x)
    mx = x.max(-1, keepdims=True)
    with np.errstate(invalid="ignore"):
        e = np.exp((x - mx).astype(np.float64))
    s = e.sum(-1, keepdims=True).astype(F32) + SOFTMAX_EPSILON
    return (e.astype(F32) * (F32(1) / s)).astype(dt)


def _hadd(a, b):
    return (a.astype(np.float16) + b.astype(np.float16)).astype(np.float16)


def _deq_add_bias(q, clip_max, bias, dt):
    """dequantize + bias as the reference adds them: float add for T=float, half2 add of the
    rounded dequantised value for T=half (transform_kernels.cu:377-381)."""
    d = dequantize(q, clip_max)
    if dt == np.float16:
        return _hadd(d.astype(np.float16), np.asarray(bias, np.float16)).astype(F32)
    return d + _f(bias)


def launch_quant_bias_add_transform_20314(inp, bias, clip_max, dim0, dim1, dim2, dim3, dim4,
                                          out_clip_max=None):
    """transform_kernels.cu:253-424: int8 [d0,d1,d2,d3,d4] -> T [d2,d0,d3,d1,d4] with
    dequantise + bias (and an optional fake quantisation of the result)."""
    dt = np.asarray(bias).dtype
    q = np.asarray(inp, np.int8).reshape(dim0, dim1, dim2, dim3, dim4)
    b = np.asarray(bias).reshape(1, 1, dim2, dim3, dim4)
    v = _deq_add_bias(q, _f(clip_max).reshape(-1)[0], np.broadcast_to(b, q.shape), dt)
    if out_clip_max is not None:
        v = fake_quantize(v.astype(dt), _f(out_clip_max).reshape(-1)[0], 6)[0]
    return np.ascontiguousarray(v.astype(dt).transpose(2, 0, 3, 1, 4))


def launch_bias_add_transform_20314(inp, bias, dim0, dim1, dim2, dim3, dim4):
    """transform_kernels.cu:140-235: T [d0,d1,d2,d3,d4] + bias [d2,d3,d4] -> [d2,d0,d3,d1,d4];
    the sum is formed in T (half2 add for T=half)."""
    dt = np.asarray(inp).dtype
    x = np.asarray(inp).reshape(dim0, dim1, dim2, dim3, dim4)
    b = np.broadcast_to(np.asarray(bias, dt).reshape(1, 1, dim2, dim3, dim4), x.shape)
    v = _hadd(x, b) if dt == np.float16 else _f(x) + _f(b)
    return np.ascontiguousarray(v.astype(dt).transpose(2, 0, 3, 1, 4))


def launch_concat3_dim1(inp1, inp2, sz0, sz2, sz1_1, sz1_2):
    """general_kernels.cu:187-234: [sz0, sz1_1, sz2] ++ [sz0, sz1_2, sz2] along dimension 1."""
    b = np.asarray(inp2).reshape(sz0, sz1_2, sz2)
    if sz1_1 == 0:
        return b.copy()
    return np.concatenate([np.asarray(inp1).reshape(sz0, sz1_1, sz2), b], axis=1)


def launch_transform4d_0213(vals, batch, seq_len, hidden, nhead, trans_count):
    """transform_kernels.cu:444-560: [tc, b, nh, s, ad] -> [b, s, tc, nh, ad]."""
    v = np.asarray(vals).reshape(trans_count, batch, nhead, seq_len, hidden // nhead)
    return np.ascontiguousarray(v.transpose(1, 3, 0, 2, 4))


def launch_quant_transform4d_0213(vals, clip_max, batch, seq_len, hidden, nhead, trans_count):
    """transform_kernels.cu:567-680: the same permutation with quantisation."""
    t = launch_transform4d_0213(vals, batch, seq_len, hidden, nhead, trans_count)
    return quantize(t, _f(clip_max).reshape(-1)[0], 2)


def _gelu_f32(x):
    x = x.astype(F32)
    u = F32(0.7978845608028654) * (x + F32(0.044715) * x * x * x)
    return x * (F32(0.5) * (F32(1) + np.tanh(u.astype(np.float64)).astype(F32)))


def _gelu_half2(val):
    """dropout_kernels.cu:33-47: x^3 in half, the cdf in float, the product in half."""
    val = val.astype(np.float16)
    pow3 = (val * (val * val).astype(np.float16)).astype(np.float16)
    u = F32(0.7978845608028654) * (val.astype(F32) + F32(0.044715) * pow3.astype(F32))
    cdf = F32(0.5) * (F32(1) + np.tanh(u.astype(np.float64)).astype(F32))
    return (val * cdf.astype(np.float16)).astype(np.float16)


def _act(x, act, dt):
    if dt == np.float16:
        if act == "gelu":
            return _gelu_half2(x).astype(F32)
        return np.maximum(x.astype(np.float16).astype(F32), F32(0)).astype(np.float16).astype(F32)
    return _gelu_f32(x) if act == "gelu" else np.maximum(_f(x), F32(0))


def _bias_act(qin, bias, cmax_prev_out, act):
    dt = np.asarray(bias).dtype
    q = np.asarray(qin, np.int8)
    b = np.broadcast_to(np.asarray(bias).reshape(1, -1), q.reshape(-1, np.asarray(bias).size).shape)
    v = _deq_add_bias(q.reshape(b.shape), _f(cmax_prev_out).reshape(-1)[0], b, dt)
    return _act(v, act, dt).reshape(q.shape), dt


def launch_ls_quant_dropout_act_bias(qin, bias, cmax_out, cmax_in, act):
    """dropout_kernels.cu:856-1057 with ratio 0: ``cmax_out`` is the clip of the GEMM output
    being dequantised, ``cmax_in`` the clip of the next GEMM's input.  Returns (codes, mask)."""
    v, _ = _bias_act(qin, bias, cmax_out, act)
    return quantize(v, _f(cmax_in).reshape(-1)[0], 2)


def launch_ls_fakequant_dropout_act_bias(qin, bias, cmax_out, cmax_in, act, symmetry=True):
    """dropout_kernels.cu:1078-1302 with ratio 0.  Returns (T values, mask)."""
    v, dt = _bias_act(qin, bias, cmax_out, act)
    out, mask = fake_quantize(v, _f(cmax_in).reshape(-1)[0], 2, symmetry)
    return out.astype(dt), mask


def launch_ls_quant_dropout_res_bias(qin, cmax, bias, residual):
    """dropout_kernels.cu:1808-1967 with ratio 0: dequantise + bias + residual."""
    dt = np.asarray(bias).dtype
    q = np.asarray(qin, np.int8)
    b = np.broadcast_to(np.asarray(bias).reshape(1, -1), q.reshape(-1, np.asarray(bias).size).shape)
    v = _deq_add_bias(q.reshape(b.shape), _f(cmax).reshape(-1)[0], b, dt)
    r = np.asarray(residual).reshape(b.shape)
    if dt == np.float16:
        return _hadd(v.astype(np.float16), r).reshape(q.shape)
    return (v + _f(r)).reshape(q.shape)


def launch_ls_dropout_res_bias(vals, bias, residual):
    """dropout_kernels.cu launch_ls_dropout_res_bias with ratio 0: (x + bias) + residual."""
    dt = np.asarray(vals).dtype
    x = np.asarray(vals)
    b = np.broadcast_to(np.asarray(bias).reshape(1, -1), x.reshape(-1, np.asarray(bias).size).shape)
    r = np.asarray(residual).reshape(b.shape)
    if dt == np.float16:
        return _hadd(_hadd(x.reshape(b.shape), b), r).reshape(x.shape)
    return ((_f(x).reshape(b.shape) + _f(b)) + _f(r)).reshape(x.shape)


def igemm_i8(a_q, w_q, alpha):
    """int8 x int8 -> int32 exact, then clamp(floor(acc * alpha + 0.5), -127, 127)."""
    acc = a_q.astype(np.int64) @ w_q.astype(np.int64).T
    f = acc.astype(F32) * F32(alpha)
    return np.minimum(np.maximum(np.floor(f + F32(0.5)), -Q), Q).astype(np.int8)


def gemm_T(x, w):
    """cublas_gemm_ex of FeedForward::Forward (feed_forward.h:36-44): out = x @ w^T with
    float32 accumulation, stored as T."""
    dt = np.asarray(x).dtype
    return (np.asarray(x).astype(np.float64) @ np.asarray(w).astype(np.float64).T).astype(F32).astype(dt)


def strided_batch_gemm(a, b, m, n, k, alpha, beta=0.0, op_a=0, op_b=0, c=None):
    """ops/includes/strided_batch_gemm.h:45-57 (cublasGemmStridedBatchedEx, float32
    accumulation): per batch element, column-major, C (m x n) = alpha op(A) op(B) + beta C.
    As row-major arrays: A [bsz, m, k] if op_a = T else [bsz, k, m]; B [bsz, n, k] if op_b = N
    else [bsz, k, n]; result [bsz, n, m] of the operands' type."""
    dt = np.asarray(a).dtype
    a64 = np.asarray(a).astype(np.float64)
    b64 = np.asarray(b).astype(np.float64)
    am = a64.reshape(-1, m, k) if op_a else a64.reshape(-1, k, m).transpose(0, 2, 1)  # [bsz, m, k]
    bm = b64.reshape(-1, k, n).transpose(0, 2, 1) if op_b else b64.reshape(-1, n, k)  # [bsz, n, k]
    out = F32(alpha) * np.einsum("bjk,bik->bji", bm, am).astype(F32)
    if beta != 0.0:
        out = out + F32(beta) * _f(c).reshape(out.shape)
    return out.astype(dt)


def split_params(para, hidden, inter):
    """transformer_encoder_layer.h:66-105 assign_weight_ptr: views into the flat blob."""
    hs, ims = hidden, inter
    sizes = [("attn_qkvw", hs * hs * 3), ("attn_qkvb", hs * 3), ("attn_ow", hs * hs),
             ("attn_ob", hs), ("attn_nw", hs), ("attn_nb", hs), ("inter_w", hs * ims),
             ("inter_b", ims), ("output_w", hs * ims), ("output_b", hs), ("ffn_nw", hs),
             ("ffn_nb", hs), ("clip_max", 12)]
    out, off = {}, 0
    for name, n in sizes:
        out[name] = para[off:off + n]
        off += n
    assert off == para.size
    out["attn_qkvw"] = out["attn_qkvw"].reshape(3 * hs, hs)
    out["attn_ow"] = out["attn_ow"].reshape(hs, hs)
    out["inter_w"] = out["inter_w"].reshape(ims, hs)
    out["output_w"] = out["output_w"].reshape(hs, ims)
    return out


def encoder_layer_forward(para, x, mask, nhead, inter, pre_ln, act, mask_future=False, taps=None):
    """layers/transformer_encoder_layer.cpp:66-293 in quantised mode, dropout off.
    x: T [B, S, H]; mask: T [B, S] additive (0 / -1e8-like); para: flat T blob."""
    dt = x.dtype
    bsz, seq, hs = x.shape
    p = split_params(np.asarray(para), hs, inter)
    cm = _f(p["clip_max"])
    qkv_c, out_c, inter_c, ffn2_c, cache_c = cm[0:3], cm[3:6], cm[6:9], cm[9:11], cm[11]
    tok = bsz * seq
    hd = hs // nhead
    taps = {} if taps is None else taps
    inp = np.asarray(x).reshape(tok, hs)

    # ---- attention block (:66-185)
    ln_in = launch_layer_norm(inp, p["attn_nw"], p["attn_nb"])[0] if pre_ln else inp
    qin, _, alpha = launch_quantize(ln_in, qkv_c, 2, True)
    qw, _ = launch_quantize(p["attn_qkvw"], qkv_c[1:], 4)
    qout = igemm_i8(qin, qw, alpha)
    taps["qkv_q"] = qout
    qkv = launch_quant_bias_add_transform_20314(
        qout, p["attn_qkvb"], qkv_c[2], bsz, seq, 3, nhead, hd,
        cache_c if mask_future else None)
    taps["qkv"] = qkv
    q, k, v = (qkv[i].reshape(bsz * nhead, seq, hd) for i in range(3))
    alpha_s = F32(dt.type(1.0) / dt.type(np.sqrt(F32(hd))))
    sc = (alpha_s * np.einsum("bid,bjd->bij", q.astype(np.float64), k.astype(np.float64))
          .astype(F32)).astype(dt)
    pr = launch_attn_softmax(sc.reshape(bsz, nhead, seq, seq), mask, mask_future)
    ctx = np.einsum("bij,bjd->bid", pr.reshape(bsz * nhead, seq, seq).astype(np.float64),
                    v.astype(np.float64)).astype(F32).astype(dt)
    attn_o_inp = launch_transform4d_0213(ctx, bsz, seq, hs, nhead, 1).reshape(tok, hs)
    taps["attn_ctx"] = attn_o_inp
    qin, _, alpha = launch_quantize(attn_o_inp, out_c, 2, True)
    qw, _ = launch_quantize(p["attn_ow"], out_c[1:], 4)
    qout = igemm_i8(qin, qw, alpha)
    taps["attn_out_q"] = qout
    attn_out = launch_ls_quant_dropout_res_bias(qout, out_c[2], p["attn_ob"], inp)
    if not pre_ln:
        attn_out = launch_layer_norm(attn_out, p["attn_nw"], p["attn_nb"])[0]
    taps["attn_out"] = attn_out

    # ---- feed-forward block (:188-250)
    ff1_inp = launch_layer_norm(attn_out, p["ffn_nw"], p["ffn_nb"])[0] if pre_ln else attn_out
    qin, _, alpha = launch_quantize(ff1_inp, inter_c, 2, True)
    qw, _ = launch_quantize(p["inter_w"], inter_c[1:], 4)
    relu_inp = igemm_i8(qin, qw, alpha)
    taps["ffn1_q"] = relu_inp
    ff2_inp, _ = launch_ls_fakequant_dropout_act_bias(
        relu_inp, p["inter_b"], inter_c[2], ffn2_c[0], act, symmetry=(act != "relu"))
    taps["ff2_inp"] = ff2_inp
    fake_w, _ = launch_fake_quantize(p["output_w"], ffn2_c[1:], 4)
    out = gemm_T(ff2_inp, fake_w)
    out = launch_ls_dropout_res_bias(out, p["output_b"], attn_out)
    if not pre_ln:
        out = launch_layer_norm(out, p["ffn_nw"], p["ffn_nb"])[0]
    return out.reshape(bsz, seq, hs)


def split_decoder_params(para, hidden, inter, layer_id, nlayer):
    """transformer_decoder_layer.h:100-168 assign_weight_ptr: views into the flat blob."""
    hs, ims = hidden, inter
    sizes = [("attn_qkvw", hs * hs * 3), ("attn_qkvb", hs * 3), ("attn_ow", hs * hs),
             ("attn_ob", hs), ("attn_nw", hs), ("attn_nb", hs),
             ("encdec_attn_qw", hs * hs), ("encdec_attn_qb", hs), ("encdec_attn_ow", hs * hs),
             ("encdec_attn_ob", hs), ("encdec_attn_nw", hs), ("encdec_attn_nb", hs),
             ("inter_w", hs * ims), ("inter_b", ims), ("output_w", hs * ims), ("output_b", hs),
             ("ffn_nw", hs), ("ffn_nb", hs), ("clip_max", 24)]
    if layer_id == 0:
        sizes += [("encdec_attn_kvw", nlayer * 2 * hs * hs), ("encdec_attn_kvb", nlayer * 2 * hs)]
    out, off = {}, 0
    for name, n in sizes:
        out[name] = para[off:off + n]
        off += n
    assert off == para.size, (off, para.size)
    for name, rows in (("attn_qkvw", 3 * hs), ("attn_ow", hs), ("encdec_attn_qw", hs),
                       ("encdec_attn_ow", hs), ("inter_w", ims), ("output_w", hs)):
        out[name] = out[name].reshape(rows, -1)
    if layer_id == 0:
        out["encdec_attn_kvw"] = out["encdec_attn_kvw"].reshape(nlayer * 2 * hs, hs)
    return out


def _attention(q, k, v, bsz, nhead, mask, mask_future):
    """StridedBatchGemm (scores, scaled in T) + launch_attn_softmax + StridedBatchGemm
    (context) + launch_transform4d_0213, as the layers chain them
    (transformer_decoder_layer.cpp:182-205).  q T [bsz * nhead, from, hd]; k, v [.., to, hd]."""
    dt = q.dtype
    bh, fl, hd = q.shape
    tl = k.shape[1]
    alpha_s = F32(dt.type(1.0) / dt.type(np.sqrt(F32(hd))))
    sc = (alpha_s * np.einsum("bid,bjd->bij", q.astype(np.float64), k.astype(np.float64))
          .astype(F32)).astype(dt)
    pr = launch_attn_softmax(sc.reshape(bsz, nhead, fl, tl), mask, mask_future)
    ctx = np.einsum("bij,bjd->bid", pr.reshape(bh, fl, tl).astype(np.float64),
                    v.astype(np.float64)).astype(F32).astype(dt)
    return launch_transform4d_0213(ctx, bsz, fl, nhead * hd, nhead, 1).reshape(bsz * fl, nhead * hd)


def _quant_linear_i8(x, w, cmax3):
    """launch_quantize of the input (start bit 2) and the weight (start bit 4), int8 GEMM to
    int8 with alpha = cmax_in * cmax_w / (cmax_out * 127)."""
    qin, _, alpha = launch_quantize(x, cmax3, 2, True)
    qw, _ = launch_quantize(w, cmax3[1:], 4)
    return igemm_i8(qin, qw, alpha)


def decoder_encdec_kv(para0, enc_out, nhead, inter, nlayer):
    """transformer_decoder_layer.cpp:236-262 encdec_kv_fw of layer 0 in quantised mode: the
    cross-attention k and v of every decoder layer, T [nlayer * 2, B, nhead, S_src, hd].  Only
    the weight is fake-quantised (clip value encdec_kv_cmax[1]); the product is in T."""
    bsz, src, hs = enc_out.shape
    p = split_decoder_params(np.asarray(para0), hs, inter, 0, nlayer)
    kv_c = _f(p["clip_max"])[18:23]
    fake_w, _ = launch_fake_quantize(p["encdec_attn_kvw"], kv_c[1:], 4)
    kv = gemm_T(np.asarray(enc_out).reshape(bsz * src, hs), fake_w)
    return launch_bias_add_transform_20314(kv, p["encdec_attn_kvb"], bsz, src, nlayer * 2, nhead,
                                           hs // nhead)


def decoder_layer_forward(para, layer_id, nlayer, x, encdec_kv, enc_mask, nhead, inter, pre_ln,
                          act, cache=None, beam=1, taps=None):
    """layers/transformer_decoder_layer.cpp:91-547 in quantised mode, dropout off.

    cache None: x T [B, trg_len, H], self attention over the whole target sequence with future
    positions masked.  cache a dict: one decoding step, x T [B * beam, 1, H];
    ``cache["k"]`` / ``cache["v"]`` hold T [B * beam * nhead, step, hd] (absent at step 0) and
    are replaced by the arrays one position longer (:173-180).  encdec_kv: the array of
    :func:`decoder_encdec_kv`; enc_mask T [B, S_src] additive.  Returns T like x."""
    x = np.asarray(x)
    dt = x.dtype
    hs = x.shape[-1]
    hd = hs // nhead
    p = split_decoder_params(np.asarray(para), hs, inter, layer_id, nlayer)
    cm = _f(p["clip_max"])
    qkv_c, out_c, eq_c, eo_c, inter_c, ffn2_c, cache_c = (cm[0:3], cm[3:6], cm[6:9], cm[9:12],
                                                         cm[12:15], cm[15:18], cm[23])
    taps = {} if taps is None else taps
    predict = cache is not None
    if predict:
        assert x.shape[1] == 1 and x.shape[0] % beam == 0
        batch, trg_len = x.shape[0] // beam, beam  # :67-70: trg_seq_len is the beam size
        sa_batch, from_len = x.shape[0], 1
    else:
        batch, trg_len = x.shape[0], x.shape[1]
        sa_batch, from_len = batch, trg_len
    tok = batch * trg_len
    inp = x.reshape(tok, hs)
    ln = lambda v, w, b: launch_layer_norm(v, p[w], p[b])[0]

    # ---- self attention (:91-233)
    ln_in = ln(inp, "attn_nw", "attn_nb") if pre_ln else inp
    qout = _quant_linear_i8(ln_in, p["attn_qkvw"], qkv_c)
    qkv = launch_quant_bias_add_transform_20314(qout, p["attn_qkvb"], qkv_c[2], sa_batch,
                                                from_len, 3, nhead, hd, cache_c)
    q, k, v = (qkv[i].reshape(sa_batch * nhead, from_len, hd) for i in range(3))
    if predict:
        step = 0 if cache.get("k") is None else cache["k"].shape[1]
        k = launch_concat3_dim1(cache.get("k"), k, sa_batch * nhead, hd, step, 1)
        v = launch_concat3_dim1(cache.get("v"), v, sa_batch * nhead, hd, step, 1)
        cache["k"], cache["v"] = k, v
    ctx = _attention(q, k, v, sa_batch, nhead, None, not predict)
    taps["attn_ctx"] = ctx
    qout = _quant_linear_i8(ctx, p["attn_ow"], out_c)
    h1 = launch_ls_quant_dropout_res_bias(qout, out_c[2], p["attn_ob"], inp)
    if not pre_ln:
        h1 = ln(h1, "attn_nw", "attn_nb")
    taps["attn_out"] = h1

    # ---- cross attention (:278-412): batch sequences of trg_len queries each
    ln_in = ln(h1, "encdec_attn_nw", "encdec_attn_nb") if pre_ln else h1
    qout = _quant_linear_i8(ln_in, p["encdec_attn_qw"], eq_c)
    eq = launch_quant_bias_add_transform_20314(qout, p["encdec_attn_qb"], eq_c[2], batch, trg_len,
                                               1, nhead, hd, None)
    src = encdec_kv.shape[3]
    ek = np.asarray(encdec_kv)[2 * layer_id].reshape(batch * nhead, src, hd)
    ev = np.asarray(encdec_kv)[2 * layer_id + 1].reshape(batch * nhead, src, hd)
    ctx = _attention(eq[0].reshape(batch * nhead, trg_len, hd), ek, ev, batch, nhead, enc_mask,
                     False)
    taps["encdec_ctx"] = ctx
    qout = _quant_linear_i8(ctx, p["encdec_attn_ow"], eo_c)
    h2 = launch_ls_quant_dropout_res_bias(qout, eo_c[2], p["encdec_attn_ob"], h1)
    if not pre_ln:
        h2 = ln(h2, "encdec_attn_nw", "encdec_attn_nb")
    taps["encdec_out"] = h2

    # ---- feed-forward (:415-483)
    ff1_inp = ln(h2, "ffn_nw", "ffn_nb") if pre_ln else h2
    relu_inp = _quant_linear_i8(ff1_inp, p["inter_w"], inter_c)
    ff2_inp, _ = launch_ls_fakequant_dropout_act_bias(
        relu_inp, p["inter_b"], inter_c[2], ffn2_c[0], act, symmetry=(act != "relu"))
    fake_w, _ = launch_fake_quantize(p["output_w"], ffn2_c[1:], 4)
    out = gemm_T(ff2_inp, fake_w)
    out = launch_ls_dropout_res_bias(out, p["output_b"], h2)
    if not pre_ln:
        out = ln(out, "ffn_nw", "ffn_nb")
    return out.reshape(x.shape)


def quant_linear_forward(x, weight, clip_max3):
    """layers/quant_linear_layer.cpp:22-45 (int8 branch): quantise input and weight, int8
    GEMM to int8 with alpha, dequantise with clip_max[2]."""
    dt = np.asarray(x).dtype
    cm = _f(clip_max3)
    qin, _, alpha = launch_quantize(x, cm, 2, True)
    qw, _ = launch_quantize(weight, cm[1:], 4)
    return launch_dequantize(igemm_i8(qin, qw, alpha), cm[2:], dt)
