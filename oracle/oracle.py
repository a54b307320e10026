"""ctypes/numpy front-end of the CPU oracle (``libls_oracle.so``).

TEST INFRASTRUCTURE ONLY: imported by ``tests/``, by the smoke check and by the
``cpu_baseline`` leg of the benchmark -- never by the shipped package.

Arrays typed ``T`` are ``numpy.float16`` or ``numpy.float32``; the dtype of the
first T-typed argument selects the variant.  Functions return fresh arrays and do
not modify their inputs unless the name of the argument says so.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libls_oracle.so")


def build(force=False):
    """Compile the C oracle with ``make`` (gcc)."""
    if force and os.path.exists(_LIB_PATH):
        os.remove(_LIB_PATH)
    subprocess.check_call(["make", "-s", "-C", _HERE])
    return _LIB_PATH


def _load():
    if not os.path.exists(_LIB_PATH):
        build()
    return ctypes.CDLL(_LIB_PATH)


_lib = _load()
_c = ctypes
_vp = _c.c_void_p


def _p(a):
    return None if a is None else _c.c_void_p(a.ctypes.data)


def _f16(a):
    if a.dtype == np.float16:
        return 1
    if a.dtype == np.float32:
        return 0
    raise TypeError("T arrays must be float16 or float32, got %s" % a.dtype)


def _c_arr(a, dtype=None):
    a = np.ascontiguousarray(a)
    if dtype is not None and a.dtype != dtype:
        raise TypeError("expected %s, got %s" % (dtype, a.dtype))
    return a


_lib.lso_h2f.restype = _c.c_float
_lib.lso_h2f.argtypes = [_c.c_uint16]
_lib.lso_f2h.restype = _c.c_uint16
_lib.lso_f2h.argtypes = [_c.c_float]
_lib.lso_float2int8.restype = _c.c_int8
_lib.lso_float2int8.argtypes = [_c.c_float, _c.c_float]
_lib.lso_posfloat2int8.restype = _c.c_int8
_lib.lso_posfloat2int8.argtypes = [_c.c_float, _c.c_float, _c.c_float]
_lib.lso_requant_acc.restype = _c.c_int8
_lib.lso_requant_acc.argtypes = [_c.c_int32, _c.c_float]


def h2f(bits):
    return _lib.lso_h2f(int(bits))


def f2h(x):
    return _lib.lso_f2h(float(x))


def float2int8(x, quant_scale):
    return _lib.lso_float2int8(float(x), float(quant_scale))


def posfloat2int8(x, quant_scale, clip_max):
    return _lib.lso_posfloat2int8(float(x), float(quant_scale), float(clip_max))


def requant_acc(acc, alpha):
    return _lib.lso_requant_acc(int(acc), float(alpha))


def quantize_tensor(x, quant_scale):
    x = _c_arr(x)
    out = np.empty(x.shape, np.int8)
    _lib.lso_quantize_tensor(_p(x), _p(out), _c.c_long(x.size), _c.c_float(quant_scale), _f16(x))
    return out


def dequantize_tensor(x, dequant_scale, dtype=np.float16):
    x = _c_arr(x, np.int32)
    out = np.empty(x.shape, dtype)
    _lib.lso_dequantize_tensor(_p(x), _p(out), _c.c_long(x.size), _c.c_float(dequant_scale), _f16(out))
    return out


def norm_layer_resual_i8O(inp, scale, bias, residual_bias, quant_scale, is_post_ln):
    """-> (int8 LN output, updated residual stream)."""
    inp = _c_arr(inp).copy()
    tokens, hidden = inp.shape
    out = np.empty(inp.shape, np.int8)
    _lib.lso_norm_layer_resual_i8O(_p(inp), _p(out), _p(_c_arr(scale)), _p(_c_arr(bias)),
                                   _p(_c_arr(residual_bias)), tokens, hidden,
                                   _c.c_float(quant_scale), int(is_post_ln), _f16(inp))
    return out, inp


def residual_bias_ln_i8O(inp, scale, bias, residual_bias, residual, dequant_scale,
                         quant_scale, is_post_ln, colsum=None):
    """``inp`` int8 or int32 GEMM output -> (int8 LN output, updated residual)."""
    inp = _c_arr(inp)
    if inp.dtype not in (np.int8, np.int32):
        raise TypeError("input must be int8 or int32")
    residual = _c_arr(residual).copy()
    tokens, hidden = residual.shape
    out = np.empty(residual.shape, np.int8)
    rb = None if residual_bias is None else _c_arr(residual_bias)
    cs = None if colsum is None else _c_arr(colsum)
    _lib.lso_residual_bias_ln_i8O(_p(inp), int(inp.dtype == np.int32), _p(_c_arr(scale)),
                                  _p(_c_arr(bias)), _p(rb), _p(out), _p(residual), tokens,
                                  hidden, _c.c_float(dequant_scale), _c.c_float(quant_scale),
                                  int(is_post_ln), _p(cs), _f16(residual))
    return out, residual


def residual_bias_ln_i32I(inp, scale, bias, residual, dequant_scale, colsum=None):
    inp = _c_arr(inp, np.int32)
    residual = _c_arr(residual)
    tokens, hidden = residual.shape
    out = np.empty_like(residual)
    cs = None if colsum is None else _c_arr(colsum)
    _lib.lso_residual_bias_ln_i32I(_p(inp), _p(_c_arr(scale)), _p(_c_arr(bias)), _p(residual),
                                   _p(out), tokens, hidden, _c.c_float(dequant_scale), _p(cs),
                                   _f16(residual))
    return out


def bias_gelu_i8I_i8O(inp, bias, dequant_scale, quant_scale):
    inp = _c_arr(inp, np.int8)
    tokens, feat = inp.shape
    out = np.empty_like(inp)
    bias = _c_arr(bias)
    _lib.lso_bias_gelu_i8I_i8O(_p(inp), _p(out), _p(bias), tokens, feat, _c.c_float(dequant_scale),
                               _c.c_float(quant_scale), _f16(bias))
    return out


def bias_relu_i8I_i8O(inp, bias, dequant_scale, quant_scale, clip_max, narrow_clip):
    inp = _c_arr(inp, np.int8)
    tokens, feat = inp.shape
    out = np.empty_like(inp)
    bias = _c_arr(bias)
    _lib.lso_bias_relu_i8I_i8O(_p(inp), _p(out), _p(bias), tokens, feat, _c.c_float(dequant_scale),
                               _c.c_float(quant_scale), _c.c_float(clip_max), int(narrow_clip),
                               _f16(bias))
    return out


def arrange_encself_qkv_i8I(ori_qkv, qkv_bias, batch, seq_len, head_num, dequant_scale):
    """[B*S, 3H] int8 -> [3, B, h, S, d] T."""
    ori_qkv = _c_arr(ori_qkv, np.int8)
    qkv_bias = _c_arr(qkv_bias)
    hidden = ori_qkv.shape[1] // 3
    d = hidden // head_num
    out = np.empty((3, batch, head_num, seq_len, d), qkv_bias.dtype)
    _lib.lso_arrange_encself_qkv_i8I(_p(ori_qkv), _p(qkv_bias), _p(out),
                                     _c.c_long(batch * seq_len * hidden), batch, seq_len, d,
                                     head_num, _c.c_float(dequant_scale), _f16(qkv_bias))
    return out


def arrange_encself_qkv_i8I_i8O(ori_qkv, qkv_bias, batch, seq_len, head_num, dequant_scale,
                                quant_scale):
    """-> (q, k, v int8 [B,h,S,d], dequantised v T)."""
    ori_qkv = _c_arr(ori_qkv, np.int8)
    qkv_bias = _c_arr(qkv_bias)
    hidden = ori_qkv.shape[1] // 3
    d = hidden // head_num
    shp = (batch, head_num, seq_len, d)
    q, k, v = (np.empty(shp, np.int8) for _ in range(3))
    dv = np.empty(shp, qkv_bias.dtype)
    _lib.lso_arrange_encself_qkv_i8I_i8O(_p(ori_qkv), _p(qkv_bias), _p(q), _p(k), _p(v), _p(dv),
                                         batch, seq_len, d, head_num, _c.c_float(dequant_scale),
                                         _c.c_float(quant_scale), _f16(qkv_bias))
    return q, k, v, dv


def arrange_atten_output_i8O(ori_q, quant_scale):
    """[B, h, S, d] T -> [B*S, h*d] int8."""
    ori_q = _c_arr(ori_q)
    b, h, s, d = ori_q.shape
    out = np.empty((b * s, h * d), np.int8)
    _lib.lso_arrange_atten_output_i8O(_p(ori_q), _p(out), b * s, s, d, h, _c.c_float(quant_scale),
                                      _f16(ori_q))
    return out


def correlation_softmax_encself(correlation, pad_mask):
    """[B, h, S, S] T scores, [B, S] int32 mask (1 = pad) -> probabilities."""
    c = _c_arr(correlation).copy()
    b, h, s, _ = c.shape
    m = _c_arr(pad_mask, np.int32)
    _lib.lso_correlation_softmax_encself(_p(c), _p(m), b, s, h, _f16(c))
    return c


def attn_scores(q, k, alpha):
    q, k = _c_arr(q), _c_arr(k)
    b, h, s, d = q.shape
    out = np.empty((b, h, s, s), q.dtype)
    _lib.lso_attn_scores(_p(q), _p(k), _p(out), b * h, s, d, _c.c_float(alpha), _f16(q))
    return out


def attn_context(probs, v):
    probs, v = _c_arr(probs), _c_arr(v)
    b, h, s, d = v.shape
    out = np.empty((b, h, s, d), v.dtype)
    _lib.lso_attn_context(_p(probs), _p(v), _p(out), b * h, s, d, _f16(v))
    return out


def gemm_i8_i32(a, w):
    """a [M,K] int8, w [N,K] int8 -> [M,N] int32."""
    a, w = _c_arr(a, np.int8), _c_arr(w, np.int8)
    m, k = a.shape
    n = w.shape[0]
    assert w.shape[1] == k
    out = np.empty((m, n), np.int32)
    _lib.lso_gemm_i8_i32(_p(a), _p(w), _p(out), m, n, k)
    return out


def gemm_i8_i8(a, w, alpha):
    a, w = _c_arr(a, np.int8), _c_arr(w, np.int8)
    m, k = a.shape
    n = w.shape[0]
    assert w.shape[1] == k
    out = np.empty((m, n), np.int8)
    _lib.lso_gemm_i8_i8(_p(a), _p(w), _p(out), m, n, k, _c.c_float(alpha))
    return out


def enc_emb_i8I(token_emb, pos_emb, tokens, pad_id, dequant_scale, scaled):
    """-> (embedding [B,S,H] T, pad mask [B,S] int32)."""
    token_emb = _c_arr(token_emb, np.int8)
    pos_emb = _c_arr(pos_emb)
    tokens = _c_arr(tokens, np.int32)
    b, s = tokens.shape
    hidden = token_emb.shape[1]
    out = np.empty((b, s, hidden), pos_emb.dtype)
    mask = np.empty((b, s), np.int32)
    _lib.lso_enc_emb_i8I(_p(token_emb), _p(pos_emb), _p(tokens), _p(out), _p(mask), int(pad_id), b,
                         s, hidden, _c.c_float(dequant_scale), int(scaled), _f16(pos_emb))
    return out, mask


def scaled_colsum(inp, scale):
    inp = _c_arr(inp)
    rows, cols = inp.shape
    out = np.empty((cols,), inp.dtype)
    _lib.lso_scaled_colsum(_p(inp), _p(out), rows, cols, _c.c_float(scale), _f16(inp))
    return out


# --------------------------------------------------------------------------- #
# whole encoder stack
# --------------------------------------------------------------------------- #
class _BertWeights(_c.Structure):
    _fields_ = [(n, _c.c_int) for n in ("n_layer", "hidden", "inner", "head_num", "max_step",
                                        "vocab", "padding_id", "is_post_ln", "use_gelu", "f16")] + [
        ("tok_emb_q", _vp), ("pos_emb", _vp), ("final_ln_scale", _vp), ("final_ln_bias", _vp),
        ("emb_clip_max", _c.c_float),
        ("ln1_scale", _c.POINTER(_vp)), ("ln1_bias", _c.POINTER(_vp)),
        ("w_qkv", _c.POINTER(_vp)), ("b_qkv", _c.POINTER(_vp)),
        ("w_out", _c.POINTER(_vp)), ("b_out", _c.POINTER(_vp)),
        ("ln2_scale", _c.POINTER(_vp)), ("ln2_bias", _c.POINTER(_vp)),
        ("w_ffn1", _c.POINTER(_vp)), ("b_ffn1", _c.POINTER(_vp)),
        ("w_ffn2", _c.POINTER(_vp)), ("b_ffn2", _c.POINTER(_vp)),
        ("ffn2_colsum", _c.POINTER(_vp)), ("clip_max", _c.POINTER(_c.c_float)),
        ("clip_stride", _c.c_int), ("emb_scaled", _c.c_int)]


class _BertTaps(_c.Structure):
    _fields_ = [("tap_layer", _c.c_int)] + [(n, _vp) for n in (
        "ln1_q", "qkv_q", "ctx", "ctx_q", "out_q", "ln2_q", "ffn1_q", "act_q", "ffn2_acc")]


_PER_LAYER = ("ln1_scale", "ln1_bias", "w_qkv", "b_qkv", "w_out", "b_out", "ln2_scale",
              "ln2_bias", "w_ffn1", "b_ffn1", "w_ffn2", "b_ffn2")


def quant_bert_encoder(weights, token_ids, tap_layer=None):
    """Run the whole int8 encoder stack.

    ``weights``: dict with the config ints (n_layer, hidden, inner, head_num,
    max_step, vocab, padding_id, is_post_ln, use_gelu), ``tok_emb_q`` int8
    [vocab,H], ``pos_emb``/``final_ln_scale``/``final_ln_bias`` T,
    ``emb_clip_max`` float, ``clip_max`` float32 [n_layer*11] and, per name in
    ``_PER_LAYER``, a list of n_layer arrays (int8 weights as [N,K]); optional
    ``ffn2_colsum`` list.  Returns (output [B,S,H] T, pad_mask, taps dict).
    """
    token_ids = _c_arr(token_ids, np.int32)
    b, s = token_ids.shape
    L, H, I = weights["n_layer"], weights["hidden"], weights["inner"]
    T = weights["pos_emb"].dtype
    keep = []  # keep temporaries alive

    def ptr_array(arrs):
        arr = (_vp * L)()
        for i, a in enumerate(arrs):
            if a is None:
                arr[i] = None
            else:
                a = np.ascontiguousarray(a)
                keep.append(a)
                arr[i] = a.ctypes.data
        keep.append(arr)
        return _c.cast(arr, _c.POINTER(_vp))

    w = _BertWeights()
    for n in ("n_layer", "hidden", "inner", "head_num", "max_step", "vocab", "padding_id",
              "is_post_ln", "use_gelu"):
        setattr(w, n, int(weights[n]))
    w.f16 = 1 if T == np.float16 else 0
    for n in ("tok_emb_q", "pos_emb", "final_ln_scale", "final_ln_bias"):
        a = np.ascontiguousarray(weights[n])
        keep.append(a)
        setattr(w, n, a.ctypes.data)
    w.emb_clip_max = float(weights["emb_clip_max"])
    for n in _PER_LAYER:
        setattr(w, n, ptr_array(weights[n]))
    cs = weights.get("ffn2_colsum")
    w.ffn2_colsum = ptr_array(cs) if cs is not None else _c.cast(None, _c.POINTER(_vp))
    clip = np.ascontiguousarray(weights["clip_max"], np.float32)
    w.clip_stride = int(weights.get("clip_stride", 11))
    w.emb_scaled = int(weights.get("emb_scaled", 0))
    assert clip.size == L * w.clip_stride
    w.clip_max = clip.ctypes.data_as(_c.POINTER(_c.c_float))

    out = np.empty((b, s, H), T)
    mask = np.empty((b, s), np.int32)
    taps_out = {}
    taps = None
    if tap_layer is not None:
        M = b * s
        d = H // weights["head_num"]
        taps = _BertTaps()
        taps.tap_layer = int(tap_layer)
        shapes = {"ln1_q": ((M, H), np.int8), "qkv_q": ((M, 3 * H), np.int8),
                  "ctx": ((b, weights["head_num"], s, d), T), "ctx_q": ((M, H), np.int8),
                  "out_q": ((M, H), np.int8), "ln2_q": ((M, H), np.int8),
                  "ffn1_q": ((M, I), np.int8), "act_q": ((M, I), np.int8),
                  "ffn2_acc": ((M, H), np.int32)}
        for n, (shp, dt) in shapes.items():
            taps_out[n] = np.empty(shp, dt)
            setattr(taps, n, taps_out[n].ctypes.data)
    rc = _lib.lso_quant_bert_encoder(_c.byref(w), _p(token_ids), b, s, _p(out), _p(mask),
                                     _c.byref(taps) if taps is not None else None)
    if rc != 0:
        raise RuntimeError("lso_quant_bert_encoder failed with code %d" % rc)
    return out, mask, taps_out


# --------------------------------------------------------------------------- #
# decoder half
# --------------------------------------------------------------------------- #
_lib.lso_length_norm.restype = _c.c_float
_lib.lso_length_norm.argtypes = [_c.c_int, _c.c_float]
_lib.lso_select_beam_rough_topk_i8I.restype = _c.c_int


def _fl(x):
    return _c.c_float(float(x))


def length_norm(length, alpha):
    return _lib.lso_length_norm(int(length), float(alpha))


def dec_emb_i8I(token_emb, pos_emb, tokens, step, dequant_scale, scaled, vocab_major=False):
    """tokens [rows, max_step] int32; token_emb [hidden, vocab] (or [vocab, hidden] when
    ``vocab_major``) -> [rows, hidden] T."""
    token_emb = _c_arr(token_emb, np.int8)
    pos_emb = _c_arr(pos_emb)
    tokens = _c_arr(tokens, np.int32)
    rows, max_step = tokens.shape
    vocab, hidden = token_emb.shape if vocab_major else token_emb.shape[::-1]
    out = np.empty((rows, hidden), pos_emb.dtype)
    _lib.lso_dec_emb_i8I(_p(token_emb), _p(pos_emb), _p(tokens), _p(out), rows, hidden, vocab,
                         int(step), max_step, _fl(dequant_scale), int(scaled), int(vocab_major),
                         _f16(pos_emb))
    return out


def arrange_decself_qkv_i8I_i8O(ori_qkv, qkv_bias, k_cache, v_cache, step_id, dequant_scale,
                                quant_scale):
    """Writes step ``step_id`` of the caches [rows, head, max_step, d] in place; returns new_q."""
    ori_qkv = _c_arr(ori_qkv, np.int8)
    qkv_bias = _c_arr(qkv_bias)
    assert k_cache.flags.c_contiguous and v_cache.flags.c_contiguous
    rows, head_num, max_step, d = k_cache.shape
    new_q = np.empty((rows, head_num * d), np.int8)
    _lib.lso_arrange_decself_qkv_i8I_i8O(_p(ori_qkv), _p(qkv_bias), _p(new_q), _p(k_cache),
                                         _p(v_cache), rows, head_num, d, max_step, int(step_id),
                                         _fl(dequant_scale), _fl(quant_scale), _f16(qkv_bias))
    return new_q


def decself_scores(q, k_cache, step_num):
    q = _c_arr(q, np.int8)
    k_cache = _c_arr(k_cache, np.int8)
    rows, head_num, max_step, d = k_cache.shape
    out = np.zeros((rows * head_num, max_step), np.int32)
    _lib.lso_decself_scores(_p(q), _p(k_cache), _p(out), rows, head_num, d, max_step,
                            int(step_num))
    return out


def fuse_softmax_new_value_i32I_i8O(logits, v_cache, step_num, attn_scale, dequant_scale,
                                    quant_scale):
    logits = _c_arr(logits, np.int32)
    v_cache = _c_arr(v_cache, np.int8)
    rows, head_num, max_step, d = v_cache.shape
    out = np.empty((rows, head_num * d), np.int8)
    _lib.lso_fuse_softmax_new_value_i32I_i8O(_p(logits), _p(v_cache), _p(out), rows * head_num,
                                             int(step_num), max_step, head_num, d,
                                             _fl(attn_scale), _fl(dequant_scale),
                                             _fl(quant_scale))
    return out


def arrange_encdec_q_i8I(ori_q, q_bias, beam_size, head_num, dequant_scale):
    ori_q = _c_arr(ori_q, np.int8)
    q_bias = _c_arr(q_bias)
    rows, hidden = ori_q.shape
    d = hidden // head_num
    out = np.empty((rows // beam_size, head_num, beam_size, d), q_bias.dtype)
    _lib.lso_arrange_encdec_q_i8I(_p(ori_q), _p(q_bias), _p(out), rows, beam_size, d, head_num,
                                  _fl(dequant_scale), _f16(q_bias))
    return out


def arrange_encdec_kv(ori_kv, kv_bias, batch, seq_len, n_layer, head_num):
    """ori_kv [batch*seq_len, n_layer, 2, H] -> (k, v) each [n_layer, batch, head, seq_len, d]."""
    ori_kv = _c_arr(ori_kv)
    kv_bias = _c_arr(kv_bias)
    hidden = ori_kv.shape[-1]
    d = hidden // head_num
    k = np.empty((n_layer, batch, head_num, seq_len, d), ori_kv.dtype)
    v = np.empty_like(k)
    _lib.lso_arrange_encdec_kv(_p(ori_kv), _p(kv_bias), _p(k), _p(v),
                               _c.c_long(batch * seq_len * hidden), batch, seq_len, n_layer, d,
                               head_num, _f16(ori_kv))
    return k, v


def correlation_softmax_encdec(correlation, pad_mask):
    """correlation [batch, head*beam, seq_len] T -> probabilities (copy)."""
    out = np.array(correlation, copy=True, order="C")
    pad_mask = _c_arr(pad_mask, np.int32)
    batch, hb, seq_len = out.shape
    _lib.lso_correlation_softmax_encdec(_p(out), _p(pad_mask), batch, hb, seq_len, _f16(out))
    return out


def attn_scores_rect(q, k, alpha):
    """q [BH, n_q, d], k [BH, n_k, d] -> [BH, n_q, n_k]."""
    q = _c_arr(q)
    k = _c_arr(k)
    bh, n_q, d = q.shape
    n_k = k.shape[1]
    out = np.empty((bh, n_q, n_k), q.dtype)
    _lib.lso_attn_scores_rect(_p(q), _p(k), _p(out), bh, n_q, n_k, d, _fl(alpha), _f16(q))
    return out


def attn_context_rect(probs, v):
    probs = _c_arr(probs)
    v = _c_arr(v)
    bh, n_q, n_k = probs.shape
    d = v.shape[2]
    out = np.empty((bh, n_q, d), probs.dtype)
    _lib.lso_attn_context_rect(_p(probs), _p(v), _p(out), bh, n_q, n_k, d, _f16(probs))
    return out


def gemm_T(a, b):
    """[M,K] @ [K,N] in T with wide accumulation."""
    a = _c_arr(a)
    b = _c_arr(b)
    m, k = a.shape
    n = b.shape[1]
    out = np.empty((m, n), a.dtype)
    _lib.lso_gemm_T(_p(a), _p(b), _p(out), m, n, k, _f16(a))
    return out


def select_beam_rough_topk_i8I(logits, logit_bias, seq_probs, seq_score, alive_seq, dequant_scale,
                               length_norm_value, cur_step, max_thread_per_block, beam_size,
                               end_id):
    """Returns (can_idx[:total], can_score[:total], num_beam_can [rows+1])."""
    logits = _c_arr(logits, np.int8)
    logit_bias = _c_arr(logit_bias)
    seq_probs = _c_arr(seq_probs, np.float32)
    seq_score = _c_arr(seq_score, np.float32)
    alive_seq = _c_arr(alive_seq, np.int32)
    rows, vocab = logits.shape
    max_step = alive_seq.shape[1]
    can_idx = np.empty(rows * vocab, np.int32)
    can_score = np.empty(rows * vocab, np.float32)
    num = np.zeros(rows + 1, np.int32)
    total = _lib.lso_select_beam_rough_topk_i8I(
        _p(logits), _p(logit_bias), _p(seq_probs), _p(seq_score), _p(alive_seq),
        _fl(dequant_scale), _p(can_idx), _p(can_score), _p(num), vocab, max_step,
        _fl(length_norm_value), int(cur_step), rows, int(max_thread_per_block), int(beam_size),
        int(end_id), _f16(logit_bias))
    return can_idx[:total].copy(), can_score[:total].copy(), num


def scan_sort_candidates(can_idx, can_score, num_beam_can):
    """Returns sorted copies and the scanned count array."""
    can_idx = np.array(can_idx, np.int32, copy=True)
    can_score = np.array(can_score, np.float32, copy=True)
    num = np.array(num_beam_can, np.int32, copy=True)
    _lib.lso_scan_sort_candidates(_p(can_idx), _p(can_score), _p(num), num.size - 1)
    return can_idx, can_score, num


def refresh_result(can_idx, can_score, num_scanned, alive_seq, seq_probs, seq_score, vocab_size,
                   cur_step, length_norm_value, end_id, beam_size):
    """``num_scanned``: the scanned array including slot 0.  Returns (new_alive_seq,
    seq_probs, seq_score, num_finished) -- copies."""
    can_idx = _c_arr(can_idx, np.int32)
    can_score = _c_arr(can_score, np.float32)
    num = _c_arr(num_scanned, np.int32)
    alive_seq = _c_arr(alive_seq, np.int32)
    rows, max_step = alive_seq.shape
    new_alive = np.array(alive_seq, copy=True)
    probs = np.array(seq_probs, np.float32, copy=True)
    score = np.array(seq_score, np.float32, copy=True)
    fin = _c.c_int(0)
    _lib.lso_refresh_result(_p(can_idx), _p(can_score), _c.c_void_p(num.ctypes.data + 4),
                            _p(alive_seq), _p(new_alive), _p(probs), _p(score), _c.byref(fin),
                            int(vocab_size), int(cur_step), _fl(length_norm_value), int(end_id),
                            rows // beam_size, int(beam_size), max_step)
    return new_alive, probs, score, fin.value


def refresh_cache_i8(num_scanned, can_idx, k_old, v_old, k_new, v_new, beam_size, vocab_size,
                     cur_step, end_id):
    """Caches [n_layer, rows, head, max_step, d]; k_new / v_new updated in place."""
    num = _c_arr(num_scanned, np.int32)
    can_idx = _c_arr(can_idx, np.int32)
    n_layer, rows, head_num, max_step, d = k_old.shape
    for a in (k_old, v_old, k_new, v_new):
        assert a.flags.c_contiguous and a.dtype == np.int8
    _lib.lso_refresh_cache_i8(_c.c_void_p(num.ctypes.data + 4), _p(can_idx), _p(k_old), _p(v_old),
                              _p(k_new), _p(v_new), _c.c_long(rows * head_num * max_step * d),
                              n_layer, rows // beam_size, int(beam_size), d, head_num,
                              int(vocab_size), int(cur_step), max_step, int(end_id))


def write_trg_tokenid_pos_penalty(alive_seq, seq_score, beam_size, out_len):
    alive_seq = _c_arr(alive_seq, np.int32)
    rows, max_step = alive_seq.shape
    score = np.array(seq_score, np.float32, copy=True)
    out = np.empty((rows // beam_size, out_len), np.int32)
    _lib.lso_write_trg_tokenid_pos_penalty(_p(alive_seq), _p(score), _p(out), max_step,
                                           int(beam_size), rows // beam_size, int(out_len))
    return out, score


def write_trg_tokenid_neg_penalty(alive_seq, seq_score, beam_size, end_id, out_len):
    alive_seq = _c_arr(alive_seq, np.int32)
    seq_score = _c_arr(seq_score, np.float32)
    rows, max_step = alive_seq.shape
    out = np.empty((rows // beam_size, out_len), np.int32)
    _lib.lso_write_trg_tokenid_neg_penalty(_p(alive_seq), _p(seq_score), _p(out), max_step,
                                           int(beam_size), int(end_id), rows // beam_size,
                                           int(out_len))
    return out


def write_topk_result(alive_seq, seq_score, beam_size, end_id, out_len):
    alive_seq = _c_arr(alive_seq, np.int32)
    rows, max_step = alive_seq.shape
    score = np.array(seq_score, np.float32, copy=True)
    out = np.empty((rows, out_len), np.int32)
    _lib.lso_write_topk_result(_p(alive_seq), _p(score), _p(out), max_step, int(beam_size),
                               int(end_id), rows, int(out_len))
    return out, score


_DEC_INTS = ("n_layer", "hidden", "inner", "head_num", "max_step", "vocab", "beam_size",
             "extra_decode_length", "start_id", "end_id", "is_post_ln", "use_gelu", "f16")
_DEC_GLOBAL = ("tok_emb_q", "pos_emb", "out_ln_scale", "out_ln_bias", "encdec_kv_kernel",
               "encdec_kv_bias", "logit_bias")
_DEC_PER_LAYER = ("self_ln_scale", "self_ln_bias", "w_self_qkv", "b_self_qkv", "w_self_out",
                  "b_self_out", "encdec_ln_scale", "encdec_ln_bias", "w_encdec_q", "b_encdec_q",
                  "w_encdec_out", "b_encdec_out", "ffn_ln_scale", "ffn_ln_bias", "w_ffn1",
                  "b_ffn1", "w_ffn2", "b_ffn2", "ffn2_colsum")


class _DecWeights(_c.Structure):
    _fields_ = ([(n, _c.c_int) for n in _DEC_INTS] + [("length_penalty", _c.c_float)] +
                [(n, _vp) for n in _DEC_GLOBAL] +
                [(n, _c.c_float) for n in ("emb_clip_max", "output_ln_clip_max",
                                           "logits_clip_max")] +
                [(n, _c.POINTER(_vp)) for n in _DEC_PER_LAYER] +
                [("clip_max", _c.POINTER(_c.c_float))])


class _DecTrace(_c.Structure):
    _fields_ = [("forced_logits", _vp), ("forced_steps", _c.c_int), ("logits_record", _vp),
                ("alive_seq_record", _vp), ("seq_probs_record", _vp), ("steps_run", _c.c_int),
                ("early_stopped", _c.c_int)]


def quant_decoder(weights, enc_out, pad_mask, is_benchmark=False, output_topk=True,
                  forced_logits=None, record=False):
    """Beam-search decode.  ``weights``: dict with the ints of ``_DEC_INTS`` (f16 is
    derived), ``length_penalty``, the arrays of ``_DEC_GLOBAL``, the three clip floats,
    per-layer lists named in ``_DEC_PER_LAYER`` (``ffn2_colsum`` None for GELU) and
    ``clip_max`` float32 [n_layer*19].

    Returns a dict: ``ids`` [batch, k, out_len] (k = beam_size when ``output_topk`` else 1),
    ``scores`` [batch, k], ``steps_run``, ``early_stopped`` and, with ``record``, the
    per-step ``logits`` [steps, rows, vocab], ``alive_seq`` [steps, rows, max_step] and
    ``seq_probs`` [steps, rows].
    """
    enc_out = _c_arr(enc_out)
    pad_mask = _c_arr(pad_mask, np.int32)
    batch, seq_len, H = enc_out.shape
    L, beam, V, max_step = (weights["n_layer"], weights["beam_size"], weights["vocab"],
                            weights["max_step"])
    rows = batch * beam
    T = enc_out.dtype
    keep = []

    def ptr_array(arrs):
        arr = (_vp * L)()
        for i, a in enumerate(arrs):
            if a is not None:
                a = np.ascontiguousarray(a)
                keep.append(a)
                arr[i] = a.ctypes.data
        keep.append(arr)
        return _c.cast(arr, _c.POINTER(_vp))

    w = _DecWeights()
    for n in _DEC_INTS:
        if n != "f16":
            setattr(w, n, int(weights[n]))
    w.f16 = 1 if T == np.float16 else 0
    w.length_penalty = float(weights["length_penalty"])
    for n in _DEC_GLOBAL:
        a = np.ascontiguousarray(weights[n])
        if n != "tok_emb_q" and a.dtype != T:
            raise TypeError("%s must be %s" % (n, T))
        keep.append(a)
        setattr(w, n, a.ctypes.data)
    for n in ("emb_clip_max", "output_ln_clip_max", "logits_clip_max"):
        setattr(w, n, float(weights[n]))
    for n in _DEC_PER_LAYER:
        v = weights.get(n)
        setattr(w, n, ptr_array(v) if v is not None else _c.cast(None, _c.POINTER(_vp)))
    clip = np.ascontiguousarray(weights["clip_max"], np.float32)
    assert clip.size == L * 19
    w.clip_max = clip.ctypes.data_as(_c.POINTER(_c.c_float))

    tr = _DecTrace()
    rec = {}
    if forced_logits is not None:
        forced_logits = _c_arr(forced_logits, np.int8)
        assert forced_logits.shape[1:] == (rows, V)
        tr.forced_logits = forced_logits.ctypes.data
        tr.forced_steps = forced_logits.shape[0]
    if record:
        rec["logits"] = np.zeros((max_step, rows, V), np.int8)
        rec["alive_seq"] = np.zeros((max_step, rows, max_step), np.int32)
        rec["seq_probs"] = np.zeros((max_step, rows), np.float32)
        tr.logits_record = rec["logits"].ctypes.data
        tr.alive_seq_record = rec["alive_seq"].ctypes.data
        tr.seq_probs_record = rec["seq_probs"].ctypes.data
    k = beam if output_topk else 1
    result = np.zeros((batch * k * max_step,), np.int32)
    scores = np.zeros((rows,), np.float32)
    out_len = _c.c_int(0)
    rc = _lib.lso_quant_decoder(_c.byref(w), _p(enc_out), _p(pad_mask), batch, seq_len,
                                int(is_benchmark), int(output_topk), _p(result),
                                _c.byref(out_len), _p(scores), _c.byref(tr))
    if rc != 0:
        raise RuntimeError("lso_quant_decoder failed with code %d" % rc)
    n = out_len.value
    out = {"ids": result[:batch * k * n].reshape(batch, k, n).copy(),
           "scores": scores[:batch * k].reshape(batch, k).copy(),
           "steps_run": tr.steps_run, "early_stopped": bool(tr.early_stopped)}
    for name, a in rec.items():
        out[name] = a[:tr.steps_run]
    return out
