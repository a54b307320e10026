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
        ("ffn2_colsum", _c.POINTER(_vp)), ("clip_max", _c.POINTER(_c.c_float))]


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
    assert clip.size == L * 11
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
