"""GPT half of the CPU oracle's numpy front-end.  TEST INFRASTRUCTURE ONLY, like the rest
of ``oracle/``."""
import ctypes as _c

import numpy as np

from .oracle import _c_arr, _f16, _fl, _lib, _p, _vp


def gpt_embedding_i8I(token_emb, pos_emb, token_id, real_seq_len, padding_id, pos_offset,
                      dequant_scale):
    """token_emb [vocab, hidden] int8, token_id [batch, seq_len].  Returns (output
    [batch, seq_len, hidden] T, updated real_seq_len copy)."""
    token_emb = _c_arr(token_emb, np.int8)
    pos_emb = _c_arr(pos_emb)
    token_id = _c_arr(token_id, np.int32)
    batch, seq_len = token_id.shape
    hidden = token_emb.shape[1]
    out = np.empty((batch, seq_len, hidden), pos_emb.dtype)
    rsl = np.array(real_seq_len, np.int32, copy=True)
    _lib.lso_gpt_embedding_i8I(_p(token_emb), _p(pos_emb), _p(token_id), _p(out), _p(rsl),
                               int(padding_id), int(pos_offset), _fl(dequant_scale), batch, seq_len,
                               hidden, _f16(pos_emb))
    return out, rsl


def gpt_scores_i8(q, k):
    """q, k [BH, S, d] int8 -> [BH, S, S] int32."""
    q = _c_arr(q, np.int8)
    k = _c_arr(k, np.int8)
    bh, s, d = q.shape
    out = np.empty((bh, s, s), np.int32)
    _lib.lso_gpt_scores_i8(_p(q), _p(k), _p(out), bh, s, d)
    return out


def correlation_softmax_gpt_i32I(correlation, real_seq_len, head_num, attn_scale, dequant_scale,
                                 dtype=np.float16):
    """correlation [batch*head, S, S] int32 -> probabilities T."""
    correlation = _c_arr(correlation, np.int32)
    rsl = _c_arr(real_seq_len, np.int32)
    bh, s, _ = correlation.shape
    out = np.empty((bh, s, s), dtype)
    _lib.lso_correlation_softmax_gpt_i32I(_p(correlation), _p(out), _p(rsl), bh // head_num, s,
                                          head_num, _fl(attn_scale), _fl(dequant_scale), _f16(out))
    return out


def attention_mask_weights_i32I(correlation, real_seq_len, head_num, dst_seq_len, attn_scale,
                                dequant_scale, out):
    """correlation [batch, head * dst_seq_len, src_seq_len] int32; ``out`` (same shape, float16
    or float32) is updated in place: rows of queries beyond the real length keep their values."""
    correlation = _c_arr(correlation, np.int32)
    rsl = _c_arr(real_seq_len, np.int32)
    batch, rows, src = correlation.shape
    assert rows == head_num * dst_seq_len and out.shape == correlation.shape
    assert out.flags["C_CONTIGUOUS"]
    _lib.lso_attention_mask_weights_i32I(_p(correlation), _p(out), _p(rsl), batch, dst_seq_len, src,
                                         head_num, _fl(attn_scale), _fl(dequant_scale), _f16(out))
    return out


def arrange_qkv_with_cache_i8I_i8O(ori_qkv, qkv_bias, k_cache, v_cache, dequant_scale, quant_scale):
    """ori_qkv [batch, 3H]; caches [batch, head, seq_len-1, d].  Returns (new_q
    [batch, head, 1, d], new_k, new_v [batch, head, seq_len, d])."""
    ori_qkv = _c_arr(ori_qkv, np.int8)
    qkv_bias = _c_arr(qkv_bias)
    k_cache = _c_arr(k_cache, np.int8)
    v_cache = _c_arr(v_cache, np.int8)
    batch, heads, old_len, d = k_cache.shape
    seq_len = old_len + 1
    new_q = np.empty((batch, heads, 1, d), np.int8)
    new_k = np.empty((batch, heads, seq_len, d), np.int8)
    new_v = np.empty_like(new_k)
    _lib.lso_arrange_qkv_with_cache_i8I_i8O(_p(ori_qkv), _p(qkv_bias), _p(new_q), _p(new_k),
                                            _p(k_cache), _p(new_v), _p(v_cache), batch, seq_len, d,
                                            heads, _fl(dequant_scale), _fl(quant_scale),
                                            _f16(qkv_bias))
    return new_q, new_k, new_v


def topk_sample_i8I_greedy(logits, old_input_ids, logits_seq_len, eos_id, dequant_scale):
    """logits [batch*logits_seq_len, vocab]; old ids [batch, seq_len].  Returns (new ids
    [batch, seq_len+1], sampled ids [batch], unfinished flag)."""
    logits = _c_arr(logits, np.int8)
    old = np.asarray(old_input_ids, np.int32)
    batch, seq_len = old.shape
    vocab = logits.shape[-1]
    buf = np.zeros(batch * seq_len + batch, np.int32)
    buf[:batch * seq_len] = old.reshape(-1)
    new = np.empty((batch, seq_len + 1), np.int32)
    unf = _c.c_int(0)
    _lib.lso_topk_sample_i8I_greedy(_p(logits), _p(buf), _p(new), vocab, batch, seq_len,
                                    int(logits_seq_len), _c.byref(unf), int(eos_id),
                                    _fl(dequant_scale))
    return new, buf[batch * seq_len:].copy(), unf.value


def ppl_i8I(logits, input_ids, real_seq_len, dequant_scale):
    logits = _c_arr(logits, np.int8)
    input_ids = _c_arr(input_ids, np.int32)
    rsl = _c_arr(real_seq_len, np.int32)
    batch, seq_len = input_ids.shape
    vocab = logits.shape[-1]
    ppl = np.zeros(batch, np.float32)
    _lib.lso_ppl_i8I(_p(logits), _p(input_ids), _p(rsl), _p(ppl), vocab, _fl(dequant_scale), batch,
                     seq_len)
    return ppl


_GPT_INTS = ("n_layer", "hidden", "inner", "head_num", "max_step", "vocab", "padding_id", "eos_id",
             "extra_decode_length", "f16")
_GPT_GLOBAL = ("tok_emb_q", "pos_emb", "out_ln_scale", "out_ln_bias")
_GPT_PER_LAYER = ("ln1_scale", "ln1_bias", "w_qkv", "b_qkv", "w_out", "b_out", "ln2_scale",
                  "ln2_bias", "w_ffn1", "b_ffn1", "w_ffn2", "b_ffn2")


class _GptWeights(_c.Structure):
    _fields_ = ([(n, _c.c_int) for n in _GPT_INTS] + [(n, _vp) for n in _GPT_GLOBAL] +
                [(n, _c.c_float) for n in ("emb_clip_max", "output_ln_clip_max",
                                           "logits_clip_max")] +
                [(n, _c.POINTER(_vp)) for n in _GPT_PER_LAYER] +
                [("clip_max", _c.POINTER(_c.c_float))])


def _weights_struct(weights, keep):
    L = weights["n_layer"]
    T = np.asarray(weights["pos_emb"]).dtype

    def ptr_array(arrs):
        arr = (_vp * L)()
        for i, a in enumerate(arrs):
            a = np.ascontiguousarray(a)
            keep.append(a)
            arr[i] = a.ctypes.data
        keep.append(arr)
        return _c.cast(arr, _c.POINTER(_vp))

    w = _GptWeights()
    for n in _GPT_INTS:
        if n != "f16":
            setattr(w, n, int(weights[n]))
    w.f16 = 1 if T == np.float16 else 0
    for n in _GPT_GLOBAL:
        a = np.ascontiguousarray(weights[n])
        keep.append(a)
        setattr(w, n, a.ctypes.data)
    for n in ("emb_clip_max", "output_ln_clip_max", "logits_clip_max"):
        setattr(w, n, float(weights[n]))
    for n in _GPT_PER_LAYER:
        setattr(w, n, ptr_array(weights[n]))
    clip = np.ascontiguousarray(weights["clip_max"], np.float32)
    assert clip.size == L * 12
    keep.append(clip)
    w.clip_max = clip.ctypes.data_as(_c.POINTER(_c.c_float))
    return w


def quant_gpt_ppl(weights, token_ids):
    token_ids = _c_arr(token_ids, np.int32)
    batch, seq_len = token_ids.shape
    keep = []
    w = _weights_struct(weights, keep)
    ppl = np.zeros(batch, np.float32)
    rc = _lib.lso_quant_gpt_ppl(_c.byref(w), _p(token_ids), batch, seq_len, _p(ppl))
    if rc != 0:
        raise RuntimeError("lso_quant_gpt_ppl failed with code %d" % rc)
    return ppl


def quant_gpt_sample(weights, token_ids, is_benchmark=False, forced_logits=None, record=False):
    """Greedy generation.  Returns dict: ``ids`` [batch, out_len], ``steps_run`` and, with
    ``record``, ``logits`` [steps, batch, vocab] (last-position logits of every step)."""
    token_ids = _c_arr(token_ids, np.int32)
    batch, seq_len = token_ids.shape
    keep = []
    w = _weights_struct(weights, keep)
    max_step, V = weights["max_step"], weights["vocab"]
    out = np.zeros(batch * max_step, np.int32)
    out_len, steps = _c.c_int(0), _c.c_int(0)
    rec = np.zeros((max_step, batch, V), np.int8) if record else None
    forced_steps = 0
    if forced_logits is not None:
        forced_logits = _c_arr(forced_logits, np.int8)
        assert forced_logits.shape[1:] == (batch, V)
        forced_steps = forced_logits.shape[0]
    rc = _lib.lso_quant_gpt_sample(_c.byref(w), _p(token_ids), batch, seq_len, int(is_benchmark),
                                   _p(out), _c.byref(out_len), _p(forced_logits), forced_steps,
                                   _p(rec), _c.byref(steps))
    if rc != 0:
        raise RuntimeError("lso_quant_gpt_sample failed with code %d" % rc)
    res = {"ids": out[:batch * out_len.value].reshape(batch, out_len.value).copy(),
           "steps_run": steps.value}
    if record:
        res["logits"] = rec[:steps.value]
    return res


_GPT_CLIP_NAMES = ["multihead_project_kernel_qkv_clip_max", "multihead_project_kernel_output_clip_max",
                   "ffn_first_kernel_clip_max", "ffn_second_kernel_clip_max", "multihead_ln_clip_max",
                   "multihead_project_output_clip_max", "ffn_ln_clip_max", "ffn_first_act_clip_max",
                   "multihead_qkv_dense_clip_max", "multihead_output_dense_clip_max",
                   "ffn_first_output_clip_max", "self_qkv_bias_out_clip_max"]


def gpt_weights_from_message(msg, cfg, dtype=np.float16):
    """QuantGpt message dict -> weights dict of the oracle.

    Loader semantics of the reference (inference/proto/quant_gpt_weight.cc:36-245): sizes come
    from the tensors; the token embedding is stored [hidden, vocab]
    (examples/inference/python/export/huggingface/ls_torch_hf_quant_gpt2_export.py:138-143) and
    its transpose serves both the row lookup and, as [N, K] codes, the logits GEMM; 12 clip values per layer in the order of
    ``_GPT_CLIP_NAMES``; extra_decode_length <= 0 means max_step.
    """
    from .model_io import _codes
    H, I = cfg["hidden"], cfg["inner"]
    emb, conf = msg["src_embedding"], msg["model_conf"]

    def T(v):
        return np.asarray(v, np.float32).astype(dtype)

    extra = conf.get("extra_decode_length", 0)
    w = dict(n_layer=len(msg["encoder_stack"]), hidden=H, inner=I, head_num=conf["head_num"],
             max_step=cfg["max_step"], vocab=cfg["vocab"], padding_id=conf.get("src_padding_id", 0),
             eos_id=conf.get("eos_id", 0),
             extra_decode_length=extra if extra > 0 else cfg["max_step"])
    w["tok_emb_q"] = _codes(emb["token_embedding"], H, cfg["vocab"])  # -> [vocab, hidden]
    w["pos_emb"] = T(emb["position_embedding"]).reshape(cfg["max_step"], H)
    w["out_ln_scale"] = T(emb["norm_scale"])
    w["out_ln_bias"] = T(emb["norm_bias"])
    for n in ("emb_clip_max", "output_ln_clip_max", "logits_clip_max"):
        w[n] = np.float32(emb[n])
    names = {"ln1_scale": "multihead_norm_scale", "ln1_bias": "multihead_norm_bias",
             "b_qkv": "multihead_project_bias_qkv", "b_out": "multihead_project_bias_output",
             "ln2_scale": "ffn_norm_scale", "ln2_bias": "ffn_norm_bias",
             "b_ffn1": "ffn_first_bias", "b_ffn2": "ffn_second_bias"}
    kernels = {"w_qkv": ("multihead_project_kernel_qkv", H, 3 * H),
               "w_out": ("multihead_project_kernel_output", H, H),
               "w_ffn1": ("ffn_first_kernel", H, I), "w_ffn2": ("ffn_second_kernel", I, H)}
    per = {k: [] for k in list(names) + list(kernels)}
    clip = []
    for l in msg["encoder_stack"]:
        for k, n in names.items():
            per[k].append(T(l[n]))
        for k, (n, r, c) in kernels.items():
            per[k].append(_codes(l[n], r, c))
        clip += [np.float32(l[n]) for n in _GPT_CLIP_NAMES]
    w.update(per)
    w["clip_max"] = np.asarray(clip, np.float32)
    return w
