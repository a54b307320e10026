"""Model-file (message dict) -> oracle weights.  TEST INFRASTRUCTURE ONLY, like the
rest of ``oracle/``: used by the tests, the smoke check and the benchmark's
``cpu_baseline`` leg."""
import numpy as np


def oracle_weights_from_message(msg, cfg, dtype=np.float16):
    """QuantBert message dict (file form) -> weights dict of the oracle's encoder.

    Follows the loader of the reference: kernels are stored [in, out] as uint8 =
    code + 127 and the engine multiplies with the transposed [out, in] int8 codes
    (inference/proto/quant_bert_weight.cc, model/quant_bert_encoder.cc.cu:132-154);
    float vectors are cast to T; the ReLU column sum is taken over the T-rounded
    dequantised FFN2 kernel (model/quant_bert_encoder.cc.cu:156-175).
    """
    from . import oracle
    H, I, L = cfg["hidden"], cfg["inner"], cfg["n_layer"]
    emb = msg["src_embedding"]

    def codes(u8, rows, cols, transpose=True):
        q = np.clip(np.asarray(u8, np.int32).reshape(rows, cols) - 127, -127, 127).astype(np.int8)
        return np.ascontiguousarray(q.T) if transpose else q

    def T(v):
        return np.asarray(v, np.float32).astype(dtype)

    names = ["multihead_project_kernel_qkv_clip_max", "multihead_project_kernel_output_clip_max",
             "ffn_first_kernel_clip_max", "ffn_second_kernel_clip_max", "multihead_ln_clip_max",
             "multihead_project_output_clip_max", "ffn_ln_clip_max", "ffn_first_act_clip_max",
             "multihead_qkv_dense_clip_max", "multihead_output_dense_clip_max",
             "ffn_first_output_clip_max"]
    w = dict(cfg)
    w["tok_emb_q"] = codes(emb["token_embedding"], cfg["vocab"], H, transpose=False)
    w["pos_emb"] = T(emb["position_embedding"]).reshape(cfg["max_step"], H)
    w["final_ln_scale"] = T(emb["norm_scale"])
    w["final_ln_bias"] = T(emb["norm_bias"])
    w["emb_clip_max"] = np.float32(emb["emb_clip_max"])
    per = {k: [] for k in ("ln1_scale", "ln1_bias", "w_qkv", "b_qkv", "w_out", "b_out", "ln2_scale",
                           "ln2_bias", "w_ffn1", "b_ffn1", "w_ffn2", "b_ffn2", "ffn2_colsum")}
    clip = []
    for l in msg["encoder_stack"]:
        per["ln1_scale"].append(T(l["multihead_norm_scale"]))
        per["ln1_bias"].append(T(l["multihead_norm_bias"]))
        per["w_qkv"].append(codes(l["multihead_project_kernel_qkv"], H, 3 * H))
        per["b_qkv"].append(T(l["multihead_project_bias_qkv"]))
        per["w_out"].append(codes(l["multihead_project_kernel_output"], H, H))
        per["b_out"].append(T(l["multihead_project_bias_output"]))
        per["ln2_scale"].append(T(l["ffn_norm_scale"]))
        per["ln2_bias"].append(T(l["ffn_norm_bias"]))
        per["w_ffn1"].append(codes(l["ffn_first_kernel"], H, I))
        per["b_ffn1"].append(T(l["ffn_first_bias"]))
        per["w_ffn2"].append(codes(l["ffn_second_kernel"], I, H))
        per["b_ffn2"].append(T(l["ffn_second_bias"]))
        clip += [np.float32(l[n]) for n in names]
        if cfg["use_gelu"]:
            per["ffn2_colsum"].append(None)
        else:
            c3, c7 = np.float32(l["ffn_second_kernel_clip_max"]), np.float32(l["ffn_first_act_clip_max"])
            u8 = np.asarray(l["ffn_second_kernel"], np.float32).reshape(I, H)
            deq = ((u8 - np.float32(127)) * c3 / np.float32(127)).astype(dtype)
            per["ffn2_colsum"].append(oracle.scaled_colsum(deq, float(c7 / np.float32(2))))
    w.update(per)
    if cfg["use_gelu"]:
        w["ffn2_colsum"] = None
    w["clip_max"] = np.asarray(clip, np.float32)
    return w


_ENC_CLIP_NAMES = ["multihead_project_kernel_qkv_clip_max", "multihead_project_kernel_output_clip_max",
                   "ffn_first_kernel_clip_max", "ffn_second_kernel_clip_max", "multihead_ln_clip_max",
                   "multihead_project_output_clip_max", "ffn_ln_clip_max", "ffn_first_act_clip_max",
                   "multihead_qkv_dense_clip_max", "multihead_output_dense_clip_max",
                   "ffn_first_output_clip_max", "ffn_second_output_clip_max"]

_DEC_CLIP_NAMES = ["self_project_kernel_qkv_clip_max", "self_project_kernel_output_clip_max",
                   "encdec_project_kernel_q_clip_max", "encdec_project_kernel_output_clip_max",
                   "ffn_first_kernel_clip_max", "ffn_second_kernel_clip_max", "self_ln_clip_max",
                   "self_project_output_clip_max", "encdec_ln_clip_max",
                   "encdec_project_output_clip_max", "ffn_ln_clip_max", "ffn_first_act_clip_max",
                   "self_qkv_dense_clip_max", "self_output_dense_clip_max",
                   "encdec_q_dense_clip_max", "encdec_output_dense_clip_max",
                   "ffn_first_output_clip_max", "ffn_second_output_clip_max",
                   "self_qkv_bias_out_clip_max"]


def _codes(u8, rows, cols, transpose=True):
    q = np.clip(np.asarray(u8, np.int32).reshape(rows, cols) - 127, -127, 127).astype(np.int8)
    return np.ascontiguousarray(q.T) if transpose else q


def _dequant(u8, clip, dtype):
    """tools/util.cc.cu:346-348 followed by the cast to T."""
    return ((np.asarray(u8, np.float32) - np.float32(127)) * np.float32(clip) /
            np.float32(127)).astype(dtype)


def oracle_transformer_weights_from_message(msg, cfg, dtype=np.float16):
    """QuantTransformer message dict -> (encoder weights, decoder weights) of the oracle.

    Loader semantics of the reference (inference/proto/quant_transformer_weight.cc:35-510):
    sizes come from the tensors, trg_end_id 0 means vocab-1, the clip tables are 12 floats per
    encoder layer and 19 per decoder layer in the order of ``_ENC_CLIP_NAMES`` /
    ``_DEC_CLIP_NAMES``, and the target embedding is stored [hidden, vocab] (it is the logits
    kernel); the oracle multiplies with [N, K] codes, so every kernel is transposed here.
    """
    from . import oracle
    H, I = cfg["hidden"], cfg["inner"]
    conf = msg["model_conf"]

    def T(v):
        return np.asarray(v, np.float32).astype(dtype)

    def colsum(u8, c_w, c_act):
        deq = _dequant(np.asarray(u8).reshape(I, H), c_w, dtype)
        return oracle.scaled_colsum(deq, float(np.float32(c_act) / np.float32(2)))

    use_gelu = bool(conf.get("use_gelu", False))
    is_post_ln = bool(conf.get("is_post_ln", False))
    # ---- encoder ----
    se = msg["src_embedding"]
    enc = dict(n_layer=len(msg["encoder_stack"]), hidden=H, inner=I, head_num=conf["head_num"],
               max_step=cfg["max_step"], vocab=cfg["src_vocab"],
               padding_id=conf.get("src_padding_id", 0), is_post_ln=is_post_ln, use_gelu=use_gelu,
               clip_stride=12, emb_scaled=1)
    enc["tok_emb_q"] = _codes(se["token_embedding"], cfg["src_vocab"], H, transpose=False)
    enc["pos_emb"] = T(se["position_embedding"]).reshape(cfg["max_step"], H)
    enc["final_ln_scale"] = T(se["norm_scale"])
    enc["final_ln_bias"] = T(se["norm_bias"])
    enc["emb_clip_max"] = np.float32(se["emb_clip_max"])
    per = {k: [] for k in ("ln1_scale", "ln1_bias", "w_qkv", "b_qkv", "w_out", "b_out", "ln2_scale",
                           "ln2_bias", "w_ffn1", "b_ffn1", "w_ffn2", "b_ffn2", "ffn2_colsum")}
    clip = []
    for l in msg["encoder_stack"]:
        per["ln1_scale"].append(T(l["multihead_norm_scale"]))
        per["ln1_bias"].append(T(l["multihead_norm_bias"]))
        per["w_qkv"].append(_codes(l["multihead_project_kernel_qkv"], H, 3 * H))
        per["b_qkv"].append(T(l["multihead_project_bias_qkv"]))
        per["w_out"].append(_codes(l["multihead_project_kernel_output"], H, H))
        per["b_out"].append(T(l["multihead_project_bias_output"]))
        per["ln2_scale"].append(T(l["ffn_norm_scale"]))
        per["ln2_bias"].append(T(l["ffn_norm_bias"]))
        per["w_ffn1"].append(_codes(l["ffn_first_kernel"], H, I))
        per["b_ffn1"].append(T(l["ffn_first_bias"]))
        per["w_ffn2"].append(_codes(l["ffn_second_kernel"], I, H))
        per["b_ffn2"].append(T(l["ffn_second_bias"]))
        clip += [np.float32(l[n]) for n in _ENC_CLIP_NAMES]
        per["ffn2_colsum"].append(None if use_gelu else colsum(
            l["ffn_second_kernel"], l["ffn_second_kernel_clip_max"], l["ffn_first_act_clip_max"]))
    enc.update(per)
    if use_gelu:
        enc["ffn2_colsum"] = None
    enc["clip_max"] = np.asarray(clip, np.float32)

    # ---- decoder ----
    te = msg["trg_embedding"]
    V = cfg["trg_vocab"]
    Ld = len(msg["decoder_stack"])
    end_id = conf.get("trg_end_id", 0) or V - 1
    dec = dict(n_layer=Ld, hidden=H, inner=I, head_num=conf["head_num"], max_step=cfg["max_step"],
               vocab=V, beam_size=conf["beam_size"],
               extra_decode_length=conf.get("extra_decode_length", 0),
               start_id=conf.get("trg_start_id", 0), end_id=end_id, is_post_ln=is_post_ln,
               use_gelu=use_gelu, length_penalty=np.float32(conf.get("length_penalty", 0.0)))
    dec["tok_emb_q"] = _codes(te["token_embedding"], H, V)  # [vocab, hidden]
    dec["pos_emb"] = T(te["position_embedding"]).reshape(cfg["max_step"], H)
    dec["out_ln_scale"] = T(te["norm_scale"])
    dec["out_ln_bias"] = T(te["norm_bias"])
    kv = np.asarray(te["encode_output_project_kernel_kv"]).reshape(Ld, H, 2 * H)
    kv_clip = np.asarray(te["encode_output_project_kernel_kv_clip_max"], np.float32)
    # file: per layer [hidden, 2*hidden]; the GEMM kernel is [hidden, n_layer*2*hidden]
    # (model/quant_decoder.cc.cu:497-501 with lda = kv_dim): the flat buffer is re-read with
    # that leading dimension, exactly as the reference hands it to cuBLAS.
    flat = np.concatenate([_dequant(kv[l], kv_clip[l], dtype).reshape(-1) for l in range(Ld)])
    dec["encdec_kv_kernel"] = np.ascontiguousarray(flat.reshape(H, Ld * 2 * H))
    dec["encdec_kv_bias"] = T(te["encode_output_project_bias_kv"])
    dec["logit_bias"] = T(te["shared_bias"])
    dec["emb_clip_max"] = np.float32(te["emb_clip_max"])
    dec["output_ln_clip_max"] = np.float32(te["output_ln_clip_max"])
    dec["logits_clip_max"] = np.float32(te["logits_clip_max"])
    names = {"self_ln_scale": "self_norm_scale", "self_ln_bias": "self_norm_bias",
             "b_self_qkv": "self_project_bias_qkv", "b_self_out": "self_project_bias_output",
             "encdec_ln_scale": "encdec_norm_scale", "encdec_ln_bias": "encdec_norm_bias",
             "b_encdec_q": "encdec_project_bias_q", "b_encdec_out": "encdec_project_bias_output",
             "ffn_ln_scale": "ffn_norm_scale", "ffn_ln_bias": "ffn_norm_bias",
             "b_ffn1": "ffn_first_bias", "b_ffn2": "ffn_second_bias"}
    kernels = {"w_self_qkv": ("self_project_kernel_qkv", H, 3 * H),
               "w_self_out": ("self_project_kernel_output", H, H),
               "w_encdec_q": ("encdec_project_kernel_q", H, H),
               "w_encdec_out": ("encdec_project_kernel_output", H, H),
               "w_ffn1": ("ffn_first_kernel", H, I), "w_ffn2": ("ffn_second_kernel", I, H)}
    per = {k: [] for k in list(names) + list(kernels) + ["ffn2_colsum"]}
    clip = []
    for l in msg["decoder_stack"]:
        for k, n in names.items():
            per[k].append(T(l[n]))
        for k, (n, r, c) in kernels.items():
            per[k].append(_codes(l[n], r, c))
        clip += [np.float32(l[n]) for n in _DEC_CLIP_NAMES]
        per["ffn2_colsum"].append(None if use_gelu else colsum(
            l["ffn_second_kernel"], l["ffn_second_kernel_clip_max"], l["ffn_first_act_clip_max"]))
    dec.update(per)
    if use_gelu:
        dec["ffn2_colsum"] = None
    dec["clip_max"] = np.asarray(clip, np.float32)
    return enc, dec
