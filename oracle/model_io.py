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
