"""Random-init quantised model files in the reference's own on-disk format.

There is no network for checkpoints, so the benchmark, the smoke check and the
tests run on synthetic models: weights ~ N(0, 0.02) quantised per tensor with
clip_max = 4 sigma, stored exactly as LightSeq's exporters store them (uint8 =
code + 127 plus a clip_max float, lightseq/training/ops/pytorch/export_quant.py:12-20)
in a ``quant_bert.proto`` message, so they load through the same
``QuantBert(path, max_batch)`` entry point as an exported checkpoint would.
Activation clip values are analytic 4-sigma estimates for random-init weights.
"""
import numpy as np

from . import proto

W_STD = 0.02


def quantize_u8(x, clip):
    """float array -> stored uint8 (= symmetric int8 code + 127)."""
    scale = np.float32(clip) / np.float32(127)
    q = np.floor(x.astype(np.float32) / scale + np.float32(0.5))
    return (np.clip(q, -127, 127) + 127).astype(np.uint8)


def bert_config(name):
    """Shapes of the named synthetic configurations."""
    cfgs = {
        # BERT-base-shaped int8 encoder stack (b32, s128)
        "bert_base": dict(n_layer=12, hidden=768, inner=3072, head_num=12, max_step=512,
                          vocab=30522, padding_id=0, is_post_ln=True, use_gelu=True),
        # Transformer-base-shaped single encoder layer (b8, s64), ReLU, post-LN
        "transformer_base_layer": dict(n_layer=1, hidden=512, inner=2048, head_num=8, max_step=128,
                                       vocab=1000, padding_id=0, is_post_ln=True, use_gelu=False),
        "tiny": dict(n_layer=2, hidden=128, inner=256, head_num=2, max_step=64, vocab=200,
                     padding_id=0, is_post_ln=True, use_gelu=True),
    }
    return dict(cfgs[name])


def make_quant_bert(cfg, seed=0, ln_noise=0.02):
    """Build the QuantBert message (a dict for :func:`proto.encode`)."""
    rng = np.random.default_rng(seed)
    H, I, L = cfg["hidden"], cfg["inner"], cfg["n_layer"]
    clip_w = 4 * W_STD

    def normal(*shape, std=W_STD):
        return rng.standard_normal(shape, dtype=np.float32) * np.float32(std)

    def ln_params():
        return ((1 + normal(H, std=ln_noise)).astype(np.float32), normal(H, std=ln_noise))

    g_final, b_final = ln_params()
    emb = {
        "token_embedding": quantize_u8(normal(cfg["vocab"], H), clip_w).reshape(-1),
        "position_embedding": normal(cfg["max_step"], H).reshape(-1),
        "norm_scale": g_final, "norm_bias": b_final, "emb_clip_max": clip_w,
    }
    proj = 4 * W_STD * np.sqrt(H)  # 4 sigma of x @ W for x ~ N(0, 1)
    layers = []
    for _ in range(L):
        g1, b1 = ln_params()
        g2, b2 = ln_params()
        ctx_clip = proj / 4  # attention averages over many keys
        act_clip = proj if cfg["use_gelu"] else proj * 0.75
        layers.append({
            "multihead_norm_scale": g1, "multihead_norm_bias": b1,
            "multihead_project_kernel_qkv": quantize_u8(normal(H, 3 * H), clip_w).reshape(-1),
            "multihead_project_bias_qkv": normal(3 * H),
            "multihead_project_kernel_output": quantize_u8(normal(H, H), clip_w).reshape(-1),
            "multihead_project_bias_output": normal(H),
            "ffn_norm_scale": g2, "ffn_norm_bias": b2,
            "ffn_first_kernel": quantize_u8(normal(H, I), clip_w).reshape(-1),
            "ffn_first_bias": normal(I),
            "ffn_second_kernel": quantize_u8(normal(I, H), clip_w).reshape(-1),
            "ffn_second_bias": normal(H),
            "multihead_project_kernel_qkv_clip_max": clip_w,
            "multihead_project_kernel_output_clip_max": clip_w,
            "ffn_first_kernel_clip_max": clip_w, "ffn_second_kernel_clip_max": clip_w,
            "multihead_ln_clip_max": 4.0,
            "multihead_project_output_clip_max": float(ctx_clip),
            "ffn_ln_clip_max": 4.0,
            "ffn_first_act_clip_max": float(act_clip),
            "multihead_qkv_dense_clip_max": float(proj),
            "multihead_output_dense_clip_max": float(proj * ctx_clip / 4),
            "ffn_first_output_clip_max": float(proj),
        })
    conf = {"head_num": cfg["head_num"], "src_padding_id": cfg["padding_id"],
            "is_post_ln": cfg["is_post_ln"], "use_gelu": cfg["use_gelu"], "multilg_type": 0}
    return {"src_embedding": emb, "encoder_stack": layers, "model_conf": conf}


def write_quant_bert(path, cfg, seed=0, ln_noise=0.02):
    """Write a synthetic QuantBert model file; returns the message dict."""
    msg = make_quant_bert(cfg, seed=seed, ln_noise=ln_noise)
    with open(path, "wb") as f:
        f.write(proto.encode("QuantBert", msg))
    return msg


def make_token_ids(cfg, batch, seq_len, seed=0, min_len=None):
    """Token ids uniform over the vocabulary (excluding the pad id), per-sequence
    valid lengths uniform in [min_len, seq_len], right padded with the pad id."""
    rng = np.random.default_rng(seed + 1)
    min_len = seq_len // 4 if min_len is None else min_len
    ids = rng.integers(1, cfg["vocab"], size=(batch, seq_len), dtype=np.int32)
    if cfg["padding_id"] != 0:
        ids[ids == cfg["padding_id"]] = 0
    lens = rng.integers(min_len, seq_len + 1, size=batch)
    lens[0] = seq_len
    ids[np.arange(seq_len)[None, :] >= lens[:, None]] = cfg["padding_id"]
    return ids, lens


# --------------------------------------------------------------------------- #
# QuantTransformer (encoder + decoder with beam search)
# --------------------------------------------------------------------------- #
def transformer_config(name):
    """Shapes of the named synthetic encoder-decoder configurations."""
    cfgs = {
        # Transformer-big-shaped en-de model: 6+6 layers, hidden 1024, 16 heads, beam 4
        "transformer_big": dict(n_enc_layer=6, n_dec_layer=6, hidden=1024, inner=4096, head_num=16,
                                max_step=64, src_vocab=32000, trg_vocab=32000, padding_id=0,
                                start_id=2, end_id=3, beam_size=4, extra_decode_length=50,
                                length_penalty=0.6, is_post_ln=False, use_gelu=False),
        "tiny": dict(n_enc_layer=2, n_dec_layer=2, hidden=128, inner=256, head_num=4, max_step=32,
                     src_vocab=300, trg_vocab=320, padding_id=0, start_id=2, end_id=3, beam_size=4,
                     extra_decode_length=12, length_penalty=0.6, is_post_ln=False, use_gelu=False),
    }
    return dict(cfgs[name])


def make_quant_transformer(cfg, seed=0, ln_noise=0.02, eos_bias=None, w_std=None):
    """Build the QuantTransformer message (a dict for :func:`proto.encode`).

    ``eos_bias`` is added to the end-of-sentence entry of the logit bias so that
    random-init models finish some beams before the length limit; the default is
    1.5 sigma of the logits.  ``w_std`` is the standard deviation of the layer kernels
    (default: ``cfg["w_std"]`` or 0.02); the embedding tables always use 0.02.  Larger layer
    kernels make the sublayers, and so the context, matter next to the tied embedding.
    """
    rng = np.random.default_rng(seed)
    H, I = cfg["hidden"], cfg["inner"]
    Le, Ld = cfg["n_enc_layer"], cfg["n_dec_layer"]
    w_std = float(cfg.get("w_std", W_STD) if w_std is None else w_std)
    clip_e = 4 * W_STD
    clip_w = 4 * w_std

    def normal(*shape, std=W_STD):
        return rng.standard_normal(shape, dtype=np.float32) * np.float32(std)

    def ln_params():
        return ((1 + normal(H, std=ln_noise)).astype(np.float32), normal(H, std=ln_noise))

    def qk(rows, cols):
        return quantize_u8(normal(rows, cols, std=w_std), clip_w).reshape(-1)

    def qe(rows, cols):
        return quantize_u8(normal(rows, cols), clip_e).reshape(-1)

    proj = float(4 * w_std * np.sqrt(H))  # 4 sigma of x @ W for x ~ N(0, 1)
    ctx_clip = proj / 4
    act_clip = proj if cfg["use_gelu"] else proj * 0.75

    g, b = ln_params()
    src_emb = {
        "token_embedding": qe(cfg["src_vocab"], H),
        "position_embedding": normal(cfg["max_step"], H).reshape(-1),
        "norm_scale": g, "norm_bias": b, "emb_clip_max": clip_e,
    }
    enc_layers = []
    for _ in range(Le):
        g1, b1 = ln_params()
        g2, b2 = ln_params()
        enc_layers.append({
            "multihead_norm_scale": g1, "multihead_norm_bias": b1,
            "multihead_project_kernel_qkv": qk(H, 3 * H), "multihead_project_bias_qkv": normal(3 * H),
            "multihead_project_kernel_output": qk(H, H), "multihead_project_bias_output": normal(H),
            "ffn_norm_scale": g2, "ffn_norm_bias": b2,
            "ffn_first_kernel": qk(H, I), "ffn_first_bias": normal(I),
            "ffn_second_kernel": qk(I, H), "ffn_second_bias": normal(H),
            "multihead_project_kernel_qkv_clip_max": clip_w,
            "multihead_project_kernel_output_clip_max": clip_w,
            "ffn_first_kernel_clip_max": clip_w, "ffn_second_kernel_clip_max": clip_w,
            "multihead_ln_clip_max": 4.0, "multihead_project_output_clip_max": ctx_clip,
            "ffn_ln_clip_max": 4.0, "ffn_first_act_clip_max": act_clip,
            "multihead_qkv_dense_clip_max": proj,
            "multihead_output_dense_clip_max": proj * ctx_clip / 4,
            "ffn_first_output_clip_max": proj, "ffn_second_output_clip_max": proj,
        })

    g, b = ln_params()
    logit_sigma = W_STD * np.sqrt(H)
    shared_bias = normal(cfg["trg_vocab"], std=0.1 * logit_sigma)
    shared_bias[cfg["end_id"]] += np.float32(1.5 * logit_sigma if eos_bias is None else eos_bias)
    # the embedding table is stored [hidden, vocab]: it is the logits kernel
    trg_emb = {
        "token_embedding": qe(H, cfg["trg_vocab"]),
        # a strong position signal keeps the random-init decoder from repeating one token
        "position_embedding": normal(cfg["max_step"], H, std=0.1).reshape(-1),
        "norm_scale": g, "norm_bias": b,
        "encode_output_project_kernel_kv": np.concatenate([qk(H, 2 * H) for _ in range(Ld)]),
        "encode_output_project_bias_kv": normal(2 * H * Ld),
        "shared_bias": shared_bias,
        "emb_clip_max": clip_e,
        "encode_output_project_kernel_kv_clip_max": np.full(Ld, clip_w, np.float32),
        "output_ln_clip_max": 4.0, "logits_clip_max": float(4 * logit_sigma),
    }
    dec_layers = []
    for _ in range(Ld):
        g1, b1 = ln_params()
        g2, b2 = ln_params()
        g3, b3 = ln_params()
        dec_layers.append({
            "self_norm_scale": g1, "self_norm_bias": b1,
            "self_project_kernel_qkv": qk(H, 3 * H), "self_project_bias_qkv": normal(3 * H),
            "self_project_kernel_output": qk(H, H), "self_project_bias_output": normal(H),
            "encdec_norm_scale": g2, "encdec_norm_bias": b2,
            "encdec_project_kernel_q": qk(H, H), "encdec_project_bias_q": normal(H),
            "encdec_project_kernel_output": qk(H, H), "encdec_project_bias_output": normal(H),
            "ffn_norm_scale": g3, "ffn_norm_bias": b3,
            "ffn_first_kernel": qk(H, I), "ffn_first_bias": normal(I),
            "ffn_second_kernel": qk(I, H), "ffn_second_bias": normal(H),
            "self_project_kernel_qkv_clip_max": clip_w, "self_project_kernel_output_clip_max": clip_w,
            "encdec_project_kernel_q_clip_max": clip_w,
            "encdec_project_kernel_output_clip_max": clip_w,
            "ffn_first_kernel_clip_max": clip_w, "ffn_second_kernel_clip_max": clip_w,
            "self_ln_clip_max": 4.0, "self_project_output_clip_max": proj / 2,
            "encdec_ln_clip_max": 4.0, "encdec_project_output_clip_max": ctx_clip,
            "ffn_ln_clip_max": 4.0, "ffn_first_act_clip_max": act_clip,
            "self_qkv_dense_clip_max": proj, "self_output_dense_clip_max": proj * proj / 8,
            "encdec_q_dense_clip_max": proj, "encdec_output_dense_clip_max": proj * ctx_clip / 4,
            "ffn_first_output_clip_max": proj, "ffn_second_output_clip_max": proj,
            "self_qkv_bias_out_clip_max": proj,
        })
    conf = {"head_num": cfg["head_num"], "beam_size": cfg["beam_size"],
            "extra_decode_length": cfg["extra_decode_length"],
            "length_penalty": cfg["length_penalty"], "src_padding_id": cfg["padding_id"],
            "trg_start_id": cfg["start_id"], "diverse_lambda": 0.0,
            "sampling_method": cfg.get("sampling_method", "beam_search"),
            "topp": cfg.get("topp", 0.75), "topk": cfg.get("topk", 1),
            "trg_end_id": cfg["end_id"], "is_post_ln": cfg["is_post_ln"],
            "no_scale_embedding": False, "use_gelu": cfg["use_gelu"], "multilg_type": 0}
    return {"src_embedding": src_emb, "encoder_stack": enc_layers, "trg_embedding": trg_emb,
            "decoder_stack": dec_layers, "model_conf": conf}


def write_quant_transformer(path, cfg, seed=0, ln_noise=0.02, eos_bias=None, w_std=None):
    """Write a synthetic QuantTransformer model file; returns the message dict."""
    msg = make_quant_transformer(cfg, seed=seed, ln_noise=ln_noise, eos_bias=eos_bias,
                                 w_std=w_std)
    with open(path, "wb") as f:
        f.write(proto.encode("QuantTransformer", msg))
    return msg


# --------------------------------------------------------------------------- #
# QuantGpt (decoder-only, greedy / perplexity)
# --------------------------------------------------------------------------- #
def gpt_config(name):
    """Shapes of the named synthetic decoder-only configurations."""
    cfgs = {
        # GPT-2-medium-shaped: 24 layers, hidden 1024, 16 heads, GELU, pre-LN, vocab 50257
        "gpt2_medium": dict(n_layer=24, hidden=1024, inner=4096, head_num=16, max_step=640,
                            vocab=50257, padding_id=50256, eos_id=50256, topk=1,
                            extra_decode_length=128, sampling_method="topk"),
        "tiny": dict(n_layer=2, hidden=128, inner=256, head_num=4, max_step=48, vocab=300,
                     padding_id=0, eos_id=299, topk=1, extra_decode_length=16,
                     sampling_method="topk"),
    }
    return dict(cfgs[name])


def make_quant_gpt(cfg, seed=0, ln_noise=0.02, w_std=None):
    """Build the QuantGpt message (a dict for :func:`proto.encode`).  The token embedding is
    stored [hidden, vocab] as the reference's exporter writes it."""
    rng = np.random.default_rng(seed)
    H, I, L = cfg["hidden"], cfg["inner"], cfg["n_layer"]
    w_std = float(cfg.get("w_std", W_STD) if w_std is None else w_std)
    clip_e, clip_w = 4 * W_STD, 4 * w_std

    def normal(*shape, std=W_STD):
        return rng.standard_normal(shape, dtype=np.float32) * np.float32(std)

    def ln_params():
        return ((1 + normal(H, std=ln_noise)).astype(np.float32), normal(H, std=ln_noise))

    def qk(rows, cols):
        return quantize_u8(normal(rows, cols, std=w_std), clip_w).reshape(-1)

    proj = float(4 * w_std * np.sqrt(H))
    g, b = ln_params()
    logit_sigma = W_STD * np.sqrt(H)
    emb = {
        "token_embedding": quantize_u8(normal(H, cfg["vocab"]), clip_e).reshape(-1),
        "position_embedding": normal(cfg["max_step"], H, std=0.1).reshape(-1),
        "norm_scale": g, "norm_bias": b, "emb_clip_max": clip_e,
        "output_ln_clip_max": 4.0, "logits_clip_max": float(4 * logit_sigma),
    }
    layers = []
    for _ in range(L):
        g1, b1 = ln_params()
        g2, b2 = ln_params()
        layers.append({
            "multihead_norm_scale": g1, "multihead_norm_bias": b1,
            "multihead_project_kernel_qkv": qk(H, 3 * H), "multihead_project_bias_qkv": normal(3 * H),
            "multihead_project_kernel_output": qk(H, H), "multihead_project_bias_output": normal(H),
            "ffn_norm_scale": g2, "ffn_norm_bias": b2,
            "ffn_first_kernel": qk(H, I), "ffn_first_bias": normal(I),
            "ffn_second_kernel": qk(I, H), "ffn_second_bias": normal(H),
            "multihead_project_kernel_qkv_clip_max": clip_w,
            "multihead_project_kernel_output_clip_max": clip_w,
            "ffn_first_kernel_clip_max": clip_w, "ffn_second_kernel_clip_max": clip_w,
            "multihead_ln_clip_max": 4.0, "multihead_project_output_clip_max": proj / 2,
            "ffn_ln_clip_max": 4.0, "ffn_first_act_clip_max": proj,
            "multihead_qkv_dense_clip_max": proj,
            "multihead_output_dense_clip_max": proj * proj / 8,
            "ffn_first_output_clip_max": proj, "self_qkv_bias_out_clip_max": proj,
        })
    conf = {"head_num": cfg["head_num"], "src_padding_id": cfg["padding_id"],
            "sampling_method": cfg.get("sampling_method", "topk"), "topp": cfg.get("topp", 0.75),
            "topk": cfg.get("topk", 1), "eos_id": cfg["eos_id"],
            "extra_decode_length": cfg["extra_decode_length"]}
    return {"src_embedding": emb, "encoder_stack": layers, "model_conf": conf}


def write_quant_gpt(path, cfg, seed=0, ln_noise=0.02, w_std=None):
    """Write a synthetic QuantGpt model file; returns the message dict."""
    msg = make_quant_gpt(cfg, seed=seed, ln_noise=ln_noise, w_std=w_std)
    with open(path, "wb") as f:
        f.write(proto.encode("QuantGpt", msg))
    return msg
