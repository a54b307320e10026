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
