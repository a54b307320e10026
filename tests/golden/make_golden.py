#!/usr/bin/env python3
"""Writes the golden fixtures of the int8 layer path (``fixtures.npz``).

The reference stores no golden vectors for this path (its tests draw random inputs
and compare against PyTorch on the GPU), so these are produced by this repository's
pinned CPU oracle on small seeded inputs: for every kernel of the encoder path the
inputs, the scalar arguments and the expected outputs.  Run from the repository root:

    python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

from oracle import oracle  # noqa: E402
from oracle.model_io import oracle_weights_from_message  # noqa: E402
from lightseq_amd import synthetic  # noqa: E402

OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "fixtures.npz")


def main():
    rng = np.random.default_rng(20240)
    F16 = np.float16
    fx = {}
    tokens, H, I = 6, 64, 128
    g = (1 + 0.1 * rng.standard_normal(H)).astype(F16)
    b = (0.1 * rng.standard_normal(H)).astype(F16)
    rb = (0.1 * rng.standard_normal(H)).astype(F16)
    cs = (0.2 * rng.standard_normal(H)).astype(F16)
    x = (1.5 * rng.standard_normal((tokens, H))).astype(F16)
    fx.update(ln_g=g, ln_b=b, ln_rb=rb, ln_cs=cs, ln_x=x)
    fx["quant_out"] = oracle.quantize_tensor(x, 127 / 4.0)
    for post in (0, 1):
        q, res = oracle.norm_layer_resual_i8O(x, g, b, rb, 127 / 4.0, post)
        fx["ln_first_q_%d" % post], fx["ln_first_res_%d" % post] = q, res
    acc8 = rng.integers(-127, 128, size=(tokens, H), dtype=np.int8)
    acc32 = rng.integers(-200000, 200000, size=(tokens, H), dtype=np.int32)
    fx.update(ln_acc8=acc8, ln_acc32=acc32)
    for post in (0, 1):
        q, res = oracle.residual_bias_ln_i8O(acc8, g, b, rb, x, 2.0 / 127, 127 / 4.0, post)
        fx["ln_i8_q_%d" % post], fx["ln_i8_res_%d" % post] = q, res
        q, res = oracle.residual_bias_ln_i8O(acc32, g, b, rb, x, 1e-5, 127 / 4.0, post, cs)
        fx["ln_i32_q_%d" % post], fx["ln_i32_res_%d" % post] = q, res
    fx["ln_i32_out"] = oracle.residual_bias_ln_i32I(acc32, g, b, x, 1e-5, cs)
    fx["deq_out"] = oracle.dequantize_tensor(acc32, 1e-5, F16)

    a = rng.integers(-127, 128, size=(tokens, I), dtype=np.int8)
    ab = (0.3 * rng.standard_normal(I)).astype(F16)
    fx.update(act_in=a, act_bias=ab)
    fx["gelu_out"] = oracle.bias_gelu_i8I_i8O(a, ab, 2.2 / 127, 127 / 2.2)
    fx["relu_out"] = oracle.bias_relu_i8I_i8O(a, ab, 2.2 / 127, 127 / 1.65, 1.65, False)
    fx["relu_narrow_out"] = oracle.bias_relu_i8I_i8O(a, ab, 2.2 / 127, 127 / 1.65, 1.65, True)

    B, S, h, d = 2, 5, 2, 32
    qkv = rng.integers(-127, 128, size=(B * S, 3 * h * d), dtype=np.int8)
    qb = (0.3 * rng.standard_normal(3 * h * d)).astype(F16)
    mask = np.array([[0, 0, 0, 0, 0], [0, 0, 0, 1, 1]], np.int32)
    fx.update(att_qkv=qkv, att_bias=qb, att_mask=mask)
    arranged = oracle.arrange_encself_qkv_i8I(qkv, qb, B, S, h, 2.2 / 127)
    fx["att_arranged"] = arranged
    probs = oracle.correlation_softmax_encself(oracle.attn_scores(arranged[0], arranged[1], np.sqrt(1 / d)), mask)
    fx["att_probs"] = probs
    ctx = oracle.attn_context(probs, arranged[2])
    fx["att_ctx"] = ctx
    fx["att_ctx_q"] = oracle.arrange_atten_output_i8O(ctx, 127 / 0.5)

    M, N, K = 37, 21, 96
    ga = rng.integers(-127, 128, size=(M, K), dtype=np.int8)
    gw = rng.integers(-127, 128, size=(N, K), dtype=np.int8)
    fx.update(gemm_a=ga, gemm_w=gw)
    fx["gemm_i32"] = oracle.gemm_i8_i32(ga, gw)
    fx["gemm_i8"] = oracle.gemm_i8_i8(ga, gw, 4.0 * 0.08 / (2.2 * 127))

    for name, over in (("gelu_post", {}), ("relu_pre", {"use_gelu": False, "is_post_ln": False})):
        cfg = synthetic.bert_config("tiny")
        cfg.update(over)
        msg = synthetic.make_quant_bert(cfg, seed=11)
        ids, _ = synthetic.make_token_ids(cfg, 2, 12, seed=11)
        out, pm, _ = oracle.quant_bert_encoder(oracle_weights_from_message(msg, cfg), ids)
        fx["stack_%s_ids" % name] = ids
        fx["stack_%s_out" % name] = out
    np.savez_compressed(OUT, **fx)
    print("wrote %s: %d arrays, %d bytes" % (OUT, len(fx), os.path.getsize(OUT)))


if __name__ == "__main__":
    main()
