"""GPU parity of the whole int8 encoder stack (QuantBert) against the CPU oracle,
through the model C ABI, on synthetic model files in the reference's format.

Bars: int32 FFN2 accumulators bit-exact wherever their int8 inputs agree, int8
activations within +-1 code on <= 0.1 % of elements, fp16 layer outputs within
2e-2 absolute at valid (non-padded) positions.
"""
import numpy as np
import pytest
import torch

from conftest import assert_codes_close
from helpers import DEV, oracle_weights_from_message

pytestmark = pytest.mark.gpu


def _build(tmp_path, cfg_name, seed, **over):
    from lightseq_amd import synthetic
    cfg = synthetic.bert_config(cfg_name)
    cfg.update(over)
    path = str(tmp_path / ("%s_%d.pb" % (cfg_name, seed)))
    msg = synthetic.write_quant_bert(path, cfg, seed=seed)
    return cfg, msg, path


def _valid(ids, cfg):
    return ids != cfg["padding_id"]


@pytest.mark.parametrize("cfg_name,batch,seq,over", [
    ("tiny", 3, 20, {}),
    ("tiny", 2, 33, {"use_gelu": False}),
    ("tiny", 2, 16, {"is_post_ln": False}),
    ("tiny", 1, 64, {"is_post_ln": False, "use_gelu": False}),
    ("tiny", 2, 24, {"hidden": 256, "inner": 512, "head_num": 2}),   # 128-wide heads
    # heads of 64 at hidden 256: the layers run the QKV + attention kernel (<= 128 tokens) ...
    ("tiny", 3, 33, {"hidden": 256, "inner": 512, "head_num": 4}),
    # ... and the GEMM followed by the multi-block attention kernel beyond 128 tokens
    ("tiny", 2, 160, {"hidden": 256, "inner": 512, "head_num": 4, "max_step": 192}),
])
def test_tiny_stack_with_taps(tmp_path, oracle, cfg_name, batch, seq, over):
    from lightseq_amd import inference, synthetic
    cfg, msg, path = _build(tmp_path, cfg_name, 3, **over)
    ids, _ = synthetic.make_token_ids(cfg, batch, seq, seed=5)
    w = oracle_weights_from_message(msg, cfg)
    M, H, I = batch * seq, cfg["hidden"], cfg["inner"]
    model = inference.QuantBert(path, batch)
    for layer in range(cfg["n_layer"]):
        want, want_mask, taps = oracle.quant_bert_encoder(w, ids, tap_layer=layer)
        bufs = {}
        for name, shape, dt in [("ln1_q", (M, H), torch.int8), ("qkv_q", (M, 3 * H), torch.int8),
                                ("ctx_q", (M, H), torch.int8), ("out_q", (M, H), torch.int8),
                                ("ln2_q", (M, H), torch.int8), ("ffn1_q", (M, I), torch.int8),
                                ("act_q", (M, I), torch.int8), ("ffn2_acc", (M, H), torch.int32)]:
            bufs[name] = torch.zeros(shape, dtype=dt, device=DEV)
            model.set_tap(layer, name, bufs[name])
        got = model.infer_fp16(ids)
        valid = _valid(ids, cfg).reshape(-1)
        for name in ("ln1_q", "qkv_q", "ctx_q", "out_q", "ln2_q", "ffn1_q", "act_q"):
            g = bufs[name].cpu().numpy()
            # padded query rows of the attention context are don't-care downstream.  Both runs
            # are free-running here: the first layer sees identical inputs and meets the per-kernel
            # bar; one flipped code there perturbs a whole accumulator row of the next GEMM, so
            # deeper stages are held to "never more than one code" with a drift allowance (the
            # stage-by-stage check on identical inputs is test_bert_base_two_layers_full_width)
            assert_codes_close(g[valid], taps[name][valid], max_frac=3e-3 if layer == 0 else 0.1,
                               what="%s layer %d" % (name, layer))
        # int32 accumulators: exact given the kernel's own int8 inputs
        act = bufs["act_q"].cpu().numpy()
        w2 = w["w_ffn2"][layer]
        exact = np.rint(act.astype(np.float64) @ w2.astype(np.float64).T).astype(np.int64)
        np.testing.assert_array_equal(bufs["ffn2_acc"].cpu().numpy().astype(np.int64), exact)
        for name in bufs:
            model.set_tap(layer, name, None)
    v = _valid(ids, cfg)
    np.testing.assert_allclose(got.astype(np.float32)[v], want.astype(np.float32)[v], atol=2e-2, rtol=0)
    model.close()


def test_transformer_base_layer_config(tmp_path, oracle):
    """One Transformer-base-shaped int8 encoder layer: batch 8, seq 64, hidden 512,
    8 heads, FFN 2048 ReLU, post-LN, all-ones mask, seed 0."""
    from lightseq_amd import inference, synthetic
    cfg, msg, path = _build(tmp_path, "transformer_base_layer", 0)
    ids, _ = synthetic.make_token_ids(cfg, 8, 64, seed=0, min_len=64)  # no padding
    w = oracle_weights_from_message(msg, cfg)
    want, _, _ = oracle.quant_bert_encoder(w, ids)
    model = inference.QuantBert(path, 8)
    got = model.infer(ids)
    assert got.dtype == np.float32 and got.shape == (8, 64, 512)
    np.testing.assert_allclose(got, want.astype(np.float32), atol=2e-2, rtol=0)
    model.close()


def test_transformer_base_layer_vs_quantisation_aware_layer(tmp_path, oracle):
    """The same single layer against the float quantisation-aware layer the int8 engine is
    exported from (training/ops/pytorch/torch_transformer_layers.py:537-679), restated in
    oracle/qat.py.  In a post-LN model file the layer norms are rotated by one position
    (examples/inference/python/export/huggingface/ls_torch_hf_quant_bert_export.py:159-177):
    "multihead_norm" of layer 0 is the embedding layer norm, "ffn_norm" follows the attention
    block and the norm stored with the embedding closes the layer.  The engine does not
    quantise the fc2 output, so that quantiser of the module is off."""
    from lightseq_amd import inference, synthetic
    from oracle import qat
    cfg, msg, path = _build(tmp_path, "transformer_base_layer", 0)
    ids, _ = synthetic.make_token_ids(cfg, 8, 64, seed=0, min_len=64)
    H, I = cfg["hidden"], cfg["inner"]
    emb, l = msg["src_embedding"], msg["encoder_stack"][0]

    def weight(name, rows, cols):
        clip = np.float32(l[name + "_clip_max"])
        codes = np.asarray(l[name], np.int32).reshape(rows, cols) - 127
        return np.ascontiguousarray((codes.astype(np.float32) * (clip / np.float32(127))).T)

    f = lambda v: np.asarray(v, np.float32)
    p = {"qkv_w": weight("multihead_project_kernel_qkv", H, 3 * H),
         "qkv_b": f(l["multihead_project_bias_qkv"]),
         "out_w": weight("multihead_project_kernel_output", H, H),
         "out_b": f(l["multihead_project_bias_output"]),
         "ln1_w": f(l["ffn_norm_scale"]), "ln1_b": f(l["ffn_norm_bias"]),
         "fc1_w": weight("ffn_first_kernel", H, I), "fc1_b": f(l["ffn_first_bias"]),
         "fc2_w": weight("ffn_second_kernel", I, H), "fc2_b": f(l["ffn_second_bias"]),
         "ln2_w": f(emb["norm_scale"]), "ln2_b": f(emb["norm_bias"])}
    amax = {"qkv_in": l["multihead_ln_clip_max"], "qkv_w": l["multihead_project_kernel_qkv_clip_max"],
            "qkv_out": l["multihead_qkv_dense_clip_max"],
            "out_in": l["multihead_project_output_clip_max"],
            "out_w": l["multihead_project_kernel_output_clip_max"],
            "out_out": l["multihead_output_dense_clip_max"], "fc1_in": l["ffn_ln_clip_max"],
            "fc1_w": l["ffn_first_kernel_clip_max"], "fc1_out": l["ffn_first_output_clip_max"],
            "fc2_in": l["ffn_first_act_clip_max"], "fc2_w": l["ffn_second_kernel_clip_max"],
            "fc2_out": 0.0}
    tok = (np.asarray(emb["token_embedding"], np.float32).reshape(cfg["vocab"], H) - 127) * (
        np.float32(emb["emb_clip_max"]) / 127)
    x0 = tok[ids] + f(emb["position_embedding"]).reshape(cfg["max_step"], H)[None, :64]
    x = qat.layer_norm(x0, f(l["multihead_norm_scale"]), f(l["multihead_norm_bias"]), eps=1e-12)
    want = qat.encoder_layer(x, p, amax, cfg["head_num"], False, "relu", None,
                             fc2_output_quant=False)
    model = inference.QuantBert(path, 8)
    got = model.infer(ids)
    model.close()
    d = np.abs(got.astype(np.float64) - want)
    assert d.max() < 2e-2, (d.max(), d.mean())


TAP_SPECS = [("ln1_q", "H", "i8"), ("qkv_q", "3H", "i8"), ("ctx_q", "H", "i8"), ("out_q", "H", "i8"),
             ("ln2_q", "H", "i8"), ("ffn1_q", "I", "i8"), ("act_q", "I", "i8"), ("ffn2_acc", "H", "i32"),
             ("res_attn", "H", "f16"), ("res_ffn", "H", "f16")]


# taps that leave the layer on its fused kernels (the others make it take the unfused route)
PASSIVE_TAPS = ("ln1_q", "ctx_q", "ln2_q", "act_q")


def _run_with_taps(model, ids, layer, M, H, I, only=None):
    width = {"H": H, "3H": 3 * H, "I": I}
    dts = {"i8": torch.int8, "i32": torch.int32, "f16": torch.float16}
    bufs = {}
    for name, wd, dt in TAP_SPECS:
        if only is not None and name not in only:
            continue
        bufs[name] = torch.zeros((M, width[wd]), dtype=dts[dt], device=DEV)
        model.set_tap(layer, name, bufs[name])
    out = model.infer_fp16(ids)
    taps = {k: v.cpu().numpy() for k, v in bufs.items()}
    for name in bufs:
        model.set_tap(layer, name, None)
    return out, taps


def _check_encoder_layer_stages(oracle, w, cfg, t, layer, B, S, mask, valid):
    """Every stage of encoder layer `layer` against the oracle's kernel for that stage, each fed
    the GPU's own stage input (the taps `t`): GEMM codes and the FFN2 accumulator bit for bit,
    attention / layer-norm / activation codes to the +-1 code / 0.1 % bar.  Returns the oracle's
    int8 input of the next layer (or None for the last layer)."""
    H, I, h = cfg["hidden"], cfg["inner"], cfg["head_num"]
    Q = np.float32(127)
    c = w["clip_max"][layer * 11:(layer + 1) * 11]
    np.testing.assert_array_equal(
        t["qkv_q"], oracle.gemm_i8_i8(t["ln1_q"], w["w_qkv"][layer], c[0] * c[4] / (c[8] * Q)))
    np.testing.assert_array_equal(
        t["out_q"], oracle.gemm_i8_i8(t["ctx_q"], w["w_out"][layer], c[1] * c[5] / (c[9] * Q)))
    np.testing.assert_array_equal(
        t["ffn1_q"], oracle.gemm_i8_i8(t["ln2_q"], w["w_ffn1"][layer], c[2] * c[6] / (c[10] * Q)))
    np.testing.assert_array_equal(t["ffn2_acc"], oracle.gemm_i8_i32(t["act_q"], w["w_ffn2"][layer]))
    qkv = oracle.arrange_encself_qkv_i8I(t["qkv_q"], w["b_qkv"][layer], B, S, h, c[8] / Q)
    probs = oracle.correlation_softmax_encself(
        oracle.attn_scores(qkv[0], qkv[1], np.sqrt(1.0 / (H // h))), mask)
    ctx_q = oracle.arrange_atten_output_i8O(oracle.attn_context(probs, qkv[2]), Q / c[5])
    assert_codes_close(t["ctx_q"][valid], ctx_q[valid], what="ctx_q layer %d" % layer)
    ln2_q, _ = oracle.residual_bias_ln_i8O(t["out_q"], w["ln2_scale"][layer], w["ln2_bias"][layer],
                                           w["b_ffn2"][layer], t["res_attn"], c[9] / Q, Q / c[6],
                                           cfg["is_post_ln"])
    assert_codes_close(t["ln2_q"], ln2_q, what="ln2_q layer %d" % layer)
    if cfg["use_gelu"]:
        act_q = oracle.bias_gelu_i8I_i8O(t["ffn1_q"], w["b_ffn1"][layer], c[10] / Q, Q / c[7])
    else:
        act_q = oracle.bias_relu_i8I_i8O(t["ffn1_q"], w["b_ffn1"][layer], c[10] / Q, Q / c[7], c[7], True)
    assert_codes_close(t["act_q"], act_q, what="act_q layer %d" % layer)
    if layer == w["n_layer"] - 1:
        return None
    cn = w["clip_max"][(layer + 1) * 11:(layer + 2) * 11]
    dq = c[3] * c[7] / (Q * Q)
    ln1_next, _ = oracle.residual_bias_ln_i8O(t["ffn2_acc"], w["ln1_scale"][layer + 1],
                                              w["ln1_bias"][layer + 1], w["b_out"][layer + 1],
                                              t["res_ffn"], dq, Q / cn[4], cfg["is_post_ln"])
    return ln1_next


def test_bert_base_every_layer_stage_by_stage(tmp_path, oracle):
    """The benchmark stack itself (12 layers, hidden 768, 12 heads, FFN 3072 GELU, batch 32 x
    seq 128, ragged lengths): every stage of every layer against the oracle's kernel for it,
    fed the GPU's own stage input; and the fused kernels a layer normally runs (QKV + attention,
    out-projection + layer norm, FFN1 + table) leave the same bytes in place as the unfused
    kernels that the taps switch the layer to."""
    from lightseq_amd import inference, synthetic
    cfg, msg, path = _build(tmp_path, "bert_base", 4, vocab=2000, max_step=128)
    B, S, H, I = 32, 128, cfg["hidden"], cfg["inner"]
    M = B * S
    ids, lens = synthetic.make_token_ids(cfg, B, S, seed=4, min_len=32)
    w = oracle_weights_from_message(msg, cfg)
    assert w["n_layer"] == 12
    mask = (ids == cfg["padding_id"]).astype(np.int32)
    valid = _valid(ids, cfg).reshape(-1)
    model = inference.QuantBert(path, B)
    ln1_next = None
    for layer in range(12):
        _, t = _run_with_taps(model, ids, layer, M, H, I)
        if ln1_next is not None:
            assert_codes_close(t["ln1_q"], ln1_next, what="ln1_q layer %d" % layer)
        ln1_next = _check_encoder_layer_stages(oracle, w, cfg, t, layer, B, S, mask, valid)
        # the same layer on its fused kernels
        _, f = _run_with_taps(model, ids, layer, M, H, I, only=PASSIVE_TAPS)
        for name in PASSIVE_TAPS:
            if name == "ctx_q":   # padded queries: zeros on both routes, but compare what matters
                np.testing.assert_array_equal(f[name][valid], t[name][valid])
            else:
                np.testing.assert_array_equal(f[name], t[name])
    model.close()


def test_bert_base_two_layers_full_width(tmp_path, oracle):
    """BERT-base width (hidden 768, 12 heads, FFN 3072 GELU), batch 32 x seq 128 with
    ragged valid lengths, cut to 2 layers so the oracle finishes in seconds.

    A +-1 code difference in one int8 activation perturbs every accumulator of its row
    in the next GEMM and flips further codes there, so two correct implementations
    drift apart layer by layer.  Parity is therefore checked per stage, each stage of
    the oracle being fed the GPU's own input of that stage; the end-to-end output is
    checked statistically."""
    from lightseq_amd import inference, synthetic
    cfg, msg, path = _build(tmp_path, "bert_base", 1, n_layer=2, vocab=2000, max_step=128)
    B, S, H, I, h = 32, 128, cfg["hidden"], cfg["inner"], cfg["head_num"]
    M, Q = B * S, np.float32(127)
    ids, lens = synthetic.make_token_ids(cfg, B, S, seed=2, min_len=32)
    w = oracle_weights_from_message(msg, cfg)
    want, want_mask, _ = oracle.quant_bert_encoder(w, ids)
    model = inference.QuantBert(path, B)
    valid = _valid(ids, cfg).reshape(-1)
    for layer in range(2):
        got, t = _run_with_taps(model, ids, layer, M, H, I)
        c = w["clip_max"][layer * 11:(layer + 1) * 11]
        # int8 GEMMs with requantising epilogue: bit exact given the same int8 input
        np.testing.assert_array_equal(
            t["qkv_q"], oracle.gemm_i8_i8(t["ln1_q"], w["w_qkv"][layer], c[0] * c[4] / (c[8] * Q)))
        np.testing.assert_array_equal(
            t["out_q"], oracle.gemm_i8_i8(t["ctx_q"], w["w_out"][layer], c[1] * c[5] / (c[9] * Q)))
        np.testing.assert_array_equal(
            t["ffn1_q"], oracle.gemm_i8_i8(t["ln2_q"], w["w_ffn1"][layer], c[2] * c[6] / (c[10] * Q)))
        # FFN2: int32 accumulators bit exact
        np.testing.assert_array_equal(t["ffn2_acc"], oracle.gemm_i8_i32(t["act_q"], w["w_ffn2"][layer]))
        # attention block from the GPU's own qkv codes
        qkv = oracle.arrange_encself_qkv_i8I(t["qkv_q"], w["b_qkv"][layer], B, S, h, c[8] / Q)
        probs = oracle.correlation_softmax_encself(
            oracle.attn_scores(qkv[0], qkv[1], np.sqrt(1.0 / (H // h))), want_mask)
        ctx_q = oracle.arrange_atten_output_i8O(oracle.attn_context(probs, qkv[2]), Q / c[5])
        assert_codes_close(t["ctx_q"][valid], ctx_q[valid], what="ctx_q layer %d" % layer)
        # LayerNorm after attention, from the GPU's own GEMM output and residual stream
        ln2_q, _ = oracle.residual_bias_ln_i8O(t["out_q"], w["ln2_scale"][layer], w["ln2_bias"][layer],
                                               w["b_ffn2"][layer], t["res_attn"], c[9] / Q, Q / c[6],
                                               cfg["is_post_ln"])
        assert_codes_close(t["ln2_q"], ln2_q, what="ln2_q layer %d" % layer)
        act_q = oracle.bias_gelu_i8I_i8O(t["ffn1_q"], w["b_ffn1"][layer], c[10] / Q, Q / c[7])
        assert_codes_close(t["act_q"], act_q, what="act_q layer %d" % layer)
        dq = c[3] * c[7] / (Q * Q)
        if layer == 0:
            cn = w["clip_max"][11:22]
            ln1_next, _ = oracle.residual_bias_ln_i8O(t["ffn2_acc"], w["ln1_scale"][1], w["ln1_bias"][1],
                                                      w["b_out"][1], t["res_ffn"], dq, Q / cn[4],
                                                      cfg["is_post_ln"])
            _, t_next = _run_with_taps(model, ids, 1, M, H, I)
            assert_codes_close(t_next["ln1_q"], ln1_next, what="ln1_q layer 1")
        else:
            final = oracle.residual_bias_ln_i32I(t["ffn2_acc"], w["final_ln_scale"], w["final_ln_bias"],
                                                 t["res_ffn"], dq)
            np.testing.assert_allclose(got.reshape(M, H).astype(np.float32), final.astype(np.float32),
                                       atol=8e-3, rtol=0)
    # end to end against the oracle's own run: drift from code flips stays small
    v = _valid(ids, cfg)
    diff = np.abs(got.astype(np.float32)[v] - want.astype(np.float32)[v])
    assert diff.mean() <= 5e-3, diff.mean()
    assert np.quantile(diff, 0.999) <= 3e-2, np.quantile(diff, 0.999)
    assert diff.max() <= 0.1, diff.max()
    model.close()


def test_bert_base_free_running_drift_against_the_oracle(tmp_path, oracle):
    """The benchmark stack whole (12 layers, b32 x s128, ragged lengths), GPU and oracle each
    running free: how far the fp16 outputs sit apart on the valid positions.  Every stage is
    held to its bar on equal inputs by the stage-by-stage test; a code that rounds the other way
    at one stage changes the inputs of all later ones, so the end-to-end distance is a
    statistic -- stated here as mean, 99.9th percentile and maximum, and asserted."""
    from lightseq_amd import inference, synthetic
    cfg, msg, path = _build(tmp_path, "bert_base", 4, vocab=2000, max_step=128)
    ids, lens = synthetic.make_token_ids(cfg, 32, 128, seed=4, min_len=32)
    want, _, _ = oracle.quant_bert_encoder(oracle_weights_from_message(msg, cfg), ids)
    model = inference.QuantBert(path, 32)
    got = model.infer_fp16(ids)
    model.close()
    v = _valid(ids, cfg)
    diff = np.abs(got.astype(np.float32)[v] - want.astype(np.float32)[v])
    scale = np.abs(want.astype(np.float32)[v]).mean()
    print("12-layer drift: mean %.3e, 99.9th percentile %.3e, max %.3e (mean |output| %.3f)" %
          (diff.mean(), np.quantile(diff, 0.999), diff.max(), scale))
    # observed: 2.0e-2, 8.4e-2, 0.125 at a mean |output| of 0.80
    assert diff.mean() <= 3e-2 and np.quantile(diff, 0.999) <= 0.12 and diff.max() <= 0.2


@pytest.mark.parametrize("preset,kw,B,S", [("bert_base", dict(n_layer=3, vocab=2000, max_step=128), 32, 128),
                                            ("bert_base", dict(n_layer=2, vocab=2000, max_step=128), 5, 77),
                                            ("tiny", dict(), 4, 24)])
def test_feed_forward_segment_route_leaves_the_same_bytes(tmp_path, preset, kw, B, S):
    """The layers run with their feed-forward half as one launch (XCD-local barriers) give the
    output of the three launches, byte for byte; the route is taken where the shape is covered
    and two runs in a row work (the barrier counters go on)."""
    from lightseq_amd import inference, kernels, synthetic
    cfg, msg, path = _build(tmp_path, preset, 6, **kw)
    ids, lens = synthetic.make_token_ids(cfg, B, S, seed=6, min_len=max(1, S // 4))
    model = inference.QuantBert(path, B)
    want = model.infer_fp16(ids)
    prev = kernels.ffn_segment_in_models(True)
    try:
        model.set_profiling(True)
        got = [model.infer_fp16(ids) for _ in range(3)]
        prof = model.get_profile()
        model.set_profiling(False)
    finally:
        kernels.ffn_segment_in_models(prev)
    for g in got:
        np.testing.assert_array_equal(g, want)
    names = {p["site"]: p["kernel"] for p in prof if p["launches"]}
    if kernels.ffn_segment_supported(B * S, cfg["hidden"], cfg["inner"]):
        assert names.get("ffn1") == "ffn_segment_kernel" and "ffn2" not in names, names
    np.testing.assert_array_equal(model.infer_fp16(ids), want)   # and back on the three launches
    model.close()


def test_bert_base_full_stack_properties(tmp_path):
    """The benchmark workload itself (12 layers, b32 x s128): size-independent
    properties.  A sequence's output does not depend on what else is in the batch
    (every kernel is row- or sequence-independent), runs are deterministic, and the
    final LayerNorm leaves every valid row with the statistics of its scale/bias."""
    from lightseq_amd import inference, synthetic
    cfg, msg, path = _build(tmp_path, "bert_base", 0, vocab=3000)
    ids, lens = synthetic.make_token_ids(cfg, 32, 128, seed=0, min_len=32)
    model = inference.QuantBert(path, 32)
    out = model.infer_fp16(ids)
    assert np.isfinite(out.astype(np.float32)).all()
    np.testing.assert_array_equal(out, model.infer_fp16(ids))
    for b in (0, 7, 31):
        alone = model.infer_fp16(ids[b:b + 1])
        np.testing.assert_array_equal(alone[0], out[b])
    perm = np.random.default_rng(0).permutation(32)
    np.testing.assert_array_equal(model.infer_fp16(ids[perm]), out[perm])
    g = np.asarray(msg["src_embedding"]["norm_scale"], np.float32)
    beta = np.asarray(msg["src_embedding"]["norm_bias"], np.float32)
    z = (out.astype(np.float32) - beta) / g
    v = ids != cfg["padding_id"]
    np.testing.assert_allclose(z[v].mean(-1), 0.0, atol=2e-2)
    np.testing.assert_allclose(z[v].std(-1), 1.0, atol=2e-2)
    model.close()


def test_reference_module_name_runs_unchanged(tmp_path):
    """A script written against the reference's module runs as it is."""
    import lightseq.inference as lsi
    from lightseq_amd import synthetic
    cfg, _msg, path = _build(tmp_path, "tiny", 2)
    ids, _ = synthetic.make_token_ids(cfg, 3, 12, seed=1)
    model = lsi.QuantBert(path, 4)
    out = model.infer(ids)
    assert out.shape == (3, 12, cfg["hidden"]) and out.dtype == np.float32
    assert np.isfinite(out).all() and np.abs(out).max() > 0


def test_token_ids_outside_the_table_are_clamped(tmp_path):
    """An id below 0 or beyond the vocabulary must not become a read outside the embedding
    table: the model clamps it (the decoder and GPT embeddings do the same)."""
    from lightseq_amd import inference, synthetic
    cfg, _msg, path = _build(tmp_path, "tiny", 4)
    ids, _ = synthetic.make_token_ids(cfg, 2, 16, seed=6)
    bad = ids.copy()
    pos = [(0, 1), (0, 3), (1, 0), (1, 2)]
    for (b, t), v in zip(pos, (cfg["vocab"], cfg["vocab"] + 12345, 2 ** 31 - 1, cfg["vocab"] + 1)):
        assert ids[b, t] != cfg["padding_id"]
        bad[b, t] = v
    clamped = np.minimum(bad, cfg["vocab"] - 1)
    model = inference.QuantBert(path, 2)
    got = model.infer_fp16(bad)
    want = model.infer_fp16(clamped)
    np.testing.assert_array_equal(got.view(np.uint16), want.view(np.uint16))
    # negative ids read row 0 of the table (they are not the padding id, so they stay unmasked)
    neg = ids.copy()
    neg[0, 1], neg[1, 2] = -7, -(2 ** 31)
    out = model.infer_fp16(neg)
    assert np.isfinite(out.astype(np.float32)).all()
    model.close()


def test_model_interface_and_errors(tmp_path):
    from lightseq_amd import inference, synthetic
    from lightseq_amd.lib import LSHError
    cfg, msg, path = _build(tmp_path, "tiny", 0)
    model = inference.QuantBert(path, 4)
    assert model.get_input_size() == 1 and model.get_output_size() == 1
    assert model.get_input_name(0) == "token_ids" and model.get_output_name(0) == "encoder_output"
    assert model.get_input_max_shape(0) == [4, cfg["max_step"]]
    assert model.get_output_max_shape(0) == [4, cfg["max_step"], cfg["hidden"]]
    assert model.get_input_dtype(0) == 2 and model.get_output_dtype(0) == 4
    ids, _ = synthetic.make_token_ids(cfg, 2, 10)
    out = model.infer(ids)
    assert out.shape == (2, 10, cfg["hidden"]) and np.isfinite(out).all()
    assert model.get_output_shape(0) == [2, 10, cfg["hidden"]]
    # same input twice -> identical output (no state leaks between calls)
    np.testing.assert_array_equal(out, model.infer(ids))
    with pytest.raises(LSHError, match="batch size of input greater than max_batch_size"):
        model.infer(np.ones((5, 4), np.int32))
    big = np.ones((1, cfg["max_step"] + 1), np.int32)
    with pytest.raises(LSHError, match="seq len of input greater than max_step"):
        model.infer(big)
    model.close()
    with pytest.raises(LSHError, match="not found"):
        inference.QuantBert(str(tmp_path / "missing.pb"), 1)
    with pytest.raises(LSHError, match="Model not supported"):
        inference.LSModel("NoSuchModel", path, 1)
    bad = tmp_path / "bad.pb"
    bad.write_bytes(b"\x0a\x03abc")
    with pytest.raises(LSHError):
        inference.QuantBert(str(bad), 1)
