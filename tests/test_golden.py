"""Golden fixtures (tests/golden/fixtures.npz, written by tests/golden/make_golden.py):
the oracle must keep reproducing them bit for bit on the CPU, and the HIP path must
match them on the GPU to the parity bar."""
import os

import numpy as np
import pytest
import torch

from conftest import assert_codes_close

FX = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "fixtures.npz"))
DEV = "cuda:0"


def _stack_cfg(name):
    from lightseq_amd import synthetic
    cfg = synthetic.bert_config("tiny")
    if name == "relu_pre":
        cfg.update(use_gelu=False, is_post_ln=False)
    return cfg


def test_oracle_reproduces_fixtures(oracle):
    f = FX
    g, b, rb, cs, x = f["ln_g"], f["ln_b"], f["ln_rb"], f["ln_cs"], f["ln_x"]
    eq = np.testing.assert_array_equal
    eq(oracle.quantize_tensor(x, 127 / 4.0), f["quant_out"])
    for post in (0, 1):
        q, res = oracle.norm_layer_resual_i8O(x, g, b, rb, 127 / 4.0, post)
        eq(q, f["ln_first_q_%d" % post]); eq(res, f["ln_first_res_%d" % post])
        q, res = oracle.residual_bias_ln_i8O(f["ln_acc8"], g, b, rb, x, 2.0 / 127, 127 / 4.0, post)
        eq(q, f["ln_i8_q_%d" % post]); eq(res, f["ln_i8_res_%d" % post])
        q, res = oracle.residual_bias_ln_i8O(f["ln_acc32"], g, b, rb, x, 1e-5, 127 / 4.0, post, cs)
        eq(q, f["ln_i32_q_%d" % post]); eq(res, f["ln_i32_res_%d" % post])
    eq(oracle.residual_bias_ln_i32I(f["ln_acc32"], g, b, x, 1e-5, cs), f["ln_i32_out"])
    eq(oracle.bias_gelu_i8I_i8O(f["act_in"], f["act_bias"], 2.2 / 127, 127 / 2.2), f["gelu_out"])
    eq(oracle.bias_relu_i8I_i8O(f["act_in"], f["act_bias"], 2.2 / 127, 127 / 1.65, 1.65, True), f["relu_narrow_out"])
    eq(oracle.gemm_i8_i32(f["gemm_a"], f["gemm_w"]), f["gemm_i32"])
    eq(oracle.gemm_i8_i8(f["gemm_a"], f["gemm_w"], 4.0 * 0.08 / (2.2 * 127)), f["gemm_i8"])
    arranged = oracle.arrange_encself_qkv_i8I(f["att_qkv"], f["att_bias"], 2, 5, 2, 2.2 / 127)
    eq(arranged, f["att_arranged"])
    eq(oracle.attn_context(f["att_probs"], arranged[2]), f["att_ctx"])
    from lightseq_amd import synthetic
    from oracle.model_io import oracle_weights_from_message
    for name in ("gelu_post", "relu_pre"):
        cfg = _stack_cfg(name)
        msg = synthetic.make_quant_bert(cfg, seed=11)
        out, _, _ = oracle.quant_bert_encoder(oracle_weights_from_message(msg, cfg), f["stack_%s_ids" % name])
        eq(out, f["stack_%s_out" % name])


def _d(a):
    return torch.from_numpy(np.ascontiguousarray(a)).to(DEV)


def _n(t):
    torch.cuda.synchronize()
    return t.cpu().numpy()


@pytest.mark.gpu
def test_hip_kernels_match_fixtures():
    from lightseq_amd import kernels as K
    f = FX
    g, b, rb, cs = (_d(f[k]) for k in ("ln_g", "ln_b", "ln_rb", "ln_cs"))
    tokens, H = f["ln_x"].shape
    out = torch.zeros((tokens, H), dtype=torch.int8, device=DEV)
    K.launch_quantize_tensor(_d(f["ln_x"]), out, tokens, H, 127 / 4.0)
    np.testing.assert_array_equal(_n(out), f["quant_out"])
    for post in (0, 1):
        x = _d(f["ln_x"])
        K.ker_norm_layer_resual_i8O_launcher(tokens, H, x, out, g, b, rb, 1024, 127 / 4.0, bool(post))
        assert_codes_close(_n(out), f["ln_first_q_%d" % post], max_frac=5e-3)
        np.testing.assert_allclose(_n(x).astype(np.float32), f["ln_first_res_%d" % post].astype(np.float32), atol=4e-3)
        x = _d(f["ln_x"])
        K.ker_residual_bias_ln_i8I_i8O_launcher(_d(f["ln_acc8"]), g, b, rb, out, x, tokens, H, 2.0 / 127,
                                                127 / 4.0, 1024, bool(post))
        assert_codes_close(_n(out), f["ln_i8_q_%d" % post], max_frac=5e-3)
        np.testing.assert_allclose(_n(x).astype(np.float32), f["ln_i8_res_%d" % post].astype(np.float32), atol=8e-3)
        x = _d(f["ln_x"])
        K.ker_residual_bias_ln_i32I_i8O_launcher(_d(f["ln_acc32"]), g, b, rb, out, x, tokens, H, 1e-5,
                                                 127 / 4.0, 1024, bool(post), False, False, cs)
        assert_codes_close(_n(out), f["ln_i32_q_%d" % post], max_frac=5e-3)
        np.testing.assert_allclose(_n(x).astype(np.float32), f["ln_i32_res_%d" % post].astype(np.float32), atol=8e-3)
    x = _d(f["ln_x"])
    K.ker_residual_bias_ln_i32I_launcher(_d(f["ln_acc32"]), g, b, x, x, tokens, H, 1e-5, 1024, False, cs)
    np.testing.assert_allclose(_n(x).astype(np.float32), f["ln_i32_out"].astype(np.float32), atol=4e-3)
    deq = torch.zeros((tokens, H), dtype=torch.float16, device=DEV)
    K.launch_dequantize_tensor(_d(f["ln_acc32"]), deq, tokens, H, 1e-5)
    np.testing.assert_allclose(_n(deq).astype(np.float32), f["deq_out"].astype(np.float32), rtol=2e-3)

    I = f["act_in"].shape[1]
    o8 = torch.zeros(f["act_in"].shape, dtype=torch.int8, device=DEV)
    K.ker_bias_gelu_i8I_i8O_launcher(tokens, _d(f["act_in"]), o8, _d(f["act_bias"]), I, 2.2 / 127, 127 / 2.2)
    assert_codes_close(_n(o8), f["gelu_out"], max_frac=5e-3)
    K.ker_bias_relu_i8I_i8O_launcher(tokens, _d(f["act_in"]), o8, _d(f["act_bias"]), I, 2.2 / 127, 127 / 1.65,
                                     1.65, False, False, False)
    assert_codes_close(_n(o8), f["relu_out"], max_frac=5e-3)
    K.ker_bias_relu_i8I_i8O_launcher(tokens, _d(f["act_in"]), o8, _d(f["act_bias"]), I, 2.2 / 127, 127 / 1.65,
                                     1.65, False, False, True)
    assert_codes_close(_n(o8), f["relu_narrow_out"], max_frac=5e-3)

    B, S, h, d = 2, 5, 2, 32
    arr = torch.zeros((3, B, h, S, d), dtype=torch.float16, device=DEV)
    K.ker_arrange_encself_qkv_i8I_launcher(B * S, h * d, _d(f["att_qkv"]), _d(f["att_bias"]), arr, B * S * h * d,
                                           S, d, h, 1024, 2.2 / 127)
    np.testing.assert_allclose(_n(arr).astype(np.float32), f["att_arranged"].astype(np.float32), atol=2e-3)
    ctx = torch.zeros((B, h, S, d), dtype=torch.float16, device=DEV)
    ctx_q = torch.zeros((B * S, h * d), dtype=torch.int8, device=DEV)
    K.encself_attention(arr[0], arr[1], arr[2], _d(f["att_mask"]), ctx, ctx_q, 127 / 0.5, B, S, h, d)
    np.testing.assert_allclose(_n(ctx).astype(np.float32), f["att_ctx"].astype(np.float32), atol=2e-3)
    assert_codes_close(_n(ctx_q), f["att_ctx_q"], max_frac=1e-2)

    M, Kk = f["gemm_a"].shape
    N = f["gemm_w"].shape[0]
    c32 = torch.zeros((M, N), dtype=torch.int32, device=DEV)
    K.gemm_i8_i32o(_d(f["gemm_a"]), _d(f["gemm_w"]), c32, M, N, Kk)
    np.testing.assert_array_equal(_n(c32), f["gemm_i32"])
    c8 = torch.zeros((M, N), dtype=torch.int8, device=DEV)
    K.gemm_i8_i8o(_d(f["gemm_a"]), _d(f["gemm_w"]), c8, M, N, Kk, 4.0 * 0.08 / (2.2 * 127))
    np.testing.assert_array_equal(_n(c8), f["gemm_i8"])


@pytest.mark.gpu
@pytest.mark.parametrize("name", ["gelu_post", "relu_pre"])
def test_hip_stack_matches_fixture(tmp_path, name):
    from lightseq_amd import inference, synthetic
    cfg = _stack_cfg(name)
    path = str(tmp_path / "m.pb")
    synthetic.write_quant_bert(path, cfg, seed=11)
    ids = FX["stack_%s_ids" % name]
    model = inference.QuantBert(path, ids.shape[0])
    got = model.infer(ids)
    v = ids != cfg["padding_id"]
    np.testing.assert_allclose(got[v], FX["stack_%s_out" % name].astype(np.float32)[v], atol=2e-2, rtol=0)
    model.close()
