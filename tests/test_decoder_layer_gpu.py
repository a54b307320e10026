"""GPU parity of the csrc decoder layer (TransformerDecoderLayer behind
``ls_create_transformer_decoder_layer_fp16`` / ``ls_transformer_decoder_layer_fw_fp16``) and
of the operators it adds (launch_bias_add_transform_20314, launch_concat3_dim1, the attention
core with its own number of keys) against the numpy restatement in oracle/layer_ops.py.
Bars: permutation kernels bit-exact; fp16 layer outputs within 2e-2 absolute."""
import numpy as np
import pytest
import torch

from helpers import DEV, to_dev, to_np, torch_dtype

pytestmark = pytest.mark.gpu

HS, NH, IMS, NLAYER = 128, 4, 256, 2
HD = HS // NH


def _lo():
    from oracle import layer_ops
    return layer_ops


def _ops():
    from lightseq_amd import ops
    return ops


@pytest.mark.parametrize("dtype", [np.float16, np.float32])
def test_bias_add_transform_20314(rng, dtype):
    d0, d1, d2, d3, d4 = 3, 5, 4, 2, 32
    x = rng.standard_normal((d0, d1, d2, d3, d4)).astype(dtype)
    b = rng.standard_normal((d2, d3, d4)).astype(dtype)
    out = torch.zeros(d2, d0, d3, d1, d4, dtype=torch_dtype(dtype), device=DEV)
    _ops().launch_bias_add_transform_20314(out, to_dev(x), to_dev(b), d0, d1, d2, d3, d4)
    np.testing.assert_array_equal(to_np(out),
                                  _lo().launch_bias_add_transform_20314(x, b, d0, d1, d2, d3, d4))


@pytest.mark.parametrize("dtype", [np.float16, np.float32])
@pytest.mark.parametrize("step", [0, 1, 37])
def test_concat3_dim1(rng, dtype, step):
    sz0, sz2 = 24, 32
    old = rng.standard_normal((sz0, step, sz2)).astype(dtype)
    new = rng.standard_normal((sz0, 1, sz2)).astype(dtype)
    out = torch.zeros(sz0, step + 1, sz2, dtype=torch_dtype(dtype), device=DEV)
    _ops().launch_concat3_dim1(to_dev(old) if step else None, to_dev(new), out, sz0, sz2, step, 1)
    np.testing.assert_array_equal(to_np(out), np.concatenate([old, new], 1))


def test_small_kernel_argument_errors():
    from lightseq_amd import lib
    out = torch.zeros(64, dtype=torch.half, device=DEV)
    with pytest.raises(lib.LSHError, match="multiple of the vector"):
        _ops().launch_concat3_dim1(out, out, out, 1, 4, 1, 1)
    with pytest.raises(lib.LSHError, match="null pointer"):
        _ops().launch_concat3_dim1(None, out, out, 1, 8, 1, 1)
    with pytest.raises(lib.LSHError, match="multiple of the vector"):
        _ops().launch_bias_add_transform_20314(out, out, out, 1, 1, 1, 1, 4)
    with pytest.raises(lib.LSHError, match="bad arguments"):  # causal needs as many keys as queries
        _ops().layer_cross_attention(out, out, out, None, out, 1, 1, 2, 1, 32, True)


@pytest.mark.parametrize("from_len,to_len,hd", [(1, 1, 64), (1, 77, 64), (4, 50, 32), (4, 300, 64),
                                                (70, 33, 128), (200, 129, 32)])
def test_cross_attention(rng, from_len, to_len, hd):
    """Queries and keys of different counts: one decoding step over a cache, a beam of queries
    over the source sentence, a whole target sequence over the source."""
    lo = _lo()
    batch, heads = 3, 2
    q = rng.standard_normal((batch * heads, from_len, hd)).astype(np.float16)
    k, v = (rng.standard_normal((batch * heads, to_len, hd)).astype(np.float16) for _ in range(2))
    pad = np.zeros((batch, to_len), np.float32)
    pad[1, to_len - to_len // 3:] = -1e8
    with np.errstate(over="ignore"):
        pad = pad.astype(np.float16)
    want = lo._attention(q, k, v, batch, heads, pad, False).reshape(batch, from_len, heads * hd)
    out = torch.zeros(batch, from_len, heads * hd, dtype=torch.float16, device=DEV)
    _ops().layer_cross_attention(to_dev(q), to_dev(k), to_dev(v), to_dev(pad), out, batch, from_len,
                                 to_len, heads, hd)
    np.testing.assert_allclose(to_np(out).astype(np.float64), want.astype(np.float64), atol=3e-3)
    # without a mask
    want = lo._attention(q, k, v, batch, heads, None, False).reshape(batch, from_len, heads * hd)
    _ops().layer_cross_attention(to_dev(q), to_dev(k), to_dev(v), None, out, batch, from_len,
                                 to_len, heads, hd)
    np.testing.assert_allclose(to_np(out).astype(np.float64), want.astype(np.float64), atol=3e-3)


# ---- the layer ----------------------------------------------------------------------------------
def _case(seed, batch, trg, src):
    from test_oracle_decoder_layer import decoder_params, pack_decoder_para
    rng = np.random.default_rng(seed)
    # Clip values near 4 sigma of what they quantise (activations ~ N(0, 1), weights
    # ~ N(0, 0.03), GEMM outputs ~ N(0, 0.35)), as a trained model has them: one int8 step of any
    # of these tensors, which a different summation order in the kernel before it may flip,
    # then moves the layer output by less than the 2e-2 bar.
    ps = [decoder_params(rng, i, NLAYER, HS, IMS, w_std=0.03) for i in range(NLAYER)]
    paras = [pack_decoder_para(p, i, act_clip=4.0, w_clip=0.12, out_clip=1.5)
             for i, p in enumerate(ps)]
    x = rng.standard_normal((batch, trg, HS)).astype(np.float16)
    enc = rng.standard_normal((batch, src, HS)).astype(np.float16)
    pad = np.zeros((batch, src), np.float32)
    pad[batch - 1, src - src // 3:] = 1
    with np.errstate(over="ignore"):
        mask = (pad * -1e8).astype(np.float16)
    return paras, x, enc, pad, mask


def _make_stack(paras, pre_ln, act, max_tokens, max_seq):
    from lightseq_amd.layers import LSTransformerDecoderLayer as L
    L.new_stack()
    config = L.get_config(max_batch_tokens=max_tokens, max_seq_len=max_seq, hidden_size=HS,
                          intermediate_size=IMS, nhead=NH, attn_prob_dropout_ratio=0.1,
                          activation_dropout_ratio=0.1, hidden_dropout_ratio=0.1,
                          pre_layer_norm=pre_ln, fp16=True, local_rank=0, nlayer=NLAYER,
                          activation_fn=act)
    layers = []
    for para in paras:
        layer = L(config).to(DEV).half().eval()
        assert layer.para.numel() == para.size
        with torch.no_grad():
            layer.para.copy_(to_dev(para))
        layer.enable_quant()
        layers.append(layer)
    return layers


def _release(layers):
    for layer in layers:
        layer.release()


@pytest.mark.parametrize("pre_ln,act", [(False, "relu"), (True, "gelu")])
def test_decoder_layer_whole_sequence_matches_restatement(pre_ln, act):
    lo = _lo()
    batch, trg, src = 3, 21, 30
    paras, x, enc, pad, mask = _case(11, batch, trg, src)
    layers = _make_stack(paras, pre_ln, act, 128, 64)
    try:
        kv = lo.decoder_encdec_kv(paras[0], enc, NH, IMS, NLAYER)
        enc_t = to_dev(enc).transpose(0, 1)  # the layer takes [src_len, batch, hidden]
        for lid, layer in enumerate(layers):
            with torch.no_grad():
                got = to_np(layer(to_dev(x), enc_t, to_dev(pad)))
            want = lo.decoder_layer_forward(paras[lid], lid, NLAYER, x, kv, mask, NH, IMS, pre_ln,
                                            act)
            d = np.abs(got.astype(np.float64) - want.astype(np.float64))
            assert d.max() < 2e-2 and d.mean() < 1e-3, (lid, d.max(), d.mean())
            with torch.no_grad():
                again = to_np(layer(to_dev(x), enc_t, to_dev(pad)))
            np.testing.assert_array_equal(again, got)
    finally:
        _release(layers)


@pytest.mark.parametrize("pre_ln", [False, True])
def test_decoding_steps_match_restatement_and_the_whole_sequence_pass(pre_ln):
    """Step by step with caches, beams of 3 carrying the same token: every step within 2e-2 of
    the restatement's step, the caches equal to its caches up to one int8 step of the
    fake-quantised k / v on a few elements, and the steps within 2e-2 of the rows of the
    layer's own whole-sequence pass."""
    lo = _lo()
    batch, trg, src, beam = 2, 9, 12, 3
    paras, x, enc, pad, mask = _case(12, batch, trg, src)
    layers = _make_stack(paras, pre_ln, "relu", 64, 32)
    try:
        kv = lo.decoder_encdec_kv(paras[0], enc, NH, IMS, NLAYER)
        enc_t = to_dev(enc).transpose(0, 1)
        with torch.no_grad():
            full = [to_np(layer(to_dev(x), enc_t, to_dev(pad))) for layer in layers]
        caches = [{} for _ in layers]
        want_caches = [{} for _ in layers]
        for t in range(trg):
            xt = np.repeat(x[:, t:t + 1], beam, axis=0)
            for lid, layer in enumerate(layers):
                with torch.no_grad():
                    got = to_np(layer(to_dev(xt), enc_t, to_dev(pad), cache=caches[lid]))
                want = lo.decoder_layer_forward(paras[lid], lid, NLAYER, xt, kv, mask, NH, IMS,
                                                pre_ln, "relu", cache=want_caches[lid], beam=beam)
                d = np.abs(got.astype(np.float64) - want.astype(np.float64))
                assert d.max() < 2e-2 and d.mean() < 1e-3, (t, lid, d.max(), d.mean())
                rows = np.repeat(full[lid][:, t:t + 1], beam, axis=1).reshape(got.shape)
                assert np.abs(got.astype(np.float64) - rows).max() < 2e-2, (t, lid)
                assert caches[lid]["dec_self_k"].shape == (batch * beam, NH, t + 1, HD)
                for name, key in (("dec_self_k", "k"), ("dec_self_v", "v")):
                    c = to_np(caches[lid][name]).reshape(want_caches[lid][key].shape)
                    dc = np.abs(c.astype(np.float64) - want_caches[lid][key])
                    assert dc.max() <= 4.0 / 127 + 1e-3 and (dc > 0).mean() < 5e-3, (t, lid, name)
        # the shared cross-attention k/v that layer 0 wrote at step 0
        got_kv = to_np(caches[0]["encdec_kv"]).reshape(kv.shape)
        np.testing.assert_allclose(got_kv.astype(np.float64), kv.astype(np.float64), atol=4e-3)
    finally:
        _release(layers)


def test_decoder_layer_argument_errors():
    from lightseq_amd import lib
    paras, x, enc, pad, mask = _case(13, 2, 4, 6)
    layers = _make_stack(paras, False, "relu", 16, 8)
    try:
        xd, enc_t, padd = to_dev(x), to_dev(enc).transpose(0, 1), to_dev(pad)
        layers[0].train()
        with pytest.raises(lib.LSHError, match="training mode"):
            layers[0](xd, enc_t, padd)
        layers[0].eval()
        layers[0].disable_quant()
        with pytest.raises(lib.LSHError, match="quantised path"):
            layers[0](xd, enc_t, padd)
        layers[0].enable_quant()
        with pytest.raises(ValueError, match="exceeds the limit"):
            layers[0](torch.zeros(2, 9, HS, dtype=torch.half, device=DEV), enc_t, padd)
        with pytest.raises(lib.LSHError, match="cache pointers"):
            lib.call("ls_transformer_decoder_layer_fw_fp16", 0, lib.ptr(xd), lib.ptr(xd), None,
                     lib.ptr(xd), 2, 1, 6, 0, None, 0, 0, 1)
        with pytest.raises(lib.LSHError, match="does not exist"):
            lib.call("ls_transformer_decoder_layer_fw_fp16", 99999, None, None, None, None, 1, 1,
                     1, -1, None, 0, 0, 1)
        import ctypes
        n = ctypes.c_longlong(0)
        lib.call("ls_layer_param_count", b"TransformerDecoderLayer", 0, ctypes.byref(n))
        assert n.value == paras[0].size
        lib.call("ls_layer_param_count", b"TransformerDecoderLayer", 1, ctypes.byref(n))
        assert n.value == paras[1].size
    finally:
        _release(layers)
    with pytest.raises(lib.LSHError, match="does not exist"):
        layers[0](xd, enc_t, padd)
