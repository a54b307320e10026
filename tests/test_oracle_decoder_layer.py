"""Pins the numpy restatement of the csrc decoder layer (oracle/layer_ops.py
decoder_layer_forward / decoder_encdec_kv) without a GPU:

* against torch's own ``nn.TransformerDecoderLayer`` in float64 with the same weights: the
  quantised layer is that layer plus int8 noise, so with biases and layer-norm offsets of
  order 0.3 a dropped bias, a swapped k/v slice, a wrong layer offset into the shared k/v or a
  transposed weight moves the output by far more than the tolerance;
* a decoding step with caches must reproduce, bit for bit, the row of the whole-sequence pass
  (the masked scores underflow to exact zeros), which pins the cache concatenation, the step
  arithmetic and the beam layout of the cross attention;
* the two small kernels against numpy one-liners.
"""
import numpy as np
import pytest
import torch

from oracle import layer_ops as lo

F32 = np.float32
HS, NH, IMS, NLAYER = 64, 2, 128, 2


def decoder_params(rng, layer_id, nlayer=NLAYER, hs=HS, ims=IMS, w_std=0.08, b_std=0.3):
    g = lambda *shape: rng.standard_normal(shape)
    p = {}
    for name, rows, cols in (("attn_qkvw", 3 * hs, hs), ("attn_ow", hs, hs),
                             ("encdec_attn_qw", hs, hs), ("encdec_attn_ow", hs, hs),
                             ("inter_w", ims, hs), ("output_w", hs, ims)):
        p[name] = np.clip(g(rows, cols) * w_std, -4 * w_std, 4 * w_std)
    for name, n in (("attn_qkvb", 3 * hs), ("attn_ob", hs), ("encdec_attn_qb", hs),
                    ("encdec_attn_ob", hs), ("inter_b", ims), ("output_b", hs)):
        p[name] = g(n) * b_std
    for pre in ("attn", "encdec_attn", "ffn"):
        p[pre + "_nw"] = 1 + 0.1 * g(hs)
        p[pre + "_nb"] = b_std * g(hs)
    if layer_id == 0:
        p["encdec_attn_kvw"] = np.clip(g(nlayer * 2 * hs, hs) * w_std, -4 * w_std, 4 * w_std)
        p["encdec_attn_kvb"] = g(nlayer * 2 * hs) * b_std
    return {k: v.astype(np.float16).astype(F32) for k, v in p.items()}


ORDER = ["attn_qkvw", "attn_qkvb", "attn_ow", "attn_ob", "attn_nw", "attn_nb", "encdec_attn_qw",
         "encdec_attn_qb", "encdec_attn_ow", "encdec_attn_ob", "encdec_attn_nw", "encdec_attn_nb",
         "inter_w", "inter_b", "output_w", "output_b", "ffn_nw", "ffn_nb"]


def pack_decoder_para(p, layer_id, act_clip=8.0, w_clip=0.32, out_clip=None, dtype=np.float16):
    """Flat blob in the order of transformer_decoder_layer.h:100-168; by default wide
    activation clips so that nothing saturates and the layer stays close to its float
    counterpart.  out_clip: clip value of the int8 GEMM outputs, when it shall differ."""
    out_clip = act_clip if out_clip is None else out_clip
    clips = [act_clip, w_clip, out_clip] * 6 + [act_clip, w_clip, 0, 0, 0] + [act_clip]
    parts = [p[k].reshape(-1) for k in ORDER] + [np.array(clips)]
    if layer_id == 0:
        parts += [p["encdec_attn_kvw"].reshape(-1), p["encdec_attn_kvb"]]
    return np.concatenate(parts).astype(dtype)


def torch_decoder_layer(p, kvw, kvb, pre_ln, act):
    ref = torch.nn.TransformerDecoderLayer(HS, NH, IMS, dropout=0.0, activation=act,
                                           batch_first=True, norm_first=pre_ln,
                                           layer_norm_eps=1e-8).double().eval()
    t = lambda a: torch.from_numpy(np.asarray(a, np.float64))
    with torch.no_grad():
        ref.self_attn.in_proj_weight.copy_(t(p["attn_qkvw"]))
        ref.self_attn.in_proj_bias.copy_(t(p["attn_qkvb"]))
        ref.self_attn.out_proj.weight.copy_(t(p["attn_ow"]))
        ref.self_attn.out_proj.bias.copy_(t(p["attn_ob"]))
        ref.multihead_attn.in_proj_weight.copy_(t(np.concatenate([p["encdec_attn_qw"], kvw])))
        ref.multihead_attn.in_proj_bias.copy_(t(np.concatenate([p["encdec_attn_qb"], kvb])))
        ref.multihead_attn.out_proj.weight.copy_(t(p["encdec_attn_ow"]))
        ref.multihead_attn.out_proj.bias.copy_(t(p["encdec_attn_ob"]))
        ref.linear1.weight.copy_(t(p["inter_w"])); ref.linear1.bias.copy_(t(p["inter_b"]))
        ref.linear2.weight.copy_(t(p["output_w"])); ref.linear2.bias.copy_(t(p["output_b"]))
        for norm, pre in ((ref.norm1, "attn"), (ref.norm2, "encdec_attn"), (ref.norm3, "ffn")):
            norm.weight.copy_(t(p[pre + "_nw"])); norm.bias.copy_(t(p[pre + "_nb"]))
    return ref


def make_case(seed, batch=2, trg=7, src=9):
    rng = np.random.default_rng(seed)
    ps = [decoder_params(rng, i) for i in range(NLAYER)]
    paras = [pack_decoder_para(p, i) for i, p in enumerate(ps)]
    x = rng.standard_normal((batch, trg, HS)).astype(np.float16)
    enc = rng.standard_normal((batch, src, HS)).astype(np.float16)
    pad = np.zeros((batch, src), bool)
    pad[1, src - 3:] = True
    with np.errstate(over="ignore"):
        mask = (pad * -1e8).astype(np.float16)  # -inf in fp16, as the reference's mask
    return ps, paras, x, enc, pad, mask


@pytest.mark.parametrize("pre_ln,act", [(False, "relu"), (True, "gelu")])
def test_decoder_layer_is_torch_decoder_layer_plus_int8_noise(pre_ln, act):
    ps, paras, x, enc, pad, mask = make_case(3)
    kv = lo.decoder_encdec_kv(paras[0], enc, NH, IMS, NLAYER)
    assert kv.shape == (NLAYER * 2, 2, NH, 9, HS // NH) and kv.dtype == np.float16
    causal = torch.triu(torch.ones(7, 7, dtype=torch.bool), 1)
    for lid in range(NLAYER):
        got = lo.decoder_layer_forward(paras[lid], lid, NLAYER, x, kv, mask, NH, IMS, pre_ln, act)
        rows = slice(2 * lid * HS, (2 * lid + 2) * HS)
        ref = torch_decoder_layer(ps[lid], ps[0]["encdec_attn_kvw"][rows],
                                  ps[0]["encdec_attn_kvb"][rows], pre_ln, act)
        with torch.no_grad():
            want = ref(torch.from_numpy(x.astype(np.float64)),
                       torch.from_numpy(enc.astype(np.float64)), tgt_mask=causal,
                       memory_key_padding_mask=torch.from_numpy(pad)).numpy()
        d = np.abs(got.astype(np.float64) - want)
        scale = np.abs(want).mean()
        # int8 steps of 8/127 on unit-variance activations: a few percent of the output scale
        assert d.mean() < 0.04 * scale and d.max() < 0.5 * scale, (lid, d.mean(), d.max(), scale)
        # what a structural mistake costs: the other layer's k/v slice is already far outside
        other = slice(2 * (1 - lid) * HS, (2 * (1 - lid) + 2) * HS)
        wrong = torch_decoder_layer(ps[lid], ps[0]["encdec_attn_kvw"][other],
                                    ps[0]["encdec_attn_kvb"][other], pre_ln, act)
        with torch.no_grad():
            w2 = wrong(torch.from_numpy(x.astype(np.float64)),
                       torch.from_numpy(enc.astype(np.float64)), tgt_mask=causal,
                       memory_key_padding_mask=torch.from_numpy(pad)).numpy()
        assert np.abs(w2 - want).mean() > 5 * d.mean()


@pytest.mark.parametrize("pre_ln", [False, True])
def test_decoding_steps_reproduce_the_whole_sequence_pass(pre_ln):
    ps, paras, x, enc, pad, mask = make_case(5, batch=2, trg=6, src=5)
    beam = 3
    kv = lo.decoder_encdec_kv(paras[0], enc, NH, IMS, NLAYER)
    for lid in range(NLAYER):
        full = lo.decoder_layer_forward(paras[lid], lid, NLAYER, x, kv, mask, NH, IMS, pre_ln,
                                        "relu")
        cache = {}
        for t in range(x.shape[1]):
            # every beam of a sentence carries the same token: rows b * beam + j
            xt = np.repeat(x[:, t:t + 1], beam, axis=0)
            out = lo.decoder_layer_forward(paras[lid], lid, NLAYER, xt, kv, mask, NH, IMS, pre_ln,
                                           "relu", cache=cache, beam=beam)
            assert cache["k"].shape == (2 * beam * NH, t + 1, HS // NH)
            np.testing.assert_array_equal(out.reshape(2, beam, HS),
                                          np.repeat(full[:, t:t + 1], beam, axis=1))


def test_small_kernels_against_numpy(rng):
    d0, d1, d2, d3, d4 = 2, 3, 4, 2, 8
    for dt in (np.float16, np.float32):
        x = rng.standard_normal((d0, d1, d2, d3, d4)).astype(dt)
        b = rng.standard_normal((d2, d3, d4)).astype(dt)
        got = lo.launch_bias_add_transform_20314(x, b, d0, d1, d2, d3, d4)
        assert got.dtype == dt and got.shape == (d2, d0, d3, d1, d4)
        for c in range(d2):
            for h in range(d3):
                np.testing.assert_array_equal(got[c, :, h], (x[:, :, c, h] + b[c, h]).astype(dt))
    a = rng.standard_normal((3, 4, 8)).astype(np.float16)
    b = rng.standard_normal((3, 1, 8)).astype(np.float16)
    np.testing.assert_array_equal(lo.launch_concat3_dim1(a, b, 3, 8, 4, 1),
                                  np.concatenate([a, b], 1))
    np.testing.assert_array_equal(lo.launch_concat3_dim1(None, b, 3, 8, 0, 1), b)
