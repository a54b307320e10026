"""GPU parity of the int8 GPT path: its kernels through the C ABI and the QuantGpt model
through the model C ABI, against the CPU oracle.

Bars: integer work (cache writes / re-layout, int32 scores, sampled ids given equal logits)
bit-exact; int8 activations within +-1 code on <= 0.1 % of the elements; fp16 values within
the tolerance written in each test.  Whole-run token equality is checked stage-conditionally
(the oracle consumes the GPU's logits in its arg-max) and, on small models, free-running.
"""
import os

import numpy as np
import pytest
import torch

from conftest import assert_codes_close
from helpers import DEV, to_dev, to_np

pytestmark = pytest.mark.gpu

DTYPES = [np.float16, np.float32]
TD = {np.float16: torch.float16, np.float32: torch.float32}


def _k():
    from lightseq_amd import kernels
    return kernels


def _og():
    from oracle import gpt
    return gpt


def _codes(rng, shape):
    return rng.integers(-127, 128, size=shape, dtype=np.int8)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("batch,seq,hidden,vocab,offset", [(3, 7, 128, 50, 0), (2, 1, 1024, 300, 9),
                                                           (1, 16, 72, 20, 3)])
def test_gpt_embedding(rng, dtype, batch, seq, hidden, vocab, offset):
    table = _codes(rng, (vocab, hidden))
    pos = (rng.standard_normal((seq + offset + 2, hidden)) * 0.1).astype(dtype)
    pad = 0
    ids = rng.integers(0, vocab, size=(batch, seq), dtype=np.int32)
    ids[0, seq // 2:] = pad
    rsl0 = rng.integers(0, 5, size=batch).astype(np.int32)
    dq = 0.08 / 127
    want, want_rsl = _og().gpt_embedding_i8I(table, pos, ids, rsl0, pad, offset, dq)
    out = torch.zeros(batch, seq, hidden, dtype=TD[dtype], device=DEV)
    rsl = to_dev(rsl0)
    _k().ker_gpt_embedding_i8I_launcher(batch, seq, hidden, to_dev(table), to_dev(pos), to_dev(ids),
                                        out, rsl, pad, offset, dq)
    np.testing.assert_array_equal(to_np(out), want)
    np.testing.assert_array_equal(to_np(rsl), want_rsl)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("batch,heads,seq,d", [(2, 3, 9, 16), (1, 4, 130, 32), (3, 2, 64, 64)])
def test_gpt_scores_and_softmax(rng, dtype, batch, heads, seq, d):
    bh = batch * heads
    q, k = _codes(rng, (bh, seq, d)), _codes(rng, (bh, seq, d))
    want_sc = _og().gpt_scores_i8(q, k)
    sc = torch.zeros(bh, seq, seq, dtype=torch.int32, device=DEV)
    _k().gpt_scores_i8_i32o(to_dev(k), to_dev(q), sc, bh, seq, d)
    np.testing.assert_array_equal(to_np(sc), want_sc)

    rsl = rng.integers(max(1, seq // 2), seq + 1, size=batch).astype(np.int32)
    rsl[0] = seq
    dq, attn_scale = 4.0 / 127, float(np.float16(np.sqrt(1.0 / d)))
    want = _og().correlation_softmax_gpt_i32I(want_sc, rsl, heads, attn_scale, dq, dtype)
    out = torch.full((bh, seq, seq), 7.0, dtype=TD[dtype], device=DEV)
    _k().ker_correlation_softmax_gpt_i32I_launcher(batch, seq, heads, sc, out, to_dev(rsl),
                                                   attn_scale, dq)
    got = to_np(out).astype(np.float32)
    tol = 1e-3 if dtype == np.float16 else 2e-6
    np.testing.assert_allclose(got, want.astype(np.float32), atol=tol, rtol=0)
    assert not np.triu(got, 1).any()  # nothing to the right of the diagonal


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("batch,heads,seq,d", [(2, 3, 5, 16), (3, 16, 1, 64), (1, 2, 40, 10)])
def test_arrange_qkv_with_cache(rng, dtype, batch, heads, seq, d):
    H = heads * d
    ori = _codes(rng, (batch, 3 * H))
    bias = (rng.standard_normal(3 * H) * 0.5).astype(dtype)
    kc, vc = _codes(rng, (batch, heads, seq - 1, d)), _codes(rng, (batch, heads, seq - 1, d))
    dq, qs = 3.0 / 127, 127 / 2.5
    wq, wk, wv = _og().arrange_qkv_with_cache_i8I_i8O(ori, bias, kc, vc, dq, qs)
    q = torch.zeros(batch, heads, 1, d, dtype=torch.int8, device=DEV)
    nk = torch.zeros(batch, heads, seq, d, dtype=torch.int8, device=DEV)
    nv = torch.zeros_like(nk)
    kcd = to_dev(kc) if seq > 1 else torch.zeros(1, dtype=torch.int8, device=DEV)
    vcd = to_dev(vc) if seq > 1 else torch.zeros(1, dtype=torch.int8, device=DEV)
    _k().ker_arrange_qkv_with_cache_i8I_i8O_launcher(batch * seq, H, to_dev(ori), to_dev(bias), q,
                                                     nk, kcd, nv, vcd, seq, d, heads, dq, qs)
    np.testing.assert_array_equal(to_np(q), wq)
    np.testing.assert_array_equal(to_np(nk), wk)
    np.testing.assert_array_equal(to_np(nv), wv)


@pytest.mark.parametrize("batch,seq,vocab,lsl", [(4, 6, 300, 6), (3, 9, 50257, 1), (2, 1, 77, 1)])
def test_topk_sample_greedy(rng, batch, seq, vocab, lsl):
    eos = 5
    logits = np.clip(rng.standard_normal((batch * lsl, vocab)) * 30, -127, 127).astype(np.int8)
    logits[(0 + 1) * lsl - 1, 17:20] = 127  # a three-way tie at the maximum: lowest id wins
    old = rng.integers(6, vocab, size=(batch, seq), dtype=np.int32)
    old[1, -1] = eos  # an ended sequence stays ended
    if batch > 2:
        logits[(2 + 1) * lsl - 1, eos] = 127
        logits[(2 + 1) * lsl - 1, :eos] = -5
    w_new, w_last, w_unf = _og().topk_sample_i8I_greedy(logits, old, lsl, eos, 0.02)
    assert w_last[0] == 17 and w_last[1] == eos
    buf = torch.zeros(batch * seq + batch, dtype=torch.int32, device=DEV)
    buf[:batch * seq] = to_dev(old.reshape(-1))
    new = torch.zeros(batch, seq + 1, dtype=torch.int32, device=DEV)
    unf = torch.zeros(1, dtype=torch.int32, device=DEV)
    _k().ker_topk_sample_i8I_launcher(batch, seq, lsl, 1024, to_dev(logits), buf, new, None, vocab,
                                      1, unf, None, eos, 0.02)
    np.testing.assert_array_equal(to_np(new), w_new)
    np.testing.assert_array_equal(to_np(buf)[batch * seq:], w_last)
    assert int(to_np(unf)[0]) == w_unf

    # the in-place step of the model gives the same tokens
    max_step = seq + 3
    ids = torch.zeros(batch, max_step, dtype=torch.int32, device=DEV)
    ids[:, :seq] = to_dev(old)
    last = torch.zeros(batch, dtype=torch.int32, device=DEV)
    unf2 = torch.zeros(1, dtype=torch.int32, device=DEV)
    last_rows = to_dev(np.ascontiguousarray(logits.reshape(batch, lsl, vocab)[:, -1]))
    _k().gpt_greedy_step(last_rows, ids, last, vocab, max_step, seq, batch, unf2, eos)
    np.testing.assert_array_equal(to_np(ids)[:, :seq + 1], w_new)
    np.testing.assert_array_equal(to_np(last), w_last)
    assert int(to_np(unf2)[0]) == w_unf


def test_topk_sample_errors():
    from lightseq_amd.lib import LSHError
    z8 = torch.zeros(64, dtype=torch.int8, device=DEV)
    zi = torch.zeros(64, dtype=torch.int32, device=DEV)
    with pytest.raises(LSHError, match="generator state"):  # random sampling without its state
        _k().ker_topk_sample_i8I_launcher(1, 4, 1, 1024, z8, zi, zi, None, 16, 4, zi, None, 1, 0.1)
    with pytest.raises(LSHError, match=r"\[1,2,4,8,16,32\]"):
        _k().ker_topk_sample_i8I_launcher(1, 4, 1, 1024, z8, zi, zi, None, 16, 3, zi, None, 1, 0.1)


@pytest.mark.parametrize("batch,seq,vocab", [(3, 8, 300), (2, 5, 5000), (3, 40, 50257)])
def test_ppl(rng, batch, seq, vocab):
    logits = np.clip(rng.standard_normal((batch * seq, vocab)) * 30, -127, 127).astype(np.int8)
    ids = rng.integers(0, vocab, size=(batch, seq), dtype=np.int32)
    rsl = np.array([seq, max(2, seq - 3), 1][:batch], np.int32)
    want = _og().ppl_i8I(logits, ids, rsl, 0.02)
    ppl = torch.zeros(batch, dtype=torch.float32, device=DEV)
    _k().ker_ppl_i8I_launcher(batch, seq, 1024, to_dev(logits), to_dev(ids), to_dev(rsl), ppl,
                              vocab, 0.02)
    np.testing.assert_allclose(to_np(ppl), want, rtol=2e-5, atol=1e-5)
    # one workgroup per position + an ordered sum: the same bits (what the model runs)
    ppl2 = torch.zeros(batch, dtype=torch.float32, device=DEV)
    ws = torch.full((batch * seq,), 7.0, dtype=torch.float32, device=DEV)
    _k().ker_ppl_i8I_workspace(batch, seq, to_dev(logits), to_dev(ids), to_dev(rsl), ppl2, vocab, 0.02, ws)
    np.testing.assert_array_equal(to_np(ppl2).view(np.uint32), to_np(ppl).view(np.uint32))


@pytest.mark.parametrize("batch,heads,seq,d,max_step", [(2, 2, 9, 32, 16), (2, 16, 130, 64, 160),
                                                        (1, 4, 64, 64, 64), (3, 2, 200, 32, 256),
                                                        # the prompt length of the generation benchmark
                                                        (2, 4, 512, 64, 640)])
def test_prefill_attention_fused(oracle, rng, batch, heads, seq, d, max_step):
    """gpt_arrange_qkv_prefill + gpt_prefill_attention == the reference's unfused chain."""
    H, M, bh = heads * d, batch * seq, batch * heads
    ori = _codes(rng, (M, 3 * H))
    bias = (rng.standard_normal(3 * H) * 0.5).astype(np.float16)
    dq_in, qs_cache = 3.0 / 127, 127 / 3.2
    rsl = rng.integers(max(1, seq // 2), seq + 1, size=batch).astype(np.int32)
    rsl[0] = seq
    q8, k8, v8, dv = oracle.arrange_encself_qkv_i8I_i8O(ori, bias, batch, seq, heads, dq_in, qs_cache)
    sc = _og().gpt_scores_i8(q8.reshape(bh, seq, d), k8.reshape(bh, seq, d))
    attn_scale = float(np.float16(np.sqrt(1.0 / d)))
    pr = _og().correlation_softmax_gpt_i32I(sc, rsl, heads, attn_scale, 1.0 / qs_cache, np.float16)
    ctx = oracle.attn_context(pr, dv)
    qs_out = 127 / 1.6
    want_q = oracle.arrange_atten_output_i8O(ctx.reshape(batch, heads, seq, d), qs_out)

    qc = torch.zeros(batch, heads, seq, d, dtype=torch.float16, device=DEV)
    kc, vd = torch.zeros_like(qc), torch.zeros_like(qc)
    kcache = torch.zeros(batch, heads, max_step, d, dtype=torch.int8, device=DEV)
    vcache = torch.zeros_like(kcache)
    _k().gpt_arrange_qkv_prefill(M, H, to_dev(ori), to_dev(bias), qc, kc, vd, kcache, vcache, seq,
                                 d, heads, max_step, dq_in, qs_cache)
    np.testing.assert_array_equal(to_np(qc), q8.astype(np.float16))
    np.testing.assert_array_equal(to_np(kc), k8.astype(np.float16))
    np.testing.assert_array_equal(to_np(vd), dv)
    np.testing.assert_array_equal(to_np(kcache)[:, :, :seq], k8)
    np.testing.assert_array_equal(to_np(vcache)[:, :, :seq], v8)
    assert not to_np(kcache)[:, :, seq:].any()

    ctx_d = torch.zeros(batch, heads, seq, d, dtype=torch.float16, device=DEV)
    ctx_q = torch.zeros(M, H, dtype=torch.int8, device=DEV)
    _k().gpt_prefill_attention(qc, kc, vd, to_dev(rsl), ctx_d, ctx_q, qs_out, 1.0 / qs_cache, batch,
                               seq, heads, d)
    got = to_np(ctx_d).astype(np.float32).reshape(ctx.shape)
    np.testing.assert_allclose(got, ctx.astype(np.float32), atol=4e-3, rtol=0)
    assert_codes_close(to_np(ctx_q), want_q.reshape(M, H), max_frac=5e-3, what="gpt ctx_q")
    # padded queries give zeros
    for b in range(batch):
        assert not to_np(ctx_q).reshape(batch, seq, H)[b, rsl[b]:].any()


@pytest.mark.parametrize("batch,heads,seq,max_step", [(2, 2, 9, 16), (2, 16, 130, 160), (1, 4, 64, 64),
                                                      (3, 2, 200, 256), (2, 4, 512, 640),
                                                      (1, 2, 1000, 1024), (3, 4, 384, 384)])
def test_prefill_attention_on_codes(oracle, rng, batch, heads, seq, max_step):
    """gpt_arrange_qkv_prefill_i8 + gpt_prefill_attention_i8 (int8 codes end to end, what the
    model runs for heads of 64) == the reference's unfused chain, ragged real lengths included;
    and the same context codes as the fp16-storage pair."""
    d = 64
    H, M, bh = heads * d, batch * seq, batch * heads
    ori = _codes(rng, (M, 3 * H))
    bias = (rng.standard_normal(3 * H) * 0.5).astype(np.float16)
    dq_in, qs_cache = 3.0 / 127, 127 / 3.2
    rsl = rng.integers(max(1, seq // 2), seq + 1, size=batch).astype(np.int32)
    rsl[0] = seq
    q8, k8, v8, dv = oracle.arrange_encself_qkv_i8I_i8O(ori, bias, batch, seq, heads, dq_in, qs_cache)
    sc = _og().gpt_scores_i8(q8.reshape(bh, seq, d), k8.reshape(bh, seq, d))
    attn_scale = float(np.float16(np.sqrt(1.0 / d)))
    pr = _og().correlation_softmax_gpt_i32I(sc, rsl, heads, attn_scale, 1.0 / qs_cache, np.float16)
    ctx = oracle.attn_context(pr, dv)
    qs_out = 127 / 1.6
    want_q = oracle.arrange_atten_output_i8O(ctx.reshape(batch, heads, seq, d), qs_out)

    k = _k()
    assert k.gpt_prefill_i8_supported(seq, heads, d)
    assert not k.gpt_prefill_i8_supported(seq, heads, 32)
    assert not k.gpt_prefill_i8_supported(1025, heads, d)
    qc = torch.full((batch, heads, seq, d), 7, dtype=torch.int8, device=DEV)
    kcache = torch.zeros(batch, heads, max_step, d, dtype=torch.int8, device=DEV)
    vcache = torch.zeros_like(kcache)
    orid, biasd, rsld = to_dev(ori), to_dev(bias), to_dev(rsl)
    k.gpt_arrange_qkv_prefill_i8(M, H, orid, biasd, qc, kcache, vcache, seq, d, heads, max_step,
                                 dq_in, qs_cache)
    np.testing.assert_array_equal(to_np(qc), q8)
    np.testing.assert_array_equal(to_np(kcache)[:, :, :seq], k8)
    np.testing.assert_array_equal(to_np(vcache)[:, :, :seq], v8)
    assert not to_np(kcache)[:, :, seq:].any() and not to_np(vcache)[:, :, seq:].any()

    ctx_q = torch.full((M, H), 5, dtype=torch.int8, device=DEV)
    k.gpt_prefill_attention_i8(qc, kcache, vcache, rsld, ctx_q, qs_out, 1.0 / qs_cache, qs_cache,
                               batch, seq, heads, d, max_step)
    got = to_np(ctx_q)
    assert_codes_close(got, want_q.reshape(M, H), max_frac=5e-3, what="gpt ctx_q (codes)")
    for b in range(batch):  # padded queries give zeros
        assert not got.reshape(batch, seq, H)[b, rsl[b]:].any()

    # the fp16-storage pair on the same input: same score integers, same rounding points
    qf = torch.zeros(batch, heads, seq, d, dtype=torch.float16, device=DEV)
    kf, vf = torch.zeros_like(qf), torch.zeros_like(qf)
    kc2, vc2 = torch.zeros_like(kcache), torch.zeros_like(vcache)
    k.gpt_arrange_qkv_prefill(M, H, orid, biasd, qf, kf, vf, kc2, vc2, seq, d, heads, max_step,
                              dq_in, qs_cache)
    assert torch.equal(kc2, kcache) and torch.equal(vc2, vcache)
    ctx_q2 = torch.zeros(M, H, dtype=torch.int8, device=DEV)
    k.gpt_prefill_attention(qf, kf, vf, rsld, None, ctx_q2, qs_out, 1.0 / qs_cache, batch, seq,
                            heads, d)
    assert torch.equal(ctx_q2, ctx_q)


def test_prefill_on_codes_rejects_what_it_does_not_cover(rng):
    k = _k()
    q = torch.zeros(1, 2, 16, 32, dtype=torch.int8, device=DEV)
    c = torch.zeros(1, 2, 16, 32, dtype=torch.int8, device=DEV)
    out = torch.zeros(16, 64, dtype=torch.int8, device=DEV)
    rsl = torch.full((1,), 16, dtype=torch.int32, device=DEV)
    with pytest.raises(RuntimeError, match="heads of 64"):
        k.gpt_prefill_attention_i8(q, c, c, rsl, out, 1.0, 1.0, 1.0, 1, 16, 2, 32, 16)
    ori = torch.zeros(16, 3 * 72, dtype=torch.int8, device=DEV)
    bias = torch.zeros(3 * 72, dtype=torch.float16, device=DEV)
    with pytest.raises(RuntimeError, match="multiple of 128"):
        k.gpt_arrange_qkv_prefill_i8(16, 72, ori, bias, q, c, c, 16, 24, 3, 16, 1.0, 1.0)


# --------------------------------------------------------------------------- #
# model
# --------------------------------------------------------------------------- #
def _make(tmp_path, cfg, seed, **kw):
    from lightseq_amd import synthetic
    path = os.path.join(str(tmp_path), "gpt_%d.pb" % seed)
    msg = synthetic.write_quant_gpt(path, cfg, seed=seed, **kw)
    return path, msg


def _prompt(cfg, batch, seq, seed, pad_tail=0):
    rng = np.random.default_rng(seed + 100)
    hi = cfg["vocab"] - 1
    ids = rng.integers(1, hi, size=(batch, seq), dtype=np.int32)
    ids[ids == cfg["padding_id"]] = 1
    ids[ids == cfg["eos_id"]] = 1
    if pad_tail:
        ids[-1, seq - pad_tail:] = cfg["padding_id"]
    return ids


def _run_sample(path, cfg, ids, max_batch, benchmark=False):
    from lightseq_amd.inference import QuantGpt
    model = QuantGpt(path, max_batch)
    rec = torch.zeros(cfg["max_step"], ids.shape[0], cfg["vocab"], dtype=torch.int8, device=DEV)
    model.set_step_record(rec, cfg["max_step"])
    model.benchmark_mode(benchmark)
    out = model.sample(ids)
    steps = model.steps_run()
    logits = rec.cpu().numpy()[:steps]
    model.close()
    return out, steps, logits


def _check_sample(msg, cfg, ids, out, steps, logits, benchmark=False):
    w = _og().gpt_weights_from_message(msg, cfg, np.float16)
    r = _og().quant_gpt_sample(w, ids, is_benchmark=benchmark, forced_logits=logits, record=True)
    assert r["steps_run"] == steps
    np.testing.assert_array_equal(r["ids"], out)
    diff = np.abs(r["logits"].astype(np.int32) - logits.astype(np.int32))
    frac, frac2 = float((diff != 0).mean()), float((diff > 1).mean())
    print("steps %d: %.3f%% of logit codes differ, %.4f%% by more than one code, max %d" %
          (steps, 100 * frac, 100 * frac2, diff.max()))
    # every int8-output GEMM turns one flipped input code into +-1 flips on a few percent
    # of its outputs, so rows that saw a flip upstream are decorrelated at the rounding level
    # (every stage of a cached step is held to its own bar, on the GPU's own stage inputs, by
    # test_cached_step_stage_by_stage_at_gpt2_medium_width; this bounds the drift of two runs
    # that each read their own caches)
    assert diff.max() <= 4
    assert frac2 <= 1e-2 and frac <= 0.25
    return w, r


@pytest.mark.parametrize("seed,batch,seq,pad_tail", [(1, 3, 9, 0), (2, 2, 17, 4), (3, 1, 5, 0),
                                                      (4, 4, 12, 3)])
def test_tiny_gpt_sample(tmp_path, seed, batch, seq, pad_tail):
    from lightseq_amd import synthetic
    cfg = synthetic.gpt_config("tiny")
    path, msg = _make(tmp_path, cfg, seed, w_std=0.2)
    ids = _prompt(cfg, batch, seq, seed, pad_tail)
    out, steps, logits = _run_sample(path, cfg, ids, max_batch=4)
    assert out.shape[0] == batch and out.shape[1] == seq + steps
    np.testing.assert_array_equal(out[:, :seq], ids)
    w, _ = _check_sample(msg, cfg, ids, out, steps, logits)
    if pad_tail == 0:
        free = _og().quant_gpt_sample(w, ids)
        assert free["ids"].shape == out.shape
        same = float((free["ids"] == out).all(axis=1).mean())
        assert same == 1.0, "only %.0f%% of the sequences agree with the free-running oracle" % (
            100 * same)


def test_gpt_benchmark_mode_and_eos(tmp_path):
    from lightseq_amd import synthetic
    cfg = synthetic.gpt_config("tiny")
    path, msg = _make(tmp_path, cfg, 1, w_std=0.2)
    ids = _prompt(cfg, 3, 9, 1)
    out, steps, logits = _run_sample(path, cfg, ids, max_batch=3, benchmark=True)
    limit = min(cfg["max_step"], ids.shape[1] + cfg["extra_decode_length"])
    assert out.shape[1] == limit
    _check_sample(msg, cfg, ids, out, steps, logits, benchmark=True)
    # once a sequence produced <eos> it keeps producing it
    for row in out:
        hit = np.nonzero(row[ids.shape[1]:] == cfg["eos_id"])[0]
        if hit.size:
            assert (row[ids.shape[1] + hit[0]:] == cfg["eos_id"]).all()


def test_tiny_gpt_ppl(tmp_path):
    from lightseq_amd import synthetic
    from lightseq_amd.inference import QuantGpt
    cfg = synthetic.gpt_config("tiny")
    cfg["sampling_method"] = "ppl"
    path, msg = _make(tmp_path, cfg, 6, w_std=0.2)
    ids = _prompt(cfg, 3, 11, 6, pad_tail=4)
    model = QuantGpt(path, 3)
    assert model.get_output_dtype(0) == 1 and model.get_output_max_shape(0) == [3]
    got = model.ppl(ids)
    model.close()
    w = _og().gpt_weights_from_message(msg, cfg, np.float16)
    want = _og().quant_gpt_ppl(w, ids)
    assert got.shape == (3,)
    # mean log-likelihood over ~10 positions, each moved by a few flipped logit codes at most
    np.testing.assert_allclose(got, want, rtol=2e-3, atol=2e-3)


def test_gpt_interface_and_errors(tmp_path):
    from lightseq_amd import synthetic
    from lightseq_amd.inference import LSModel, QuantGpt
    from lightseq_amd.lib import LSHError
    cfg = synthetic.gpt_config("tiny")
    path, _ = _make(tmp_path, cfg, 8, w_std=0.2)
    model = QuantGpt(path, 2)
    assert model.get_input_name(0) == "token_ids" and model.get_output_name(0) == "result"
    assert model.get_input_max_shape(0) == [2, cfg["max_step"]]
    assert model.get_output_max_shape(0) == [2, cfg["max_step"]]
    assert model.get_input_dtype(0) == 2 and model.get_output_dtype(0) == 2
    a = model.sample(_prompt(cfg, 2, 7, 1))
    b = model.sample(_prompt(cfg, 2, 7, 1))
    np.testing.assert_array_equal(a, b)
    with pytest.raises(LSHError, match="max_batch_size"):
        model.sample(_prompt(cfg, 3, 5, 0))
    model.close()
    bad = dict(cfg, topk=3)
    path2 = os.path.join(str(tmp_path), "topk3.pb")
    synthetic.write_quant_gpt(path2, bad, seed=1)
    with pytest.raises(LSHError, match=r"\[1,2,4,8,16,32\].*topk = 3"):
        LSModel("QuantGpt", path2, 2)


def test_gpt2_medium_shape(tmp_path):
    """GPT-2-medium-shaped model (hidden 1024, 16 heads, inner 4096, vocabulary 50257) with
    fewer layers and a shorter prompt so that the oracle finishes in seconds."""
    from lightseq_amd import synthetic
    cfg = synthetic.gpt_config("gpt2_medium")
    cfg.update(n_layer=2, max_step=96, extra_decode_length=8)
    path, msg = _make(tmp_path, cfg, 12, w_std=0.05)
    ids = _prompt(cfg, 2, 48, 12, pad_tail=5)
    out, steps, logits = _run_sample(path, cfg, ids, max_batch=2)
    assert steps >= 1 and out.shape[1] == 48 + steps
    _check_sample(msg, cfg, ids, out, steps, logits)


GPT_TAPS_I8 = ["ln1_q", "self_q", "ctx_q", "out_q", "ln2_q", "next_ln_q"]
GPT_TAPS_F16 = ["res_in", "res_attn", "res_out"]


def _gpt_step_taps(path, cfg, ids, layer, step):
    """One sample() with every intermediate of layer `layer` at cached step `step` tapped."""
    from lightseq_amd.inference import QuantGpt
    batch = ids.shape[0]
    H, I, h = cfg["hidden"], cfg["inner"], cfg["head_num"]
    model = QuantGpt(path, batch)
    t = {n: torch.zeros(batch, H, dtype=torch.int8, device=DEV) for n in GPT_TAPS_I8}
    t.update({n: torch.zeros(batch, H, dtype=torch.float16, device=DEV) for n in GPT_TAPS_F16})
    t["act_q"] = torch.zeros(batch, I, dtype=torch.int8, device=DEV)
    t["ffn2_acc"] = torch.zeros(batch, H, dtype=torch.int32, device=DEV)
    for n in ("k_cache", "v_cache"):
        t[n] = torch.zeros(batch, h, cfg["max_step"], H // h, dtype=torch.int8, device=DEV)
    for n, buf in t.items():
        model.set_tap(layer, "dec." + n, buf)
    model.set_tap_step(step)
    model.benchmark_mode(True)   # no early stop: the tapped step is reached
    model.sample(ids)
    steps = model.steps_run()
    out = {n: buf.cpu().numpy() for n, buf in t.items()}
    model.close()
    return out, steps


def _check_gpt_step_stages(w, cfg, tp, layer, pos):
    """Every stage of one layer of a cached step (the new token sits at position `pos`) against
    the oracle's kernel for that stage, each fed the GPU's own stage input
    (model/quant_gpt_encoder.cc.cu:560-760): int8 GEMM outputs, the appended cache rows and the
    int32 FFN2 accumulator bit for bit, layer-norm and attention codes within one code on at most
    0.1 % of the elements."""
    from oracle import oracle
    Q = np.float32(127)
    c = w["clip_max"][layer * 12:(layer + 1) * 12]
    h, H = cfg["head_num"], cfg["hidden"]
    d = H // h
    W = lambda name: w[name][layer]
    eq = np.testing.assert_array_equal

    codes = oracle.gemm_i8_i8(tp["ln1_q"], W("w_qkv"), c[0] * c[4] / (c[8] * Q))
    k_c, v_c = tp["k_cache"].copy(), tp["v_cache"].copy()
    k_c[:, :, pos, :] = 99
    v_c[:, :, pos, :] = 99
    new_q = oracle.arrange_decself_qkv_i8I_i8O(codes, W("b_qkv"), k_c, v_c, pos, c[8] / Q, Q / c[11])
    eq(tp["self_q"], new_q)
    eq(tp["k_cache"][:, :, :pos + 1], k_c[:, :, :pos + 1])
    eq(tp["v_cache"][:, :, :pos + 1], v_c[:, :, :pos + 1])
    scores = oracle.decself_scores(tp["self_q"], tp["k_cache"], pos + 1)
    attn_scale = float(np.float16(np.sqrt(np.float32(1.0) / np.float32(d))))
    ctx = oracle.fuse_softmax_new_value_i32I_i8O(scores, tp["v_cache"], pos + 1, attn_scale, c[11] / Q,
                                                 Q / c[5])
    assert_codes_close(tp["ctx_q"], ctx, max_frac=1e-3, what="cached self-attention context")
    eq(tp["out_q"], oracle.gemm_i8_i8(tp["ctx_q"], W("w_out"), c[1] * c[5] / (c[9] * Q)))
    ln_q, res = oracle.residual_bias_ln_i8O(tp["out_q"], W("ln2_scale"), W("ln2_bias"), W("b_ffn2"),
                                            tp["res_in"], c[9] / Q, Q / c[6], False)
    assert_codes_close(tp["ln2_q"], ln_q, max_frac=1e-3, what="layer norm before the FFN")
    np.testing.assert_allclose(tp["res_attn"].astype(np.float32), res.astype(np.float32), atol=2e-2)

    codes = oracle.gemm_i8_i8(tp["ln2_q"], W("w_ffn1"), c[2] * c[6] / (c[10] * Q))
    eq(tp["act_q"], oracle.bias_gelu_i8I_i8O(codes, W("b_ffn1"), c[10] / Q, Q / c[7]))
    eq(tp["ffn2_acc"], oracle.gemm_i8_i32(tp["act_q"], W("w_ffn2")))
    if layer == w["n_layer"] - 1:
        sc_, bi_, rb_, clip = w["out_ln_scale"], w["out_ln_bias"], None, w["output_ln_clip_max"]
    else:
        sc_, bi_, rb_ = w["ln1_scale"][layer + 1], w["ln1_bias"][layer + 1], w["b_out"][layer + 1]
        clip = w["clip_max"][(layer + 1) * 12 + 4]
    ln_q, res = oracle.residual_bias_ln_i8O(tp["ffn2_acc"], sc_, bi_, rb_, tp["res_attn"],
                                            c[3] * c[7] / (Q * Q), Q / clip, False)
    assert_codes_close(tp["next_ln_q"], ln_q, max_frac=1e-3, what="layer norm after the FFN")
    np.testing.assert_allclose(tp["res_out"].astype(np.float32), res.astype(np.float32), atol=2e-2)


@pytest.mark.parametrize("layer", [0, 1])
def test_cached_step_stage_by_stage_at_gpt2_medium_width(tmp_path, layer):
    """One cached step of a GPT-2-medium-shaped model (hidden 1024, 16 heads, inner 4096), stage
    by stage through the step taps, at the first cached step, a middle one and the last."""
    from lightseq_amd import synthetic
    cfg = synthetic.gpt_config("gpt2_medium")
    cfg.update(n_layer=2, max_step=96, extra_decode_length=24)
    path, msg = _make(tmp_path, cfg, 12, w_std=0.05)
    prompt_len = 48
    ids = _prompt(cfg, 2, prompt_len, 12)
    w = _og().gpt_weights_from_message(msg, cfg, np.float16)
    last = None
    for step in (1, 11, -1):
        if step < 0:
            step = last
        tp, steps = _gpt_step_taps(path, cfg, ids, layer, step)
        last = steps - 1
        assert 1 <= step < steps
        assert np.abs(tp["ln1_q"]).max() > 0 and np.abs(tp["ffn2_acc"]).max() > 0
        _check_gpt_step_stages(w, cfg, tp, layer, prompt_len + step - 1)


def test_gpt2_medium_full_size_properties(tmp_path):
    """The generation benchmark at its stated size -- 24 layers, hidden 1024, 16 heads, inner
    4096, vocabulary 50257, batch 16, prompt 512, 128 generated tokens, greedy -- through
    QuantGpt.  The oracle would take minutes here, so the run is held to what must be true at
    any size: every generated token is the first arg-max of that step's recorded logits, the
    prompt is kept, the run is deterministic, and a sequence's tokens do not depend on the rest
    of its batch."""
    from lightseq_amd import synthetic
    from lightseq_amd.inference import QuantGpt
    cfg = synthetic.gpt_config("gpt2_medium")
    batch, prompt, new = 16, 512, 128
    assert cfg["n_layer"] == 24 and cfg["max_step"] >= prompt + new
    cfg.update(extra_decode_length=new)
    path, _ = _make(tmp_path, cfg, 21)
    ids = _prompt(cfg, batch, prompt, 21)
    model = QuantGpt(path, batch)
    rec = torch.zeros(new, batch, cfg["vocab"], dtype=torch.int8, device=DEV)
    model.set_step_record(rec, new)
    model.benchmark_mode(True)   # no early stop: all 128 steps run
    out = model.sample(ids)
    steps = model.steps_run()
    assert steps == new and out.shape == (batch, prompt + new)
    np.testing.assert_array_equal(out[:, :prompt], ids)
    logits = rec.cpu().numpy()
    gen = out[:, prompt:]
    eos = cfg["eos_id"]
    done = np.zeros(batch, bool)
    for t in range(steps):
        want = logits[t].astype(np.int32).argmax(axis=1)   # numpy: first maximum = lowest id
        live = ~done
        np.testing.assert_array_equal(gen[live, t], want[live], err_msg="step %d" % t)
        assert (gen[done, t] == eos).all()                  # finished rows stay on <eos>
        done |= gen[:, t] == eos
    # deterministic; the record of a second run is the same bytes
    rec2 = torch.zeros_like(rec)
    model.set_step_record(rec2, new)
    out2 = model.sample(ids)
    np.testing.assert_array_equal(out2, out)
    assert torch.equal(rec, rec2)
    # a sequence does not depend on the rest of its batch
    model.set_step_record(None, 0)
    sub = model.sample(ids[5:8])
    np.testing.assert_array_equal(sub, out[5:8])
    # the steps replayed as HIP graphs (seen, captured, replayed twice) give the same tokens
    model.graph_mode(True)
    for rep in range(4):
        np.testing.assert_array_equal(model.sample(ids), out, err_msg="graph run %d" % rep)
    captured, replayed = model.graph_stats()
    assert captured == new - 1 and replayed == 3 * captured, (captured, replayed)
    model.close()


@pytest.mark.parametrize("benchmark", [False, True])
def test_graph_replay_of_the_steps_equals_eager(tmp_path, benchmark):
    """Steps replayed as HIP graphs give the eager run's tokens: several replays, with eager work
    of this program (another batch shape, a torch kernel, synchronisations) between them."""
    from lightseq_amd import synthetic
    from lightseq_amd.inference import QuantGpt
    cfg = synthetic.gpt_config("tiny")
    path, _ = _make(tmp_path, cfg, 5, w_std=0.2)
    ids = _prompt(cfg, 3, 9, 5)
    other = _prompt(cfg, 2, 6, 6)
    model = QuantGpt(path, 4)
    model.benchmark_mode(benchmark)
    want, want_other = model.sample(ids), model.sample(other)
    steps = model.steps_run()
    model.graph_mode(True)
    scratch = torch.zeros(1 << 16, device=DEV)
    for rep in range(5):       # 1st: eager (keys seen), 2nd: capture + launch, then replays
        got = model.sample(ids)
        np.testing.assert_array_equal(got, want, err_msg="replay %d" % rep)
        scratch.add_(1.0)
        torch.cuda.synchronize()
        if rep % 2 == 0:
            np.testing.assert_array_equal(model.sample(other), want_other)
    captured, replayed = model.graph_stats()
    assert captured >= 1 and replayed >= 3 * captured, (captured, replayed)
    # recording switches the graphs off and still gives the same tokens
    rec = torch.zeros(cfg["max_step"], 3, cfg["vocab"], dtype=torch.int8, device=DEV)
    model.set_step_record(rec, cfg["max_step"])
    np.testing.assert_array_equal(model.sample(ids), want)
    assert model.graph_stats()[1] == replayed
    assert model.graph_nodes() >= 7 * cfg["n_layer"]
    prepare_ms, steps_ms, loop_steps = model.phase_times()
    assert loop_steps == model.steps_run() - 1 and steps_ms > 0 and prepare_ms > 0
    model.graph_mode(False)
    model.set_step_record(None, 0)
    np.testing.assert_array_equal(model.sample(ids), want)
    assert steps >= 1
    model.close()
