"""Pins the GPT half of the CPU oracle with checks that do not restate its code: numpy /
scipy library routines in float64, layout identities, closed forms, and the consistency of
the two attention routes of the model (prompt pass vs cached step)."""
import numpy as np
import pytest
from scipy.special import log_softmax, softmax

from conftest import assert_codes_close


def _og():
    from oracle import gpt
    return gpt


def _codes(rng, shape):
    return rng.integers(-127, 128, size=shape, dtype=np.int8)


@pytest.mark.parametrize("dtype", [np.float16, np.float32])
def test_gpt_embedding(rng, dtype):
    batch, seq, hidden, vocab, offset, pad = 3, 6, 24, 40, 5, 0
    table = _codes(rng, (vocab, hidden))
    pos = (rng.standard_normal((seq + offset, hidden)) * 0.1).astype(dtype)
    ids = rng.integers(1, vocab, size=(batch, seq), dtype=np.int32)
    ids[1, 4:] = pad
    dq = np.float32(0.08 / 127)
    out, rsl = _og().gpt_embedding_i8I(table, pos, ids, np.array([2, 0, 7], np.int32), pad, offset, dq)
    want = (table[ids].astype(np.float32) * dq +
            pos[offset:offset + seq].astype(np.float32)[None]).astype(dtype)
    want[ids == pad] = 0
    np.testing.assert_array_equal(out, want)
    np.testing.assert_array_equal(rsl, np.array([2 + 6, 0 + 4, 7 + 6]))


def test_scores_and_causal_softmax(rng):
    batch, heads, seq, d = 2, 3, 9, 8
    bh = batch * heads
    q, k = _codes(rng, (bh, seq, d)), _codes(rng, (bh, seq, d))
    sc = _og().gpt_scores_i8(q, k)
    np.testing.assert_array_equal(sc, np.einsum("bid,bjd->bij", q.astype(np.int64), k.astype(np.int64)))
    rsl = np.array([seq, 5], np.int32)
    dq, a = 4.0 / 127, 0.35
    pr = _og().correlation_softmax_gpt_i32I(sc, rsl, heads, a, dq, np.float32)
    x = sc.astype(np.float64) * a * dq * dq
    x = np.where(np.triu(np.ones((seq, seq), bool), 1)[None], -np.inf, x)
    want = softmax(x, axis=-1).reshape(batch, heads, seq, seq)
    want[1, :, 5:, :] = 0  # queries at or beyond the real length
    np.testing.assert_allclose(pr.reshape(want.shape), want, atol=2e-6)
    pr16 = _og().correlation_softmax_gpt_i32I(sc, rsl, heads, a, dq, np.float16)
    np.testing.assert_allclose(pr16.astype(np.float64).reshape(want.shape), want, atol=1e-3)


@pytest.mark.parametrize("dtype", [np.float16, np.float32])
@pytest.mark.parametrize("dst,src", [(1, 7), (4, 9), (6, 6)])
def test_attention_mask_weights(rng, dtype, dst, src):
    """The last `dst` queries over `src` keys against scipy's soft-max in float64 with the mask
    written independently (key j visible to query i iff j <= i + src - dst); queries at or
    beyond the real length keep what the output buffer held."""
    batch, heads = 3, 2
    corr = rng.integers(-40000, 40000, size=(batch, heads * dst, src)).astype(np.int32)
    rsl = np.array([src, max(src - dst + 1, 1), src - 1], np.int32)
    attn_scale, dq = np.float32(0.125), np.float32(2.0 / 127)
    out = np.full(corr.shape, 7.0, dtype)
    _og().attention_mask_weights_i32I(corr, rsl, heads, dst, attn_scale, dq, out)
    x = corr.astype(np.float64) * float(attn_scale) * float(dq) * float(dq)
    qpos = (np.arange(heads * dst) % dst) + src - dst
    visible = np.arange(src)[None, :] <= qpos[:, None]
    want = softmax(np.where(visible[None], x, -np.inf), axis=-1)
    assert (qpos < rsl[0]).all() and not (qpos < rsl[2]).all()
    for b in range(batch):
        live = qpos < rsl[b]
        tol = 2e-3 if dtype == np.float16 else 1e-6
        np.testing.assert_allclose(out[b][live].astype(np.float64), want[b][live], atol=tol)
        assert np.all(out[b][live][~visible[live]] == 0)
        assert np.all(out[b][~live] == 7.0)
    # a dropped scale factor or a shifted mask fails: one-hot rows where one key dominates
    corr2 = np.zeros((1, dst, src), np.int32)
    corr2[0, :, 0] = 30_000_000
    out2 = np.zeros(corr2.shape, np.float32)
    _og().attention_mask_weights_i32I(corr2, np.array([src], np.int32), 1, dst, attn_scale, dq, out2)
    np.testing.assert_allclose(out2[0, :, 0], 1.0, atol=1e-6)


@pytest.mark.parametrize("dtype", [np.float16, np.float32])
def test_arrange_qkv_with_cache(rng, dtype):
    batch, heads, old_len, d = 2, 3, 4, 8
    H = heads * d
    ori = _codes(rng, (batch, 3 * H))
    bias = (rng.standard_normal(3 * H) * 0.5).astype(dtype)
    kc, vc = _codes(rng, (batch, heads, old_len, d)), _codes(rng, (batch, heads, old_len, d))
    dq, qs = np.float32(3.0 / 127), np.float32(127 / 2.5)
    nq, nk, nv = _og().arrange_qkv_with_cache_i8I_i8O(ori, bias, kc, vc, dq, qs)
    val = ori.astype(np.float32) * dq + bias.astype(np.float32)[None]
    codes = np.clip(np.floor(val * qs + np.float32(0.5)), -127, 127).astype(np.int8)
    codes = codes.reshape(batch, 3, heads, 1, d)
    np.testing.assert_array_equal(nq, codes[:, 0])
    np.testing.assert_array_equal(nk, np.concatenate([kc, codes[:, 1]], axis=2))
    np.testing.assert_array_equal(nv, np.concatenate([vc, codes[:, 2]], axis=2))


def test_greedy_is_first_argmax(rng):
    batch, seq, vocab, eos = 5, 4, 90, 7
    logits = np.clip(rng.standard_normal((batch, vocab)) * 30, -127, 127).astype(np.int8)
    logits[0, [11, 50, 80]] = 127
    logits[3, eos] = 127
    logits[3, :eos] = -9
    old = rng.integers(8, vocab, size=(batch, seq), dtype=np.int32)
    old[2, -1] = eos
    new, last, unf = _og().topk_sample_i8I_greedy(logits, old, 1, eos, 0.02)
    want = logits.argmax(axis=1)
    want[2] = eos
    np.testing.assert_array_equal(last, want)
    np.testing.assert_array_equal(new[:, :seq], old)
    np.testing.assert_array_equal(new[:, seq], want)
    assert last[0] == 11 and last[3] == eos and unf == 1
    # everything ended or sampling <eos>: nothing unfinished
    old[:, -1] = eos
    _, last, unf = _og().topk_sample_i8I_greedy(logits, old, 1, eos, 0.02)
    assert (last == eos).all() and unf == 0


def test_ppl_is_mean_nll(rng):
    batch, seq, vocab = 3, 7, 50
    logits = np.clip(rng.standard_normal((batch * seq, vocab)) * 30, -127, 127).astype(np.int8)
    ids = rng.integers(0, vocab, size=(batch, seq), dtype=np.int32)
    rsl = np.array([7, 4, 1], np.int32)
    dq = 0.03
    got = _og().ppl_i8I(logits, ids, rsl, dq)
    lp = log_softmax(logits.astype(np.float64).reshape(batch, seq, vocab) * dq, axis=-1)
    for b in range(batch):
        n = rsl[b] - 1
        want = -np.mean([lp[b, s, ids[b, s + 1]] for s in range(n)]) if n > 0 else 0.0
        assert abs(got[b] - want) < 1e-4
    # uniform logits: the perplexity exponent is log(vocab)
    flat = np.zeros((seq, vocab), np.int8)
    got = _og().ppl_i8I(flat, ids[:1], np.array([seq], np.int32), dq)
    assert abs(got[0] - np.log(vocab)) < 1e-5


def _tiny(seed, **over):
    from lightseq_amd import synthetic
    cfg = synthetic.gpt_config("tiny")
    cfg.update(over)
    msg = synthetic.make_quant_gpt(cfg, seed=seed, w_std=0.2)
    return cfg, _og().gpt_weights_from_message(msg, cfg, np.float16)


def test_cached_step_matches_prompt_pass():
    """The logits a cached step gives for position n equal, up to the different rounding
    points of the two attention routes, the logits of a prompt pass over the n+1 tokens."""
    cfg, w = _tiny(2)
    rng = np.random.default_rng(5)
    ids = rng.integers(1, cfg["vocab"] - 1, size=(2, 8), dtype=np.int32)
    a = _og().quant_gpt_sample(w, ids, is_benchmark=True, record=True)
    k = 3
    longer = a["ids"][:, :ids.shape[1] + k].astype(np.int32)
    b = _og().quant_gpt_sample(w, np.ascontiguousarray(longer), is_benchmark=True, record=True)
    diff = np.abs(a["logits"][k].astype(np.int32) - b["logits"][0].astype(np.int32))
    # the routes round differently (fp16 probabilities and values in the prompt pass, float
    # in the cached step) and every requantisation amplifies that: a few codes out of a
    # spread of ~32 codes, against ~45 codes between unrelated logit rows
    assert diff.max() <= 8 and diff.mean() < 1.5, (diff.max(), diff.mean())
    corr = np.corrcoef(a["logits"][k].astype(np.float64).ravel(),
                       b["logits"][0].astype(np.float64).ravel())[0, 1]
    assert corr > 0.995, corr
    # and the continuation is the same text
    n = min(a["ids"].shape[1], b["ids"].shape[1])
    assert (a["ids"][:, :n] == b["ids"][:, :n]).mean() > 0.9


def test_sample_invariants():
    cfg, w = _tiny(3)
    rng = np.random.default_rng(6)
    ids = rng.integers(1, cfg["vocab"] - 1, size=(3, 6), dtype=np.int32)
    full = _og().quant_gpt_sample(w, ids, is_benchmark=True, record=True)
    limit = min(cfg["max_step"], ids.shape[1] + cfg["extra_decode_length"])
    assert full["ids"].shape == (3, limit) and full["steps_run"] == limit - ids.shape[1]
    np.testing.assert_array_equal(full["ids"][:, :6], ids)
    # greedy: every generated token is the first arg-max of the recorded logits
    for t in range(full["steps_run"]):
        prev = full["ids"][:, 6 + t - 1]
        want = np.where(prev == cfg["eos_id"], cfg["eos_id"], full["logits"][t].argmax(axis=1))
        np.testing.assert_array_equal(full["ids"][:, 6 + t], want)
    # sequences are independent
    one = _og().quant_gpt_sample(w, ids[1:2], is_benchmark=True)
    np.testing.assert_array_equal(one["ids"][0], full["ids"][1])
    # replaying a run's own logits changes nothing
    again = _og().quant_gpt_sample(w, ids, is_benchmark=True, forced_logits=full["logits"])
    np.testing.assert_array_equal(again["ids"], full["ids"])


def test_ppl_model_close_to_uniform_for_random_weights():
    cfg, w = _tiny(4)
    rng = np.random.default_rng(7)
    ids = rng.integers(1, cfg["vocab"] - 1, size=(2, 12), dtype=np.int32)
    ppl = _og().quant_gpt_ppl(w, ids)
    assert ppl.shape == (2,) and np.all(np.abs(ppl - np.log(cfg["vocab"])) < 1.0)
