"""Pins the decoder half of the CPU oracle with checks that do not restate its code:
library routines (numpy integer matmul, scipy softmax / log_softmax in float64), a literal
lane-by-lane simulation of the reference's shuffle network, brute-force top-k over all
candidates, layout identities written as reshapes / transposes, and invariants of the whole
decoder (greedy = arg-max of its own logits, batch invariance, replay of its own logits).
"""
import numpy as np
import pytest
from scipy.special import log_softmax, softmax

from conftest import assert_codes_close


def _codes(rng, shape):
    return rng.integers(-127, 128, size=shape, dtype=np.int8)


def _quant(x, qs):
    """float array -> int8 codes, numpy float32 arithmetic."""
    y = np.floor(x.astype(np.float32) * np.float32(qs) + np.float32(0.5))
    return np.clip(y, -127, 127).astype(np.int8)


# --------------------------------------------------------------------------- #
# embedding and layout kernels
# --------------------------------------------------------------------------- #
@pytest.mark.parametrize("dtype", [np.float16, np.float32])
def test_dec_emb(oracle, rng, dtype):
    rows, hidden, vocab, max_step, step = 6, 40, 30, 8, 5
    table = _codes(rng, (hidden, vocab))
    pos = (rng.standard_normal((max_step, hidden)) * 0.1).astype(dtype)
    tokens = rng.integers(0, vocab, size=(rows, max_step), dtype=np.int32)
    dq = np.float32(0.08 / 127)
    a = oracle.dec_emb_i8I(table, pos, tokens, step, dq, True, False)
    b = oracle.dec_emb_i8I(np.ascontiguousarray(table.T), pos, tokens, step, dq, True, True)
    np.testing.assert_array_equal(a, b)  # the two table layouts hold the same matrix
    scale = np.float32(dq * np.sqrt(np.float32(hidden)))
    want = (table.T[tokens[:, step]].astype(np.float32) * scale +
            pos[step].astype(np.float32)[None, :]).astype(dtype)
    np.testing.assert_array_equal(a, want)
    c = oracle.dec_emb_i8I(table, pos, tokens, step, dq, False, False)
    want_c = (table.T[tokens[:, step]].astype(np.float32) * dq + pos[step].astype(np.float32)).astype(dtype)
    np.testing.assert_array_equal(c, want_c)


@pytest.mark.parametrize("dtype", [np.float16, np.float32])
def test_arrange_decself_qkv(oracle, rng, dtype):
    rows, heads, d, max_step, step = 5, 3, 8, 6, 4
    H = heads * d
    ori = _codes(rng, (rows, 3 * H))
    bias = (rng.standard_normal(3 * H) * 0.5).astype(dtype)
    k0, v0 = _codes(rng, (rows, heads, max_step, d)), _codes(rng, (rows, heads, max_step, d))
    k, v = k0.copy(), v0.copy()
    dq, qs = np.float32(3.0 / 127), np.float32(127 / 2.5)
    q = oracle.arrange_decself_qkv_i8I_i8O(ori, bias, k, v, step, dq, qs)
    val = ori.astype(np.float32) * dq + bias.astype(np.float32)[None, :]
    codes = _quant(val, qs).reshape(rows, 3, heads, d)
    np.testing.assert_array_equal(q, codes[:, 0].reshape(rows, H))
    np.testing.assert_array_equal(k[:, :, step], codes[:, 1])
    np.testing.assert_array_equal(v[:, :, step], codes[:, 2])
    keep = np.arange(max_step) != step
    np.testing.assert_array_equal(k[:, :, keep], k0[:, :, keep])
    np.testing.assert_array_equal(v[:, :, keep], v0[:, :, keep])


def test_decself_scores_are_integer_matmul(oracle, rng):
    rows, heads, d, max_step, step_num = 4, 3, 16, 12, 9
    q = _codes(rng, (rows, heads * d))
    k = _codes(rng, (rows, heads, max_step, d))
    got = oracle.decself_scores(q, k, step_num)
    want = np.einsum("rhd,rhjd->rhj", q.reshape(rows, heads, d).astype(np.int64),
                     k.astype(np.int64)).reshape(rows * heads, max_step)
    np.testing.assert_array_equal(got[:, :step_num], want[:, :step_num])
    assert not got[:, step_num:].any()


def test_fuse_softmax_new_value_vs_float64(oracle, rng):
    rows, heads, d, max_step, step_num = 6, 4, 16, 40, 33
    v = _codes(rng, (rows, heads, max_step, d))
    logits = rng.integers(-40000, 40000, size=(rows * heads, max_step), dtype=np.int32)
    dq, attn_scale, qs = 4.0 / 127, 0.25, 127 / 1.5
    got = oracle.fuse_softmax_new_value_i32I_i8O(logits, v, step_num, attn_scale, dq, qs)
    p = softmax(logits[:, :step_num].astype(np.float64) * dq * dq * attn_scale, axis=-1)
    ctx = np.einsum("bj,bjd->bd", p, v.reshape(rows * heads, max_step, d)[:, :step_num].astype(np.float64)) * dq
    want = np.clip(np.floor(ctx * qs + 0.5), -127, 127).astype(np.int8).reshape(rows, heads * d)
    assert_codes_close(got, want, max_frac=3e-3, what="new value vs float64")
    # one step: the softmax is 1 and the output is the requantised value itself
    one = oracle.fuse_softmax_new_value_i32I_i8O(logits, v, 1, attn_scale, dq, qs)
    np.testing.assert_array_equal(one, _quant(v[:, :, 0].astype(np.float32) * np.float32(dq), qs).reshape(rows, -1))


@pytest.mark.parametrize("dtype", [np.float16, np.float32])
def test_encdec_layouts(oracle, rng, dtype):
    batch, seq, layers, heads, d, beam = 2, 5, 3, 2, 4, 3
    H = heads * d
    ori = rng.standard_normal((batch * seq, layers, 2, H)).astype(dtype)
    bias = (rng.standard_normal((layers, 2, H)) * 0.3).astype(dtype)
    k, v = oracle.arrange_encdec_kv(ori, bias, batch, seq, layers, heads)
    s = (ori.astype(np.float32) + bias.astype(np.float32)[None]).astype(dtype)
    s = s.reshape(batch, seq, layers, 2, heads, d).transpose(2, 3, 0, 4, 1, 5)  # l, kv, b, h, s, d
    np.testing.assert_array_equal(k, s[:, 0])
    np.testing.assert_array_equal(v, s[:, 1])

    rows = batch * beam
    oq = _codes(rng, (rows, H))
    qb = (rng.standard_normal(H) * 0.5).astype(dtype)
    dq = np.float32(3.0 / 127)
    got = oracle.arrange_encdec_q_i8I(oq, qb, beam, heads, dq)
    if dtype == np.float16:  # half(code*dq) + bias as a half add
        val = ((oq.astype(np.float32) * dq).astype(np.float16).astype(np.float32) +
               qb.astype(np.float32)).astype(np.float16)
    else:
        val = oq.astype(np.float32) * dq + qb
    want = val.reshape(batch, beam, heads, d).transpose(0, 2, 1, 3)
    np.testing.assert_array_equal(got, want)


def test_encdec_attention_chain_vs_float64(oracle, rng):
    batch, heads, beam, seq, d = 2, 3, 4, 11, 16
    bh = batch * heads
    q = rng.standard_normal((bh, beam, d)).astype(np.float16)
    k = rng.standard_normal((bh, seq, d)).astype(np.float16)
    v = rng.standard_normal((bh, seq, d)).astype(np.float16)
    lens = np.array([seq, 6])
    mask = (np.arange(seq)[None, :] >= lens[:, None]).astype(np.int32)
    sc = oracle.attn_scores_rect(q, k, float(np.sqrt(1.0 / d)))
    pr = oracle.correlation_softmax_encdec(sc.reshape(batch, heads * beam, seq), mask)
    ctx = oracle.attn_context_rect(pr.reshape(bh, beam, seq), v)
    s64 = np.einsum("bid,bjd->bij", q.astype(np.float64), k.astype(np.float64)) / np.sqrt(d)
    s64 = s64.reshape(batch, heads * beam, seq)
    s64 = np.where(mask[:, None, :] != 0, -np.inf, s64)
    p64 = softmax(s64, axis=-1)
    c64 = np.einsum("bij,bjd->bid", p64.reshape(bh, beam, seq), v.astype(np.float64))
    np.testing.assert_allclose(pr.astype(np.float64), p64, atol=2e-3)
    np.testing.assert_allclose(ctx.astype(np.float64), c64, atol=6e-3)
    assert not pr[1, :, 6:].any()


def test_gemm_T(oracle, rng):
    a = rng.standard_normal((9, 32)).astype(np.float16)
    b = (rng.standard_normal((32, 21)) * 0.1).astype(np.float16)
    got = oracle.gemm_T(a, b)
    want = (a.astype(np.float64) @ b.astype(np.float64)).astype(np.float16)
    np.testing.assert_array_equal(got, want)
    a32, b32 = a.astype(np.float32), b.astype(np.float32)
    np.testing.assert_allclose(oracle.gemm_T(a32, b32), a32.astype(np.float64) @ b32, rtol=1e-6)


# --------------------------------------------------------------------------- #
# beam search
# --------------------------------------------------------------------------- #
def test_length_norm(oracle):
    for length in (1, 2, 7, 64):
        assert abs(oracle.length_norm(length, 0.6) - ((5 + length) / 6.0) ** -0.6) < 1e-6
        assert oracle.length_norm(length, 0.0) == 1.0
        assert oracle.length_norm(length, -1.0) == np.float32(1.0) / np.float32(length)


def _rough_threshold_by_lanes(lgt, threads, K):
    """inference/kernels/common.h:118-137 executed lane by lane for a block of `threads`
    threads, thread t owning the vocabulary ids congruent to t."""
    NEG = np.float32(-100000000.0)
    tmax = np.full(threads, NEG, np.float32)
    for vid, x in enumerate(lgt):
        t = vid % threads
        tmax[t] = max(tmax[t], x)
    shared = np.zeros(32, np.float32)
    for w in range(threads // 32):
        shared[w] = tmax[w * 32:(w + 1) * 32].max()
    # warp 0 after the broadcast load
    val = np.array([shared[l] if l < (threads >> 5) else np.float32(0) for l in range(32)],
                   np.float32)
    m = 16
    while m >= K:
        val = np.array([max(val[l], val[l ^ m]) for l in range(32)], np.float32)
        m >>= 1
    m = K >> 1
    while m > 0:
        val = np.array([min(val[l], val[l ^ m]) for l in range(32)], np.float32)
        m >>= 1
    return val[0]


def _beam_inputs(rng, batch, beam, vocab, max_step, cur_step, end_id, finished=()):
    rows = batch * beam
    logits = np.clip(rng.standard_normal((rows, vocab)) * 32, -127, 127).astype(np.int8)
    bias = (rng.standard_normal(vocab) * 0.05).astype(np.float16)
    alive = rng.integers(4, vocab, size=(rows, max_step), dtype=np.int32)
    for r in finished:
        alive[r, cur_step] = end_id
    probs = (-rng.random(rows) * 5).astype(np.float32)
    if cur_step == 0:
        probs = np.where(np.arange(rows) % beam == 0, 0.0, -1000.0).astype(np.float32)
    score = (-rng.random(rows) * 8 - 2000.0 * (np.arange(rows) // beam)).astype(np.float32)
    return logits, bias, probs, score, alive


@pytest.mark.parametrize("threads,beam,vocab", [(1024, 4, 3000), (1024, 8, 700), (256, 2, 1000),
                                                 (64, 16, 500), (1024, 1, 2000), (1024, 32, 4000)])
def test_select_candidates_match_shuffle_network(oracle, rng, threads, beam, vocab):
    batch, max_step, cur_step, end_id = 2, 8, 3, 3
    logits, bias, probs, score, alive = _beam_inputs(rng, batch, beam, vocab, max_step, cur_step,
                                                     end_id, finished=(1,))
    dq = np.float32(2.5 / 127)
    ln = oracle.length_norm(cur_step + 1, 0.6)
    idx, sc, num = oracle.select_beam_rough_topk_i8I(logits, bias, probs, score, alive, dq, ln,
                                                     cur_step, threads, beam, end_id)
    assert num[0] == idx.size == num[1:].sum()
    pos = 0
    for row in range(batch * beam):
        n = num[1 + row]
        b, j = divmod(row, beam)
        if row == 1:  # finished beam: one <eos> candidate carrying its score
            assert n == 1 and idx[pos] == end_id + j * vocab and sc[pos] == score[row]
            pos += n
            continue
        lgt = logits[row].astype(np.float32) * dq + bias.astype(np.float32)
        thr = _rough_threshold_by_lanes(lgt, threads, beam)
        want = np.nonzero(lgt >= thr)[0]
        np.testing.assert_array_equal(idx[pos:pos + n] - j * vocab, want)
        assert n >= beam  # "rough but safe": never fewer than beam_size candidates
        # scores: (prefix log-prob + log_softmax) * length_norm + batch offset
        lp = log_softmax(lgt.astype(np.float64))
        want_sc = (probs[row] + lp[want]) * ln - 2000.0 * b
        np.testing.assert_allclose(sc[pos:pos + n], want_sc, rtol=1e-6, atol=1e-3)
        pos += n


def test_scan_sort(oracle, rng):
    num = np.array([0, 3, 1, 4, 2], np.int32)
    num[0] = num[1:].sum()
    idx = rng.integers(0, 1000, size=num[0]).astype(np.int32)
    sc = rng.choice(np.array([-1.0, -2.0, -3.5, -7.25], np.float32), size=num[0])  # many ties
    s_idx, s_sc, s_num = oracle.scan_sort_candidates(idx, sc, num)
    order = np.argsort(-sc, kind="stable")
    np.testing.assert_array_equal(s_sc, sc[order])
    np.testing.assert_array_equal(s_idx, idx[order])
    np.testing.assert_array_equal(s_num[1:], np.cumsum(num[1:]) - num[1:])
    assert s_num[0] == num[0]


@pytest.mark.parametrize("cur_step,finished", [(0, ()), (3, ()), (5, (0, 5, 6)), (2, (0, 1, 2, 3))])
def test_search_step_is_exact_topk(oracle, rng, cur_step, finished):
    """select + sort + refresh picks, per sentence, the beam_size best of all
    beam_size * vocab continuations by total log-probability (float64 brute force)."""
    batch, beam, vocab, max_step, end_id = 2, 4, 600, 10, 3
    logits, bias, probs, score, alive = _beam_inputs(rng, batch, beam, vocab, max_step, cur_step,
                                                     end_id, finished=finished)
    dq = np.float32(2.5 / 127)
    ln = oracle.length_norm(cur_step + 1, 0.6)
    idx, sc, num = oracle.select_beam_rough_topk_i8I(logits, bias, probs, score, alive, dq, ln,
                                                     cur_step, 1024, beam, end_id)
    s_idx, s_sc, s_num = oracle.scan_sort_candidates(idx, sc, num)
    new_alive, new_probs, new_score, fin = oracle.refresh_result(
        s_idx, s_sc, s_num, alive, probs, score, vocab, cur_step, ln, end_id, beam)
    n_fin = 0
    for b in range(batch):
        cands = []  # (total score, parent beam, token)
        for j in range(beam):
            row = b * beam + j
            if cur_step != 0 and alive[row, cur_step] == end_id:
                cands.append((float(score[row]) + 2000.0 * b, j, end_id))
                continue
            lgt = logits[row].astype(np.float64) * float(dq) + bias.astype(np.float64)
            tot = (float(probs[row]) + log_softmax(lgt)) * float(ln)
            cands += [(tot[t], j, t) for t in range(vocab)]
        cands.sort(key=lambda c: -c[0])
        for j in range(beam):
            tot, parent, tok = cands[j]
            row = b * beam + j
            assert new_alive[row, cur_step + 1] == tok
            np.testing.assert_array_equal(new_alive[row, :cur_step + 1],
                                          alive[b * beam + parent, :cur_step + 1])
            assert (new_alive[row, cur_step + 2:] == end_id).all()
            if tok == end_id:
                n_fin += 1
                assert abs(new_score[row] + 2000.0 * b - tot) < 2e-3
                assert new_probs[row] == probs[row]  # untouched
            else:
                assert abs(new_probs[row] - tot / float(ln)) < 2e-3
                assert new_score[row] == score[row]
    assert fin == n_fin


def test_refresh_cache_is_a_gather(oracle, rng):
    layers, batch, beam, heads, max_step, d, vocab, end_id, cur_step = 2, 2, 4, 2, 6, 8, 50, 3, 3
    rows = batch * beam
    shape = (layers, rows, heads, max_step, d)
    k_old, v_old = _codes(rng, shape), _codes(rng, shape)
    k_new, v_new = _codes(rng, shape), _codes(rng, shape)
    k0, v0 = k_new.copy(), v_new.copy()
    parents = rng.integers(0, beam, size=rows)
    toks = rng.integers(4, vocab, size=rows)
    toks[[1, 6]] = end_id
    # two candidates per row; each sentence's winners sit first in its segment
    num = np.zeros(rows + 1, np.int32)
    num[1:] = np.arange(rows) * 2
    num[0] = rows * 2
    can_idx = np.zeros(rows * 2, np.int32)
    for b in range(batch):
        for j in range(beam):
            can_idx[num[1 + b * beam] + j] = parents[b * beam + j] * vocab + toks[b * beam + j]
    oracle.refresh_cache_i8(num, can_idx, k_old, v_old, k_new, v_new, beam, vocab, cur_step, end_id)
    for row in range(rows):
        b = row // beam
        src = b * beam + parents[row]
        if toks[row] == end_id:  # finished beams keep whatever the new buffer held
            np.testing.assert_array_equal(k_new[:, row], k0[:, row])
            continue
        np.testing.assert_array_equal(k_new[:, row, :, :cur_step + 1], k_old[:, src, :, :cur_step + 1])
        np.testing.assert_array_equal(v_new[:, row, :, :cur_step + 1], v_old[:, src, :, :cur_step + 1])
        np.testing.assert_array_equal(k_new[:, row, :, cur_step + 1:], k0[:, row, :, cur_step + 1:])
        np.testing.assert_array_equal(v_new[:, row, :, cur_step + 1:], v0[:, row, :, cur_step + 1:])


def test_output_writers(oracle, rng):
    batch, beam, max_step, out_len, end_id = 3, 4, 12, 7, 3
    rows = batch * beam
    alive = rng.integers(0, 6, size=(rows, max_step), dtype=np.int32)
    score = (-rng.random(rows) * 20 - 2000.0 * (np.arange(rows) // beam)).astype(np.float32)
    out, sc = oracle.write_trg_tokenid_pos_penalty(alive, score, beam, out_len)
    np.testing.assert_array_equal(out, alive[::beam, 1:out_len + 1])
    np.testing.assert_allclose(sc[:batch], score[::beam] + 2000.0 * np.arange(batch), atol=1e-3)
    out = oracle.write_trg_tokenid_neg_penalty(alive, score, beam, end_id, out_len)
    for b in range(batch):
        rec = score[b * beam:(b + 1) * beam].astype(np.float64) + 2000.0 * b
        lens = (alive[b * beam:(b + 1) * beam, 1:out_len + 1] != end_id).sum(axis=1)
        best = int(np.argmax(rec / (lens + 1e-12)))
        np.testing.assert_array_equal(out[b], alive[b * beam + best, 1:out_len + 1])
    out, sc = oracle.write_topk_result(alive, score, beam, end_id, out_len)
    np.testing.assert_array_equal(out[:, :-1], alive[:, 1:out_len])
    assert (out[:, -1] == end_id).all()
    np.testing.assert_allclose(sc, score + 2000.0 * (np.arange(rows) // beam), atol=1e-3)


# --------------------------------------------------------------------------- #
# whole decoder: invariants of the orchestration
# --------------------------------------------------------------------------- #
def _tiny_model(seed, **over):
    from lightseq_amd import synthetic
    from oracle import model_io
    cfg = synthetic.transformer_config("tiny")
    cfg.update(over)
    sigma = 0.02 * np.sqrt(cfg["hidden"])
    msg = synthetic.make_quant_transformer(cfg, seed=seed, eos_bias=2.5 * sigma, w_std=0.2)
    enc_w, dec_w = model_io.oracle_transformer_weights_from_message(msg, cfg, np.float16)
    ids, _ = synthetic.make_token_ids(dict(vocab=cfg["src_vocab"], padding_id=0), 3, 9, seed=seed)
    return cfg, enc_w, dec_w, ids


def test_decoder_greedy_follows_its_logits(oracle):
    cfg, enc_w, dec_w, ids = _tiny_model(3, beam_size=1, length_penalty=-1.0)
    enc_out, mask, _ = oracle.quant_bert_encoder(enc_w, ids)
    r = oracle.quant_decoder(dec_w, enc_out, mask, record=True)
    dq = np.float32(dec_w["logits_clip_max"]) / np.float32(127)
    bias = dec_w["logit_bias"].astype(np.float32)
    done = np.zeros(ids.shape[0], bool)
    for t in range(r["steps_run"]):
        lgt = r["logits"][t].astype(np.float32) * dq + bias[None, :]
        tok = r["alive_seq"][t][:, t + 1]
        want = np.where(done, dec_w["end_id"], lgt.argmax(axis=1))
        np.testing.assert_array_equal(tok, want)
        done |= tok == dec_w["end_id"]
    # the running log-probability is the sum of the chosen log-softmax terms
    lp = np.zeros(ids.shape[0])
    alive_mask = np.ones(ids.shape[0], bool)
    for t in range(min(3, r["steps_run"])):
        lgt = r["logits"][t].astype(np.float64) * float(dq) + bias.astype(np.float64)
        tok = r["alive_seq"][t][:, t + 1]
        lp += log_softmax(lgt, axis=1)[np.arange(len(tok)), tok]
        alive_mask &= tok != dec_w["end_id"]
        np.testing.assert_allclose(r["seq_probs"][t][alive_mask], lp[alive_mask], atol=2e-3)


def test_decoder_batch_invariance_and_replay(oracle):
    cfg, enc_w, dec_w, ids = _tiny_model(5)
    enc_out, mask, _ = oracle.quant_bert_encoder(enc_w, ids)
    full = oracle.quant_decoder(dec_w, enc_out, mask, record=True, is_benchmark=True)
    one = oracle.quant_decoder(dec_w, enc_out[1:2], mask[1:2], is_benchmark=True)
    np.testing.assert_array_equal(one["ids"][0], full["ids"][1])
    # feeding a run its own logits back changes nothing
    again = oracle.quant_decoder(dec_w, enc_out, mask, forced_logits=full["logits"], record=True,
                                 is_benchmark=True)
    np.testing.assert_array_equal(again["ids"], full["ids"])
    np.testing.assert_array_equal(again["alive_seq"], full["alive_seq"])
    # early stop only shortens the output
    short = oracle.quant_decoder(dec_w, enc_out, mask)
    n = short["ids"].shape[2]
    if short["early_stopped"]:
        np.testing.assert_array_equal(short["ids"], full["ids"][:, :, :n])
        assert (full["ids"][:, :, n:] == dec_w["end_id"]).all()
    else:
        np.testing.assert_array_equal(short["ids"], full["ids"])


def test_decoder_rejects_bad_shapes(oracle):
    cfg, enc_w, dec_w, ids = _tiny_model(1)
    enc_out = np.zeros((1, cfg["max_step"] + 1, cfg["hidden"]), np.float16)
    mask = np.zeros((1, cfg["max_step"] + 1), np.int32)
    with pytest.raises(RuntimeError):
        oracle.quant_decoder(dec_w, enc_out, mask)
