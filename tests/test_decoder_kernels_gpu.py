"""GPU parity: decoder-step and beam-search kernels against the CPU oracle, called
through the C ABI, on seeded inputs.

Bars: integer work (cache writes, int32 scores, sequence / cache refresh, token
output, candidate sets) bit-exact; int8 activations within +-1 code on <= 0.1 % of the
elements; fp16 / fp32 values within the tolerance written in each test.
"""
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


def _randT(rng, shape, dtype, scale=1.0):
    return (rng.standard_normal(shape) * scale).astype(dtype)


def _codes(rng, shape):
    return rng.integers(-127, 128, size=shape, dtype=np.int8)


# --------------------------------------------------------------------------- #
# embedding
# --------------------------------------------------------------------------- #
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("vocab_major", [False, True])
@pytest.mark.parametrize("batch,beam,hidden,vocab,max_step,step", [(2, 4, 128, 300, 16, 0),
                                                                    (3, 2, 1024, 1000, 32, 31),
                                                                    (1, 1, 72, 50, 8, 3)])
def test_dec_emb(oracle, rng, dtype, vocab_major, batch, beam, hidden, vocab, max_step, step):
    rows = batch * beam
    table = _codes(rng, (vocab, hidden) if vocab_major else (hidden, vocab))
    pos = _randT(rng, (max_step, hidden), dtype, 0.1)
    tokens = rng.integers(0, vocab, size=(rows, max_step), dtype=np.int32)
    dq = 0.08 / 127
    want = oracle.dec_emb_i8I(table, pos, tokens, step, dq, True, vocab_major)
    out = torch.zeros(rows, hidden, dtype=TD[dtype], device=DEV)
    _k().launch_dec_emb_i8I(to_dev(table), to_dev(pos), to_dev(tokens), None, None, out, batch,
                            beam, hidden, vocab, step, max_step, 0, dq, True, vocab_major)
    np.testing.assert_array_equal(to_np(out), want)


def test_dec_emb_errors():
    from lightseq_amd.lib import LSHError
    t = torch.zeros(64, dtype=torch.int8, device=DEV)
    p = torch.zeros(64, dtype=torch.float16, device=DEV)
    tok = torch.zeros(8, dtype=torch.int32, device=DEV)
    with pytest.raises(LSHError, match="step < max_step"):
        _k().launch_dec_emb_i8I(t, p, tok, None, None, p, 1, 1, 8, 8, 8, 8, 0, 1.0, True)
    with pytest.raises(LSHError, match="multilingle"):
        _k().launch_dec_emb_i8I(t, p, tok, None, None, p, 1, 1, 8, 8, 0, 8, 1, 1.0, True)


# --------------------------------------------------------------------------- #
# self attention
# --------------------------------------------------------------------------- #
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("rows,heads,d,max_step,step", [(8, 4, 32, 16, 0), (6, 16, 64, 64, 37),
                                                        (3, 2, 20, 8, 7)])
def test_arrange_decself_qkv(oracle, rng, dtype, rows, heads, d, max_step, step):
    H = heads * d
    ori = _codes(rng, (rows, 3 * H))
    bias = _randT(rng, (3 * H,), dtype, 0.5)
    kc = _codes(rng, (rows, heads, max_step, d))
    vc = _codes(rng, (rows, heads, max_step, d))
    dq, qs = 3.0 / 127, 127 / 2.5
    kw, vw = kc.copy(), vc.copy()
    want_q = oracle.arrange_decself_qkv_i8I_i8O(ori, bias, kw, vw, step, dq, qs)
    kd, vd = to_dev(kc), to_dev(vc)
    q = torch.zeros(rows, H, dtype=torch.int8, device=DEV)
    _k().ker_arrange_decself_qkv_i8I_i8O_launcher(rows, H, to_dev(ori), to_dev(bias), q, kd, vd,
                                                  heads, d, max_step, step, 1024, dq, qs)
    np.testing.assert_array_equal(to_np(q), want_q)
    np.testing.assert_array_equal(to_np(kd), kw)
    np.testing.assert_array_equal(to_np(vd), vw)


@pytest.mark.parametrize("rows,heads,d,max_step,step_num", [(8, 4, 32, 16, 1), (4, 16, 64, 64, 64),
                                                            (5, 3, 20, 200, 131), (2, 2, 8, 1024, 1000),
                                                            (16, 16, 64, 640, 577),
                                                            (3, 4, 128, 256, 200)])
def test_decself_attention(oracle, rng, rows, heads, d, max_step, step_num):
    q = _codes(rng, (rows, heads * d))
    kc = _codes(rng, (rows, heads, max_step, d))
    vc = _codes(rng, (rows, heads, max_step, d))
    bh = rows * heads
    want_scores = oracle.decself_scores(q, kc, step_num)
    scores = torch.zeros(bh, max_step, dtype=torch.int32, device=DEV)
    qd, kd, vd = to_dev(q), to_dev(kc), to_dev(vc)
    _k().decself_scores_i8_i32o(kd, qd, scores, bh, step_num, max_step, d)
    got_scores = to_np(scores)
    np.testing.assert_array_equal(got_scores[:, :step_num], want_scores[:, :step_num])
    assert not got_scores[:, step_num:].any()  # nothing written past the current step

    # realistic magnitudes: logits of a few units after scaling
    dq = 4.0 / 127
    attn_scale = float(np.float16(np.sqrt(1.0 / d)))
    small = (want_scores // 4).astype(np.int32)
    qs = 127 / 1.5
    want = oracle.fuse_softmax_new_value_i32I_i8O(small, vc, step_num, attn_scale, dq, qs)
    out = torch.zeros(rows, heads * d, dtype=torch.int8, device=DEV)
    _k().ker_fuse_softmax_new_value_i32I_i8O_launcher(to_dev(small), vd, out, bh, step_num,
                                                      max_step, heads, d, attn_scale, dq, qs)
    assert_codes_close(to_np(out), want, what="fuse_softmax_new_value")

    # the fused kernel reproduces the pair: bit for bit where it shares the ascending-step
    # value sum (head sizes off the fast path), to the int8 bar where it sums as a tree
    want2 = torch.zeros_like(out)
    _k().ker_fuse_softmax_new_value_i32I_i8O_launcher(scores, vd, want2, bh, step_num, max_step,
                                                      heads, d, attn_scale, dq / 8, qs)
    fused = torch.zeros_like(out)
    _k().decself_attention_i8(qd, kd, vd, fused, bh, step_num, max_step, heads, d, attn_scale,
                              dq / 8, qs)
    if d in (32, 64, 128):
        assert_codes_close(to_np(fused), to_np(want2), what="decself_attention vs pair")
    else:
        np.testing.assert_array_equal(to_np(fused), to_np(want2))
    ref2 = oracle.fuse_softmax_new_value_i32I_i8O(want_scores, vc, step_num, attn_scale, dq / 8, qs)
    assert_codes_close(to_np(fused), ref2, what="decself_attention")


# --------------------------------------------------------------------------- #
# encoder-decoder attention
# --------------------------------------------------------------------------- #
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("batch,beam,heads,d", [(2, 4, 4, 32), (3, 1, 16, 64), (1, 8, 3, 10)])
def test_arrange_encdec_q(oracle, rng, dtype, batch, beam, heads, d):
    rows, H = batch * beam, heads * d
    ori = _codes(rng, (rows, H))
    bias = _randT(rng, (H,), dtype, 0.5)
    dq = 3.0 / 127
    want = oracle.arrange_encdec_q_i8I(ori, bias, beam, heads, dq)
    out = torch.zeros(batch, heads, beam, d, dtype=TD[dtype], device=DEV)
    _k().ker_arrange_encdec_q_i8I_launcher(rows, H, to_dev(ori), to_dev(bias), out, beam, d, heads,
                                           1024, dq)
    np.testing.assert_array_equal(to_np(out), want)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("batch,seq,layers,heads,d", [(2, 7, 2, 4, 32), (3, 33, 6, 8, 64),
                                                      (1, 5, 1, 3, 10)])
def test_arrange_encdec_kv(oracle, rng, dtype, batch, seq, layers, heads, d):
    H = heads * d
    ori = _randT(rng, (batch * seq, layers, 2, H), dtype)
    bias = _randT(rng, (layers, 2, H), dtype, 0.3)
    wk, wv = oracle.arrange_encdec_kv(ori, bias, batch, seq, layers, heads)
    # a layer stride larger than the data, as the model allocates it (max sizes)
    stride = batch * seq * H + 64
    k = torch.zeros(layers * stride, dtype=TD[dtype], device=DEV)
    v = torch.zeros(layers * stride, dtype=TD[dtype], device=DEV)
    _k().ker_arrange_encdec_kv_launcher(batch * seq, layers, H, to_dev(ori), to_dev(bias), k, v,
                                        stride, seq, d, heads, 1024)
    gk = to_np(k).reshape(layers, stride)[:, :batch * seq * H].reshape(wk.shape)
    gv = to_np(v).reshape(layers, stride)[:, :batch * seq * H].reshape(wv.shape)
    np.testing.assert_array_equal(gk, wk)
    np.testing.assert_array_equal(gv, wv)


def _pad_mask(rng, batch, seq):
    lens = rng.integers(max(1, seq // 3), seq + 1, size=batch)
    lens[0] = seq
    return (np.arange(seq)[None, :] >= lens[:, None]).astype(np.int32)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("batch,hb,seq", [(2, 16, 7), (3, 64, 64), (2, 8, 200), (1, 4, 1)])
def test_softmax_encdec(oracle, rng, dtype, batch, hb, seq):
    corr = _randT(rng, (batch, hb, seq), dtype, 2.0)
    mask = _pad_mask(rng, batch, seq)
    want = oracle.correlation_softmax_encdec(corr, mask)
    c = to_dev(corr)
    _k().ker_correlation_softmax_encdec_launcher(batch, hb, seq, c, to_dev(mask))
    got = to_np(c).astype(np.float32)
    tol = 1e-3 if dtype == np.float16 else 2e-6  # one fp16 ulp of a probability < 1
    np.testing.assert_allclose(got, want.astype(np.float32), atol=tol, rtol=0)
    assert not got[np.broadcast_to(mask[:, None, :] != 0, got.shape)].any()


@pytest.mark.parametrize("batch,beam,heads,d,seq", [(2, 4, 4, 32, 9), (2, 4, 16, 64, 64),
                                                    (3, 1, 2, 64, 130), (1, 8, 3, 10, 5)])
def test_encdec_attention_fused(oracle, rng, batch, beam, heads, d, seq):
    q = _randT(rng, (batch, heads, beam, d), np.float16)
    k = _randT(rng, (batch, heads, seq, d), np.float16)
    v = _randT(rng, (batch, heads, seq, d), np.float16)
    mask = _pad_mask(rng, batch, seq)
    bh = batch * heads
    sc = oracle.attn_scores_rect(q.reshape(bh, beam, d), k.reshape(bh, seq, d),
                                 float(np.sqrt(np.float32(1.0) / np.float32(d))))
    pr = oracle.correlation_softmax_encdec(sc.reshape(batch, heads * beam, seq), mask)
    ctx = oracle.attn_context_rect(pr.reshape(bh, beam, seq), v.reshape(bh, seq, d))
    qs = 127 / 1.0
    want_q = oracle.arrange_atten_output_i8O(ctx.reshape(batch, heads, beam, d), qs)
    ctx_d = torch.zeros(batch, heads, beam, d, dtype=torch.float16, device=DEV)
    ctx_q = torch.zeros(batch * beam, heads * d, dtype=torch.int8, device=DEV)
    _k().encdec_attention(to_dev(q), to_dev(k), to_dev(v), to_dev(mask), ctx_d, ctx_q, qs, batch,
                          beam, heads, seq, d)
    got = to_np(ctx_d).astype(np.float32).reshape(ctx.shape)
    # fp16 context values below ~2 in magnitude: 2e-3 is two ulps
    np.testing.assert_allclose(got, ctx.astype(np.float32), atol=2e-3, rtol=0)
    assert_codes_close(to_np(ctx_q), want_q.reshape(batch * beam, heads * d), max_frac=5e-3,
                       what="encdec ctx_q")


@pytest.mark.parametrize("m,n,k", [(64, 128, 64), (100, 200, 128), (512, 1536, 256), (7, 33, 16)])
def test_gemm_f16_nt(oracle, rng, m, n, k):
    a = _randT(rng, (m, k), np.float16)
    w = _randT(rng, (n, k), np.float16, 0.05)
    want = oracle.gemm_T(a, np.ascontiguousarray(w.T)).astype(np.float32)
    c = torch.zeros(m, n, dtype=torch.float16, device=DEV)
    _k().gemm_f16_nt(to_dev(a), to_dev(w), c, m, n, k)
    got = to_np(c).astype(np.float32)
    # fp32 accumulation rounded once to fp16: at most one fp16 ulp from the wide sum
    np.testing.assert_allclose(got, want, atol=1e-3, rtol=1.5e-3)
    f64 = a.astype(np.float64) @ w.astype(np.float64).T
    np.testing.assert_allclose(got, f64, atol=1e-3, rtol=1.5e-3)


# --------------------------------------------------------------------------- #
# beam search
# --------------------------------------------------------------------------- #
def _beam_state(rng, batch, beam, vocab, max_step, cur_step, end_id, dtype, finished_frac=0.3,
                tie_bias=False):
    rows = batch * beam
    logits = np.clip(rng.standard_normal((rows, vocab)) * 32, -127, 127).astype(np.int8)
    bias = np.zeros(vocab, dtype) if tie_bias else _randT(rng, (vocab,), dtype, 0.05)
    alive = rng.integers(4, vocab, size=(rows, max_step), dtype=np.int32)
    alive[:, 0] = 2
    fin = np.zeros(rows, bool)
    if cur_step > 0:
        fin = rng.random(rows) < finished_frac
        alive[fin, cur_step] = end_id
    if cur_step == 0:
        probs = np.where(np.arange(rows) % beam == 0, 0.0, -1000.0).astype(np.float32)
    else:
        probs = (-rng.random(rows) * 5 * cur_step).astype(np.float32)
    score = (-rng.random(rows) * 8 - 2000.0 * (np.arange(rows) // beam)).astype(np.float32)
    return logits, bias, probs, score, alive, fin


BEAM_CASES = [  # batch, beam, vocab, max_step, cur_step, threads
    (2, 4, 320, 16, 0, 1024),
    (3, 4, 1000, 32, 5, 1024),
    (2, 8, 32000, 64, 17, 1024),
    (4, 2, 777, 16, 3, 256),
    (2, 1, 500, 16, 2, 1024),
    (1, 32, 5000, 16, 4, 1024),
    (2, 16, 2100, 16, 1, 32),
    (2, 4, 32768, 16, 2, 1024),   # largest vocabulary of the register-resident top-k kernel
    (1, 4, 40000, 16, 2, 1024),   # beyond it: the looping kernel
]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("batch,beam,vocab,max_step,cur_step,threads", BEAM_CASES)
def test_select_beam_rough_topk(oracle, rng, dtype, batch, beam, vocab, max_step, cur_step,
                                threads):
    end_id = 3
    logits, bias, probs, score, alive, _ = _beam_state(rng, batch, beam, vocab, max_step, cur_step,
                                                       end_id, dtype)
    rows = batch * beam
    dq = 2.5 / 127
    ln = oracle.length_norm(cur_step + 1, 0.6)
    assert _k().length_norm(cur_step + 1, 0.6) == ln
    w_idx, w_score, w_num = oracle.select_beam_rough_topk_i8I(logits, bias, probs, score, alive, dq,
                                                              ln, cur_step, threads, beam, end_id)
    can_idx = torch.full((rows * vocab,), -1, dtype=torch.int32, device=DEV)
    can_score = torch.zeros(rows * vocab, dtype=torch.float32, device=DEV)
    num = torch.zeros(rows + 1, dtype=torch.int32, device=DEV)
    _k().select_beam_rough_topk_i8I_launcher(to_dev(logits), to_dev(bias), to_dev(probs),
                                             to_dev(score), to_dev(alive), dq, can_idx, can_score,
                                             num, vocab, max_step, ln, cur_step, rows, threads,
                                             beam, 0.0, end_id)
    g_num = to_np(num)
    np.testing.assert_array_equal(g_num, w_num)
    total = int(g_num[0])
    assert total >= 1 and (g_num[1:] >= 1).all()
    np.testing.assert_array_equal(to_np(can_idx)[:total], w_idx)
    # scores: sums of exp / log differ in the last bits; |score| reaches 2000 * batch
    np.testing.assert_allclose(to_np(can_score)[:total], w_score, rtol=2e-6, atol=2e-4)


def _oracle_step(oracle, logits, bias, probs, score, alive, dq, ln, cur_step, beam, end_id, vocab):
    idx, sc, num = oracle.select_beam_rough_topk_i8I(logits, bias, probs, score, alive, dq, ln,
                                                     cur_step, 1024, beam, end_id)
    s_idx, s_sc, s_num = oracle.scan_sort_candidates(idx, sc, num)
    new_alive, new_probs, new_score, fin = oracle.refresh_result(
        s_idx, s_sc, s_num, alive, probs, score, vocab, cur_step, ln, end_id, beam)
    return s_idx, s_sc, s_num, new_alive, new_probs, new_score, fin


@pytest.mark.parametrize("batch,beam,vocab,max_step,cur_step,threads", BEAM_CASES)
def test_refresh_result_and_cache(oracle, rng, batch, beam, vocab, max_step, cur_step, threads):
    end_id = 3
    dtype = np.float16
    logits, bias, probs, score, alive, _ = _beam_state(rng, batch, beam, vocab, max_step, cur_step,
                                                       end_id, dtype)
    # make <eos> attractive so that some beams finish in this step
    logits[:, end_id] = 120
    rows = batch * beam
    dq = 2.5 / 127
    ln = oracle.length_norm(cur_step + 1, 0.6)
    s_idx, s_sc, s_num, w_alive, w_probs, w_score, w_fin = _oracle_step(
        oracle, logits, bias, probs, score, alive, dq, ln, cur_step, beam, end_id, vocab)
    d_idx, d_sc, d_num = to_dev(s_idx), to_dev(s_sc), to_dev(s_num)
    new_alive = torch.zeros(rows, max_step, dtype=torch.int32, device=DEV)
    p_d, s_d = to_dev(probs), to_dev(score)
    fin = torch.zeros(1, dtype=torch.int32, device=DEV)
    _k().ker_refresh_result(d_idx, d_sc, d_num.data_ptr() + 4, to_dev(alive), new_alive, p_d, s_d,
                            fin, vocab, cur_step, ln, 0.0, end_id, batch, beam, max_step)
    np.testing.assert_array_equal(to_np(new_alive), w_alive)
    np.testing.assert_array_equal(to_np(p_d), w_probs)
    np.testing.assert_array_equal(to_np(s_d), w_score)
    assert int(to_np(fin)[0]) == w_fin

    # cache reorder from the same sorted candidates
    layers, heads, d = 2, 2, 16
    shape = (layers, rows, heads, max_step, d)
    k_old, v_old = _codes(rng, shape), _codes(rng, shape)
    k_new, v_new = _codes(rng, shape), _codes(rng, shape)
    wk, wv = k_new.copy(), v_new.copy()
    oracle.refresh_cache_i8(s_num, s_idx, k_old, v_old, wk, wv, beam, vocab, cur_step, end_id)
    kn, vn = to_dev(k_new), to_dev(v_new)
    _k().ker_refresh_cache_launcher_i8(layers, rows * 2, 1024, d_num.data_ptr() + 4, d_idx,
                                       to_dev(k_old), to_dev(v_old), kn, vn,
                                       rows * heads * max_step * d, beam, d, heads, vocab, cur_step,
                                       max_step, False, end_id)
    np.testing.assert_array_equal(to_np(kn), wk)
    np.testing.assert_array_equal(to_np(vn), wv)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("tie_bias", [False, True])
@pytest.mark.parametrize("batch,beam,vocab,max_step,cur_step,threads", BEAM_CASES)
def test_beam_search_step(oracle, rng, dtype, tie_bias, batch, beam, vocab, max_step, cur_step,
                          threads):
    """The sort-free search step picks the beams the reference pipeline picks."""
    end_id = 3
    logits, bias, probs, score, alive, _ = _beam_state(rng, batch, beam, vocab, max_step, cur_step,
                                                       end_id, dtype, tie_bias=tie_bias)
    logits[::2, end_id] = 100
    rows = batch * beam
    dq = 2.5 / 127
    ln = oracle.length_norm(cur_step + 1, 0.6)
    s_idx, s_sc, s_num, w_alive, w_probs, w_score, w_fin = _oracle_step(
        oracle, logits, bias, probs, score, alive, dq, ln, cur_step, beam, end_id, vocab)
    new_alive = torch.zeros(rows, max_step, dtype=torch.int32, device=DEV)
    p_d, s_d = to_dev(probs), to_dev(score)
    top_s = torch.zeros(rows * beam, dtype=torch.float32, device=DEV)
    top_i = torch.zeros(rows * beam, dtype=torch.int32, device=DEV)
    parent = torch.full((rows,), -7, dtype=torch.int32, device=DEV)
    fin = torch.zeros(1, dtype=torch.int32, device=DEV)
    _k().beam_search_step_i8I(to_dev(logits), to_dev(bias), p_d, s_d, to_dev(alive), new_alive,
                              top_s, top_i, parent, fin, dq, vocab, max_step, ln, cur_step, batch,
                              beam, end_id)
    np.testing.assert_array_equal(to_np(new_alive), w_alive)
    assert int(to_np(fin)[0]) == w_fin
    # parents: the winning candidates' source beams, -1 where the new token is <eos>
    picks = np.stack([s_idx[s_num[1 + b * beam] + np.arange(beam)] for b in range(batch)])
    want_parent = np.where(picks % vocab == end_id, -1, picks // vocab).reshape(-1)
    np.testing.assert_array_equal(to_np(parent), want_parent)
    live = want_parent >= 0
    np.testing.assert_allclose(to_np(p_d)[live], w_probs[live], rtol=2e-6, atol=2e-4)
    np.testing.assert_allclose(to_np(s_d)[~live], w_score[~live], rtol=2e-6, atol=2e-4)
    # untouched slots keep their old values
    np.testing.assert_array_equal(to_np(p_d)[~live], probs[~live])
    np.testing.assert_array_equal(to_np(s_d)[live], score[live])

    # cache reorder by parent table == reorder from the sorted candidates
    layers, heads, d = 2, 2, 16
    shape = (layers, rows, heads, max_step, d)
    k_old, v_old = _codes(rng, shape), _codes(rng, shape)
    k_new, v_new = _codes(rng, shape), _codes(rng, shape)
    wk, wv = k_new.copy(), v_new.copy()
    oracle.refresh_cache_i8(s_num, s_idx, k_old, v_old, wk, wv, beam, vocab, cur_step, end_id)
    kn, vn = to_dev(k_new), to_dev(v_new)
    _k().refresh_cache_by_parent_i8(layers, rows, parent, to_dev(k_old), to_dev(v_old), kn, vn,
                                    rows * heads * max_step * d, beam, d, heads, cur_step, max_step)
    np.testing.assert_array_equal(to_np(kn), wk)
    np.testing.assert_array_equal(to_np(vn), wv)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("tie_bias", [False, True])
@pytest.mark.parametrize("batch,beam,vocab,cur_step", [(2, 8, 32000, 17), (16, 4, 32000, 9), (2, 4, 32768, 2),
                                                       (3, 2, 8208, 0), (1, 32, 16384, 4), (2, 4, 9000 - 8, 3),
                                                       (2, 4, 5008, 3), (1, 4, 40000, 2)])
def test_beam_search_step_with_the_rows_dealt_to_several_workgroups(oracle, rng, dtype, tie_bias, batch,
                                                                     beam, vocab, cur_step):
    """lsh_beam_search_step_ws_i8I picks the beams the reference pipeline picks and the beams of
    lsh_beam_search_step_i8I (vocabularies of 8208 .. 32768 ids run the split kernels, the last
    two cases fall back), finished beams included."""
    end_id, max_step = 3, 24
    logits, bias, probs, score, alive, _ = _beam_state(rng, batch, beam, vocab, max_step, cur_step,
                                                       end_id, dtype, tie_bias=tie_bias)
    logits[::2, end_id] = 100
    rows = batch * beam
    dq = 2.5 / 127
    ln = oracle.length_norm(cur_step + 1, 0.6)
    s_idx, s_sc, s_num, w_alive, w_probs, w_score, w_fin = _oracle_step(
        oracle, logits, bias, probs, score, alive, dq, ln, cur_step, beam, end_id, vocab)
    nbytes = _k().beam_search_step_workspace(batch, beam, vocab)
    assert (nbytes > 0) == (8192 < vocab <= 32768 and vocab % 16 == 0)
    if nbytes:
        assert nbytes == rows * -(-vocab // 8192) * 2 * beam * 4
    out = []
    for ws in (torch.zeros(max(nbytes, 8) // 4, dtype=torch.float32, device=DEV), None):
        new_alive = torch.zeros(rows, max_step, dtype=torch.int32, device=DEV)
        p_d, s_d = to_dev(probs), to_dev(score)
        top_s = torch.zeros(rows * beam, dtype=torch.float32, device=DEV)
        top_i = torch.zeros(rows * beam, dtype=torch.int32, device=DEV)
        parent = torch.full((rows,), -7, dtype=torch.int32, device=DEV)
        fin = torch.zeros(1, dtype=torch.int32, device=DEV)
        _k().beam_search_step_ws_i8I(to_dev(logits), to_dev(bias), p_d, s_d, to_dev(alive), new_alive,
                                     top_s, top_i, parent, fin, dq, vocab, max_step, ln, cur_step, batch,
                                     beam, end_id, ws)
        out.append((to_np(new_alive), to_np(parent), int(to_np(fin)[0]), to_np(p_d), to_np(s_d)))
    (a_alive, a_parent, a_fin, a_p, a_s), (b_alive, b_parent, b_fin, b_p, b_s) = out
    np.testing.assert_array_equal(a_alive, w_alive)
    assert a_fin == w_fin
    picks = np.stack([s_idx[s_num[1 + b * beam] + np.arange(beam)] for b in range(batch)])
    want_parent = np.where(picks % vocab == end_id, -1, picks // vocab).reshape(-1)
    np.testing.assert_array_equal(a_parent, want_parent)
    live = want_parent >= 0
    np.testing.assert_allclose(a_p[live], w_probs[live], rtol=2e-6, atol=2e-4)
    np.testing.assert_allclose(a_s[~live], w_score[~live], rtol=2e-6, atol=2e-4)
    np.testing.assert_array_equal(a_p[~live], probs[~live])
    np.testing.assert_array_equal(a_s[live], score[live])
    # against the one-workgroup-per-row step: same sequences, parents, count; scores to the last place
    np.testing.assert_array_equal(a_alive, b_alive)
    np.testing.assert_array_equal(a_parent, b_parent)
    assert a_fin == b_fin
    np.testing.assert_allclose(a_p, b_p, rtol=1e-6, atol=1e-5)
    np.testing.assert_allclose(a_s, b_s, rtol=1e-6, atol=1e-5)


@pytest.mark.parametrize("batch,beam,max_step,out_len", [(3, 4, 16, 9), (8, 4, 32, 31), (2, 1, 8, 1),
                                                         (5, 8, 16, 15)])
def test_output_writers(oracle, rng, batch, beam, max_step, out_len):
    end_id, vocab = 3, 100
    rows = batch * beam
    alive = rng.integers(0, 6, size=(rows, max_step), dtype=np.int32)
    score = (-rng.random(rows) * 20 - 2000.0 * (np.arange(rows) // beam)).astype(np.float32)
    a_d = to_dev(alive)

    w_out, w_score = oracle.write_trg_tokenid_pos_penalty(alive, score, beam, out_len)
    out = torch.zeros(batch, out_len, dtype=torch.int32, device=DEV)
    s_d = to_dev(score)
    _k().ker_write_trg_tokenid_pos_penalty(a_d, s_d, out, max_step, beam, batch, out_len)
    np.testing.assert_array_equal(to_np(out), w_out)
    np.testing.assert_array_equal(to_np(s_d), w_score)

    w_out = oracle.write_trg_tokenid_neg_penalty(alive, score, beam, end_id, out_len)
    out.zero_()
    _k().ker_write_trg_tokenid_neg_penalty(a_d, to_dev(score), out, max_step, beam, vocab, end_id,
                                           batch, out_len)
    np.testing.assert_array_equal(to_np(out), w_out)

    w_out, w_score = oracle.write_topk_result(alive, score, beam, end_id, out_len)
    out2 = torch.zeros(rows, out_len, dtype=torch.int32, device=DEV)
    s_d = to_dev(score)
    _k().ker_write_topk_result(a_d, s_d, out2, vocab, max_step, beam, end_id, rows, out_len)
    np.testing.assert_array_equal(to_np(out2), w_out)
    np.testing.assert_array_equal(to_np(s_d), w_score)


def test_beam_argument_errors():
    from lightseq_amd.lib import LSHError
    z8 = torch.zeros(64, dtype=torch.int8, device=DEV)
    zh = torch.zeros(64, dtype=torch.float16, device=DEV)
    zf = torch.zeros(64, dtype=torch.float32, device=DEV)
    zi = torch.zeros(64, dtype=torch.int32, device=DEV)
    with pytest.raises(LSHError, match="beam_size"):
        _k().select_beam_rough_topk_i8I_launcher(z8, zh, zf, zf, zi, 1.0, zi, zf, zi, 8, 8, 1.0, 0,
                                                 3, 1024, 3, 0.0, 1)
    with pytest.raises(LSHError, match="diverse"):
        _k().select_beam_rough_topk_i8I_launcher(z8, zh, zf, zf, zi, 1.0, zi, zf, zi, 8, 8, 1.0, 0,
                                                 4, 1024, 4, 0.5, 1)
    with pytest.raises(LSHError, match="COL32"):
        _k().select_beam_rough_topk_i8I_launcher(z8, zh, zf, zf, zi, 1.0, zi, zf, zi, 8, 8, 1.0, 0,
                                                 4, 1024, 4, 0.0, 1, in_col32=True)
    with pytest.raises(LSHError, match="must differ"):
        _k().beam_search_step_i8I(z8, zh, zf, zf, zi, zi, zf, zi, zi, zi, 1.0, 8, 8, 1.0, 0, 1, 4,
                                  1)
