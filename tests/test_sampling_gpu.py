"""GPU parity of the GPT random-sampling launchers (top-k with k > 1, top-p) against the CPU
restatement in oracle/sampling.py, through the C ABI.  The uniform number of a draw is defined
by (seed, sequence, draw index), so the sampled token is decided -- except where the number
falls within 1e-5 of a boundary of the cumulative distribution (the float sums run in another
order on the GPU); the oracle flags those draws and they are compared by membership only."""
import os

import numpy as np
import pytest
import torch

from helpers import DEV, to_dev, to_np
from oracle import sampling as S

pytestmark = pytest.mark.gpu


def _k():
    from lightseq_amd import kernels
    return kernels


def _logits(rng, rows, vocab, spread=35):
    return np.clip(rng.standard_normal((rows, vocab)) * spread, -127, 127).astype(np.int8)


def test_generator_numbers_are_the_philox_words():
    """1024 equal logits: every class is a candidate of probability 1/1024, so the chosen id is
    ceil(1024 x) - 1 and reveals the uniform number of every (sequence, draw)."""
    k = _k()
    batch, vocab, seed = 5, 1024, 0x1234567890ABCDEF
    state = k.rng_setup(batch, seed)
    logits = to_dev(np.full((batch, vocab), 17, np.int8))
    max_step = 12
    ids = torch.ones(batch, max_step, dtype=torch.int32, device=DEV)
    last = torch.zeros(batch, dtype=torch.int32, device=DEV)
    unf = torch.zeros(1, dtype=torch.int32, device=DEV)
    for draw in range(6):
        k.gpt_sample_step(logits, ids, last, vocab, max_step, 1 + draw, batch, unf, vocab + 5, 32, 0.0,
                          0.1, state)
        got = to_np(last)
        for b in range(batch):
            x = float(S.uniform_of_draw(seed, b, draw))
            want = int(np.ceil(1024 * x)) - 1
            assert abs(int(got[b]) - want) <= (abs(1024 * x - round(1024 * x)) < 1e-2), (b, draw, x, got[b])
    st = to_np(state).view(np.uint32).reshape(batch, 4)
    assert (st[:, 3] == 6).all() and (st[:, 2] == np.arange(batch)).all()


@pytest.mark.parametrize("vocab,k", [(1000, 2), (1024, 4), (5000, 8), (50257, 4), (32000, 16), (2077, 32)])
def test_topk_sampling_launcher_against_the_oracle(rng, vocab, k):
    kk = _k()
    batch, seq, lsl, eos, scale, seed = 6, 5, 2, 3, 0.09, 99 + k
    logits = _logits(rng, batch * lsl, vocab)
    old = rng.integers(4, vocab, size=(batch, seq), dtype=np.int32)
    old[2, -1] = eos  # an ended sequence stays ended and draws nothing
    state = kk.rng_setup(batch, seed)
    buf = torch.zeros(batch * seq + batch, dtype=torch.int32, device=DEV)
    buf[:batch * seq] = to_dev(old.reshape(-1))
    new = torch.zeros(batch, seq + 1, dtype=torch.int32, device=DEV)
    unf = torch.zeros(1, dtype=torch.int32, device=DEV)
    for draw in range(2):  # the second launch uses the next number of every live sequence
        kk.ker_topk_sample_i8I_launcher(batch, seq, lsl, 1024, to_dev(logits), buf, new, None, vocab, k,
                                        unf, state, eos, scale)
        got = to_np(new)
        np.testing.assert_array_equal(got[:, :seq], old)
        np.testing.assert_array_equal(to_np(buf)[batch * seq:], got[:, seq])
        for b in range(batch):
            if b == 2:
                assert got[b, seq] == eos
                continue
            row = logits[(b + 1) * lsl - 1]
            tok, amb, cand, _ = S.topk_sample_row(row, k, scale, S.uniform_of_draw(seed, b, draw))
            assert got[b, seq] in cand
            if not amb:
                assert got[b, seq] == tok, (b, draw)
        assert int(to_np(unf)[0]) == 1
    st = to_np(state).view(np.uint32).reshape(batch, 4)
    assert st[:, 3].tolist() == [2, 2, 0, 2, 2, 2]


@pytest.mark.parametrize("vocab,p", [(900, 0.5), (1024, 0.9), (50257, 0.75), (32000, 0.2), (7001, 1.0),
                                     (4096, 0.01)])
def test_topp_sampling_launcher_against_the_oracle(rng, vocab, p):
    kk = _k()
    batch, seq, lsl, eos, scale, seed = 5, 3, 1, 2, 0.12, 5
    logits = _logits(rng, batch * lsl, vocab, spread=25)
    logits[0, 11] = 127  # a row with a dominant id
    old = rng.integers(3, vocab, size=(batch, seq), dtype=np.int32)
    state = kk.rng_setup(batch, seed)
    buf = torch.zeros(batch * seq + batch, dtype=torch.int32, device=DEV)
    buf[:batch * seq] = to_dev(old.reshape(-1))
    new = torch.zeros(batch, seq + 1, dtype=torch.int32, device=DEV)
    unf = torch.zeros(1, dtype=torch.int32, device=DEV)
    kk.ker_topp_sample_i8I_launcher(batch, seq, lsl, 1024, to_dev(logits), buf, new, None, vocab, p, unf,
                                    state, eos, scale)
    got = to_np(new)
    for b in range(batch):
        tok, amb, cand, _ = S.topp_sample_row(logits[b], p, scale, S.uniform_of_draw(seed, b, 0))
        if not amb:
            assert got[b, seq] in cand and got[b, seq] == tok, b


def test_sampled_frequencies_follow_the_candidate_probabilities(rng):
    """4000 draws of one row (one sequence, draw after draw) against the oracle's probabilities."""
    kk = _k()
    vocab, k, scale = 3000, 8, 0.05
    row = _logits(rng, 1, vocab, spread=20)
    _, _, cand, probs = S.topk_sample_row(row[0], k, scale, 0.5)
    state = kk.rng_setup(1, 2024)
    max_step = 4002
    ids = torch.ones(1, max_step, dtype=torch.int32, device=DEV)
    last = torch.zeros(1, dtype=torch.int32, device=DEV)
    unf = torch.zeros(1, dtype=torch.int32, device=DEV)
    rowd = to_dev(row)
    for d in range(4000):
        kk.gpt_sample_step(rowd, ids, last, vocab, max_step, 1 + d, 1, unf, vocab + 1, k, 0.0, scale, state)
    drawn = to_np(ids)[0, 1:4001]
    assert set(drawn.tolist()) <= set(cand.tolist())
    for i, pr in zip(cand, probs):
        assert abs((drawn == i).mean() - pr) < 4 * np.sqrt(pr * (1 - pr) / 4000) + 2e-3


def test_sampling_launchers_reject_bad_arguments():
    from lightseq_amd.lib import LSHError
    kk = _k()
    z8 = torch.zeros(64, dtype=torch.int8, device=DEV)
    zi = torch.zeros(64, dtype=torch.int32, device=DEV)
    st = kk.rng_setup(2, 1)
    with pytest.raises(LSHError, match=r"\[1,2,4,8,16,32\]"):
        kk.gpt_sample_step(z8, zi, zi, 16, 8, 2, 2, zi, 1, 3, 0.5, 0.1, st)
    with pytest.raises(LSHError, match="topp"):
        kk.gpt_sample_step(z8, zi, zi, 16, 8, 2, 2, zi, 1, 0, 1.5, 0.1, st)
    with pytest.raises(LSHError):
        kk.ker_topp_sample_i8I_launcher(1, 4, 1, 1024, z8, zi, zi, None, 16, 0.0, zi, st, 1, 0.1)
    with pytest.raises(LSHError, match="generator state"):
        kk.ker_topp_sample_i8I_launcher(1, 4, 1, 1024, z8, zi, zi, None, 16, 0.5, zi, None, 1, 0.1)


@pytest.mark.parametrize("method,topk,topp", [("topk", 4, 0.75), ("topk", 32, 0.75), ("topp", 1, 0.6)])
def test_quant_gpt_with_random_sampling(tmp_path, method, topk, topp):
    """QuantGpt loads a model file that asks for random sampling (topk = 4 is the format's
    default), gives the same tokens for the same seed, and every sampled token is the oracle's
    choice for the step's recorded logits and the (seed, sequence, draw) number."""
    from lightseq_amd import synthetic
    from lightseq_amd.inference import QuantGpt
    cfg = synthetic.gpt_config("tiny")
    cfg.update(sampling_method=method, topk=topk, topp=topp)
    path = os.path.join(str(tmp_path), "sample.pb")
    msg = synthetic.write_quant_gpt(path, cfg, seed=3, w_std=0.2)
    scale = float(msg["src_embedding"]["logits_clip_max"]) / 127.0
    rng = np.random.default_rng(1)
    ids = rng.integers(1, cfg["vocab"] - 1, size=(3, 6), dtype=np.int32)
    ids[ids == cfg["eos_id"]] = 1
    model = QuantGpt(path, 3)
    a = model.sample(ids)            # seed 0 at load
    model.set_seed(0)
    rec = torch.zeros(cfg["max_step"], 3, cfg["vocab"], dtype=torch.int8, device=DEV)
    model.set_step_record(rec, cfg["max_step"])
    b = model.sample(ids)
    steps = model.steps_run()
    np.testing.assert_array_equal(a, b)
    model.set_step_record(None, 0)
    model.set_seed(12345)
    c = model.sample(ids)
    assert c.shape[0] == 3
    model.close()
    logits = rec.cpu().numpy()[:steps]
    draws = np.zeros(3, np.int64)
    seq = ids.shape[1]
    checked = 0
    for s in range(steps):
        for r in range(3):
            if b[r, seq + s - 1] == cfg["eos_id"]:
                assert b[r, seq + s] == cfg["eos_id"]
                continue
            x = S.uniform_of_draw(0, r, int(draws[r]))
            draws[r] += 1
            if method == "topp":
                tok, amb, cand, _ = S.topp_sample_row(logits[s, r], topp, scale, x)
            else:
                tok, amb, cand, _ = S.topk_sample_row(logits[s, r], topk, scale, x)
            assert b[r, seq + s] in cand
            if not amb:
                assert b[r, seq + s] == tok, (s, r)
                checked += 1
    assert checked >= steps



# ---- encoder-decoder launchers: logit = code * scale + bias[id], ids in place ---------------
def _dec_case(rng, batch, vocab, max_step, cur_len, eos, bias_dtype, spread=30):
    logits = _logits(rng, batch, vocab, spread)
    bias = (rng.standard_normal(vocab) * 2).astype(bias_dtype)
    ids = rng.integers(eos + 1, vocab, size=(batch, max_step), dtype=np.int32)
    return logits, bias, ids


@pytest.mark.parametrize("bias_dtype", [np.float16, np.float32])
@pytest.mark.parametrize("vocab,k", [(1000, 1), (32000, 1), (1024, 2), (5000, 4), (32000, 8), (2077, 32)])
def test_decoder_topk_sampling_launcher_against_the_oracle(rng, vocab, k, bias_dtype):
    kk = _k()
    batch, max_step, cur_len, eos, scale, seed = 6, 9, 4, 2, 0.09, 40 + k
    logits, bias, ids = _dec_case(rng, batch, vocab, max_step, cur_len, eos, bias_dtype)
    ids[2, cur_len - 1] = eos          # an ended row: another end token, no draw, no flag
    if k == 1:
        logits[4, :] = 5               # ties at the maximum go to the first id (bias breaks none)
        bias_tie = bias.copy()
        bias_tie[:] = 0
    state = kk.rng_setup(batch, seed)
    d_ids, d_unf = to_dev(ids), torch.zeros(1, dtype=torch.int32, device=DEV)
    want = ids.copy()
    draws = np.zeros(batch, np.int64)
    for step in range(2):
        cl = cur_len + step
        kk.ker_topk_sample_i8I_dec_launcher(batch, cl, max_step, 1, 1024, to_dev(logits), to_dev(bias),
                                            d_ids, None, vocab, k, d_unf, None if k == 1 else state,
                                            eos, scale)
        got = to_np(d_ids)
        unf, amb = S.dec_sample_step(logits, bias, want, cl, eos, scale, k=k, seed=seed, draws=draws)
        for b in range(batch):
            if b in amb:
                want[b, cl] = got[b, cl]   # a draw at a boundary of the distribution: either side
        np.testing.assert_array_equal(got, want, err_msg="step %d" % step)
        assert int(to_np(d_unf)[0]) == unf == 1
    if k > 1:
        st = to_np(state).view(np.uint32).reshape(batch, 4)
        assert st[:, 3].tolist() == [2, 2, 0, 2, 2, 2]
    else:
        d2 = to_dev(ids)
        kk.ker_topk_sample_i8I_dec_launcher(batch, cur_len, max_step, 1, 1024, to_dev(logits),
                                            to_dev(bias_tie), d2, None, vocab, 1, d_unf, None, eos, scale)
        assert int(to_np(d2)[4, cur_len]) == 0


@pytest.mark.parametrize("vocab,p", [(900, 0.5), (1024, 0.9), (32000, 0.75), (7001, 1.0), (4096, 0.01)])
def test_decoder_topp_sampling_launcher_against_the_oracle(rng, vocab, p):
    kk = _k()
    batch, max_step, cur_len, eos, scale, seed = 5, 6, 1, 2, 0.12, 5
    logits, bias, ids = _dec_case(rng, batch, vocab, max_step, cur_len, eos, np.float16, spread=25)
    logits[0, 11] = 127
    bias[11] = 3.0                     # a row with a dominant id
    ids[3, 0] = eos                    # cur_len == 1: the start column never ends a row (:1917)
    state = kk.rng_setup(batch, seed)
    d_ids, d_unf = to_dev(ids), torch.zeros(1, dtype=torch.int32, device=DEV)
    kk.ker_topp_sample_i8I_dec_launcher(batch, cur_len, max_step, 1, 1024, to_dev(logits), to_dev(bias),
                                        d_ids, None, vocab, p, d_unf, state, eos, scale)
    got = to_np(d_ids)
    np.testing.assert_array_equal(got[:, :cur_len], ids[:, :cur_len])
    np.testing.assert_array_equal(got[:, cur_len + 1:], ids[:, cur_len + 1:])
    for b in range(batch):
        tok, amb, cand, _ = S.dec_topp_sample_row(logits[b], bias, p, scale, S.uniform_of_draw(seed, b, 0))
        if not amb:
            assert got[b, cur_len] in cand and got[b, cur_len] == tok, b


def test_decoder_sampling_uses_the_last_logits_row_of_a_sequence(rng):
    kk = _k()
    batch, lsl, vocab, max_step, eos, scale = 3, 4, 3000, 5, 1, 0.1
    logits = _logits(rng, batch * lsl, vocab)
    bias = np.zeros(vocab, np.float32)
    ids = np.full((batch, max_step), 7, np.int32)
    d_ids, d_unf = to_dev(ids), torch.zeros(1, dtype=torch.int32, device=DEV)
    kk.ker_topk_sample_i8I_dec_launcher(batch, 2, max_step, lsl, 1024, to_dev(logits), to_dev(bias),
                                        d_ids, None, vocab, 1, d_unf, None, eos, scale)
    got = to_np(d_ids)
    for b in range(batch):
        assert got[b, 2] == int(np.argmax(logits[(b + 1) * lsl - 1]))


def test_decoder_sampling_launchers_reject_bad_arguments():
    from lightseq_amd.lib import LSHError
    kk = _k()
    z8 = torch.zeros(64, dtype=torch.int8, device=DEV)
    zi = torch.zeros(64, dtype=torch.int32, device=DEV)
    zb = torch.zeros(16, dtype=torch.float16, device=DEV)
    st = kk.rng_setup(2, 1)
    with pytest.raises(LSHError, match=r"\[1,2,4,8,16,32\]"):
        kk.ker_topk_sample_i8I_dec_launcher(2, 2, 8, 1, 1024, z8, zb, zi, None, 16, 3, zi, st, 1, 0.1)
    with pytest.raises(LSHError, match="generator state"):
        kk.ker_topk_sample_i8I_dec_launcher(2, 2, 8, 1, 1024, z8, zb, zi, None, 16, 4, zi, None, 1, 0.1)
    with pytest.raises(LSHError, match="topp"):
        kk.ker_topp_sample_i8I_dec_launcher(2, 2, 8, 1, 1024, z8, zb, zi, None, 16, 1.5, zi, st, 1, 0.1)
    with pytest.raises(LSHError):   # the column to write lies outside the row
        kk.ker_topk_sample_i8I_dec_launcher(2, 8, 8, 1, 1024, z8, zb, zi, None, 16, 1, zi, None, 1, 0.1)
    with pytest.raises(LSHError, match="COL32|col32"):
        kk.ker_topk_sample_i8I_dec_launcher(2, 2, 8, 1, 1024, z8, zb, zi, None, 16, 1, zi, None, 1, 0.1,
                                            in_col32=True)


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
@pytest.mark.parametrize("dst,src", [(1, 640), (5, 9), (16, 16), (3, 1024)])
def test_attention_mask_weights_launcher(rng, dtype, dst, src):
    from oracle import gpt as og
    kk = _k()
    batch, heads = 3, 4
    corr = rng.integers(-30000, 30000, size=(batch, heads * dst, src)).astype(np.int32)
    rsl = np.array([src, max(src - dst + 1, 1), src - 1], np.int32)
    attn_scale, dq = 0.125, 2.0 / 127
    npdt = np.float16 if dtype == torch.float16 else np.float32
    want = np.full(corr.shape, 3.0, npdt)
    og.attention_mask_weights_i32I(corr, rsl, heads, dst, attn_scale, dq, want)
    out = torch.full(corr.shape, 3.0, dtype=dtype, device=DEV)
    kk.ker_attention_mask_weights_i32I_launcher(batch, dst, src, heads, to_dev(corr), out, to_dev(rsl),
                                                attn_scale, dq)
    got = to_np(out).astype(np.float32)
    tol = 1e-3 if dtype == torch.float16 else 2e-6   # float sums run in another order
    np.testing.assert_allclose(got, want.astype(np.float32), atol=tol)
    np.testing.assert_array_equal(got == 3.0, want.astype(np.float32) == 3.0)  # untouched rows
