"""The CPU restatement of the GPT random-sampling kernels (oracle/sampling.py), pinned by what
does not depend on it: the published Philox4x32-10 known-answer vectors, a lane-by-lane run of
the reference's shuffle network, brute-force nucleus and soft-max computations."""
import numpy as np
import pytest
from scipy.special import softmax

from oracle import sampling as S


def test_philox_known_answers():
    """Random123 kat_vectors, philox4x32 with 10 rounds."""
    assert S.philox4x32_10((0, 0, 0, 0), (0, 0)) == [0x6627e8d5, 0xe169c58d, 0xbc57ac4c, 0x9b00dbd8]
    assert S.philox4x32_10((0xffffffff,) * 4, (0xffffffff,) * 2) == \
        [0x408f276d, 0x41c83b0e, 0xa20bc7c6, 0x6d5451fd]
    assert S.philox4x32_10((0x243f6a88, 0x85a308d3, 0x13198a2e, 0x03707344), (0xa4093822, 0x299f31d0)) == \
        [0xd16cfe09, 0x94fdcceb, 0x5001e420, 0x24126ea1]


def test_uniforms_lie_in_the_half_open_unit_interval_and_look_uniform():
    xs = np.array([S.uniform_of_draw(7, r, d) for r in range(8) for d in range(500)], np.float64)
    assert xs.min() > 0.0 and xs.max() <= 1.0
    assert abs(xs.mean() - 0.5) < 0.02 and abs(xs.var() - 1 / 12) < 0.01
    # rows and draws give different numbers; the seed's high word matters
    assert S.uniform_of_draw(7, 0, 0) != S.uniform_of_draw(7, 1, 0) != S.uniform_of_draw(7, 0, 1)
    assert S.uniform_of_draw(7, 3, 5) != S.uniform_of_draw(7 + (1 << 32), 3, 5)


def _shuffle_network_kth(thread_max, k):
    """kernels/common.h:118-137 lane by lane: warp maxima, then xor-butterflies over 32 lanes
    (max for masks 16..k, min for masks k/2..1); lane 0's value."""
    val = [float(thread_max[32 * w:32 * w + 32].max()) for w in range(32)]
    mask = 16
    while mask >= k:
        val = [max(val[l], val[l ^ mask]) for l in range(32)]
        mask >>= 1
    mask = k >> 1
    while mask > 0:
        val = [min(val[l], val[l ^ mask]) for l in range(32)]
        mask >>= 1
    assert len(set(val)) == 1 or k < 32  # every lane agrees once the min steps cover all groups
    return val[0]


@pytest.mark.parametrize("k", [2, 4, 8, 16, 32])
def test_rough_kth_is_the_shuffle_network(k):
    rng = np.random.default_rng(k)
    for _ in range(20):
        cm = rng.integers(-128, 128, size=1024).astype(np.int32)
        got = S.rough_kth_code(cm, k)
        assert got == int(_shuffle_network_kth(cm, k))
        # "rough but safe": never above the true k-th largest of the warp maxima
        warp = np.sort(cm.reshape(32, 32).max(axis=1))[::-1]
        assert got <= warp[k - 1]


@pytest.mark.parametrize("k", [2, 8, 32])
def test_topk_candidates_and_probabilities_by_brute_force(k):
    rng = np.random.default_rng(10 + k)
    V, scale = 3000, 0.11
    codes = np.clip(rng.standard_normal(V) * 40, -127, 127).astype(np.int8)
    tok, amb, ids, probs = S.topk_sample_row(codes, k, scale, 0.5)
    kth = S.rough_kth_code(S._class_max(codes), k)
    # brute force: per class the first id of the class maximum, kept when it reaches the threshold
    want = []
    for t in range(1024):
        cls = np.arange(t, V, 1024)
        best = cls[np.argmax(codes[cls])]
        if codes[best] >= kth:
            want.append(int(best))
    assert sorted(ids.tolist()) == sorted(want)
    assert len(want) >= k  # the threshold never cuts below k candidates
    np.testing.assert_allclose(probs, softmax(codes[ids].astype(np.float64) * scale), rtol=1e-5)
    assert tok in want


def test_choice_walks_the_classes_in_thread_order():
    codes = np.full(2048, -100, np.int8)
    # one peak in each of the warps 0..3 (a group modulo 4 each): the rough 4th maximum is 90
    codes[[5, 1064, 70, 1124]] = [100, 90, 100, 100]  # classes 5, 40, 70, 100
    codes[1029] = 100  # class 5 again, a later id: the first one stays the class's candidate
    _, _, ids, probs = S.topk_sample_row(codes, 4, 0.05, 0.5)
    assert ids.tolist() == [5, 1064, 70, 1124]
    edges = np.cumsum(probs)
    for x, want in [(1e-6, 5), (edges[0] - 1e-3, 5), (edges[0] + 1e-3, 1064), (edges[1] + 1e-3, 70),
                    (edges[2] + 1e-3, 1124), (1.0, 1124)]:
        assert S.topk_sample_row(codes, 4, 0.05, x)[0] == want
    # frequencies follow the probabilities
    rng = np.random.default_rng(0)
    draws = [S.topk_sample_row(codes, 4, 0.05, x)[0] for x in rng.uniform(0, 1, 3000)]
    for i, p in zip(ids, probs):
        assert abs(draws.count(int(i)) / 3000 - p) < 0.03


@pytest.mark.parametrize("p", [0.05, 0.5, 0.9, 1.0])
def test_topp_threshold_by_brute_force(p):
    rng = np.random.default_rng(int(p * 100))
    V, scale = 5000, 0.15
    codes = np.clip(rng.standard_normal(V) * 35, -127, 127).astype(np.int8)
    cm = S._class_max(codes)
    thr, _ = S.topp_threshold_code(cm, p, scale)
    # brute force over the sorted class maxima in float64
    srt = np.sort(cm)[::-1].astype(np.float64) * np.float64(np.float32(scale))
    ex = np.exp(np.maximum(srt - srt[0], -64.0))
    pre, total, want = 0.0, ex.sum(), srt[0]
    for v, e in zip(srt, ex):
        pre += e
        if pre > p * total:
            break
        want = v
    assert thr == int(round(want / np.float64(np.float32(scale))))
    if p == 1.0:
        assert thr == cm.min()
    tok, _, ids, probs = S.topp_sample_row(codes, p, scale, 0.3)
    assert set(codes[ids] >= thr) == {True} and abs(probs.sum() - 1) < 1e-9 and tok in ids
    # the nucleus holds at least p of the class-maximum mass, or is the single largest class
    mass = ex[srt >= thr * np.float64(np.float32(scale)) - 1e-9].sum() / total
    assert mass <= p + 1e-9 or (srt >= want).sum() == (srt == srt[0]).sum() or thr == int(cm.max())


def test_topp_keeps_the_largest_when_it_alone_exceeds_p():
    codes = np.full(4096, -90, np.int8)
    codes[77] = 120
    tok, amb, ids, probs = S.topp_sample_row(codes, 0.3, 0.2, 0.9)
    assert ids.tolist() == [77] and tok == 77


# ---- encoder-decoder form: logit = code * scale + bias[id] ---------------------------------
def _row(rng, V, spread=35):
    return np.clip(rng.standard_normal(V) * spread, -127, 127).astype(np.int8)


@pytest.mark.parametrize("k", [2, 4, 32])
def test_decoder_topk_reduces_to_the_code_form_without_bias(k):
    """With a zero bias the float route must give what the int8-code route gives (the two are
    written separately: float thresholds and comparisons here, integer ones there)."""
    rng = np.random.default_rng(30 + k)
    V, scale = 4000, 0.07
    codes = _row(rng, V)
    for x in [0.01, 0.37, 0.99]:
        a = S.dec_topk_sample_row(codes, np.zeros(V, np.float16), k, scale, x)
        b = S.topk_sample_row(codes, k, scale, x)
        assert a[0] == b[0] and a[2].tolist() == b[2].tolist()
        np.testing.assert_allclose(a[3], b[3], rtol=1e-6)


@pytest.mark.parametrize("p", [0.1, 0.6, 1.0])
def test_decoder_topp_reduces_to_the_code_form_without_bias(p):
    rng = np.random.default_rng(int(p * 10))
    V, scale = 6000, 0.12
    codes = _row(rng, V)
    a = S.dec_topp_sample_row(codes, np.zeros(V, np.float32), p, scale, 0.41)
    b = S.topp_sample_row(codes, p, scale, 0.41)
    assert a[0] == b[0] and a[2].tolist() == b[2].tolist()
    np.testing.assert_allclose(a[3], b[3], rtol=1e-6)


def test_decoder_bias_enters_the_threshold_the_candidates_and_the_probabilities():
    """Brute force in float64 with a bias large enough to reorder the ids: a route that dropped
    the bias anywhere (class maxima, threshold test, exps) gives other candidates or weights."""
    rng = np.random.default_rng(5)
    V, scale, k = 3000, 0.05, 8
    codes = _row(rng, V, 20)
    bias = (rng.standard_normal(V) * 3).astype(np.float16)
    logit = codes.astype(np.float64) * np.float64(np.float32(scale)) + bias.astype(np.float64)
    tok, _, ids, probs = S.dec_topk_sample_row(codes, bias, k, scale, 0.5)
    cmax = np.array([logit[t::1024].max() for t in range(1024)])
    warp = cmax.reshape(32, 32).max(axis=1)
    kth = min(warp[g::k].max() for g in range(k))
    want = [int(np.arange(t, V, 1024)[np.argmax(logit[t::1024])]) for t in range(1024)
            if cmax[t] >= kth - 1e-6]
    assert sorted(ids.tolist()) == sorted(want) and len(want) >= k
    np.testing.assert_allclose(probs, softmax(logit[ids]), rtol=2e-4)
    assert sorted(ids.tolist()) != sorted(S.topk_sample_row(codes, k, scale, 0.5)[2].tolist())
    # greedy: the bias decides
    bias2 = np.zeros(V, np.float32)
    bias2[1234] = 100.0
    assert S.dec_greedy_row(codes, bias2, scale) == 1234
    assert S.dec_greedy_row(np.zeros(V, np.int8), np.zeros(V, np.float32), scale) == 0  # first of ties


def test_decoder_topp_nucleus_by_brute_force_with_bias():
    rng = np.random.default_rng(8)
    V, scale, p = 5000, 0.1, 0.5
    codes = _row(rng, V, 25)
    bias = (rng.standard_normal(V) * 2).astype(np.float32)
    logit = S.biased_logits(codes, bias, scale).astype(np.float64)
    cm = np.array([logit[t::1024].max() for t in range(1024)])
    srt = np.sort(cm)[::-1]
    ex = np.exp(np.maximum(srt - srt[0], -64.0))
    pre, total, want = 0.0, ex.sum(), srt[0]
    for v, e in zip(srt, ex):
        pre += e
        if pre > p * total:
            break
        want = v
    thr, _ = S.dec_topp_threshold(S._class_max_f(logit.astype(np.float32)), p)
    assert abs(float(thr) - want) < 1e-6
    tok, _, ids, probs = S.dec_topp_sample_row(codes, bias, p, scale, 0.77)
    assert (logit[ids] >= want - 1e-6).all() and tok in ids and abs(probs.sum() - 1) < 1e-9


def test_decoder_step_keeps_ended_rows_and_reports_the_flag():
    rng = np.random.default_rng(2)
    V, eos, max_step = 2000, 7, 6
    logits = np.stack([_row(rng, V) for _ in range(3)])
    bias = np.zeros(V, np.float16)
    ids = np.full((3, max_step), 1, np.int32)
    ids[1, 2] = eos
    draws = np.zeros(3, np.int64)
    unf, _ = S.dec_sample_step(logits, bias, ids, 3, eos, 0.1, k=4, seed=11, draws=draws)
    assert ids[1, 3] == eos and draws.tolist() == [1, 0, 1] and unf == 1
    assert ids[0, 3] == S.dec_topk_sample_row(logits[0], bias, 4, 0.1, S.uniform_of_draw(11, 0, 0))[0]
    # every row picks the end token: nothing unfinished
    bias_eos = np.zeros(V, np.float32)
    bias_eos[eos] = 1000.0
    ids2 = np.full((3, max_step), 1, np.int32)
    unf, _ = S.dec_sample_step(logits, bias_eos, ids2, 1, eos, 0.1, k=1)
    assert unf == 0 and (ids2[:, 1] == eos).all()
