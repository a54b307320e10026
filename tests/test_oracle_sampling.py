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
