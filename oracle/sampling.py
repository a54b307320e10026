"""CPU restatement of the GPT random-sampling kernels.  TEST INFRASTRUCTURE ONLY, like the
rest of ``oracle/``.

Follows ``ker_topk_sample_i8I<k>`` (inference/kernels/gptKernels_int8.cc.cu:252-420) and
``ker_topp_sample_i8I`` (:465-640) as they act with 1024 threads per block, which is what
the model launches (inference/model/quant_gpt_encoder.cc.cu:399-487): thread t sees the
vocabulary ids congruent to t modulo 1024 (a *class*), the candidate set holds at most one id
per class, and the choice walks the classes in thread order with one uniform number.

What the reference leaves open, and what is fixed here instead:

* the uniform numbers come from a cuRAND state seeded with ``clock()``
  (kernels/transformerKernels.cc.cu:2270-2274): no stream of numbers is defined by the
  source.  Here they are Philox4x32-10 outputs (key = seed, counter = (draw, 0, row, 0), word
  0), mapped to (0, 1] as ``curand_uniform`` maps 32 bits; ``philox4x32_10`` is pinned by the
  published known-answer vectors of that generator.
* ``ker_topp_sample_i8I`` compares every thread's prefix sum with a threshold that only the
  last thread assigns (:533-539: the other threads read an uninitialised local), so its
  nucleus is undefined behaviour; restated here is what the code intends: the nucleus is the
  longest prefix of the descending class maxima whose exp-sum stays within p of the total, and
  at least the largest one.  **Parity unpinned** for top-p.
* float sums over the 1024 threads run in the order of the reference's shuffle trees and
  ``cub::BlockScan``; here they are float64, and a draw that falls within ``AMBIGUOUS`` of a
  boundary of the cumulative distribution is reported as ambiguous instead of decided.
"""
import numpy as np

THREADS = 1024
LOGIT_THRESH_MIN = -64.0  # kernels/transformerKernels.h:11
AMBIGUOUS = 1e-5


def philox4x32_10(counter, key):
    """Philox4x32-10 (Salmon et al., "Parallel random numbers: as easy as 1, 2, 3", SC'11):
    counter 4 x uint32, key 2 x uint32 -> 4 x uint32."""
    c = [int(x) & 0xFFFFFFFF for x in counter]
    k = [int(x) & 0xFFFFFFFF for x in key]
    for _ in range(10):
        p0 = 0xD2511F53 * c[0]
        p1 = 0xCD9E8D57 * c[2]
        c = [((p1 >> 32) ^ c[1] ^ k[0]) & 0xFFFFFFFF, p1 & 0xFFFFFFFF,
             ((p0 >> 32) ^ c[3] ^ k[1]) & 0xFFFFFFFF, p0 & 0xFFFFFFFF]
        k = [(k[0] + 0x9E3779B9) & 0xFFFFFFFF, (k[1] + 0xBB67AE85) & 0xFFFFFFFF]
    return c


def uniform_of_draw(seed, row, draw):
    """The uniform number in (0, 1] of draw ``draw`` of sequence ``row`` (float32, as
    ``curand_uniform`` forms it: x * 2^-32 + 2^-33)."""
    x = philox4x32_10((draw & 0xFFFFFFFF, 0, row, 0), (seed & 0xFFFFFFFF, (seed >> 32) & 0xFFFFFFFF))[0]
    return np.float32(np.float32(x) * np.float32(2.0 ** -32) + np.float32(2.0 ** -33))


def _class_max(codes):
    """Per-class maximum code of one row (class t: ids t, t + 1024, ...); -129 = empty class."""
    v = len(codes)
    cm = np.full(THREADS, -129, np.int32)
    for t in range(min(THREADS, v)):
        cm[t] = int(codes[t::THREADS].max())
    return cm


def rough_kth_code(class_max, k):
    """kernels/common.h:118-137 on the class maxima: maxima of the 32 warps of 32 threads, the
    maximum over the warps that agree modulo k, the minimum over the k groups."""
    warp = class_max.reshape(32, 32).max(axis=1)
    return int(min(warp[g::k].max() for g in range(k)))


def _candidates(codes, threshold_code, dequant_scale):
    """Step 2 of both kernels (:318-345, :565-590): per class, among the ids whose logit is at
    least the threshold, the first one with the largest exp(max(logit - max, thresh_min)).
    Returns (class index, token id, exp) arrays over the classes that hold a candidate."""
    s = np.float32(dequant_scale)
    logit = codes.astype(np.float32) * s
    mx = logit.max()
    ex = np.exp(np.maximum(logit - mx, np.float32(LOGIT_THRESH_MIN)).astype(np.float32)).astype(np.float32)
    thr = np.float32(threshold_code) * s if threshold_code > -129 else np.float32(-np.inf)
    ts, ids, es = [], [], []
    for t in range(min(THREADS, len(codes))):
        idx = np.arange(t, len(codes), THREADS)
        ok = logit[idx] >= thr
        if not ok.any():
            continue
        cand = idx[ok]
        j = int(np.argmax(ex[cand]))  # first of the largest
        ts.append(t)
        ids.append(int(cand[j]))
        es.append(float(ex[cand[j]]))
    return np.array(ts), np.array(ids), np.array(es, np.float64)


def _choose(ts, ids, es, x):
    """:347-395: probabilities, inclusive prefix in thread order, the first thread whose prefix
    reaches x; when rounding leaves none, the lowest thread of the largest probability.
    Returns (token id, ambiguous)."""
    p = es / es.sum()
    pre = np.cumsum(p)
    x = float(x)
    hit = np.nonzero(x <= pre)[0]
    amb = bool(np.any(np.abs(pre[:-1] - x) < AMBIGUOUS)) or (len(hit) == 0)
    if len(hit) == 0:
        return int(ids[int(np.argmax(p))]), amb
    return int(ids[hit[0]]), amb


def topk_sample_row(codes, k, dequant_scale, x):
    """One row of ``ker_topk_sample_i8I<k>``, k in {2, 4, 8, 16, 32}: (token id, ambiguous,
    candidate ids, candidate probabilities)."""
    codes = np.asarray(codes, np.int8)
    kth = rough_kth_code(_class_max(codes), k)
    ts, ids, es = _candidates(codes, kth, dequant_scale)
    tok, amb = _choose(ts, ids, es, x)
    return tok, amb, ids, es / es.sum()


def topp_threshold_code(class_max, p, dequant_scale):
    """The smallest class maximum inside the nucleus (:497-547 as intended): class maxima in
    descending order, exps, inclusive prefix; the nucleus is the prefix within p of the total,
    and never empty.  Returns (code, ambiguous: a prefix sum lies at the boundary)."""
    s = np.float32(dequant_scale)
    srt = np.sort(class_max[class_max > -129])[::-1]
    logit = srt.astype(np.float32) * s
    ex = np.exp(np.maximum(logit - logit[0], np.float32(LOGIT_THRESH_MIN)).astype(np.float32)).astype(np.float64)
    # absent classes (vocabulary below 1024 ids) hold -inf: exp(thresh_min) each, as the kernel adds
    total = ex.sum() + (THREADS - len(srt)) * float(np.exp(np.float32(LOGIT_THRESH_MIN)))
    pre = np.cumsum(ex)
    inside = np.nonzero(pre <= p * total)[0]
    amb = bool(np.any(np.abs(pre - p * total) < AMBIGUOUS * total))
    return (int(srt[inside[-1]]) if len(inside) else int(srt[0])), amb


def topp_sample_row(codes, p, dequant_scale, x):
    """One row of ``ker_topp_sample_i8I``: (token id, ambiguous, candidate ids, probabilities)."""
    codes = np.asarray(codes, np.int8)
    thr, amb0 = topp_threshold_code(_class_max(codes), p, dequant_scale)
    ts, ids, es = _candidates(codes, thr, dequant_scale)
    tok, amb = _choose(ts, ids, es, x)
    return tok, amb or amb0, ids, es / es.sum()


# ---------------------------------------------------------------------------------------------
# Encoder-decoder model: ker_topk_sample_i8I<k> / ker_topp_sample_i8I of
# inference/kernels/transformerKernels_int8.cc.cu:1908-2290.  A logit is
# float(code) * dequant_scale + logit_bias[id] (:1945-1947), so everything runs on float32
# logits; the class structure, the candidate rule and the choice are those above.
#
# Not defined by the reference, fixed here (parity unpinned):
# * whether the compiler fuses the product and the sum of a logit: rounded separately here;
# * k == 1: every thread holding the maximum stores its id (:2047-2049, a race): the first id;
# * top-p: the class maximum is formed as fmaxf(m, code * scale) + bias inside the loop over the
#   class's ids (:2136-2137), which adds up the bias of every id; restated is the maximum of the
#   biased logits, and the intended nucleus as for the GPT kernel.
# ---------------------------------------------------------------------------------------------
def biased_logits(codes, bias, dequant_scale):
    """float32 logits of one row: the product and the sum rounded separately."""
    prod = (np.asarray(codes, np.int8).astype(np.float32) * np.float32(dequant_scale)).astype(np.float32)
    return (prod + np.asarray(bias).astype(np.float32)).astype(np.float32)


def _class_max_f(logit):
    """Per-class maximum logit (class t: ids t, t + 1024, ...); -inf = empty class."""
    cm = np.full(THREADS, -np.inf, np.float32)
    for t in range(min(THREADS, len(logit))):
        cm[t] = logit[t::THREADS].max()
    return cm


def rough_kth_value(class_max, k):
    """kernels/common.h:118-137 on float class maxima."""
    warp = class_max.reshape(32, 32).max(axis=1)
    return np.float32(min(warp[g::k].max() for g in range(k)))


def _candidates_f(logit, thr):
    """Step 2 (:1969-1990, :2185-2204): per class, among the ids whose logit reaches the
    threshold, the first one with the largest exp(max(logit - max, thresh_min))."""
    mx = logit.max()
    ex = np.exp(np.maximum(logit - mx, np.float32(LOGIT_THRESH_MIN)).astype(np.float32)).astype(np.float32)
    ts, ids, es = [], [], []
    for t in range(min(THREADS, len(logit))):
        idx = np.arange(t, len(logit), THREADS)
        ok = logit[idx] >= thr
        if not ok.any():
            continue
        cand = idx[ok]
        j = int(np.argmax(ex[cand]))
        ts.append(t)
        ids.append(int(cand[j]))
        es.append(float(ex[cand[j]]))
    return np.array(ts), np.array(ids), np.array(es, np.float64)


def dec_greedy_row(codes, bias, dequant_scale):
    """k == 1: the first id of the largest logit."""
    return int(np.argmax(biased_logits(codes, bias, dequant_scale)))


def dec_topk_sample_row(codes, bias, k, dequant_scale, x):
    """One row of the decoder's ``ker_topk_sample_i8I<k>``, k in {2, 4, 8, 16, 32}: (token id,
    ambiguous, candidate ids, candidate probabilities)."""
    logit = biased_logits(codes, bias, dequant_scale)
    kth = rough_kth_value(_class_max_f(logit), k)
    ts, ids, es = _candidates_f(logit, kth)
    tok, amb = _choose(ts, ids, es, x)
    return tok, amb, ids, es / es.sum()


def dec_topp_threshold(class_max, p):
    """The smallest class maximum inside the nucleus: (value, ambiguous)."""
    srt = np.sort(class_max[np.isfinite(class_max)])[::-1]
    ex = np.exp(np.maximum(srt - srt[0], np.float32(LOGIT_THRESH_MIN)).astype(np.float32)).astype(np.float64)
    total = ex.sum() + (THREADS - len(srt)) * float(np.exp(np.float32(LOGIT_THRESH_MIN)))
    pre = np.cumsum(ex)
    inside = np.nonzero(pre <= p * total)[0]
    amb = bool(np.any(np.abs(pre - p * total) < AMBIGUOUS * total))
    return (np.float32(srt[inside[-1]]) if len(inside) else np.float32(srt[0])), amb


def dec_topp_sample_row(codes, bias, p, dequant_scale, x):
    """One row of the decoder's ``ker_topp_sample_i8I``."""
    logit = biased_logits(codes, bias, dequant_scale)
    thr, amb0 = dec_topp_threshold(_class_max_f(logit), p)
    ts, ids, es = _candidates_f(logit, thr)
    tok, amb = _choose(ts, ids, es, x)
    return tok, amb or amb0, ids, es / es.sum()


def dec_sample_step(logits, bias, ids, cur_len, eos_id, dequant_scale, k=0, p=0.0, seed=0, draws=None):
    """One step of QuantDecoder::sample / ::topk_greedy_search
    (inference/model/quant_decoder.cc.cu:952-998, 1101-1130) on ids [rows, max_step] in place:
    a row whose last token is ``eos_id`` gets another one and draws nothing; otherwise column
    ``cur_len`` receives the token.  ``draws`` [rows] counts the uniform numbers used per row
    (updated).  Returns (unfinished flag, list of rows whose draw was ambiguous)."""
    rows = ids.shape[0]
    unfinished, ambiguous = 0, []
    for b in range(rows):
        if cur_len > 1 and ids[b, cur_len - 1] == eos_id:
            ids[b, cur_len] = eos_id
            continue
        if k == 1:
            tok = dec_greedy_row(logits[b], bias, dequant_scale)
        else:
            x = uniform_of_draw(seed, b, int(draws[b]))
            draws[b] += 1
            if k > 1:
                tok, amb, _, _ = dec_topk_sample_row(logits[b], bias, k, dequant_scale, x)
            else:
                tok, amb, _, _ = dec_topp_sample_row(logits[b], bias, p, dequant_scale, x)
            if amb:
                ambiguous.append(b)
        ids[b, cur_len] = tok
        if tok != eos_id:
            unfinished = 1
    return unfinished, ambiguous
