"""GPU: the beam-search step that allocates nothing (``lsh_beam_search_step_noalloc_i8I_f16``)
against the entry point it is a variant of (``lsh_beam_search_step_i8I_f16``, whose
proposal workspace the caller brings), through the C ABI.

Both run the same kernels, so every output must be identical bit for bit.  Two calls in a
row share the library's static workspace, the second with a smaller input: what the first
call left behind must not leak into the second.  A step beyond the static workspace's
65536 proposals is rejected.
"""
import numpy as np
import pytest
import torch

from helpers import DEV, to_dev, to_np

pytestmark = pytest.mark.gpu


def _k():
    from lightseq_amd import kernels
    return kernels


def _state(rng, batch, beam, vocab, max_step, cur_step, end_id):
    rows = batch * beam
    logits = np.clip(rng.standard_normal((rows, vocab)) * 32, -127, 127).astype(np.int8)
    logits[::2, end_id] = 100
    bias = (rng.standard_normal(vocab) * 0.05).astype(np.float16)
    alive = rng.integers(4, vocab, size=(rows, max_step), dtype=np.int32)
    alive[:, 0] = 2
    if cur_step > 0:
        alive[rng.random(rows) < 0.3, cur_step] = end_id
        probs = (-rng.random(rows) * 5 * cur_step).astype(np.float32)
    else:
        probs = np.where(np.arange(rows) % beam == 0, 0.0, -1000.0).astype(np.float32)
    score = (-rng.random(rows) * 8 - 2000.0 * (np.arange(rows) // beam)).astype(np.float32)
    return logits, bias, probs, score, alive


def _run(state, batch, beam, vocab, max_step, cur_step, end_id, static):
    logits, bias, probs, score, alive = state
    rows = batch * beam
    new_alive = torch.zeros(rows, max_step, dtype=torch.int32, device=DEV)
    p_d, s_d = to_dev(probs), to_dev(score)
    parent = torch.full((rows,), -7, dtype=torch.int32, device=DEV)
    fin = torch.full((1,), -1, dtype=torch.int32, device=DEV)
    dq, ln = 2.5 / 127, _k().length_norm(cur_step + 1, 0.6)
    if static:
        _k().beam_search_step_noalloc_i8I(to_dev(logits), to_dev(bias), p_d, s_d, to_dev(alive),
                                          new_alive, parent, fin, dq, vocab, max_step, ln, cur_step,
                                          batch, beam, end_id)
    else:
        top_s = torch.zeros(rows * beam, dtype=torch.float32, device=DEV)
        top_i = torch.zeros(rows * beam, dtype=torch.int32, device=DEV)
        _k().beam_search_step_i8I(to_dev(logits), to_dev(bias), p_d, s_d, to_dev(alive), new_alive,
                                  top_s, top_i, parent, fin, dq, vocab, max_step, ln, cur_step,
                                  batch, beam, end_id)
    return [to_np(t).copy() for t in (new_alive, p_d, s_d, parent, fin)]


# (first call, second call): batch, beam, vocab, max_step, cur_step
PAIRS = [
    ((16, 4, 32000, 66, 17), (3, 4, 1000, 32, 5)),       # Transformer-big step, then a small one
    ((4, 8, 5000, 16, 4), (2, 2, 777, 16, 0)),
    ((2, 32, 2100, 16, 1), (1, 4, 40000, 16, 2)),        # widest beam; then the looping top-k
]


@pytest.mark.parametrize("first,second", PAIRS)
def test_noalloc_step_equals_workspace_step_twice_in_a_row(rng, first, second):
    end_id = 3
    for batch, beam, vocab, max_step, cur_step in (first, second):
        state = _state(rng, batch, beam, vocab, max_step, cur_step, end_id)
        want = _run(state, batch, beam, vocab, max_step, cur_step, end_id, static=False)
        got = _run(state, batch, beam, vocab, max_step, cur_step, end_id, static=True)
        for g, w, what in zip(got, want, ("alive_seq", "seq_probs", "seq_score", "parent",
                                          "num_finished")):
            np.testing.assert_array_equal(g, w, err_msg=what)
        assert got[4][0] >= 0


def test_noalloc_step_rejects_sizes_beyond_its_workspace():
    from lightseq_amd.lib import LSHError
    z8 = torch.zeros(64, dtype=torch.int8, device=DEV)
    zh = torch.zeros(64, dtype=torch.float16, device=DEV)
    zf = torch.zeros(64, dtype=torch.float32, device=DEV)
    zi = torch.zeros(64, dtype=torch.int32, device=DEV)
    zj = torch.zeros(64, dtype=torch.int32, device=DEV)
    with pytest.raises(LSHError, match="65536"):
        _k().beam_search_step_noalloc_i8I(z8, zh, zf, zf, zi, zj, zi, zi, 1.0, 8, 8, 1.0, 0, 65, 32,
                                          1)
    with pytest.raises(LSHError, match="beam_size"):
        _k().beam_search_step_noalloc_i8I(z8, zh, zf, zf, zi, zj, zi, zi, 1.0, 8, 8, 1.0, 0, 1, 33,
                                          1)
