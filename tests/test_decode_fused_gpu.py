"""GPU parity of the fused decode-step launches against the launcher sequences they replace,
through the C ABI: integer outputs bit for bit.
"""
import numpy as np
import pytest
import torch

from helpers import DEV, to_dev, to_np

pytestmark = pytest.mark.gpu


def _k():
    from lightseq_amd import kernels
    return kernels


@pytest.mark.parametrize("M,heads,d,K,max_step,step", [(16, 16, 64, 1024, 40, 7), (64, 16, 64, 1024, 24, 23),
                                                       (3, 4, 32, 256, 9, 0), (7, 2, 128, 384, 5, 4),
                                                       (200, 4, 64, 256, 6, 2)])
def test_qkv_product_with_cache_append_equals_the_pair(rng, M, heads, d, K, max_step, step):
    """lsh_gemm_i8_decself_qkv_i8o == lsh_gemm_i8_i8o followed by
    ker_arrange_decself_qkv_i8I_i8O: q codes, and the cache slots (all other slots untouched)."""
    H = heads * d
    a = rng.integers(-127, 128, size=(M, K), dtype=np.int8)
    w = rng.integers(-127, 128, size=(3 * H, K), dtype=np.int8)
    bias = (rng.standard_normal(3 * H) * 0.4).astype(np.float16)
    alpha = 2.5 / (np.sqrt(K) * 127)
    ds, qs = 3.0 / 127, 127 / 3.5
    fill = rng.integers(-127, 128, size=(2, M, heads, max_step, d), dtype=np.int8)

    # reference sequence
    c = torch.zeros((M, 3 * H), dtype=torch.int8, device=DEV)
    _k().gemm_i8_i8o(to_dev(a), to_dev(w), c, M, 3 * H, K, alpha)
    q0 = torch.zeros((M, H), dtype=torch.int8, device=DEV)
    kv0 = to_dev(fill.copy())
    _k().ker_arrange_decself_qkv_i8I_i8O_launcher(M, H, c, to_dev(bias), q0, kv0[0], kv0[1], heads, d,
                                                  max_step, step, 1024, ds, qs)
    # fused
    q1 = torch.full((M, H), 5, dtype=torch.int8, device=DEV)
    kv1 = to_dev(fill.copy())
    _k().gemm_i8_decself_qkv_i8o(to_dev(a), to_dev(w), to_dev(bias), q1, kv1[0], kv1[1], M, H, K, heads,
                                 max_step, step, alpha, ds, qs)
    np.testing.assert_array_equal(to_np(q1), to_np(q0))
    np.testing.assert_array_equal(to_np(kv1), to_np(kv0))
    # only slot `step` of the caches changed
    got = to_np(kv1)
    keep = np.ones(max_step, dtype=bool)
    keep[step] = False
    np.testing.assert_array_equal(got[:, :, :, keep, :], fill[:, :, :, keep, :])


def test_qkv_product_with_cache_append_rejects_bad_arguments(rng):
    from lightseq_amd.lib import LSHError
    M, heads, d, K, max_step = 4, 2, 24, 128, 4  # d not a multiple of 16
    H = heads * d
    a = torch.zeros((M, K), dtype=torch.int8, device=DEV)
    w = torch.zeros((3 * H, K), dtype=torch.int8, device=DEV)
    bias = torch.zeros(3 * H, dtype=torch.float16, device=DEV)
    q = torch.zeros((M, H), dtype=torch.int8, device=DEV)
    kv = torch.zeros((2, M, heads, max_step, d), dtype=torch.int8, device=DEV)
    with pytest.raises(LSHError):
        _k().gemm_i8_decself_qkv_i8o(a, w, bias, q, kv[0], kv[1], M, H, K, heads, max_step, 0, 1e-3, 1e-2,
                                     30.0)
    d = 32
    H = heads * d
    w = torch.zeros((3 * H, K), dtype=torch.int8, device=DEV)
    bias = torch.zeros(3 * H, dtype=torch.float16, device=DEV)
    q = torch.zeros((M, H), dtype=torch.int8, device=DEV)
    kv = torch.zeros((2, M, heads, max_step, d), dtype=torch.int8, device=DEV)
    with pytest.raises(LSHError):  # step outside the cache
        _k().gemm_i8_decself_qkv_i8o(a, w, bias, q, kv[0], kv[1], M, H, K, heads, max_step, max_step, 1e-3,
                                     1e-2, 30.0)


@pytest.mark.parametrize("B,beam,heads,S,d", [(3, 4, 2, 37, 64), (2, 2, 3, 64, 32), (1, 4, 2, 130, 128),
                                              (16, 4, 16, 64, 64), (2, 2, 2, 200, 64), (2, 3, 2, 300, 32),
                                              (1, 5, 2, 60, 128), (2, 1, 4, 128, 64)])
def test_cross_attention_vector_kernel_equals_the_scalar_one(rng, B, beam, heads, S, d):
    """lsh_encdec_attention_f16 picks a vector-load kernel for 16-byte aligned operands and
    head sizes 32 / 64 / 128; for sources longer than 16 loads of a wavefront cover (8192 / d
    keys) it sums in the same order as the general kernel, so a query buffer shifted by 8 bytes
    (general kernel) gives the same context bits and codes.  Shorter sources run the kernel that
    keeps keys, values and probabilities in registers and sums in another order: the same fp16
    rounding points, context within one fp16 step of the magnitudes involved and codes within
    +-1 on at most 0.5 % of the elements."""
    q = (rng.standard_normal((B, heads, beam, d)) * 0.7).astype(np.float16)
    k = (rng.standard_normal((B, heads, S, d)) * 0.7).astype(np.float16)
    v = (rng.standard_normal((B, heads, S, d)) * 0.7).astype(np.float16)
    mask = np.zeros((B, S), dtype=np.int32)
    for b in range(B):
        mask[b, rng.integers(S // 2, S + 1):] = 1
    qs = 127 / 1.5
    outs = []
    for shift in (0, 4):  # halfs: 0 keeps the 16-byte alignment, 4 breaks it
        qbuf = torch.zeros(q.size + 8, dtype=torch.float16, device=DEV)
        qd = qbuf[shift:shift + q.size].view(B, heads, beam, d)
        qd.copy_(to_dev(q))
        ctx = torch.zeros((B, heads, beam, d), dtype=torch.float16, device=DEV)
        ctx_q = torch.zeros((B * beam, heads * d), dtype=torch.int8, device=DEV)
        _k().encdec_attention(qd, to_dev(k), to_dev(v), to_dev(mask), ctx, ctx_q, qs, B, beam, heads, S, d)
        outs.append((to_np(ctx), to_np(ctx_q)))
    if S > 16 * (512 // d):
        np.testing.assert_array_equal(outs[0][0].view(np.uint16), outs[1][0].view(np.uint16))
        np.testing.assert_array_equal(outs[0][1], outs[1][1])
    else:
        from conftest import assert_codes_close
        np.testing.assert_allclose(outs[0][0].astype(np.float32), outs[1][0].astype(np.float32), atol=2e-3,
                                   rtol=2e-3)
        assert_codes_close(outs[0][1], outs[1][1], max_frac=5e-3)


@pytest.mark.parametrize("batch,beam,heads,d,K", [(16, 4, 16, 64, 1024), (3, 2, 4, 32, 256), (2, 1, 2, 128, 384),
                                                  (40, 4, 4, 64, 256)])
def test_cross_attention_q_product_equals_the_pair(rng, batch, beam, heads, d, K):
    """lsh_gemm_i8_encdec_q_f16 == lsh_gemm_i8_i8o followed by ker_arrange_encdec_q_i8I, bit for bit."""
    M, H = batch * beam, heads * d
    a = rng.integers(-127, 128, size=(M, K), dtype=np.int8)
    w = rng.integers(-127, 128, size=(H, K), dtype=np.int8)
    bias = (rng.standard_normal(H) * 0.4).astype(np.float16)
    alpha, ds = 2.5 / (np.sqrt(K) * 127), 3.0 / 127
    c = torch.zeros((M, H), dtype=torch.int8, device=DEV)
    _k().gemm_i8_i8o(to_dev(a), to_dev(w), c, M, H, K, alpha)
    q0 = torch.zeros((batch, heads, beam, d), dtype=torch.float16, device=DEV)
    _k().ker_arrange_encdec_q_i8I_launcher(M, H, c, to_dev(bias), q0, beam, d, heads, 1024, ds)
    q1 = torch.full((batch, heads, beam, d), 3.0, dtype=torch.float16, device=DEV)
    _k().gemm_i8_encdec_q(to_dev(a), to_dev(w), to_dev(bias), q1, M, H, K, beam, heads, alpha, ds)
    np.testing.assert_array_equal(to_np(q1).view(np.uint16), to_np(q0).view(np.uint16))


@pytest.mark.parametrize("M,heads,K,max_step,step", [
    (16, 16, 1024, 700, 639),   # GPT-2-medium decode step near the end: the cache requested first
    (16, 16, 1024, 1030, 256),  # ... every count of cache rows per lane of that kernel
    (16, 16, 1024, 1030, 383),
    (16, 16, 1024, 1030, 384),
    (3, 8, 512, 1030, 511),
    (16, 16, 1024, 1030, 767),
    (5, 2, 128, 1030, 1023),
    (2, 8, 512, 1030, 1024),    # ... and beyond it: rounds
    (16, 16, 1024, 700, 200),   # ... and where the stand-alone attention has the same group shape
    (16, 16, 1024, 200, 100),
    (64, 16, 1024, 66, 63),     # Transformer-big beam step: one wavefront per row
    (64, 16, 1024, 66, 0),
    (5, 8, 512, 40, 17),        # rows not a multiple of the row group, head count a multiple of 8
    (3, 2, 128, 300, 130),      # few heads, ragged row group
    (9, 4, 256, 90, 64),
])
def test_qkv_product_cache_append_and_attention_in_one_launch(rng, M, heads, K, max_step, step):
    """lsh_decself_qkv_attention_i8_f16 == lsh_gemm_i8_decself_qkv_i8o_f16 followed by
    lsh_decself_attention_i8: q codes and caches byte for byte; context codes byte for byte
    where the group shapes agree (more than 128 and at most 1024 cached steps), else within one
    code on at most 0.1 % (another summation tree)."""
    from conftest import assert_codes_close
    d, H = 64, heads * 64
    assert K == H
    x = rng.integers(-127, 128, size=(M, K), dtype=np.int8)
    w = rng.integers(-127, 128, size=(3 * H, K), dtype=np.int8)
    bias = (rng.standard_normal(3 * H) * 0.4).astype(np.float16)
    alpha = 2.5 / (np.sqrt(K) * 127)
    ds, qs = 3.0 / 127, 127 / 3.5
    attn_scale, cache_dq, ctx_qs = 0.125, 3.5 / 127, 127 / 2.0
    fill = rng.integers(-127, 128, size=(2, M, heads, max_step, d), dtype=np.int8)
    k = _k()
    xd, wd, bd = to_dev(x), to_dev(w), to_dev(bias)

    q0 = torch.zeros((M, H), dtype=torch.int8, device=DEV)
    kv0 = to_dev(fill.copy())
    ctx0 = torch.zeros((M, H), dtype=torch.int8, device=DEV)
    k.gemm_i8_decself_qkv_i8o(xd, wd, bd, q0, kv0[0], kv0[1], M, H, K, heads, max_step, step, alpha, ds, qs)
    k.decself_attention_i8(q0, kv0[0], kv0[1], ctx0, M * heads, step + 1, max_step, heads, d, attn_scale,
                           cache_dq, ctx_qs)

    q1 = torch.full((M, H), 5, dtype=torch.int8, device=DEV)
    kv1 = to_dev(fill.copy())
    ctx1 = torch.full((M, H), 7, dtype=torch.int8, device=DEV)
    k.decself_qkv_attention_i8(xd, wd, bd, q1, kv1[0], kv1[1], ctx1, M, H, heads, max_step, step, alpha, ds,
                               qs, attn_scale, cache_dq, ctx_qs)
    np.testing.assert_array_equal(to_np(q1), to_np(q0))
    np.testing.assert_array_equal(to_np(kv1), to_np(kv0))
    if 128 < step + 1 <= 1024:
        np.testing.assert_array_equal(to_np(ctx1), to_np(ctx0))
    else:
        assert_codes_close(to_np(ctx1), to_np(ctx0))


def test_qkv_product_and_attention_in_one_launch_rejects_what_it_does_not_cover():
    from lightseq_amd.lib import LSHError
    k = _k()

    def call(M, heads, d, max_step, step):
        H = heads * d
        z = lambda *s: torch.zeros(s, dtype=torch.int8, device=DEV)  # noqa: E731
        k.decself_qkv_attention_i8(z(M, H), z(3 * H, H), torch.zeros(3 * H, dtype=torch.float16, device=DEV),
                                   z(M, H), z(M, heads, max_step, d), z(M, heads, max_step, d), z(M, H), M, H,
                                   heads, max_step, step, 1e-3, 1e-2, 30.0, 0.125, 1e-2, 30.0)

    call(4, 2, 64, 8, 3)  # covered
    for bad in [(4, 2, 32, 8, 3),      # heads of 32: hidden != heads * 64
                (4, 3, 64, 8, 3),      # hidden 192 is not a multiple of 128
                (4, 32, 64, 8, 3),     # hidden 2048
                (4, 2, 64, 8, 8),      # step outside the cache
                (4, 2, 64, 5000, 3)]:  # cache longer than 4096
        with pytest.raises(LSHError):
            call(*bad)



@pytest.mark.parametrize("rows,hidden,vocab,step,post_ln,with_rb", [(64, 1024, 32000, 17, True, True),
                                                                      (16, 512, 1000, 0, False, True),
                                                                      (5, 768, 333, 3, True, True),
                                                                      (3, 132, 50, 6, False, True)])
def test_target_embedding_and_first_layer_norm_in_one_launch(rng, rows, hidden, vocab, step, post_ln, with_rb):
    """lsh_dec_emb_norm_layer_i8O_f16 == lsh_launch_dec_emb_i8I_vocab_major_f16 followed by
    lsh_ker_norm_layer_resual_i8O_f16 with the row kernel: codes and residual stream byte for
    byte (ids outside the table are clamped by both)."""
    k = _k()
    max_step = 9 + step
    emb = to_dev(rng.integers(-127, 128, size=(vocab, hidden), dtype=np.int8))
    pos = to_dev((rng.standard_normal((max_step, hidden)) * 0.5).astype(np.float16))
    tokens = rng.integers(0, vocab, size=(rows, max_step), dtype=np.int32)
    tokens[0, step] = vocab + 7  # outside the table
    tokens = to_dev(tokens)
    g = to_dev((1 + 0.1 * rng.standard_normal(hidden)).astype(np.float16))
    b = to_dev((0.1 * rng.standard_normal(hidden)).astype(np.float16))
    rb = to_dev((0.1 * rng.standard_normal(hidden)).astype(np.float16)) if with_rb else None
    dq, qs = 0.6 / 127, 127 / 3.0

    res0 = torch.zeros((rows, hidden), dtype=torch.float16, device=DEV)
    q0 = torch.zeros((rows, hidden), dtype=torch.int8, device=DEV)
    prev = k.layer_norm_row_kernel(True)
    try:
        k.launch_dec_emb_i8I(emb, pos, tokens, None, None, res0, rows, 1, hidden, vocab, step, max_step, 0,
                             dq, True, vocab_major=True)
        k.ker_norm_layer_resual_i8O_launcher(rows, hidden, res0, q0, g, b, rb, 1024, qs, post_ln)
    finally:
        k.layer_norm_row_kernel(prev)

    res1 = torch.full((rows, hidden), 3.0, dtype=torch.float16, device=DEV)
    q1 = torch.full((rows, hidden), 9, dtype=torch.int8, device=DEV)
    k.dec_emb_norm_layer_i8O(emb, pos, tokens, res1, q1, g, b, rb, rows, hidden, vocab, step, max_step, dq,
                             True, qs, post_ln)
    np.testing.assert_array_equal(to_np(q1), to_np(q0))
    np.testing.assert_array_equal(to_np(res1).view(np.uint16), to_np(res0).view(np.uint16))


@pytest.mark.parametrize("batch,hidden,vocab,pos,post_ln", [(16, 1024, 50257, 512, False), (5, 768, 333, 0, True),
                                                          (3, 132, 50, 6, False)])
def test_gpt_step_embedding_and_first_layer_norm_in_one_launch(rng, batch, hidden, vocab, pos, post_ln):
    """lsh_gpt_emb_step_norm_layer_i8O_f16 == lsh_ker_gpt_embedding_i8I_f16 (one position per
    sequence) followed by lsh_ker_norm_layer_resual_i8O_f16 with the row kernel: codes, residual
    stream and token counts byte for byte; a padding token embeds to zeros and is not counted;
    the flag word is cleared."""
    from lightseq_amd.lib import LSHError
    k = _k()
    max_step = pos + 4
    pad = vocab - 1
    emb = to_dev(rng.integers(-127, 128, size=(vocab, hidden), dtype=np.int8))
    pe = to_dev((rng.standard_normal((max_step, hidden)) * 0.5).astype(np.float16))
    ids = rng.integers(0, vocab - 1, size=(batch,), dtype=np.int32)
    ids[1] = pad
    ids = to_dev(ids)
    g = to_dev((1 + 0.1 * rng.standard_normal(hidden)).astype(np.float16))
    b = to_dev((0.1 * rng.standard_normal(hidden)).astype(np.float16))
    rb = to_dev((0.1 * rng.standard_normal(hidden)).astype(np.float16))
    dq, qs = 0.6 / 127, 127 / 3.0
    lens = rng.integers(1, 40, size=(batch,), dtype=np.int32)

    res0 = torch.zeros((batch, hidden), dtype=torch.float16, device=DEV)
    q0 = torch.zeros((batch, hidden), dtype=torch.int8, device=DEV)
    len0 = to_dev(lens.copy())
    prev = k.layer_norm_row_kernel(True)
    try:
        k.ker_gpt_embedding_i8I_launcher(batch, 1, hidden, emb, pe, ids, res0, len0, pad, pos, dq)
        k.ker_norm_layer_resual_i8O_launcher(batch, hidden, res0, q0, g, b, rb, 1024, qs, post_ln)
    finally:
        k.layer_norm_row_kernel(prev)

    res1 = torch.full((batch, hidden), 3.0, dtype=torch.float16, device=DEV)
    q1 = torch.full((batch, hidden), 9, dtype=torch.int8, device=DEV)
    len1 = to_dev(lens.copy())
    flag = torch.full((1,), 5, dtype=torch.int32, device=DEV)
    k.gpt_emb_step_norm_layer_i8O(emb, pe, ids, res1, q1, g, b, rb, len1, flag, batch, hidden, vocab, pad, pos,
                                  max_step, dq, qs, post_ln)
    np.testing.assert_array_equal(to_np(q1), to_np(q0))
    np.testing.assert_array_equal(to_np(res1).view(np.uint16), to_np(res0).view(np.uint16))
    np.testing.assert_array_equal(to_np(len1), to_np(len0))
    assert to_np(len1)[1] == lens[1] and to_np(len1)[0] == lens[0] + 1
    assert int(to_np(flag)[0]) == 0
    with pytest.raises(LSHError):  # position outside the table
        k.gpt_emb_step_norm_layer_i8O(emb, pe, ids, res1, q1, g, b, rb, len1, flag, batch, hidden, vocab, pad,
                                      max_step, max_step, dq, qs, post_ln)


@pytest.mark.parametrize("batch,beam,heads,S", [(16, 4, 16, 64), (3, 2, 4, 37), (2, 1, 2, 128), (5, 3, 8, 9),
                                                (2, 4, 16, 100)])
def test_cross_attention_q_product_and_attention_in_one_launch(rng, batch, beam, heads, S):
    """lsh_encdec_q_attention_f16 == lsh_gemm_i8_encdec_q_f16 followed by lsh_encdec_attention_f16:
    the int8 context byte for byte (padded source positions included); what it does not cover
    is refused."""
    from lightseq_amd.lib import LSHError
    k = _k()
    d = 64
    M, H = batch * beam, heads * d
    x = to_dev(rng.integers(-127, 128, size=(M, H), dtype=np.int8))
    w = to_dev(rng.integers(-127, 128, size=(H, H), dtype=np.int8))
    bias = to_dev((rng.standard_normal(H) * 0.4).astype(np.float16))
    alpha, ds = 2.5 / (np.sqrt(H) * 127), 3.0 / 127
    kk = to_dev((rng.standard_normal((batch, heads, S, d)) * 0.7).astype(np.float16))
    vv = to_dev((rng.standard_normal((batch, heads, S, d)) * 0.7).astype(np.float16))
    mask = np.zeros((batch, S), dtype=np.int32)
    for b in range(batch):
        mask[b, S - int(rng.integers(0, max(1, S // 2))):] = 1
    mask[0, :] = 0
    mask = to_dev(mask)
    qs = 127 / 1.5

    q0 = torch.zeros((batch, heads, beam, d), dtype=torch.float16, device=DEV)
    ctx0 = torch.zeros((M, H), dtype=torch.int8, device=DEV)
    k.gemm_i8_encdec_q(x, w, bias, q0, M, H, H, beam, heads, alpha, ds)
    k.encdec_attention(q0, kk, vv, mask, None, ctx0, qs, batch, beam, heads, S, d)
    ctx1 = torch.full((M, H), 7, dtype=torch.int8, device=DEV)
    k.encdec_q_attention(x, w, bias, kk, vv, mask, ctx1, qs, batch, beam, heads, S, H, alpha, ds)
    np.testing.assert_array_equal(to_np(ctx1), to_np(ctx0))

    with pytest.raises(LSHError):  # the context over the input rows
        k.encdec_q_attention(x, w, bias, kk, vv, mask, x, qs, batch, beam, heads, S, H, alpha, ds)
    with pytest.raises(LSHError):  # more than four beams
        k.encdec_q_attention(x, w, bias, kk, vv, mask, ctx1, qs, 1, 5, heads, S, H, alpha, ds)
    with pytest.raises(LSHError):  # a source beyond the short kernel
        k.encdec_q_attention(x, w, bias, kk, vv, mask, ctx1, qs, batch, beam, heads, 129, H, alpha, ds)
