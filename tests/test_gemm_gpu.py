"""GPU parity of the int8 MFMA GEMM through the C ABI.

int32 accumulators are bit-exact against the oracle's integer triple loop (small
shapes) and against an exact float64 BLAS product (large shapes: |acc| <= K*127^2
< 2^53, so the float64 product of integer matrices is exact).  int8 outputs follow
clamp(floor(acc*alpha + 0.5), -127, 127) bit-exactly given exact accumulators.
"""
import numpy as np
import pytest
import torch

from helpers import DEV, to_dev, to_np

pytestmark = pytest.mark.gpu

SMALL = [(1, 1, 16), (3, 5, 16), (32, 32, 32), (33, 31, 48), (64, 16, 128), (130, 70, 144),
         (257, 129, 272), (300, 513, 400), (128, 256, 1024)]
LARGE = [(4096, 2304, 768), (4096, 768, 768), (4096, 3072, 768), (4096, 768, 3072),
         (512, 1536, 512), (512, 2048, 512), (4096, 4096, 1024), (4096, 1024, 4096),
         (1000, 30522 // 6, 128), (64, 1000, 1024),
         # ragged rows and columns in the 128x64 kernel (column tails of 40 and of 8), a single K step
         (200, 1000, 1536), (130, 72, 256), (256, 192, 128),
         # one output tile per workgroup: 256 x 256 with ragged rows and a 16-column last tile,
         # 256 x 192 with ragged rows and the shortest K loop it takes, 256 x 128 (K loop = ring depth)
         (4000, 3088, 768), (3900, 3072, 384), (8192, 1024, 384), (8192, 1024, 1024),
         # 128 x 96 tiles on 4 wavefronts (narrow outputs), ragged rows, both ring depths
         (4000, 768, 384), (3000, 960, 1536),
         # decode-step shapes (rows = batch x beam of one step)
         (16, 3072, 1024), (16, 1024, 4096), (16, 50257, 1024), (64, 32000, 1024),
         (64, 4096, 1024), (33, 1000, 256), (1, 64, 128), (48, 40, 384)]


def _k():
    from lightseq_amd import kernels
    return kernels


def _exact_i32(a, w):
    return np.rint(a.astype(np.float64) @ w.astype(np.float64).T).astype(np.int64)


@pytest.mark.parametrize("M,N,K", SMALL)
def test_gemm_i32_small_vs_oracle(oracle, rng, M, N, K):
    a = rng.integers(-127, 128, size=(M, K), dtype=np.int8)
    w = rng.integers(-127, 128, size=(N, K), dtype=np.int8)
    want = oracle.gemm_i8_i32(a, w)
    np.testing.assert_array_equal(want, _exact_i32(a, w))  # the oracle itself, against BLAS
    c = torch.full((M, N), 7, dtype=torch.int32, device=DEV)
    _k().gemm_i8_i32o(to_dev(a), to_dev(w), c, M, N, K)
    np.testing.assert_array_equal(to_np(c), want)


@pytest.mark.parametrize("M,N,K", SMALL)
def test_gemm_i8_small_vs_oracle(oracle, rng, M, N, K):
    a = rng.integers(-127, 128, size=(M, K), dtype=np.int8)
    w = rng.integers(-127, 128, size=(N, K), dtype=np.int8)
    alpha = 3.0 / (np.sqrt(K) * 127)
    want = oracle.gemm_i8_i8(a, w, alpha)
    c = torch.full((M, N), 7, dtype=torch.int8, device=DEV)
    _k().gemm_i8_i8o(to_dev(a), to_dev(w), c, M, N, K, alpha)
    np.testing.assert_array_equal(to_np(c), want)


@pytest.mark.parametrize("M,N,K", LARGE)
def test_gemm_large_exact(rng, M, N, K):
    a = rng.integers(-127, 128, size=(M, K), dtype=np.int8)
    w = rng.integers(-127, 128, size=(N, K), dtype=np.int8)
    ref = _exact_i32(a, w)
    c = torch.zeros((M, N), dtype=torch.int32, device=DEV)
    _k().gemm_i8_i32o(to_dev(a), to_dev(w), c, M, N, K)
    np.testing.assert_array_equal(to_np(c).astype(np.int64), ref)
    alpha = np.float32(4.0 * 0.08 / (6.0 * 127))
    f = ref.astype(np.float32) * alpha  # |acc| < 2^24 for K <= 1024; larger K: same float cast as the kernel
    want8 = np.clip(np.floor(f + np.float32(0.5)), -127, 127).astype(np.int8)
    c8 = torch.zeros((M, N), dtype=torch.int8, device=DEV)
    _k().gemm_i8_i8o(to_dev(a), to_dev(w), c8, M, N, K, float(alpha))
    np.testing.assert_array_equal(to_np(c8), want8)


def test_gemm_extreme_values(rng):
    """All-(-127) x all-(-127) at K=4096 reaches the largest accumulator of the path."""
    M, N, K = 64, 64, 4096
    a = np.full((M, K), -127, np.int8)
    w = np.full((N, K), -127, np.int8)
    c = torch.zeros((M, N), dtype=torch.int32, device=DEV)
    _k().gemm_i8_i32o(to_dev(a), to_dev(w), c, M, N, K)
    assert np.all(to_np(c) == K * 127 * 127)


def test_gemm_linearity(rng):
    """Size-independent property at full size: (A1 + A2) W^T == A1 W^T + A2 W^T."""
    M, N, K = 4096, 3072, 768
    a1 = rng.integers(-60, 61, size=(M, K), dtype=np.int8)
    a2 = rng.integers(-60, 61, size=(M, K), dtype=np.int8)
    w = rng.integers(-127, 128, size=(N, K), dtype=np.int8)
    wd = to_dev(w)
    outs = []
    for a in (a1, a2, (a1 + a2).astype(np.int8)):
        c = torch.zeros((M, N), dtype=torch.int32, device=DEV)
        _k().gemm_i8_i32o(to_dev(a), wd, c, M, N, K)
        outs.append(c)
    assert torch.equal(outs[0] + outs[1], outs[2])


def test_gemm_rejects_bad_k():
    from lightseq_amd.lib import LSHError
    a = torch.zeros((4, 8), dtype=torch.int8, device=DEV)
    c = torch.zeros((4, 4), dtype=torch.int32, device=DEV)
    with pytest.raises(LSHError):
        _k().gemm_i8_i32o(a, a, c, 4, 4, 8)


@pytest.mark.parametrize("M,N,K", [(4096, 2304, 768), (4096, 4096, 1024), (4000, 3088, 768), (8192, 1024, 384),
                                   (4096, 768, 3072), (4096, 768, 768)])
def test_tile_kernel_equals_persistent_kernels(rng, M, N, K):
    """The one-tile-per-workgroup kernel and the persistent kernels give the same bytes."""
    k = _k()
    a = to_dev(rng.integers(-127, 128, size=(M, K), dtype=np.int8))
    w = to_dev(rng.integers(-127, 128, size=(N, K), dtype=np.int8))
    alpha = 3.0 / (np.sqrt(K) * 127)
    outs = []
    prev = k.gemm_i8_tile_kernel(True)
    try:
        for on in (True, False):
            k.gemm_i8_tile_kernel(on)
            c32 = torch.zeros((M, N), dtype=torch.int32, device=DEV)
            c8 = torch.zeros((M, N), dtype=torch.int8, device=DEV)
            k.gemm_i8_i32o(a, w, c32, M, N, K)
            k.gemm_i8_i8o(a, w, c8, M, N, K, alpha)
            outs.append((c32, c8))
    finally:
        k.gemm_i8_tile_kernel(prev)
    assert torch.equal(outs[0][0], outs[1][0]) and torch.equal(outs[0][1], outs[1][1])


def test_fused_gelu_epilogue_at_the_microbenchmark_shape(oracle, rng):
    """4096 x 4096 x 1024 with clip values 4.0 / 0.08 / 6.0: the fused bias + GELU + requant
    epilogue (arithmetic and tabulated) against the oracle's stand-alone kernel on the exact
    int8 product."""
    M, N, K = 4096, 4096, 1024
    a = rng.integers(-127, 128, size=(M, K), dtype=np.int8)
    w = rng.integers(-127, 128, size=(N, K), dtype=np.int8)
    bias = (0.02 * rng.standard_normal(N)).astype(np.float16)
    c_in, c_w, c_out, c_act = 4.0, 0.08, 6.0, 6.0
    alpha = np.float32(c_in * c_w / (c_out * 127))
    f = _exact_i32(a, w).astype(np.float32) * alpha
    prod8 = np.clip(np.floor(f + np.float32(0.5)), -127, 127).astype(np.int8)
    ds, qs = c_out / 127, 127 / c_act
    want = oracle.bias_gelu_i8I_i8O(prod8, bias, ds, qs)
    k = _k()
    ad, wd, bd = to_dev(a), to_dev(w), to_dev(bias)
    got = torch.zeros((M, N), dtype=torch.int8, device=DEV)
    k.gemm_i8_bias_gelu_i8o(ad, wd, got, bd, M, N, K, float(alpha), ds, qs)
    from conftest import assert_codes_close
    assert_codes_close(to_np(got), want, what="fused GELU epilogue vs oracle")
    lut = torch.zeros((N, 256), dtype=torch.int8, device=DEV)
    k.build_act_lut(lut, bd, N, ds, qs, c_act, 0)
    via_lut = torch.zeros_like(got)
    k.gemm_i8_lut_i8o(ad, wd, via_lut, lut, M, N, K, float(alpha))
    assert torch.equal(via_lut, got)


@pytest.mark.parametrize("M,N,K", [(256, 256, 128), (300, 3072, 768), (4096, 3072, 768), (77, 160, 48),
                                   (4000, 3088, 768), (8192, 1024, 384), (4096, 768, 768),
                                   (16, 4096, 1024), (64, 4096, 1024),
                                   # ragged columns with the table rows in LDS (last tile: 40 and 16 columns)
                                   (200, 1000, 256), (130, 208, 384)])
@pytest.mark.parametrize("act", ["gelu", "relu", "relu_narrow"])
def test_fused_bias_act_epilogue_equals_unfused_pair(rng, M, N, K, act):
    """GEMM + bias/activation/requant in one kernel == int8-output GEMM followed by the
    stand-alone kernel, byte for byte."""
    k = _k()
    a = to_dev(rng.integers(-127, 128, size=(M, K), dtype=np.int8))
    w = to_dev(rng.integers(-127, 128, size=(N, K), dtype=np.int8))
    bias = to_dev((0.3 * rng.standard_normal(N)).astype(np.float16))
    alpha, ds, qs, clip = 3.0 / (np.sqrt(K) * 127), 2.2 / 127, 127 / 1.65, 1.65
    tmp = torch.zeros((M, N), dtype=torch.int8, device=DEV)
    want = torch.zeros_like(tmp)
    got = torch.zeros_like(tmp)
    k.gemm_i8_i8o(a, w, tmp, M, N, K, alpha)
    if act == "gelu":
        k.ker_bias_gelu_i8I_i8O_launcher(M, tmp, want, bias, N, ds, qs)
        k.gemm_i8_bias_gelu_i8o(a, w, got, bias, M, N, K, alpha, ds, qs)
    else:
        narrow = act == "relu_narrow"
        k.ker_bias_relu_i8I_i8O_launcher(M, tmp, want, bias, N, ds, qs, clip, False, False, narrow)
        k.gemm_i8_bias_relu_i8o(a, w, got, bias, M, N, K, alpha, ds, qs, clip, narrow)
    assert torch.equal(got, want)
    # and the same epilogue as a per-column table of the 256 codes
    lut = torch.zeros((N, 256), dtype=torch.int8, device=DEV)
    k.build_act_lut(lut, bias, N, ds, qs, clip, {"gelu": 0, "relu": 1, "relu_narrow": 2}[act])
    via_lut = torch.zeros_like(tmp)
    k.gemm_i8_lut_i8o(a, w, via_lut, lut, M, N, K, alpha)
    assert torch.equal(via_lut, want)


@pytest.mark.parametrize("B,S,h,d,K", [(2, 16, 2, 64, 128), (32, 128, 12, 64, 768), (3, 10, 4, 16, 64)])
def test_fused_qkv_arrange_epilogue_equals_unfused_pair(rng, B, S, h, d, K):
    k = _k()
    H, M = h * d, B * S
    a = to_dev(rng.integers(-127, 128, size=(M, K), dtype=np.int8))
    w = to_dev(rng.integers(-127, 128, size=(3 * H, K), dtype=np.int8))
    bias = to_dev((0.3 * rng.standard_normal(3 * H)).astype(np.float16))
    alpha, ds = 3.0 / (np.sqrt(K) * 127), 2.2 / 127
    tmp = torch.zeros((M, 3 * H), dtype=torch.int8, device=DEV)
    want = torch.zeros((3, B, h, S, d), dtype=torch.float16, device=DEV)
    got = torch.zeros_like(want)
    k.gemm_i8_i8o(a, w, tmp, M, 3 * H, K, alpha)
    k.ker_arrange_encself_qkv_i8I_launcher(M, H, tmp, bias, want, M * H, S, d, h, 1024, ds)
    k.gemm_i8_qkv_arrange(a, w, got, bias, M * H, M, H, K, S, h, alpha, ds)
    assert torch.equal(got.view(torch.int16), want.view(torch.int16))


def test_fused_qkv_arrange_rejects_small_heads(rng):
    from lightseq_amd.lib import LSHError
    k = _k()
    a = torch.zeros((8, 16), dtype=torch.int8, device=DEV)
    w = torch.zeros((3 * 8, 16), dtype=torch.int8, device=DEV)
    out = torch.zeros((3, 8, 8), dtype=torch.float16, device=DEV)
    bias = torch.zeros(24, dtype=torch.float16, device=DEV)
    with pytest.raises(LSHError):
        k.gemm_i8_qkv_arrange(a, w, out, bias, 64, 8, 8, 16, 8, 1, 1.0, 1.0)


@pytest.mark.parametrize("M,N,K,ksplit", [(16, 3072, 1024, 1), (16, 1024, 4096, 8), (64, 1024, 4096, 4),
                                          (64, 32000, 1024, 1), (16, 50257, 1024, 1), (1, 48, 256, 1),
                                          (17, 1000, 768, 1), (33, 40, 512, 2), (48, 4096, 1024, 1),
                                          (5, 8, 2048, 2), (64, 1024, 4096, 16)])
def test_decode_step_kernels_give_the_same_bytes(rng, M, N, K, ksplit):
    """Products of at most 64 rows: the 16 x 16 x 64 kernel and the 32 x 32 x 32 kernel agree bit
    for bit -- int32 planes, requantised codes, the table epilogue -- and with the exact product."""
    k = _k()
    a = rng.integers(-127, 128, size=(M, K), dtype=np.int8)
    w = rng.integers(-127, 128, size=(N, K), dtype=np.int8)
    ad, wd = to_dev(a), to_dev(w)
    alpha = 3.0 / (np.sqrt(K) * 127)
    lut = to_dev(rng.integers(-127, 128, size=(N, 256), dtype=np.int8))
    outs = []
    prev = k.gemm_i8_decode_kernel_16x16(True)
    try:
        for on in (True, False):
            k.gemm_i8_decode_kernel_16x16(on)
            planes = torch.full((ksplit, M, N), 7, dtype=torch.int32, device=DEV)
            assert k.gemm_i8_i32o_splitk(ad, wd, planes, M, N, K, ksplit) == ksplit
            c8 = torch.full((M, N), 9, dtype=torch.int8, device=DEV)
            k.gemm_i8_i8o(ad, wd, c8, M, N, K, alpha)
            cl = torch.full((M, N), 9, dtype=torch.int8, device=DEV)
            k.gemm_i8_lut_i8o(ad, wd, cl, lut, M, N, K, alpha)
            outs.append((planes, c8, cl))
    finally:
        k.gemm_i8_decode_kernel_16x16(prev)
    for x, y in zip(*outs):
        assert torch.equal(x, y)
    np.testing.assert_array_equal(to_np(outs[0][0]).astype(np.int64).sum(0), _exact_i32(a, w))
    # the table epilogue is the table entry of the requantised code
    codes = to_np(outs[0][1]).astype(np.int64) + 128
    np.testing.assert_array_equal(to_np(outs[0][2]), np.take_along_axis(to_np(lut).T, codes, axis=0))


@pytest.mark.parametrize("M,N,K,ksplit", [(4096, 768, 3072, 2), (16, 1024, 4096, 8), (64, 1024, 4096, 4),
                                          (300, 256, 1024, 4), (33, 96, 256, 2)])
def test_split_k_planes_sum_to_the_product(rng, M, N, K, ksplit):
    a = rng.integers(-127, 128, size=(M, K), dtype=np.int8)
    w = rng.integers(-127, 128, size=(N, K), dtype=np.int8)
    c = torch.full((ksplit, M, N), 7, dtype=torch.int32, device=DEV)
    used = _k().gemm_i8_i32o_splitk(to_dev(a), to_dev(w), c, M, N, K, ksplit)
    assert used == ksplit
    planes = to_np(c).astype(np.int64)
    np.testing.assert_array_equal(planes.sum(0), _exact_i32(a, w))
    kp = K // ksplit
    np.testing.assert_array_equal(planes[1], _exact_i32(a[:, kp:2 * kp], w[:, kp:2 * kp]))
    # a split that does not divide K into whole 128-byte steps is not applied
    c1 = torch.zeros((3, M, N), dtype=torch.int32, device=DEV)
    assert _k().gemm_i8_i32o_splitk(to_dev(a), to_dev(w), c1, M, N, K, 3) == (3 if (K // 128) % 3 == 0 else 1)
    assert _k().gemm_i8_preferred_ksplit(4096, 768, 3072) == 1  # encoder sizes: not worth the planes
    assert _k().gemm_i8_preferred_ksplit(16, 1024, 4096) == 4
    assert _k().gemm_i8_preferred_ksplit(4096, 3072, 768) == 1


@pytest.mark.parametrize("rows,hidden,nparts", [(16, 1024, 8), (4096, 768, 2), (37, 512, 4)])
def test_layer_norm_over_accumulator_planes(rng, rows, hidden, nparts):
    planes = rng.integers(-20000, 20000, size=(nparts, rows, hidden), dtype=np.int32)
    total = planes.sum(0).astype(np.int32)
    g = (1 + 0.1 * rng.standard_normal(hidden)).astype(np.float16)
    b = (0.1 * rng.standard_normal(hidden)).astype(np.float16)
    rb = (0.1 * rng.standard_normal(hidden)).astype(np.float16)
    res = rng.standard_normal((rows, hidden)).astype(np.float16)
    outs = []
    for inp, n in ((planes, nparts), (total, 1)):
        q = torch.zeros(rows, hidden, dtype=torch.int8, device=DEV)
        r = to_dev(res.copy())
        _k().ker_residual_bias_ln_planes_i32I_i8O(to_dev(inp), n, rows * hidden, to_dev(g), to_dev(b),
                                                  to_dev(rb), q, r, rows, hidden, 3e-4, 127 / 4.0, True)
        outs.append((to_np(q), to_np(r)))
    np.testing.assert_array_equal(outs[0][0], outs[1][0])
    np.testing.assert_array_equal(outs[0][1], outs[1][1])


@pytest.mark.parametrize("M,H", [(4096, 768), (1000, 1024), (300, 512), (17, 768), (8192, 1024)])
@pytest.mark.parametrize("post_ln", [True, False])
def test_fused_outproj_layernorm_equals_unfused_pair(rng, M, H, post_ln):
    """Out-projection GEMM + residual LayerNorm + quantisation in one kernel == the int8-output
    GEMM followed by ker_residual_bias_ln_i8I_i8O, byte for byte (int8 output and fp16 residual)."""
    k = _k()
    a = to_dev(rng.integers(-127, 128, size=(M, H), dtype=np.int8))
    w = to_dev(rng.integers(-127, 128, size=(H, H), dtype=np.int8))
    g = to_dev((1 + 0.1 * rng.standard_normal(H)).astype(np.float16))
    b = to_dev((0.1 * rng.standard_normal(H)).astype(np.float16))
    rb = to_dev((0.1 * rng.standard_normal(H)).astype(np.float16))
    res = rng.standard_normal((M, H)).astype(np.float16)
    alpha, dq, qs = 3.0 / (np.sqrt(H) * 127), 2.5 / 127, 127 / 4.0
    tmp = torch.zeros((M, H), dtype=torch.int8, device=DEV)
    want_q, want_r = torch.zeros_like(tmp), to_dev(res.copy())
    k.gemm_i8_i8o(a, w, tmp, M, H, H, alpha)
    k.ker_residual_bias_ln_i8I_i8O_launcher(tmp, g, b, rb, want_q, want_r, M, H, dq, qs, 1024, post_ln)
    wt = torch.zeros_like(w)
    k.tile_weight_16x64(w, wt, H, H)
    got_q, got_r = torch.full_like(tmp, 7), to_dev(res.copy())
    k.gemm_i8_residual_ln_i8O(a, wt, alpha, g, b, rb, got_q, got_r, M, H, H, dq, qs, post_ln)
    assert torch.equal(got_q, want_q)
    assert torch.equal(got_r.view(torch.int16), want_r.view(torch.int16))


def test_fused_outproj_layernorm_rejects_other_sizes():
    from lightseq_amd.lib import LSHError
    z8 = torch.zeros(640 * 640, dtype=torch.int8, device=DEV)
    zh = torch.zeros(640 * 16, dtype=torch.float16, device=DEV)
    with pytest.raises(LSHError, match="512, 768, 1024"):
        _k().gemm_i8_residual_ln_i8O(z8, z8, 1.0, zh, zh, zh, z8, zh, 16, 640, 640, 1.0, 1.0, True)
