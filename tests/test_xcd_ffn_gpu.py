"""The feed-forward segment of an encoder layer as one launch (lsh_ffn_segment_i8_f16: FFN1 with
the tabulated epilogue -> FFN2 -> layer norm, rows dealt to the XCDs, XCD-local barriers)
against the three launches it replaces, byte for byte, and against the oracle's kernels."""
import numpy as np
import pytest
import torch

from conftest import assert_codes_close
from helpers import DEV, to_dev, to_np

pytestmark = pytest.mark.gpu


def _k():
    from lightseq_amd import kernels
    return kernels


def _case(rng, M, H, I, relu):
    x = rng.integers(-127, 128, size=(M, H), dtype=np.int8)
    w1 = rng.integers(-127, 128, size=(I, H), dtype=np.int8)
    w2 = rng.integers(-127, 128, size=(H, I), dtype=np.int8)
    b1 = (rng.standard_normal(I) * 0.3).astype(np.float16)
    res = rng.standard_normal((M, H)).astype(np.float16)
    gam = (1 + 0.1 * rng.standard_normal(H)).astype(np.float16)
    bet = (0.1 * rng.standard_normal(H)).astype(np.float16)
    rb = (0.1 * rng.standard_normal(H)).astype(np.float16)
    colsum = (0.05 * rng.standard_normal(H)).astype(np.float16) if relu else None
    # accumulators of K random products spread ~ 127^2 sqrt(K) / 3: alpha brings them to codes
    alpha1 = 127.0 / (127 * 127 * np.sqrt(H) / 1.5)
    ds1, qs1, clip = 3.0 / 127, 127 / 2.0, 2.0
    dq2 = 2.0 / (127 * 127 * np.sqrt(I) / 3)
    return dict(x=x, w1=w1, w2=w2, b1=b1, res=res, gam=gam, bet=bet, rb=rb, colsum=colsum,
                alpha1=alpha1, ds1=ds1, qs1=qs1, clip=clip, dq2=dq2, qs_out=127 / 3.0)


def _three_launches(k, c, M, H, I, relu, final, post_ln):
    dev = {n: (to_dev(v) if isinstance(v, np.ndarray) else v) for n, v in c.items()}
    lut = torch.zeros((I, 256), dtype=torch.int8, device=DEV)
    k.build_act_lut(lut, dev["b1"], I, c["ds1"], c["qs1"], c["clip"], 2 if relu else 0)
    act = torch.zeros((M, I), dtype=torch.int8, device=DEV)
    k.gemm_i8_lut_i8o(dev["x"], dev["w1"], act, lut, M, I, H, c["alpha1"])
    acc = torch.zeros((M, H), dtype=torch.int32, device=DEV)
    k.gemm_i8_i32o(act, dev["w2"], acc, M, H, I)
    res = dev["res"].clone()
    if final:
        out = torch.zeros((M, H), dtype=torch.float16, device=DEV)
        k.ker_residual_bias_ln_i32I_launcher(acc, dev["gam"], dev["bet"], res, out, M, H, c["dq2"], 1024,
                                             False, dev["colsum"])
        return lut, act, acc, res, out, None
    out_q = torch.zeros((M, H), dtype=torch.int8, device=DEV)
    k.ker_residual_bias_ln_i32I_i8O_launcher(acc, dev["gam"], dev["bet"], dev["rb"], out_q, res, M, H,
                                             c["dq2"], c["qs_out"], 1024, post_ln, False, False,
                                             dev["colsum"])
    return lut, act, acc, res, None, out_q


SHAPES = [  # M, H, I, relu, final, post_ln
    (4096, 768, 3072, False, False, True),     # the benchmark layer
    (4096, 768, 3072, False, True, True),      # ... and its last layer
    (512, 512, 2048, True, False, True),       # Transformer-base layer, ReLU with column sums
    (1024, 1024, 4096, True, False, False),    # Transformer-big encoder, pre-LN
    (1000, 768, 3072, False, False, True),     # rows that do not split evenly
    (24, 256, 512, False, True, False),        # three rows per XCD
    (4096 + 128, 384, 1536, False, False, True),
]


@pytest.mark.parametrize("M,H,I,relu,final,post_ln", SHAPES)
def test_segment_equals_the_three_launches(rng, M, H, I, relu, final, post_ln):
    k = _k()
    if not k.ffn_segment_supported(M, H, I):
        pytest.skip("shape not covered by the segment kernel")
    c = _case(rng, M, H, I, relu)
    lut, act_w, acc_w, res_w, out_w, outq_w = _three_launches(k, c, M, H, I, relu, final, post_ln)
    dev = {n: (to_dev(v) if isinstance(v, np.ndarray) else v) for n, v in c.items()}
    sync = k.FfnSegmentSync()
    for rep in range(3):   # the counters go on from launch to launch
        act = torch.full((M, I), 5, dtype=torch.int8, device=DEV)
        acc = torch.full((M, H), 7, dtype=torch.int32, device=DEV)
        res = dev["res"].clone()
        out = torch.zeros((M, H), dtype=torch.float16, device=DEV) if final else None
        out_q = None if final else torch.full((M, H), 9, dtype=torch.int8, device=DEV)
        k.ffn_segment_i8(dev["x"], dev["w1"], lut, c["alpha1"], act, dev["w2"], acc, res, out, out_q,
                         dev["gam"], dev["bet"], None if final else dev["rb"], dev["colsum"], M, H, I,
                         c["dq2"], 0.0 if final else c["qs_out"], post_ln, final, sync)
        torch.cuda.synchronize()
        assert sync.error() == 0, "the kernel gave up: error word %d" % sync.error()
        np.testing.assert_array_equal(to_np(act), to_np(act_w), err_msg="activation codes, launch %d" % rep)
        np.testing.assert_array_equal(to_np(acc), to_np(acc_w), err_msg="accumulators, launch %d" % rep)
        if final:
            np.testing.assert_array_equal(to_np(out), to_np(out_w))
            np.testing.assert_array_equal(to_np(res), to_np(dev["res"]))   # only read
        else:
            np.testing.assert_array_equal(to_np(out_q), to_np(outq_w))
            np.testing.assert_array_equal(to_np(res), to_np(res_w))
    assert sync.launches.value == 3
    assert 20 < float(act_w.float().abs().mean()) < 110 and float(acc_w.float().abs().mean()) > 1000


def test_segment_against_the_oracle(oracle, rng):
    """Not only HIP against HIP: the oracle's kernels on the same inputs (int8 GEMM + bias + GELU
    + requantisation, int32 GEMM, residual + layer norm + quantisation)."""
    k = _k()
    M, H, I = 256, 256, 1024
    c = _case(rng, M, H, I, False)
    dev = {n: (to_dev(v) if isinstance(v, np.ndarray) else v) for n, v in c.items()}
    lut = torch.zeros((I, 256), dtype=torch.int8, device=DEV)
    k.build_act_lut(lut, dev["b1"], I, c["ds1"], c["qs1"], c["clip"], 0)
    act = torch.zeros((M, I), dtype=torch.int8, device=DEV)
    acc = torch.zeros((M, H), dtype=torch.int32, device=DEV)
    res = dev["res"].clone()
    out_q = torch.zeros((M, H), dtype=torch.int8, device=DEV)
    sync = k.FfnSegmentSync()
    k.ffn_segment_i8(dev["x"], dev["w1"], lut, c["alpha1"], act, dev["w2"], acc, res, None, out_q,
                     dev["gam"], dev["bet"], dev["rb"], None, M, H, I, c["dq2"], c["qs_out"], True, False,
                     sync)
    torch.cuda.synchronize()
    assert sync.error() == 0
    ffn1 = oracle.gemm_i8_i8(c["x"], c["w1"], c["alpha1"])
    want_act = oracle.bias_gelu_i8I_i8O(ffn1, c["b1"], c["ds1"], c["qs1"])
    assert_codes_close(to_np(act), want_act, what="activation codes")
    np.testing.assert_array_equal(to_np(acc), oracle.gemm_i8_i32(to_np(act), c["w2"]))
    want_q, want_res = oracle.residual_bias_ln_i8O(to_np(acc), c["gam"], c["bet"], c["rb"], c["res"],
                                                   c["dq2"], c["qs_out"], True)
    assert_codes_close(to_np(out_q), want_q, what="layer-norm codes")
    np.testing.assert_allclose(to_np(res).astype(np.float32), want_res.astype(np.float32), atol=2e-3)


def test_segment_gives_up_when_its_workgroups_cannot_all_arrive():
    """The bounded wait, forced from the host: the counters are made to look as if a workgroup of
    every XCD were missing (one arrival short of every target), with a small poll limit.  Every
    workgroup gives up, the kernel ends, and the error word says so."""
    k = _k()
    M, H, I = 256, 256, 512
    z8 = lambda *s: torch.zeros(s, dtype=torch.int8, device=DEV)
    f16 = lambda *s: torch.ones(s, dtype=torch.float16, device=DEV)
    sync = k.FfnSegmentSync()
    sync.launches.value = 6            # targets start at 6 * 64 while the counters stand at zero
    res = f16(M, H)
    k.ffn_segment_i8(z8(M, H), z8(I, H), z8(I, 256), 1e-3, z8(M, I), z8(H, I),
                     torch.zeros((M, H), dtype=torch.int32, device=DEV), res, None, z8(M, H), f16(H),
                     f16(H), f16(H), None, M, H, I, 1e-3, 10.0, True, False, sync, spin_limit=200)
    torch.cuda.synchronize()
    assert sync.error() == 1
    sync.reset()
    assert sync.error() == 0
    # a launch count of the wrong parity looks like places taken twice: the other error bit
    sync.launches.value = 1
    k.ffn_segment_i8(z8(M, H), z8(I, H), z8(I, 256), 1e-3, z8(M, I), z8(H, I),
                     torch.zeros((M, H), dtype=torch.int32, device=DEV), res, None, z8(M, H), f16(H),
                     f16(H), f16(H), None, M, H, I, 1e-3, 10.0, True, False, sync, spin_limit=200)
    torch.cuda.synchronize()
    assert sync.error() & 2


def test_segment_rejects_what_it_does_not_cover():
    from lightseq_amd.lib import LSHError
    k = _k()
    assert not k.ffn_segment_supported(4096, 760, 3072)
    assert not k.ffn_segment_supported(4096, 2048, 8192)
    assert not k.ffn_segment_supported(4, 768, 3072)
    z8 = lambda *s: torch.zeros(s, dtype=torch.int8, device=DEV)
    f16 = lambda *s: torch.ones(s, dtype=torch.float16, device=DEV)
    sync = k.FfnSegmentSync()
    with pytest.raises(LSHError):
        k.ffn_segment_i8(z8(64, 760), z8(3072, 760), z8(3072, 256), 1e-3, z8(64, 3072), z8(760, 3072),
                         torch.zeros((64, 760), dtype=torch.int32, device=DEV), f16(64, 760), None,
                         z8(64, 760), f16(760), f16(760), f16(760), None, 64, 760, 3072, 1e-3, 10.0, True,
                         False, sync)
    assert sync.launches.value == 0
