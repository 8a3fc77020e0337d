"""Bit-exact parity of the uint8 (LOWP) kernels and engine against the CPU oracle."""
import ctypes as C

import numpy as np
import pytest

import cases
import gpu_util as G
from thnets_amd import api, configs

pytestmark = pytest.mark.gpu


def test_quantize_dequantize_bit_exact(hiplib, oracle):
    g = cases.rng(10)
    for x in (g.standard_normal((2, 3, 5, 7), dtype=np.float32), g.uniform(0, 1, (4, 11)).astype(np.float32),
              -g.uniform(0, 3, 50).astype(np.float32), np.zeros(9, np.float32),
              g.standard_normal(300000, dtype=np.float32) * 100):
        dx = api.DeviceArray(hiplib, x)
        dq = api.DeviceArray(hiplib, nbytes=x.size)
        m, s = C.c_float(), C.c_float()
        hiplib.thhip_quantize(dx.ptr, dq.ptr, x.size, C.byref(m), C.byref(s))
        hiplib.thhip_sync()
        q, mo, so = oracle.lowp_quantize(x)
        assert (m.value, s.value) == (mo, so)
        assert np.array_equal(dq.get(x.shape, np.uint8), q)
        dy = api.DeviceArray(hiplib, nbytes=x.nbytes)
        hiplib.thhip_dequantize(dq.ptr, dy.ptr, x.size, mo, so)
        hiplib.thhip_sync()
        assert np.array_equal(dy.get(x.shape, np.float32), oracle.lowp_dequantize(q, mo, so))


def _lowp_case(i, rngv=16.0, seed=0):
    B, Ci, H, W, Co, kH, kW, dH, dW, pH, pW = cases.CONV_CASES[i]
    g = cases.rng(1000 + i + seed)
    x = g.uniform(-3, 3, (B, Ci, H, W)).astype(np.float32)
    w = g.standard_normal((Co, Ci, kH, kW), dtype=np.float32) * np.float32(np.sqrt(2.0 / (Ci * kH * kW)))
    b = g.standard_normal(Co, dtype=np.float32) * np.float32(0.5)
    return x, w, b, (dH, dW), (pH, pW)


@pytest.mark.parametrize("i", range(len(cases.CONV_CASES)))
def test_conv_u8_bit_exact(hiplib, oracle, i):
    x, w, b, d, p = _lowp_case(i)
    rngv = 16.0
    om, osub = float(np.float32(255) / np.float32(rngv)), -rngv / 2
    xq, im, isub = oracle.lowp_quantize(x)
    wq, wm, wsub = oracle.lowp_quantize(w)
    bq, bm, bsub = oracle.lowp_quantize(b)
    want = oracle.lowp_conv2d(xq, im, isub, wq, wm, wsub, bq, bm, bsub, om, osub, d, p)
    prm = oracle.lowp_mm_params(wm, wsub, im, isub, om, osub)
    zero = int(np.round(np.float32(-isub) * np.float32(im)))
    addend = np.array([oracle.lowp_bias_addend(int(c), bm, bsub, om) for c in bq], np.int32)
    got = G.conv2d_u8(hiplib, xq, wq, addend, d, p, zero, prm)
    assert got.shape == want.shape
    assert np.array_equal(got, want), "mismatching codes: %d of %d" % ((got != want).sum(), got.size)
    # fused threshold on the codes
    thr = oracle.lowp_scale_float(om, osub, 0.0)
    got = G.conv2d_u8(hiplib, xq, wq, addend, d, p, zero, prm, act=1, thr=thr, val=thr)
    assert np.array_equal(got, oracle.lowp_threshold(want, thr, thr))


def test_conv_u8_wrapping_requantisation_and_extreme_offsets(hiplib, oracle):
    g = cases.rng(1100)
    xq = g.integers(0, 256, (2, 5, 7, 6), dtype=np.uint8)
    wq = g.integers(0, 256, (9, 5, 3, 3), dtype=np.uint8)
    for prm in (dict(a_off=-128, b_off=-128, c_off=1000, c_mult=77, c_shift=12),
                dict(a_off=0, b_off=0, c_off=0, c_mult=9000, c_shift=20),          # products beyond 2^31 wrap
                dict(a_off=-255, b_off=3, c_off=-12345, c_mult=511, c_shift=18),
                dict(a_off=-100, b_off=-7, c_off=5, c_mult=1, c_shift=0)):
        col = np.stack([oracle.lowp_unfold(xq[t], (3, 3), (1, 1), (1, 1), 77) for t in range(2)])
        want = np.stack([oracle.lowp_gemm(wq.reshape(9, 45), col[t], **prm) for t in range(2)]).reshape(2, 9, 7, 6)
        got = G.conv2d_u8(hiplib, xq, wq, None, (1, 1), (1, 1), 77, prm)
        assert np.array_equal(got, want), prm


def test_conv_u8_split_k_bit_exact(hiplib, oracle):
    rngv = 16.0
    om, osub = float(np.float32(255) / np.float32(rngv)), -rngv / 2
    try:
        for (bm, bn, sk) in [(64, 64, 2), (64, 64, 5), (128, 128, 3), (128, 64, 4)]:
            hiplib.thhip_conv_set_tuning(bm, bn, sk, sk % 3)
            for i in (1, 5, 10):
                x, w, b, d, p = _lowp_case(i, seed=50)
                xq, im, isub = oracle.lowp_quantize(x)
                wq, wm, wsub = oracle.lowp_quantize(w)
                bq, bm_, bsub = oracle.lowp_quantize(b)
                want = oracle.lowp_conv2d(xq, im, isub, wq, wm, wsub, bq, bm_, bsub, om, osub, d, p)
                prm = oracle.lowp_mm_params(wm, wsub, im, isub, om, osub)
                zero = int(np.round(np.float32(-isub) * np.float32(im)))
                addend = np.array([oracle.lowp_bias_addend(int(c), bm_, bsub, om) for c in bq], np.int32)
                got = G.conv2d_u8(hiplib, xq, wq, addend, d, p, zero, prm)
                assert np.array_equal(got, want), (bm, bn, sk, i)
    finally:
        hiplib.thhip_conv_set_tuning(0, 0, 0, 0)


def test_lowpgemm_drop_in(hiplib, oracle):
    g = cases.rng(1101)
    for (m, n, k) in ((3, 5, 7), (64, 3025, 363), (100, 1, 900), (130, 77, 65)):
        a = g.integers(0, 256, (m, k), dtype=np.uint8)
        b = g.integers(0, 256, (k, n), dtype=np.uint8)
        c = np.zeros((m, n), np.uint8)
        G.note("lowpgemm %s" % ((m, n, k),))
        hiplib.lowpgemm(1, 1, 1, m, n, k, a.ctypes.data, b.ctypes.data, c.ctypes.data, k, n, n, -117, -128, 32513, 1028, 18)
        assert np.array_equal(c, oracle.lowp_gemm(a, b, -117, -128, 32513, 1028, 18))


# (B, Ci, H, W, Co, kH, kW, dH, dW, padH, padW): shapes for the channels-last memory order
CL_CASES = [
    (2, 64, 9, 11, 36, 3, 3, 1, 1, 1, 1),
    (3, 128, 7, 7, 200, 5, 5, 2, 2, 2, 2),
    (1, 192, 13, 13, 68, 1, 1, 1, 1, 0, 0),
    (5, 64, 6, 6, 132, 6, 6, 1, 1, 0, 0),
    (2, 16, 10, 10, 8, 3, 3, 1, 1, 1, 1),       # K = 144 ends inside a K-tile
    (2, 48, 5, 6, 40, 2, 3, 1, 1, 0, 1),
    (2, 64, 9, 7, 80, 3, 3, 1, 1, 1, 1),         # 16-byte channels-last stores; the last accumulator has 16 of 32 planes
    (2, 3, 21, 19, 64, 7, 7, 2, 2, 3, 3),       # plane-major in only (generic K order), channels-last out
    (3, 3, 35, 35, 64, 11, 11, 4, 4, 2, 2),     # the image layer: also through the four-plane pixel copy
    (2, 1, 9, 12, 12, 3, 3, 1, 1, 1, 1),
    (2, 4, 8, 7, 20, 5, 2, 2, 1, 2, 0),
    (1, 2, 6, 30, 8, 1, 9, 1, 3, 0, 4),
]


@pytest.mark.parametrize("i", range(len(CL_CASES)))
def test_conv_u8_channels_last_bit_exact(hiplib, oracle, i):
    """Every combination of memory orders gives the codes of the plane-major restatement,
    including the bias add's tail rule (which goes by the position inside the plane),
    the fused threshold, forced tiles and a K split."""
    B, Ci, H, W, Co, kH, kW, dH, dW, pH, pW = CL_CASES[i]
    g = cases.rng(1300 + i)
    x = g.uniform(-3, 3, (B, Ci, H, W)).astype(np.float32)
    w = g.standard_normal((Co, Ci, kH, kW), dtype=np.float32) * np.float32(np.sqrt(2.0 / (Ci * kH * kW)))
    b = g.standard_normal(Co, dtype=np.float32) * np.float32(0.5)
    d, p = (dH, dW), (pH, pW)
    rngv = 16.0
    om, osub = float(np.float32(255) / np.float32(rngv)), -rngv / 2
    xq, im, isub = oracle.lowp_quantize(x)
    wq, wm, wsub = oracle.lowp_quantize(w)
    bq, bm, bsub = oracle.lowp_quantize(b)
    want = oracle.lowp_conv2d(xq, im, isub, wq, wm, wsub, bq, bm, bsub, om, osub, d, p)
    prm = oracle.lowp_mm_params(wm, wsub, im, isub, om, osub)
    zero = int(np.round(np.float32(-isub) * np.float32(im)))
    addend = np.array([oracle.lowp_bias_addend(int(c), bm, bsub, om) for c in bq], np.int32)
    thr = oracle.lowp_scale_float(om, osub, 0.0)
    orders = [(0, 1)] + ([(1, 0), (1, 1)] if Ci % 16 == 0 else []) + ([(2, 0), (2, 1)] if Ci <= 4 else [])
    try:
        for tune in ((0, 0, 0, 0), (64, 64, 3, 2), (128, 128, 1, 0), (64, 128, 2, 1), (128, 64, 1, 4)):
            hiplib.thhip_conv_set_tuning(*tune)
            for (x_cl, y_cl) in orders:
                # Ci a multiple of the K-tile: the scalar tap walk, then the per-thread decode
                for generic in ((0, 1) if x_cl == 1 and Ci % 64 == 0 else (0,)):
                    hiplib.thhip_conv_set_generic_cl(generic)
                    got = G.conv2d_u8(hiplib, xq, wq, addend, d, p, zero, prm, x_cl=x_cl, y_cl=y_cl)
                    assert np.array_equal(got, want), (tune, x_cl, y_cl, generic, int((got != want).sum()))
                    got = G.conv2d_u8(hiplib, xq, wq, addend, d, p, zero, prm, act=1, thr=thr, val=thr, x_cl=x_cl, y_cl=y_cl)
                    assert np.array_equal(got, oracle.lowp_threshold(want, thr, thr)), (tune, x_cl, y_cl, generic)
    finally:
        hiplib.thhip_conv_set_generic_cl(0)
        hiplib.thhip_conv_set_tuning(0, 0, 0, 0)


DIRECT_CASES = [c for c in CL_CASES if c[1] % 64 == 0] + [
    (2, 64, 20, 17, 260, 3, 3, 1, 1, 1, 1),      # several tiles along both axes, partial ones
    (1, 128, 30, 30, 72, 1, 1, 1, 1, 0, 0),      # two K-tiles
    (1, 64, 12, 12, 40, 1, 1, 1, 1, 0, 0),       # one K-tile
    (3, 192, 13, 13, 384, 3, 3, 1, 1, 1, 1),     # an AlexNet layer: every border position reads the tail
]


@pytest.mark.parametrize("i", range(len(DIRECT_CASES)))
def test_conv_u8_loaded_straight_into_lds_bit_exact(hiplib, oracle, i):
    """Channels-last codes whose tensor is followed by a tail of the padding code: the kernel
    that loads its operands straight into LDS (re-centring and column sums done on the
    fragments, padding fetched from the tail) gives the codes of the restatement, on every
    tile shape, with the bias add's tail rule and the fused threshold."""
    B, Ci, H, W, Co, kH, kW, dH, dW, pH, pW = DIRECT_CASES[i]
    g = cases.rng(1500 + i)
    x = g.uniform(-3, 3, (B, Ci, H, W)).astype(np.float32)
    w = g.standard_normal((Co, Ci, kH, kW), dtype=np.float32) * np.float32(np.sqrt(2.0 / (Ci * kH * kW)))
    b = g.standard_normal(Co, dtype=np.float32) * np.float32(0.5)
    d, p = (dH, dW), (pH, pW)
    rngv = 16.0
    om, osub = float(np.float32(255) / np.float32(rngv)), -rngv / 2
    xq, im, isub = oracle.lowp_quantize(x)
    wq, wm, wsub = oracle.lowp_quantize(w)
    bq, bm, bsub = oracle.lowp_quantize(b)
    want = oracle.lowp_conv2d(xq, im, isub, wq, wm, wsub, bq, bm, bsub, om, osub, d, p)
    prm = oracle.lowp_mm_params(wm, wsub, im, isub, om, osub)
    zero = int(np.round(np.float32(-isub) * np.float32(im)))
    addend = np.array([oracle.lowp_bias_addend(int(c), bm, bsub, om) for c in bq], np.int32)
    thr = oracle.lowp_scale_float(om, osub, 0.0)
    try:
        # (64 x 64 tiles, fourth argument: one K group, or two that share the tile and split its K-tiles)
        for tune in ((0, 0, 0, 0), (64, 64, 9, 1), (64, 64, 9, 2), (128, 64, 9, 0), (64, 128, 9, 0), (128, 128, 9, 0)):
            hiplib.thhip_conv_set_tuning(*tune)
            for y_cl in (1, 0):
                for tail in (64, 200):
                    got = G.conv2d_u8(hiplib, xq, wq, addend, d, p, zero, prm, x_cl=1, y_cl=y_cl, tail=tail)
                    assert np.array_equal(got, want), (tune, y_cl, tail, int((got != want).sum()))
                got = G.conv2d_u8(hiplib, xq, wq, addend, d, p, zero, prm, act=1, thr=thr, val=thr, x_cl=1, y_cl=y_cl, tail=64)
                assert np.array_equal(got, oracle.lowp_threshold(want, thr, thr)), (tune, y_cl)
    finally:
        hiplib.thhip_conv_set_tuning(0, 0, 0, 0)


def test_maxpool_and_relayout_channels_last(hiplib, oracle):
    g = cases.rng(1400)
    for (B, Cn, H, W, kH, kW, dH, dW, pH, pW, ceil) in ((2, 8, 13, 13, 3, 3, 2, 2, 0, 0, 0), (3, 64, 27, 27, 3, 3, 2, 2, 0, 0, 0),
                                                       (1, 12, 7, 9, 2, 2, 2, 2, 1, 1, 1), (2, 4, 10, 8, 2, 3, 1, 2, 0, 1, 0)):
        q = g.integers(0, 256, (B, Cn, H, W), dtype=np.uint8)
        G.note("relayout/maxpool_u8_cl %s" % ((B, Cn, H, W, kH, kW, dH, dW, pH, pW, ceil),))
        dq = api.DeviceArray(hiplib, q)
        dcl = api.DeviceArray(hiplib, nbytes=q.size)
        hiplib.thhip_relayout_u8(dq.ptr, dcl.ptr, B, Cn, H * W, 1)
        hiplib.thhip_sync()
        cl = dcl.get((B, H, W, Cn), np.uint8)
        assert np.array_equal(cl, q.transpose(0, 2, 3, 1))
        dback = api.DeviceArray(hiplib, nbytes=q.size)
        hiplib.thhip_relayout_u8(dcl.ptr, dback.ptr, B, Cn, H * W, 0)
        hiplib.thhip_sync()
        assert np.array_equal(dback.get(q.shape, np.uint8), q)
        want = oracle.lowp_maxpool(q, kH, kW, dH, dW, pH, pW, ceil)
        oH, oW = want.shape[2:]
        dy = api.DeviceArray(hiplib, nbytes=want.size)
        hiplib.thhip_maxpool_u8_cl(dcl.ptr, dy.ptr, B, Cn, H, W, oH, oW, kH, kW, dH, dW, pH, pW)
        hiplib.thhip_sync()
        assert np.array_equal(dy.get((B, oH, oW, Cn), np.uint8).transpose(0, 3, 1, 2), want)


def test_image_layer_with_pooling_bit_exact(hiplib, oracle):
    """thhip_conv2d_u8_image_pool (image layer + Threshold + 3x3 / stride 2 max pooling in one
    kernel) against the restatement's convolution, threshold and pooling run one after the
    other: AlexNet's stem shape, one to four planes, kernel rows of 11, 7, 4 and 5 taps (whole
    and partial groups of four pixels), other vertical strides, images wide and high enough
    for several workgroups per image (and ragged last ones), 64 and 128 output planes,
    parameters that wrap, and the unclamped last positions of a plane."""
    g = cases.rng(1900)
    prms = (dict(a_off=-117, b_off=-128, c_off=32513, c_mult=1028, c_shift=18),
            dict(a_off=-255, b_off=3, c_off=-12345, c_mult=511, c_shift=14),
            dict(a_off=-100, b_off=-90, c_off=5000, c_mult=700, c_shift=17))
    #        B  Ci  H    W   Co   kH  kW dH padH padW
    shapes = ((2, 3, 224, 224, 64, 11, 11, 4, 2, 2),
              (3, 3, 35, 36, 64, 11, 11, 4, 2, 2),
              (1, 1, 47, 52, 64, 7, 7, 4, 3, 3),
              (2, 4, 31, 480, 128, 3, 4, 2, 0, 1),
              (1, 2, 300, 40, 64, 5, 5, 3, 1, 0),
              (2, 3, 27, 28, 64, 11, 9, 4, 0, 5))
    for ci, (B, Ci, H, W, Co, kH, kW, dH, pH, pW) in enumerate(shapes):
        xq = g.integers(0, 256, (B, Ci, H, W), dtype=np.uint8)
        wq = g.integers(0, 256, (Co, Ci, kH, kW), dtype=np.uint8)
        addend = g.integers(-60, 61, Co).astype(np.int32)
        prm = prms[ci % len(prms)]
        zero = 128 if ci % 2 == 0 else 77
        oH, oW = (H + 2 * pH - kH) // dH + 1, (W + 2 * pW - kW) // 4 + 1
        assert hiplib.thhip_conv2d_u8_image_pool_supported(B, Ci, H, W, Co, kH, kW, dH, 4, pH, pW, 3, 3, 2, 2, 0, 0, 0)
        # the restatement, step by step: im2col with the padding code, GEMM, bias add (with its tail), threshold, pooling
        conv = np.empty((B, Co, oH, oW), np.uint8)
        for b in range(B):
            col = oracle.lowp_unfold(xq[b], (kH, kW), (dH, 4), (pH, pW), zero)
            plain = oracle.lowp_gemm(wq.reshape(Co, -1), col, **prm)
            for o in range(Co):
                conv[b, o] = oracle.lowp_add(plain[o], int(addend[o])).reshape(oH, oW)
        thr = oracle.lowp_threshold(conv, 100, 97)
        want = oracle.lowp_maxpool(thr, 3, 3, 2, 2)
        ph, pw = want.shape[2:]
        G.note("conv2d_u8_image_pool x%s w%s dH%d pad(%d,%d) prm%s zero%d" % (xq.shape, wq.shape, dH, pH, pW, prm, zero))
        wp = hiplib.thhip_conv_pack_weight_u8_layout(wq.ctypes.data, Co, Ci, kH, kW, 2)
        dx, da = api.DeviceArray(hiplib, xq), api.DeviceArray(hiplib, addend)
        dy = api.DeviceArray(hiplib, nbytes=B * ph * pw * Co)
        hiplib.thhip_conv2d_u8_image_pool(dx.ptr, wp, da.ptr, dy.ptr, B, Ci, H, W, Co, kH, kW, dH, 4, pH, pW, zero,
                                          prm["a_off"], prm["b_off"], prm["c_off"], prm["c_mult"], prm["c_shift"], 1, 100, 97)
        hiplib.thhip_sync()
        got = dy.get((B, ph, pw, Co), np.uint8).transpose(0, 3, 1, 2)
        assert np.array_equal(got, want), (ci, int((got != want).sum()))
        # without a bias addend and without a threshold
        want2 = oracle.lowp_maxpool(np.stack([oracle.lowp_gemm(wq.reshape(Co, -1), oracle.lowp_unfold(
            xq[b], (kH, kW), (dH, 4), (pH, pW), zero), **prm).reshape(Co, oH, oW) for b in range(B)]), 3, 3, 2, 2)
        hiplib.thhip_conv2d_u8_image_pool(dx.ptr, wp, None, dy.ptr, B, Ci, H, W, Co, kH, kW, dH, 4, pH, pW, zero,
                                          prm["a_off"], prm["b_off"], prm["c_off"], prm["c_mult"], prm["c_shift"], 0, 0, 0)
        hiplib.thhip_sync()
        assert np.array_equal(dy.get((B, ph, pw, Co), np.uint8).transpose(0, 3, 1, 2), want2), ci
        hiplib.thhip_free(wp)
    # shapes the kernel leaves to the general path
    assert not hiplib.thhip_conv2d_u8_image_pool_supported(1, 3, 224, 224, 64, 11, 11, 4, 2, 2, 2, 3, 3, 2, 2, 0, 0, 0)   # stride 2
    assert not hiplib.thhip_conv2d_u8_image_pool_supported(1, 3, 224, 224, 64, 11, 11, 4, 4, 2, 2, 2, 2, 2, 2, 0, 0, 0)   # 2x2 pooling
    assert not hiplib.thhip_conv2d_u8_image_pool_supported(1, 3, 224, 224, 48, 11, 11, 4, 4, 2, 2, 3, 3, 2, 2, 0, 0, 0)   # 48 planes
    assert not hiplib.thhip_conv2d_u8_image_pool_supported(1, 5, 224, 224, 64, 11, 11, 4, 4, 2, 2, 3, 3, 2, 2, 0, 0, 0)   # 5 planes


def test_conv_u8_patch_bit_exact(hiplib, oracle):
    """thhip_conv2d_u8_patch (input patch kept in LDS, optional 3x3 / stride 2 pooling) against
    the restatement step by step: AlexNet's conv2-5 shapes, several bands per image with and
    without pooling, kernels of 1x1, 2x3, 3x3 and 5x5 taps, one to eight blocks of 64 input
    planes (the whole patch in LDS before the K loop, or streamed block by block with weight
    rings of three and five K-tiles), a last band shorter than the others, padding codes other
    than 128, wrapping parameters, and the unclamped last positions of a plane."""
    g = cases.rng(2000)
    prms = (dict(a_off=-117, b_off=-128, c_off=32513, c_mult=1028, c_shift=18),
            dict(a_off=-255, b_off=3, c_off=-12345, c_mult=511, c_shift=14),
            dict(a_off=-100, b_off=-90, c_off=5000, c_mult=700, c_shift=19))
    #        B  Ci   H   W   Co  kH kW padH padW pool
    shapes = ((2, 192, 13, 13, 384, 3, 3, 1, 1, 0),
              (2, 64, 27, 27, 192, 5, 5, 2, 2, 1),
              (3, 256, 13, 13, 256, 3, 3, 1, 1, 1),
              (2, 64, 27, 27, 64, 5, 5, 2, 2, 0),
              (1, 128, 9, 20, 64, 2, 3, 0, 1, 0),
              (2, 384, 13, 13, 128, 3, 3, 1, 1, 0),
              (1, 64, 40, 60, 64, 3, 3, 1, 1, 1),
              (1, 64, 7, 100, 128, 3, 3, 0, 0, 0),
              (2, 128, 13, 13, 64, 1, 1, 0, 0, 0),
              (1, 512, 13, 13, 64, 3, 3, 1, 1, 1),
              (1, 64, 23, 23, 64, 3, 3, 1, 1, 1),
              (2, 128, 11, 11, 64, 5, 5, 2, 2, 1),       # streamed patch, weight ring of five
              (2, 128, 14, 14, 64, 3, 3, 1, 1, 1),       # streamed, ring of three, pooled
              (1, 192, 6, 6, 64, 3, 3, 0, 0, 0),
              (1, 128, 9, 9, 64, 3, 5, 1, 2, 0),         # 15 taps: three groups of five
              (1, 128, 9, 9, 64, 3, 2, 1, 1, 0),         # 6 taps: an even number of groups of three - not streamed
              (1, 128, 20, 20, 64, 3, 3, 1, 1, 0))       # a patch of more than 256 pixels - not streamed
    for ci, (B, Ci, H, W, Co, kH, kW, pH, pW, pool) in enumerate(shapes):
        xq = g.integers(0, 256, (B, Ci, H, W), dtype=np.uint8)
        wq = g.integers(0, 256, (Co, Ci, kH, kW), dtype=np.uint8)
        addend = g.integers(-60, 61, Co).astype(np.int32)
        prm = prms[ci % len(prms)]
        zero = 128 if ci % 2 == 0 else 77
        oH, oW = H + 2 * pH - kH + 1, W + 2 * pW - kW + 1
        assert hiplib.thhip_conv2d_u8_patch_supported(B, Ci, H, W, Co, kH, kW, 1, 1, pH, pW, pool), ci
        conv = np.empty((B, Co, oH, oW), np.uint8)
        for b in range(B):
            col = oracle.lowp_unfold(xq[b], (kH, kW), (1, 1), (pH, pW), zero)
            plain = oracle.lowp_gemm(wq.reshape(Co, -1), col, **prm)
            for o in range(Co):
                conv[b, o] = oracle.lowp_add(plain[o], int(addend[o])).reshape(oH, oW)
        want = oracle.lowp_threshold(conv, 100, 97)
        if pool:
            want = oracle.lowp_maxpool(want, 3, 3, 2, 2)
        yh, yw = want.shape[2:]
        G.note("conv2d_u8_patch x%s w%s pad(%d,%d) pool%d prm%s zero%d" % (xq.shape, wq.shape, pH, pW, pool, prm, zero))
        wp = hiplib.thhip_conv_pack_weight_u8_patch(wq.ctypes.data, Co, Ci, kH, kW)
        dx = api.DeviceArray(hiplib, np.ascontiguousarray(xq.transpose(0, 2, 3, 1)))
        da = api.DeviceArray(hiplib, addend)
        dy = api.DeviceArray(hiplib, nbytes=B * yh * yw * Co)
        hiplib.thhip_memset(dy.ptr, 0x5a, B * yh * yw * Co)
        hiplib.thhip_conv2d_u8_patch(dx.ptr, wp, da.ptr, dy.ptr, B, Ci, H, W, Co, kH, kW, 1, 1, pH, pW, zero,
                                     prm["a_off"], prm["b_off"], prm["c_off"], prm["c_mult"], prm["c_shift"], 1, 100, 97, pool)
        hiplib.thhip_sync()
        got = dy.get((B, yh, yw, Co), np.uint8).transpose(0, 3, 1, 2)
        assert np.array_equal(got, want), (ci, int((got != want).sum()))
        hiplib.thhip_free(wp)
    assert not hiplib.thhip_conv2d_u8_patch_supported(1, 64, 13, 13, 64, 3, 3, 2, 2, 1, 1, 0)    # stride 2
    assert not hiplib.thhip_conv2d_u8_patch_supported(1, 96, 13, 13, 64, 3, 3, 1, 1, 1, 1, 0)    # 96 planes
    assert not hiplib.thhip_conv2d_u8_patch_supported(1, 4096, 13, 13, 64, 3, 3, 1, 1, 1, 1, 0)  # one output row: a patch of 180 KB
    assert not hiplib.thhip_conv2d_u8_patch_supported(1, 64, 13, 300, 64, 3, 3, 1, 1, 1, 1, 0)   # rows of 300 positions


def _linear_u8(hiplib, xq, wq, addend, prm, act=0, thr=0, val=0):
    B, K = xq.shape
    nOut = wq.shape[0]
    G.note("linear_batched_u8 B=%d K=%d nOut=%d prm%s act=%d" % (B, K, nOut, prm, act))
    assert hiplib.thhip_linear_batched_u8_supported(B, K, nOut)
    wp = hiplib.thhip_linear_pack_weight_u8(wq.ctypes.data, nOut, K)
    rs = hiplib.thhip_u8_rowsums(wq.ctypes.data, nOut, K)
    dx = api.DeviceArray(hiplib, xq)
    da = api.DeviceArray(hiplib, np.ascontiguousarray(addend, np.int32)) if addend is not None else None
    dy = api.DeviceArray(hiplib, nbytes=B * nOut)
    hiplib.thhip_linear_batched_u8(dx.ptr, wp, rs, da.ptr if da else None, dy.ptr, B, K, nOut, prm["a_off"], prm["b_off"],
                                   prm["c_off"], prm["c_mult"], prm["c_shift"], act, thr, val)
    hiplib.thhip_sync()
    y = dy.get((B, nOut), np.uint8)
    hiplib.thhip_free(wp)
    hiplib.thhip_free(rs)
    return y


def test_linear_batched_u8_bit_exact(hiplib, oracle):
    """One-position layers through the matrix kernel: against the GEMM + bias add of the
    restatement (a plane of one element is all tail: no lower clamp), ragged rows,
    batches (one, two and four groups of sixteen columns) and K tails (K % 64 of 16, 48;
    fewer K-steps than wavefronts), layers wide enough for two row blocks per workgroup, with
    wrapping parameters."""
    g = cases.rng(1200)
    prms = (dict(a_off=-117, b_off=-128, c_off=32513, c_mult=1028, c_shift=18),
            dict(a_off=-255, b_off=3, c_off=-12345, c_mult=511, c_shift=14),
            dict(a_off=0, b_off=0, c_off=0, c_mult=9000, c_shift=20))
    shapes = ((1, 16, 1), (2, 144, 37), (33, 1024, 100), (64, 2064, 70), (17, 4096, 130), (64, 9216, 64),
              (16, 1088, 16), (32, 64, 33), (48, 4144, 17), (5, 6400, 1000),
              # wide layers, two blocks of sixteen rows per workgroup: whole, a ragged last block, an odd number of blocks
              (64, 1024, 4096), (20, 320, 4090), (33, 128, 4104))
    for ci, (B, K, nOut) in enumerate(shapes):
        xq = g.integers(0, 256, (B, K), dtype=np.uint8)
        wq = g.integers(0, 256, (nOut, K), dtype=np.uint8)
        addend = g.integers(-40, 41, nOut).astype(np.int32)
        prm = prms[ci % len(prms)]
        plain = oracle.lowp_gemm(wq, np.ascontiguousarray(xq.T), **prm).T        # [B][nOut]
        biased = np.stack([[oracle.lowp_add(plain[b, o:o + 1], int(addend[o]))[0] for o in range(nOut)]
                           for b in range(B)]).astype(np.uint8)
        assert np.array_equal(_linear_u8(hiplib, xq, wq, None, prm), plain), (B, K, nOut)
        assert np.array_equal(_linear_u8(hiplib, xq, wq, addend, prm), biased), (B, K, nOut)
        got = _linear_u8(hiplib, xq, wq, addend, prm, act=1, thr=100, val=97)
        assert np.array_equal(got, oracle.lowp_threshold(biased, 100, 97)), (B, K, nOut)
    assert not hiplib.thhip_linear_batched_u8_supported(65, 1024, 10)
    assert not hiplib.thhip_linear_batched_u8_supported(4, 1000, 10)


def test_threshold_and_softmax_u8_bit_exact(hiplib, oracle):
    q = cases.rng(1102).integers(0, 256, (3, 1000), dtype=np.uint8)
    y = G.unary(hiplib, hiplib.thhip_threshold_u8, q, q.shape, G.U8, q.size, 127, 127, 1)
    assert np.array_equal(y, oracle.lowp_threshold(q, 127, 127, 1))
    for shape in [(3, 1000), (1000,), (2, 21, 3, 3)]:
        q = cases.rng(1103).integers(0, 256, shape, dtype=np.uint8)
        if len(shape) == 1:
            nframe, dim, stride = 1, shape[0], 1
        elif len(shape) == 2:
            nframe, dim, stride = shape[0], shape[1], 1
        else:
            nframe, dim, stride = shape[0], shape[1], shape[2] * shape[3]
        dx = api.DeviceArray(hiplib, q)
        dy = api.DeviceArray(hiplib, nbytes=q.size)
        hiplib.thhip_softmax_u8.restype = C.c_float
        om = hiplib.thhip_softmax_u8(dx.ptr, dy.ptr, nframe, dim, stride, 7.96875, -16.0)
        hiplib.thhip_sync()
        want, wm, _ = oracle.lowp_softmax(q, 7.96875, -16.0)
        assert np.array_equal(dy.get(shape, np.uint8), want)
        assert om == np.float32(wm)


def test_engine_small_network_bit_exact_every_layer(hiplib, oracle):
    g = cases.rng(17)
    w1 = g.standard_normal((6, 3, 3, 3), dtype=np.float32) * np.float32(0.3)
    w2 = g.standard_normal((5, 6, 2, 2), dtype=np.float32) * np.float32(0.3)
    layers = [configs.conv(w1, g.standard_normal(6, dtype=np.float32) * np.float32(0.1), 1, 1), configs.relu(),
              configs.maxpool(2, 2),
              configs.conv(w2, g.standard_normal(5, dtype=np.float32) * np.float32(0.1), 1, 0), configs.relu(),
              {"type": "softmax"}]
    x = g.uniform(-2, 2, (5, 3, 8, 8)).astype(np.float32)
    net = api.HipNetwork(layers, lowp_range=16.0)
    y = net.process_float(x)
    xq, im, isub = oracle.lowp_quantize(x)
    outs = []
    q, m, s = oracle.lowp_run_layers(layers, xq, im, isub, 16.0, collect=outs)
    for i in (1, 2, 4, 5):      # conv outputs hold the fused threshold, compare after it
        assert np.array_equal(net.module_output(i).astype(np.uint8), outs[i][0]), i
    assert np.array_equal(y, oracle.lowp_dequantize(q, m, s).ravel())
    # a second forward on the same engine instance gives the same codes (the reference
    # loses its quantisation parameters after the first)
    assert np.array_equal(net.process_float(x), y)
    net.free()


def _oracle_load_images(oracle, imgs, mean, std, bgr):
    n, (H, W) = len(imgs), imgs[0].shape[:2]
    dst = np.empty((n, 3, H, W), np.uint8)
    ptrs = (C.c_void_p * n)(*[im.ctypes.data for im in imgs])
    m, s = C.c_float(), C.c_float()
    oracle.lib.orc_lowp_load_images(dst.ctypes.data_as(C.POINTER(C.c_ubyte)), ptrs, n, W, H, W * 3,
                                    (C.c_float * 3)(*mean), (C.c_float * 3)(*std), bgr, C.byref(m), C.byref(s))
    return dst, m.value, s.value


def test_process_images_uint8_engine(hiplib, oracle):
    """THProcessImages on the uint8 engine: the image loader's codes (fixed range from
    mean / std, values outside 0..255 wrapping like the reference's build) bit for bit,
    then the same network codes and de-quantised result as the restatement."""
    g = cases.rng(1500)
    mean, std = (0.485, 0.456, 0.406), (0.229, 0.224, 0.225)
    imgs = [np.ascontiguousarray(g.integers(0, 256, (9, 11, 3), dtype=np.uint8)) for _ in range(3)]
    for bgr in (0, 1):
        want, wm, ws = _oracle_load_images(oracle, imgs, mean, std, bgr)
        m, s_ = C.c_float(), C.c_float()
        for i, im in enumerate(imgs):
            dsrc = api.DeviceArray(hiplib, im)
            ddst = api.DeviceArray(hiplib, nbytes=3 * 9 * 11)
            hiplib.thhip_rgb2code(ddst.ptr, dsrc.ptr, 11, 9, 33, (C.c_float * 3)(*mean), (C.c_float * 3)(*std), bgr,
                                  C.byref(m), C.byref(s_))
            hiplib.thhip_sync()
            assert np.array_equal(ddst.get((3, 9, 11), np.uint8), want[i]), (bgr, i)
        assert (m.value, s_.value) == (wm, ws)
    w1 = g.standard_normal((8, 3, 3, 3), dtype=np.float32) * np.float32(0.3)
    w2 = g.standard_normal((5, 8, 2, 2), dtype=np.float32) * np.float32(0.3)
    layers = [configs.conv(w1, g.standard_normal(8, dtype=np.float32) * np.float32(0.1), 1, 1), configs.relu(),
              configs.maxpool(2, 2),
              configs.conv(w2, g.standard_normal(5, dtype=np.float32) * np.float32(0.1), 1, 0), configs.relu()]
    imgs = [np.ascontiguousarray(g.integers(0, 256, (8, 10, 3), dtype=np.uint8)) for _ in range(4)]
    net = api.HipNetwork(layers, mean, std, lowp_range=16.0)
    for bgr in (0, 1):
        y = net.process_images(imgs, bgr=bgr)
        xq, im_, isub = _oracle_load_images(oracle, imgs, mean, std, bgr)
        outs = []
        q, mo, so = oracle.lowp_run_layers(layers, xq, im_, isub, 16.0, collect=outs)
        assert np.array_equal(net.module_output(4).astype(np.uint8), outs[4][0]), bgr
        assert np.array_equal(y, oracle.lowp_dequantize(q, mo, so).ravel()), bgr
    net.free()


def _device_codes(hiplib, net, q):
    """uint8 codes -> a device tensor struct the engine accepts (test-side construction:
    storage marked as engine-owned device memory, extra reference so it is never freed
    by the library)."""
    from thnets_amd import abi
    dev = api.DeviceArray(hiplib, np.ascontiguousarray(q, np.uint8))
    st = abi.THFloatStorage(dev.ptr, 2, abi.TH_MUSTFREE_HIP + abi.THHIP_U8)
    t = abi.ABI.THFloatTensor()
    t.nDimension = q.ndim
    stride = 1
    for i in range(q.ndim - 1, -1, -1):
        t.size[i] = q.shape[i]
        t.stride[i] = stride
        stride *= q.shape[i]
    t.storage = C.pointer(st)
    return t, (dev, st)


def _fused_expectation(layers, outs, i, got_shape):
    """What module i's buffer holds: its own codes, those of the Threshold folded into
    it, or - when the convolution ran with its Threshold and max pooling as one kernel -
    the pooled codes.  Returns (index into outs, fused pooling?)."""
    j = i
    if i + 1 < len(layers) and layers[i + 1]["type"] == "threshold":
        j = i + 1
    if tuple(got_shape[1:]) != tuple(outs[j][0].shape[1:]):
        j = next(k for k in range(i + 1, len(layers)) if layers[k]["type"] == "maxpool")
        assert layers[i]["type"] in ("conv", "threshold") and j <= i + 2, (i, got_shape, outs[j][0].shape)
        return j, True
    return j, False


def test_alexnet_lowp_full_size_bit_exact_all_64_images(hiplib, oracle):
    """Configuration 5 at its real layer shapes and batch size.  Every code of every
    module output of ALL 64 images is compared with the CPU oracle (run here, one
    image at a time with the batch's quantisation, as the reference's engine has to be
    driven) and with the committed checksums tests/golden/alexnet_lowp_b64_golden.npz;
    the codes of the last layer also with the fixture's full copy.  Then images 0, 3,
    40 and 63 as a batch of four must give, module by module, the same codes as their
    rows of the batch of 64 (a result must not depend on the batch an image is in)."""
    import os
    import zlib
    gold = np.load(os.path.join(os.path.dirname(__file__), "golden", "alexnet_lowp_b64_golden.npz"))
    cfg = configs.alexnet_lowp(batch=64)
    layers = cfg["layers"]
    x = oracle.normalize(cfg["input"], cfg["mean"], cfg["std"])
    net = api.HipNetwork(layers, lowp_range=cfg["range"])
    xq, im, isub = oracle.lowp_quantize(x)              # one min/max over the whole batch
    assert (np.float32(im), np.float32(isub)) == tuple(gold["input/quant"])
    G.note("alexnet lowp b64 forward")
    t, keep = _device_codes(hiplib, net, xq)
    assert hiplib.THHipNetwork_setInputQuant(net.handle, im, isub) == 0
    hiplib.THForward(net.handle, C.addressof(t))
    last = net.nelem - 1
    got64 = [net.module_output(i).astype(np.uint8) for i in range(net.nelem)]
    assert got64[last].shape == (64, 1000, 1, 1)
    # the oracle on all 64 images, eight at a time
    parts = []
    for b0 in range(0, 64, 8):
        outs = []
        oracle.lowp_run_layers(layers, xq[b0:b0 + 8], im, isub, cfg["range"], collect=outs)
        parts.append(outs)
    outs = [(np.concatenate([p[i][0] for p in parts]), parts[0][i][1], parts[0][i][2]) for i in range(len(layers))]
    fused_pool = False
    images_checked = np.zeros(64, bool)
    for i in range(len(layers)):
        j, fused = _fused_expectation(layers, outs, i, got64[i].shape)
        fused_pool |= fused
        want = outs[j][0]
        differ = (got64[i] != want).reshape(64, -1).sum(axis=1)
        assert not differ.any(), "module %d (%s): images %s differ in %d codes" % (
            i, layers[i]["type"], np.flatnonzero(differ).tolist(), differ.sum())
        # the committed fixture, image by image
        crc = np.array([zlib.crc32(got64[i][b].tobytes()) for b in range(64)], np.uint32)
        assert np.array_equal(crc, gold["module%d/crc" % j]), (i, np.flatnonzero(crc != gold["module%d/crc" % j]))
        assert np.array_equal(got64[i].reshape(64, -1).sum(axis=1, dtype=np.int64), gold["module%d/sum" % j])
        assert net.module_quant(i) == (np.float32(outs[i][1]), np.float32(outs[i][2])) == tuple(gold["module%d/quant" % i])
        images_checked |= ~differ.astype(bool)
    assert images_checked.all() and images_checked.size == 64
    assert np.array_equal(got64[last].reshape(64, -1), gold["last/codes"])
    assert fused_pool, "the image layer of AlexNet should take the fused convolution + pooling kernel"
    # the logits carry information (not saturated everywhere)
    assert len(np.unique(got64[last])) > 20
    # the same images in a small batch: the same codes
    sel = [0, 3, 40, 63]
    G.note("alexnet lowp b4 forward")
    t2, keep2 = _device_codes(hiplib, net, xq[sel])
    hiplib.THHipNetwork_setInputQuant(net.handle, im, isub)
    hiplib.THForward(net.handle, C.addressof(t2))
    for i in range(len(layers)):
        got = net.module_output(i).astype(np.uint8)
        assert np.array_equal(got, got64[i][sel]), "module %d: a batch of 4 and a batch of 64 differ" % i
    net.free()
