"""Parity of every hand-written HIP kernel, called through the C ABI, against the CPU
oracle on the same seeded inputs and against the reference-made golden vectors.

Tolerances (from the task's contract): fp32 GEMM-shaped results max|err| <= 1e-3 *
max|ref| (observed ~1e-6; the tests hold them to 2e-5); fp16 / bf16 2e-2 relative to
max|ref|; everything that is not a sum (threshold, pooling, batchnorm, image loading,
uint8 codes) bit-exact.
"""
import os

import numpy as np
import pytest

import cases
import gpu_util as G

pytestmark = pytest.mark.gpu

GOLD = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "fp32_golden.npz"))
FP32_TOL = 2e-5
HALF_TOL = 2e-2


@pytest.mark.parametrize("i", range(len(cases.CONV_CASES)))
def test_conv_f32_vs_oracle_and_golden(hiplib, oracle, i):
    x, s = cases.conv_case(i)
    d, p = (s["dH"], s["dW"]), (s["padH"], s["padW"])
    y = G.conv2d(hiplib, x, s["weight"], s["bias"], d, p)
    G.assert_close(y, oracle.conv2d(x, s["weight"], s["bias"], d, p), FP32_TOL, "oracle")
    G.assert_close(y, GOLD["conv%d" % i], FP32_TOL, "golden")
    # fused Threshold epilogue == Threshold applied afterwards (bit-exact)
    ya = G.conv2d(hiplib, x, s["weight"], s["bias"], d, p, act=1, thr=0.1, val=-0.5)
    assert np.array_equal(ya, np.where(y > np.float32(0.1), y, np.float32(-0.5)))
    # no bias
    G.assert_close(G.conv2d(hiplib, x, s["weight"], None, d, p), oracle.conv2d(x, s["weight"], None, d, p), FP32_TOL)
    # both K-tile depths of the fp32 kernel (the launcher picks one by layer width)
    try:
        for chunks in (2, 4):
            hiplib.thhip_conv_set_ktile(chunks)
            G.assert_close(G.conv2d(hiplib, x, s["weight"], s["bias"], d, p), GOLD["conv%d" % i], FP32_TOL, "ktile %d" % chunks)
    finally:
        hiplib.thhip_conv_set_ktile(0)


def test_conv_f32_ktile_depths_tap_major_and_split(hiplib, oracle):
    """Tap-major fp32 layers (planes in blocks of 32) at both K-tile depths, with forced
    tiles and K splits that start inside a block."""
    g = cases.rng(910)
    for (B, Ci, H, W, Co, k, dd, pp) in ((2, 32, 9, 10, 70, 3, 1, 1), (1, 96, 7, 7, 130, 3, 2, 1), (3, 64, 6, 5, 64, 1, 1, 0),
                                         (2, 32, 23, 17, 300, 3, 1, 1)):
        x = g.uniform(-1, 1, (B, Ci, H, W)).astype(np.float32)
        w = g.standard_normal((Co, Ci, k, k), dtype=np.float32) * np.float32(np.sqrt(2.0 / (Ci * k * k)))
        b = g.standard_normal(Co, dtype=np.float32) * np.float32(0.1)
        want = oracle.conv2d(x, w, b, (dd, dd), (pp, pp))
        try:
            for chunks in (2, 4):
                hiplib.thhip_conv_set_ktile(chunks)
                for tune in ((0, 0, 0, 0), (64, 64, 3, 0), (128, 64, 2, 2), (128, 128, 5, 0), (64, 128, 1, 1)):
                    hiplib.thhip_conv_set_tuning(*tune)
                    G.assert_close(G.conv2d(hiplib, x, w, b, (dd, dd), (pp, pp)), want, FP32_TOL, str((chunks, tune)))
            # every way of cutting the tile grid over the XCDs, with ragged rectangles and a K split
            hiplib.thhip_conv_set_ktile(0)
            for parts in (1, 2, 4, 8):
                hiplib.thhip_conv_set_xcd_parts(parts)
                for tune in ((64, 64, 0, 0), (64, 64, 2, 0)):
                    hiplib.thhip_conv_set_tuning(*tune)
                    G.assert_close(G.conv2d(hiplib, x, w, b, (dd, dd), (pp, pp)), want, FP32_TOL, str((parts, tune)))
        finally:
            hiplib.thhip_conv_set_ktile(0)
            hiplib.thhip_conv_set_xcd_parts(0)
            hiplib.thhip_conv_set_tuning(0, 0, 0, 0)


def test_conv_f32_loaded_straight_into_lds(hiplib, oracle):
    """The fp32 kernel whose operands go from global memory straight to LDS (plane-major
    tensors, planes in blocks of 32): K-tile counts 1..13 around the edges of its
    three-stage pipeline, partial tiles on both axes, strides, padding, the folded
    batch-norm factor and the fused threshold, both tile shapes and K-tile depths."""
    from thnets_amd import api
    g = cases.rng(913)
    shapes = [(2, 32, 9, 10, 70, 1, 1, 0), (1, 64, 7, 7, 130, 1, 2, 0), (1, 96, 6, 5, 64, 1, 1, 0), (2, 32, 12, 11, 36, 2, 1, 1),
              (1, 160, 5, 5, 40, 1, 1, 0), (1, 192, 6, 6, 72, 1, 1, 0), (1, 224, 4, 7, 33, 1, 1, 0), (2, 32, 23, 17, 300, 3, 1, 1),
              (1, 96, 7, 7, 130, 3, 2, 1), (3, 64, 14, 14, 96, 3, 1, 1), (1, 416, 4, 4, 64, 1, 1, 0), (1, 64, 20, 20, 64, 5, 1, 2)]
    try:
        for (B, Ci, H, W, Co, k, dd, pp) in shapes:
            x = g.uniform(-1, 1, (B, Ci, H, W)).astype(np.float32)
            w = g.standard_normal((Co, Ci, k, k), dtype=np.float32) * np.float32(np.sqrt(2.0 / (Ci * k * k)))
            b = g.standard_normal(Co, dtype=np.float32) * np.float32(0.1)
            want = np.maximum(oracle.conv2d(x, w, b, (dd, dd), (pp, pp)), 0)
            # K-tiles of 32, of 16; then K split in 2, 3 and 7 parts (last argument / 10), more parts than K-tiles included
            for tune in ((64, 64, 9, 0), (128, 64, 9, 0), (64, 64, 9, 2), (128, 64, 9, 2), (64, 64, 9, 20), (128, 64, 9, 32), (64, 64, 9, 70)):
                G.note("fp32 straight to LDS %s tile %s" % ((B, Ci, H, W, Co, k, dd, pp), tune))
                hiplib.thhip_conv_set_tuning(*tune)
                got = G.conv2d(hiplib, x, w, b, (dd, dd), (pp, pp), act=1, thr=0.0, val=0.0)
                G.assert_close(got, want, FP32_TOL, str((Ci, Co, k, tune)))
    finally:
        hiplib.thhip_conv_set_tuning(0, 0, 0, 0)


def test_conv_f32_last_tiles_cut_along_k(hiplib, oracle):
    """fp32 tiles loaded straight into LDS: the tiles an XCD cannot spread evenly over its
    CUs are cut along K and summed in order by a second kernel.  Layers where every tile
    is cut (few tiles), where only the last ones are (784 tiles: 98 per XCD), with
    partial tiles on both axes, the folded batch-norm factor and the threshold; every
    limit on the parts, 1 = never cut; the same call twice gives the same bits."""
    g = cases.rng(917)
    # last entry: the M tiles cut into that many groups over the XCDs (0: by weight size)
    shapes = [(4, 64, 112, 112, 64, 3, 1, 1, 0), (1, 64, 20, 20, 64, 5, 1, 2, 0), (2, 96, 30, 30, 70, 3, 1, 1, 0),
              (5, 128, 28, 28, 128, 3, 1, 1, 0), (3, 256, 27, 27, 100, 3, 2, 1, 0), (4, 64, 112, 112, 128, 3, 1, 1, 2)]
    try:
        for (B, Ci, H, W, Co, k, dd, pp, mparts) in shapes:
            hiplib.thhip_conv_set_xcd_parts(mparts)
            x = g.uniform(-1, 1, (B, Ci, H, W)).astype(np.float32)
            w = g.standard_normal((Co, Ci, k, k), dtype=np.float32) * np.float32(np.sqrt(2.0 / (Ci * k * k)))
            b = g.standard_normal(Co, dtype=np.float32) * np.float32(0.1)
            sc = g.uniform(0.5, 1.5, Co).astype(np.float32)
            plain = oracle.conv2d(x, w, None, (dd, dd), (pp, pp))
            want = np.maximum(plain * sc[None, :, None, None] + b[None, :, None, None], 0)
            for parts in (1, 2, 8, 64):
                G.note("fp32 last tiles cut along K %s parts %d" % ((B, Ci, H, W, Co, k, dd, pp), parts))
                hiplib.thhip_conv_set_tail_parts(parts)
                got = G.conv2d_layout(hiplib, x, w, b, (dd, dd), (pp, pp), act=1, dtype=G.F32, scale=sc)
                G.assert_close(got, want, FP32_TOL, str((Ci, Co, k, parts)))
                again = G.conv2d_layout(hiplib, x, w, b, (dd, dd), (pp, pp), act=1, dtype=G.F32, scale=sc)
                assert np.array_equal(got, again), "cut tiles: results depend on timing"
    finally:
        hiplib.thhip_conv_set_tail_parts(8)
        hiplib.thhip_conv_set_xcd_parts(0)


def test_conv_f32_image_layer_with_pooling(hiplib, oracle):
    """thhip_conv2d_image_pool (an fp32 image layer, its folded batch norm factor, Threshold and the
    3x3 / stride 2 max pooling in one kernel) against the oracle's convolution -> factor and shift ->
    Threshold -> max pooling: ResNet's 7x7 / stride 2 stem at 224 x 224 and 112 x 112, pooling padding 1
    and 0 (the padding must never win a maximum: all-negative planes without a Threshold), one to four
    input planes, other kernels and strides, 128 output planes, a last group of pooled rows that is
    not full; and the layers it leaves to the other kernels."""
    from thnets_amd import api
    g = cases.rng(941)
    #         B  Ci   H    W   Co  k  d pad ppad
    shapes = [(2, 3, 224, 224, 64, 7, 2, 3, 1), (1, 3, 112, 112, 128, 7, 2, 3, 1), (2, 3, 115, 115, 64, 7, 2, 3, 0),
              (1, 1, 57, 111, 64, 3, 2, 1, 1), (1, 4, 60, 58, 64, 5, 2, 2, 0), (1, 2, 100, 224, 64, 4, 4, 0, 1),
              (1, 3, 84, 56, 64, 3, 1, 1, 1)]
    for (B, Ci, H, W, Co, k, d, pad, ppad) in shapes:
        x = g.uniform(-1, 1, (B, Ci, H, W)).astype(np.float32)
        w = g.standard_normal((Co, Ci, k, k), dtype=np.float32) * np.float32(np.sqrt(2.0 / (Ci * k * k)))
        b = g.standard_normal(Co, dtype=np.float32) * np.float32(0.1)
        b[::3] -= np.float32(40)       # whole planes far below zero
        sc = (g.uniform(0.5, 1.5, Co) * g.choice([-1.0, 1.0], Co)).astype(np.float32)
        oH, oW = (H + 2 * pad - k) // d + 1, (W + 2 * pad - k) // d + 1
        pH, pW = oracle.pool_outsize(oH, oW, 3, 3, 2, 2, ppad, ppad, 0)
        raw = oracle.conv2d(x, w, None, (d, d), (pad, pad))
        for act, scale in ((1, sc), (0, sc), (1, None)):
            G.note("image layer + pooling %s act %d scale %s" % ((B, Ci, H, W, Co, k, d, pad, ppad), act, scale is not None))
            assert hiplib.thhip_conv2d_image_pool_supported(B, Ci, H, W, Co, k, k, d, d, pad, pad, 3, 3, 2, 2, ppad, ppad, 0, G.F32, 0), \
                (B, Ci, H, W, Co, k, d, pad, ppad)
            dx = api.DeviceArray(hiplib, x)
            wp = hiplib.thhip_conv_pack_weight_layout(np.ascontiguousarray(w).ctypes.data, Co, Ci, k, k, G.F32, 0)
            db = api.DeviceArray(hiplib, b)
            ds = api.DeviceArray(hiplib, scale) if scale is not None else None
            dy = api.DeviceArray(hiplib, nbytes=B * Co * pH * pW * 4)
            hiplib.thhip_memset(dy.ptr, 0x7f, B * Co * pH * pW * 4)
            hiplib.thhip_conv2d_image_pool(dx.ptr, wp, ds.ptr if ds else None, db.ptr, dy.ptr, B, Ci, H, W, Co, k, k, d, d, pad, pad,
                                           ppad, act, 0.25, -0.5, G.F32)
            hiplib.thhip_sync()
            got = dy.get((B, Co, pH, pW), np.float32)
            hiplib.thhip_free(wp)
            v = raw * scale[None, :, None, None] if scale is not None else raw
            v = v + b[None, :, None, None]
            if act:
                v = np.where(v > np.float32(0.25), v, np.float32(-0.5)).astype(np.float32)
            want = oracle.maxpool(v, 3, 3, 2, 2, ppad, ppad, 0)
            G.assert_close(got, want, FP32_TOL, str((B, Ci, H, W, Co, k, d, pad, ppad, act)))
    sup = hiplib.thhip_conv2d_image_pool_supported
    assert not sup(2, 3, 224, 224, 64, 7, 7, 2, 2, 3, 3, 2, 2, 2, 2, 0, 0, 0, G.F32, 0)       # a 2x2 pooling
    assert not sup(2, 3, 224, 224, 64, 7, 7, 2, 2, 3, 3, 3, 3, 2, 2, 1, 1, 1, G.F32, 0)       # ceil mode
    assert not sup(2, 3, 224, 224, 64, 7, 7, 2, 2, 3, 3, 3, 3, 2, 2, 1, 1, 0, G.F16, 0)       # a half type
    assert not sup(2, 8, 224, 224, 64, 7, 7, 2, 2, 3, 3, 3, 3, 2, 2, 1, 1, 0, G.F32, 0)       # eight planes
    assert not sup(2, 3, 224, 224, 96, 7, 7, 2, 2, 3, 3, 3, 3, 2, 2, 1, 1, 0, G.F32, 0)       # 96 output planes
    assert not sup(2, 3, 200, 200, 64, 7, 7, 2, 2, 3, 3, 3, 3, 2, 2, 1, 1, 0, G.F32, 0)       # pooled rows of 50 positions


def test_conv_f32_k_split_with_a_pooling_of_any_window(hiplib, oracle):
    """fp32 layers of a few tiles split K and a second kernel adds the parts; that kernel also takes a max
    pooling that follows (any window, stride, padding, rounding): the same bits as the convolution entry
    point followed by the pooling one, the oracle's values, on AlexNet's batch-1 layers (planes in blocks of
    32 or not), with the folded factor, with and without the threshold; layers it does not take."""
    from thnets_amd import api
    g = cases.rng(931)
    # (B, Ci, H, W, Co, k, d, pad), (pool kH, kW, dH, dW, padH, padW, ceil)
    shapes = [((1, 3, 224, 224, 64, 11, 4, 2), (3, 3, 2, 2, 0, 0, 0)), ((1, 64, 27, 27, 192, 5, 1, 2), (3, 3, 2, 2, 0, 0, 0)),
              ((1, 256, 13, 13, 256, 3, 1, 1), (3, 3, 2, 2, 0, 0, 0)), ((2, 96, 20, 21, 70, 3, 1, 1), (2, 2, 2, 2, 0, 0, 1)),
              ((3, 40, 17, 15, 33, 3, 1, 0), (3, 2, 2, 1, 1, 1, 1)), ((1, 128, 9, 9, 100, 3, 1, 1), (9, 9, 1, 1, 0, 0, 0))]
    for (B, Ci, H, W, Co, k, d, pad), (pkH, pkW, pdH, pdW, ppH, ppW, ceil) in shapes:
        x = g.uniform(-1, 1, (B, Ci, H, W)).astype(np.float32)
        w = g.standard_normal((Co, Ci, k, k), dtype=np.float32) * np.float32(np.sqrt(2.0 / (Ci * k * k)))
        b = g.standard_normal(Co, dtype=np.float32) * np.float32(0.1)
        sc = (g.uniform(0.5, 1.5, Co) * g.choice([-1.0, 1.0], Co)).astype(np.float32)
        oH, oW = (H + 2 * pad - k) // d + 1, (W + 2 * pad - k) // d + 1
        pH, pW = oracle.pool_outsize(oH, oW, pkH, pkW, pdH, pdW, ppH, ppW, ceil)
        raw = oracle.conv2d(x, w, None, (d, d), (pad, pad)) * sc[None, :, None, None] + b[None, :, None, None]
        for act in (1, 0):
            G.note("conv + pooling of any window %s %s act %d" % ((B, Ci, H, W, Co, k, d, pad), (pkH, pkW, pdH, pdW, ppH, ppW, ceil), act))
            assert hiplib.thhip_conv2d_poolk_supported(B, Ci, H, W, Co, k, k, d, d, pad, pad, pkH, pkW, pdH, pdW, ppH, ppW, ceil, G.F32)
            unpooled = G.conv2d_layout(hiplib, x, w, b, (d, d), (pad, pad), act=act, dtype=G.F32, scale=sc)
            ref = G.unary(hiplib, hiplib.thhip_maxpool, unpooled, (B, Co, pH, pW), G.F32, B, Co, oH, oW, pH, pW, pkH, pkW, pdH, pdW,
                          ppH, ppW, G.F32)
            dx = api.DeviceArray(hiplib, x)
            wp = hiplib.thhip_conv_pack_weight_layout(np.ascontiguousarray(w).ctypes.data, Co, Ci, k, k, G.F32, 0)
            db, ds = api.DeviceArray(hiplib, b), api.DeviceArray(hiplib, sc)
            dy = api.DeviceArray(hiplib, nbytes=B * Co * pH * pW * 4)
            hiplib.thhip_conv2d_poolk(dx.ptr, wp, ds.ptr, db.ptr, dy.ptr, B, Ci, H, W, Co, k, k, d, d, pad, pad,
                                      pkH, pkW, pdH, pdW, ppH, ppW, ceil, act, 0.0, 0.0, G.F32)
            hiplib.thhip_sync()
            got = dy.get((B, Co, pH, pW), np.float32)
            hiplib.thhip_free(wp)
            assert np.array_equal(got.view(np.uint32), ref.view(np.uint32)), ((B, Ci, H, W, Co, k), int((got != ref).sum()))
            want = oracle.maxpool(np.maximum(raw, 0) if act else raw, pkH, pkW, pdH, pdW, ppH, ppW, ceil)
            G.assert_close(got, want, FP32_TOL, str((B, Ci, H, W, Co, k, d, pad)))
    # a large layer: windows of up to four values only (four lanes per pooled value)
    assert hiplib.thhip_conv2d_poolk_supported(16, 512, 14, 14, 512, 3, 3, 1, 1, 1, 1, 2, 2, 2, 2, 0, 0, 0, G.F32)
    assert not hiplib.thhip_conv2d_poolk_supported(16, 512, 14, 14, 512, 3, 3, 1, 1, 1, 1, 3, 3, 2, 2, 0, 0, 0, G.F32)
    # layers of many tiles run without a K split, the half types have their own fused poolings
    assert not hiplib.thhip_conv2d_poolk_supported(16, 64, 112, 112, 64, 3, 3, 1, 1, 1, 1, 3, 3, 2, 2, 0, 0, 0, G.F32)
    assert not hiplib.thhip_conv2d_poolk_supported(1, 64, 27, 27, 192, 5, 5, 1, 1, 2, 2, 3, 3, 2, 2, 0, 0, 0, G.F16)
    assert not hiplib.thhip_conv2d_poolk_supported(1, 64, 27, 27, 192, 5, 5, 1, 1, 2, 2, 3, 3, 2, 2, 2, 2, 0, G.F32)   # padding over half the window


@pytest.mark.parametrize("dtype", [G.F16, G.BF16])
def test_conv_half_last_tiles_cut_along_k(hiplib, oracle, dtype):
    """Half-type tiles loaded straight into LDS (channels-last input): the tiles an XCD
    cannot spread evenly over its CUs are cut along K, as on the fp32 path, where at least
    one whole round of tiles precedes them.  518 tiles of 128x128 (64 or 65 per XCD, two
    resident per CU: one tile cut on some XCDs, none on others; 100 of 128 planes), 265
    tiles of 256x256 (33 per XCD, one per CU), a layer of few tiles (never cut); both
    output orders, the factor and the threshold, every limit on the parts (1 = never
    cut), same bits twice."""
    g = cases.rng(919)
    # last entry: the M tiles cut into that many groups over the XCDs (0: by weight size)
    shapes = [(8, 64, 91, 91, 100, 3, 1, 1, (128, 128, 9, 0), 0), (8, 128, 92, 92, 256, 3, 1, 1, (256, 256, 0, 0), 0),
              (3, 96, 27, 27, 100, 3, 2, 1, (64, 128, 9, 0), 0), (8, 64, 91, 91, 256, 3, 1, 1, (128, 128, 9, 0), 2)]
    try:
        for (B, Ci, H, W, Co, k, dd, pp, tune, mparts) in shapes:
            hiplib.thhip_conv_set_xcd_parts(mparts)
            x = g.uniform(-1, 1, (B, Ci, H, W)).astype(np.float32)
            w = g.standard_normal((Co, Ci, k, k), dtype=np.float32) * np.float32(np.sqrt(2.0 / (Ci * k * k)))
            b = g.standard_normal(Co, dtype=np.float32) * np.float32(0.1)
            sc = g.uniform(0.5, 1.5, Co).astype(np.float32)
            plain = oracle.conv2d(x, w, None, (dd, dd), (pp, pp))
            want = np.maximum(plain * sc[None, :, None, None] + b[None, :, None, None], 0)
            hiplib.thhip_conv_set_tuning(*tune)
            for y_cl in (1, 0):
                for parts in (1, 2, 8):
                    G.note("half last tiles cut along K %s parts %d y_cl %d" % ((B, Ci, H, W, Co, k, dd, pp, tune), parts, y_cl))
                    hiplib.thhip_conv_set_tail_parts(parts)
                    got = G.conv2d_layout(hiplib, x, w, b, (dd, dd), (pp, pp), act=1, dtype=dtype, x_cl=1, y_cl=y_cl, scale=sc)
                    G.assert_close(got, want, HALF_TOL, str((Ci, Co, k, parts, y_cl)))
                    again = G.conv2d_layout(hiplib, x, w, b, (dd, dd), (pp, pp), act=1, dtype=dtype, x_cl=1, y_cl=y_cl, scale=sc)
                    assert np.array_equal(got, again), "cut tiles: results depend on timing"
    finally:
        hiplib.thhip_conv_set_tail_parts(8)
        hiplib.thhip_conv_set_tuning(0, 0, 0, 0)
        hiplib.thhip_conv_set_xcd_parts(0)


@pytest.mark.parametrize("dtype", [G.F16, G.BF16])
@pytest.mark.parametrize("i", [0, 1, 3, 5, 10])
def test_conv_half_vs_fp32_oracle(hiplib, oracle, i, dtype):
    x, s = cases.conv_case(i)
    d, p = (s["dH"], s["dW"]), (s["padH"], s["padW"])
    y = G.conv2d(hiplib, x, s["weight"], s["bias"], d, p, dtype=dtype)
    G.assert_close(y, oracle.conv2d(x, s["weight"], s["bias"], d, p), HALF_TOL, "half conv")


def test_conv_f32_tile_shapes_and_invariants(hiplib, oracle):
    g = cases.rng(900)
    # shapes that select each tile configuration, with ragged M / N / K
    for (B, Ci, H, W, Co, k, d, p) in [(2, 16, 72, 72, 130, 3, 1, 1),    # 128x128 tiles, M tail
                                       (1, 24, 40, 40, 200, 3, 1, 1),    # 128x64
                                       (3, 9, 160, 160, 48, 3, 1, 1),    # 64x128
                                       (1, 5, 17, 17, 7, 3, 1, 1)]:      # 64x64
        x = g.uniform(-1, 1, (B, Ci, H, W)).astype(np.float32)
        w = g.standard_normal((Co, Ci, k, k), dtype=np.float32) * np.float32(0.1)
        b = g.standard_normal(Co, dtype=np.float32)
        y = G.conv2d(hiplib, x, w, b, (d, d), (p, p))
        G.assert_close(y, oracle.conv2d(x, w, b, (d, d), (p, p)), FP32_TOL, str((B, Ci, H, W, Co)))
        # batch == images one at a time (bit-exact: same tiles per column)
        y0 = G.conv2d(hiplib, x[:1], w, b, (d, d), (p, p))
        G.assert_close(y0[0], y[0], 1e-6)
    # delta kernel shifts the input exactly; zero weights give the bias planes exactly
    x = g.standard_normal((1, 2, 8, 9), dtype=np.float32)
    w = np.zeros((2, 2, 3, 3), np.float32)
    w[0, 0, 0, 2] = 1.0
    w[1, 1, 2, 1] = 1.0
    y = G.conv2d(hiplib, x, w, None, (1, 1), (1, 1))
    xp = np.pad(x, ((0, 0), (0, 0), (1, 1), (1, 1)))
    assert np.array_equal(y[0, 0], xp[0, 0, 0:8, 2:11]) and np.array_equal(y[0, 1], xp[0, 1, 2:10, 1:10])
    b = np.array([0.5, -2.0], np.float32)
    y = G.conv2d(hiplib, x, np.zeros_like(w), b, (1, 1), (1, 1))
    assert np.array_equal(y, np.broadcast_to(b[None, :, None, None], y.shape))
    # linearity in the weights: conv(w1 + w2) == conv(w1) + conv(w2) up to rounding
    w1 = g.standard_normal((9, 2, 3, 3), dtype=np.float32)
    w2 = g.standard_normal((9, 2, 3, 3), dtype=np.float32)
    s = G.conv2d(hiplib, x, w1 + w2, None, (1, 1), (1, 1))
    G.assert_close(s, G.conv2d(hiplib, x, w1, None, (1, 1), (1, 1)) + G.conv2d(hiplib, x, w2, None, (1, 1), (1, 1)), 1e-5)


def test_conv_split_k_and_forced_tiles(hiplib, oracle):
    # every tile shape and several split-K factors give the same answer as the oracle;
    # repeated launches reuse the scratch counters correctly
    try:
        for (bm, bn) in [(64, 64), (128, 64), (64, 128), (128, 128)]:
            for sk in (1, 2, 3, 7):
                hiplib.thhip_conv_set_tuning(bm, bn, sk, sk % 3)
                for i in (4, 5, 10):
                    x, s = cases.conv_case(i)
                    d, p = (s["dH"], s["dW"]), (s["padH"], s["padW"])
                    want = oracle.conv2d(x, s["weight"], s["bias"], d, p)
                    for rep in range(2):
                        y = G.conv2d(hiplib, x, s["weight"], s["bias"], d, p, act=1, thr=0.0, val=0.0)
                        G.assert_close(y, np.maximum(want, 0), FP32_TOL, "tile %dx%d splitk %d case %d" % (bm, bn, sk, i))
        hiplib.thhip_conv_set_tuning(64, 64, 4, 2)
        x, s = cases.conv_case(10)
        y = G.conv2d(hiplib, x, s["weight"], s["bias"], (1, 1), (1, 1), dtype=G.F16)
        G.assert_close(y, oracle.conv2d(x, s["weight"], s["bias"], (1, 1), (1, 1)), HALF_TOL)
    finally:
        hiplib.thhip_conv_set_tuning(0, 0, 0, 0)


def test_pack_unpack_roundtrip(hiplib):
    import ctypes as C
    from thnets_amd import api
    g = cases.rng(901)
    # plane counts that select the tap-major K order (multiples of 16) and the plain one
    for (Co, Ci, kHW) in [(5, 7, 1), (64, 3, 9), (130, 64, 9), (33, 1000, 1), (40, 32, 25), (200, 256, 36)]:
        w = g.standard_normal((Co, Ci * kHW), dtype=np.float32)
        wp = hiplib.thhip_conv_pack_weight(w.ctypes.data, Co, Ci, kHW, G.F32)
        rows = hiplib.thhip_conv_unpack_rows(wp, Co, Ci, kHW, G.F32)
        hiplib.thhip_sync()
        back = np.empty_like(w)
        hiplib.thhip_memcpy_d2h(back.ctypes.data, rows, back.nbytes)
        assert np.array_equal(back, w)
        hiplib.thhip_free(wp)
        hiplib.thhip_free(rows)


@pytest.mark.parametrize("i", range(len(cases.LINEAR_CASES)))
def test_gemv_vs_oracle_and_golden(hiplib, oracle, i):
    x, s = cases.linear_case(i)
    if x.ndim != 1:
        pytest.skip("matrix input goes through the convolution kernel (network tests)")
    y = G.gemv(hiplib, x, s["weight"], s["bias"])
    G.assert_close(y, oracle.linear(x, s["weight"], s["bias"]), FP32_TOL, "oracle")
    G.assert_close(y, GOLD["linear%d" % i], FP32_TOL, "golden")
    ya = G.gemv(hiplib, x, s["weight"], s["bias"], act=1, thr=0.0, val=0.0)
    assert np.array_equal(ya, np.maximum(y, 0))
    for dt in (G.F16, G.BF16):
        G.assert_close(G.gemv(hiplib, x, s["weight"], s["bias"], dtype=dt), y, HALF_TOL)


def test_gemv_ragged_sizes(hiplib, oracle):
    g = cases.rng(902)
    for (nOut, nIn) in [(1, 1), (3, 5), (1000, 4096), (4099, 1027), (9000, 64)]:
        x = g.standard_normal(nIn, dtype=np.float32)
        w = g.standard_normal((nOut, nIn), dtype=np.float32)
        b = g.standard_normal(nOut, dtype=np.float32)
        G.assert_close(G.gemv(hiplib, x, w, b), oracle.linear(x, w, b), FP32_TOL, str((nOut, nIn)))


def test_linear_batched_vs_oracle_and_golden(hiplib, oracle):
    from thnets_amd import api
    g = cases.rng(906)
    shapes = [(4, 128, 64), (16, 512, 100), (2, 64, 17), (16, 4096, 1000), (32, 1028, 515), (17, 200, 33), (7, 25088, 48),
              (16, 1024, 1100), (20, 516, 1030), (64, 1024, 260), (45, 516, 1030), (128, 256, 48)]   # the last: slices of 64 (of 32 with the row blocks forced)
    for (B, nIn, nOut) in shapes:
        assert hiplib.thhip_linear_batched_supported(B, nIn, nOut, G.F32)
        x = g.standard_normal((B, nIn), dtype=np.float32)
        w = g.standard_normal((nOut, nIn), dtype=np.float32) * np.float32(np.sqrt(2.0 / nIn))
        b = g.standard_normal(nOut, dtype=np.float32)
        G.note("linear_batched %s" % ((B, nIn, nOut),))
        dx, dw, db = api.DeviceArray(hiplib, x), api.DeviceArray(hiplib, w), api.DeviceArray(hiplib, b)
        dy = api.DeviceArray(hiplib, nbytes=B * nOut * 4)
        for rb in (0, 1, 4):        # chosen by width, one and four row blocks per wavefront
            hiplib.thhip_linear_batched_set_tuning(rb)
            hiplib.thhip_linear_batched(dx.ptr, dw.ptr, db.ptr, dy.ptr, B, nIn, nOut, 0, 0.0, 0.0, G.F32)
            hiplib.thhip_sync()
            y = dy.get((B, nOut), np.float32)
            G.assert_close(y, oracle.linear(x, w, b), FP32_TOL, str((B, nIn, nOut, rb)))
        hiplib.thhip_linear_batched_set_tuning(0)
        hiplib.thhip_linear_batched(dx.ptr, dw.ptr, None, dy.ptr, B, nIn, nOut, 1, 0.0, 0.0, G.F32)
        hiplib.thhip_sync()
        G.assert_close(dy.get((B, nOut), np.float32), np.maximum(oracle.linear(x, w, None), 0), FP32_TOL)
    assert not hiplib.thhip_linear_batched_supported(129, 128, 64, G.F32)
    assert not hiplib.thhip_linear_batched_supported(4, 130, 64, G.F32)
    assert hiplib.thhip_linear_batched_supported(4, 128, 64, G.F16)
    assert not hiplib.thhip_linear_batched_supported(4, 132, 64, G.F16)        # half rows come in 16-byte vectors
    for i in (2, 3):
        x, s = cases.linear_case(i)
        B, nIn = x.shape
        nOut = s["weight"].shape[0]
        dx, dw, db = api.DeviceArray(hiplib, x), api.DeviceArray(hiplib, s["weight"]), api.DeviceArray(hiplib, s["bias"])
        dy = api.DeviceArray(hiplib, nbytes=B * nOut * 4)
        if not hiplib.thhip_linear_batched_supported(B, nIn, nOut, G.F32):
            continue
        hiplib.thhip_linear_batched(dx.ptr, dw.ptr, db.ptr, dy.ptr, B, nIn, nOut, 0, 0.0, 0.0, G.F32)
        hiplib.thhip_sync()
        G.assert_close(dy.get((B, nOut), np.float32), GOLD["linear%d" % i], FP32_TOL)


@pytest.mark.parametrize("dt", [G.F16, G.BF16])
def test_conv_half_channels_last(hiplib, oracle, dt):
    """fp16 / bf16 convolution with channels-last tensors on either side, the folded
    batch-norm factor and the fused threshold: against the fp32 restatement on the
    rounded operands, and against the same kernel on plane-major tensors."""
    from thnets_amd import api
    g = cases.rng(908)
    shapes = [(2, 8, 9, 11, 36, 3, 3, 1, 1, 1, 1), (3, 64, 7, 7, 200, 5, 5, 2, 2, 2, 2), (1, 24, 13, 13, 68, 1, 1, 1, 1, 0, 0),
              (5, 16, 6, 6, 132, 6, 6, 1, 1, 0, 0), (2, 3, 21, 19, 64, 7, 7, 2, 2, 3, 3), (2, 128, 8, 8, 64, 3, 3, 1, 1, 1, 1)]
    for (B, Ci, H, W, Co, kH, kW, dH, dW, pH, pW) in shapes:
        x = g.uniform(-1, 1, (B, Ci, H, W)).astype(np.float32)
        w = g.standard_normal((Co, Ci, kH, kW), dtype=np.float32) * np.float32(np.sqrt(2.0 / (Ci * kH * kW)))
        b = g.standard_normal(Co, dtype=np.float32) * np.float32(0.1)
        sc = g.uniform(0.5, 1.5, Co).astype(np.float32)
        xr = api.from_device_dtype(api.to_device_dtype(hiplib, x, dt), x.shape, dt)
        wr = api.from_device_dtype(api.to_device_dtype(hiplib, w, dt), w.shape, dt)
        raw = oracle.conv2d(xr, wr, None, (dH, dW), (pH, pW))
        want = np.maximum(raw * sc[None, :, None, None] + b[None, :, None, None], 0)
        base = G.conv2d_layout(hiplib, x, w, b, (dH, dW), (pH, pW), act=1, dtype=dt, scale=sc)
        G.assert_close(base, want, HALF_TOL, "plane-major")
        orders = [(0, 1)] + ([(1, 0), (1, 1)] if Ci % 8 == 0 else [])
        try:
            for (x_cl, y_cl) in orders:
                # Ci a multiple of the K-tile: the scalar tap walk, then the per-thread decode
                for generic in ((0, 1) if x_cl == 1 and Ci % 32 == 0 else (0,)):
                    hiplib.thhip_conv_set_generic_cl(generic)
                    for tune in ((0, 0, 0, 0), (128, 128, 2, 0)):
                        hiplib.thhip_conv_set_tuning(*tune)
                        got = G.conv2d_layout(hiplib, x, w, b, (dH, dW), (pH, pW), act=1, dtype=dt, x_cl=x_cl, y_cl=y_cl, scale=sc)
                        G.assert_close(got, want, HALF_TOL, str((x_cl, y_cl, generic, tune)))
                        G.assert_close(got, base, 1e-2, "vs plane-major " + str((x_cl, y_cl, generic, tune)))
        finally:
            hiplib.thhip_conv_set_generic_cl(0)
            hiplib.thhip_conv_set_tuning(0, 0, 0, 0)


def test_conv_f32_with_table_add_in_the_epilogue(hiplib, oracle):
    """fp32 convolution -> (factor, bias) -> two-input table add -> Threshold(0, 0) in one kernel:
    bit for bit the convolution followed by thhip_axpby2 (the same sums in the same order, one
    rounding per operation), both operand orders, layers that split K (the finishing kernel adds),
    layers with tiles cut along K, 1x1 strided projections; and against the restatement with the
    reference's a - b."""
    from thnets_amd import api
    g = cases.rng(5300)
    shapes = [(4, 64, 56, 56, 64, 3, 3, 1, 1, 1, 1), (8, 32, 30, 30, 96, 3, 3, 1, 1, 1, 1), (4, 256, 14, 14, 256, 3, 3, 1, 1, 1, 1),
              (6, 64, 56, 56, 128, 1, 1, 2, 2, 0, 0), (2, 512, 7, 7, 512, 3, 3, 1, 1, 1, 1), (32, 128, 28, 28, 128, 3, 3, 1, 1, 1, 1)]
    for (B, Ci, H, W, Co, kH, kW, dH, dW, pH, pW) in shapes:
        x = g.uniform(-1, 1, (B, Ci, H, W)).astype(np.float32)
        w = g.standard_normal((Co, Ci, kH, kW), dtype=np.float32) * np.float32(np.sqrt(2.0 / (Ci * kH * kW)))
        b = g.standard_normal(Co, dtype=np.float32) * np.float32(0.1)
        sc = g.uniform(0.5, 1.5, Co).astype(np.float32)
        oH, oW = (H + 2 * pH - kH) // dH + 1, (W + 2 * pW - kW) // dW + 1
        r = g.standard_normal((B, Co, oH, oW), dtype=np.float32)
        args = (B, Ci, H, W, Co, kH, kW, dH, dW, pH, pW)
        assert hiplib.thhip_conv2d_residual_supported(*args, G.F32), args
        wp = hiplib.thhip_conv_pack_weight_layout(w.ctypes.data, Co, Ci, kH, kW, G.F32, 0)
        dx, db, ds, dr = (api.DeviceArray(hiplib, a) for a in (x, b, sc, r))
        n = B * Co * oH * oW
        dy, dz, dq = (api.DeviceArray(hiplib, nbytes=n * 4) for _ in range(3))
        raw = oracle.conv2d(x, w, None, (dH, dW), (pH, pW)) * sc[None, :, None, None] + b[None, :, None, None]
        for mode in (1, 2):
            for act in (0, 1):
                G.note("conv + table add fp32 %s mode %d act %d" % (args, mode, act))
                hiplib.thhip_conv2d_layout(dx.ptr, wp, ds.ptr, db.ptr, dy.ptr, *args, 0, 0.0, 0.0, G.F32, 0, 0)
                if mode == 1:
                    hiplib.thhip_axpby2(dy.ptr, dr.ptr, dz.ptr, n, n, -1.0, act, G.F32)
                else:
                    hiplib.thhip_axpby2(dr.ptr, dy.ptr, dz.ptr, n, n, -1.0, act, G.F32)
                hiplib.thhip_conv2d_residual(dx.ptr, wp, ds.ptr, db.ptr, dr.ptr, mode, -1.0, act, dq.ptr, *args, 0, 0.0, 0.0, G.F32)
                hiplib.thhip_sync()
                plain, fused = dz.get((B, Co, oH, oW), np.float32), dq.get((B, Co, oH, oW), np.float32)
                assert np.array_equal(plain, fused), (args, mode, act, np.abs(plain - fused).max())
                want = raw - r if mode == 1 else r - raw
                if act:
                    want = np.maximum(want, 0)
                G.assert_close(fused, want, FP32_TOL, "conv + table add " + str(args))
        hiplib.thhip_free(wp)
    assert not hiplib.thhip_conv2d_residual_supported(2, 3, 32, 32, 64, 3, 3, 1, 1, 1, 1, G.F32)
    assert not hiplib.thhip_conv2d_residual_supported(2, 64, 32, 32, 64, 3, 3, 1, 1, 1, 1, G.F16)


def test_conv_f32_rows_with_their_own_taps(hiplib, oracle):
    """fp32 plane-major layers whose planes are not whole blocks of 32 on the kernel that loads
    straight into LDS with a (plane, tap) of its own per K row: many tiles at stride 1 (7x7 on
    three planes, 5x5 on twenty), few tiles with strides and a K split (11x11 / stride 4 on
    three planes, 3x3 / stride 2 on 48), K values past the last plane in the last K-tile.
    Against the restatement and against the register-staged kernel (a forced tile)."""
    g = cases.rng(5500)
    shapes = [(40, 3, 64, 64, 64, 7, 1, 3), (8, 20, 40, 40, 64, 5, 1, 2), (2, 3, 227, 227, 64, 11, 4, 2), (2, 48, 30, 30, 96, 3, 2, 1),
              (3, 33, 17, 19, 70, 1, 1, 0), (1, 5, 9, 9, 64, 3, 1, 1)]
    for (B, Ci, H, W, Co, k, d, pad) in shapes:
        x = g.uniform(-1, 1, (B, Ci, H, W)).astype(np.float32)
        w = g.standard_normal((Co, Ci, k, k), dtype=np.float32) * np.float32(np.sqrt(2.0 / (Ci * k * k)))
        b = g.standard_normal(Co, dtype=np.float32) * np.float32(0.1)
        sc = g.uniform(0.5, 1.5, Co).astype(np.float32)
        raw = oracle.conv2d(x, w, None, (d, d), (pad, pad))
        for (scale, act) in ((None, 0), (sc, 1)):
            want = raw * (scale[None, :, None, None] if scale is not None else 1) + b[None, :, None, None]
            if act:
                want = np.where(want > 0.05, want, np.float32(0.05))      # (continuous: a sum next to the threshold moves the result little)
            kw = dict(act=act, thr=0.05, val=0.05, dtype=G.F32, scale=scale)
            G.note("fp32 rows kernel %s act %d" % ((B, Ci, H, W, Co, k, d, pad), act))
            got = G.conv2d_layout(hiplib, x, w, b, (d, d), (pad, pad), **kw)
            G.assert_close(got, want, FP32_TOL, "fp32 rows kernel " + str((B, Ci, H, W, Co, k, d, pad, act)))
            try:
                hiplib.thhip_conv_set_tuning(64, 64, 1, 0)
                staged = G.conv2d_layout(hiplib, x, w, b, (d, d), (pad, pad), **kw)
            finally:
                hiplib.thhip_conv_set_tuning(0, 0, 0, 0)
            G.assert_close(got, staged, FP32_TOL, "fp32 rows kernel against the register-staged one " + str((B, Ci, H, W, Co, k, d, pad)))


def test_conv_f32_taps_from_a_patch_in_lds(hiplib, oracle):
    """The fp32 kernel for 3x3 / stride 1 / padding 1 layers whose output is whole 16x4, 8x8 or 4x4
    patches (every tap read from one patch of the input in LDS): forced on small layers of all
    three patch shapes (a last tile of fewer than four 4x4 patches among them), two to six half
    blocks of input planes, 64 to 192 output planes, with and without the folded batch-norm factor
    and Threshold; and as the dispatcher picks it (more than 512 tiles; the last tiles of an XCD
    cut along K), alone, with the 2x2 pooling and with a table add in its epilogue, each bit for
    bit the separate kernel on the plain result.  Against the restatement."""
    from thnets_amd import api
    g = cases.rng(5400)
    small = [(2, 32, 16, 16, 64), (1, 64, 24, 24, 128), (3, 32, 8, 32, 64), (2, 96, 40, 24, 192), (1, 32, 4, 16, 64), (1, 32, 8, 8, 64),
             (2, 32, 12, 12, 64), (1, 64, 28, 28, 128), (3, 32, 4, 4, 64)]
    for (B, Ci, H, W, Co) in small:
        x = g.uniform(-1, 1, (B, Ci, H, W)).astype(np.float32)
        w = g.standard_normal((Co, Ci, 3, 3), dtype=np.float32) * np.float32(np.sqrt(2.0 / (Ci * 9)))
        b = g.standard_normal(Co, dtype=np.float32) * np.float32(0.1)
        sc = g.uniform(0.5, 1.5, Co).astype(np.float32)
        raw = oracle.conv2d(x, w, None, (1, 1), (1, 1))
        for (scale, act) in ((None, 0), (sc, 1)):
            want = raw * (scale[None, :, None, None] if scale is not None else 1) + b[None, :, None, None]
            if act:
                want = np.where(want > 0.05, want, np.float32(0.05))      # (continuous: a sum next to the threshold moves the result little)
            G.note("fp32 patch kernel, forced, %s act %d" % ((B, Ci, H, W, Co), act))
            try:
                hiplib.thhip_conv_set_tuning(64, 1, 0, 0)
                got = G.conv2d_layout(hiplib, x, w, b, (1, 1), (1, 1), act=act, thr=0.05, val=0.05, dtype=G.F32, scale=scale)
            finally:
                hiplib.thhip_conv_set_tuning(0, 0, 0, 0)
            G.assert_close(got, want, FP32_TOL, "fp32 patch kernel " + str((B, Ci, H, W, Co, act)))
    # seeded random shapes (all three patch shapes, last tiles of one to three 4x4 patches): against the kernel
    # that fetches every tap with a load of its own (another order of the sums) and against the restatement
    for it in range(16):
        B, Ci, Co = int(g.integers(1, 6)), int(g.choice([32, 64, 96, 160])), int(g.choice([64, 128, 192]))
        H, W = 4 * int(g.integers(1, 13)), 4 * int(g.integers(1, 13))
        x = g.standard_normal((B, Ci, H, W), dtype=np.float32)
        w = g.standard_normal((Co, Ci, 3, 3), dtype=np.float32) * np.float32(0.05)
        b = g.standard_normal(Co, dtype=np.float32)
        outs = []
        for tune in ((64, 1, 0, 0), (64, 64, 9, 2)):
            G.note("fp32 patch kernel, random shape %s tile %s" % ((B, Ci, H, W, Co), tune))
            try:
                hiplib.thhip_conv_set_tuning(*tune)
                outs.append(G.conv2d_layout(hiplib, x, w, b, (1, 1), (1, 1), act=1, thr=0.0, val=0.0, dtype=G.F32))
            finally:
                hiplib.thhip_conv_set_tuning(0, 0, 0, 0)
        G.assert_close(outs[0], outs[1], FP32_TOL, "fp32 patch kernel against the other " + str((B, Ci, H, W, Co)))
        want = np.maximum(oracle.conv2d(x, w, b, (1, 1), (1, 1)), np.float32(0))
        G.assert_close(outs[0], want, FP32_TOL, "fp32 patch kernel, random shape, against the restatement " + str((B, Ci, H, W, Co)))
    # as dispatched: 2048 tiles of 64 planes x 64 pixels
    for (B, Ci, H, W, Co) in ((32, 32, 64, 64, 64), (24, 64, 56, 56, 128), (44, 64, 28, 28, 256), (140, 32, 24, 40, 64)):
        x = g.uniform(-1, 1, (B, Ci, H, W)).astype(np.float32)
        w = g.standard_normal((Co, Ci, 3, 3), dtype=np.float32) * np.float32(np.sqrt(2.0 / (Ci * 9)))
        b = g.standard_normal(Co, dtype=np.float32) * np.float32(0.1)
        sc = g.uniform(0.5, 1.5, Co).astype(np.float32)
        r = g.standard_normal((B, Co, H, W), dtype=np.float32)
        args = (B, Ci, H, W, Co, 3, 3, 1, 1, 1, 1)
        assert hiplib.thhip_conv2d_pool2_supported(*args, G.F32, 0, 0) and hiplib.thhip_conv2d_residual_supported(*args, G.F32)
        wp = hiplib.thhip_conv_pack_weight_layout(w.ctypes.data, Co, Ci, 3, 3, G.F32, 0)
        dx, db, ds, dr = (api.DeviceArray(hiplib, a) for a in (x, b, sc, r))
        n = B * Co * H * W
        dy, dz, dq = (api.DeviceArray(hiplib, nbytes=n * 4) for _ in range(3))
        dp, dpq = (api.DeviceArray(hiplib, nbytes=n) for _ in range(2))
        G.note("fp32 patch kernel, dispatched, %s" % (args,))
        hiplib.thhip_conv2d_layout(dx.ptr, wp, ds.ptr, db.ptr, dy.ptr, *args, 1, 0.05, 0.05, G.F32, 0, 0)
        hiplib.thhip_maxpool(dy.ptr, dp.ptr, B, Co, H, W, H // 2, W // 2, 2, 2, 2, 2, 0, 0, G.F32)
        hiplib.thhip_conv2d_layout_pool2(dx.ptr, wp, ds.ptr, db.ptr, dpq.ptr, *args, 1, 0.05, 0.05, G.F32, 0, 0)
        hiplib.thhip_sync()
        got = dy.get((B, Co, H, W), np.float32)
        raw = oracle.conv2d(x, w, None, (1, 1), (1, 1)) * sc[None, :, None, None] + b[None, :, None, None]
        G.assert_close(got, np.where(raw > 0.05, raw, np.float32(0.05)), FP32_TOL, "fp32 patch kernel, dispatched " + str(args))
        plain, fused = dp.get((B, Co, H // 2, W // 2), np.float32), dpq.get((B, Co, H // 2, W // 2), np.float32)
        assert np.array_equal(plain, fused), (args, np.abs(plain - fused).max())
        assert np.array_equal(plain, got.reshape(B, Co, H // 2, 2, W // 2, 2).max(axis=(3, 5)))
        for mode in (1, 2):
            hiplib.thhip_conv2d_layout(dx.ptr, wp, ds.ptr, db.ptr, dy.ptr, *args, 0, 0.0, 0.0, G.F32, 0, 0)
            if mode == 1:
                hiplib.thhip_axpby2(dy.ptr, dr.ptr, dz.ptr, n, n, -1.0, 1, G.F32)
            else:
                hiplib.thhip_axpby2(dr.ptr, dy.ptr, dz.ptr, n, n, -1.0, 1, G.F32)
            hiplib.thhip_conv2d_residual(dx.ptr, wp, ds.ptr, db.ptr, dr.ptr, mode, -1.0, 1, dq.ptr, *args, 0, 0.0, 0.0, G.F32)
            hiplib.thhip_sync()
            plain, fused = dz.get((B, Co, H, W), np.float32), dq.get((B, Co, H, W), np.float32)
            assert np.array_equal(plain, fused), (args, mode, np.abs(plain - fused).max())
            G.assert_close(fused, np.maximum(raw - r if mode == 1 else r - raw, 0), FP32_TOL, "fp32 patch kernel + table add " + str(args))
        hiplib.thhip_free(wp)


def test_conv_f32_with_pooling_in_the_epilogue(hiplib, oracle):
    """fp32 convolution -> (factor, bias, Threshold) -> 2x2 / stride 2 max pooling in one
    kernel: against the pooling kernel on the plain convolution's output (the same comparisons;
    the sums differ in their last bits only where one of the two runs cut a tile along K, since
    the positions are tiled in another order) and against the restatement.
    Odd output sizes (the pooling drops the last row / column), strides, 64- and 128-plane
    tiles, tiles cut along K, both K-tile depths."""
    from thnets_amd import api
    g = cases.rng(5200)
    shapes = [(20, 32, 47, 45, 64, 3, 3, 1, 1, 1, 1), (12, 64, 64, 96, 128, 3, 3, 1, 1, 1, 1), (32, 32, 71, 70, 96, 5, 5, 2, 2, 2, 2),
              (32, 64, 36, 36, 64, 3, 3, 1, 1, 1, 1), (1, 32, 130, 129, 128, 1, 1, 1, 1, 0, 0), (16, 96, 30, 30, 192, 3, 3, 1, 1, 1, 1)]
    for (B, Ci, H, W, Co, kH, kW, dH, dW, pH, pW) in shapes:
        x = g.uniform(-1, 1, (B, Ci, H, W)).astype(np.float32)
        w = g.standard_normal((Co, Ci, kH, kW), dtype=np.float32) * np.float32(np.sqrt(2.0 / (Ci * kH * kW)))
        b = g.standard_normal(Co, dtype=np.float32) * np.float32(0.1)
        sc = g.uniform(0.5, 1.5, Co).astype(np.float32)
        oH, oW = (H + 2 * pH - kH) // dH + 1, (W + 2 * pW - kW) // dW + 1
        args = (B, Ci, H, W, Co, kH, kW, dH, dW, pH, pW, G.F32, 0, 0)
        assert hiplib.thhip_conv2d_pool2_supported(*args), args
        wp = hiplib.thhip_conv_pack_weight_layout(w.ctypes.data, Co, Ci, kH, kW, G.F32, 0)
        dx, db, ds = api.DeviceArray(hiplib, x), api.DeviceArray(hiplib, b), api.DeviceArray(hiplib, sc)
        dy = api.DeviceArray(hiplib, nbytes=B * Co * oH * oW * 4)
        dp = api.DeviceArray(hiplib, nbytes=B * Co * (oH // 2) * (oW // 2) * 4)
        dq = api.DeviceArray(hiplib, nbytes=B * Co * (oH // 2) * (oW // 2) * 4)
        for (scale, act) in ((None, 0), (ds, 1)):
            G.note("conv+pool fp32 %s act %d" % (args, act))
            sp = scale.ptr if scale else None
            hiplib.thhip_conv2d_layout(dx.ptr, wp, sp, db.ptr, dy.ptr, B, Ci, H, W, Co, kH, kW, dH, dW, pH, pW, act, 0.05, 0.05, G.F32, 0, 0)
            hiplib.thhip_maxpool(dy.ptr, dp.ptr, B, Co, oH, oW, oH // 2, oW // 2, 2, 2, 2, 2, 0, 0, G.F32)
            hiplib.thhip_conv2d_layout_pool2(dx.ptr, wp, sp, db.ptr, dq.ptr, B, Ci, H, W, Co, kH, kW, dH, dW, pH, pW, act, 0.05, 0.05,
                                             G.F32, 0, 0)
            hiplib.thhip_sync()
            plain = dp.get((B, Co, oH // 2, oW // 2), np.float32)
            fused = dq.get((B, Co, oH // 2, oW // 2), np.float32)
            G.assert_close(fused, plain, 4e-6, "conv+pool vs conv, pool " + str(args))
            raw = oracle.conv2d(x, w, None, (dH, dW), (pH, pW))
            want = raw * (sc[None, :, None, None] if scale else 1) + b[None, :, None, None]
            if act:
                want = np.where(want > 0.05, want, np.float32(0.05))      # (continuous: a sum next to the threshold moves the result little)
            want = want[:, :, :oH // 2 * 2, :oW // 2 * 2].reshape(B, Co, oH // 2, 2, oW // 2, 2).max(axis=(3, 5))
            G.assert_close(fused, want, FP32_TOL, "conv+pool " + str(args))
        hiplib.thhip_free(wp)
    # layers the K split takes, and forced tiles, are not pooled in the epilogue
    assert not hiplib.thhip_conv2d_pool2_supported(16, 512, 14, 14, 512, 3, 3, 1, 1, 1, 1, G.F32, 0, 0)
    assert not hiplib.thhip_conv2d_pool2_supported(16, 3, 224, 224, 64, 3, 3, 1, 1, 1, 1, G.F32, 0, 0)


@pytest.mark.parametrize("dt", [G.F32, G.F16, G.BF16])
def test_conv_image_layer_from_lds_patch(hiplib, oracle, dt):
    """The 3 -> 64 n planes, 3x3, stride 1, padding 1 image layer that runs from an input
    patch in LDS: ragged widths and heights (part tiles, part bands), one to four rows per
    workgroup (batch x height decides), 64 / 128 / 192 planes, with and without the folded
    batch-norm factor and Threshold, channels-last output for the half types; against the
    fp32 restatement on the rounded operands and against the generic kernel (a forced tile)."""
    from thnets_amd import api
    g = cases.rng(4100 + dt)
    tol = FP32_TOL if dt == G.F32 else HALF_TOL
    shapes = [(1, 7, 5, 64), (2, 33, 70, 64), (1, 224, 224, 64), (3, 40, 31, 128), (40, 13, 32, 64), (300, 3, 9, 64),
              (2, 1, 1, 192), (1, 600, 97, 64)]
    for (B, H, W, Co) in shapes:
        x = g.uniform(-1, 1, (B, 3, H, W)).astype(np.float32)
        w = g.standard_normal((Co, 3, 3, 3), dtype=np.float32) * np.float32(0.3)
        b = g.standard_normal(Co, dtype=np.float32) * np.float32(0.1)
        sc = g.uniform(0.5, 1.5, Co).astype(np.float32)
        xr = api.from_device_dtype(api.to_device_dtype(hiplib, x, dt), x.shape, dt)
        wr = api.from_device_dtype(api.to_device_dtype(hiplib, w, dt), w.shape, dt)
        raw = oracle.conv2d(xr, wr, None, (1, 1), (1, 1))
        for (scale, act) in ((None, 0), (sc, 1)):
            want = raw * (scale[None, :, None, None] if scale is not None else 1) + b[None, :, None, None]
            if act:
                want = np.where(want > 0.05, want, np.float32(-0.5))
            kw = dict(act=act, thr=0.05, val=-0.5, dtype=dt, scale=scale)
            got = G.conv2d_layout(hiplib, x, w, b, (1, 1), (1, 1), **kw)
            G.assert_close(got, want, tol, "stem " + str((B, H, W, Co, act)))
            try:
                hiplib.thhip_conv_set_tuning(64, 64, 1, 0)
                generic = G.conv2d_layout(hiplib, x, w, b, (1, 1), (1, 1), **kw)
            finally:
                hiplib.thhip_conv_set_tuning(0, 0, 0, 0)
            G.assert_close(got, generic, 2e-6 if dt == G.F32 else 1e-2, "stem vs generic " + str((B, H, W, Co, act)))
            if dt != G.F32:
                cl = G.conv2d_layout(hiplib, x, w, b, (1, 1), (1, 1), y_cl=1, **kw)
                assert np.array_equal(cl, got), "channels-last output " + str((B, H, W, Co, act))


@pytest.mark.parametrize("dt", [G.F16, G.BF16])
def test_conv_half_wide_tile(hiplib, oracle, dt):
    """The tiles whose operands go from global memory straight to LDS, every shape: K-tile
    counts around every edge of their pipelines (prologue of up to four tiles, steady state in
    rounds of three or four, drain), partial tiles along both axes, padding, strides, both
    output orders."""
    from thnets_amd import api
    g = cases.rng(911)
    shapes = [(2, 32, 12, 13, 300, 1, 1, 1, 1, 0, 0), (1, 64, 20, 17, 260, 1, 1, 1, 1, 0, 0), (1, 96, 9, 9, 40, 1, 1, 1, 1, 0, 0),
              (2, 32, 10, 10, 72, 2, 2, 1, 1, 1, 1), (1, 160, 8, 8, 64, 1, 1, 1, 1, 0, 0), (1, 224, 6, 7, 36, 1, 1, 1, 1, 0, 0),
              (1, 256, 5, 9, 132, 1, 1, 2, 1, 0, 0), (1, 32, 11, 11, 64, 3, 3, 1, 1, 1, 1), (1, 352, 7, 6, 68, 1, 1, 1, 1, 0, 0),
              (1, 384, 6, 6, 260, 1, 1, 1, 1, 0, 0), (3, 64, 7, 7, 200, 5, 5, 2, 2, 2, 2), (2, 64, 16, 16, 512, 3, 3, 1, 1, 1, 1),
              (1, 128, 9, 10, 72, 1, 1, 1, 1, 0, 0), (1, 192, 8, 8, 36, 1, 1, 1, 1, 0, 0), (2, 64, 9, 9, 40, 2, 2, 1, 1, 1, 0),
              (1, 320, 7, 5, 260, 1, 1, 1, 1, 0, 0)]
    try:
        for (B, Ci, H, W, Co, kH, kW, dH, dW, pH, pW) in shapes:
            x = g.uniform(-1, 1, (B, Ci, H, W)).astype(np.float32)
            w = g.standard_normal((Co, Ci, kH, kW), dtype=np.float32) * np.float32(np.sqrt(2.0 / (Ci * kH * kW)))
            b = g.standard_normal(Co, dtype=np.float32) * np.float32(0.1)
            sc = g.uniform(0.5, 1.5, Co).astype(np.float32)
            xr = api.from_device_dtype(api.to_device_dtype(hiplib, x, dt), x.shape, dt)
            wr = api.from_device_dtype(api.to_device_dtype(hiplib, w, dt), w.shape, dt)
            raw = oracle.conv2d(xr, wr, None, (dH, dW), (pH, pW))
            want = np.maximum(raw * sc[None, :, None, None] + b[None, :, None, None], 0)
            for y_cl in (1, 0):
                G.note("wide tile %s y_cl %d dtype %d" % ((B, Ci, H, W, Co, kH, kW, dH, dW, pH, pW), y_cl, dt))
                hiplib.thhip_conv_set_tuning(128, 128, 0, 0)
                narrow = G.conv2d_layout(hiplib, x, w, b, (dH, dW), (pH, pW), act=1, dtype=dt, x_cl=1, y_cl=y_cl, scale=sc)
                # 256 positions: eight and four waves, K-tiles of 32 in four LDS stages.  The smaller tiles
                # (third argument 9: the kernel that loads straight into LDS): four waves, four stages.
                # (fourth argument, 64 x 64 tiles: one K group, or two that share the tile and split its K-tiles)
                for tune in ((256, 256, 0, 0), (128, 256, 0, 0), (128, 128, 9, 0), (128, 64, 9, 0), (64, 128, 9, 0), (64, 64, 9, 1),
                             (64, 64, 9, 2)):
                    hiplib.thhip_conv_set_tuning(*tune)
                    got = G.conv2d_layout(hiplib, x, w, b, (dH, dW), (pH, pW), act=1, dtype=dt, x_cl=1, y_cl=y_cl, scale=sc)
                    G.assert_close(got, want, HALF_TOL, str((Ci, Co, kH, y_cl, tune)))
                    G.assert_close(got, narrow, 1e-2, "vs the register-staged 128x128 tile " + str((Ci, Co, kH, y_cl, tune)))
    finally:
        hiplib.thhip_conv_set_tuning(0, 0, 0, 0)


@pytest.mark.parametrize("dt", [G.F16, G.BF16])
def test_conv_half_patch_kernel(hiplib, oracle, dt):
    """3x3 stride-1 convolutions of 64 to 512 planes whose taps come from an input patch in LDS:
    images smaller and larger than the 8 x 32 tile, partial tiles on both axes, padding 0, 1
    and 2, plane counts that leave a partial 64-row tile, both output orders."""
    from thnets_amd import api
    g = cases.rng(912)
    shapes = [(2, 5, 7, 64, 1, 1, 64), (1, 8, 32, 128, 1, 1, 64), (3, 19, 45, 72, 1, 1, 64), (1, 40, 33, 200, 0, 0, 64),
              (2, 9, 70, 36, 2, 1, 64), (1, 16, 64, 260, 1, 0, 64), (1, 3, 3, 64, 0, 0, 64),
              (2, 11, 37, 72, 1, 1, 128), (1, 8, 32, 128, 0, 1, 128), (1, 21, 9, 40, 1, 1, 128),   # 128 planes: four blocks of 32
              (1, 13, 40, 72, 1, 1, 256), (2, 8, 33, 64, 1, 1, 512)]                                 # eight and sixteen blocks
    try:
        for (B, H, W, Co, pH, pW, Ci) in shapes:
            x = g.uniform(-1, 1, (B, Ci, H, W)).astype(np.float32)
            w = g.standard_normal((Co, Ci, 3, 3), dtype=np.float32) * np.float32(np.sqrt(2.0 / (Ci * 9)))
            b = g.standard_normal(Co, dtype=np.float32) * np.float32(0.1)
            sc = g.uniform(0.5, 1.5, Co).astype(np.float32)
            xr = api.from_device_dtype(api.to_device_dtype(hiplib, x, dt), x.shape, dt)
            wr = api.from_device_dtype(api.to_device_dtype(hiplib, w, dt), w.shape, dt)
            raw = oracle.conv2d(xr, wr, None, (1, 1), (pH, pW))
            want = np.maximum(raw * sc[None, :, None, None] + b[None, :, None, None], 0)
            for y_cl in (1, 0):
                G.note("patch kernel %s y_cl %d dtype %d" % ((B, Ci, H, W, Co, pH, pW), y_cl, dt))
                hiplib.thhip_conv_set_tuning(64, 64, 0, 0)
                narrow = G.conv2d_layout(hiplib, x, w, b, (1, 1), (pH, pW), act=1, dtype=dt, x_cl=1, y_cl=y_cl, scale=sc)
                hiplib.thhip_conv_set_tuning(64, 1, 0, 0)
                got = G.conv2d_layout(hiplib, x, w, b, (1, 1), (pH, pW), act=1, dtype=dt, x_cl=1, y_cl=y_cl, scale=sc)
                G.assert_close(got, want, HALF_TOL, str((B, H, W, Co, pH, pW, y_cl)))
                G.assert_close(got, narrow, 1e-2, "vs the 64x64 tile " + str((B, H, W, Co, pH, pW, y_cl)))
    finally:
        hiplib.thhip_conv_set_tuning(0, 0, 0, 0)


@pytest.mark.parametrize("dt", [G.F16, G.BF16])
def test_conv_half_patch_kernel_with_pooling(hiplib, oracle, dt):
    """Convolution, threshold and the 2x2 / stride 2 max pooling that follows in one kernel:
    the same values as the convolution entry point followed by the pooling (bit for bit on
    the kernel that keeps an input patch in LDS: the pooling compares the rounded outputs; on
    the tiles loaded straight into LDS up to the last bit of a sum, where one of the two runs
    cut a tile along K), and the oracle's within the half tolerance; odd output sizes (the
    last row / column is dropped), both output orders, the folded batch-norm factor with
    negative entries; 64 and 128 planes (patch kernel), and 256 x 256, 128 x 128 and 64 x 64
    tiles with one and two K groups, 1x1 and strided layers (tiles loaded straight into LDS)."""
    import ctypes as C
    from thnets_amd import api
    g = cases.rng(914)
    shapes = [(8, 64, 33, 47, 72, 3, 1, 1, True), (16, 128, 40, 64, 72, 3, 1, 1, True), (40, 64, 17, 19, 132, 3, 1, 0, True),
              (4, 64, 40, 64, 200, 3, 1, 1, True),
              (16, 256, 56, 56, 256, 3, 1, 1, False), (16, 512, 28, 28, 512, 3, 1, 1, False), (4, 512, 14, 14, 512, 3, 1, 1, False),
              (3, 32, 21, 23, 40, 1, 1, 0, False), (2, 96, 30, 31, 264, 5, 2, 2, False), (1, 64, 8, 8, 64, 3, 1, 1, False)]
    for (B, Ci, H, W, Co, k, d, pad, exact) in shapes:
        x = g.uniform(-1, 1, (B, Ci, H, W)).astype(np.float32)
        w = g.standard_normal((Co, Ci, k, k), dtype=np.float32) * np.float32(np.sqrt(2.0 / (Ci * k * k)))
        b = g.standard_normal(Co, dtype=np.float32) * np.float32(0.1)
        sc = (g.uniform(0.5, 1.5, Co) * g.choice([-1.0, 1.0], Co)).astype(np.float32)
        oH, oW = (H + 2 * pad - k) // d + 1, (W + 2 * pad - k) // d + 1
        pH, pW = oH // 2, oW // 2
        xr = api.from_device_dtype(api.to_device_dtype(hiplib, x, dt), x.shape, dt)
        wr = api.from_device_dtype(api.to_device_dtype(hiplib, w, dt), w.shape, dt)
        raw = oracle.conv2d(xr, wr, None, (d, d), (pad, pad))
        act = np.maximum(raw * sc[None, :, None, None] + b[None, :, None, None], 0)
        want = act[:, :, :2 * pH, :2 * pW].reshape(B, Co, pH, 2, pW, 2).max(axis=(3, 5))
        for y_cl in (1, 0):
            G.note("conv + pool %s y_cl %d dtype %d" % ((B, Ci, H, W, Co, k, d, pad), y_cl, dt))
            assert hiplib.thhip_conv2d_pool2_supported(B, Ci, H, W, Co, k, k, d, d, pad, pad, dt, 1, y_cl)
            # (the same output order: the channels-last epilogue rounds a*s + b to the half type once, the plane-major
            # one to fp32 first, which differs in the last bit of one value in 50 000)
            unpooled = G.conv2d_layout(hiplib, x, w, b, (d, d), (pad, pad), act=1, dtype=dt, x_cl=1, y_cl=y_cl if exact else 0, scale=sc)
            ref = unpooled[:, :, :2 * pH, :2 * pW].reshape(B, Co, pH, 2, pW, 2).max(axis=(3, 5))
            dx = api.to_device_dtype(hiplib, np.ascontiguousarray(x.transpose(0, 2, 3, 1)), dt)
            wp = hiplib.thhip_conv_pack_weight_layout(np.ascontiguousarray(w).ctypes.data, Co, Ci, k, k, dt, 1)
            db, ds = api.DeviceArray(hiplib, b), api.DeviceArray(hiplib, sc)
            dy = api.DeviceArray(hiplib, nbytes=B * Co * pH * pW * 2)
            hiplib.thhip_conv2d_layout_pool2(dx.ptr, wp, ds.ptr, db.ptr, dy.ptr, B, Ci, H, W, Co, k, k, d, d, pad, pad,
                                             1, 0.0, 0.0, dt, 1, y_cl)
            hiplib.thhip_sync()
            if y_cl:
                got = np.ascontiguousarray(api.from_device_dtype(dy, (B, pH, pW, Co), dt).transpose(0, 3, 1, 2))
            else:
                got = api.from_device_dtype(dy, (B, Co, pH, pW), dt)
            hiplib.thhip_free(wp)
            if exact:
                assert np.array_equal(got, ref), (B, Ci, H, W, Co, pad, y_cl, int((got != ref).sum()))
            else:
                G.assert_close(got, ref, 1e-2, "vs convolution, pooling " + str((B, Ci, H, W, Co, k, d, pad, y_cl)))
                assert (got != ref).mean() < 1e-3, (B, Ci, H, W, Co, k, d, pad, y_cl, float((got != ref).mean()))
            G.assert_close(got, want, HALF_TOL, str((B, Ci, H, W, Co, k, d, pad, y_cl)))
    # layers the fused kernels do not take
    assert not hiplib.thhip_conv2d_pool2_supported(8, 24, 33, 47, 72, 3, 3, 1, 1, 1, 1, dt, 1, 1)        # planes not in blocks of 32
    assert not hiplib.thhip_conv2d_pool2_supported(8, 64, 33, 47, 72, 3, 3, 1, 1, 1, 1, dt, 0, 1)        # plane-major input
    assert not hiplib.thhip_conv2d_pool2_supported(8, 64, 3, 47, 72, 3, 3, 1, 1, 0, 0, dt, 1, 1)         # one output row
    assert not hiplib.thhip_conv2d_pool2_supported(8, 64, 33, 47, 72, 3, 3, 1, 1, 1, 1, G.F32, 1, 1)


@pytest.mark.parametrize("dt", [G.F16, G.BF16])
def test_conv_half_whole_image_patch_kernel(hiplib, oracle, dt):
    """3x3 / stride 1 / padding 1 layers of 256 and 512 planes on outputs of at most 14 x 14, one whole
    image per workgroup (VGG-16's last three convolutions): 32 and 64 planes per workgroup (forced, and as
    the dispatcher picks them by the number of workgroups), 14 x 14, 13 x 13 and 12 x 14 images, a plane
    count that leaves a partial block, both output orders; alone against the oracle and the 64 x 64 tile,
    and with the 2x2 pooling in the epilogue bit for bit the pooled plain result (odd sizes drop the last
    row and column)."""
    from thnets_amd import api
    g = cases.rng(916)
    shapes = [(16, 512, 14, 14, 512), (4, 256, 13, 13, 1024), (8, 512, 12, 14, 544), (64, 256, 14, 14, 256), (6, 256, 14, 11, 736)]
    try:
        for (B, Ci, H, W, Co) in shapes:
            x = g.uniform(-1, 1, (B, Ci, H, W)).astype(np.float32)
            w = g.standard_normal((Co, Ci, 3, 3), dtype=np.float32) * np.float32(np.sqrt(2.0 / (Ci * 9)))
            b = g.standard_normal(Co, dtype=np.float32) * np.float32(0.1)
            sc = (g.uniform(0.5, 1.5, Co) * g.choice([-1.0, 1.0], Co)).astype(np.float32)
            xr = api.from_device_dtype(api.to_device_dtype(hiplib, x, dt), x.shape, dt)
            wr = api.from_device_dtype(api.to_device_dtype(hiplib, w, dt), w.shape, dt)
            raw = oracle.conv2d(xr, wr, None, (1, 1), (1, 1))
            want = np.maximum(raw * sc[None, :, None, None] + b[None, :, None, None], 0)
            pH, pW = H // 2, W // 2
            plain = {}
            for y_cl in (1, 0):
                hiplib.thhip_conv_set_tuning(64, 64, 0, 0)
                narrow = G.conv2d_layout(hiplib, x, w, b, (1, 1), (1, 1), act=1, dtype=dt, x_cl=1, y_cl=y_cl, scale=sc)
                for planes in (3, 4, 0):      # 32 planes, 64 planes, the dispatcher's choice
                    G.note("whole-image patch kernel %s y_cl %d dtype %d planes %d" % ((B, Ci, H, W, Co), y_cl, dt, planes))
                    hiplib.thhip_conv_set_tuning(64 if planes else 0, 1 if planes else 0, 0, planes)
                    got = G.conv2d_layout(hiplib, x, w, b, (1, 1), (1, 1), act=1, dtype=dt, x_cl=1, y_cl=y_cl, scale=sc)
                    G.assert_close(got, want, HALF_TOL, str((B, Ci, H, W, Co, y_cl, planes)))
                    G.assert_close(got, narrow, 1e-2, "vs the 64x64 tile " + str((B, Ci, H, W, Co, y_cl, planes)))
                    if planes == 3:
                        plain[y_cl] = got
                    else:
                        assert np.array_equal(got, plain[y_cl]), (B, Ci, H, W, Co, y_cl, planes)   # (the same sums in the same order)
            hiplib.thhip_conv_set_tuning(0, 0, 0, 0)
            for y_cl in (1, 0):
                ref = plain[y_cl][:, :, :2 * pH, :2 * pW].reshape(B, Co, pH, 2, pW, 2).max(axis=(3, 5))
                G.note("whole-image patch kernel with pooling %s y_cl %d dtype %d" % ((B, Ci, H, W, Co), y_cl, dt))
                assert hiplib.thhip_conv2d_pool2_supported(B, Ci, H, W, Co, 3, 3, 1, 1, 1, 1, dt, 1, y_cl)
                dx = api.to_device_dtype(hiplib, np.ascontiguousarray(x.transpose(0, 2, 3, 1)), dt)
                wp = hiplib.thhip_conv_pack_weight_layout(np.ascontiguousarray(w).ctypes.data, Co, Ci, 3, 3, dt, 1)
                db, ds = api.DeviceArray(hiplib, b), api.DeviceArray(hiplib, sc)
                dy = api.DeviceArray(hiplib, nbytes=B * Co * pH * pW * 2)
                hiplib.thhip_conv2d_layout_pool2(dx.ptr, wp, ds.ptr, db.ptr, dy.ptr, B, Ci, H, W, Co, 3, 3, 1, 1, 1, 1,
                                                 1, 0.0, 0.0, dt, 1, y_cl)
                hiplib.thhip_sync()
                if y_cl:
                    got = np.ascontiguousarray(api.from_device_dtype(dy, (B, pH, pW, Co), dt).transpose(0, 3, 1, 2))
                else:
                    got = api.from_device_dtype(dy, (B, Co, pH, pW), dt)
                hiplib.thhip_free(wp)
                assert np.array_equal(got, ref), (B, Ci, H, W, Co, y_cl, int((got != ref).sum()))
    finally:
        hiplib.thhip_conv_set_tuning(0, 0, 0, 0)


def test_conv_f32_two_layers_in_one_launch(hiplib, oracle):
    """thhip_conv_pair_begin / _end: the call right after _begin is held back and shares a launch with the
    next one where both run whole on the kernel that loads its tiles straight into LDS; bit for bit the two
    calls made one after the other.  The shapes of a residual block with a projection (1x1 / stride 2
    beside 3x3 / stride 2), a first call that cannot be held back (a K split), a second call on another
    kernel (the held launch then follows it), and nothing after the held call but _end."""
    from thnets_amd import api
    g = cases.rng(930)

    class Layer:
        def __init__(self, B, Ci, H, W, Co, k, d, pad, x=None):
            self.shape = (B, Ci, H, W, Co, k, d, pad)
            self.x = x if x is not None else api.DeviceArray(hiplib, g.uniform(-1, 1, (B, Ci, H, W)).astype(np.float32))
            w = g.standard_normal((Co, Ci, k, k), dtype=np.float32) * np.float32(np.sqrt(2.0 / (Ci * k * k)))
            self.w = w
            self.b = g.standard_normal(Co, dtype=np.float32) * np.float32(0.1)
            self.db = api.DeviceArray(hiplib, self.b)
            self.wp = hiplib.thhip_conv_pack_weight(np.ascontiguousarray(w).ctypes.data, Co, Ci, k * k, G.F32)
            self.o = ((H + 2 * pad - k) // d + 1, (W + 2 * pad - k) // d + 1)
            self.y = api.DeviceArray(hiplib, nbytes=B * Co * self.o[0] * self.o[1] * 4)

        def run(self):
            B, Ci, H, W, Co, k, d, pad = self.shape
            hiplib.thhip_conv2d(self.x.ptr, self.wp, self.db.ptr, self.y.ptr, B, Ci, H, W, Co, k, k, d, d, pad, pad, 1, 0.0, 0.0, G.F32)

        def read(self):
            hiplib.thhip_sync()
            out = api.from_device_dtype(self.y, (self.shape[0], self.shape[4]) + self.o, G.F32).copy()
            hiplib.thhip_memset(self.y.ptr, 0, self.y.nbytes)
            return out

    cases_ = []
    for (B, Ci, S, Co) in ((8, 64, 56, 128), (8, 128, 28, 256), (3, 32, 30, 64)):
        a = Layer(B, Ci, S, S, Co, 1, 2, 0)
        cases_.append((a, Layer(B, Ci, S, S, Co, 3, 2, 1, x=a.x), "projection beside the first convolution"))
    a = Layer(2, 256, 14, 14, 256, 3, 1, 1)                       # few tiles, long K: split, not held back
    cases_.append((a, Layer(2, 256, 14, 14, 64, 1, 1, 0, x=a.x), "a first call with a K split"))
    a = Layer(16, 64, 28, 28, 64, 1, 1, 0)
    cases_.append((a, Layer(16, 64, 56, 56, 64, 3, 1, 1), "a second call on the patch kernel"))
    for (first, second, what) in cases_:
        G.note("two layers in one launch: " + what + " " + str(first.shape) + " " + str(second.shape))
        first.run(); second.run()
        want = (first.read(), second.read())
        hiplib.thhip_conv_pair_begin()
        first.run(); second.run()
        hiplib.thhip_conv_pair_end()
        got = (first.read(), second.read())
        assert np.array_equal(got[0], want[0]) and np.array_equal(got[1], want[1]), what
        G.assert_close(got[0], np.maximum(oracle.conv2d(api.from_device_dtype(first.x, first.shape[:4], G.F32), first.w, first.b,
                                                        (first.shape[6],) * 2, (first.shape[7],) * 2), 0), FP32_TOL, what)
        hiplib.thhip_conv_pair_begin()
        first.run()
        hiplib.thhip_conv_pair_end()
        assert np.array_equal(first.read(), want[0]), what + ", alone"
        hiplib.thhip_free(first.wp); hiplib.thhip_free(second.wp)


def test_conv_f32_cut_tiles_added_in_the_kernel(hiplib, oracle):
    """THHipSumPartsInKernel: the tiles an XCD cuts along K, added by the workgroup whose part is ready last
    (the parts meet in the XCD's L2) against the same launch followed by the kernel that adds them: the same
    bits, on both fp32 kernels that cut tiles (3x3 / stride 1 from a patch in LDS; strided and 1x1 layers with
    tiles loaded straight into LDS), with the folded factor and Threshold, with a table add, with the 2x2
    pooling; every case three times in a row (the arrival counters are left at zero).  One case against the
    restatement.  The probe launch saw workgroup b on XCD (b + r) % 8 for every b."""
    from thnets_amd import api
    g = cases.rng(7700)
    assert hiplib.thhip_xcd_map() >> 31, "the workgroups of the probe launch were not handed to the XCDs in order"
    shapes = [(32, 64, 56, 56, 64, 3, 1, 1), (24, 64, 56, 56, 128, 3, 1, 1), (44, 64, 28, 28, 256, 3, 1, 1), (12, 128, 64, 32, 128, 3, 1, 1),
              (32, 64, 56, 56, 128, 3, 2, 1), (16, 64, 40, 40, 128, 5, 1, 2), (9, 64, 75, 77, 64, 3, 1, 1), (32, 128, 56, 56, 128, 3, 2, 1)]
    cut = [0, 0]        # launches with cut tiles: tiles loaded straight into LDS, taps from a patch
    try:
        for (B, Ci, H, W, Co, k, d, pad) in shapes:
            oH, oW = (H + 2 * pad - k) // d + 1, (W + 2 * pad - k) // d + 1
            x = g.uniform(-1, 1, (B, Ci, H, W)).astype(np.float32)
            w = g.standard_normal((Co, Ci, k, k), dtype=np.float32) * np.float32(np.sqrt(2.0 / (Ci * k * k)))
            b = g.standard_normal(Co, dtype=np.float32) * np.float32(0.1)
            sc = g.uniform(0.5, 1.5, Co).astype(np.float32)
            r = g.standard_normal((B, Co, oH, oW), dtype=np.float32)
            args = (B, Ci, H, W, Co, k, k, d, d, pad, pad)
            wp = hiplib.thhip_conv_pack_weight_layout(w.ctypes.data, Co, Ci, k, k, G.F32, 0)
            dx, db, ds, dr = (api.DeviceArray(hiplib, a) for a in (x, b, sc, r))
            n = B * Co * oH * oW
            dy = api.DeviceArray(hiplib, nbytes=n * 4)
            pool = oH % 2 == 0 and oW % 2 == 0 and hiplib.thhip_conv2d_pool2_supported(*args, G.F32, 0, 0)
            res = hiplib.thhip_conv2d_residual_supported(*args, G.F32)
            outs = {}
            for mode in (0, 1, 1, 1, 0):
                G.note("cut tiles, added in the kernel %d, %s" % (mode, args))
                hiplib.THHipSumPartsInKernel(mode)
                before = hiplib.thhip_conv_cut_launches(0), hiplib.thhip_conv_cut_launches(1)
                got = []
                hiplib.thhip_memset(dy.ptr, 0xFF, n * 4)
                hiplib.thhip_conv2d_layout(dx.ptr, wp, ds.ptr, db.ptr, dy.ptr, *args, 1, 0.05, 0.05, G.F32, 0, 0)
                hiplib.thhip_sync()
                got.append(dy.get((B, Co, oH, oW), np.float32))
                after = hiplib.thhip_conv_cut_launches(0), hiplib.thhip_conv_cut_launches(1)
                assert after[mode] == before[mode] and after[1 - mode] - before[1 - mode] in (0, 1), (args, mode, before, after)
                cut[(k, d) == (3, 1)] += after[1 - mode] - before[1 - mode]
                if res:
                    hiplib.thhip_memset(dy.ptr, 0xFF, n * 4)
                    hiplib.thhip_conv2d_residual(dx.ptr, wp, None, db.ptr, dr.ptr, 2, -1.0, 1, dy.ptr, *args, 0, 0.0, 0.0, G.F32)
                    hiplib.thhip_sync()
                    got.append(dy.get((B, Co, oH, oW), np.float32))
                if pool:
                    hiplib.thhip_memset(dy.ptr, 0xFF, n * 4)
                    hiplib.thhip_conv2d_layout_pool2(dx.ptr, wp, ds.ptr, db.ptr, dy.ptr, *args, 1, 0.05, 0.05, G.F32, 0, 0)
                    hiplib.thhip_sync()
                    got.append(dy.get((B, Co, oH // 2, oW // 2), np.float32))
                if mode in outs:
                    assert all(np.array_equal(a, c) for a, c in zip(got, outs[mode])), ("not the same twice", args, mode)
                outs[mode] = got
            assert len(outs[0]) == len(outs[1]) == 1 + int(bool(res)) + int(bool(pool))
            for a, c in zip(outs[0], outs[1]):
                assert np.array_equal(a, c), (args, np.abs(a - c).max())
            if (B, Ci, H) == (9, 64, 75):
                raw = oracle.conv2d(x, w, None, (d, d), (pad, pad)) * sc[None, :, None, None] + b[None, :, None, None]
                G.assert_close(outs[1][0], np.where(raw > 0.05, raw, np.float32(0.05)), FP32_TOL, "cut tiles added in the kernel " + str(args))
            hiplib.thhip_free(wp)
        assert cut[0] >= 10 and cut[1] >= 15, cut     # (five launches a shape)
    finally:
        hiplib.THHipSumPartsInKernel(1)


@pytest.mark.parametrize("dt", [G.F16, G.BF16])
def test_conv_half_image_layer_in_front(hiplib, oracle, dt):
    """The network's image layer (3 -> 64 planes, 3x3 / stride 1 / padding 1, factor, shift, Threshold) computed
    inside the 3x3 layer of 64 input planes that follows it, with and without that layer's 2x2 pooling: against
    the oracle run on the values the device holds (the first layer's output rounded to the half type, as the
    separate kernel stores it), and against the two layers run one after the other on the device; images
    smaller than a tile, partial tiles on both axes, several tiles per workgroup, a Threshold other than ReLU
    after the first layer, plane counts of the second layer with a partial block."""
    from thnets_amd import api
    g = cases.rng(918)
    shapes = [(2, 8, 32, 64, 1), (3, 19, 46, 72, 1), (1, 5, 6, 64, 0), (40, 16, 64, 128, 1), (2, 37, 70, 136, 0), (1, 224, 224, 64, 1)]
    for (B, H, W, Co, relu1) in shapes:
        x = g.uniform(-1, 1, (B, 3, H, W)).astype(np.float32)
        w1 = g.standard_normal((64, 3, 3, 3), dtype=np.float32) * np.float32(0.3)
        b1 = g.standard_normal(64, dtype=np.float32) * np.float32(0.1)
        s1 = (g.uniform(0.5, 1.5, 64) * g.choice([-1.0, 1.0], 64)).astype(np.float32)
        w2 = g.standard_normal((Co, 64, 3, 3), dtype=np.float32) * np.float32(np.sqrt(2.0 / (64 * 9)))
        b2 = g.standard_normal(Co, dtype=np.float32) * np.float32(0.1)
        s2 = g.uniform(0.5, 1.5, Co).astype(np.float32)
        thr1, val1 = (0.0, 0.0) if relu1 else (0.05, -0.02)
        rd = lambda a: api.from_device_dtype(api.to_device_dtype(hiplib, a, dt), a.shape, dt)
        raw1 = oracle.conv2d(rd(x), rd(w1), None, (1, 1), (1, 1)) * s1[None, :, None, None] + b1[None, :, None, None]
        mid = rd(np.where(raw1 > thr1, raw1, np.float32(val1)).astype(np.float32))
        raw2 = oracle.conv2d(mid, rd(w2), None, (1, 1), (1, 1)) * s2[None, :, None, None] + b2[None, :, None, None]
        want = np.maximum(raw2, 0)
        # the two layers one after the other on the device
        first = G.conv2d_layout(hiplib, x, w1, b1, (1, 1), (1, 1), act=1, thr=thr1, val=val1, dtype=dt, x_cl=0, y_cl=1, scale=s1)
        G.assert_close(first, mid, HALF_TOL, "image layer alone " + str((B, H, W)))
        second = G.conv2d_layout(hiplib, first, w2, b2, (1, 1), (1, 1), act=1, dtype=dt, x_cl=1, y_cl=1, scale=s2)
        assert hiplib.thhip_conv2d_image_pair_supported(B, H, W, 64, Co, dt, 1)
        dx = api.to_device_dtype(hiplib, x, dt)
        wf = hiplib.thhip_conv_pack_weight_image_front(np.ascontiguousarray(w1).ctypes.data, dt)
        wp = hiplib.thhip_conv_pack_weight_layout(np.ascontiguousarray(w2).ctypes.data, Co, 64, 3, 3, dt, 1)
        d1b, d1s, d2b, d2s = (api.DeviceArray(hiplib, a) for a in (b1, s1, b2, s2))
        for pool in (0, 1):
            if pool and (H < 2 or W < 2):
                continue
            G.note("image layer in front %s pool %d dtype %d" % ((B, H, W, Co, relu1), pool, dt))
            oH, oW = (H // 2, W // 2) if pool else (H, W)
            dy = api.DeviceArray(hiplib, nbytes=B * Co * oH * oW * 2)
            hiplib.thhip_conv2d_image_pair(dx.ptr, wf, d1s.ptr, d1b.ptr, 1, thr1, val1, wp, d2s.ptr, d2b.ptr, dy.ptr,
                                           B, H, W, Co, 1, 0.0, 0.0, pool, dt)
            hiplib.thhip_sync()
            got = np.ascontiguousarray(api.from_device_dtype(dy, (B, oH, oW, Co), dt).transpose(0, 3, 1, 2))
            pooled = lambda a: a[:, :, :2 * oH, :2 * oW].reshape(B, Co, oH, 2, oW, 2).max(axis=(3, 5)) if pool else a
            G.assert_close(got, pooled(want), HALF_TOL, str((B, H, W, Co, pool)))
            G.assert_close(got, pooled(second), 1e-2, "vs the two layers one after the other " + str((B, H, W, Co, pool)))
        hiplib.thhip_free(wf)
        hiplib.thhip_free(wp)
    assert not hiplib.thhip_conv2d_image_pair_supported(2, 8, 31, 64, 64, dt, 1)      # odd width
    assert not hiplib.thhip_conv2d_image_pair_supported(2, 8, 32, 32, 64, dt, 1)      # the image layer makes 64 planes
    assert not hiplib.thhip_conv2d_image_pair_supported(2, 8, 32, 64, 512, dt, 1)
    assert not hiplib.thhip_conv2d_image_pair_supported(2, 8, 32, 64, 64, G.F32, 1)


@pytest.mark.parametrize("dt", [G.F16, G.BF16])
def test_maxpool_and_relayout_half_channels_last(hiplib, oracle, dt):
    from thnets_amd import api
    g = cases.rng(909)
    for (B, Cn, H, W, kH, kW, dH, dW, pH, pW, ceil) in ((2, 8, 13, 13, 3, 3, 2, 2, 0, 0, 0), (3, 64, 14, 14, 2, 2, 2, 2, 0, 0, 0),
                                                       (1, 16, 7, 9, 2, 2, 2, 2, 1, 1, 1), (2, 24, 10, 8, 2, 3, 1, 2, 0, 1, 0)):
        x = g.standard_normal((B, Cn, H, W), dtype=np.float32)
        dx = api.to_device_dtype(hiplib, x, dt)
        xr = api.from_device_dtype(dx, x.shape, dt)
        dcl = api.DeviceArray(hiplib, nbytes=x.size * 2)
        hiplib.thhip_relayout(dx.ptr, dcl.ptr, B, Cn, H * W, 1, dt)
        hiplib.thhip_sync()
        assert np.array_equal(api.from_device_dtype(dcl, (B, H, W, Cn), dt), xr.transpose(0, 2, 3, 1))
        dback = api.DeviceArray(hiplib, nbytes=x.size * 2)
        hiplib.thhip_relayout(dcl.ptr, dback.ptr, B, Cn, H * W, 0, dt)
        hiplib.thhip_sync()
        assert np.array_equal(api.from_device_dtype(dback, x.shape, dt), xr)
        spec = {"type": "maxpool", "kW": kW, "kH": kH, "dW": dW, "dH": dH, "padW": pW, "padH": pH, "ceil_mode": ceil}
        want = oracle.run_layers([spec], xr)
        oH, oW = want.shape[2:]
        dy = api.DeviceArray(hiplib, nbytes=want.size * 2)
        hiplib.thhip_maxpool_cl(dcl.ptr, dy.ptr, B, Cn, H, W, oH, oW, kH, kW, dH, dW, pH, pW, dt)
        hiplib.thhip_sync()
        assert np.array_equal(api.from_device_dtype(dy, (B, oH, oW, Cn), dt).transpose(0, 3, 1, 2), want)


@pytest.mark.parametrize("dt", [G.F16, G.BF16])
def test_linear_batched_half_types(hiplib, oracle, dt):
    """fp16 / bf16 storage and MFMA, fp32 accumulation: against the fp32 restatement on
    the rounded operands at the half tolerance (2e-2 of the largest reference value)."""
    from thnets_amd import api
    g = cases.rng(907)
    for (B, nIn, nOut) in [(4, 128, 64), (16, 4096, 1000), (32, 1032, 515), (17, 200, 33), (3, 25088, 40), (70, 1032, 260)]:
        x = g.standard_normal((B, nIn), dtype=np.float32)
        w = g.standard_normal((nOut, nIn), dtype=np.float32) * np.float32(np.sqrt(2.0 / nIn))
        b = g.standard_normal(nOut, dtype=np.float32)
        G.note("linear_batched half dt%d %s" % (dt, (B, nIn, nOut)))
        dx, dw = api.to_device_dtype(hiplib, x, dt), api.to_device_dtype(hiplib, w, dt)
        db = api.DeviceArray(hiplib, b)
        dy = api.DeviceArray(hiplib, nbytes=B * nOut * 2)
        xr = api.from_device_dtype(dx, x.shape, dt)
        wr = api.from_device_dtype(dw, w.shape, dt)
        want = np.maximum(oracle.linear(xr, wr, b), 0)
        for rb in (1, 4):
            hiplib.thhip_linear_batched_set_tuning(rb)
            hiplib.thhip_linear_batched(dx.ptr, dw.ptr, db.ptr, dy.ptr, B, nIn, nOut, 1, 0.0, 0.0, dt)
            hiplib.thhip_sync()
            G.assert_close(api.from_device_dtype(dy, (B, nOut), dt), want, HALF_TOL, str((B, nIn, nOut, rb)))
        hiplib.thhip_linear_batched_set_tuning(0)


def test_threshold_bit_exact(hiplib, oracle):
    x = cases.rng(700).standard_normal((2, 3, 4, 5), dtype=np.float32)
    x.ravel()[:3] = (0.0, -0.0, 0.25)
    for j, (thr, val, alpha, inplace) in enumerate([(0, 0, 0, 1), (0.25, -1.5, 0, 0), (0.25, -1.5, 0, 1), (0, 0, 0.1, 0)]):
        y = G.unary(hiplib, hiplib.thhip_threshold, x, x.shape, G.F32, x.size, thr, val, alpha, inplace, G.F32)
        assert np.array_equal(y, oracle.threshold(x, thr, val, alpha, inplace)), j
    xg = cases.rng(700).standard_normal((2, 3, 4, 5), dtype=np.float32)
    assert np.array_equal(G.unary(hiplib, hiplib.thhip_threshold, xg, xg.shape, G.F32, xg.size, 0, 0, 0, 1, G.F32),
                          GOLD["threshold0"])


def test_maxpool_f32_vector_paths_bit_exact(hiplib, oracle):
    """The fp32 pooling kernels that make several outputs per thread (2x2 / stride 2, and
    3x3 / stride 2 / padding 1 on planes whose width is a multiple of eight), against the
    oracle bit for bit: odd and even heights, signed zeros (the first maximum wins), the
    most negative float, windows that reach outside the plane."""
    g = cases.rng(930)
    for (B, Cn, H, W, k, d, pad) in [(2, 3, 16, 16, 3, 2, 1), (1, 5, 15, 24, 3, 2, 1), (2, 2, 8, 8, 3, 2, 1), (1, 2, 7, 40, 3, 2, 1),
                                     (2, 3, 12, 16, 2, 2, 0), (1, 1, 2, 8, 3, 2, 1)]:
        x = g.standard_normal((B, Cn, H, W), dtype=np.float32)
        flat = x.ravel()
        flat[g.integers(0, flat.size, flat.size // 5)] = 0.0
        flat[g.integers(0, flat.size, flat.size // 5)] = -0.0
        flat[g.integers(0, flat.size, flat.size // 7)] = -np.finfo(np.float32).max
        x[:, :, 0, :] = -np.abs(x[:, :, 0, :])      # a border row whose maxima are zeros of either sign
        want = oracle.maxpool(x, k, k, d, d, pad, pad, 0)
        oH, oW = want.shape[2:]
        G.note("maxpool fp32 vector path %s" % ((B, Cn, H, W, k, d, pad),))
        y = G.unary(hiplib, hiplib.thhip_maxpool, x, (B, Cn, oH, oW), G.F32, B, Cn, H, W, oH, oW, k, k, d, d, pad, pad, G.F32)
        assert np.array_equal(y.view(np.uint32), want.view(np.uint32)), (B, Cn, H, W, k, d, pad)


@pytest.mark.parametrize("i", range(len(cases.POOL_CASES)))
def test_pooling_bit_exact(hiplib, oracle, i):
    x = cases.pool_case(i)
    B, Cn, H, W, kH, kW, dH, dW, pH, pW, ceil = cases.POOL_CASES[i]
    oH, oW = oracle.pool_outsize(H, W, kH, kW, dH, dW, pH, pW, ceil)
    y = G.unary(hiplib, hiplib.thhip_maxpool, x, (B, Cn, oH, oW), G.F32, B, Cn, H, W, oH, oW, kH, kW, dH, dW, pH, pW, G.F32)
    assert np.array_equal(y, GOLD["maxpool%d" % i])
    cip = i % 2
    y = G.unary(hiplib, hiplib.thhip_avgpool, x, (B, Cn, oH, oW), G.F32, B, Cn, H, W, oH, oW, kH, kW, dH, dW, pH, pW, cip,
                G.F32)
    G.assert_close(y, GOLD["avgpool%d" % i], 1e-6)
    q = cases.rng(20 + i).integers(0, 256, (B, Cn, H, W), dtype=np.uint8)
    yq = G.unary(hiplib, hiplib.thhip_maxpool, q, (B, Cn, oH, oW), G.U8, B, Cn, H, W, oH, oW, kH, kW, dH, dW, pH, pW, G.U8)
    assert np.array_equal(yq, oracle.lowp_maxpool(q, kH, kW, dH, dW, pH, pW, ceil))


def test_avgpool_whole_plane(hiplib, oracle):
    """A window that is the whole plane (the pooling before a classifier) has a kernel of its own,
    sixteen lanes per plane: against the restatement, plane sizes below, at and above sixteen."""
    g = cases.rng(230)
    for (B, Cn, H, W) in ((3, 70, 7, 7), (2, 33, 5, 4), (1, 5, 13, 13), (2, 9, 4, 4), (2, 3, 3, 3)):
        x = g.standard_normal((B, Cn, H, W), dtype=np.float32)
        G.note("avgpool whole plane %s" % ((B, Cn, H, W),))
        for cip in (0, 1):
            y = G.unary(hiplib, hiplib.thhip_avgpool, x, (B, Cn, 1, 1), G.F32, B, Cn, H, W, 1, 1, H, W, 1, 1, 0, 0, cip, G.F32)
            G.assert_close(y, oracle.avgpool(x, H, W, 1, 1, 0, 0, 0, cip), 1e-6, str((B, Cn, H, W)))


def _softmax_dims(sh):
    if len(sh) == 1:
        return 1, sh[0], 1
    if len(sh) == 2:
        return sh[0], sh[1], 1
    if len(sh) == 3:
        return 1, sh[0], sh[1] * sh[2]
    return sh[0], sh[1], sh[2] * sh[3]


@pytest.mark.parametrize("i", range(len(cases.SOFTMAX_SHAPES)))
def test_softmax(hiplib, oracle, i):
    x = cases.softmax_case(i)
    sh = x.shape
    nframe, dim, stride = _softmax_dims(sh)
    y = G.unary(hiplib, hiplib.thhip_softmax, x, sh, G.F32, nframe, dim, stride, G.F32)
    G.assert_close(y, GOLD["softmax%d" % i], 1e-5)


def test_softmax_long_vectors(hiplib, oracle):
    """A few long vectors take a workgroup of sixteen wavefronts each: lengths below and above what the
    threads keep in registers (four values each), a strided one, against the restatement."""
    g = cases.rng(440)
    for sh in ((1, 1000), (2, 4096), (3, 5000), (2, 600, 3, 2), (1, 513)):
        x = (g.standard_normal(sh, dtype=np.float32) * np.float32(4.0)).astype(np.float32)
        nframe, dim, stride = _softmax_dims(sh)
        G.note("softmax %s" % (sh,))
        y = G.unary(hiplib, hiplib.thhip_softmax, x, sh, G.F32, nframe, dim, stride, G.F32)
        G.assert_close(y, oracle.softmax(x), 1e-5, str(sh))
        assert np.allclose(y.sum(axis=1), 1.0, atol=1e-4)


def test_batchnorm_and_table_add(hiplib, oracle):
    from thnets_amd import api
    x, s = cases.bn_case()
    inv = (1 / np.sqrt(s["running_var"].astype(np.float64) + s["eps"])).astype(np.float32)
    d = [api.DeviceArray(hiplib, np.ascontiguousarray(v, np.float32)) for v in (s["running_mean"], inv, s["weight"], s["bias"])]
    B, Cn = x.shape[:2]
    y = G.unary(hiplib, hiplib.thhip_batchnorm, x, x.shape, G.F32, B, Cn, x.size // (B * Cn), d[0].ptr, d[1].ptr, d[2].ptr,
                d[3].ptr, G.F32)
    G.assert_close(y, GOLD["bn0"], 1e-6)
    a = cases.rng(903).standard_normal(1000, dtype=np.float32)
    b = cases.rng(904).standard_normal(700, dtype=np.float32)
    da, db = api.DeviceArray(hiplib, a), api.DeviceArray(hiplib, b)
    dy = api.DeviceArray(hiplib, nbytes=a.nbytes)
    hiplib.thhip_axpby2(da.ptr, db.ptr, dy.ptr, a.size, b.size, -1.0, 0, G.F32)
    hiplib.thhip_sync()
    assert np.array_equal(dy.get(a.shape, np.float32), oracle.caddtable([a, b]))
    hiplib.thhip_axpby2(da.ptr, db.ptr, dy.ptr, a.size, b.size, 1.0, 1, G.F32)
    hiplib.thhip_sync()
    assert np.array_equal(dy.get(a.shape, np.float32), np.maximum(oracle.caddtable([a, b], is_csubtable=True), 0))


def test_rgb2float_bit_exact(hiplib, oracle):
    from thnets_amd import api
    g = cases.rng(905)
    img = g.integers(0, 256, (37, 53, 3), dtype=np.uint8)
    mean = np.array([0.485, 0.456, 0.406], np.float32)
    std = np.array([0.229, 0.224, 0.225], np.float32)
    dsrc = api.DeviceArray(hiplib, img)
    for bgr in (0, 1):
        dy = api.DeviceArray(hiplib, nbytes=3 * 37 * 53 * 4)
        hiplib.thhip_rgb2float(dy.ptr, dsrc.ptr, 53, 37, 53 * 3, 3, mean.ctypes.data, std.ctypes.data, bgr, G.F32)
        hiplib.thhip_sync()
        assert np.array_equal(dy.get((3, 37, 53), np.float32), oracle.rgb2float(img, mean, std, bgr))


def test_events_and_profile_counters(hiplib):
    import ctypes as C
    hiplib.thhip_profile_reset()
    hiplib.thhip_profile_enable(1)
    hiplib.thhip_event_record(0)
    x, s = cases.conv_case(0)
    G.conv2d(hiplib, x, s["weight"], s["bias"], (1, 1), (1, 1))
    hiplib.thhip_event_record(1)
    assert hiplib.thhip_event_ms(0, 1) > 0
    ms, n, work = C.c_double(), C.c_long(), C.c_double()
    hiplib.thhip_profile_get(0, C.byref(ms), C.byref(n), C.byref(work))
    hiplib.thhip_profile_enable(0)
    assert n.value == 1 and ms.value > 0
    B, Ci, H, W, Co, kH, kW = 1, 3, 19, 23, 5, 3, 3
    assert work.value == 2.0 * Co * Ci * kH * kW * (B * 19 * 23)


@pytest.mark.gpu
@pytest.mark.parametrize("dt,tol", [(G.F32, FP32_TOL), (G.F16, HALF_TOL), (G.BF16, HALF_TOL)])
@pytest.mark.parametrize("i", range(len(cases.FULLCONV_CASES)))
def test_fullconv_vs_oracle(hiplib, oracle, i, dt, tol):
    """thhip_fullconv2d (MFMA product + gather col2im) against the restatement of
    nn_SpatialFullConvolution_updateOutput, with the reference's bias factor (11), the
    textbook one (1) and a fused threshold."""
    from thnets_amd import api
    x, spec = cases.fullconv_case(i)
    w, b = spec["weight"], spec["bias"]
    Ci, Co, kH, kW = w.shape
    B, _, H, W = x.shape
    d, pad, adj = (spec["dH"], spec["dW"]), (spec["padH"], spec["padW"]), (spec["adjH"], spec["adjW"])
    xr = api.from_device_dtype(api.to_device_dtype(hiplib, x, dt), x.shape, dt)
    wr = api.from_device_dtype(api.to_device_dtype(hiplib, w, dt), w.shape, dt)
    want11 = oracle.fullconv2d(xr, wr, b, d, pad, adj)
    plain = oracle.fullconv2d(xr, wr, None, d, pad, adj)
    G.note("fullconv case %d dtype %d" % (i, dt))
    wp = hiplib.thhip_fullconv_pack_weight(np.ascontiguousarray(w).ctypes.data, Ci, Co, kH, kW, dt)
    dx = api.to_device_dtype(hiplib, x, dt)
    db = api.DeviceArray(hiplib, b) if b is not None else None
    es = 4 if dt == G.F32 else 2
    col = api.DeviceArray(hiplib, nbytes=B * Co * kH * kW * H * W * es)
    dy = api.DeviceArray(hiplib, nbytes=want11.size * es)
    for beta, act, want in ((11.0, 0, want11), (1.0, 0, plain + (b[None, :, None, None] if b is not None else 0)),
                            (11.0, 1, np.where(want11 > 0.1, want11, -2.0))):
        hiplib.thhip_fullconv2d(dx.ptr, wp, db.ptr if db else None, beta, col.ptr, dy.ptr, B, Ci, H, W, Co, kH, kW,
                                d[0], d[1], pad[0], pad[1], adj[0], adj[1], act, 0.1, -2.0, dt)
        hiplib.thhip_sync()
        got = api.from_device_dtype(dy, want11.shape, dt)
        if act and dt != G.F32:
            # values next to the threshold may fall on either side after rounding
            near = np.abs(want11 - 0.1) < tol * np.abs(want11).max()
            got, want = np.where(near, 0, got), np.where(near, 0, want)
        G.assert_close(got, want, tol, "beta %g act %d" % (beta, act))
    hiplib.thhip_free(wp)


@pytest.mark.gpu
@pytest.mark.parametrize("dt", [G.F32, G.F16, G.BF16])
def test_maxpool_indices_and_unpool_vs_oracle(hiplib, oracle, dt):
    """Pooling with indices and the gather form of SpatialMaxUnpooling: bit-exact,
    including overlapping windows, where the last window in row-major order wins."""
    from thnets_amd import api
    g = cases.rng(870)
    for (B, Cn, H, W, k, d, pad, ceil) in ((2, 3, 9, 8, 2, 2, 0, 0), (2, 5, 9, 8, 3, 2, 1, 0), (1, 4, 7, 7, 3, 1, 1, 0),
                                           (3, 2, 10, 11, 3, 2, 0, 1), (1, 1, 5, 5, 5, 5, 2, 0)):
        x = g.standard_normal((B, Cn, H, W), dtype=np.float32)
        # ties: repeated values inside windows (first maximum wins)
        x[:, :, ::3, ::2] = np.float32(0.75)
        xr = api.from_device_dtype(api.to_device_dtype(hiplib, x, dt), x.shape, dt)
        pooled, ind = oracle.maxpool_indices(xr, k, k, d, d, pad, pad, ceil)
        oH, oW = pooled.shape[2:]
        G.note("maxpool_indices/unpool %s dtype %d" % ((B, Cn, H, W, k, d, pad, ceil), dt))
        es = 4 if dt == G.F32 else 2
        dx = api.to_device_dtype(hiplib, x, dt)
        dy = api.DeviceArray(hiplib, nbytes=pooled.size * es)
        di = api.DeviceArray(hiplib, nbytes=pooled.size * 4)
        hiplib.thhip_maxpool_indices(dx.ptr, dy.ptr, di.ptr, B, Cn, H, W, oH, oW, k, k, d, d, pad, pad, dt)
        hiplib.thhip_sync()
        assert np.array_equal(api.from_device_dtype(dy, pooled.shape, dt), pooled)
        assert np.array_equal(di.get(pooled.shape, np.int32) + 1, ind.astype(np.int32))
        v = g.standard_normal(pooled.shape, dtype=np.float32)
        vr = api.from_device_dtype(api.to_device_dtype(hiplib, v, dt), v.shape, dt)
        dv = api.to_device_dtype(hiplib, v, dt)
        du = api.DeviceArray(hiplib, nbytes=x.size * es)
        hiplib.thhip_maxunpool(dv.ptr, di.ptr, du.ptr, B, Cn, H, W, oH, oW, k, k, d, d, pad, pad, dt)
        hiplib.thhip_sync()
        assert np.array_equal(api.from_device_dtype(du, x.shape, dt), oracle.maxunpool(vr, ind, H, W))


@pytest.mark.gpu
def test_maxpool_2x2_vector_path(hiplib, oracle):
    """2x2 / stride 2 pooling of fp32 planes with a width that is a multiple of four
    takes 16-byte loads; widths and heights that do not qualify take the general
    kernel.  Both bit-exact, -inf and large negative values included."""
    g = cases.rng(880)
    for (B, Cn, H, W) in ((2, 3, 8, 8), (1, 5, 6, 12), (3, 2, 224, 224), (2, 2, 7, 8), (2, 2, 8, 6), (1, 1, 2, 4)):
        x = g.standard_normal((B, Cn, H, W), dtype=np.float32)
        x[0, 0, :2, :4] = np.float32(-3e38)
        oH, oW = oracle.pool_outsize(H, W, 2, 2, 2, 2, 0, 0, 0)
        y = G.unary(hiplib, hiplib.thhip_maxpool, x, (B, Cn, oH, oW), G.F32, B, Cn, H, W, oH, oW, 2, 2, 2, 2, 0, 0, G.F32)
        assert np.array_equal(y, oracle.maxpool(x, 2, 2, 2, 2)), (B, Cn, H, W)
