"""Helpers for the GPU tests: call the kernel-level C ABI on numpy data."""
import ctypes as C

import numpy as np

from thnets_amd import abi, api

F32, F16, BF16, U8 = abi.THHIP_F32, abi.THHIP_F16, abi.THHIP_BF16, abi.THHIP_U8


def note(msg):
    print("[gpu-case] " + msg, flush=True)


def conv2d(lib, x, w, bias, d=(1, 1), pad=(0, 0), act=0, thr=0.0, val=0.0, dtype=F32):
    x = np.ascontiguousarray(x, np.float32)
    w = np.ascontiguousarray(w, np.float32)
    B, Ci, H, W = x.shape
    Co, _, kH, kW = w.shape
    K = Ci * kH * kW
    oH, oW = (H + 2 * pad[0] - kH) // d[0] + 1, (W + 2 * pad[1] - kW) // d[1] + 1
    note("conv2d x%s w%s d%s pad%s dtype%d" % (x.shape, w.shape, d, pad, dtype))
    wp = lib.thhip_conv_pack_weight(w.ctypes.data, Co, Ci, kH * kW, dtype)
    dx = api.to_device_dtype(lib, x, dtype)
    db = api.DeviceArray(lib, np.ascontiguousarray(bias, np.float32)) if bias is not None else None
    dy = api.DeviceArray(lib, nbytes=B * Co * oH * oW * (4 if dtype == F32 else 2))
    lib.thhip_conv2d(dx.ptr, wp, db.ptr if db else None, dy.ptr, B, Ci, H, W, Co, kH, kW, d[0], d[1], pad[0], pad[1],
                     act, thr, val, dtype)
    lib.thhip_sync()
    y = api.from_device_dtype(dy, (B, Co, oH, oW), dtype)
    lib.thhip_free(wp)
    return y


def conv2d_layout(lib, x, w, bias, d=(1, 1), pad=(0, 0), act=0, thr=0.0, val=0.0, dtype=F16, x_cl=0, y_cl=0, scale=None):
    """Convolution with the device tensors channels-last on either side (half types) and
    an optional per-plane factor applied before the bias; x and the result are
    [B][C][H][W] arrays."""
    x = np.ascontiguousarray(x, np.float32)
    w = np.ascontiguousarray(w, np.float32)
    B, Ci, H, W = x.shape
    Co, _, kH, kW = w.shape
    oH, oW = (H + 2 * pad[0] - kH) // d[0] + 1, (W + 2 * pad[1] - kW) // d[1] + 1
    note("conv2d_layout x%s w%s d%s pad%s dtype%d x_cl%d y_cl%d" % (x.shape, w.shape, d, pad, dtype, x_cl, y_cl))
    wp = lib.thhip_conv_pack_weight_layout(w.ctypes.data, Co, Ci, kH, kW, dtype, x_cl)
    dx = api.to_device_dtype(lib, np.ascontiguousarray(x.transpose(0, 2, 3, 1)) if x_cl else x, dtype)
    db = api.DeviceArray(lib, np.ascontiguousarray(bias, np.float32)) if bias is not None else None
    ds = api.DeviceArray(lib, np.ascontiguousarray(scale, np.float32)) if scale is not None else None
    dy = api.DeviceArray(lib, nbytes=B * Co * oH * oW * (4 if dtype == F32 else 2))
    lib.thhip_conv2d_layout(dx.ptr, wp, ds.ptr if ds else None, db.ptr if db else None, dy.ptr, B, Ci, H, W, Co, kH, kW,
                            d[0], d[1], pad[0], pad[1], act, thr, val, dtype, x_cl, y_cl)
    lib.thhip_sync()
    if y_cl:
        y = np.ascontiguousarray(api.from_device_dtype(dy, (B, oH, oW, Co), dtype).transpose(0, 3, 1, 2))
    else:
        y = api.from_device_dtype(dy, (B, Co, oH, oW), dtype)
    lib.thhip_free(wp)
    return y


def gemv(lib, x, w, bias, act=0, thr=0.0, val=0.0, dtype=F32):
    nOut, nIn = w.shape
    note("gemv %dx%d dtype%d" % (nOut, nIn, dtype))
    dx = api.to_device_dtype(lib, x, dtype)
    dw = api.to_device_dtype(lib, w, dtype)
    db = api.DeviceArray(lib, np.ascontiguousarray(bias, np.float32)) if bias is not None else None
    dy = api.DeviceArray(lib, nbytes=nOut * 4)
    lib.thhip_gemv(dx.ptr, dw.ptr, db.ptr if db else None, dy.ptr, nIn, nOut, act, thr, val, dtype)
    lib.thhip_sync()
    return api.from_device_dtype(dy, (nOut,), dtype)


def unary(lib, fn, x, out_shape, dtype, *args):
    dx = api.to_device_dtype(lib, x, dtype) if dtype != U8 else api.DeviceArray(lib, np.ascontiguousarray(x, np.uint8))
    n = int(np.prod(out_shape))
    dy = api.DeviceArray(lib, nbytes=n * {F32: 4, F16: 2, BF16: 2, U8: 1}[dtype])
    fn(dx.ptr, dy.ptr, *args)
    lib.thhip_sync()
    return api.from_device_dtype(dy, out_shape, dtype)


def conv2d_u8(lib, xq, wq, addend, d, pad, zero, prm, act=0, thr=0, val=0, x_cl=0, y_cl=0, tail=0):
    """xq and the result are [B][C][H][W] arrays; x_cl = 1 / y_cl = 1 make the device
    copies channels-last ([B][H][W][C]), x_cl = 2 asks for the four-plane pixel path
    (plane-major in memory); both call the layout entry point.  tail > 0 (with x_cl = 1):
    the device copy is followed by that many bytes of the code `zero` and the call says so."""
    xq = np.ascontiguousarray(xq, np.uint8)
    wq = np.ascontiguousarray(wq, np.uint8)
    B, Ci, H, W = xq.shape
    Co, _, kH, kW = wq.shape
    K = Ci * kH * kW
    oH, oW = (H + 2 * pad[0] - kH) // d[0] + 1, (W + 2 * pad[1] - kW) // d[1] + 1
    note("conv2d_u8 x%s w%s d%s pad%s prm%s" % (xq.shape, wq.shape, d, pad, prm))
    if x_cl:
        wp = lib.thhip_conv_pack_weight_u8_layout(wq.ctypes.data, Co, Ci, kH, kW, x_cl)
    else:
        wp = lib.thhip_conv_pack_weight_u8(wq.ctypes.data, Co, Ci, kH * kW)
    if tail:
        assert x_cl == 1
        dx = api.DeviceArray(lib, np.concatenate([np.ascontiguousarray(xq.transpose(0, 2, 3, 1)).ravel(),
                                                  np.full(tail, zero, np.uint8)]))
    else:
        dx = api.DeviceArray(lib, np.ascontiguousarray(xq.transpose(0, 2, 3, 1)) if x_cl == 1 else xq)
    da = api.DeviceArray(lib, np.ascontiguousarray(addend, np.int32)) if addend is not None else None
    dy = api.DeviceArray(lib, nbytes=B * Co * oH * oW)
    if tail:
        lib.thhip_conv2d_u8_layout_tail(dx.ptr, wp, da.ptr if da else None, dy.ptr, B, Ci, H, W, Co, kH, kW, d[0], d[1],
                                        pad[0], pad[1], zero, prm["a_off"], prm["b_off"], prm["c_off"], prm["c_mult"],
                                        prm["c_shift"], act, thr, val, x_cl, y_cl, tail)
    elif x_cl or y_cl:
        lib.thhip_conv2d_u8_layout(dx.ptr, wp, da.ptr if da else None, dy.ptr, B, Ci, H, W, Co, kH, kW, d[0], d[1],
                                   pad[0], pad[1], zero, prm["a_off"], prm["b_off"], prm["c_off"], prm["c_mult"],
                                   prm["c_shift"], act, thr, val, x_cl, y_cl)
    else:
        lib.thhip_conv2d_u8(dx.ptr, wp, da.ptr if da else None, dy.ptr, B, Ci, H, W, Co, kH, kW, d[0], d[1], pad[0],
                            pad[1], zero, prm["a_off"], prm["b_off"], prm["c_off"], prm["c_mult"], prm["c_shift"], act,
                            thr, val)
    lib.thhip_sync()
    if y_cl:
        y = np.ascontiguousarray(dy.get((B, oH, oW, Co), np.uint8).transpose(0, 3, 1, 2))
    else:
        y = dy.get((B, Co, oH, oW), np.uint8)
    lib.thhip_free(wp)
    return y


def assert_close(got, want, tol, what=""):
    got = np.asarray(got, np.float64)
    want = np.asarray(want, np.float64)
    assert got.shape == want.shape, (what, got.shape, want.shape)
    err = np.abs(got - want).max()
    ref = max(np.abs(want).max(), 1e-30)
    assert err <= tol * ref, "%s: max|err| %.3g > %.3g * max|ref| %.3g" % (what, err, tol, ref)
