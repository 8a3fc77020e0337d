"""ctypes front end of the CPU checkers.  TEST INFRASTRUCTURE ONLY.

Only tests/, the smoke run and the benchmark's cpu_baseline leg import this file;
nothing under thnets_amd/ does.  It offers

* ``Oracle``   -- liboracle.so (this repository's C restatement, thnets_oracle.c),
                  plus a layer-list executor for fp32 and uint8 networks;
* ``Reference``-- the reference's own CPU library when oracle/_ref holds a build of
                  it (made by oracle/Makefile from the reference sources), driven
                  through the same ``struct module`` arrays as the HIP engine.
"""
import ctypes as C
import os
import subprocess

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ORACLE_SO = os.path.join(HERE, "liboracle.so")
REF_SO = os.path.join(HERE, "_ref", "libthnets_ref.so")
REF_LOWP_SO = os.path.join(HERE, "_ref", "libthnets_ref_lowp.so")

_f32p = C.POINTER(C.c_float)
_u8p = C.POINTER(C.c_ubyte)


def _p(a, t=_f32p):
    return a.ctypes.data_as(t) if a is not None else None


def build(ref_root="/root/reference"):
    """Compile liboracle.so and, when the reference tree is present, oracle/_ref."""
    subprocess.check_call(["make", "-s", "-C", HERE, "REF=" + ref_root, "all"])


class Oracle:
    def __init__(self):
        if not os.path.exists(ORACLE_SO):
            build()
        self.lib = L = C.CDLL(ORACLE_SO)
        L.orc_exp_minus_approx.restype = C.c_double
        L.orc_exp_minus_approx.argtypes = [C.c_double]
        L.orc_lowp_softmax.restype = C.c_float
        L.orc_lowp_scale_float.restype = C.c_ubyte
        L.orc_lowp_scale_float.argtypes = [C.c_float, C.c_float, C.c_float]
        L.orc_lowp_bias_addend.argtypes = [C.c_ubyte, C.c_float, C.c_float, C.c_float]
        L.orc_lowp_requant.restype = C.c_ubyte

    # ---- fp32 primitives ----
    def threads(self):
        return self.lib.orc_num_threads()

    def set_threads(self, n):
        self.lib.orc_set_num_threads(int(n))

    def conv_outsize(self, i, k, d, pad):
        return self.lib.orc_conv_outsize(i, k, d, pad)

    def conv2d(self, x, w, bias, d=(1, 1), pad=(0, 0), use_unfold=False):
        x = np.ascontiguousarray(x, np.float32)
        w = np.ascontiguousarray(w, np.float32)
        B, Ci, H, W = x.shape
        Co, _, kH, kW = w.shape
        oH, oW = self.conv_outsize(H, kH, d[0], pad[0]), self.conv_outsize(W, kW, d[1], pad[1])
        y = np.empty((B, Co, oH, oW), np.float32)
        b = None if bias is None else np.ascontiguousarray(bias, np.float32)
        rc = self.lib.orc_conv2d_f32(_p(x), _p(w), _p(b), _p(y), B, Ci, H, W, Co, kH, kW, d[0], d[1], pad[0], pad[1],
                                     int(use_unfold))
        if rc:
            raise ValueError("output size is too small")
        return y

    def conv2d_f64(self, x, w, bias, d=(1, 1), pad=(0, 0)):
        x = np.ascontiguousarray(x, np.float32)
        w = np.ascontiguousarray(w, np.float32)
        B, Ci, H, W = x.shape
        Co, _, kH, kW = w.shape
        oH, oW = self.conv_outsize(H, kH, d[0], pad[0]), self.conv_outsize(W, kW, d[1], pad[1])
        y = np.empty((B, Co, oH, oW), np.float64)
        b = None if bias is None else np.ascontiguousarray(bias, np.float32)
        self.lib.orc_conv2d_f64(_p(x), _p(w), _p(b), y.ctypes.data_as(C.POINTER(C.c_double)), B, Ci, H, W, Co, kH, kW,
                                d[0], d[1], pad[0], pad[1])
        return y

    def unfold(self, x, k, d, pad):
        x = np.ascontiguousarray(x, np.float32)
        Ci, H, W = x.shape
        oH, oW = self.conv_outsize(H, k[0], d[0], pad[0]), self.conv_outsize(W, k[1], d[1], pad[1])
        col = np.empty((Ci * k[0] * k[1], oH * oW), np.float32)
        self.lib.orc_unfold_f32(_p(x), _p(col), Ci, H, W, k[0], k[1], d[0], d[1], pad[0], pad[1], oH, oW)
        return col

    def sgemm_acc(self, a, b, c):
        M, K = a.shape
        N = b.shape[1]
        self.lib.orc_sgemm_acc(M, N, K, _p(a), _p(b), _p(c))
        return c

    def linear(self, x, w, bias):
        x = np.ascontiguousarray(x, np.float32)
        w = np.ascontiguousarray(w, np.float32)
        b = None if bias is None else np.ascontiguousarray(bias, np.float32)
        nOut, nIn = w.shape
        if x.ndim == 1:
            y = np.empty(nOut, np.float32)
            self.lib.orc_linear1d_f32(_p(x), _p(w), _p(b), _p(y), nIn, nOut)
        else:
            y = np.empty((x.shape[0], nOut), np.float32)
            self.lib.orc_linear2d_f32(_p(x), _p(w), _p(b), _p(y), x.shape[0], nIn, nOut)
        return y

    def threshold(self, x, thr=0.0, val=0.0, alpha=0.0, inplace=1):
        x = np.ascontiguousarray(x, np.float32)
        y = np.empty_like(x)
        self.lib.orc_threshold_f32(_p(x), _p(y), C.c_long(x.size), C.c_float(thr), C.c_float(val), C.c_float(alpha),
                                   int(inplace))
        return y

    def pool_outsize(self, H, W, kH, kW, dH, dW, padH, padW, ceil_mode):
        oh, ow = C.c_int(), C.c_int()
        self.lib.orc_pool_outsize(H, W, kH, kW, dH, dW, padH, padW, ceil_mode, C.byref(oh), C.byref(ow))
        return oh.value, ow.value

    def maxpool(self, x, kH, kW, dH, dW, padH=0, padW=0, ceil_mode=0):
        x = np.ascontiguousarray(x, np.float32)
        B, Cn, H, W = x.shape
        oH, oW = self.pool_outsize(H, W, kH, kW, dH, dW, padH, padW, ceil_mode)
        y = np.empty((B, Cn, oH, oW), np.float32)
        self.lib.orc_maxpool_f32(_p(x), _p(y), B, Cn, H, W, oH, oW, kH, kW, dH, dW, padH, padW)
        return y

    def maxpool_indices(self, x, kH, kW, dH, dW, padH=0, padW=0, ceil_mode=0):
        """(output, indices): indices are float, position of the maximum in the input plane + 1."""
        x = np.ascontiguousarray(x, np.float32)
        B, Cn, H, W = x.shape
        oH, oW = self.pool_outsize(H, W, kH, kW, dH, dW, padH, padW, ceil_mode)
        y = np.empty((B, Cn, oH, oW), np.float32)
        ind = np.empty((B, Cn, oH, oW), np.float32)
        self.lib.orc_maxpool_indices_f32(_p(x), _p(y), _p(ind), B, Cn, H, W, oH, oW, kH, kW, dH, dW, padH, padW)
        return y, ind

    def maxunpool(self, x, ind, oH, oW):
        x = np.ascontiguousarray(x, np.float32)
        ind = np.ascontiguousarray(ind, np.float32)
        B, Cn, iH, iW = x.shape
        y = np.empty((B, Cn, oH, oW), np.float32)
        if self.lib.orc_maxunpool_f32(_p(x), _p(ind), _p(y), B, Cn, iH, iW, oH, oW):
            raise ValueError("invalid max index")
        return y

    def fullconv2d(self, x, w, bias, d=(1, 1), pad=(0, 0), adj=(0, 0)):
        """x [B,Ci,H,W], w [Ci,Co,kH,kW]; the reference's arithmetic (11 * result + bias when there is a bias)."""
        x = np.ascontiguousarray(x, np.float32)
        w = np.ascontiguousarray(w, np.float32)
        B, Ci, H, W = x.shape
        _, Co, kH, kW = w.shape
        oH, oW = (H - 1) * d[0] - 2 * pad[0] + kH + adj[0], (W - 1) * d[1] - 2 * pad[1] + kW + adj[1]
        y = np.empty((B, Co, oH, oW), np.float32)
        b = None if bias is None else np.ascontiguousarray(bias, np.float32)
        self.lib.orc_fullconv2d_f32(_p(x), _p(w), _p(b) if b is not None else None, _p(y), B, Ci, H, W, Co, kH, kW,
                                    d[0], d[1], pad[0], pad[1], adj[0], adj[1])
        return y

    def fullconv2d_f64(self, x, w, d=(1, 1), pad=(0, 0), adj=(0, 0)):
        x = np.ascontiguousarray(x, np.float32)
        w = np.ascontiguousarray(w, np.float32)
        B, Ci, H, W = x.shape
        _, Co, kH, kW = w.shape
        oH, oW = (H - 1) * d[0] - 2 * pad[0] + kH + adj[0], (W - 1) * d[1] - 2 * pad[1] + kW + adj[1]
        y = np.empty((B, Co, oH, oW), np.float64)
        self.lib.orc_fullconv2d_f64(_p(x), _p(w), y.ctypes.data_as(C.c_void_p), B, Ci, H, W, Co, kH, kW,
                                    d[0], d[1], pad[0], pad[1], adj[0], adj[1])
        return y

    def avgpool(self, x, kH, kW, dH, dW, padH=0, padW=0, ceil_mode=0, count_include_pad=1):
        x = np.ascontiguousarray(x, np.float32)
        B, Cn, H, W = x.shape
        kH = kH or H
        kW = kW or W
        oH, oW = self.pool_outsize(H, W, kH, kW, dH, dW, padH, padW, ceil_mode)
        y = np.empty((B, Cn, oH, oW), np.float32)
        self.lib.orc_avgpool_f32(_p(x), _p(y), B, Cn, H, W, oH, oW, kH, kW, dH, dW, padH, padW, count_include_pad)
        return y

    def softmax(self, x):
        x = np.ascontiguousarray(x, np.float32)
        y = np.empty_like(x)
        if x.ndim == 1:
            nframe, dim, stride = 1, x.shape[0], 1
        elif x.ndim == 2:
            nframe, dim, stride = x.shape[0], x.shape[1], 1
        elif x.ndim == 3:
            nframe, dim, stride = 1, x.shape[0], x.shape[1] * x.shape[2]
        else:
            nframe, dim, stride = x.shape[0], x.shape[1], x.shape[2] * x.shape[3]
        self.lib.orc_softmax_f32(_p(x), _p(y), C.c_long(nframe), C.c_long(dim), C.c_long(stride))
        return y

    def batchnorm(self, x, mean, var, weight, bias, eps):
        x = np.ascontiguousarray(x, np.float32)
        y = np.empty_like(x)
        B, Cn = x.shape[0], x.shape[1]
        HW = x.size // (B * Cn)
        a = [None if v is None else np.ascontiguousarray(v, np.float32) for v in (mean, var, weight, bias)]
        self.lib.orc_batchnorm_f32(_p(x), _p(y), C.c_long(B), C.c_long(Cn), C.c_long(HW), _p(a[0]), _p(a[1]), _p(a[2]),
                                   _p(a[3]), C.c_double(eps))
        return y

    def caddtable(self, ins, is_csubtable=False):
        ins = [np.ascontiguousarray(v, np.float32) for v in ins]
        out = np.empty_like(ins[0])
        arr = (_f32p * len(ins))(*[_p(v) for v in ins])
        n = (C.c_long * len(ins))(*[v.size for v in ins])
        self.lib.orc_caddtable_f32(int(is_csubtable), len(ins), arr, n, _p(out))
        return out

    def normalize(self, x, mean, std):
        x = np.array(x, np.float32, copy=True, order="C")
        B, Cn = x.shape[0], x.shape[1]
        m = np.asarray(mean, np.float32)
        s = np.asarray(std, np.float32)
        self.lib.orc_normalize_f32(_p(x), B, Cn, C.c_long(x.size // (B * Cn)), _p(m), _p(s))
        return x

    def rgb2float(self, img, mean, std, bgr=0):
        """img: uint8 [H][W][cp] (row stride = W*cp)."""
        img = np.ascontiguousarray(img, np.uint8)
        H, W, cp = img.shape
        dst = np.empty((cp, H, W), np.float32)
        m = np.asarray(mean, np.float32)
        s = np.asarray(std, np.float32)
        self.lib.orc_rgb2float(_p(dst), _p(img, _u8p), W, H, W * cp, cp, _p(m), _p(s), int(bgr))
        return dst

    # ---- fp32 network executor (forward(), thapi.c:158-235, on a layer list) ----
    def run_layers(self, layers, x, collect=None):
        """x: float32 array, 4-D [B,C,H,W] or as produced by earlier layers.  Returns
        the output; ``collect`` (a list) receives every top-level module output."""
        kept = {}       # position of a maxpool -> (indices, input height, input width), for maxunpool
        outs = []       # every output, for layers that name their inputs (thapi.c:173-193)
        for pos, spec in enumerate(layers):
            if spec.get("inputs"):
                x = outs[spec["inputs"][0]] if len(spec["inputs"]) == 1 else [outs[j] for j in spec["inputs"]]
            if spec["type"] == "maxpool":
                h, w = x.shape[-2:]
                x4 = x if x.ndim == 4 else x[None]
                y, ind = self.maxpool_indices(x4, spec["kH"], spec["kW"], spec["dH"], spec["dW"], spec["padH"], spec["padW"],
                                              spec.get("ceil_mode", 0))
                kept[pos] = (ind, h, w)
                x = y if x.ndim == 4 else y[0]
            elif spec["type"] == "maxunpool":
                ind, h, w = kept[spec["pooling"]]
                x4 = x if x.ndim == 4 else x[None]
                y = self.maxunpool(x4, ind, h, w)
                x = y if x.ndim == 4 else y[0]
            else:
                x = self._run_one(spec, x)
            outs.append(x)
            if collect is not None:
                collect.append(x if not isinstance(x, list) else [v.copy() for v in x])
        return x

    def _run_one(self, spec, x):
        k = spec["type"]
        if k == "conv":
            return self.conv2d(x, spec["weight"], spec["bias"], (spec["dH"], spec["dW"]), (spec["padH"], spec["padW"]),
                               use_unfold=spec.get("mm") == "mm")
        if k == "fullconv":
            x4 = x if x.ndim == 4 else x[None]
            y = self.fullconv2d(x4, spec["weight"], spec.get("bias"), (spec.get("dH", 1), spec.get("dW", 1)),
                                (spec.get("padH", 0), spec.get("padW", 0)), (spec.get("adjH", 0), spec.get("adjW", 0)))
            return y if x.ndim == 4 else y[0]
        if k == "linear":
            xs = np.squeeze(x)          # THFloatTensor_squeeze, Linear.c:86
            return self.linear(xs, spec["weight"], spec["bias"])
        if k == "threshold":
            return self.threshold(x, spec.get("threshold", 0.0), spec.get("val", 0.0), spec.get("alpha", 0.0),
                                  spec.get("inplace", 1))
        if k == "maxpool":
            return self.maxpool(x, spec["kH"], spec["kW"], spec["dH"], spec["dW"], spec["padH"], spec["padW"],
                                spec.get("ceil_mode", 0))
        if k == "avgpool":
            return self.avgpool(x, spec["kH"], spec["kW"], spec["dH"], spec["dW"], spec["padH"], spec["padW"],
                                spec.get("ceil_mode", 0), spec.get("count_include_pad", 1))
        if k == "view":
            # nn_View_updateOutput, View.c:84-97: [B, numElements] when B > 1 else 1-D
            n = spec["numElements"]
            b = x.shape[0] if x.ndim == 4 else 1
            if n == -1:
                n = x.size // b
            else:
                b = x.size // n
            return x.reshape(b, n) if b > 1 else x.reshape(n)
        if k == "softmax":
            return self.softmax(x)
        if k == "bn":
            return self.batchnorm(x, spec["running_mean"], spec["running_var"], spec.get("weight"), spec.get("bias"),
                                  spec.get("eps", 1e-5))
        if k == "dropout":
            return x if spec.get("v2", 1) == 1 else (x * np.float32(1 - spec.get("p", 0.5))).astype(np.float32)
        if k == "sequential":
            return self.run_layers(spec["layers"], x)
        if k == "concattable":
            return [self.run_layers(b, x) for b in spec["branches"]]
        if k in ("caddtable", "csubtable"):
            return self.caddtable(x, is_csubtable=(k == "csubtable"))
        raise ValueError(k)

    # ---- uint8 primitives ----
    def lowp_quantize(self, x):
        x = np.ascontiguousarray(x, np.float32)
        q = np.empty(x.shape, np.uint8)
        mult, sub = C.c_float(), C.c_float()
        self.lib.orc_lowp_quantize(_p(x), C.c_long(x.size), _p(q, _u8p), C.byref(mult), C.byref(sub))
        return q, mult.value, sub.value

    def lowp_dequantize(self, q, mult, sub):
        q = np.ascontiguousarray(q, np.uint8)
        x = np.empty(q.shape, np.float32)
        self.lib.orc_lowp_dequantize(_p(q, _u8p), C.c_long(q.size), C.c_float(mult), C.c_float(sub), _p(x))
        return x

    def lowp_mm_params(self, wm, wsub, im, isub, om, osub):
        out = (C.c_int * 5)()
        self.lib.orc_lowp_mm_params(C.c_float(wm), C.c_float(wsub), C.c_float(im), C.c_float(isub), C.c_float(om),
                                    C.c_float(osub), out)
        return dict(a_off=out[0], b_off=out[1], c_off=out[2], c_mult=out[3], c_shift=out[4])

    def lowp_bias_addend(self, bq, bm, bsub, om):
        return self.lib.orc_lowp_bias_addend(int(bq), bm, bsub, om)

    def lowp_gemm(self, a, b, a_off, b_off, c_off, c_mult, c_shift):
        a = np.ascontiguousarray(a, np.uint8)
        b = np.ascontiguousarray(b, np.uint8)
        m, k = a.shape
        n = b.shape[1]
        c = np.empty((m, n), np.uint8)
        self.lib.orc_lowp_gemm(m, n, k, _p(a, _u8p), _p(b, _u8p), _p(c, _u8p), k, n, n, a_off, b_off, c_off, c_mult,
                               c_shift)
        return c

    def lowp_add(self, dst, add):
        dst = np.array(dst, np.uint8, copy=True)
        self.lib.orc_lowp_add(_p(dst, _u8p), int(add), dst.size)
        return dst

    def lowp_unfold(self, x, k, d, pad, zero):
        x = np.ascontiguousarray(x, np.uint8)
        Ci, H, W = x.shape
        oH, oW = self.conv_outsize(H, k[0], d[0], pad[0]), self.conv_outsize(W, k[1], d[1], pad[1])
        col = np.empty((Ci * k[0] * k[1], oH * oW), np.uint8)
        self.lib.orc_lowp_unfold(_p(x, _u8p), _p(col, _u8p), Ci, H, W, k[0], k[1], d[0], d[1], pad[0], pad[1], oH, oW,
                                 C.c_ubyte(zero))
        return col

    def lowp_conv2d(self, xq, im, isub, wq, wm, wsub, bq, bm, bsub, om, osub, d, pad):
        xq = np.ascontiguousarray(xq, np.uint8)
        wq = np.ascontiguousarray(wq, np.uint8)
        bq = np.ascontiguousarray(bq, np.uint8)
        B, Ci, H, W = xq.shape
        Co, _, kH, kW = wq.shape
        oH, oW = self.conv_outsize(H, kH, d[0], pad[0]), self.conv_outsize(W, kW, d[1], pad[1])
        y = np.empty((B, Co, oH, oW), np.uint8)
        f = C.c_float
        rc = self.lib.orc_lowp_conv2d(_p(xq, _u8p), f(im), f(isub), _p(wq, _u8p), f(wm), f(wsub), _p(bq, _u8p), f(bm),
                                      f(bsub), _p(y, _u8p), f(om), f(osub), B, Ci, H, W, Co, kH, kW, d[0], d[1],
                                      pad[0], pad[1])
        if rc:
            raise ValueError("output size is too small")
        return y

    def lowp_scale_float(self, mult, sub, value):
        return self.lib.orc_lowp_scale_float(mult, sub, value)

    def lowp_threshold(self, q, thr, val, inplace=1):
        q = np.ascontiguousarray(q, np.uint8)
        y = np.empty_like(q)
        self.lib.orc_lowp_threshold(_p(q, _u8p), _p(y, _u8p), C.c_long(q.size), C.c_ubyte(thr), C.c_ubyte(val),
                                    int(inplace))
        return y

    def lowp_maxpool(self, q, kH, kW, dH, dW, padH=0, padW=0, ceil_mode=0):
        q = np.ascontiguousarray(q, np.uint8)
        B, Cn, H, W = q.shape
        oH, oW = self.pool_outsize(H, W, kH, kW, dH, dW, padH, padW, ceil_mode)
        y = np.empty((B, Cn, oH, oW), np.uint8)
        self.lib.orc_lowp_maxpool(_p(q, _u8p), _p(y, _u8p), B, Cn, H, W, oH, oW, kH, kW, dH, dW, padH, padW)
        return y

    def lowp_softmax(self, q, mult, sub):
        q = np.ascontiguousarray(q, np.uint8)
        y = np.empty_like(q)
        if q.ndim == 1:
            nframe, dim, stride = 1, q.shape[0], 1
        elif q.ndim == 2:
            nframe, dim, stride = q.shape[0], q.shape[1], 1
        elif q.ndim == 3:
            nframe, dim, stride = 1, q.shape[0], q.shape[1] * q.shape[2]
        else:
            nframe, dim, stride = q.shape[0], q.shape[1], q.shape[2] * q.shape[3]
        om = self.lib.orc_lowp_softmax(_p(q, _u8p), _p(y, _u8p), C.c_long(nframe), C.c_long(dim), C.c_long(stride),
                                       C.c_float(mult), C.c_float(sub))
        return y, om, 0.0

    # ---- uint8 network executor (THLowp_ToLowp + forward on a layer list) ----
    def lowp_prepare(self, layers):
        """Weight / bias quantisation of THLowp_ToLowp, lowp_basic.c:154-193."""
        prep = []
        for spec in layers:
            if spec["type"] in ("conv", "linear"):
                w = np.asarray(spec["weight"], np.float32)
                if spec["type"] == "linear":
                    w = w.reshape(w.shape[0], w.shape[1], 1, 1)
                wq, wm, wsub = self.lowp_quantize(w)
                bq, bm, bsub = self.lowp_quantize(spec["bias"])
                prep.append(dict(wq=wq, wm=wm, wsub=wsub, bq=bq, bm=bm, bsub=bsub))
            else:
                prep.append(None)
        return prep

    def lowp_run_layers(self, layers, xq, im, isub, rng, prep=None, collect=None):
        """Runs uint8 codes ``xq`` (with mult ``im``, sub ``isub``) through the network.
        Every module output uses mult = 255/range, sub = -range/2
        (lowp_basic.c:137-148).  Returns (codes, mult, sub)."""
        prep = prep or self.lowp_prepare(layers)
        om = np.float32(255) / np.float32(rng)
        osub = -np.float32(rng) / np.float32(2)
        q, m, s = xq, np.float32(im), np.float32(isub)
        for spec, p in zip(layers, prep):
            k = spec["type"]
            if k in ("conv", "linear"):
                if q.ndim == 2:
                    q = q.reshape(q.shape[0], q.shape[1], 1, 1)
                d = (spec.get("dH", 1), spec.get("dW", 1))
                pad = (spec.get("padH", 0), spec.get("padW", 0))
                q = self.lowp_conv2d(q, m, s, p["wq"], p["wm"], p["wsub"], p["bq"], p["bm"], p["bsub"], om, osub, d, pad)
                m, s = om, osub
            elif k == "threshold":
                thr = self.lowp_scale_float(m, s, spec.get("threshold", 0.0))
                val = self.lowp_scale_float(m, s, spec.get("val", 0.0))
                q = self.lowp_threshold(q, thr, val, spec.get("inplace", 1))
            elif k == "maxpool":
                q = self.lowp_maxpool(q, spec["kH"], spec["kW"], spec["dH"], spec["dW"], spec["padH"], spec["padW"],
                                      spec.get("ceil_mode", 0))
            elif k == "softmax":
                q, m, s = self.lowp_softmax(q, m, s)
            elif k == "dropout":
                pass
            else:
                raise ValueError("module %r is not supported by the uint8 engine" % k)
            if collect is not None:
                collect.append((q.copy(), float(m), float(s)))
        return q, float(m), float(s)


class Reference:
    """The reference's own CPU library, when a build of it exists in oracle/_ref."""

    @staticmethod
    def available(lowp=False):
        return os.path.exists(REF_LOWP_SO if lowp else REF_SO)

    def __init__(self, lowp=False, threads=None):
        from thnets_amd.abi import ABI, ABI_LOWP
        self.lowp = lowp
        self.abi = ABI_LOWP if lowp else ABI
        path = REF_LOWP_SO if lowp else REF_SO
        # lowpgemm is an unresolved symbol of the -DLOWP build: bind lazily
        self.lib = L = C.CDLL(path, mode=os.RTLD_LAZY)
        self._gomp = C.CDLL("libgomp.so.1")
        if threads:
            self._gomp.omp_set_num_threads(int(threads))
        L.THInit()
        self.max_threads = C.c_int.in_dll(L, "threads_num").value
        L.THFloatTensor_new.restype = C.c_void_p
        L.forward.restype = C.c_void_p
        L.forward.argtypes = [C.c_void_p, C.c_void_p]
        L.THProcessFloat.argtypes = [C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_int,
                                     C.POINTER(C.POINTER(C.c_float)), C.POINTER(C.c_int), C.POINTER(C.c_int)]

    def set_threads(self, n):
        """Thread counts must divide the batch: the reference's batched convolution
        hangs otherwise (orphaned barriers, OpenBLAS-stripped/sgemm.c:967-979)."""
        n = max(1, min(int(n), self.max_threads))
        self._gomp.omp_set_num_threads(n)
        C.c_int.in_dll(self.lib, "threads_num").value = n
        return n

    def threads_for_batch(self, batch, limit=None):
        limit = min(limit or self.max_threads, self.max_threads)
        if batch < 4:
            return limit
        return max(d for d in range(1, limit + 1) if batch % d == 0)

    def host_network(self, cfg):
        from thnets_amd.netbuild import HostNetwork
        return HostNetwork(self.lib, self.abi, resolve_cpu=True).build(cfg["layers"], cfg["mean"], cfg["std"])

    def process_float(self, hostnet, x):
        """THProcessFloat on a fresh copy (it normalises its argument in place)."""
        from thnets_amd.netbuild import tensor_to_numpy  # noqa: F401
        x = np.array(x, np.float32, copy=True, order="C")
        B, Cn, H, W = x.shape
        res = C.POINTER(C.c_float)()
        ow, oh = C.c_int(), C.c_int()
        self.set_threads(self.threads_for_batch(B))
        n = self.lib.THProcessFloat(C.addressof(hostnet.thnet), x.ctypes.data, B, W, H, Cn, C.byref(res), C.byref(ow),
                                    C.byref(oh))
        return np.ctypeslib.as_array(res, shape=(n,)).copy()

    def forward(self, hostnet, x):
        """forward() (thapi.c:158-235) on an un-normalised tensor of any plane count."""
        from thnets_amd.netbuild import tensor_to_numpy
        x = np.array(x, np.float32, copy=True, order="C")
        self.set_threads(self.threads_for_batch(x.shape[0] if x.ndim == 4 else 1))
        t = hostnet.tensor(x)
        out = self.lib.forward(C.addressof(hostnet.thnet.net.contents), C.addressof(t.contents))
        return tensor_to_numpy(self.abi, C.cast(out, self.abi.PTensor))

    def module_output(self, hostnet, idx):
        from thnets_amd.netbuild import tensor_to_numpy
        return tensor_to_numpy(self.abi, hostnet.thnet.net.contents.modules[idx].output)

    # ---- -DLOWP build only: the reference's uint8 helpers that do not need gemmlowp ----
    def _lowp_tensor(self, hostnet, q, mult, sub):
        """uint8 codes as the reference stores them: a THFloatTensor whose storage holds bytes."""
        q = np.ascontiguousarray(q, np.uint8)
        from thnets_amd.abi import THFloatStorage
        st = THFloatStorage(q.ctypes.data, 1, 0)
        t = self.abi.THFloatTensor()
        t.nDimension = q.ndim
        stride = 1
        for i in range(q.ndim - 1, -1, -1):
            t.size[i] = q.shape[i]
            t.stride[i] = stride
            stride *= q.shape[i]
        t.storage = C.pointer(st)
        t.mult, t.sub = mult, sub
        hostnet._keep += [q, st, t]
        return t

    def _lowp_read(self, pt):
        t = pt.contents
        shape = tuple(t.size[i] for i in range(t.nDimension))
        n = int(np.prod(shape))
        buf = (C.c_ubyte * n).from_address(t.storage.contents.data + t.storageOffset)
        return np.frombuffer(buf, np.uint8).reshape(shape).copy(), float(t.mult), float(t.sub)

    def lowp_quantize(self, x):
        """THLowpTensor_newFromFloatTensor (lowp_basic.c:5-38) run by the reference."""
        assert self.lowp
        from thnets_amd.netbuild import HostNetwork
        hn = HostNetwork(self.lib, self.abi)
        t = hn.tensor(np.ascontiguousarray(x, np.float32))
        self.lib.THLowpTensor_newFromFloatTensor.restype = C.c_void_p
        self.lib.THLowpTensor_newFromFloatTensor.argtypes = [C.c_void_p]
        out = self.lib.THLowpTensor_newFromFloatTensor(C.addressof(t.contents))
        return self._lowp_read(C.cast(out, self.abi.PTensor))

    def lowp_dequantize(self, q, mult, sub):
        """THFloatTensor_newFromLowpTensor (lowp_basic.c:40-58) run by the reference."""
        from thnets_amd.netbuild import HostNetwork, tensor_to_numpy
        hn = HostNetwork(self.lib, self.abi)
        t = self._lowp_tensor(hn, q, mult, sub)
        self.lib.THFloatTensor_newFromLowpTensor.restype = C.c_void_p
        self.lib.THFloatTensor_newFromLowpTensor.argtypes = [C.c_void_p]
        out = self.lib.THFloatTensor_newFromLowpTensor(C.addressof(t))
        return tensor_to_numpy(self.abi, C.cast(out, self.abi.PTensor))

    def lowp_scale_float(self, mult, sub, value):
        from thnets_amd.netbuild import HostNetwork
        hn = HostNetwork(self.lib, self.abi)
        t = self._lowp_tensor(hn, np.zeros(1, np.uint8), mult, sub)
        self.lib.THLowp_ScaleFloat.restype = C.c_ubyte
        self.lib.THLowp_ScaleFloat.argtypes = [C.c_void_p, C.c_float]
        return self.lib.THLowp_ScaleFloat(C.addressof(t), value)

    def lowp_module(self, spec, q, mult, sub, out_mult=None, out_sub=None):
        """Runs one of Lowp_Threshold / Lowp_SpatialMaxPooling / Lowp_SoftMax
        _updateOutput (lowp/lowp_*.c) on codes q; OpenMP is pinned to one thread
        (the shipped softmax shares a scratch row between threads)."""
        from thnets_amd.netbuild import HostNetwork
        fn = {"threshold": "Lowp_Threshold_updateOutput", "maxpool": "Lowp_SpatialMaxPooling_updateOutput",
              "softmax": "Lowp_SoftMax_updateOutput"}[spec["type"]]
        hn = HostNetwork(self.lib, self.abi).build([spec])
        m = hn.thnet.net.contents.modules[0]
        if out_mult is not None:
            m.output.contents.mult, m.output.contents.sub = out_mult, out_sub
        t = self._lowp_tensor(hn, np.array(q, np.uint8, copy=True), mult, sub)
        self.set_threads(1)
        f = getattr(self.lib, fn)
        f.restype = C.c_void_p
        f.argtypes = [C.c_void_p, C.c_void_p]
        out = f(C.addressof(m), C.addressof(t))
        return self._lowp_read(C.cast(out, self.abi.PTensor))

    def lowp_load_images(self, images, mean, std, bgr=0):
        """Lowp_LoadImages (lowp_basic.c:82-131) run by the reference."""
        imgs = [np.ascontiguousarray(im, np.uint8) for im in images]
        H, W = imgs[0].shape[:2]
        ptrs = (C.c_void_p * len(imgs))(*[im.ctypes.data for im in imgs])
        m = (C.c_float * 3)(*mean)
        s = (C.c_float * 3)(*std)
        self.lib.Lowp_LoadImages.restype = C.c_void_p
        self.lib.Lowp_LoadImages.argtypes = [C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_void_p, C.c_int]
        self.set_threads(1)
        out = self.lib.Lowp_LoadImages(ptrs, len(imgs), W, H, W * 3, m, s, int(bgr))
        return self._lowp_read(C.cast(out, self.abi.PTensor))
