"""Builds thnets ``struct module`` arrays in memory from numpy weights.

The reference ships no model files and its loaders (.t7 / ONNX) are outside the
path this repository accelerates, so networks are assembled the way
examples/thnets-tf.cc:112-138 of the reference does it: fill ``struct module`` by
hand.  The result is a host ("CPU description") network that
``THCreateHipNetwork`` / ``THCreateHipLowpNetwork`` turn into a device network,
exactly as the reference turns a loaded network into a cuDNN or LOWP one
(thapi.c:730-742, 784-796).

A layer list is a list of dicts; ``type`` selects the module:

    conv        weight [Co,Ci,kH,kW], bias [Co] | None, dW dH padW padH, mm="virt"|"mm"
    linear      weight [nOut,nIn], bias [nOut]
    threshold   threshold val alpha inplace          (ReLU = all zero, inplace 1)
    maxpool     kW kH dW dH padW padH ceil_mode
    avgpool     kW kH dW dH padW padH ceil_mode count_include_pad
    view        numElements
    softmax
    bn          running_mean running_var weight bias eps
    dropout     p inplace v2
    sequential  layers=[...]
    concattable branches=[[...], [...]]
    fullconv    weight [Ci,Co,kH,kW], bias [Co] | None, dW dH padW padH adjW adjH
    maxunpool   pooling=<position of its maxpool in the same list>
    caddtable | csubtable
"""
import ctypes as C

import numpy as np

from .abi import ABI, MT, THFloatStorage, ENGINE_CPU

# name of the CPU updateOutput of each module type in a thnets library
CPU_UPDATE = {
    "conv": "nn_SpatialConvolutionMM_updateOutput",
    "linear": "nn_Linear_updateOutput",
    "threshold": "nn_Threshold_updateOutput",
    "maxpool": "nn_SpatialMaxPooling_updateOutput",
    "avgpool": "nn_SpatialAveragePooling_updateOutput",
    "view": "nn_View_updateOutput",
    "softmax": "nn_SoftMax_updateOutput",
    "bn": "nn_SpatialBatchNormalization_updateOutput",
    "dropout": "nn_Dropout_updateOutput",
    "sequential": "nn_Sequential_updateOutput",
    "concattable": "nn_ConcatTable_updateOutput",
    "fullconv": "nn_SpatialFullConvolution_updateOutput",
    "maxunpool": "nn_SpatialMaxUnpooling_updateOutput",
    "caddtable": "nn_CAddTable_updateOutput",
    "csubtable": "nn_CAddTable_updateOutput",
}


def relu(inplace=1):
    return {"type": "threshold", "threshold": 0.0, "val": 0.0, "alpha": 0.0, "inplace": inplace}


def conv(weight, bias, d=1, pad=0, mm="virt"):
    return {"type": "conv", "weight": weight, "bias": bias, "dW": d, "dH": d, "padW": pad, "padH": pad, "mm": mm}


def maxpool(k, d, pad=0, ceil_mode=0):
    return {"type": "maxpool", "kW": k, "kH": k, "dW": d, "dH": d, "padW": pad, "padH": pad, "ceil_mode": ceil_mode}


class HostNetwork:
    """A THNETWORK in ctypes memory plus everything that must stay alive with it."""

    def __init__(self, lib, abi=ABI, resolve_cpu=False):
        self.lib = lib
        self.abi = abi
        self.resolve_cpu = resolve_cpu
        self._keep = []
        self.thnet = abi.THNETWORK()
        self.layers = None
        lib.THFloatTensor_new.restype = C.c_void_p

    # -- tensors -------------------------------------------------------
    def _new_lib_tensor(self):
        """An empty tensor allocated by the library (it may free / resize it)."""
        p = self.lib.THFloatTensor_new()
        return C.cast(p, self.abi.PTensor)

    def tensor(self, arr):
        """A tensor struct borrowing a float32 numpy array (mustfree = 0)."""
        if arr is None:
            return self._new_lib_tensor()
        a = np.ascontiguousarray(arr, dtype=np.float32)
        st = THFloatStorage(a.ctypes.data, 1, 0)
        t = self.abi.THFloatTensor()
        t.nDimension = a.ndim
        stride = 1
        for i in range(a.ndim - 1, -1, -1):
            t.size[i] = a.shape[i]
            t.stride[i] = stride
            stride *= a.shape[i]
        t.storage = C.pointer(st)
        t.storageOffset = 0
        self._keep += [a, st, t]
        return C.pointer(t)

    def _fn(self, kind):
        if not self.resolve_cpu:
            return None
        return C.cast(getattr(self.lib, CPU_UPDATE[kind]), C.c_void_p).value

    # -- modules -------------------------------------------------------
    def _network(self, layers):
        abi = self.abi
        n = len(layers)
        mods = (abi.module * n)()
        net = abi.network()
        net.nelem = n
        net.engine = ENGINE_CPU
        net.modules = C.cast(mods, C.POINTER(abi.module))
        self._keep += [mods, net]
        pnet = C.pointer(net)
        for i, spec in enumerate(layers):
            m = mods[i]
            kind = spec["type"]
            m.updateOutput = self._fn(kind)
            m.output = self._new_lib_tensor()
            m.net = pnet
            # graph form (thapi.c:173-193): "inputs" lists the positions, in this list, of the
            # modules whose outputs this one reads
            inputs = spec.get("inputs", [])
            m.ninputs = len(inputs)
            for j, src in enumerate(inputs):
                if not 0 <= src < i:
                    raise ValueError("layer %d names input %d, which does not come before it" % (i, src))
                m.inputs[j] = src
            if kind == "conv":
                w = np.asarray(spec["weight"], dtype=np.float32)
                co, ci, kh, kw = w.shape
                m.type = MT["MT_SpatialConvolutionVirtMM" if spec.get("mm", "virt") == "virt" else "MT_SpatialConvolutionMM"]
                c = m.SpatialConvolution
                # the MM modules keep the weight 2-D [Co][Ci*kH*kW] (thapi.c:704-707)
                c.weight = self.tensor(w.reshape(co, ci * kh * kw))
                c.bias = self.tensor(spec["bias"])
                c.finput = self._new_lib_tensor()
                c.dW, c.dH, c.padW, c.padH = spec["dW"], spec["dH"], spec["padW"], spec["padH"]
                c.kW, c.kH, c.nInputPlane, c.nOutputPlane = kw, kh, ci, co
            elif kind == "linear":
                m.type = MT["MT_Linear"]
                m.Linear.weight = self.tensor(spec["weight"])
                m.Linear.bias = self.tensor(spec["bias"])
                m.Linear.addBuffer = self._new_lib_tensor()
                m.Linear.commute = 0
            elif kind == "threshold":
                m.type = MT["MT_Threshold"]
                t = m.Threshold
                t.threshold, t.val, t.alpha = spec.get("threshold", 0.0), spec.get("val", 0.0), spec.get("alpha", 0.0)
                t.inplace = spec.get("inplace", 1)
            elif kind == "maxpool":
                m.type = MT["MT_SpatialMaxPooling"]
                p = m.SpatialMaxPooling
                for k in ("kW", "kH", "dW", "dH", "padW", "padH", "ceil_mode"):
                    setattr(p, k, spec.get(k, 0))
                p.indices = self._new_lib_tensor()
            elif kind == "avgpool":
                m.type = MT["MT_SpatialAveragePooling"]
                p = m.SpatialAveragePooling
                for k in ("kW", "kH", "dW", "dH", "padW", "padH", "ceil_mode", "count_include_pad"):
                    setattr(p, k, spec.get(k, 0))
            elif kind == "view":
                m.type = MT["MT_View"]
                m.View.numElements = spec["numElements"]
                m.View.nDimension = 0
            elif kind == "softmax":
                m.type = MT["MT_SoftMax"]
            elif kind == "bn":
                m.type = MT["MT_SpatialBatchNormalization"]
                b = m.SpatialBatchNormalization
                b.running_mean = self.tensor(spec["running_mean"])
                b.running_var = self.tensor(spec["running_var"])
                b.weight = self.tensor(spec.get("weight"))
                b.bias = self.tensor(spec.get("bias"))
                b.eps = spec.get("eps", 1e-5)
            elif kind == "dropout":
                m.type = MT["MT_Dropout"]
                m.Dropout.p, m.Dropout.inplace, m.Dropout.v2 = spec.get("p", 0.5), spec.get("inplace", 1), spec.get("v2", 1)
            elif kind == "sequential":
                m.type = MT["MT_Sequential"]
                m.Sequential.net = self._network(spec["layers"])
            elif kind == "concattable":
                m.type = MT["MT_ConcatTable"]
                # each branch is one module of the table's network; a list becomes a Sequential
                branches = [b[0] if len(b) == 1 else {"type": "sequential", "layers": b} for b in spec["branches"]]
                m.ConcatTable.net = self._network(branches)
            elif kind == "fullconv":
                w = np.asarray(spec["weight"], dtype=np.float32)
                ci, co, kh, kw = w.shape
                m.type = MT["MT_SpatialFullConvolution"]
                c = m.SpatialFullConvolution
                c.weight = self.tensor(w)
                c.bias = self.tensor(spec.get("bias"))
                c.ones = self._new_lib_tensor()
                c.columns = self._new_lib_tensor()
                c.dW, c.dH, c.padW, c.padH = spec.get("dW", 1), spec.get("dH", 1), spec.get("padW", 0), spec.get("padH", 0)
                c.adjW, c.adjH = spec.get("adjW", 0), spec.get("adjH", 0)
                c.kW, c.kH, c.nInputPlane, c.nOutputPlane = kw, kh, ci, co
            elif kind == "maxunpool":
                # names its pooling (a position in this list) by that module's nnmodule tag
                m.type = MT["MT_SpatialMaxUnpooling"]
                tag = 0x7000 + spec["pooling"]
                mods[spec["pooling"]].nnmodule = tag
                m.SpatialMaxUnpooling.pooling = tag
            elif kind == "caddtable":
                m.type = MT["MT_CAddTable"]
            elif kind == "csubtable":
                m.type = MT["MT_CSubTable"]
            else:
                raise ValueError("unknown layer type %r" % kind)
        return pnet

    def build(self, layers, mean=(0.0, 0.0, 0.0), std=(1.0, 1.0, 1.0)):
        self.layers = layers
        self.thnet.net = self._network(layers)
        for i in range(3):
            self.thnet.mean[i] = mean[i]
            self.thnet.std[i] = std[i]
        return self

    @property
    def ptr(self):
        return C.pointer(self.thnet)


def tensor_to_numpy(abi, pt, dtype=np.float32, copy=True):
    """Host tensor struct -> numpy array (contiguous tensors only)."""
    t = pt.contents
    shape = tuple(t.size[i] for i in range(t.nDimension))
    n = int(np.prod(shape)) if shape else 0
    base = t.storage.contents.data + t.storageOffset * np.dtype(dtype).itemsize
    buf = (C.c_char * (n * np.dtype(dtype).itemsize)).from_address(base)
    a = np.frombuffer(buf, dtype=dtype).reshape(shape)
    return a.copy() if copy else a
