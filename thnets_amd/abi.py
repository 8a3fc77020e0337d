"""ctypes mirror of the thnets C ABI for the conv / Linear / LOWP path.

The same structures drive two libraries:

* this repository's engine (``include/thnets_hip.h``), and
* the reference's own CPU library when a test-side build of it exists,

which is what lets a parity test hand byte-identical ``struct module`` arrays to
both.  Layout follows thnets.h:104-120 (tensor / storage), :122-232 (per-module
parameter blocks), :250-336 (``enum moduletype`` / ``struct module``), :401-407
(``struct network``) and :571-580 (``THNETWORK``) of the reference.  ``lowp=True``
adds the ``sub, mult`` members a ``-DLOWP`` build of the reference appends to
``THFloatTensor`` (thnets.h:117-119); the engine in this repository always uses
the default layout.
"""
import ctypes as C

MAXMODULEINPUTS = 16
MODULE_UNION_BYTES = 80

# enum moduletype, thnets.h:250-288
MODULE_TYPES = [
    "MT_Nil", "MT_SpatialConvolutionMM", "MT_SpatialConvolutionVirtMM", "MT_SpatialConvolution",
    "MT_SpatialMaxPooling", "MT_SpatialAveragePooling", "MT_Linear", "MT_SoftMax", "MT_Threshold",
    "MT_View", "MT_Dropout", "MT_SpatialZeroPadding", "MT_Reshape", "MT_Normalize",
    "MT_SpatialFullConvolution", "MT_SpatialMaxUnpooling", "MT_SpatialBatchNormalization",
    "MT_Sequential", "MT_Concat", "MT_ConcatTable", "MT_JoinTable", "MT_CAddTable", "MT_CSubTable",
    "MT_PReLU", "MT_Identity", "MT_Padding", "MT_LogSoftMax", "MT_Slice", "MT_Cmax", "MT_Upsample",
    "MT_LSTM", "MT_GRU", "MT_Squeeze", "MT_Unsqueeze", "MT_Sigmoid", "MT_Tanh", "MT_Transpose",
]
MT = {name: i for i, name in enumerate(MODULE_TYPES)}

# engine ids, thnets.h:401 plus the two engines this repository appends
ENGINE_CPU, ENGINE_CUDA, ENGINE_OPENCL, ENGINE_OPENCLINIT, ENGINE_LOWP, ENGINE_HIP, ENGINE_HIPLOWP = range(7)

# enum thhip_dtype
THHIP_F32, THHIP_F16, THHIP_BF16, THHIP_U8 = range(4)
# THFloatStorage.mustfree of device memory owned by the engine: 4 + the element type it holds
TH_MUSTFREE_HIP = 4


class THFloatStorage(C.Structure):
    _fields_ = [("data", C.c_void_p), ("nref", C.c_int), ("mustfree", C.c_int)]


def _tensor_type(lowp):
    fields = [
        ("size", C.c_long * 4),
        ("stride", C.c_long * 4),
        ("nDimension", C.c_int),
        ("storage", C.POINTER(THFloatStorage)),
        ("storageOffset", C.c_long),
    ]
    if lowp:
        fields += [("sub", C.c_float), ("mult", C.c_float)]
    return type("THFloatTensorLowp" if lowp else "THFloatTensor", (C.Structure,), {"_fields_": fields})


class Abi:
    """All structure types for one tensor layout (default or -DLOWP)."""

    def __init__(self, lowp=False):
        self.lowp = lowp
        T = self.THFloatTensor = _tensor_type(lowp)
        PT = self.PTensor = C.POINTER(T)

        class SpatialConvolution(C.Structure):
            _fields_ = [("bias", PT), ("weight", PT), ("finput", PT)] + [
                (n, C.c_int) for n in ("dW", "dH", "padW", "padH", "kW", "kH", "nInputPlane", "nOutputPlane",
                                       "refl_pad", "padW2", "padH2", "autopad", "dlH", "dlW")]

        class SpatialFullConvolution(C.Structure):
            _fields_ = [("bias", PT), ("weight", PT)] + [
                (n, C.c_int) for n in ("dW", "dH", "padW", "padH", "kW", "kH", "nInputPlane", "nOutputPlane",
                                       "adjW", "adjH")] + [("ones", PT), ("columns", PT)]

        class SpatialMaxUnpooling(C.Structure):
            _fields_ = [("pooling", C.c_void_p)]

        class SpatialMaxPooling(C.Structure):
            _fields_ = [(n, C.c_int) for n in ("padW", "padH", "dW", "dH", "kW", "kH", "ceil_mode",
                                               "iwidth", "iheight")] + [("indices", PT)] + [
                (n, C.c_int) for n in ("padW2", "padH2")]

        class SpatialAveragePooling(C.Structure):
            _fields_ = [(n, C.c_int) for n in ("padW", "padH", "dW", "dH", "kW", "kH", "ceil_mode", "iwidth",
                                               "iheight", "count_include_pad", "padW2", "padH2")]

        class Linear(C.Structure):
            _fields_ = [("bias", PT), ("weight", PT), ("addBuffer", PT), ("commute", C.c_int)]

        class Threshold(C.Structure):
            _fields_ = [("threshold", C.c_float), ("val", C.c_float), ("alpha", C.c_float), ("inplace", C.c_int)]

        class View(C.Structure):
            _fields_ = [("numElements", C.c_int), ("nDimension", C.c_int), ("size", C.c_long * 4)]

        class Dropout(C.Structure):
            _fields_ = [("p", C.c_float), ("inplace", C.c_int), ("v2", C.c_int)]

        class SpatialBatchNormalization(C.Structure):
            _fields_ = [("running_mean", PT), ("running_var", PT), ("weight", PT), ("bias", PT),
                        ("eps", C.c_double)]

        class network(C.Structure):
            pass

        class Sequential(C.Structure):
            _fields_ = [("net", C.POINTER(network))]

        class Concat(C.Structure):
            _fields_ = [("net", C.POINTER(network)), ("dimension", C.c_int)]

        class ModuleUnion(C.Union):
            _fields_ = [
                ("SpatialConvolution", SpatialConvolution),
                ("SpatialFullConvolution", SpatialFullConvolution),
                ("SpatialMaxUnpooling", SpatialMaxUnpooling),
                ("SpatialMaxPooling", SpatialMaxPooling),
                ("SpatialAveragePooling", SpatialAveragePooling),
                ("Linear", Linear),
                ("Threshold", Threshold),
                ("View", View),
                ("Dropout", Dropout),
                ("SpatialBatchNormalization", SpatialBatchNormalization),
                ("Sequential", Sequential),
                ("Concat", Concat),
                ("ConcatTable", Sequential),
                ("abi_pad", C.c_char * MODULE_UNION_BYTES),
            ]

        class module(C.Structure):
            _anonymous_ = ("u",)
            _fields_ = [
                ("type", C.c_int),
                ("updateOutput", C.c_void_p),
                ("nnfree", C.c_void_p),
                ("output", PT),
                ("net", C.POINTER(network)),
                ("nnmodule", C.c_void_p),
                ("outputname", C.c_char_p),
                ("ninputs", C.c_int),
                ("inputs", C.c_int * MAXMODULEINPUTS),
                ("u", ModuleUnion),
            ]

        network._fields_ = [("nelem", C.c_int), ("engine", C.c_int), ("modules", C.POINTER(module))]

        class THNETWORK(C.Structure):
            _fields_ = [
                ("netobj", C.c_void_p),
                ("statobj", C.c_void_p),
                ("net", C.POINTER(network)),
                ("pynet", C.c_void_p),
                ("allpynodes", C.c_void_p),
                ("out", PT),
                ("mean", C.c_float * 3),
                ("std", C.c_float * 3),
            ]

        self.SpatialConvolution = SpatialConvolution
        self.SpatialMaxPooling = SpatialMaxPooling
        self.SpatialFullConvolution = SpatialFullConvolution
        self.SpatialMaxUnpooling = SpatialMaxUnpooling
        self.SpatialAveragePooling = SpatialAveragePooling
        self.Linear = Linear
        self.Threshold = Threshold
        self.View = View
        self.Dropout = Dropout
        self.SpatialBatchNormalization = SpatialBatchNormalization
        self.Sequential = Sequential
        self.Concat = Concat
        self.ModuleUnion = ModuleUnion
        self.module = module
        self.network = network
        self.THNETWORK = THNETWORK

    def layout(self):
        """sizeof / offsetof table used by the ABI tests."""
        m, t, n, s = self.module, self.THFloatTensor, self.THNETWORK, self.SpatialConvolution
        return {
            "sizeof_THFloatStorage": C.sizeof(THFloatStorage),
            "sizeof_THFloatTensor": C.sizeof(t),
            "off_tensor_nDimension": t.nDimension.offset,
            "off_tensor_storage": t.storage.offset,
            "off_tensor_storageOffset": t.storageOffset.offset,
            "sizeof_module": C.sizeof(m),
            "off_module_updateOutput": m.updateOutput.offset,
            "off_module_output": m.output.offset,
            "off_module_net": m.net.offset,
            "off_module_outputname": m.outputname.offset,
            "off_module_inputs": m.inputs.offset,
            "off_module_union": m.u.offset,
            "sizeof_SpatialConvolution": C.sizeof(s),
            "off_conv_dW": s.dW.offset,
            "off_conv_nOutputPlane": s.nOutputPlane.offset,
            "sizeof_SpatialFullConvolution": C.sizeof(self.SpatialFullConvolution),
            "off_fullconv_adjW": self.SpatialFullConvolution.adjW.offset,
            "off_fullconv_ones": self.SpatialFullConvolution.ones.offset,
            "sizeof_SpatialMaxPooling": C.sizeof(self.SpatialMaxPooling),
            "off_maxpool_indices": self.SpatialMaxPooling.indices.offset,
            "sizeof_SpatialBatchNormalization": C.sizeof(self.SpatialBatchNormalization),
            "off_bn_eps": self.SpatialBatchNormalization.eps.offset,
            "sizeof_Linear": C.sizeof(self.Linear),
            "sizeof_Threshold": C.sizeof(self.Threshold),
            "sizeof_View": C.sizeof(self.View),
            "sizeof_network": C.sizeof(self.network),
            "off_network_modules": self.network.modules.offset,
            "sizeof_THNETWORK": C.sizeof(n),
            "off_thnetwork_net": n.net.offset,
            "off_thnetwork_out": n.out.offset,
            "off_thnetwork_mean": n.mean.offset,
            "off_thnetwork_std": n.std.offset,
        }


ABI = Abi(lowp=False)
ABI_LOWP = Abi(lowp=True)
