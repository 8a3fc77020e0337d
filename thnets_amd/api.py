"""Python face of the MI355X engine (``lib/libthnets_hip.so``).

Mirrors the reference's ``thnets.py`` (a ctypes wrapper around ``THInit`` /
``THLoadNetwork`` / ``THProcessFloat`` / ``THFreeNetwork``, thnets.py:11-30) for the
engine in this repository, and binds the kernel-level ``thhip_*`` C ABI for tests
and the benchmark.  There is no CPU fallback: loading fails loudly when the
library has not been built, and the library itself aborts when no GPU is visible.
"""
import ctypes as C
import os

import numpy as np

from . import abi
from .netbuild import HostNetwork

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "lib", "libthnets_hip.so")

_lib = None

c_fp = C.POINTER(C.c_float)
c_ip = C.POINTER(C.c_int)
vp = C.c_void_p

# Test and tuning hooks (process-wide switches of the kernel choice): exported by the library,
# declared in csrc/thhip_internal.h, not in the installed header.
TEST_HOOKS = {
    "thhip_conv_set_ktile": (None, [C.c_int]),
    "thhip_conv_set_tail_parts": (None, [C.c_int]),
    "thhip_xcd_map": (C.c_uint, []),
    "thhip_windowed_forwards": (C.c_long, []),
    "thhip_fault_flag": (C.POINTER(C.c_int), []),
    "thhip_conv_cut_launches": (C.c_long, [C.c_int]),
    "thhip_conv_set_xcd_parts": (None, [C.c_int]),
    "thhip_conv_set_generic_cl": (None, [C.c_int]),
    "thhip_linear_batched_set_tuning": (None, [C.c_int]),
    "thhip_conv_set_tuning": (None, [C.c_int, C.c_int, C.c_int, C.c_int]),
}

# name -> (restype, argtypes); every symbol include/thnets_hip.h declares
PROTOTYPES = {
    "THError": (None, None),
    "THFloatTensor_new": (vp, []),
    "THFloatStorage_new": (vp, [C.c_long]),
    "THFloatStorage_newwithbuffer": (vp, [vp]),
    "THFloatTensor_newWithStorage1d": (vp, [vp, C.c_long, C.c_long, C.c_long]),
    "THFloatTensor_newWithStorage2d": (vp, [vp, C.c_long, C.c_long, C.c_long, C.c_long, C.c_long]),
    "THFloatTensor_newWithTensor": (vp, [vp]),
    "THFloatTensor_data": (vp, [vp]),
    "THFloatTensor_nElement": (C.c_long, [vp]),
    "THFloatTensor_resize": (None, [vp, C.POINTER(C.c_long), C.c_int]),
    "THFloatTensor_resize4d": (None, [vp] + [C.c_long] * 4),
    "THFloatTensor_resize3d": (None, [vp] + [C.c_long] * 3),
    "THFloatTensor_resize2d": (None, [vp] + [C.c_long] * 2),
    "THFloatTensor_resize1d": (None, [vp, C.c_long]),
    "THFloatTensor_set": (None, [vp, vp]),
    "THFloatTensor_free": (None, [vp]),
    "THInit": (None, []),
    "THForward": (vp, [vp, vp]),
    "THProcessFloat": (C.c_int, [vp, vp, C.c_int, C.c_int, C.c_int, C.c_int, C.POINTER(c_fp), c_ip, c_ip]),
    "THProcessImages": (C.c_int, [vp, C.POINTER(vp), C.c_int, C.c_int, C.c_int, C.c_int, C.POINTER(c_fp), c_ip, c_ip,
                                  C.c_int]),
    "THMakeSpatial": (None, [vp, C.c_int]),
    "THUseSpatialConvolutionMM": (C.c_int, [vp, C.c_int]),
    "THFreeNetwork": (None, [vp]),
    "THLoadNetwork": (vp, [C.c_char_p]),
    "THLoadTensor": (vp, [C.c_char_p]),
    "THLastError": (C.c_int, []),
    "THCreateHipNetwork": (vp, [vp]),
    "THHipHalfFloat": (C.c_int, [C.c_int]),
    "THHipFoldBatchNorm": (C.c_int, [C.c_int]),
    "THHipImageLayerInFront": (C.c_int, [C.c_int]),
    "THHipSumPartsInKernel": (C.c_int, [C.c_int]),
    "THHipTableArithmetic": (C.c_int, [C.c_int]),
    "THCreateHipLowpNetwork": (vp, [vp, C.c_float]),
    "THHipTensor_newFromFloatTensor": (vp, [vp]),
    "THFloatTensor_newFromHipTensor": (vp, [vp]),
    "THHipNetwork_copyModuleOutput": (C.c_long, [vp, C.c_int, C.POINTER(c_fp), C.POINTER(C.c_long), c_ip]),
    "THHipNetwork_getModuleQuant": (C.c_int, [vp, C.c_int, c_fp, c_fp]),
    "THHipNetwork_setInputQuant": (C.c_int, [vp, C.c_float, C.c_float]),
    "THHipLowpTensor_newFromFloatTensor": (vp, [vp, vp]),
    "lowpgemm": (None, [C.c_int] * 6 + [vp, vp, vp] + [C.c_int] * 8),
    "thhip_device_count": (C.c_int, []),
    "thhip_malloc": (vp, [C.c_size_t]),
    "thhip_free": (None, [vp]),
    "thhip_memcpy_h2d": (None, [vp, vp, C.c_size_t]),
    "thhip_memcpy_d2h": (None, [vp, vp, C.c_size_t]),
    "thhip_memcpy_d2d": (None, [vp, vp, C.c_size_t]),
    "thhip_alloc_calls": (C.c_long, []),
    "thhip_host_malloc": (vp, [C.c_size_t]),
    "thhip_host_free": (None, [vp]),
    "thhip_memcpy_h2d_async": (None, [vp, vp, C.c_size_t]),
    "thhip_memcpy_d2h_async": (None, [vp, vp, C.c_size_t]),
    "thhip_memset": (None, [vp, C.c_int, C.c_size_t]),
    "thhip_sync": (None, []),
    "thhip_event_record": (None, [C.c_int]),
    "thhip_event_ms": (C.c_float, [C.c_int, C.c_int]),
    "thhip_profile_enable": (None, [C.c_int]),
    "thhip_profile_reset": (None, []),
    "thhip_profile_get": (None, [C.c_int, C.POINTER(C.c_double), C.POINTER(C.c_long), C.POINTER(C.c_double)]),
    "thhip_probe_mfma": (C.c_double, [C.c_int, C.c_int, C.c_double]),
    "thhip_conv_pack_weight": (vp, [vp, C.c_int, C.c_int, C.c_int, C.c_int]),
    "thhip_conv_packed_bytes": (C.c_size_t, [C.c_int, C.c_int, C.c_int, C.c_int]),
    "thhip_conv_unpack_rows": (vp, [vp, C.c_int, C.c_int, C.c_int, C.c_int]),
    "thhip_conv2d": (None, [vp, vp, vp, vp] + [C.c_int] * 11 + [C.c_int, C.c_float, C.c_float, C.c_int]),
    "thhip_conv_pack_weight_layout": (vp, [vp, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int]),
    "thhip_conv2d_layout": (None, [vp, vp, vp, vp, vp] + [C.c_int] * 11 + [C.c_int, C.c_float, C.c_float, C.c_int, C.c_int, C.c_int]),
    "thhip_relayout": (None, [vp, vp] + [C.c_int] * 5),
    "thhip_maxpool_cl": (None, [vp, vp] + [C.c_int] * 13),
    "thhip_conv2d_image_pool_supported": (C.c_int, [C.c_int] * 20),
    "thhip_conv2d_image_pool": (None, [vp, vp, vp, vp, vp] + [C.c_int] * 12 + [C.c_int, C.c_float, C.c_float, C.c_int]),
    "thhip_conv_pair_begin": (None, []),
    "thhip_conv_pair_end": (None, []),
    "thhip_conv_pack_weight_image_front": (vp, [vp, C.c_int]),
    "thhip_conv2d_image_pair_supported": (C.c_int, [C.c_int] * 7),
    "thhip_conv2d_image_pair": (None, [vp, vp, vp, vp, C.c_int, C.c_float, C.c_float, vp, vp, vp, vp] + [C.c_int] * 5 +
                                [C.c_float, C.c_float, C.c_int, C.c_int]),
    "thhip_conv2d_affine": (None, [vp, vp, vp, vp, vp] + [C.c_int] * 11 + [C.c_int, C.c_float, C.c_float, C.c_int]),
    "thhip_maxpool_indices": (None, [vp, vp, vp] + [C.c_int] * 13),
    "thhip_maxunpool": (None, [vp, vp, vp] + [C.c_int] * 13),
    "thhip_fullconv_pack_weight": (vp, [vp] + [C.c_int] * 5),
    "thhip_fullconv2d": (None, [vp, vp, vp, C.c_float, vp, vp] + [C.c_int] * 14 + [C.c_float, C.c_float, C.c_int]),
    "thhip_col2im": (None, [vp, vp, C.c_float, vp] + [C.c_int] * 13 + [C.c_float, C.c_float, C.c_int]),
    "thhip_normalize": (None, [vp, vp, C.c_int, C.c_int, C.c_long, vp, vp, C.c_int]),
    "thhip_gemv": (None, [vp, vp, vp, vp, C.c_int, C.c_int, C.c_int, C.c_float, C.c_float, C.c_int]),
    "thhip_linear_batched_supported": (C.c_int, [C.c_int] * 4),
    "thhip_linear_batched": (None, [vp, vp, vp, vp, C.c_int, C.c_int, C.c_int, C.c_int, C.c_float, C.c_float, C.c_int]),
    "thhip_linear_batched_noalloc": (C.c_int, [vp, vp, vp, vp, C.c_int, C.c_int, C.c_int, C.c_int, C.c_float, C.c_float, C.c_int]),
    "thhip_linear_batched_noalloc_init": (C.c_int, []),
    "thhip_linear_batched_noalloc_limit": (C.c_size_t, []),
    "thhip_minmax": (None, [vp, C.c_long, C.c_int, c_fp, c_fp]),
    "thhip_threshold": (None, [vp, vp, C.c_long, C.c_float, C.c_float, C.c_float, C.c_int, C.c_int]),
    "thhip_maxpool": (None, [vp, vp] + [C.c_int] * 13),
    "thhip_pool_outsize": (None, [C.c_int] * 9 + [c_ip, c_ip]),
    "thhip_avgpool": (None, [vp, vp] + [C.c_int] * 14),
    "thhip_softmax": (None, [vp, vp, C.c_long, C.c_long, C.c_long, C.c_int]),
    "thhip_batchnorm": (None, [vp, vp, C.c_long, C.c_long, C.c_long, vp, vp, vp, vp, C.c_int]),
    "thhip_axpby2": (None, [vp, vp, vp, C.c_long, C.c_long, C.c_float, C.c_int, C.c_int]),
    "thhip_convert": (None, [vp, C.c_int, vp, C.c_int, C.c_long]),
    "thhip_rgb2float": (None, [vp, vp, C.c_int, C.c_int, C.c_int, C.c_int, vp, vp, C.c_int, C.c_int]),
    "thhip_rgb2float_batch": (None, [vp, vp, C.c_int, C.c_long, C.c_int, C.c_int, C.c_int, C.c_int, vp, vp, C.c_int, C.c_int]),
    "thhip_quantize": (None, [vp, vp, C.c_long, c_fp, c_fp]),
    "thhip_dequantize": (None, [vp, vp, C.c_long, C.c_float, C.c_float]),
    "thhip_conv_pack_weight_u8": (vp, [vp, C.c_int, C.c_int, C.c_int]),
    "thhip_conv2d_u8": (None, [vp, vp, vp, vp] + [C.c_int] * 11 + [C.c_int] * 6 + [C.c_int] * 3),
    "thhip_conv_pack_weight_u8_layout": (vp, [vp, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int]),
    "thhip_conv2d_u8_layout": (None, [vp, vp, vp, vp] + [C.c_int] * 11 + [C.c_int] * 6 + [C.c_int] * 3 + [C.c_int] * 2),
    "thhip_conv2d_pool2_supported": (C.c_int, [C.c_int] * 14),
    "thhip_conv2d_poolk_supported": (C.c_int, [C.c_int] * 19),
    "thhip_conv2d_poolk": (None, [vp, vp, vp, vp, vp] + [C.c_int] * 18 + [C.c_int, C.c_float, C.c_float, C.c_int]),
    "thhip_conv2d_residual_supported": (C.c_int, [C.c_int] * 12),
    "thhip_conv2d_residual": (None, [vp, vp, vp, vp, vp, C.c_int, C.c_float, C.c_int, vp] + [C.c_int] * 11 +
                              [C.c_int, C.c_float, C.c_float, C.c_int]),
    "thhip_conv2d_layout_pool2": (None, [vp, vp, vp, vp, vp] + [C.c_int] * 11 + [C.c_int, C.c_float, C.c_float, C.c_int, C.c_int, C.c_int]),
    "thhip_conv2d_u8_layout_tail": (None, [vp, vp, vp, vp] + [C.c_int] * 11 + [C.c_int] * 6 + [C.c_int] * 3 + [C.c_int] * 3),
    "thhip_conv2d_u8_image_pool_supported": (C.c_int, [C.c_int] * 18),
    "thhip_conv2d_u8_image_pool": (None, [vp, vp, vp, vp] + [C.c_int] * 11 + [C.c_int] * 6 + [C.c_int] * 3),
    "thhip_conv2d_u8_patch_supported": (C.c_int, [C.c_int] * 12),
    "thhip_conv_pack_weight_u8_patch": (vp, [vp, C.c_int, C.c_int, C.c_int, C.c_int]),
    "thhip_conv2d_u8_patch": (None, [vp, vp, vp, vp] + [C.c_int] * 11 + [C.c_int] * 6 + [C.c_int] * 3 + [C.c_int]),
    "thhip_maxpool_u8_cl": (None, [vp, vp] + [C.c_int] * 12),
    "thhip_relayout_u8": (None, [vp, vp] + [C.c_int] * 4),
    "thhip_linear_batched_u8_supported": (C.c_int, [C.c_int] * 3),
    "thhip_u8_rowsums": (vp, [vp, C.c_int, C.c_int]),
    "thhip_linear_pack_weight_u8": (vp, [vp, C.c_int, C.c_int]),
    "thhip_linear_batched_u8": (None, [vp, vp, vp, vp, vp] + [C.c_int] * 3 + [C.c_int] * 5 + [C.c_int] * 3),
    "thhip_rgb2code": (None, [vp, vp, C.c_int, C.c_int, C.c_int, vp, vp, C.c_int, c_fp, c_fp]),
    "thhip_rgb2code_batch": (None, [vp, vp, C.c_int, C.c_long, C.c_int, C.c_int, C.c_int, vp, vp, C.c_int, c_fp, c_fp]),
    "thhip_threshold_u8": (None, [vp, vp, C.c_long, C.c_int, C.c_int, C.c_int]),
    "thhip_softmax_u8": (C.c_float, [vp, vp, C.c_long, C.c_long, C.c_long, C.c_float, C.c_float]),
}


def load_library(path=LIB_PATH):
    """dlopen the engine and attach prototypes.  No GPU is touched."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(path):
        raise RuntimeError(
            "%s is missing: build it with `make -C thnets_amd/csrc` (or __graft_entry__.build()); "
            "this package has no CPU fallback" % path)
    lib = C.CDLL(path)
    for name, (res, args) in list(PROTOTYPES.items()) + list(TEST_HOOKS.items()):
        fn = getattr(lib, name)
        if args is not None:
            fn.restype = res
            fn.argtypes = args
    _lib = lib
    return lib


def _np_dtype(dt):
    return {abi.THHIP_F32: np.float32, abi.THHIP_F16: np.float16, abi.THHIP_U8: np.uint8}[dt]


def _bf16_bits(a):
    """float32 -> bfloat16 bit patterns, round to nearest even."""
    u = np.ascontiguousarray(a, np.float32).view(np.uint32).astype(np.uint64)
    return ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)


class DeviceArray:
    """A device buffer holding a numpy array's bytes (tests and benchmarks)."""

    def __init__(self, lib, arr=None, nbytes=None):
        self.lib = lib
        self.nbytes = int(arr.nbytes if arr is not None else nbytes)
        self.ptr = lib.thhip_malloc(self.nbytes)
        if arr is not None:
            a = np.ascontiguousarray(arr)
            lib.thhip_memcpy_h2d(self.ptr, a.ctypes.data, a.nbytes)

    def get(self, shape, dtype):
        out = np.empty(shape, dtype)
        assert out.nbytes <= self.nbytes
        self.lib.thhip_memcpy_d2h(out.ctypes.data, self.ptr, out.nbytes)
        return out

    def free(self):
        if self.ptr:
            self.lib.thhip_free(self.ptr)
            self.ptr = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


def to_device_dtype(lib, arr, dtype):
    """Host float32 array -> DeviceArray in the engine dtype."""
    a = np.ascontiguousarray(arr, np.float32)
    if dtype == abi.THHIP_F32:
        return DeviceArray(lib, a)
    if dtype == abi.THHIP_F16:
        return DeviceArray(lib, a.astype(np.float16))
    if dtype == abi.THHIP_BF16:
        return DeviceArray(lib, _bf16_bits(a))
    raise ValueError(dtype)


def from_device_dtype(dev, shape, dtype):
    if dtype == abi.THHIP_F32:
        return dev.get(shape, np.float32)
    if dtype == abi.THHIP_F16:
        return dev.get(shape, np.float16).astype(np.float32)
    if dtype == abi.THHIP_BF16:
        bits = dev.get(shape, np.uint16).astype(np.uint32) << 16
        return bits.view(np.float32)
    if dtype == abi.THHIP_U8:
        return dev.get(shape, np.uint8)
    raise ValueError(dtype)


class HipNetwork:
    """A network on the engine, made from a layer list (see netbuild) or from a
    Torch7 model directory (``model.net`` + ``stat.t7``, read by ``THLoadNetwork``)."""

    def __init__(self, layers, mean=(0.0, 0.0, 0.0), std=(1.0, 1.0, 1.0), half=0, lowp_range=None,
                 make_spatial=None, fold_bn=True):
        self.lib = lib = load_library()
        lib.THInit()
        loaded = None
        if isinstance(layers, (str, bytes, os.PathLike)):
            loaded = lib.THLoadNetwork(os.fsencode(layers))
            if not loaded:
                raise IOError("THLoadNetwork(%r) failed: error %d" % (layers, lib.THLastError()))
            self.host = HostNetwork(lib, abi.ABI, resolve_cpu=False)      # only makes host tensors for upload()
            source = loaded
        else:
            self.host = HostNetwork(lib, abi.ABI, resolve_cpu=False).build(layers, mean, std)
            source = C.addressof(self.host.thnet)
        if make_spatial:
            lib.THMakeSpatial(source, int(make_spatial))
        self.half = half
        self.lowp = lowp_range is not None
        if self.lowp:
            self.handle = lib.THCreateHipLowpNetwork(source, C.c_float(lowp_range))
            self.dtype = abi.THHIP_U8
        else:
            if lib.THHipHalfFloat(half) != 0:
                raise ValueError("THHipHalfFloat(%r) refused" % half)
            old_fold = lib.THHipFoldBatchNorm(1 if fold_bn else 0)
            self.handle = lib.THCreateHipNetwork(source)
            lib.THHipFoldBatchNorm(old_fold)
            lib.THHipHalfFloat(0)
            self.dtype = (abi.THHIP_F32, abi.THHIP_F16, abi.THHIP_BF16)[half]
        if loaded:
            lib.THFreeNetwork(loaded)      # the engine copied what it needs (thnets-test.c:130-134)
        self.thnet = C.cast(self.handle, C.POINTER(abi.ABI.THNETWORK)).contents
        self._dev_in = None

    @property
    def nelem(self):
        return self.thnet.net.contents.nelem

    def process_float(self, x):
        """THProcessFloat on a copy of x ([B,C,H,W] float32); returns the flat result."""
        x = np.array(x, np.float32, copy=True, order="C")
        B, Cn, H, W = x.shape
        res = c_fp()
        ow, oh = C.c_int(), C.c_int()
        n = self.lib.THProcessFloat(self.handle, x.ctypes.data, B, W, H, Cn, C.byref(res), C.byref(ow), C.byref(oh))
        return np.ctypeslib.as_array(res, shape=(n,)).copy()

    def process_images(self, images, bgr=0):
        """THProcessImages on a list of uint8 [H][W][3] (or [H][W]) arrays."""
        imgs = [np.ascontiguousarray(im, np.uint8) for im in images]
        H, W = imgs[0].shape[:2]
        cp = 1 if imgs[0].ndim == 2 else imgs[0].shape[2]
        ptrs = (vp * len(imgs))(*[im.ctypes.data for im in imgs])
        res = c_fp()
        ow, oh = C.c_int(), C.c_int()
        n = self.lib.THProcessImages(self.handle, ptrs, len(imgs), W, H, W * cp, C.byref(res), C.byref(ow),
                                     C.byref(oh), bgr)
        return np.ctypeslib.as_array(res, shape=(n,)).copy()

    def upload(self, x):
        """Host float32 (already normalised) -> device tensor in the engine dtype
        (quantised on the device for a uint8 network); kept alive by this object and
        reused by forward()."""
        x = np.ascontiguousarray(x, np.float32)
        t = self.host.tensor(x)
        if self.lowp:
            dev = self.lib.THHipLowpTensor_newFromFloatTensor(self.handle, C.addressof(t.contents))
        else:
            self.lib.THHipHalfFloat(self.half)
            dev = self.lib.THHipTensor_newFromFloatTensor(C.addressof(t.contents))
            self.lib.THHipHalfFloat(0)
        if self._dev_in:
            self.lib.THFloatTensor_free(self._dev_in)
        self._dev_in = dev
        return dev

    def forward(self, dev=None):
        """THForward on a device tensor: kernels only, no host transfers."""
        return self.lib.THForward(self.handle, dev or self._dev_in)

    def module_output(self, idx):
        res = c_fp()
        size = (C.c_long * 4)()
        nd = C.c_int()
        n = self.lib.THHipNetwork_copyModuleOutput(self.handle, idx, C.byref(res), size, C.byref(nd))
        a = np.ctypeslib.as_array(res, shape=(n,)).copy().reshape([size[i] for i in range(nd.value)])
        C.CDLL(None).free(res)
        return a

    def module_quant(self, idx):
        m, s = C.c_float(), C.c_float()
        if self.lib.THHipNetwork_getModuleQuant(self.handle, idx, C.byref(m), C.byref(s)):
            raise ValueError("not a uint8 network")
        return m.value, s.value

    def free(self):
        if self.handle:
            if self._dev_in:
                self.lib.THFloatTensor_free(self._dev_in)
                self._dev_in = None
            self.lib.THFreeNetwork(self.handle)
            self.handle = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


class thnets:
    """Drop-in for the class in the reference's thnets.py, over the HIP engine.
    ``LoadNetwork`` takes a Torch7 model directory, as there, or a layer list."""

    def __init__(self):
        self.net = None

    def LoadNetwork(self, layers, mean=(0.0, 0.0, 0.0), std=(1.0, 1.0, 1.0), **kw):
        self.net = HipNetwork(layers, mean, std, **kw)

    def ProcessFloat(self, image):
        """image: float32 [C][H][W], as in thnets.py:20-30 (batch of one)."""
        if self.net is None:
            return None
        image = np.asarray(image, np.float32)
        return self.net.process_float(image[None])

    def FreeNetwork(self):
        if self.net is not None:
            self.net.free()
        self.net = None
