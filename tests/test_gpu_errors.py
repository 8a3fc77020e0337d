"""Failure paths of the engine, forced from the host: a fatal error is THError's message on
stderr and exit(-1) (thbasic.c:172-181), so each case runs in a child process.  No kernel
is launched with bad arguments: every check fires on the host first.  Also the per-layer
range printout of th_minmax (thapi.c:197-202)."""
import ctypes as C
import os
import subprocess
import sys

import numpy as np
import pytest

import cases
import gpu_util as G
from thnets_amd import abi, api

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

PRELUDE = r"""
import sys
sys.path.insert(0, %r)
sys.path.insert(0, %r)
import ctypes as C
import numpy as np
import cases
from thnets_amd import api, abi, netbuild
lib = api.load_library()
lib.THInit()
cfg = cases.small_networks()["tiny_cnn"]
""" % (ROOT, os.path.join(ROOT, "tests"))


def child(body):
    r = subprocess.run([sys.executable, "-c", PRELUDE + body + "\nprint('survived')\n"], capture_output=True, text=True,
                       timeout=180)
    return r


def fatal(body, message):
    G.note("fatal path: " + message)
    r = child(body)
    assert r.returncode == 255 and "survived" not in r.stdout, (r.returncode, r.stdout, r.stderr)
    assert message in r.stderr, r.stderr


def test_unsupported_module_types_are_fatal():
    """cudnn_basic.c:189-303: an engine refuses the module types it cannot run when the
    network is converted, not when it runs."""
    for name in ("MT_Concat", "MT_SpatialZeroPadding", "MT_JoinTable"):
        fatal(r"""
host = netbuild.HostNetwork(lib).build(cfg["layers"], cfg["mean"], cfg["std"])
host.thnet.net.contents.modules[1].type = abi.MT[%r]
lib.THCreateHipNetwork(C.addressof(host.thnet))
""" % name, "module type %d is not supported by the HIP engine" % abi.MT[name])
    # the uint8 engine's own list (lowp_basic.c:164-208)
    fatal(r"""
layers = cfg["layers"][:3] + [{"type": "avgpool", "kW": 2, "kH": 2, "dW": 2, "dH": 2, "padW": 0, "padH": 0, "ceil_mode": 0,
                               "count_include_pad": 1}]
host = netbuild.HostNetwork(lib).build(layers)
lib.THCreateHipLowpNetwork(C.addressof(host.thnet), C.c_float(16.0))
""", "MT_SpatialAveragePooling not supported in lowp")


def test_wrong_inputs_are_fatal():
    # a host tensor where a device tensor is expected
    fatal(r"""
net = api.HipNetwork(cfg["layers"], cfg["mean"], cfg["std"])
t = net.host.tensor(cfg["input"])
lib.THForward(net.handle, C.addressof(t.contents))
""", "module input is not a device tensor")
    # a device tensor of another element type: made under THHipHalfFloat(1), given to an fp32 network
    fatal(r"""
net = api.HipNetwork(cfg["layers"], cfg["mean"], cfg["std"])
t = net.host.tensor(cfg["input"])
lib.THHipHalfFloat(1)
dev = lib.THHipTensor_newFromFloatTensor(C.addressof(t.contents))
lib.THHipHalfFloat(0)
lib.THForward(net.handle, dev)
""", "device tensor holds fp16 elements, fp32 expected")
    # planes that do not match the first convolution
    fatal(r"""
net = api.HipNetwork(cfg["layers"], cfg["mean"], cfg["std"])
net.process_float(np.zeros((1, 4, 8, 8), np.float32))
""", "nInputPlane 3 does not match input planes 4")
    # an image smaller than the kernel (SpatialConvolutionMM.c:162-164)
    fatal(r"""
w = np.zeros((4, 3, 5, 5), np.float32)
net = api.HipNetwork([netbuild.conv(w, None, 1, 0)])
net.process_float(np.zeros((1, 3, 3, 3), np.float32))
""", "Output size is too small")
    # a CPU network handed to THProcessFloat: this library carries no CPU path
    fatal(r"""
host = netbuild.HostNetwork(lib).build(cfg["layers"], cfg["mean"], cfg["std"])
x = np.zeros((1, 3, 8, 8), np.float32)
res = api.c_fp(); ow = C.c_int(); oh = C.c_int()
lib.THProcessFloat(C.addressof(host.thnet), x.ctypes.data, 1, 8, 8, 3, C.byref(res), C.byref(ow), C.byref(oh))
""", "it carries no CPU path")


def test_a_fault_reported_by_a_kernel_is_fatal_where_nothing_can_be_repeated():
    """A kernel that adds the K parts of cut tiles through its XCD's L2 reports, through a flag in page-locked
    host memory, when the workgroups of its launch were not handed to the XCDs in one order (hip_rt.hip).  The report is
    forced from the host here (no kernel misbehaves): at a plain synchronisation it is a fatal error that says
    what to do."""
    fatal(r"""
lib.thhip_fault_flag()[0] = 1
lib.thhip_sync()
""", "a kernel reported fault 1")


def test_a_fault_reported_by_a_kernel_makes_THProcessFloat_repeat_the_forward(hiplib, oracle):
    """The same report during THProcessFloat / THProcessImages: the path that raised it is switched off
    (THHipSumPartsInKernel reads 0 afterwards), the forward pass runs once more and the call returns the
    same values as without the report."""
    cfg = cases.small_networks()["tiny_cnn"]
    net = api.HipNetwork(cfg["layers"], cfg["mean"], cfg["std"])
    g = cases.rng(4100)
    imgs = [g.integers(0, 256, (8, 8, 3), dtype=np.uint8) for _ in range(2)]
    try:
        want = net.process_float(cfg["input"])
        want_img = net.process_images(imgs)
        for call in ("float", "images"):
            assert hiplib.THHipSumPartsInKernel(1) == 1
            G.note("a reported fault during THProcess" + call)
            hiplib.thhip_fault_flag()[0] = 1
            got = net.process_float(cfg["input"]) if call == "float" else net.process_images(imgs)
            assert hiplib.thhip_fault_flag()[0] == 0
            assert np.array_equal(got, want if call == "float" else want_img)
            assert hiplib.THHipSumPartsInKernel(1) == 0, "the report did not switch the path off"
        hiplib.thhip_sync()         # nothing is left over for the next synchronisation
        ref = np.asarray(oracle.run_layers(cfg["layers"], oracle.normalize(cfg["input"], cfg["mean"], cfg["std"])))
        G.assert_close(got if call == "float" else want, ref.ravel(), 1e-4, "after the repeat")
    finally:
        hiplib.THHipSumPartsInKernel(1)
        net.free()


def test_batchnorm_with_too_few_variances_is_fatal():
    body = r"""
g = cases.rng(5)
bn = {"type": "bn", "running_mean": np.zeros(8, np.float32), "running_var": np.ones(5, np.float32),
      "weight": np.ones(8, np.float32), "bias": np.zeros(8, np.float32), "eps": 1e-5}
layers = [cfg["layers"][0], bn]
lib.THHipFoldBatchNorm(%d)
net = api.HipNetwork(layers, fold_bn=%s)
"""
    fatal(body % (1, "True"), "running_var has 5 elements, 8 expected")
    fatal(body % (0, "False"), "running_var has 5 elements, 8 expected")


def test_uint8_image_loader_refuses_one_plane_images():
    """With stride < 3 * width the reference's loader reads past the image (three bytes per
    pixel whatever the stride, lowp_basic.c:82-131); the device copy would be read out of
    bounds, so the call is refused."""
    fatal(r"""
net = api.HipNetwork(cfg["layers"][:3], cfg["mean"], cfg["std"], lowp_range=16.0)
img = np.zeros((8, 8), np.uint8)
net.process_images([img])
""", "the uint8 engine takes three-plane images only")
    fatal(r"""
d = api.DeviceArray(lib, nbytes=64)
m = (C.c_float * 3)(0.4, 0.5, 0.6); s = (C.c_float * 3)(0.2, 0.25, 0.3)
a, b = C.c_float(), C.c_float()
lib.thhip_rgb2code(d.ptr, d.ptr, 8, 8, 8, m, s, 0, C.byref(a), C.byref(b))
""", "row stride 8 is less than 3 * width 8")


def test_minmax_kernel(hiplib):
    g = cases.rng(2300)
    for n in (1, 63, 1000, 300001):
        x = g.standard_normal(n).astype(np.float32) * np.float32(3)
        if n > 10:
            x[7] = np.nan      # skipped, as `data[i] > *max` skips it
        for dt in (G.F32, G.F16, G.BF16):
            d = api.to_device_dtype(hiplib, x, dt)
            back = api.from_device_dtype(d, (n,), dt)
            mn, mx = C.c_float(), C.c_float()
            hiplib.thhip_minmax(d.ptr, n, dt, C.byref(mn), C.byref(mx))
            assert mn.value == np.nanmin(back) and mx.value == np.nanmax(back), (n, dt)
    q = g.integers(3, 250, 5000, dtype=np.uint8)
    d = api.DeviceArray(hiplib, q)
    mn, mx = C.c_float(), C.c_float()
    hiplib.thhip_minmax(d.ptr, q.size, G.U8, C.byref(mn), C.byref(mx))
    assert (mn.value, mx.value) == (float(q.min()), float(q.max()))
    hiplib.thhip_minmax(d.ptr, 0, G.F32, C.byref(mn), C.byref(mx))
    fmax = float(np.finfo(np.float32).max)
    assert mn.value == fmax and mx.value == -fmax      # THInf / -THInf (FLT_MAX, thnets.h:463), thapi.c:143-144
    # values beyond +-FLT_MAX do not move the seeds either (`data[i] > *max` is false for -inf ... FLT_MAX)
    d = api.DeviceArray(hiplib, np.array([-np.inf, -np.inf], np.float32))
    hiplib.thhip_minmax(d.ptr, 2, G.F32, C.byref(mn), C.byref(mx))
    assert mn.value == -np.inf and mx.value == -fmax


def test_th_minmax_prints_every_layer(hiplib, oracle):
    """thapi.c:197-202: with th_minmax set the executor prints "Layer i output: min=..., max=..."
    after every module of the top-level list."""
    r = child(r"""
C.c_int.in_dll(lib, "th_minmax").value = 1
net = api.HipNetwork(cfg["layers"], cfg["mean"], cfg["std"])
net.process_float(cfg["input"])
C.CDLL(None).fflush(None)
""")
    assert r.returncode == 0, r.stderr
    lines = [l for l in r.stdout.splitlines() if l.startswith("Layer ")]
    cfg = cases.small_networks()["tiny_cnn"]
    outs = []
    oracle.run_layers(cfg["layers"], oracle.normalize(cfg["input"], cfg["mean"], cfg["std"]), collect=outs)
    # a Threshold folded into its producer: the producer's printed range is already the thresholded one
    assert len(lines) == len(cfg["layers"])
    for i, line in enumerate(lines):
        assert line.startswith("Layer %d output: min=" % (i + 1))
        mn = float(line.split("min=")[1].split(",")[0])
        mx = float(line.split("max=")[1])
        want = outs[i + 1] if cfg["layers"][i]["type"] == "conv" and cfg["layers"][i + 1]["type"] == "threshold" else outs[i]
        assert abs(mn - float(want.min())) <= 2e-5 * max(1, abs(float(want.min()))) + 1e-6, (i, line)
        assert abs(mx - float(want.max())) <= 2e-5 * max(1, abs(float(want.max()))) + 1e-6, (i, line)


def test_th_minmax_where_threshold_and_pooling_run_in_the_convolution(hiplib, oracle):
    """A convolution that takes the Threshold and the 2x2 pooling after it into its epilogue writes the
    pooled tensor only, so its line (and the lines of the two modules it absorbed, which pass that tensor
    on) shows the pooled tensor's range: the maximum is the convolution's own, the minimum that of the
    window maxima.  One line per module all the same (thapi.c:197-202)."""
    r = child(r"""
g = cases.rng(77)
from thnets_amd import configs
w1 = g.standard_normal((32, 3, 3, 3), dtype=np.float32) * np.float32(0.3)
w2 = g.standard_normal((64, 32, 3, 3), dtype=np.float32) * np.float32(0.08)
layers = [configs.conv(w1, g.standard_normal(32, dtype=np.float32) * np.float32(0.1), 1, 1), configs.relu(),
          configs.conv(w2, g.standard_normal(64, dtype=np.float32) * np.float32(0.1), 1, 1), configs.relu(), configs.maxpool(2, 2)]
x = g.uniform(0, 1, (3, 3, 128, 128)).astype(np.float32)
assert lib.thhip_conv2d_pool2_supported(3, 32, 128, 128, 64, 3, 3, 1, 1, 1, 1, 0, 0, 0)
C.c_int.in_dll(lib, "th_minmax").value = 1
net = api.HipNetwork(layers, cfg["mean"], cfg["std"])
net.process_float(x.copy())
C.CDLL(None).fflush(None)
""")
    assert r.returncode == 0, r.stderr
    lines = [l for l in r.stdout.splitlines() if l.startswith("Layer ")]
    assert len(lines) == 5, lines
    from thnets_amd import configs
    g = cases.rng(77)
    w1 = g.standard_normal((32, 3, 3, 3), dtype=np.float32) * np.float32(0.3)
    w2 = g.standard_normal((64, 32, 3, 3), dtype=np.float32) * np.float32(0.08)
    layers = [configs.conv(w1, g.standard_normal(32, dtype=np.float32) * np.float32(0.1), 1, 1), configs.relu(),
              configs.conv(w2, g.standard_normal(64, dtype=np.float32) * np.float32(0.1), 1, 1), configs.relu(), configs.maxpool(2, 2)]
    x = g.uniform(0, 1, (3, 3, 128, 128)).astype(np.float32)
    cfg = cases.small_networks()["tiny_cnn"]
    outs = []
    oracle.run_layers(layers, oracle.normalize(x, cfg["mean"], cfg["std"]), collect=outs)
    want = [outs[1], outs[1], outs[4], outs[4], outs[4]]      # (thresholded; thresholded and pooled)
    for i, line in enumerate(lines):
        assert line.startswith("Layer %d output: min=" % (i + 1))
        mn = float(line.split("min=")[1].split(",")[0])
        mx = float(line.split("max=")[1])
        assert abs(mn - float(want[i].min())) <= 2e-5 * max(1, abs(float(want[i].min()))) + 1e-6, (i, line, float(want[i].min()))
        assert abs(mx - float(want[i].max())) <= 2e-5 * max(1, abs(float(want[i].max()))) + 1e-6, (i, line, float(want[i].max()))
