"""Whole networks through the drop-in API (THCreateHipNetwork + THProcessFloat /
THForward) against the CPU oracle layer by layer and against golden vectors written by
the reference's own CPU library."""
import os

import numpy as np
import pytest

import cases
import gpu_util as G
from thnets_amd import api, netbuild, configs

pytestmark = pytest.mark.gpu

GOLD = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "fp32_golden.npz"))
NET_TOL = 1e-4      # contract: 1e-3 * max|ref| per layer output


def layerwise(net, oracle, cfg, tol, folded_bn=True):
    x = oracle.normalize(cfg["input"], cfg["mean"], cfg["std"])
    outs = []
    oracle.run_layers(cfg["layers"], x, collect=outs)
    layers = cfg["layers"]
    for i, o in enumerate(outs):
        if isinstance(o, list):
            continue
        want = o
        # a Threshold folded into its producer: the producer's buffer holds the thresholded values
        # (or applied in place on the producer's buffer)
        # a batch norm folded into the convolution before it: the convolution's buffer holds the
        # normalised values (and the threshold's, if one follows the batch norm)
        if folded_bn and layers[i]["type"] == "conv" and i + 1 < len(layers) and layers[i + 1]["type"] == "bn":
            want = outs[i + 1]
            if i + 2 < len(layers) and layers[i + 2]["type"] == "threshold":
                want = outs[i + 2]
        elif i + 1 < len(layers) and layers[i + 1]["type"] == "threshold" and (
                layers[i]["type"] in ("conv", "linear", "caddtable", "fullconv") or layers[i + 1].get("inplace", 1) == 1):
            want = outs[i + 1]
        got = net.module_output(i)
        if layers[i]["type"] in ("conv", "bn", "threshold") and got.size != np.asarray(want).size:
            # a 2x2 pooling done in the convolution's epilogue: the buffer holds the pooled tensor
            j = i + 1
            while j < len(layers) and layers[j]["type"] in ("bn", "threshold"):
                j += 1
            assert j < len(layers) and layers[j]["type"] == "maxpool", (i, got.shape, np.asarray(want).shape)
            want = outs[j]
        G.assert_close(got.ravel(), np.asarray(want).ravel(), tol, "module %d %s" % (i, layers[i]["type"]))


@pytest.mark.parametrize("name", sorted(cases.small_networks().keys()))
def test_small_networks_vs_oracle_and_golden(hiplib, oracle, name):
    cfg = cases.small_networks()[name]
    G.note("network " + name)
    net = api.HipNetwork(cfg["layers"], cfg["mean"], cfg["std"])
    x0 = cfg["input"].copy()
    y = net.process_float(cfg["input"])
    assert np.array_equal(cfg["input"], x0)
    G.assert_close(y, GOLD["net_" + name], NET_TOL, "golden")
    layerwise(net, oracle, cfg, NET_TOL)
    # repeated calls are stable
    assert np.array_equal(net.process_float(cfg["input"]), y)
    net.free()


def test_batchnorm_folding_on_and_off(hiplib, oracle):
    """A batch norm after a convolution runs in the convolution's epilogue by default
    and as its own kernel with THHipFoldBatchNorm(0); both match the restatement layer
    by layer, the unfolded one as closely as any other fp32 path."""
    cfg = cases.small_networks()["resnet18_small"]
    for fold in (True, False):
        net = api.HipNetwork(cfg["layers"], cfg["mean"], cfg["std"], fold_bn=fold)
        y = net.process_float(cfg["input"])
        G.assert_close(y, GOLD["net_resnet18_small"], NET_TOL, "golden fold=%s" % fold)
        layerwise(net, oracle, cfg, NET_TOL, folded_bn=fold)
        net.free()
    # a stand-alone conv -> bn -> relu chain with awkward planes, against the double-checked layers
    g = cases.rng(1600)
    w = g.standard_normal((70, 5, 3, 3), dtype=np.float32) * np.float32(0.2)
    layers = [configs.conv(w, g.standard_normal(70, dtype=np.float32), 1, 1), configs._bn(g, 70), configs.relu(),
              configs.maxpool(2, 2)]
    x = g.standard_normal((3, 5, 10, 12), dtype=np.float32)
    want = oracle.run_layers(layers, x)
    for fold in (True, False):
        net = api.HipNetwork(layers, fold_bn=fold)
        G.assert_close(net.process_float(x), want.ravel(), NET_TOL, "conv-bn-relu fold=%s" % fold)
        net.free()


def test_process_float_normalises_callers_buffer_in_place(hiplib, oracle):
    import ctypes as C
    cfg = cases.small_networks()["tiny_cnn"]
    net = api.HipNetwork(cfg["layers"], cfg["mean"], cfg["std"])
    x = np.array(cfg["input"], np.float32, copy=True)
    res = api.c_fp()
    ow, oh = C.c_int(), C.c_int()
    B, Cn, H, W = x.shape
    n = hiplib.THProcessFloat(net.handle, x.ctypes.data, B, W, H, Cn, C.byref(res), C.byref(ow), C.byref(oh))
    assert n == 30 and (ow.value, oh.value) == (1, 1)
    assert np.array_equal(x, oracle.normalize(cfg["input"], cfg["mean"], cfg["std"]))   # thapi.c:397-402
    got = np.ctypeslib.as_array(res, shape=(n,)).copy()
    net.free()
    # the device applies the normalisation to its own copy of the raw data: same bits as the host
    # pass, on every engine (odd sizes, planes beyond the third left alone)
    g = cases.rng(95)
    for (B, Cn, H, W) in ((3, 3, 7, 5), (2, 5, 6, 9), (1, 1, 4, 4)):
        raw = g.uniform(-2, 3, (B, Cn, H, W)).astype(np.float32)
        mean, std = np.float32([0.3, -0.2, 0.7]), np.float32([0.9, 1.7, 0.31])
        want = raw.copy()
        for c in range(min(Cn, 3)):
            want[:, c] = (want[:, c] - mean[c]) / std[c]
        for dt in (G.F32, G.F16, G.BF16):
            G.note("thhip_normalize %s dtype %d" % ((B, Cn, H, W), dt))
            d_in = api.DeviceArray(hiplib, raw)
            d_out = api.DeviceArray(hiplib, nbytes=raw.size * (4 if dt == G.F32 else 2))
            hiplib.thhip_normalize(d_in.ptr, d_out.ptr, B, Cn, H * W, mean.ctypes.data, std.ctypes.data, dt)
            hiplib.thhip_sync()
            ref = api.from_device_dtype(api.to_device_dtype(hiplib, want, dt), want.shape, dt)
            assert np.array_equal(api.from_device_dtype(d_out, raw.shape, dt), ref), (B, Cn, H, W, dt)
    # and the whole call equals a forward pass on host-normalised data
    net = api.HipNetwork(cfg["layers"], cfg["mean"], cfg["std"])
    net.upload(oracle.normalize(cfg["input"], cfg["mean"], cfg["std"]))
    net.forward()
    assert np.array_equal(net.module_output(net.nelem - 1).ravel(), got)
    net.free()


def test_config1_vs_golden_sample(hiplib, oracle):
    cfg = configs.config1()
    net = api.HipNetwork(cfg["layers"])
    net.upload(cfg["input"])
    net.forward()
    y = net.module_output(1).ravel()
    G.assert_close(y[cases.sample_indices(y.size)], GOLD["config1/sample"], 2e-5)
    assert abs(y.astype(np.float64).sum() - GOLD["config1/sum"]) <= 1e-5 * abs(GOLD["config1/sum"])
    G.assert_close(y, oracle.run_layers(cfg["layers"], cfg["input"]).ravel(), 2e-5)
    net.free()


def test_alexnet_b1_vs_golden_and_layerwise(hiplib, oracle):
    cfg = configs.alexnet_owt()
    net = api.HipNetwork(cfg["layers"], cfg["mean"], cfg["std"])
    y = net.process_float(cfg["input"])
    G.assert_close(y, GOLD["alexnet_b1"], NET_TOL)
    layerwise(net, oracle, cfg, NET_TOL)
    net.free()
    # the THMakeSpatial form gives the same logits
    cfg2 = configs.alexnet_owt(softmax=False)
    a = api.HipNetwork(cfg2["layers"], cfg2["mean"], cfg2["std"])
    b = api.HipNetwork(cfg2["layers"], cfg2["mean"], cfg2["std"], make_spatial=224)
    assert b.nelem == a.nelem - 1
    G.assert_close(b.process_float(cfg2["input"]), a.process_float(cfg2["input"]), 1e-5)
    a.free()
    b.free()


@pytest.mark.parametrize("half", [1, 2])
def test_half_engine_small_vgg(hiplib, oracle, half):
    cfg = cases.small_networks()["vgg16_small"]
    net = api.HipNetwork(cfg["layers"], cfg["mean"], cfg["std"], half=half)
    y = net.process_float(cfg["input"])
    G.assert_close(y, GOLD["net_vgg16_small"], 2e-2 if half == 1 else 6e-2, "half engine")
    # every module output, read back in the reference's order although the engine keeps the
    # tensors between convolutions channels-last
    layerwise(net, oracle, cfg, 2e-2 if half == 1 else 6e-2)
    net.free()
    # the same with batch norm (folded) and residual branches, and AlexNet's 11x11 / 5x5 layers
    for name, tol in (("resnet18_small", 4e-2 if half == 1 else 1.5e-1), ("alexnet_small", 2e-2 if half == 1 else 6e-2)):
        if name not in cases.small_networks():
            continue
        c2 = cases.small_networks()[name]
        n2 = api.HipNetwork(c2["layers"], c2["mean"], c2["std"], half=half)
        G.assert_close(n2.process_float(c2["input"]), GOLD["net_" + name], tol, name)
        n2.free()


@pytest.mark.parametrize("half", [1, 2])
def test_half_engine_image_layer_in_front(hiplib, oracle, half):
    """A half network whose image layer (3 -> 64, 3x3 / stride 1 / padding 1, ReLU) is followed by a 3x3 layer of
    64 planes: with THHipImageLayerInFront(2) the second layer computes the first one's output itself (one
    launch, nothing written), with 0 both run their own kernels, with 1 (the default) the batch decides.  Every
    module output against the oracle in each mode -- the image layer's is then filled on demand -- the modes
    against each other, and a second forward of another batch through the same network."""
    from thnets_amd.netbuild import conv, relu, maxpool
    g = cases.rng(1300)
    def wgt(*shape):
        return g.standard_normal(shape, dtype=np.float32) * np.float32(np.sqrt(2.0 / np.prod(shape[1:])))
    layers = [conv(wgt(64, 3, 3, 3), wgt(64) * np.float32(0.1), 1, 1), relu(),
              conv(wgt(72, 64, 3, 3), wgt(72) * np.float32(0.1), 1, 1), relu(), maxpool(2, 2),
              conv(wgt(32, 72, 3, 3), wgt(32) * np.float32(0.1), 1, 1), relu()]
    mean, std = (0.485, 0.456, 0.406), (0.229, 0.224, 0.225)
    tol = 2e-2 if half == 1 else 6e-2
    old = hiplib.THHipImageLayerInFront(1)
    try:
        for mode in (0, 2, 1):
            hiplib.THHipImageLayerInFront(mode)
            net = api.HipNetwork(layers, mean, std, half=half)
            for (B, H, W) in ((3, 40, 66), (5, 17, 32)):
                x = g.uniform(0, 1, (B, 3, H, W)).astype(np.float32)
                cfg = {"layers": layers, "mean": mean, "std": std, "input": x}
                net.process_float(x.copy())
                layerwise(net, oracle, cfg, tol)
            net.free()
    finally:
        hiplib.THHipImageLayerInFront(old)
    # the two forms on one input
    g2 = cases.rng(1301)
    x = g2.uniform(0, 1, (4, 3, 24, 64)).astype(np.float32)
    ys = []
    try:
        for mode in (0, 2):
            hiplib.THHipImageLayerInFront(mode)
            net = api.HipNetwork(layers, mean, std, half=half)
            ys.append((net.process_float(x.copy()), net.module_output(0), net.module_output(2)))
            net.free()
    finally:
        hiplib.THHipImageLayerInFront(old)
    assert np.array_equal(ys[0][1], ys[1][1])          # the image layer's own kernel either way
    G.assert_close(ys[1][2], ys[0][2], 1e-2, "second layer, image layer in front against behind")
    G.assert_close(ys[1][0], ys[0][0], 2e-2, "network output, image layer in front against behind")


def test_process_images_matches_process_float(hiplib, oracle):
    cfg = cases.small_networks()["tiny_cnn"]
    g = cases.rng(1200)
    imgs = [g.integers(0, 256, (8, 8, 3), dtype=np.uint8) for _ in range(3)]
    net = api.HipNetwork(cfg["layers"], cfg["mean"], cfg["std"])
    y = net.process_images(imgs, bgr=0)
    x = np.stack([oracle.rgb2float(im, cfg["mean"], cfg["std"], 0) for im in imgs])
    want = oracle.run_layers(cfg["layers"], x)
    G.assert_close(y, want.ravel(), 1e-5)
    yb = net.process_images(imgs, bgr=1)
    xb = np.stack([oracle.rgb2float(im, cfg["mean"], cfg["std"], 1) for im in imgs])
    G.assert_close(yb, oracle.run_layers(cfg["layers"], xb).ravel(), 1e-5)
    net.free()


def test_process_float_uploads_a_large_batch_in_windows(hiplib, oracle):
    """THProcessFloat on eight images of 4.8 MB: the batch goes up in three pieces and the first two
    convolutions (with their Threshold and pooling) work on a piece while the next one crosses the link
    (thhip_forward_windows).  Against the oracle, fp32 and fp16; a network whose first modules run a
    kernel that knows no window (a 3x3 / stride 2 pooling after the image layer) is noticed: that call, and
    the ones after it, run on the whole batch and give the right values too."""
    g = cases.rng(8800)
    def w(co, ci, k):
        return g.standard_normal((co, ci, k, k), dtype=np.float32) * np.float32(np.sqrt(2.0 / (ci * k * k)))
    def b(n):
        return g.standard_normal(n, dtype=np.float32) * np.float32(0.1)
    bn = dict(type="bn", weight=g.uniform(0.5, 1.5, 64).astype(np.float32), bias=b(64),
              running_mean=b(64), running_var=g.uniform(0.5, 1.5, 64).astype(np.float32), eps=1e-5)
    layers = [netbuild.conv(w(32, 3, 3), b(32), 1, 1), netbuild.relu(),
              netbuild.conv(w(64, 32, 3), b(64), 1, 1), bn, netbuild.relu(), netbuild.maxpool(2, 2),
              netbuild.conv(w(8, 64, 3), b(8), 1, 1), netbuild.relu(), netbuild.maxpool(2, 2)]
    mean, std = [0.485, 0.456, 0.406], [0.229, 0.224, 0.225]
    x = g.uniform(0, 1, (8, 3, 224, 224)).astype(np.float32)
    want = np.asarray(oracle.run_layers(layers, oracle.normalize(x, mean, std))).ravel()
    for kw, tol in (({}, 1e-4), ({"half": 1}, 3e-2)):
        net = api.HipNetwork(layers, mean, std, **kw)
        before = hiplib.thhip_windowed_forwards()
        G.note("THProcessFloat in windows %s" % (kw,))
        x0 = x.copy()
        got = net.process_float(x0)
        assert hiplib.thhip_windowed_forwards() == before + 1, "the batch was not run in windows"
        G.assert_close(got, want, tol, "in windows %s" % (kw,))
        again = net.process_float(x)
        assert np.array_equal(got, again)
        net.free()
    # a 3x3 / stride 2 pooling after the image layer: its kernels take no window
    layers = [netbuild.conv(w(32, 3, 3), b(32), 1, 1), netbuild.relu(), netbuild.maxpool(3, 2),
              netbuild.conv(w(64, 32, 3), b(64), 1, 1), netbuild.relu(), netbuild.maxpool(2, 2),
              netbuild.conv(w(8, 64, 3), b(8), 1, 1), netbuild.relu()]
    want = np.asarray(oracle.run_layers(layers, oracle.normalize(x, mean, std))).ravel()
    for kw, tol in (({}, 1e-4), ({"half": 1}, 3e-2)):
        net = api.HipNetwork(layers, mean, std, **kw)
        before = hiplib.thhip_windowed_forwards()
        G.note("THProcessFloat, a module of the prefix without a window %s" % (kw,))
        got = net.process_float(x)
        G.assert_close(got, want, tol, "whole batch after the window was ignored %s" % (kw,))
        assert np.array_equal(net.process_float(x), got)
        assert hiplib.thhip_windowed_forwards() == before
        net.free()


def test_vgg16_full_size_properties(hiplib, oracle):
    """Full configuration 3 (batch 16, 224x224): too large for the CPU checker inside a
    test, so check size-independent properties: batch == images one by one, and the
    first convolution + pooling block against the oracle on one image."""
    cfg = configs.vgg16(batch=4)
    net = api.HipNetwork(cfg["layers"])
    y = net.process_float(cfg["input"]).reshape(4, -1)
    y1 = net.process_float(cfg["input"][2:3]).ravel()
    G.assert_close(y1, y[2], 1e-5, "batch vs single image")
    net.upload(cfg["input"][:1])
    net.forward()
    want = oracle.run_layers(cfg["layers"][:5], cfg["input"][:1])
    G.assert_close(net.module_output(4), want, 2e-5, "first block")
    net.free()


@pytest.mark.gpu
def test_table_arithmetic_as_named(hiplib, oracle):
    """THHipTableArithmetic(1): CAddTable adds and CSubTable subtracts (the modules' documented
    meaning), in the table add's own kernel, in the epilogue of a block's last convolution (identity
    and projection shortcuts, fp32 planes in blocks of 32) and with three inputs; the default stays
    the shipped arithmetic (CAddTable.c:59-84), which the other tests pin."""
    g = cases.rng(7100)
    def cv(ci, co, k, pad):
        w = g.standard_normal((co, ci, k, k), dtype=np.float32) * np.float32(np.sqrt(1.0 / (ci * k * k)))
        return configs.conv(w, g.standard_normal(co, dtype=np.float32) * np.float32(0.1), 1, pad)
    ident = [{"type": "dropout", "p": 0.0, "inplace": 1, "v2": 1}]
    stem = [cv(3, 32, 3, 1), configs.relu()]
    main1, main2, short2 = [cv(32, 32, 3, 1), configs.relu(), cv(32, 32, 3, 1)], [cv(32, 64, 3, 1)], [cv(32, 64, 1, 0)]
    three = [[cv(64, 8, 3, 1)], [cv(64, 8, 1, 0)], [cv(64, 8, 3, 1)]]
    x = g.uniform(-1, 1, (2, 3, 12, 12)).astype(np.float32)
    run = lambda layers, t: oracle.run_layers(layers, t)
    for kind in ("caddtable", "csubtable"):
        sign = np.float32(1 if kind == "caddtable" else -1)
        layers = stem + [{"type": "concattable", "branches": [main1, ident]}, {"type": kind}, configs.relu(),
                         {"type": "concattable", "branches": [main2, short2]}, {"type": kind}, configs.relu(),
                         {"type": "concattable", "branches": three}, {"type": kind}]
        t = run(stem, x)
        t = np.maximum(run(main1, t) + sign * t, 0)
        t = np.maximum(run(main2, t) + sign * run(short2, t), 0)
        want = run(three[0], t) + sign * run(three[1], t) + sign * run(three[2], t)
        old = hiplib.THHipTableArithmetic(1)
        try:
            assert old == 0
            net = api.HipNetwork(layers)
        finally:
            hiplib.THHipTableArithmetic(0)
        got = net.process_float(x)
        G.assert_close(got, want.ravel(), NET_TOL, "tables as named, " + kind)
        net.free()
        shipped = api.HipNetwork(layers)      # the default again: what the reference's modules compute
        G.assert_close(shipped.process_float(x), run(layers, x).ravel(), NET_TOL, "tables as shipped, " + kind)
        shipped.free()


@pytest.mark.gpu
def test_graph_form_networks(hiplib, oracle):
    """Modules that name their inputs (ninputs / inputs[], thapi.c:173-193): the residual
    network as a flat graph gives bit for bit what its ConcatTable / CAddTable form gives,
    with the batch norms folded and not; a module is folded into its producer only when it
    is the producer's sole consumer."""
    cfg = cases.small_networks()["resnet18_small"]
    graph = configs.to_graph(cfg["layers"])
    assert any(len(s["inputs"]) == 2 for s in graph) and all(s["type"] != "concattable" for s in graph)
    want = oracle.run_layers(cfg["layers"], oracle.normalize(cfg["input"], cfg["mean"], cfg["std"]))
    for fold in (1, 0):
        hiplib.THHipFoldBatchNorm(fold)
        try:
            nt = api.HipNetwork(cfg["layers"], cfg["mean"], cfg["std"])
            ng = api.HipNetwork(graph, cfg["mean"], cfg["std"])
            yt, yg = nt.process_float(cfg["input"]), ng.process_float(cfg["input"])
            assert np.array_equal(yt, yg), "graph form differs from table form (fold %d)" % fold
            G.assert_close(yg, want.ravel(), 1e-3, "graph form vs oracle")
            nt.free()
            ng.free()
        finally:
            hiplib.THHipFoldBatchNorm(1)
    # half engine: a graph stays plane-major
    ng = api.HipNetwork(graph, cfg["mean"], cfg["std"], half=1)
    G.assert_close(ng.process_float(cfg["input"]), want.ravel(), 4e-2, "graph form, fp16")
    ng.free()
    # a convolution read by two modules: its Threshold must not be folded into it
    g = cases.rng(1700)
    w0 = g.standard_normal((8, 3, 3, 3), dtype=np.float32) * np.float32(0.3)
    w1 = g.standard_normal((8, 8, 3, 3), dtype=np.float32) * np.float32(0.2)
    b = lambda: g.standard_normal(8, dtype=np.float32) * np.float32(0.1)
    layers = [dict(netbuild.conv(w0, b(), 1, 1), inputs=[]),
              dict(netbuild.relu(inplace=0), inputs=[0]),
              dict(netbuild.conv(w1, b(), 1, 1), inputs=[0]),       # reads the convolution's raw output
              {"type": "caddtable", "inputs": [1, 2]},
              dict(netbuild.relu(), inputs=[3])]
    x = g.uniform(-1, 1, (2, 3, 9, 7)).astype(np.float32)
    net = api.HipNetwork(layers)
    G.assert_close(net.process_float(x.copy()), oracle.run_layers(layers, x).ravel(), 1e-4, "two consumers")
    net.free()
    # a convolution (with its folded Threshold) read by a pooling and by another module: the pooling
    # must not be taken by the convolution, whose full output the other module needs; and the same
    # chain with the pooling as its only consumer, where it is (a layer of a few tiles: its K is split)
    w2 = g.standard_normal((8, 64, 3, 3), dtype=np.float32) * np.float32(0.05)
    w3 = g.standard_normal((64, 3, 3, 3), dtype=np.float32) * np.float32(0.3)
    b64 = g.standard_normal(64, dtype=np.float32) * np.float32(0.1)
    for shared in (1, 0):
        layers = [dict(netbuild.conv(w3, b64, 1, 1), inputs=[]),
                  dict(netbuild.relu(), inputs=[0]),
                  dict(netbuild.conv(w2, b(), 1, 1), inputs=[1]),
                  dict(netbuild.relu(), inputs=[2]),
                  dict(netbuild.maxpool(3, 2), inputs=[3]),
                  dict(netbuild.maxpool(3, 2), inputs=[3 if shared else 4])]
        if shared:
            layers.append({"type": "caddtable", "inputs": [4, 5]})
        x = g.uniform(-1, 1, (2, 3, 13, 11)).astype(np.float32)
        net = api.HipNetwork(layers)
        G.assert_close(net.process_float(x.copy()), oracle.run_layers(layers, x).ravel(), 1e-4, "pooling, shared %d" % shared)
        net.free()


@pytest.mark.gpu
@pytest.mark.parametrize("half", [1, 2])
def test_vgg16_full_size_half_engines(hiplib, oracle, half):
    """Full-size VGG-16 on the half engines (the kernels that keep an input patch in LDS and
    the tiles loaded straight into LDS all run at their real shapes): against the fp32
    engine on the same input, image by image against the batch, and the first block
    against the oracle."""
    cfg = configs.vgg16(batch=3)
    n32 = api.HipNetwork(cfg["layers"])
    want = n32.process_float(cfg["input"]).reshape(3, -1)
    n32.free()
    net = api.HipNetwork(cfg["layers"], half=half)
    tol = 3e-2 if half == 1 else 1.5e-1
    y = net.process_float(cfg["input"]).reshape(3, -1)
    G.assert_close(y, want, tol, "half engine vs fp32 engine")
    y1 = net.process_float(cfg["input"][1:2]).ravel()
    G.assert_close(y1, y[1], 1e-2 if half == 1 else 5e-2, "batch vs single image")     # (other tiles, other rounding order)
    net.upload(cfg["input"][:1])
    net.forward()
    ref = oracle.run_layers(cfg["layers"][:5], cfg["input"][:1])
    G.assert_close(net.module_output(4), ref, 2e-2 if half == 1 else 6e-2, "first block")
    net.free()


@pytest.mark.gpu
@pytest.mark.parametrize("name", ["tiny_cnn", "vgg16_small", "resnet18_small", "segnet_small"])
def test_loaded_model_directory_runs_like_the_layer_list(hiplib, oracle, tmp_path, name):
    """THLoadNetwork -> THCreateHipNetwork -> THProcessFloat on a Torch7 model
    directory gives, bit for bit, what the same weights give when the module array
    is assembled by hand, in fp32, fp16 and uint8 form; the fp32 and fp16 results are
    also held against the golden vector of the reference's CPU library and against the
    oracle on the same weights."""
    from thnets_amd import t7
    cfg = cases.small_networks()[name]
    ref = np.asarray(oracle.run_layers(cfg["layers"], oracle.normalize(cfg["input"], cfg["mean"], cfg["std"])))
    t7.save_model_dir(str(tmp_path), cfg["layers"], cfg["mean"], cfg["std"], longsize=4 if name == "tiny_cnn" else 8)
    G.note("model directory %s" % name)
    for kw in ({}, {"half": 1}) + (({"lowp_range": 16.0, "make_spatial": 8},) if name == "tiny_cnn" else ()):
        a = api.HipNetwork(str(tmp_path), **kw)
        b = api.HipNetwork(cfg["layers"], cfg["mean"], cfg["std"], **kw)
        got, want = a.process_float(cfg["input"]), b.process_float(cfg["input"])
        a.free()
        b.free()
        assert got.shape == want.shape and np.array_equal(got, want), kw
        if not kw:
            G.assert_close(got, GOLD["net_" + name], NET_TOL, "model directory against the golden vector")
            G.assert_close(got.ravel(), ref.ravel(), NET_TOL, "model directory against the oracle")
        elif "half" in kw:
            G.assert_close(got.ravel(), ref.ravel(), 3e-2, "model directory, fp16, against the oracle")


@pytest.mark.gpu
def test_command_line_driver(hiplib, oracle, tmp_path):
    """thnets-hip-test (the counterpart of thnets-test.c) on a model directory and
    a .t7 input prints the values THProcessFloat returns; a PPM image goes through
    THProcessImages."""
    import subprocess
    from thnets_amd import t7
    cfg = cases.small_networks()["tiny_cnn"]
    t7.save_model_dir(str(tmp_path), cfg["layers"], cfg["mean"], cfg["std"])
    x = cfg["input"][0]
    t7.save(str(tmp_path / "in.t7"), np.ascontiguousarray(x))
    exe = os.path.join(os.path.dirname(api.LIB_PATH), "thnets-hip-test")
    assert os.path.exists(exe), "build it with make -C thnets_amd/csrc"
    net = api.HipNetwork(cfg["layers"], cfg["mean"], cfg["std"])
    want = net.process_float(np.stack([x, x]))
    ref = np.asarray(oracle.run_layers(cfg["layers"], oracle.normalize(np.stack([x, x]), cfg["mean"], cfg["std"])))
    G.note("thnets-hip-test fp32 batch 2")
    r = subprocess.run([exe, "-m", str(tmp_path), "-i", str(tmp_path / "in.t7"), "-p", "-b", "2", "-r", "2"],
                       capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stderr
    vals = [float(l.split(":")[1]) for l in r.stdout.splitlines() if l.startswith("(")]
    assert len(vals) == want.size and np.allclose(vals, want, rtol=0, atol=5e-7)
    G.assert_close(np.asarray(vals, np.float32), ref.ravel(), NET_TOL, "printed values against the oracle")
    assert "1 run processing time:" in r.stdout
    # an 8-bit image through THProcessImages
    g = cases.rng(91)
    img = g.integers(0, 256, (8, 8, 3), dtype=np.uint8)
    with open(tmp_path / "in.ppm", "wb") as fp:
        fp.write(b"P6\n# test image\n8 8\n255\n" + img.tobytes())
    want = net.process_images([img])
    net.free()
    G.note("thnets-hip-test ppm")
    r = subprocess.run([exe, "-m", str(tmp_path), "-i", str(tmp_path / "in.ppm"), "-p", "-L", "4"],
                       capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stderr
    vals = [float(l.split(":")[1]) for l in r.stdout.splitlines() if l.startswith("(")]
    assert len(vals) == 4 and np.allclose(vals, want[:4], rtol=0, atol=5e-7)
    ximg = oracle.rgb2float(img, cfg["mean"], cfg["std"], 0)[None]
    ref = np.asarray(oracle.run_layers(cfg["layers"], ximg)).ravel()
    G.assert_close(np.asarray(vals, np.float32), ref[:4], NET_TOL, "printed values of the image against the oracle")
    # a model directory that does not exist: the reference's message, exit code 0 (thnets-test.c:199)
    r = subprocess.run([exe, "-m", str(tmp_path / "none"), "-i", "random"], capture_output=True, text=True, timeout=120)
    assert "The network could not be loaded: -1" in r.stdout
