"""Pins the fp32 CPU restatement (oracle/thnets_oracle.c) three ways:
  1. against golden vectors written by the reference's own compiled CPU library
     (tests/golden/fp32_golden.npz, made by tests/golden/make_golden.py);
  2. live against that library when oracle/_ref holds a build of it;
  3. against what the mathematics fixes (double-precision direct convolution, delta
     kernels, 1x1 convolution == Linear, batch == images one by one, numpy closed
     forms), chosen so that a dropped term, a wrong index or a transposed operand fails.
Tolerance for GEMM-shaped results: 1e-3 * max|ref| is the contract; the restatement is
held to 2e-5 * max|ref| (summation order only).  Everything else is bit-exact.
"""
import os

import numpy as np
import pytest

import cases
from thnets_amd import configs

GOLD = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "fp32_golden.npz"))
SUM_TOL = 2e-5


def close(a, b, tol=SUM_TOL):
    a = np.asarray(a, np.float64).ravel()
    b = np.asarray(b, np.float64).ravel()
    assert a.shape == b.shape
    assert np.abs(a - b).max() <= tol * max(np.abs(b).max(), 1e-30)


# ---------------------------------------------------------------- golden vectors

@pytest.mark.parametrize("i", range(len(cases.CONV_CASES)))
def test_conv_golden(oracle, i):
    x, spec = cases.conv_case(i)
    g = GOLD["conv%d" % i]
    for unfold in (False, True):
        y = oracle.conv2d(x, spec["weight"], spec["bias"], (spec["dH"], spec["dW"]), (spec["padH"], spec["padW"]),
                          use_unfold=unfold)
        assert y.shape == g.shape
        close(y, g)


@pytest.mark.parametrize("i", range(len(cases.POOL_CASES)))
def test_pool_golden(oracle, i):
    x = cases.pool_case(i)
    s = cases.pool_spec(i, "maxpool")
    y = oracle.run_layers([s], x)
    assert y.shape == GOLD["maxpool%d" % i].shape
    assert np.array_equal(y, GOLD["maxpool%d" % i])
    s = cases.pool_spec(i, "avgpool")
    y = oracle.run_layers([s], x)
    assert y.shape == GOLD["avgpool%d" % i].shape
    assert np.array_equal(y, GOLD["avgpool%d" % i])


@pytest.mark.parametrize("i", range(len(cases.LINEAR_CASES)))
def test_linear_golden(oracle, i):
    x, spec = cases.linear_case(i)
    y = oracle.run_layers([spec], x)
    g = GOLD["linear%d" % i]
    assert y.shape == g.shape
    if x.ndim == 1:
        # sequential dot, no fused multiply-add: the same arithmetic as a default build
        # of the reference (OpenBLAS-stripped/gemv_t.c:51-63)
        assert np.array_equal(y, g)
    else:
        close(y, g)


@pytest.mark.parametrize("i", range(len(cases.SOFTMAX_SHAPES)))
def test_softmax_golden(oracle, i):
    y = oracle.softmax(cases.softmax_case(i))
    assert np.array_equal(y, GOLD["softmax%d" % i])


def test_bn_threshold_caddtable_golden(oracle):
    x, spec = cases.bn_case()
    assert np.array_equal(oracle.run_layers([spec], x), GOLD["bn0"])
    g = cases.rng(700)
    xt = g.standard_normal((2, 3, 4, 5), dtype=np.float32)
    for j, (thr, val, alpha, inplace) in enumerate([(0, 0, 0, 1), (0.25, -1.5, 0, 0), (0.25, -1.5, 0, 1), (0, 0, 0.1, 0)]):
        y = oracle.threshold(xt, thr, val, alpha, inplace)
        assert np.array_equal(y, GOLD["threshold%d" % j]), j
    ws = [g.standard_normal((4, 3, 1, 1), dtype=np.float32) for _ in range(3)]
    for nb in (2, 3):
        layers = [{"type": "concattable", "branches": [[cases.conv(w, None)] for w in ws[:nb]]}, {"type": "caddtable"}]
        close(oracle.run_layers(layers, xt), GOLD["caddtable%d" % nb])


@pytest.mark.parametrize("name", sorted(cases.small_networks().keys()))
def test_small_network_golden(oracle, name):
    cfg = cases.small_networks()[name]
    x = oracle.normalize(cfg["input"], cfg["mean"], cfg["std"])
    y = oracle.run_layers(cfg["layers"], x)
    close(y, GOLD["net_" + name], 1e-4)


def test_config1_and_alexnet_golden(oracle):
    cfg = configs.config1()
    y = oracle.run_layers(cfg["layers"], cfg["input"]).ravel()
    assert tuple(GOLD["config1/shape"]) == (1, 128, 56, 56)
    close(y[cases.sample_indices(y.size)], GOLD["config1/sample"])
    assert abs(y.astype(np.float64).sum() - GOLD["config1/sum"]) <= 1e-5 * abs(GOLD["config1/sum"])
    cfg = configs.alexnet_owt()
    x = oracle.normalize(cfg["input"], cfg["mean"], cfg["std"])
    close(oracle.run_layers(cfg["layers"], x), GOLD["alexnet_b1"], 1e-4)


# ---------------------------------------------------------------- live reference

def test_reference_live_conv_and_network(oracle, reference):
    for i in (1, 3, 5, 7):
        x, spec = cases.conv_case(i)
        hn = reference.host_network({"layers": [spec], "mean": (0, 0, 0), "std": (1, 1, 1)})
        close(oracle.run_layers([spec], x), reference.forward(hn, x))
    cfg = cases.small_networks()["resnet18_small"]
    hn = reference.host_network(cfg)
    yr = reference.process_float(hn, cfg["input"])
    x = oracle.normalize(cfg["input"], cfg["mean"], cfg["std"])
    close(oracle.run_layers(cfg["layers"], x), yr, 1e-4)
    # a second forward on the same reference network gives the same answer
    assert np.array_equal(yr, reference.process_float(hn, cfg["input"]))


def test_reference_live_normalisation_is_in_place(oracle, reference):
    cfg = cases.small_networks()["tiny_cnn"]
    hn = reference.host_network(cfg)
    close(reference.process_float(hn, cfg["input"]),
          oracle.run_layers(cfg["layers"], oracle.normalize(cfg["input"], cfg["mean"], cfg["std"])), 1e-5)


# ---------------------------------------------------------------- mathematics

@pytest.mark.parametrize("i", range(len(cases.CONV_CASES)))
def test_conv_vs_double_direct(oracle, i):
    x, spec = cases.conv_case(i)
    d, p = (spec["dH"], spec["dW"]), (spec["padH"], spec["padW"])
    close(oracle.conv2d(x, spec["weight"], spec["bias"], d, p), oracle.conv2d_f64(x, spec["weight"], spec["bias"], d, p),
          1e-5)


def test_double_direct_vs_numpy_brute_force(oracle):
    g = cases.rng(1)
    x = g.standard_normal((2, 3, 6, 5))
    w = g.standard_normal((4, 3, 3, 2))
    b = g.standard_normal(4)
    dH, dW, pH, pW = 2, 1, 1, 2
    oH, oW = (6 + 2 * pH - 3) // dH + 1, (5 + 2 * pW - 2) // dW + 1
    xp = np.zeros((2, 3, 6 + 2 * pH, 5 + 2 * pW))
    xp[:, :, pH:pH + 6, pW:pW + 5] = x.astype(np.float32)
    ref = np.zeros((2, 4, oH, oW))
    for oy in range(oH):
        for ox in range(oW):
            patch = xp[:, :, oy * dH:oy * dH + 3, ox * dW:ox * dW + 2]
            ref[:, :, oy, ox] = np.einsum("bchw,ochw->bo", patch, w.astype(np.float32).astype(np.float64)) + \
                b.astype(np.float32)
    y = oracle.conv2d_f64(x.astype(np.float32), w.astype(np.float32), b.astype(np.float32), (dH, dW), (pH, pW))
    assert np.abs(y - ref).max() < 1e-12


def test_unfold_matches_definition_and_mm_equals_virtmm(oracle):
    g = cases.rng(2)
    x = g.standard_normal((3, 7, 6), dtype=np.float32)
    col = oracle.unfold(x, (3, 2), (2, 1), (1, 1))
    oH, oW = (7 + 2 - 3) // 2 + 1, (6 + 2 - 2) // 1 + 1
    assert col.shape == (3 * 3 * 2, oH * oW)
    for k in range(col.shape[0]):
        c, kh, kw = k // 6, (k % 6) // 2, k % 2
        for y in range(oH):
            for xx in range(oW):
                iy, ix = y * 2 - 1 + kh, xx - 1 + kw
                want = x[c, iy, ix] if 0 <= iy < 7 and 0 <= ix < 6 else 0.0
                assert col[k, y * oW + xx] == want
    w = g.standard_normal((5, 3, 3, 2), dtype=np.float32)
    a = oracle.conv2d(x[None], w, None, (2, 1), (1, 1), use_unfold=True)
    b = oracle.conv2d(x[None], w, None, (2, 1), (1, 1), use_unfold=False)
    assert np.array_equal(a, b)


def test_delta_kernel_shifts_input_and_zero_weights_give_bias(oracle):
    g = cases.rng(3)
    x = g.standard_normal((1, 2, 8, 9), dtype=np.float32)
    w = np.zeros((2, 2, 3, 3), np.float32)
    w[0, 0, 0, 2] = 1.0      # output plane 0 = plane 0 shifted by (-1, +1)
    w[1, 1, 2, 1] = 1.0      # output plane 1 = plane 1 shifted by (+1, 0)
    y = oracle.conv2d(x, w, None, (1, 1), (1, 1))
    xp = np.pad(x, ((0, 0), (0, 0), (1, 1), (1, 1)))
    assert np.array_equal(y[0, 0], xp[0, 0, 0:8, 2:11])
    assert np.array_equal(y[0, 1], xp[0, 1, 2:10, 1:10])
    b = np.array([0.5, -2.0], np.float32)
    y = oracle.conv2d(x, np.zeros_like(w), b, (1, 1), (1, 1))
    assert np.array_equal(y, np.broadcast_to(b[None, :, None, None], y.shape))


def test_1x1_conv_equals_linear_and_batch_equals_single_images(oracle):
    g = cases.rng(4)
    x = g.standard_normal((5, 24), dtype=np.float32)
    w = g.standard_normal((7, 24), dtype=np.float32)
    b = g.standard_normal(7, dtype=np.float32)
    lin = oracle.linear(x, w, b)
    cv = oracle.conv2d(x.reshape(5, 24, 1, 1), w.reshape(7, 24, 1, 1), b).reshape(5, 7)
    close(lin, cv, 1e-6)
    close(lin, x.astype(np.float64) @ w.astype(np.float64).T + b, 1e-6)
    for i in range(5):
        close(oracle.linear(x[i], w, b), lin[i], 1e-6)
    xi, spec = cases.conv_case(5)
    yb = oracle.run_layers([spec], xi)
    for t in range(xi.shape[0]):
        assert np.array_equal(oracle.run_layers([spec], xi[t:t + 1])[0], yb[t])


def test_threshold_closed_forms(oracle):
    x = np.array([-2.0, -0.0, 0.0, 0.25, 0.3, 5.0, np.inf, -np.inf], np.float32)
    assert np.array_equal(oracle.threshold(x, 0, 0, 0, 1), np.where(x <= 0, np.float32(0), x))
    assert np.array_equal(oracle.threshold(x, 0.25, -1, 0, 0), np.where(x > 0.25, x, np.float32(-1)))
    assert np.array_equal(oracle.threshold(x, 0.25, -1, 0, 1), np.where(x <= 0.25, np.float32(-1), x))
    with np.errstate(invalid="ignore"):
        assert np.array_equal(oracle.threshold(x[:6], 9, 9, 0.5, 0), np.where(x[:6] >= 0, x[:6], x[:6] * np.float32(0.5)))


def test_pool_geometry_and_values_brute_force(oracle):
    # floor / ceil and the "last window must start inside" rule
    assert oracle.pool_outsize(55, 55, 3, 3, 2, 2, 0, 0, 0) == (27, 27)
    assert oracle.pool_outsize(13, 13, 3, 3, 2, 2, 0, 0, 1) == (6, 6)
    assert oracle.pool_outsize(14, 14, 3, 3, 2, 2, 0, 0, 1) == (7, 7)
    assert oracle.pool_outsize(112, 112, 3, 3, 2, 2, 1, 1, 0) == (56, 56)
    assert oracle.pool_outsize(6, 6, 3, 3, 3, 3, 1, 1, 1) == (3, 3)
    assert oracle.pool_outsize(5, 5, 2, 2, 2, 2, 1, 1, 1) == (3, 3)   # ceil gives 4, last starts at 6 >= 5+1
    for i in range(len(cases.POOL_CASES)):
        x = cases.pool_case(i)
        B, Cn, H, W, kH, kW, dH, dW, pH, pW, ceil = cases.POOL_CASES[i]
        y = oracle.maxpool(x, kH, kW, dH, dW, pH, pW, ceil)
        ya = oracle.avgpool(x, kH, kW, dH, dW, pH, pW, ceil, count_include_pad=1)
        oH, oW = y.shape[2:]
        for oy in range(oH):
            for ox in range(oW):
                hs, ws = oy * dH - pH, ox * dW - pW
                he, we = min(hs + kH, H), min(ws + kW, W)
                win = x[:, :, max(hs, 0):he, max(ws, 0):we]
                assert np.array_equal(y[:, :, oy, ox], win.max(axis=(2, 3)))
                pool = (min(hs + kH, H + pH) - hs) * (min(ws + kW, W + pW) - ws)
                close(ya[:, :, oy, ox], win.astype(np.float64).sum(axis=(2, 3)) / pool, 1e-5)


def test_softmax_polynomial_and_normalisation(oracle):
    # the routine is 1 / (1 + x/8 + x^2/128 + x^3/3072 + x^4/98304)^8, an 8th-power
    # truncated exponential: exact value at 0, close to exp(-x) for small x, 0 from 13 on
    f = oracle.lib.orc_exp_minus_approx
    assert f(0.0) == 1.0
    assert f(13.0) == 0.0 and f(50.0) == 0.0
    for v in (0.1, 0.5, 1.0, 2.0, 5.0, 10.0):
        p = 1 + v / 8 + v * v * 0.0078125 + v ** 3 * 0.00032552083 + v ** 4 * 1.0172526e-5
        assert abs(f(v) - p ** -8) < 1e-14
        assert abs(f(v) - np.exp(-v)) < 1e-4
    x = cases.softmax_case(1)
    y = oracle.softmax(x)
    close(y.sum(axis=1), np.ones(3), 1e-5)
    assert np.array_equal(np.argmax(y, 1), np.argmax(x, 1))
    y4 = oracle.softmax(cases.softmax_case(3))
    close(y4.sum(axis=1), np.ones((2, 3, 3)), 1e-5)


def test_batchnorm_and_caddtable_closed_forms(oracle):
    x, s = cases.bn_case()
    y = oracle.run_layers([s], x)
    inv = (1 / np.sqrt(s["running_var"].astype(np.float64) + 1e-5)).astype(np.float32)
    want = ((x - s["running_mean"][None, :, None, None]) * inv[None, :, None, None]) * s["weight"][None, :, None, None] \
        + s["bias"][None, :, None, None]
    assert np.array_equal(y, want.astype(np.float32))
    a = np.arange(6, dtype=np.float32) + 5
    b = np.arange(4, dtype=np.float32) + 3
    c = np.ones(2, np.float32)
    # two inputs subtract (and copy the tail); CSubTable adds; three inputs count the first twice
    assert np.array_equal(oracle.caddtable([a, b]), np.concatenate([a[:4] - b, a[4:]]))
    assert np.array_equal(oracle.caddtable([a, b], is_csubtable=True), np.concatenate([a[:4] + b, a[4:]]))
    want3 = 2 * a
    want3[:4] += b
    want3[:2] += c
    assert np.array_equal(oracle.caddtable([a, b, c]), want3)


def test_rgb2float_closed_form(oracle):
    g = cases.rng(5)
    img = g.integers(0, 256, (5, 7, 3), dtype=np.uint8)
    mean, std = (0.485, 0.456, 0.406), (0.229, 0.224, 0.225)
    for bgr in (0, 1):
        y = oracle.rgb2float(img, mean, std, bgr)
        src = img[:, :, ::-1] if bgr else img
        want = (src.transpose(2, 0, 1).astype(np.float32) * np.float32(0.003921568) -
                np.asarray(mean, np.float32)[:, None, None]) * (np.float32(1) / np.asarray(std, np.float32))[:, None, None]
        assert np.array_equal(y, want.astype(np.float32))


def test_graph_form_equals_table_form(oracle):
    """Layers that name their inputs (the reference's executor for graph formats,
    thapi.c:173-193): laying a ConcatTable / CAddTable network out as a flat graph changes
    nothing, bit for bit, and every named input must come earlier in the list."""
    from thnets_amd import configs, netbuild
    cfg = cases.small_networks()["resnet18_small"]
    x = oracle.normalize(cfg["input"], cfg["mean"], cfg["std"])
    graph = configs.to_graph(cfg["layers"])
    assert np.array_equal(oracle.run_layers(graph, x), oracle.run_layers(cfg["layers"], x))
    # an identity branch disappears: such an add reads the main branch and, earlier in the list, the block input
    adds = [s for s in graph if s["type"] == "caddtable"]
    assert adds and all(len(s["inputs"]) == 2 for s in adds) and any(s["inputs"][0] > s["inputs"][1] for s in adds)
    for i, s in enumerate(graph):
        assert all(0 <= j < i for j in s["inputs"])
