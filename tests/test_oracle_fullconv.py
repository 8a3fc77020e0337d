"""Pins the restatements of SpatialFullConvolution, the pooling indices and
SpatialMaxUnpooling (oracle/thnets_oracle.c):
  1. golden vectors written by the reference's own compiled CPU library
     (tests/golden/fp32_golden.npz: fullconv*, maxunpool*, net_segnet_small);
  2. live against that library where oracle/_ref holds a build of it;
  3. mathematics: the scatter definition in double precision, the adjoint identity
     <fullconv(x), y> == <x, conv(y)> with the (separately pinned) convolution, a
     stride-1 full convolution == a padded convolution with the flipped kernel, brute
     force unpooling in Python; the bias rule (11 * sum + bias) shows against all three.
"""
import os

import numpy as np
import pytest

import cases

GOLD = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "fp32_golden.npz"))
SUM_TOL = 2e-5


def close(a, b, tol=SUM_TOL):
    a = np.asarray(a, np.float64).ravel()
    b = np.asarray(b, np.float64).ravel()
    assert a.shape == b.shape
    assert np.abs(a - b).max() <= tol * max(np.abs(b).max(), 1e-30)


def run(oracle, spec, x):
    return oracle.run_layers([spec], x)


@pytest.mark.parametrize("i", range(len(cases.FULLCONV_CASES)))
def test_fullconv_golden_and_definition(oracle, i):
    x, spec = cases.fullconv_case(i)
    y = run(oracle, spec, x)
    assert y.shape == GOLD["fullconv%d" % i].shape
    close(y, GOLD["fullconv%d" % i])
    d, pad, adj = (spec["dH"], spec["dW"]), (spec["padH"], spec["padW"]), (spec["adjH"], spec["adjW"])
    exact = oracle.fullconv2d_f64(x, spec["weight"], d, pad, adj)
    if spec["bias"] is None:
        close(y, exact)
    else:       # SpatialFullConvolution.c:231-237: beta = 11 in the bias GEMM
        close(y, 11.0 * exact + spec["bias"].astype(np.float64)[None, :, None, None])


@pytest.mark.parametrize("i", range(len(cases.FULLCONV_CASES)))
def test_fullconv_is_the_adjoint_of_the_convolution(oracle, i):
    """<fullconv_w(x), y> == <x, conv_w(y)> for every y when the convolution of y
    (weight read as [Ci out][Co in][kH][kW], same stride and pad) lands on x's extent."""
    x, spec = cases.fullconv_case(i)
    d, pad, adj = (spec["dH"], spec["dW"]), (spec["padH"], spec["padW"]), (spec["adjH"], spec["adjW"])
    full = oracle.fullconv2d_f64(x, spec["weight"], d, pad, adj)
    g = cases.rng(850 + i)
    y = g.standard_normal(full.shape).astype(np.float32)
    back = oracle.conv2d_f64(y, spec["weight"], None, d, pad)
    assert back.shape == x.shape        # (oH + 2 pad - k) // d + 1 == H, also with adj < d
    lhs, rhs = float((full * y).sum()), float((x.astype(np.float64) * back).sum())
    assert abs(lhs - rhs) <= 1e-9 * max(abs(lhs), abs(rhs), 1.0)


def test_stride1_fullconv_is_a_padded_convolution_with_the_flipped_kernel(oracle):
    g = cases.rng(860)
    x = g.standard_normal((2, 5, 6, 7), dtype=np.float32)
    w = g.standard_normal((5, 4, 3, 3), dtype=np.float32)
    full = oracle.fullconv2d(x, w, None, (1, 1), (1, 1))
    wc = np.ascontiguousarray(w[:, :, ::-1, ::-1].transpose(1, 0, 2, 3))
    close(full, oracle.conv2d(x, wc, None, (1, 1), (1, 1)))


def brute_unpool(x, ind, oH, oW):
    B, Cn, iH, iW = x.shape
    y = np.zeros((B, Cn, oH * oW), np.float32)
    for b in range(B):
        for c in range(Cn):
            for e in range(iH * iW):
                y[b, c, int(ind[b, c].ravel()[e]) - 1] = x[b, c].ravel()[e]
    return y.reshape(B, Cn, oH, oW)


@pytest.mark.parametrize("j,geom", list(enumerate([(2, 2, 0), (3, 2, 1), (3, 1, 1)])))
def test_maxunpool_golden_and_brute_force(oracle, j, geom):
    k, d, pad = geom
    g = cases.rng(701)
    xp = g.standard_normal((2, 3, 9, 8), dtype=np.float32)
    layers = [cases.maxpool(k, d, pad), {"type": "threshold", "threshold": -0.2, "val": 7.0, "alpha": 0, "inplace": 0},
              {"type": "maxunpool", "pooling": 0}]
    y = oracle.run_layers(layers, xp)
    assert np.array_equal(y, GOLD["maxunpool%d" % j])
    pooled, ind = oracle.maxpool_indices(xp, k, k, d, d, pad, pad)
    assert np.array_equal(pooled, oracle.maxpool(xp, k, k, d, d, pad, pad))
    # the index names the first maximum of the window
    flat = xp.reshape(2, 3, -1)
    assert np.array_equal(np.take_along_axis(flat, (ind.reshape(2, 3, -1) - 1).astype(np.int64), 2).reshape(pooled.shape), pooled)
    t = oracle.threshold(pooled, -0.2, 7.0, 0.0, 0)
    assert np.array_equal(y, brute_unpool(t, ind, 9, 8))
    # unpooling a pooling's own output puts every maximum back in its place
    back = oracle.maxunpool(pooled, ind, 9, 8)
    mask = back != 0
    assert np.array_equal(back[mask], xp[mask])


def test_segnet_small_golden(oracle):
    cfg = cases.small_networks()["segnet_small"]
    x = oracle.normalize(cfg["input"], cfg["mean"], cfg["std"])
    y = oracle.run_layers(cfg["layers"], x)
    close(y.ravel(), GOLD["net_segnet_small"], 1e-4)


@pytest.mark.parametrize("i", range(len(cases.FULLCONV_CASES)))
def test_fullconv_live_reference(oracle, reference, i):
    x, spec = cases.fullconv_case(i)
    hn = reference.host_network({"layers": [spec], "mean": (0, 0, 0), "std": (1, 1, 1)})
    close(run(oracle, spec, x), reference.forward(hn, x))


def test_segnet_small_live_reference(oracle, reference):
    cfg = cases.small_networks()["segnet_small"]
    want = reference.process_float(reference.host_network(cfg), cfg["input"])
    x = oracle.normalize(cfg["input"], cfg["mean"], cfg["std"])
    close(oracle.run_layers(cfg["layers"], x).ravel(), want, 1e-4)
