"""Seeded test cases shared by the golden-vector generator, the CPU tests and the GPU
tests.  Inputs are regenerated from the seed everywhere; only outputs are stored."""
import numpy as np

from thnets_amd import configs
from thnets_amd.netbuild import conv, maxpool, relu


def rng(seed):
    return np.random.Generator(np.random.PCG64(seed))


# (B, Ci, H, W, Co, kH, kW, dH, dW, padH, padW) -- edge cases the reference's geometry
# code distinguishes: stride 4 / pad 2 (AlexNet conv1), stride 2 / pad 3 (ResNet stem),
# 1x1 with and without stride, non-square kernels and strides, pad wider than the
# kernel reach, a single output position, output planes that are not tile multiples.
CONV_CASES = [
    (1, 3, 19, 23, 5, 3, 3, 1, 1, 1, 1),
    (2, 7, 17, 13, 70, 5, 5, 2, 2, 2, 2),
    (3, 16, 9, 9, 130, 1, 1, 1, 1, 0, 0),
    (1, 3, 35, 35, 64, 11, 11, 4, 4, 2, 2),
    (2, 3, 30, 30, 16, 7, 7, 2, 2, 3, 3),
    (4, 33, 14, 14, 200, 3, 3, 2, 2, 1, 1),
    (5, 8, 6, 6, 16, 6, 6, 1, 1, 0, 0),
    (2, 5, 12, 10, 9, 3, 2, 1, 2, 0, 1),
    (1, 4, 8, 8, 33, 1, 1, 2, 2, 0, 0),
    (6, 2, 5, 5, 3, 3, 3, 1, 1, 2, 2),
    (1, 64, 14, 14, 96, 3, 3, 1, 1, 1, 1),
]


def conv_case(i):
    B, Ci, H, W, Co, kH, kW, dH, dW, pH, pW = CONV_CASES[i]
    g = rng(100 + i)
    x = g.uniform(-1, 1, (B, Ci, H, W)).astype(np.float32)
    w = (g.standard_normal((Co, Ci, kH, kW), dtype=np.float32) * np.float32(np.sqrt(2.0 / (Ci * kH * kW))))
    b = (g.standard_normal(Co, dtype=np.float32) * np.float32(0.1))
    spec = {"type": "conv", "weight": w, "bias": b, "dW": dW, "dH": dH, "padW": pW, "padH": pH, "mm": "virt"}
    return x, spec


# (B, C, H, W, kH, kW, dH, dW, padH, padW, ceil_mode)
POOL_CASES = [
    (2, 3, 55, 55, 3, 3, 2, 2, 0, 0, 0),
    (1, 4, 13, 13, 3, 3, 2, 2, 0, 0, 1),
    (2, 5, 28, 28, 3, 3, 2, 2, 1, 1, 0),
    (3, 2, 7, 9, 2, 2, 2, 2, 1, 1, 1),
    (1, 3, 6, 6, 3, 3, 3, 3, 1, 1, 1),
    (2, 2, 10, 8, 2, 3, 1, 2, 0, 1, 0),
]


def pool_case(i):
    B, Cn, H, W = POOL_CASES[i][:4]
    return rng(200 + i).standard_normal((B, Cn, H, W), dtype=np.float32)


def pool_spec(i, kind="maxpool"):
    _, _, _, _, kH, kW, dH, dW, pH, pW, ceil = POOL_CASES[i]
    s = {"type": kind, "kW": kW, "kH": kH, "dW": dW, "dH": dH, "padW": pW, "padH": pH, "ceil_mode": ceil}
    if kind == "avgpool":
        s["count_include_pad"] = i % 2
    return s


LINEAR_CASES = [(1, 37, 11), (1, 1024, 300), (4, 129, 65), (16, 512, 100), (1, 9216, 64)]


def linear_case(i):
    B, nIn, nOut = LINEAR_CASES[i]
    g = rng(300 + i)
    x = g.standard_normal((B, nIn), dtype=np.float32)
    if B == 1:
        x = x[0]
    w = g.standard_normal((nOut, nIn), dtype=np.float32) * np.float32(np.sqrt(2.0 / nIn))
    b = g.standard_normal(nOut, dtype=np.float32) * np.float32(0.1)
    return x, {"type": "linear", "weight": w, "bias": b}


SOFTMAX_SHAPES = [(10,), (3, 1000), (7, 4, 5), (2, 21, 3, 3)]


def softmax_case(i):
    return (rng(400 + i).standard_normal(SOFTMAX_SHAPES[i], dtype=np.float32) * np.float32(4.0)).astype(np.float32)


def bn_case(seed=500, shape=(3, 6, 5, 4)):
    g = rng(seed)
    x = g.standard_normal(shape, dtype=np.float32)
    c = shape[1]
    spec = {"type": "bn", "running_mean": g.standard_normal(c, dtype=np.float32) * np.float32(0.3),
            "running_var": g.uniform(0.5, 1.5, c).astype(np.float32),
            "weight": g.uniform(0.5, 1.5, c).astype(np.float32),
            "bias": g.standard_normal(c, dtype=np.float32) * np.float32(0.1), "eps": 1e-5}
    return x, spec


def small_networks():
    """Whole networks small enough for the CPU checkers: name -> config dict."""
    nets = {}
    nets["vgg16_small"] = configs.vgg16(seed=3, batch=2, scale=1 / 8, side=32)
    nets["resnet18_small"] = configs.resnet18(seed=4, batch=4, scale=1 / 8, side=64)
    g = rng(600)
    w1 = g.standard_normal((8, 3, 3, 3), dtype=np.float32) * np.float32(0.3)
    w2 = g.standard_normal((10, 8 * 4 * 4), dtype=np.float32) * np.float32(0.1)
    nets["tiny_cnn"] = {
        "name": "tiny_cnn",
        "layers": [conv(w1, g.standard_normal(8, dtype=np.float32) * np.float32(0.1), 1, 1), relu(), maxpool(2, 2),
                   {"type": "view", "numElements": 128},
                   {"type": "linear", "weight": w2, "bias": g.standard_normal(10, dtype=np.float32) * np.float32(0.1)},
                   {"type": "softmax"}],
        "input": g.uniform(0, 1, (3, 3, 8, 8)).astype(np.float32),
        "mean": (0.4, 0.5, 0.6), "std": (0.2, 0.25, 0.3)}
    g = rng(601)

    def wgt(*shape):
        fan = np.prod(shape[1:]) if len(shape) == 4 else shape[0]
        return (g.standard_normal(shape, dtype=np.float32) * np.float32(np.sqrt(1.0 / fan))).astype(np.float32)

    def fullconv(w, b, d=1, pad=0, adj=0):
        return {"type": "fullconv", "weight": w, "bias": b, "dW": d, "dH": d, "padW": pad, "padH": pad, "adjW": adj, "adjH": adj}
    # encoder / decoder: poolings whose indices steer SpatialMaxUnpooling, full convolutions
    # with and without a bias (the reference scales by 11 when there is one), strides 1 and 2
    nets["segnet_small"] = {
        "name": "segnet_small",
        "layers": [conv(wgt(8, 3, 3, 3), wgt(8) * np.float32(0.1), 1, 1), relu(), maxpool(2, 2),
                   conv(wgt(16, 8, 3, 3), wgt(16) * np.float32(0.1), 1, 1), relu(), maxpool(3, 2, 1),
                   fullconv(wgt(16, 16, 3, 3) * np.float32(0.1), wgt(16) * np.float32(0.1), 1, 1),
                   {"type": "maxunpool", "pooling": 5},
                   fullconv(wgt(16, 8, 3, 3) * np.float32(0.1), wgt(8) * np.float32(0.1), 1, 1), relu(),
                   {"type": "maxunpool", "pooling": 2},
                   fullconv(wgt(8, 4, 2, 2), None, 2, 0),
                   fullconv(wgt(4, 3, 3, 3) * np.float32(0.1), wgt(3) * np.float32(0.1), 2, 1, 1)],
        "input": g.uniform(0, 1, (2, 3, 16, 16)).astype(np.float32),
        "mean": (0.4, 0.5, 0.6), "std": (0.2, 0.25, 0.3)}
    return nets


# (B, Ci, H, W, Co, kH, kW, dH, dW, padH, padW, adjH, adjW, bias)
FULLCONV_CASES = [
    (2, 8, 5, 6, 4, 3, 3, 1, 1, 1, 1, 0, 0, True),
    (1, 16, 7, 7, 12, 2, 2, 2, 2, 0, 0, 0, 0, False),
    (3, 5, 4, 9, 7, 3, 3, 2, 2, 1, 1, 1, 1, True),
    (2, 32, 8, 8, 16, 4, 4, 2, 2, 1, 1, 0, 0, True),
    (1, 3, 6, 5, 2, 5, 3, 3, 2, 2, 0, 2, 1, False),
    (2, 64, 12, 12, 3, 2, 2, 2, 2, 0, 0, 0, 0, True),
]


def fullconv_case(i):
    B, Ci, H, W, Co, kH, kW, dH, dW, pH, pW, aH, aW, has_bias = FULLCONV_CASES[i]
    g = rng(800 + i)
    x = g.standard_normal((B, Ci, H, W), dtype=np.float32)
    w = g.standard_normal((Ci, Co, kH, kW), dtype=np.float32) * np.float32(np.sqrt(1.0 / (Ci * kH * kW)))
    b = g.standard_normal(Co, dtype=np.float32) * np.float32(0.5) if has_bias else None
    spec = {"type": "fullconv", "weight": w, "bias": b, "dW": dW, "dH": dH, "padW": pW, "padH": pH, "adjW": aW, "adjH": aH}
    return x, spec


def sample_indices(n, count=4096, seed=7):
    """Deterministic strided sample of a flat tensor (for large outputs)."""
    if n <= count:
        return np.arange(n)
    return np.sort(rng(seed).choice(n, count, replace=False))


def tensor_summary(y):
    """What the full-size golden files keep of one module output: shape, a strided sample,
    sum, sum of squares and max|.| of the whole tensor, and the sum of every (image, plane)
    slice (every element is in one of them) -- float64 accumulation, stored as float32."""
    a = np.ascontiguousarray(y, np.float32)
    flat = a.ravel()
    d = flat.astype(np.float64)
    out = {"shape": np.array(a.shape, np.int64), "sample": flat[sample_indices(flat.size)],
           "sum": np.array(d.sum()), "sumsq": np.array((d * d).sum()), "absmax": np.array(np.abs(flat).max())}
    if a.ndim == 4:
        out["psum"] = d.reshape(a.shape[0] * a.shape[1], -1).sum(axis=1).astype(np.float32)
    elif a.ndim == 2:
        out["psum"] = d.reshape(a.shape).sum(axis=1).astype(np.float32)
    else:
        out["psum"] = np.array([d.sum()], np.float32)
    return out
