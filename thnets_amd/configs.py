"""Seeded synthetic networks for the five benchmark / parity configurations.

No model files exist for the reference offline, so every network is random-init
with a fixed seed: weights He-normal (sigma = sqrt(2 / fan_in)), biases N(0, 0.01),
from numpy's PCG64 stream ``np.random.Generator(np.random.PCG64(seed))``.  The same
function is called by the engine side and the checker side, so both see identical
bytes.  ``scale`` < 1 shrinks channel counts (and the image, for the whole-network
configurations) so that a CPU checker finishes in seconds; scale = 1 is the real
shape.
"""
import numpy as np

from .netbuild import conv, maxpool, relu

IMAGENET_MEAN = (0.485, 0.456, 0.406)
IMAGENET_STD = (0.229, 0.224, 0.225)


def _rng(seed):
    return np.random.Generator(np.random.PCG64(seed))


def _he(rng, shape, fan_in):
    return (rng.standard_normal(shape, dtype=np.float32) * np.float32(np.sqrt(2.0 / fan_in))).astype(np.float32)


def _bias(rng, n):
    return (rng.standard_normal(n, dtype=np.float32) * np.float32(0.01)).astype(np.float32)


def _conv(rng, ci, co, k, d=1, pad=0):
    return conv(_he(rng, (co, ci, k, k), ci * k * k), _bias(rng, co), d=d, pad=pad)


def _linear(rng, nin, nout):
    return {"type": "linear", "weight": _he(rng, (nout, nin), nin), "bias": _bias(rng, nout)}


def config1(seed=1):
    """Single conv 64->128 3x3/s1/p1 on 1x64x56x56 + ReLU (GEMM M=128 K=576 N=3136)."""
    rng = _rng(seed)
    x = rng.uniform(-1.0, 1.0, (1, 64, 56, 56)).astype(np.float32)
    layers = [_conv(rng, 64, 128, 3, 1, 1), relu()]
    return {"name": "config1_conv64x128", "layers": layers, "input": x, "mean": (0, 0, 0), "std": (1, 1, 1)}


def alexnet_owt(seed=2, batch=1, spatial=False, softmax=True):
    """AlexNet-OWT shape (profilealexnetowt.lua:8-31 of the reference, Dropout left
    out as the configuration lists none).  ``spatial`` gives the THMakeSpatial form
    (thapi.c:642-690): View dropped, fc6 a 6x6 convolution, fc7/fc8 1x1."""
    rng = _rng(seed)
    layers = [
        _conv(rng, 3, 64, 11, 4, 2), relu(), maxpool(3, 2),
        _conv(rng, 64, 192, 5, 1, 2), relu(), maxpool(3, 2),
        _conv(rng, 192, 384, 3, 1, 1), relu(),
        _conv(rng, 384, 256, 3, 1, 1), relu(),
        _conv(rng, 256, 256, 3, 1, 1), relu(), maxpool(3, 2),
    ]
    fc6, fc7, fc8 = _linear(rng, 9216, 4096), _linear(rng, 4096, 4096), _linear(rng, 4096, 1000)
    if spatial:
        def as_conv(lin, ci, k):
            w = lin["weight"].reshape(lin["weight"].shape[0], ci, k, k)
            return conv(w, lin["bias"], d=1, pad=0)
        layers += [as_conv(fc6, 256, 6), relu(), as_conv(fc7, 4096, 1), relu(), as_conv(fc8, 4096, 1)]
    else:
        layers += [{"type": "view", "numElements": 9216}, fc6, relu(), fc7, relu(), fc8]
    if softmax:
        layers.append({"type": "softmax"})
    x = _rng(seed + 1000).uniform(0.0, 1.0, (batch, 3, 224, 224)).astype(np.float32)
    return {"name": "alexnet_owt_b%d%s" % (batch, "_spatial" if spatial else ""), "layers": layers, "input": x,
            "mean": IMAGENET_MEAN, "std": IMAGENET_STD}


VGG16_PLAN = (64, 64, "M", 128, 128, "M", 256, 256, 256, "M", 512, 512, 512, "M", 512, 512, 512, "M")


def vgg16(seed=3, batch=16, scale=1.0, side=224):
    """VGG-16 shape: thirteen 3x3/p1 convolutions, maxpool 2/2 after each block,
    then Linear 25088->4096->4096->1000, ReLU throughout."""
    rng = _rng(seed)
    layers = []
    ci = 3
    s = side
    for v in VGG16_PLAN:
        if v == "M":
            layers.append(maxpool(2, 2))
            s //= 2
        else:
            co = max(4, int(round(v * scale)))
            layers += [_conv(rng, ci, co, 3, 1, 1), relu()]
            ci = co
    nflat = ci * s * s
    h = max(8, int(round(4096 * scale)))
    nout = max(8, int(round(1000 * scale)))
    layers += [{"type": "view", "numElements": nflat}, _linear(rng, nflat, h), relu(), _linear(rng, h, h), relu(),
               _linear(rng, h, nout)]
    x = _rng(seed + 1000).uniform(0.0, 1.0, (batch, 3, side, side)).astype(np.float32)
    return {"name": "vgg16_b%d_s%g_%d" % (batch, scale, side), "layers": layers, "input": x,
            "mean": (0, 0, 0), "std": (1, 1, 1)}


def _bn(rng, c):
    return {"type": "bn",
            "running_mean": (rng.standard_normal(c, dtype=np.float32) * np.float32(0.1)).astype(np.float32),
            "running_var": rng.uniform(0.5, 1.5, c).astype(np.float32),
            "weight": rng.uniform(0.5, 1.5, c).astype(np.float32),
            "bias": (rng.standard_normal(c, dtype=np.float32) * np.float32(0.1)).astype(np.float32),
            "eps": 1e-5}


def _basic_block(rng, ci, co, stride):
    main = [_conv(rng, ci, co, 3, stride, 1), _bn(rng, co), relu(), _conv(rng, co, co, 3, 1, 1), _bn(rng, co)]
    if stride != 1 or ci != co:
        short = [_conv(rng, ci, co, 1, stride, 0), _bn(rng, co)]
    else:
        short = [{"type": "dropout", "p": 0.0, "inplace": 1, "v2": 1}]  # nn.Identity stand-in (Dropout.c:37-53)
    # the reference's CAddTable with two inputs computes branch0 - branch1 (CAddTable.c:59-67)
    return [{"type": "concattable", "branches": [main, short]}, {"type": "caddtable"}, relu()]


def resnet18(seed=4, batch=32, scale=1.0, side=224):
    """ResNet-18 shape: stem 7x7/s2/p3, BN, ReLU, maxpool 3/2/p1, four stages of two
    basic blocks, average pool over the remaining extent, Linear 512->1000.  The
    residual "addition" uses the reference's CAddTable arithmetic (a - b)."""
    rng = _rng(seed)
    w = [max(4, int(round(v * scale))) for v in (64, 128, 256, 512)]
    layers = [_conv(rng, 3, w[0], 7, 2, 3), _bn(rng, w[0]), relu(), maxpool(3, 2, pad=1)]
    ci = w[0]
    for i, co in enumerate(w):
        layers += _basic_block(rng, ci, co, 1 if i == 0 else 2)
        layers += _basic_block(rng, co, co, 1)
        ci = co
    s = side // 32
    layers += [{"type": "avgpool", "kW": s, "kH": s, "dW": 1, "dH": 1, "padW": 0, "padH": 0, "ceil_mode": 0,
                "count_include_pad": 1},
               {"type": "view", "numElements": ci}, _linear(rng, ci, max(8, int(round(1000 * scale))))]
    x = _rng(seed + 1000).uniform(0.0, 1.0, (batch, 3, side, side)).astype(np.float32)
    return {"name": "resnet18_b%d_s%g_%d" % (batch, scale, side), "layers": layers, "input": x,
            "mean": (0, 0, 0), "std": (1, 1, 1)}


def to_graph(layers):
    """The same network as a flat list whose layers name their inputs ("inputs": positions
    in the list), the form the reference's graph loaders produce and its executor routes by
    (thapi.c:173-193): ConcatTable branches are laid out one after the other, an identity
    branch disappears (the table add reads the block's input directly), the table add names
    the branch ends."""
    out, prev, ends = [], None, None
    for spec in layers:
        if spec["type"] == "concattable":
            ends = []
            for branch in spec["branches"]:
                p = prev
                if not (len(branch) == 1 and branch[0]["type"] == "dropout"):
                    for s in branch:
                        out.append(dict(s, inputs=[p] if p is not None else []))
                        p = len(out) - 1
                ends.append(p)
            continue
        if spec["type"] in ("caddtable", "csubtable"):
            out.append(dict(spec, inputs=list(ends)))
        else:
            out.append(dict(spec, inputs=[prev] if prev is not None else []))
        prev = len(out) - 1
    return out


def alexnet_lowp(seed=2, batch=64):
    """Configuration 5: the AlexNet-OWT weights in THMakeSpatial form, to be run
    through the uint8 engine with range 32.  No SoftMax: bit-exactness is asserted on
    the codes of every layer up to fc8."""
    cfg = alexnet_owt(seed=seed, batch=batch, spatial=True, softmax=False)
    cfg["name"] = "alexnet_owt_lowp_b%d" % batch
    cfg["range"] = 32.0
    return cfg
