"""THLoadNetwork / THLoadTensor (Torch7 model directories, thapi.c:244-333, thload.c).

No GPU is needed: the loader is host code.  The reference ships no .t7 file, so
the files come from this repository's writer (thnets_amd/t7.py); the writer is
pinned by the reference's own reader where oracle/_ref exists (the same files
load there and its CPU forward gives the outputs of the network they were made
from), and the loader by comparing the `struct module` array it builds with the
one assembled by hand from the same weights.
"""
import ctypes as C
import os
import subprocess
import sys

import numpy as np
import pytest

import cases
from thnets_amd import abi, api, t7
from thnets_amd.abi import ABI, MT
from thnets_amd.netbuild import conv, maxpool, relu, tensor_to_numpy

ERR_OPENFILE, ERR_READFILE, ERR_NOTIMPLEMENTED, ERR_CORRUPTED, ERR_WRONGOBJECT = -1, -2, -3, -4, -5
MT_NAME = {v: k for k, v in MT.items()}


@pytest.fixture(scope="module")
def lib():
    return api.load_library()       # dlopen only: no GPU call is made in this file


def _tensor(pt):
    if not pt or not pt.contents.storage:
        return None
    return tensor_to_numpy(ABI, pt)


def describe(pnet):
    """struct network* -> nested python description (types, parameters, weights)."""
    out = []
    net = pnet.contents
    for i in range(net.nelem):
        m = net.modules[i]
        name = MT_NAME[m.type]
        d = {"type": name}
        if name.startswith("MT_SpatialConvolution"):
            c = m.SpatialConvolution
            d["type"] = "conv"
            for k in ("dW", "dH", "padW", "padH", "kW", "kH", "nInputPlane", "nOutputPlane"):
                d[k] = getattr(c, k)
            d["weight"], d["bias"] = _tensor(c.weight), _tensor(c.bias)
        elif name == "MT_Linear":
            d["weight"], d["bias"] = _tensor(m.Linear.weight), _tensor(m.Linear.bias)
        elif name == "MT_Threshold":
            d.update(threshold=m.Threshold.threshold, val=m.Threshold.val, alpha=m.Threshold.alpha)
        elif name in ("MT_SpatialMaxPooling", "MT_SpatialAveragePooling"):
            p = m.SpatialMaxPooling
            for k in ("kW", "kH", "dW", "dH", "padW", "padH", "ceil_mode"):
                d[k] = getattr(p, k)
            if name == "MT_SpatialAveragePooling":
                d["count_include_pad"] = m.SpatialAveragePooling.count_include_pad
        elif name == "MT_SpatialFullConvolution":
            c = m.SpatialFullConvolution
            for k in ("dW", "dH", "padW", "padH", "adjW", "adjH", "kW", "kH", "nInputPlane", "nOutputPlane"):
                d[k] = getattr(c, k)
            d["weight"], d["bias"] = _tensor(c.weight), _tensor(c.bias)
        elif name == "MT_SpatialMaxUnpooling":
            # which module of this network it names (by that module's loader object)
            d["pooling"] = [j for j in range(net.nelem) if net.modules[j].nnmodule and
                            net.modules[j].nnmodule == m.SpatialMaxUnpooling.pooling]
        elif name == "MT_View":
            d["numElements"] = m.View.numElements
        elif name == "MT_SpatialBatchNormalization":
            b = m.SpatialBatchNormalization
            d.update(running_mean=_tensor(b.running_mean), running_var=_tensor(b.running_var), weight=_tensor(b.weight),
                     bias=_tensor(b.bias), eps=b.eps)
        elif name in ("MT_Sequential", "MT_ConcatTable"):
            d["net"] = describe(m.Sequential.net)
        out.append(d)
    return out


def same(a, b, path="net"):
    assert type(a) is type(b), path
    if isinstance(a, list):
        assert len(a) == len(b), path
        for i, (x, y) in enumerate(zip(a, b)):
            same(x, y, "%s[%d]" % (path, i))
    elif isinstance(a, dict):
        assert sorted(a) == sorted(b), path
        for k in a:
            same(a[k], b[k], path + "." + k)
    elif isinstance(a, np.ndarray):
        assert a.shape == b.shape and np.array_equal(a, b), path
    else:
        assert a == b, (path, a, b)


def load(lib, path):
    h = lib.THLoadNetwork(str(path).encode())
    return C.cast(h, C.POINTER(ABI.THNETWORK)) if h else None


def built_description(lib, cfg):
    from thnets_amd.netbuild import HostNetwork
    host = HostNetwork(lib, ABI).build(cfg["layers"], cfg["mean"], cfg["std"])
    return describe(host.thnet.net), host


@pytest.mark.parametrize("name", ["tiny_cnn", "vgg16_small", "resnet18_small", "segnet_small"])
@pytest.mark.parametrize("variant", ["long8", "long4", "conv4d_boolceil"])
def test_loaded_network_equals_hand_built(lib, tmp_path, name, variant):
    cfg = cases.small_networks()[name]
    t7.save_model_dir(str(tmp_path), cfg["layers"], cfg["mean"], cfg["std"], longsize=4 if variant == "long4" else 8,
                      conv_as_4d=variant == "conv4d_boolceil", boolean_ceil=variant == "conv4d_boolceil")
    net = load(lib, tmp_path)
    assert net, lib.THLastError()
    try:
        want, _keep = built_description(lib, cfg)
        same(describe(net.contents.net), want)
        assert net.contents.net.contents.engine == abi.ENGINE_CPU
        assert np.allclose(list(net.contents.mean), cfg["mean"], rtol=0, atol=0) or \
            np.array_equal(np.float32(list(net.contents.mean)), np.float32(cfg["mean"]))
        assert np.array_equal(np.float32(list(net.contents.std)), np.float32(cfg["std"]))
    finally:
        lib.THFreeNetwork(net)


def test_shared_storage_double_tensors_and_missing_stat(lib, tmp_path):
    """Flattened parameters (every weight a view into one storage), Double tensors,
    a module shared by reference, no stat.t7."""
    g = cases.rng(77)
    flat = t7.Storage(g.standard_normal(4 * 6 + 4 + 3 * 4 + 3).astype(np.float64))
    lin1 = t7.Obj("nn.Linear", weight=t7.TensorView(flat, 0, [4, 6], [6, 1]), bias=t7.TensorView(flat, 24, [4], [1]))
    lin2 = t7.Obj("nn.Linear", weight=t7.TensorView(flat, 28, [3, 4], [4, 1]), bias=t7.TensorView(flat, 40, [3], [1]))
    act = t7.Obj("nn.ReLU", threshold=0, val=0, inplace=True)
    model = t7.Obj("nn.Sequential", modules=[lin1, act, lin2, act, t7.Obj("nn.Identity"), t7.Obj("nn.SoftMax")], train=False)
    os.makedirs(tmp_path / "m")
    t7.save(str(tmp_path / "m" / "model.net"), model)
    net = load(lib, tmp_path / "m")
    assert net, lib.THLastError()
    try:
        d = describe(net.contents.net)
        f = flat.data.astype(np.float32)
        assert [m["type"] for m in d] == ["MT_Linear", "MT_Threshold", "MT_Linear", "MT_Threshold", "MT_Dropout", "MT_SoftMax"]
        assert np.array_equal(d[0]["weight"], f[:24].reshape(4, 6)) and np.array_equal(d[0]["bias"], f[24:28])
        assert np.array_equal(d[2]["weight"], f[28:40].reshape(3, 4)) and np.array_equal(d[2]["bias"], f[40:43])
        assert list(net.contents.mean) == [0, 0, 0] and list(net.contents.std) == [1, 1, 1]
    finally:
        lib.THFreeNetwork(net)


def test_make_spatial_on_a_loaded_network(lib, tmp_path):
    """THMakeSpatial (thapi.c:642-690) drops the View and turns Linear into a
    size x size convolution over the same weight memory; freeing stays clean."""
    cfg = cases.small_networks()["tiny_cnn"]
    t7.save_model_dir(str(tmp_path), cfg["layers"], cfg["mean"], cfg["std"])
    net = load(lib, tmp_path)
    try:
        lib.THMakeSpatial(net, 8)
        d = describe(net.contents.net)
        assert [m["type"] for m in d] == ["conv", "MT_Threshold", "MT_SpatialMaxPooling", "conv", "MT_SoftMax"]
        fc = d[3]
        assert (fc["kW"], fc["kH"], fc["nInputPlane"], fc["nOutputPlane"]) == (4, 4, 8, 10)
        assert np.array_equal(fc["weight"], cfg["layers"][4]["weight"])
    finally:
        lib.THFreeNetwork(net)


def test_load_tensor(lib, tmp_path):
    g = cases.rng(78)
    x = g.standard_normal((2, 3, 5, 4)).astype(np.float32)
    st = t7.Storage(np.arange(40, dtype=np.float64))
    for nm, obj, want in (("a.t7", x, x), ("b.t7", t7.TensorView(st, 3, [3, 4], [8, 2]),
                                         np.arange(40, dtype=np.float32)[3:][:24].reshape(3, 8)[:, ::2][:, :4])):
        for ls in (8, 4):
            t7.save(str(tmp_path / nm), obj, ls)
            h = lib.THLoadTensor(str(tmp_path / nm).encode())
            assert h, lib.THLastError()
            got = tensor_to_numpy(ABI, C.cast(h, ABI.PTensor))
            lib.THFloatTensor_free(h)
            assert np.array_equal(got, want)
    t7.save(str(tmp_path / "n.t7"), {"a": 1})
    assert not lib.THLoadTensor(str(tmp_path / "n.t7").encode()) and lib.THLastError() == ERR_WRONGOBJECT


def test_recoverable_errors(lib, tmp_path):
    """Loader failures return 0 and leave a code (thnets.h:16-22), like the reference."""
    assert load(lib, tmp_path / "nowhere") is None and lib.THLastError() == ERR_OPENFILE
    cfg = cases.small_networks()["tiny_cnn"]
    t7.save_model_dir(str(tmp_path), cfg["layers"], cfg["mean"], cfg["std"])
    whole = open(tmp_path / "model.net", "rb").read()
    for cut in (3, 40, len(whole) // 2, len(whole) - 5):
        open(tmp_path / "model.net", "wb").write(whole[:cut])
        assert load(lib, tmp_path) is None and lib.THLastError() in (ERR_READFILE, ERR_CORRUPTED), cut
    open(tmp_path / "model.net", "wb").write(b"\x63\x00\x00\x00" + whole[4:])
    assert load(lib, tmp_path) is None and lib.THLastError() == ERR_CORRUPTED
    t7.save(str(tmp_path / "model.net"), {"not": "a module"})
    assert load(lib, tmp_path) is None and lib.THLastError() == ERR_WRONGOBJECT
    # a stat.t7 that is not {mean, std} (thapi.c:308-318)
    t7.save_model_dir(str(tmp_path), cfg["layers"], cfg["mean"], cfg["std"])
    t7.save(str(tmp_path / "stat.t7"), {"mean": np.float32([1, 2, 3])})
    assert load(lib, tmp_path) is None and lib.THLastError() == ERR_WRONGOBJECT


FATAL = r"""
import sys
sys.path.insert(0, %r)
from thnets_amd import api
lib = api.load_library()
lib.THLoadNetwork(%r)
print("survived")
"""


def test_unknown_module_is_fatal(tmp_path):
    """thload.c:776: THError -> message on stderr and exit(-1)."""
    model = t7.Obj("nn.Sequential", modules=[t7.Obj("nn.SpatialFractionalMaxPooling", kW=2)])
    t7.save(str(tmp_path / "model.net"), model)
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, "-c", FATAL % (root, str(tmp_path).encode())], capture_output=True, text=True, timeout=120)
    assert r.returncode != 0 and "survived" not in r.stdout
    assert "Unknown module type nn.SpatialFractionalMaxPooling" in r.stderr


def test_python_reader_round_trip(tmp_path):
    g = cases.rng(79)
    w = g.standard_normal((3, 4)).astype(np.float32)
    obj = {"n": 1.5, "s": "text", "b": True, "nil": None, "list": [1, 2, 3], "t": w,
           "o": t7.Obj("nn.Linear", weight=w, bias=np.float64([1, 2, 3])), "ls": t7.Storage(np.int64([7, 8]))}
    for ls in (8, 4):
        t7.save(str(tmp_path / "x.t7"), obj, ls)
        r = t7.load(str(tmp_path / "x.t7"), ls)
        assert r["n"] == 1.5 and r["s"] == "text" and r["b"] is True and r["nil"] is None
        assert r["list"] == {1.0: 1.0, 2.0: 2.0, 3.0: 3.0}
        assert np.array_equal(r["t"], w) and r["o"].cls == "nn.Linear"
        assert r["o"].fields["weight"] is r["t"]                  # written once, referenced after
        assert np.array_equal(r["o"].fields["bias"], [1, 2, 3]) and np.array_equal(r["ls"].data, [7, 8])


# ---- the writer against the reference's own reader and CPU forward ----

@pytest.mark.parametrize("name", ["tiny_cnn", "vgg16_small", "resnet18_small", "segnet_small"])
def test_reference_reads_the_same_files(reference, tmp_path, name):
    """The files this repository writes load in the reference (THLoadNetwork,
    thapi.c:244-333) and its CPU forward on them equals its forward on the network
    assembled by hand from the same weights."""
    cfg = cases.small_networks()[name]
    t7.save_model_dir(str(tmp_path), cfg["layers"], cfg["mean"], cfg["std"])
    L = reference.lib
    L.THLoadNetwork.restype = C.c_void_p
    L.THLoadNetwork.argtypes = [C.c_char_p]
    h = L.THLoadNetwork(str(tmp_path).encode())
    assert h
    net = C.cast(h, C.POINTER(reference.abi.THNETWORK))
    assert np.array_equal(np.float32(list(net.contents.mean)), np.float32(cfg["mean"]))
    assert np.array_equal(np.float32(list(net.contents.std)), np.float32(cfg["std"]))

    class Loaded:
        thnet = net.contents
    got = reference.process_float(Loaded, cfg["input"])
    want = reference.process_float(reference.host_network(cfg), cfg["input"])
    assert got.shape == want.shape and np.array_equal(got, want)
