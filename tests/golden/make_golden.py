"""Writes tests/golden/fp32_golden.npz with outputs of the REFERENCE's own CPU library.

Run in a container where oracle/_ref has been built from the mounted reference tree
(`make -C oracle`).  Inputs and weights are regenerated from seeds by tests/cases.py
and thnets_amd/configs.py, so only outputs are stored (large ones as a strided
sample plus sum / sum of squares).  The library is driven through the same
`struct module` arrays the HIP engine receives; nothing from the reference is
imported as Python.

    python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

import cases  # noqa: E402
from oracle.oracle_py import Reference  # noqa: E402
from thnets_amd import configs  # noqa: E402


def run_single(ref, spec, x):
    hn = ref.host_network({"layers": [spec], "mean": (0, 0, 0), "std": (1, 1, 1)})
    return ref.forward(hn, x)


def summary(prefix, y, out):
    flat = np.ascontiguousarray(y, np.float32).ravel()
    idx = cases.sample_indices(flat.size)
    out[prefix + "/shape"] = np.array(y.shape, np.int64)
    out[prefix + "/sample"] = flat[idx]
    out[prefix + "/sum"] = np.array(flat.astype(np.float64).sum())
    out[prefix + "/sumsq"] = np.array((flat.astype(np.float64) ** 2).sum())


def main():
    ref = Reference()
    out = {}
    for i in range(len(cases.CONV_CASES)):
        x, spec = cases.conv_case(i)
        out["conv%d" % i] = run_single(ref, spec, x)
        spec_mm = dict(spec, mm="mm")
        assert np.array_equal(run_single(ref, spec_mm, x), out["conv%d" % i]), "MM and VirtMM differ"
    for i in range(len(cases.POOL_CASES)):
        x = cases.pool_case(i)
        out["maxpool%d" % i] = run_single(ref, cases.pool_spec(i, "maxpool"), x)
        out["avgpool%d" % i] = run_single(ref, cases.pool_spec(i, "avgpool"), x)
    for i in range(len(cases.LINEAR_CASES)):
        x, spec = cases.linear_case(i)
        out["linear%d" % i] = run_single(ref, spec, x)
    for i in range(len(cases.SOFTMAX_SHAPES)):
        out["softmax%d" % i] = run_single(ref, {"type": "softmax"}, cases.softmax_case(i))
    x, spec = cases.bn_case()
    out["bn0"] = run_single(ref, spec, x)
    g = cases.rng(700)
    xt = g.standard_normal((2, 3, 4, 5), dtype=np.float32)
    for j, (thr, val, alpha, inplace) in enumerate([(0, 0, 0, 1), (0.25, -1.5, 0, 0), (0.25, -1.5, 0, 1), (0, 0, 0.1, 0)]):
        out["threshold%d" % j] = run_single(ref, {"type": "threshold", "threshold": thr, "val": val, "alpha": alpha,
                                                   "inplace": inplace}, xt)
    # the table "addition" as shipped: two and three branches of 1x1 convolutions
    ws = [g.standard_normal((4, 3, 1, 1), dtype=np.float32) for _ in range(3)]
    for nb in (2, 3):
        layers = [{"type": "concattable", "branches": [[cases.conv(w, None)] for w in ws[:nb]]}, {"type": "caddtable"}]
        hn = ref.host_network({"layers": layers, "mean": (0, 0, 0), "std": (1, 1, 1)})
        out["caddtable%d" % nb] = ref.forward(hn, xt)
    for i in range(len(cases.FULLCONV_CASES)):
        x, spec = cases.fullconv_case(i)
        out["fullconv%d" % i] = run_single(ref, spec, x)
    # a pooling with overlapping windows, its indices, and the unpooling of a second tensor by them
    g = cases.rng(701)
    xp = g.standard_normal((2, 3, 9, 8), dtype=np.float32)
    for j, (k, d, pad) in enumerate([(2, 2, 0), (3, 2, 1), (3, 1, 1)]):
        layers = [cases.maxpool(k, d, pad), {"type": "threshold", "threshold": -0.2, "val": 7.0, "alpha": 0, "inplace": 0},
                  {"type": "maxunpool", "pooling": 0}]
        hn = ref.host_network({"layers": layers, "mean": (0, 0, 0), "std": (1, 1, 1)})
        out["maxunpool%d" % j] = ref.forward(hn, xp)
    for name, cfg in cases.small_networks().items():
        hn = ref.host_network(cfg)
        out["net_" + name] = ref.process_float(hn, cfg["input"])
    cfg = configs.config1()
    summary("config1", run_single_net(ref, cfg), out)
    cfg = configs.alexnet_owt()
    hn = ref.host_network(cfg)
    out["alexnet_b1"] = ref.process_float(hn, cfg["input"])
    path = os.path.join(ROOT, "tests", "golden", "fp32_golden.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, os.path.getsize(path), "bytes,", len(out), "arrays")


def run_single_net(ref, cfg):
    hn = ref.host_network(cfg)
    return ref.forward(hn, cfg["input"])


if __name__ == "__main__":
    main()
