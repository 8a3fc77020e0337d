"""Writes tests/golden/fullsize_golden.npz: every module output of the two full-size
benchmark networks, VGG-16 at batch 16 and ResNet-18 at batch 32 (224 x 224), as the
REFERENCE's own CPU library computes them.

Run in a container where oracle/_ref has been built from the mounted reference tree
(`make -C oracle`).  The library is driven through the same `struct module` arrays the
HIP engine receives, one module's updateOutput at a time (its executor, thapi.c:158-235,
frees every output as soon as the next module has run), walking ConcatTable branches
and their Sequential containers the way ConcatTable.c:20-50 and Sequential.c:20-51 do,
so the outputs of the modules inside the residual blocks are seen too.  A module's output
is summarised right after its call, before an in-place Threshold (Threshold.c:47-53)
overwrites it.  Outputs are numbered like the flat graph form of the network
(thnets_amd.configs.to_graph): positions of a ConcatTable and of an identity branch do
not appear.  Thread counts divide the batch (the batched convolution hangs otherwise,
OpenBLAS-stripped/sgemm.c:967-979).  Inputs and weights are regenerated from seeds, so
only summaries of the outputs are stored (tests/cases.py:tensor_summary).

    python tests/golden/make_golden_fullsize.py
"""
import ctypes as C
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

import cases  # noqa: E402
from oracle.oracle_py import Reference  # noqa: E402
from thnets_amd import configs  # noqa: E402
from thnets_amd.netbuild import tensor_to_numpy  # noqa: E402

UPDATE = C.CFUNCTYPE(C.c_void_p, C.c_void_p, C.c_void_p)


def stepwise(ref, cfg):
    """Runs cfg's network module by module; returns the list of output summaries in
    graph-form order."""
    hn = ref.host_network(cfg)
    x = np.array(cfg["input"], np.float32, copy=True, order="C")
    ref.set_threads(ref.threads_for_batch(x.shape[0]))
    ref.lib.THFloatTensor_set.argtypes = [C.c_void_p, C.c_void_p]
    ref.lib.THFloatTensor_set.restype = None
    outs = []

    def call(mod, tin, record=True):
        out = UPDATE(mod.updateOutput)(C.addressof(mod), tin)
        if record:
            y = tensor_to_numpy(ref.abi, C.cast(out, ref.abi.PTensor), copy=False)
            outs.append(cases.tensor_summary(y))
        return out

    cur = C.addressof(hn.tensor(x).contents)
    mods = hn.thnet.net.contents.modules
    for i, spec in enumerate(cfg["layers"]):
        m = mods[i]
        if spec["type"] != "concattable":
            cur = call(m, cur)
            continue
        table = m.ConcatTable.net.contents
        for j, branch in enumerate(spec["branches"]):
            bm = table.modules[j]
            if len(branch) == 1:
                call(bm, cur, record=branch[0]["type"] != "dropout")
                continue
            seq = bm.Sequential.net.contents
            t = cur
            for k in range(len(branch)):
                t = call(seq.modules[k], t)
            ref.lib.THFloatTensor_set(C.cast(bm.output, C.c_void_p), t)      # Sequential.c:49
        cur = C.addressof(m)        # "the table is the module itself", ConcatTable.c:49
    return outs, hn


def main():
    ref = Reference()
    out = {}
    for name, cfg in (("vgg16_b16", configs.vgg16(batch=16)), ("resnet18_b32", configs.resnet18(batch=32))):
        t0 = time.time()
        outs, hn = stepwise(ref, cfg)
        graph = configs.to_graph(cfg["layers"])
        assert len(outs) == len(graph), (len(outs), len(graph))
        for pos, s in enumerate(outs):
            for k, v in s.items():
                out["%s/%d/%s" % (name, pos, k)] = v
        # the module-by-module walk must be what the library's own executor computes
        y = ref.process_float(ref.host_network(cfg), cfg["input"])
        assert np.array_equal(y[cases.sample_indices(y.size)], outs[-1]["sample"]), name
        out["%s/output" % name] = y
        print(name, "%d outputs, %.1f s" % (len(outs), time.time() - t0), flush=True)
        del hn
    path = os.path.join(ROOT, "tests", "golden", "fullsize_golden.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, os.path.getsize(path), "bytes,", len(out), "arrays")


if __name__ == "__main__":
    main()
