"""Writes tests/golden/alexnet_lowp_b64_golden.npz: configuration 5 (the AlexNet-OWT
shape through the uint8 path, range 32) for ALL 64 images of the batch.

The codes come from the CPU restatement under oracle/ (`lowp_run_layers`: one image
at a time with the batch's one (mult, sub), the way the reference's LOWP engine has
to be driven - lowp/lowp_SpatialConvolution.c:124-187, lowp/lowp_basic.c:5-38,
299-321).  Stored per module: the CRC-32 and the sum of every image's codes and the
module's (mult, sub); in full: the codes of the last module (64 x 1000) and the
quantisation of the input.  Inputs and weights are regenerated from seeds by
thnets_amd/configs.py.

    python tests/golden/make_golden_lowp.py
"""
import os
import sys
import zlib

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

from oracle.oracle_py import Oracle  # noqa: E402
from thnets_amd import configs  # noqa: E402

PATH = os.path.join(ROOT, "tests", "golden", "alexnet_lowp_b64_golden.npz")


def image_checksums(q):
    """(CRC-32, sum) of each image's codes of one module output [B, ...]."""
    q = np.ascontiguousarray(q, np.uint8)
    crc = np.array([zlib.crc32(q[b].tobytes()) for b in range(q.shape[0])], np.uint32)
    tot = q.reshape(q.shape[0], -1).sum(axis=1, dtype=np.int64)
    return crc, tot


def main():
    oracle = Oracle()
    cfg = configs.alexnet_lowp(batch=64)
    x = oracle.normalize(cfg["input"], cfg["mean"], cfg["std"])
    xq, im, isub = oracle.lowp_quantize(x)
    out = {"input/quant": np.array([im, isub], np.float32)}
    out["input/crc"], out["input/sum"] = image_checksums(xq)
    outs = []
    for b0 in range(0, 64, 8):
        part = []
        q, m, s = oracle.lowp_run_layers(cfg["layers"], xq[b0:b0 + 8], im, isub, cfg["range"], collect=part)
        outs.append(part)
    for i in range(len(cfg["layers"])):
        q = np.concatenate([part[i][0] for part in outs])
        assert all(part[i][1:] == outs[0][i][1:] for part in outs)
        out["module%d/shape" % i] = np.array(q.shape, np.int64)
        out["module%d/quant" % i] = np.array(outs[0][i][1:], np.float32)
        out["module%d/crc" % i], out["module%d/sum" % i] = image_checksums(q)
    out["last/codes"] = q.reshape(64, -1)
    np.savez_compressed(PATH, **out)
    print("wrote", PATH, os.path.getsize(PATH), "bytes")


if __name__ == "__main__":
    main()
