"""thhip_linear_batched_noalloc -- the entry point that allocates nothing -- against
thhip_linear_batched (same kernels: the same bits) and against the CPU oracle, through
the C ABI: two calls in a row, the second with a smaller input, so what the first call
left in the fixed device array must not leak into the second; then a batch that runs in
two slices, the half types, and the rejection of a shape whose partial sums do not fit."""
import numpy as np
import pytest

import cases
import gpu_util as G
from thnets_amd import api

pytestmark = pytest.mark.gpu


def both(lib, oracle, B, nIn, nOut, act, dtype, seed, tol):
    g = cases.rng(seed)
    x = g.standard_normal((B, nIn), dtype=np.float32)
    w = g.standard_normal((nOut, nIn), dtype=np.float32) * np.float32(np.sqrt(2.0 / nIn))
    b = g.standard_normal(nOut, dtype=np.float32) * np.float32(0.1)
    G.note("linear_batched_noalloc B=%d %d->%d act=%d dtype=%d" % (B, nIn, nOut, act, dtype))
    dx, dw = api.to_device_dtype(lib, x, dtype), api.to_device_dtype(lib, w, dtype)
    db = api.DeviceArray(lib, b)
    es = 4 if dtype == G.F32 else 2
    dy0 = api.DeviceArray(lib, nbytes=B * nOut * es)
    dy1 = api.DeviceArray(lib, nbytes=B * nOut * es)
    lib.thhip_memset(dy0.ptr, 0xFF, B * nOut * es)
    lib.thhip_memset(dy1.ptr, 0xFF, B * nOut * es)
    lib.thhip_linear_batched(dx.ptr, dw.ptr, db.ptr, dy0.ptr, B, nIn, nOut, act, 0.1, -0.5, dtype)
    # the property the entry point is named for: not one allocating request (device or page-locked
    # memory, events) reaches the HIP runtime during the call, with the per-launch profiler off and on
    for prof in (0, 1):
        lib.thhip_profile_enable(prof)
        if prof:        # the profiler's event pool fills on first use; the library's own calls may allocate
            lib.thhip_linear_batched(dx.ptr, dw.ptr, db.ptr, dy0.ptr, B, nIn, nOut, act, 0.1, -0.5, dtype)
        before = lib.thhip_alloc_calls()
        rc = lib.thhip_linear_batched_noalloc(dx.ptr, dw.ptr, db.ptr, dy1.ptr, B, nIn, nOut, act, 0.1, -0.5, dtype)
        assert rc == 0
        assert lib.thhip_alloc_calls() == before, "thhip_linear_batched_noalloc allocated (profiling %d)" % prof
    lib.thhip_profile_enable(0)
    lib.thhip_sync()
    want = api.from_device_dtype(dy0, (B, nOut), dtype)
    got = api.from_device_dtype(dy1, (B, nOut), dtype)
    assert np.array_equal(got, want), "differs from thhip_linear_batched"
    ref = oracle.linear(x, w, b)
    if act:
        ref = np.where(ref > np.float32(0.1), ref, np.float32(-0.5)).astype(np.float32)
    G.assert_close(got, ref, tol, "vs oracle")


def test_noalloc_linear_two_calls_second_smaller(hiplib, oracle):
    assert hiplib.thhip_linear_batched_noalloc_init() == 0
    assert hiplib.thhip_linear_batched_noalloc_limit() == 8 << 20
    # a wide layer (four row blocks per wavefront, K split 8: 2 MiB of partial sums) ...
    both(hiplib, oracle, 16, 25088, 4096, 1, G.F32, 2100, 2e-5)
    # ... then a small ragged one that reuses the front of the same array
    both(hiplib, oracle, 5, 516, 70, 0, G.F32, 2101, 2e-5)
    both(hiplib, oracle, 3, 1024, 33, 1, G.F32, 2102, 2e-5)
    # 40 rows (four column groups), 100 rows (two slices), and the half types
    both(hiplib, oracle, 40, 4096, 1000, 0, G.F32, 2103, 2e-5)
    both(hiplib, oracle, 100, 1024, 1100, 1, G.F32, 2106, 2e-5)
    both(hiplib, oracle, 16, 4096, 4096, 0, G.F16, 2104, 2e-2)   # (no threshold: a rounded value may fall on its other side)
    both(hiplib, oracle, 7, 2048, 100, 0, G.BF16, 2105, 6e-2)


def test_noalloc_linear_rejects_what_does_not_fit(hiplib, capfd):
    """32 rows x 100000 outputs x 4 bytes of partial sums > 8 MiB: refused before anything
    is launched (the operands are never touched, so small buffers stand in for them)."""
    d = api.DeviceArray(hiplib, nbytes=4096)
    assert hiplib.thhip_linear_batched_noalloc(d.ptr, d.ptr, None, d.ptr, 32, 1024, 100000, 0, 0.0, 0.0, G.F32) == -2
    assert "needs 12800000 bytes" in capfd.readouterr().err
    assert hiplib.thhip_linear_batched_noalloc(d.ptr, d.ptr, None, d.ptr, 4, 1023, 8, 0, 0.0, 0.0, G.F32) == -1
    hiplib.thhip_sync()
