"""Benchmark of the MI355X thnets engine on the reference's headline workloads.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

One "step" is one THForward of the VGG-16-shape network (fp32, batch 16, 3x224x224,
synthetic seeded input and weights) with the input already resident in HBM; the
value is whole-job images/second.  The same run also measures the convolution kernel
family with HIP events inside the timed region, on the engine's stream: one pair around every run of
convolution launches that nothing else on the stream interrupts (-> "roofline"),
times the same network through THProcessFloat call by call as the reference's CLI does
(-> "process_float": best and mean of at least 20 calls after 2 warm-ups, host
transfers included), THProcessImages on 64 8-bit images beside the same batch as
floats (-> "process_images"), times the uint8 AlexNet-OWT batch-64 network (-> "roofline_int8"
and "extra"), the fp16 VGG-16, AlexNet-OWT batch 1 and ResNet-18 networks (-> "extra"),
what the matrix cores sustain from registers alone (-> "extra"), and the CPU baseline
on the host cores (-> "cpu_baseline": the reference's own CPU library when oracle/_ref
holds a build of it, else this repository's C restatement).  Prints one JSON line.
"""
import argparse
import ctypes as C
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

from thnets_amd import api, configs  # noqa: E402

PEAK_TFLOPS_FP32_MFMA = 157.3
PEAK_TOPS_INT8_MFMA = 5030.0


def counter_traffic(profile, key):
    """HBM bytes per launch as the counter summary under profiles/ states them: the line
    `<key> = <bytes>` of that file (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE of this program,
    scaled against a plain copy of known size), or None when the summary is not there."""
    try:
        with open(os.path.join(ROOT, "profiles", profile)) as f:
            for line in f:
                if line.strip().startswith(key + " ="):
                    return float(line.split("=")[1].split()[0])
    except OSError:
        pass
    return None


def profile_get(lib, fam):
    ms, n, work = C.c_double(), C.c_long(), C.c_double()
    lib.thhip_profile_get(fam, C.byref(ms), C.byref(n), C.byref(work))
    return ms.value, n.value, work.value


def timed_forward(lib, net, steps, warmup, families, profiled=True, timed_families=None, reps=1):
    """W untimed + K timed THForward calls; returns ms/step and per-family
    (ms, launches, work) measured with an event pair around every run of launches of one family
    (no event between two launches of a run: one there costs 3-5 us of stream time, which shows on
    networks of short kernels).  profiled=True: the launches of `timed_families` (default: all of
    `families`) carry their events in the timed steps themselves; the other families, and every
    family with profiled=False, are measured in K further steps.  reps > 1 (the legs under
    "extra" only, never the headline): the K timed steps are run that many times and the
    fastest run counts (a 15 ms run right after a network was built sees the clocks ramp)."""
    if timed_families is None:
        timed_families = families
    if not profiled:
        timed_families = ()
    for _ in range(warmup):
        net.forward()
    lib.thhip_sync()
    best = None
    for _ in range(max(reps, 1)):
        lib.thhip_profile_reset()
        lib.thhip_profile_enable(sum(2 << f for f in timed_families))
        t0 = time.perf_counter()
        lib.thhip_event_record(0)
        for _ in range(steps):
            net.forward()
        lib.thhip_event_record(1)
        lib.thhip_sync()
        wall_ms = (time.perf_counter() - t0) * 1e3 / steps
        dev_ms = lib.thhip_event_ms(0, 1) / steps
        if best is None or max(wall_ms, dev_ms) < max(best[0], best[1]):
            best = (wall_ms, dev_ms, {f: profile_get(lib, f) for f in timed_families})
    wall_ms, dev_ms, fam = best
    rest = [f for f in families if f not in timed_families]
    if rest:
        lib.thhip_profile_reset()
        lib.thhip_profile_enable(1)
        for _ in range(steps):
            net.forward()
        lib.thhip_sync()
        fam.update({f: profile_get(lib, f) for f in rest})
    lib.thhip_profile_enable(0)
    return max(wall_ms, dev_ms), fam


def cpu_baseline(cfg, seconds_budget=25.0):
    """Times the CPU path on this host: THProcessFloat of the reference's own library
    (kind "reference") or the C restatement (kind "port") on the same network."""
    from oracle.oracle_py import Oracle, Reference
    batch = cfg["input"].shape[0]
    cores = os.cpu_count() or 1
    try:
        cores = min(cores, len(os.sched_getaffinity(0)))
    except AttributeError:
        pass
    if Reference.available():
        ref = Reference()
        threads = ref.set_threads(ref.threads_for_batch(batch, limit=min(cores, 16)))
        hn = ref.host_network(cfg)
        ref.process_float(hn, cfg["input"])          # warm-up
        times = []
        t_end = time.perf_counter() + seconds_budget
        while len(times) < 5 and (not times or time.perf_counter() < t_end):
            t0 = time.perf_counter()
            ref.process_float(hn, cfg["input"])
            times.append(time.perf_counter() - t0)
        kind = "reference"
    else:
        orc = Oracle()
        threads = min(orc.threads(), cores, 16)
        orc.set_threads(threads)
        x = orc.normalize(cfg["input"], cfg["mean"], cfg["std"])
        times = []
        t_end = time.perf_counter() + seconds_budget
        while len(times) < 3 and (not times or time.perf_counter() < t_end):
            t0 = time.perf_counter()
            orc.run_layers(cfg["layers"], x)
            times.append(time.perf_counter() - t0)
        kind = "port"
    best = min(times)
    return {"value": round(batch / best, 3), "unit": "images/s", "cores": int(threads), "kind": kind,
            "sample": "%d THProcessFloat calls of the same %s network (batch %d) after one warm-up; best of them"
                      % (len(times), cfg["name"], batch),
            "mean_value": round(batch / (sum(times) / len(times)), 3)}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    # (twenty: the first ~50 ms of work after an idle spell run 1-4 % slower while the clocks settle;
    # measured on one box, 3 warm-up steps 4148 / 4173 images/s, 20 warm-up steps 4204 / 4197)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-int8", action="store_true", help="skip the uint8 AlexNet leg")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this engine runs on one GPU; --gpus %d is not supported (images are independent, so "
              "more GPUs would each take a slice of the batch with replicated weights)" % args.gpus, file=sys.stderr)
        sys.exit(2)

    lib = api.load_library()
    lib.THInit()

    # A plain device-to-device copy of known size: under `rocprofv3 --pmc FETCH_SIZE`
    # / `WRITE_SIZE` its dispatch calibrates the counters (256 MiB read, 256 MiB written).
    cal_bytes = 256 << 20
    ca, cb = api.DeviceArray(lib, nbytes=cal_bytes), api.DeviceArray(lib, nbytes=cal_bytes)
    lib.thhip_memset(ca.ptr, 1, cal_bytes)
    lib.thhip_memcpy_d2d(cb.ptr, ca.ptr, cal_bytes)
    lib.thhip_sync()
    ca.free()
    cb.free()

    # ---- VGG-16 fp32 batch 16 (the headline) ----
    cfg = configs.vgg16(batch=16)
    net = api.HipNetwork(cfg["layers"], cfg["mean"], cfg["std"])
    net.upload(cfg["input"])
    # the convolutions (the roofline's kernel) carry their events in the timed steps; the
    # Linear and pooling figures under "extra" come from a second pass
    ms, fam = timed_forward(lib, net, args.steps, args.warmup, (0, 1, 3), timed_families=(0,))
    conv_ms, conv_n, conv_flops = fam[0]
    value = 16.0 / (ms * 1e-3)
    achieved = conv_flops / (conv_ms * 1e-3) / 1e12 if conv_ms > 0 else 0.0
    roofline = {"bound": "mfma", "achieved": round(achieved, 3), "peak": PEAK_TFLOPS_FP32_MFMA, "unit": "TFLOP/s",
                "frac": round(achieved / PEAK_TFLOPS_FP32_MFMA, 4),
                "traffic": counter_traffic("conv_f32_vgg16_fp32_b16_counters.md", "conv_hbm_bytes_per_launch"),
                "kernel": "conv_f32_patch_kernel (implicit-GEMM convolution, every tap of a 3x3 layer read from one input patch "
                          "per plane in LDS: nine of the 13 convolutions of a step, four of them with the 2x2 max pooling that "
                          "follows in their epilogue; the K parts of an XCD's last tiles added in the kernel) and "
                          "conv_f32_direct_kernel (operands loaded straight into LDS: the three 14x14 layers, K split in three, with "
                          "the kernel that sums the parts); the image layer on conv_stem_kernel<fp32>",
                "launches_per_step": conv_n / args.steps, "avg_launch_ms": round(conv_ms / max(conv_n, 1), 5),
                "flops_per_launch": conv_flops / max(conv_n, 1)}
    extra = {"vgg16_conv_ms_per_step": round(conv_ms / args.steps, 4),
             "vgg16_batched_fc_ms_per_step": round(fam[1][0] / args.steps, 4),
             "vgg16_other_kernels_ms_per_step": round(fam[3][0] / args.steps, 4),
             "method_of_the_other_networks": "each of the networks below: at least twenty warm-up steps (ten at batch 64), then the fastest of three "
                                             "runs of K steps without events; kernel-family rates from K further "
                                             "steps with an event pair around every run of launches of a family"}
    # the HBM-bound kernels of the same step against the 8 TB/s peak: batched Linear (weights read once)
    # and max pooling (input read + output written once)
    if fam[1][0] > 0:
        extra["vgg16_batched_fc_GB/s"] = round(fam[1][2] / (fam[1][0] * 1e-3) / 1e9, 1)
        extra["vgg16_batched_fc_frac_of_hbm_peak"] = round(fam[1][2] / (fam[1][0] * 1e-3) / 8e12, 4)
    if fam[3][0] > 0:
        extra["vgg16_pooling_GB/s"] = round(fam[3][2] / (fam[3][0] * 1e-3) / 1e9, 1)
        extra["vgg16_pooling_frac_of_hbm_peak"] = round(fam[3][2] / (fam[3][0] * 1e-3) / 8e12, 4)
    # the same step through the drop-in call, timed the way the reference's CLI times it (thnets-test.c:161-200:
    # a loop of THProcessFloat calls; its first GPU run is dropped): host normalisation + H2D + kernels + D2H,
    # 2 warm-up calls, then every call on its own (the call normalises its argument in place: each gets a
    # fresh copy, made outside the timed region)
    calls = max(args.steps, 20)
    res, ow, oh = C.POINTER(C.c_float)(), C.c_int(), C.c_int()
    times = []
    for i in range(calls + 2):
        x = np.array(cfg["input"], np.float32, copy=True, order="C")
        t0 = time.perf_counter()
        lib.THProcessFloat(net.handle, x.ctypes.data, 16, 224, 224, 3, C.byref(res), C.byref(ow), C.byref(oh))
        if i >= 2:
            times.append(time.perf_counter() - t0)
    process_float = {"images_per_sec_best": round(16.0 / min(times), 1),
                     "images_per_sec_mean": round(16.0 * len(times) / sum(times), 1), "calls": len(times), "warmup": 2,
                     "what": "B / wall time of one THProcessFloat call of the same network (normalisation on the host, "
                             "H2D of the input, all kernels, D2H of the result): PCIe-inclusive, never `value`"}
    net.free()

    # ---- VGG-16 fp16 batch 16 (THHipHalfFloat(1): fp16 storage and MFMA, fp32 accumulation) ----
    nh = api.HipNetwork(cfg["layers"], cfg["mean"], cfg["std"], half=1)
    nh.upload(cfg["input"])
    msh, famh = timed_forward(lib, nh, args.steps, max(args.warmup, 20), (0, 1, 3), profiled=False, reps=3)
    hc_ms, hc_n, hc_fl = famh[0]
    extra["vgg16_fp16_b16"] = {
        "images_per_sec": round(16.0 / (msh * 1e-3), 1), "ms_per_step": round(msh, 4),
        "conv_TFLOP/s": round(hc_fl / (hc_ms * 1e-3) / 1e12, 1) if hc_ms > 0 else None,
        "frac_of_fp16_mfma_peak": round(hc_fl / (hc_ms * 1e-3) / 1e12 / 2500.0, 4) if hc_ms > 0 else None,
        "workload": "VGG-16 shape, fp16 storage and MFMA, batch 16 (BASELINE configs[2], fp16 leg)"}
    nh.free()

    # ---- the same at batch 64: enough whole 256 x 256 tiles for every layer of 256 planes and more ----
    cfg64 = configs.vgg16(batch=64)
    nh = api.HipNetwork(cfg64["layers"], cfg64["mean"], cfg64["std"], half=1)
    nh.upload(cfg64["input"])
    msh, famh = timed_forward(lib, nh, max(args.steps // 2, 5), max(args.warmup, 10), (0, 1, 3), profiled=False, reps=3)
    hc_ms, hc_n, hc_fl = famh[0]
    extra["vgg16_fp16_b64"] = {
        "images_per_sec": round(64.0 / (msh * 1e-3), 1), "ms_per_step": round(msh, 4),
        "conv_TFLOP/s": round(hc_fl / (hc_ms * 1e-3) / 1e12, 1) if hc_ms > 0 else None,
        "frac_of_fp16_mfma_peak": round(hc_fl / (hc_ms * 1e-3) / 1e12 / 2500.0, 4) if hc_ms > 0 else None,
        "workload": "VGG-16 shape, fp16 storage and MFMA, batch 64"}
    nh.free()
    del cfg64

    # ---- AlexNet-OWT fp32 batch 1 (GEMV-bound Linear layers) ----
    c2 = configs.alexnet_owt()
    n2 = api.HipNetwork(c2["layers"], c2["mean"], c2["std"])
    x2 = c2["input"].copy()
    for c in range(3):
        x2[:, c] = (x2[:, c] - np.float32(c2["mean"][c])) / np.float32(c2["std"][c])
    n2.upload(x2)
    ms2, fam2 = timed_forward(lib, n2, max(args.steps, 20), max(args.warmup, 20), (0, 1, 3), profiled=False, reps=3)
    gv_ms, gv_n, gv_bytes = fam2[1]
    extra["alexnet_owt_fp32_b1"] = {
        "images_per_sec": round(1e3 / ms2, 1), "ms_per_step": round(ms2, 4),
        "gemv_GB/s": round(gv_bytes / (gv_ms * 1e-3) / 1e9, 1) if gv_ms > 0 else None,
        "gemv_frac_of_hbm_peak": round(gv_bytes / (gv_ms * 1e-3) / 8e12, 4) if gv_ms > 0 else None,
        "workload": "AlexNet-OWT fp32 batch 1 (BASELINE configs[1])"}
    n2.free()

    # ---- ResNet-18 fp32 batch 32 (1x1 projections, batch norm folded into the conv epilogue) ----
    c4 = configs.resnet18(batch=32)
    n4 = api.HipNetwork(c4["layers"], c4["mean"], c4["std"])
    x4 = c4["input"].copy()
    for c in range(3):
        x4[:, c] = (x4[:, c] - np.float32(c4["mean"][c])) / np.float32(c4["std"][c])
    n4.upload(x4)
    ms4, fam4 = timed_forward(lib, n4, max(args.steps, 20), max(args.warmup, 20), (0, 1, 3), profiled=False, reps=3)
    cv_ms, cv_n, cv_fl = fam4[0]
    extra["resnet18_fp32_b32"] = {
        "images_per_sec": round(32.0 / (ms4 * 1e-3), 1), "ms_per_step": round(ms4, 4),
        "conv_TFLOP/s": round(cv_fl / (cv_ms * 1e-3) / 1e12, 2) if cv_ms > 0 else None,
        "workload": "ResNet-18 shape fp32 batch 32 (BASELINE configs[3]), residual add with the reference's a - b arithmetic"}
    n4.free()

    # ---- uint8 AlexNet-OWT batch 64 ----
    roofline_int8 = None
    if not args.no_int8:
        c5 = configs.alexnet_lowp(batch=64)
        x5 = c5["input"].copy()
        for c in range(3):
            x5[:, c] = (x5[:, c] - np.float32(c5["mean"][c])) / np.float32(c5["std"][c])
        n5 = api.HipNetwork(c5["layers"], c5["mean"], c5["std"], lowp_range=c5["range"])
        n5.upload(x5)
        ms5, fam5 = timed_forward(lib, n5, max(args.steps, 20), max(args.warmup, 20), (2, 3), profiled=False, reps=3)
        i8_ms, i8_n, i8_ops = fam5[2]
        i8_tops = i8_ops / (i8_ms * 1e-3) / 1e12 if i8_ms > 0 else 0.0
        extra["int8_alexnet_owt_b64"] = {
            "images_per_sec": round(64.0 / (ms5 * 1e-3), 1), "ms_per_step": round(ms5, 4),
            "conv_i8_TOP/s": round(i8_tops, 2), "frac_of_int8_mfma_peak": round(i8_tops / PEAK_TOPS_INT8_MFMA, 4),
            "dtype": "u8 x u8 -> i32", "workload": "AlexNet-OWT THMakeSpatial form, range 32 (BASELINE configs[4])"}
        # the uint8 convolution family (the eight layers of a step, fc6-8 as one-position convolutions) like `roofline`:
        # ops = 2 M K N B per launch over the time of the launches (events around the run of them, in a second pass of K steps)
        roofline_int8 = {
            "bound": "mfma", "achieved": round(i8_tops, 3), "peak": PEAK_TOPS_INT8_MFMA, "unit": "TOP/s",
            "frac": round(i8_tops / PEAK_TOPS_INT8_MFMA, 4),
            "traffic": counter_traffic("conv_u8_alexnet_owt_b64_counters.md", "conv_hbm_bytes_per_launch"),
            "kernel": "conv_u8_image_pool_kernel (conv1 with its pooling), conv_u8_patch_kernel (conv2-5: the input patch of a band "
                      "resident in LDS or streamed plane block by plane block, pooling in the epilogue where one follows), "
                      "linear_u8_kernel (fc6-8) (uint8 AlexNet-OWT batch 64: eight launches per step)",
            "launches_per_step": i8_n / max(args.steps, 20), "avg_launch_ms": round(i8_ms / max(i8_n, 1), 5),
            "ops_per_launch": i8_ops / max(i8_n, 1),
            "cpu_baseline": None,
            "cpu_baseline_note": "no CPU baseline of the reference's LOWP path can exist for this workload: its GEMM is "
                                 "gemmlowp, which the reference does not carry (lowp/gemm8.cc includes it from a directory "
                                 "the user must fetch), and its uint8 forward holds one image (batch 64 is 64 engine "
                                 "constructions); parity is against this repository's restatement, image by image"}
        n5.free()

    # ---- THProcessImages on the device: 64 interleaved 8-bit 224 x 224 x 3 images cross the link as bytes and become
    # normalised planes (float engines) or codes (uint8 engine) there (thapi.c:452-563); beside it the same batch as
    # floats through THProcessFloat (four times the bytes, normalised by the call) ----
    process_images = None
    if not args.no_int8:
        g = np.random.Generator(np.random.PCG64(77))
        imgs = [np.ascontiguousarray(g.integers(0, 256, (224, 224, 3), dtype=np.uint8)) for _ in range(64)]
        ptrs = (C.c_void_p * 64)(*[im.ctypes.data for im in imgs])
        xf = np.ascontiguousarray(np.stack(imgs).transpose(0, 3, 1, 2).astype(np.float32) / np.float32(255))
        c6 = configs.alexnet_lowp(batch=1)        # AlexNet-OWT, THMakeSpatial form, no SoftMax
        process_images = {"workload": "AlexNet-OWT shape, batch 64 of 224x224x3 8-bit images; best / mean images/s of 10 "
                                      "calls after 2 warm-ups, host transfers included"}
        res, ow, oh = C.POINTER(C.c_float)(), C.c_int(), C.c_int()
        for name, kw in (("fp32", {}), ("uint8", {"lowp_range": c6["range"]})):
            n6 = api.HipNetwork(c6["layers"], c6["mean"], c6["std"], **kw)
            t_img, t_flt = [], []
            for i in range(12):
                t0 = time.perf_counter()
                lib.THProcessImages(n6.handle, ptrs, 64, 224, 224, 672, C.byref(res), C.byref(ow), C.byref(oh), 0)
                if i >= 2:
                    t_img.append(time.perf_counter() - t0)
            for i in range(12):
                x = np.array(xf, np.float32, copy=True, order="C")
                t0 = time.perf_counter()
                lib.THProcessFloat(n6.handle, x.ctypes.data, 64, 224, 224, 3, C.byref(res), C.byref(ow), C.byref(oh))
                if i >= 2:
                    t_flt.append(time.perf_counter() - t0)
            process_images[name] = {
                "THProcessImages_images_per_sec_best": round(64.0 / min(t_img), 1),
                "THProcessImages_images_per_sec_mean": round(64.0 * len(t_img) / sum(t_img), 1),
                "THProcessFloat_images_per_sec_best": round(64.0 / min(t_flt), 1),
                "THProcessFloat_images_per_sec_mean": round(64.0 * len(t_flt) / sum(t_flt), 1)}
            n6.free()

    # ---- what the matrix cores sustain from registers alone on this device (no memory traffic), for scale ----
    extra["mfma_register_loop"] = {
        "fp32_32x32x2_TFLOP/s_by_waves_per_simd": {str(w): round(lib.thhip_probe_mfma(0, w, 30.0) / 1e12, 1) for w in (1, 2, 3, 4)},
        "fp16_32x32x16_TFLOP/s": round(lib.thhip_probe_mfma(1, 2, 600.0) / 1e12, 1),
        "int8_32x32x32_TOP/s": round(lib.thhip_probe_mfma(3, 2, 600.0) / 1e12, 1),
        "what": "MFMAs on four accumulators per wavefront with operands (random values) in registers and nothing else; "
                "fp32 for about 30 ms per occupancy, fp16 and int8 with two wavefronts per SIMD for about 600 ms (their "
                "rate climbs over the first few hundred ms of such a loop and falls with the operands' bit activity: all "
                "zeros run at 2480 / 4960); the published peaks are 157.3 / 2500 / 5030"}

    cpu = None
    if not args.no_cpu:
        cpu = cpu_baseline(cfg)

    line = {
        "metric": "images/sec VGG-16 fp32 b16 (+ int8 AlexNet-OWT b64 under extra); % MFMA peak under roofline",
        "value": round(value, 2), "unit": "images/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": "VGG-16 shape, fp32, batch 16, 3x224x224, THForward with the input resident in HBM "
                               "(BASELINE configs[2])", "batch": 16},
        "roofline": roofline, "cpu_baseline": cpu, "process_float": process_float, "process_images": process_images, "roofline_int8": roofline_int8,
        "extra": extra,
    }
    print(json.dumps(line))


if __name__ == "__main__":
    main()
