#!/usr/bin/env python3
"""Benchmark of the PINK hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload cfg1]

A step is one pass of the hot path over one batch of synthetic input: the whole
image set of the workload, mapped (cfg1) or trained in order (cfg0/2/3/4), with the
images already resident in HBM when the timed region starts.  Default workload: cfg1
(mapping 20 000 images, uint8 distances, 720 variants) with the SOM obtained by
training cfg0 for one epoch on the GPU first (untimed).

Prints ONE JSON line with the throughput, a `roofline` object for the kernel class
that takes most of the time (durations from HIP events recorded on the library's own
stream around every launch) and a `cpu_baseline` object (the CPU oracle timed on a
bounded sample of the same workload on this host's cores).
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0          # MI355X HBM3E, published
MFMA_INT8_PEAK_TOPS = 5000.0   # MI355X dense int8 MFMA, published
FP32_PEAK_TFLOPS = 157.3       # MI355X vector fp32 (packed FMA), published

DTYPE_NAME = {0: "f32", 1: "u16", 2: "u8"}


# Peaks measured on the MI355X box used for this work with small microbenchmarks (independent
# MFMA / fma streams on all CUs): the clock settles near 2.0-2.2 GHz under load.  Reported next to
# the published figures, never instead of them.
MEASURED_INT8_MFMA_TOPS = 4130.0
MEASURED_FMA_NOPACK_TFLOPS = 72.5

# HBM bytes per image from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE (profiles/cfg1_map_u8_hbm_traffic.txt),
# scaled by the same counters' readings for a 256 MiB device-to-device copy (FETCH x2.0, WRITE x1.0).
MEASURED_TRAFFIC_PER_IMAGE = {
    ("cfg1", 3, "rotate"): 49.2e3 + 103.8e3,     # image + part of the geometry table read; units written
    ("cfg1", 3, "distance"): 107.3e3 + 0.8e3,    # units read once; keys written
}


def algorithmic_per_image(w, E, path):
    """Algorithmic bytes / operations per image for each kernel class.  `path` is the distance
    kernel in use (capi.KERNEL_VALU / _MFMA / _MFMA_SYM): the matrix-core paths never write the
    float variants, their rotation kernel emits the packed distance operand directly."""
    elem = {0: 4, 1: 2, 2: 1}[w.ed_type]
    S, R, N = w.neuron_size, w.R, w.som_size
    nrr = max(w.num_rot // 4, 1)
    kp = -(-E // 64) * 64
    # k_rotate: image read once; a trainer's launch stores two of every base rotation's symmetries as
    # float32 (the base rotation and its quarter turn, one when there is a single rotation) and the
    # region of all R variants in the distance type; a mapper's launch stores the packed region only
    stored = nrr * (2 if w.num_rot > 1 else 1) if w.mode == "train" else 0
    rot_bytes = w.image_size * 4 + stored * S * 4 + R * E * elem
    if w.ed_type != 0 and (path == 1 or w.channels > 1):     # integer distances on the vector ALU, or multi-channel
        rot_bytes = w.image_size * 4 + R * S * 4          # all variants; a kernel of its own packs the region
    if path == 2:      # uint8 MFMA, symmetries on the image side: ceil(nrr/4) tiles of 32 rows + norms
        rot_bytes = w.image_size * 4 + -(-nrr // 4) * 32 * (kp + 4)
    elif path == 3:    # uint8 MFMA, symmetries on the SOM side: ceil(nrr/32) units of 32 rows + 1 KiB of norm entries
        rot_bytes = w.image_size * 4 + -(-nrr // 32) * (32 * kp + 1024)
    # every operand element read once: all R variants and the N neurons, or, where the symmetries sit on
    # the SOM side (operand in registers), the units of the base rotations the rotation kernel wrote + the keys
    dist_bytes = (R + N) * E * elem
    if path == 3:
        dist_bytes = -(-nrr // 32) * (32 * kp + 1024) + N * 8
    return {
        "rotate": {"bytes": rot_bytes},
        # region of every variant read as float32 and written in the distance type
        "pack": {"bytes": R * E * (4 + elem)},
        # one subtract-square-accumulate = 2 operations
        "distance": {"bytes": dist_bytes, "ops": 2 * N * R * E},
        # SOM read + written, one variant read per neuron
        "update": {"bytes": 3 * N * S * 4},
        "finalize": {"bytes": N * 16},
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=None,
                    help="timed steps (default: 30 for the mapping workload, whose step takes a few ms, 3 for training)")
    ap.add_argument("--warmup", type=int, default=None, help="untimed steps before them (default: 10 mapping, 1 training)")
    ap.add_argument("--workload", default="cfg1", choices=["cfg0", "cfg1", "cfg2", "cfg3", "cfg4"])
    ap.add_argument("--images", type=int, default=0, help="override the number of images per step")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--host-buffers", action="store_true",
                    help="also time one step through the host-pointer entry points (PCIe transfers included); "
                         "reported as `pcie_inclusive`, never as `value`")
    ap.add_argument("--kernel", default="auto", choices=["auto", "valu", "mfma", "mfma_sym", "mfma_gemm"])
    ap.add_argument("--calibrate-copy", type=int, default=0, metavar="MIB",
                    help="also run one plain device-to-device copy of this many MiB (a kernel of known "
                         "traffic, to scale rocprofv3 FETCH_SIZE / WRITE_SIZE readings)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU; --gpus %d is not supported (every figure is a "
              "single-MI355X figure)" % args.gpus, file=sys.stderr)
        sys.exit(2)

    import torch
    from pink_amd import capi, synthetic

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(3)
    dev = torch.device("cuda:0")
    w = synthetic.WORKLOADS[args.workload]
    # a mapping step is a few milliseconds of GPU time: enough of them that the clocks have settled
    if args.steps is None:
        args.steps = 30 if w.mode == "map" else 3
    if args.warmup is None:
        args.warmup = 10 if w.mode == "map" else 1
    n_images = args.images or w.n_images
    kernel_choice = {"auto": capi.KERNEL_AUTO, "valu": capi.KERNEL_VALU, "mfma": capi.KERNEL_MFMA,
                     "mfma_sym": capi.KERNEL_MFMA_SYM, "mfma_gemm": capi.KERNEL_MFMA_GEMM}[args.kernel]

    t0 = time.time()
    imgs_host = synthetic.images(w, n_images)
    som0 = synthetic.initial_som(w)
    if w.mode == "map":
        # the SOM of cfg0 after one epoch, trained here on the GPU (set-up, not timed)
        w0 = synthetic.WORKLOADS["cfg0"]
        with synthetic.make_context(w0) as tr:
            tr.set_som(som0)
            tr.train(synthetic.images(w0))
            som0 = tr.get_som()
    setup_s = time.time() - t0

    ctx = synthetic.make_context(w, kernel_choice=kernel_choice)
    E = ctx.region_size
    ctx.set_som(som0)
    d_imgs = torch.from_numpy(imgs_host).to(dev)
    d_heat = torch.empty((n_images, w.som_size), dtype=torch.float32, device=dev)
    d_best = torch.empty((n_images, w.som_size), dtype=torch.int32, device=dev)
    d_bmu = torch.empty((n_images,), dtype=torch.int32, device=dev)
    torch.cuda.synchronize()
    if args.calibrate_copy:
        src = torch.empty(args.calibrate_copy << 20, dtype=torch.uint8, device=dev)
        dst = torch.empty_like(src)
        dst.copy_(src)            # reads and writes exactly calibrate_copy MiB each
        torch.cuda.synchronize()
        del src, dst

    def step():
        if w.mode == "map":
            ctx.map_device(d_imgs.data_ptr(), n_images, d_heat.data_ptr(), d_best.data_ptr())
        else:
            ctx.train_device(d_imgs.data_ptr(), n_images, d_bmu.data_ptr())

    for _ in range(args.warmup):
        if w.mode == "train":
            ctx.set_som(som0)
        step()
    ctx.synchronize()

    # ---- timed region: exactly `steps` steps, nothing but the path's own launches on the stream ----
    if w.mode == "train":
        ctx.set_som(som0)
    ctx.set_profiling(False)
    torch.cuda.synchronize()
    ctx.synchronize()
    t_start = time.perf_counter()
    for _ in range(args.steps):
        step()
    ctx.synchronize()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t_start
    # ---- per-kernel durations: HIP events around every launch, on the context's stream, in a pass of
    # their own right after the timed one (the event records cost a mapper several per cent of its
    # throughput and a trainer, with thousands of launches per second, much more)
    ctx.set_profiling(True)
    if w.mode == "map":
        for _ in range(args.steps):
            step()
        prof_images = n_images * args.steps
        measured = "the %d timed steps repeated with per-launch HIP events" % args.steps
    else:
        prof_images = min(n_images, 256)
        ctx.train_device(d_imgs.data_ptr(), prof_images, d_bmu.data_ptr())
        measured = "separate pass of %d images with per-launch HIP events" % prof_images
    times = ctx.kernel_times()
    ctx.set_profiling(False)

    value = n_images * args.steps / elapsed
    path = ctx.distance_kernel
    alg = algorithmic_per_image(w, E, path)
    total_ms = sum(ms for _, ms in times.values()) or 1e-9
    dominant = max(times, key=lambda k: times[k][1])
    # The distance + argmin kernel is the one the path is priced on (its operation count is the
    # algorithm's); where another class is ahead of it by less than a tenth, the roofline object still
    # describes the distance kernel, so that the line does not flip between two near-equal kernels.
    if times["distance"][1] >= 0.9 * times[dominant][1]:
        dominant = "distance"
    launches, ms = times[dominant]
    avg_ms = ms / max(launches, 1)
    imgs_per_launch = prof_images / max(launches, 1)
    per_s = imgs_per_launch / (avg_ms * 1e-3)
    notes = None
    if dominant == "distance" and w.ed_type == capi.FLOAT:
        # direct float32 form on the vector ALU: subtract + fma per pair element, counted as 2 ops
        bound, unit, peak = "mfma", "TFLOP/s", FP32_PEAK_TFLOPS
        achieved = alg["distance"]["ops"] * per_s / 1e12
        notes = ("compute bound on the vector ALU, not on MFMA: bit-faithful sequential fma per (neuron, rotation); "
                 "packed FP32 is disabled in this build, so the attainable rate is half the published "
                 "157.3 TFLOP/s (measured %.1f TFLOP/s fma)" % MEASURED_FMA_NOPACK_TFLOPS)
    elif dominant == "distance" and path == capi.KERNEL_MFMA_SYM:
        bound, unit, peak = "mfma", "TOP/s", MFMA_INT8_PEAK_TOPS
        achieved = alg["distance"]["ops"] * per_s / 1e12
        notes = "int8 MFMA; measured MFMA peak on this box %.0f TOP/s" % MEASURED_INT8_MFMA_TOPS
    else:
        bound, unit, peak = "hbm", "GB/s", HBM_PEAK_GBS
        achieved = alg[dominant]["bytes"] * per_s / 1e9
        if dominant == "rotate" and path != capi.KERNEL_VALU:
            notes = ("vector-ALU bound (exact bilinear arithmetic per operand byte), far from HBM: "
                     "algorithmic bytes = image read + packed operand written")
    traffic = MEASURED_TRAFFIC_PER_IMAGE.get((args.workload, path, dominant))
    roofline = {
        "kernel": dominant, "bound": bound, "achieved": round(achieved, 3), "peak": peak, "unit": unit,
        "frac": round(achieved / peak, 5),
        "traffic": round(traffic * imgs_per_launch) if traffic else None,
        "algorithmic_bytes_per_launch": round(alg[dominant]["bytes"] * imgs_per_launch),
        "avg_launch_ms": round(avg_ms, 6), "launches": launches, "images_per_launch": imgs_per_launch,
        "measured": measured,
        "share_of_kernel_time": round(ms / total_ms, 4),
        "kernel_ms": {k: round(v[1], 4) for k, v in times.items()},
        "distance_path": {1: "vector ALU", 2: "int8 MFMA, image-side symmetries", 3: "int8 MFMA, SOM-side symmetries",
                          4: "int8 MFMA GEMM, split k"}[path],
    }
    if notes:
        roofline["note"] = notes
    # the distance kernel's own fractions, whichever kernel dominates
    d_launches, d_ms = times["distance"]
    if d_launches:
        d_per_s = prof_images / (d_ms * 1e-3)
        dist = {"ops_per_s": alg["distance"]["ops"] * d_per_s, "share_of_kernel_time": round(d_ms / total_ms, 4)}
        if w.ed_type == capi.FLOAT:
            dist["frac_of_fp32_157.3TF"] = round(dist["ops_per_s"] / 1e12 / FP32_PEAK_TFLOPS, 5)
            dist["frac_of_measured_nopack_fma"] = round(dist["ops_per_s"] / 1e12 / MEASURED_FMA_NOPACK_TFLOPS, 5)
        else:
            dist["frac_of_int8_mfma_5POPs"] = round(dist["ops_per_s"] / 1e12 / MFMA_INT8_PEAK_TOPS, 5)
            dist["hbm_frac_algorithmic_bytes"] = round(alg["distance"]["bytes"] * d_per_s / 1e9 / HBM_PEAK_GBS, 5)
        dist["ops_per_s"] = round(dist["ops_per_s"] / 1e12, 3)
        roofline["distance_kernel"] = dist
    r_launches, r_ms = times["rotate"]
    if r_launches:
        r_per_s = prof_images / (r_ms * 1e-3)
        roofline["rotate_kernel"] = {"share_of_kernel_time": round(r_ms / total_ms, 4),
                                     "hbm_frac_algorithmic_bytes": round(alg["rotate"]["bytes"] * r_per_s / 1e9 / HBM_PEAK_GBS, 5),
                                     "us_per_image": round(r_ms * 1e3 / prof_images, 4)}

    pcie = None
    if args.host_buffers:
        if w.mode == "train":
            ctx.set_som(som0)
        t = time.perf_counter()
        if w.mode == "map":
            ctx.map(imgs_host)
        else:
            ctx.train(imgs_host)
        dt = time.perf_counter() - t
        pcie = {"value": round(n_images / dt, 2), "unit": "images/s",
                "what": "one step through pink_hip_%s with pageable host buffers: H2D of the images, "
                        "D2H of the results and the device allocations included" % w.mode}

    cpu = None
    if not args.no_cpu_baseline:
        import oracle as O
        s = O.shape(w.som_size, w.channels, w.image_dim, w.neuron_dim, w.num_rot, w.use_flip, w.ed_dim,
                    w.ed_shape, w.ed_type)
        F = synthetic.update_factors(w) if w.mode == "train" else None

        def cpu_run(n):
            t = time.perf_counter()
            if w.mode == "map":
                O.map_images(s, som0, imgs_host[:n])
            else:
                O.train(s, som0.copy(), imgs_host[:n], F)
            return time.perf_counter() - t

        cpu_run(min(2, n_images))                      # warm-up
        probe_n = min(4, n_images)
        probe = cpu_run(probe_n)
        n_cpu = int(max(probe_n, min(n_images, 12.0 / max(probe / probe_n, 1e-6))))
        dt = cpu_run(n_cpu)
        cpu = {"value": round(n_cpu / dt, 3), "unit": "images/s", "cores": O.num_threads(), "kind": "port",
               "sample": "%d images of %s, %.1f s, OpenMP over rotations" % (n_cpu, w.name, dt)}

    out = {
        "metric": ("map" if w.mode == "map" else "train") + " images/sec @%d rot x flip" % w.R,
        "value": round(value, 2), "unit": "images/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(elapsed / args.steps * 1e3, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": DTYPE_NAME[w.ed_type], "data": "synthetic",
        "config": {"workload": w.name, "mode": w.mode, "images_per_step": n_images, "som_size": w.som_size,
                   "neuron": [w.channels, w.neuron_dim, w.neuron_dim], "image": [w.channels, w.image_dim, w.image_dim],
                   "variants": w.R, "region_elements": E, "distance_kernel": args.kernel,
                   "som": "cfg0 trained 1 epoch on the GPU" if w.mode == "map" else "mt19937(1234) U[0,1)"},
        "roofline": roofline, "cpu_baseline": cpu, "setup_s": round(setup_s, 2),
    }
    if pcie:
        out["pcie_inclusive"] = pcie
    ctx.close()
    print(json.dumps(out))


if __name__ == "__main__":
    main()
