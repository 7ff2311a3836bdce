#!/usr/bin/env python3
"""Benchmark of the PINK hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload cfg0]

A step is one pass of the hot path over one batch of synthetic input: the image set of the
workload trained in order (cfg0/2/3/4: every image sees the weights the image before it left,
the final SOM copied back to the host at the end of the step, Trainer::update_som) or mapped
(cfg1), with the images already resident in HBM when the timed region starts.

Default workload: cfg0, the configuration the metric is quoted on -- training a 10x10 SOM in
float32 on 2 000 images of 64x64 with 360 rotations x flip (720 variants).  The same JSON line
carries, under `all_configs`, the other four configurations on a bounded number of images each
(fixed step counts, whatever --steps says).

Prints ONE JSON line with the throughput, a `roofline` object for the kernel class that takes
most of the time (durations from HIP events recorded on the library's own stream around every
launch, in a pass of the same step right after the timed one), a `cpu_baseline` object (the CPU
oracle timed on a bounded sample of the same workload on this host's cores) and
`host_inclusive` (the same step through the host-pointer entry points: H2D of the images and D2H
of the results inside the clock; never `value`).
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
FP32_PEAK_TFLOPS = 157.3       # MI355X fp32 (vector with packed FMA, and fp32 MFMA), published

DTYPE_NAME = {0: "f32", 1: "u16", 2: "u8"}

# Peaks measured on an MI355X of this pool with small microbenchmarks (independent MFMA / fma
# streams on all CUs): the clock settles near 2.0-2.2 GHz under load.  Reported next to the
# published figures, never instead of them.
MEASURED_INT8_MFMA_TOPS = 4130.0
MEASURED_VALU_LANE_OPS_T = 50.0     # subtract / fma stream, eight waves per SIMD: 3.15 clk per wave instruction at 2.4 GHz

# HBM bytes per image of one kernel class from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, each scaled
# by what the same counter reads for a device-to-device copy of known size; (bytes, the summary
# under profiles/ that holds the readings).  Not measured in the run that prints the line.
COUNTER_TRAFFIC_PER_IMAGE = {
    ("cfg0", "distance"): (12.280e6 + 3.239e6, "profiles/cfg0_train_f32_counters.txt"),   # with the update of the image before
    ("cfg0", "update"): ((28.133e6 + 0.774e6 + 1.706e6 + 1.184e6) / 48, "profiles/cfg0_train_f32_counters.txt"),   # per group of 48
    ("cfg1", "rotate"): ((96.042e6 + 207.618e6) / 2048, "profiles/cfg1_map_u8_counters.txt"),
    ("cfg1", "distance"): ((214.632e6 + 1.639e6) / 2048, "profiles/cfg1_map_u8_counters.txt"),
    ("cfg2", "distance"): (32.971e6 + 0.069e6, "profiles/cfg2_train_u16_counters.txt"),
    ("cfg2", "update"): (28.845e6 + 17.831e6, "profiles/cfg2_train_u16_counters.txt"),
    ("cfg3", "distance"): (252.417e6 + 0.576e6, "profiles/cfg3_train_f32_3ch_counters.txt"),
    # the operand rows per image and a sixteenth of the launch that brings the neurons' full images up to date
    ("cfg3", "update"): (73.894e6 + 47.153e6 + (323.973e6 + 95.049e6) / 16, "profiles/cfg3_train_f32_3ch_counters.txt"),
    ("cfg4", "update"): ((85.604e6 + 0.835e6) / 256, "profiles/cfg4_train_u8_counters.txt"),     # the resident launch of 256 images
}

# Images per step of the workloads that ride along in `all_configs` (the headline workload always
# runs its whole image set): bounded so that the default run stays within minutes; training is
# sequential, so the rate per image does not depend on how many follow.
SIDE_IMAGES = {"cfg0": 2000, "cfg1": 20000, "cfg2": 1500, "cfg3": 600, "cfg4": 20000}
SIDE_STEPS = {"cfg0": (1, 3), "cfg1": (5, 20), "cfg2": (1, 2), "cfg3": (1, 2), "cfg4": (1, 2)}   # (warm-up, timed)


def algorithmic_per_image(w, E, path):
    """Algorithmic bytes / operations per image for each kernel class.  `path` is the distance
    kernel in use (capi.KERNEL_VALU / _MFMA / _MFMA_SYM / _MFMA_GEMM): the matrix-core mapping paths
    never write the float variants, their rotation kernel emits the packed distance operand directly."""
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


def distance_path_name(w, path, times):
    """The kernel that computed the distances in this run, by the library's path and what was launched."""
    from pink_amd import capi
    if w.ed_type == capi.FLOAT and path != capi.KERNEL_MFMA_F32:
        if w.mode == "train" and 0 < times["update"][0] < times["distance"][0]:
            return "float32 vector ALU, one (neuron, variant) pair per lane, DPP broadcast; the launch also applies the update of the image before"
        return "float32 vector ALU, one (neuron, variant) pair per lane"
    if w.mode == "train" and path == capi.KERNEL_MFMA_GEMM and times["distance"][0] == 0:
        return ("int8 MFMA inside the resident launch of a small uint8 trainer (one launch per group of images: distances, "
                "best match, update; one block per neuron, a 64-bit word per block and image exchanged through memory)")
    return {capi.KERNEL_VALU: "integer vector ALU", capi.KERNEL_MFMA: "int8 MFMA, image-side symmetries, SOM operand in LDS",
            capi.KERNEL_MFMA_SYM: "int8 MFMA, SOM-side symmetries, SOM operand in registers",
            capi.KERNEL_MFMA_GEMM: "int8 MFMA GEMM, one launch, 64x64 or 32x32 tiles over the whole k range, finished by their blocks",
            capi.KERNEL_MFMA_F32: "float32 MFMA GEMM (recast, on request)"}[path]


def cpu_baseline(w, som0, imgs_host, budget_s, quick=False):
    """The CPU path on a bounded sample of the workload, on this host's cores.

    `value`: the oracle run with the reference's own parallel structure
    (generate_euclidean_distance_matrix.h:45-56: per neuron an `omp parallel for` over the rotations, one call
    through a function pointer and one `omp critical` section per pair) in float32, the arithmetic the
    reference's CPU path uses whatever the distance type (it has no integer mode).  `port`: the oracle's own,
    leaner evaluation (sixteen variants side by side in vector registers, neurons and variant blocks spread
    over the threads) in the workload's distance type: the faster CPU figure, not what the reference runs."""
    import oracle as O
    from pink_amd import capi, synthetic
    F = synthetic.update_factors(w) if w.mode == "train" else None
    threads = O.num_threads()

    def shape(ed_type):
        return O.shape(w.som_size, w.channels, w.image_dim, w.neuron_dim, w.num_rot, w.use_flip, w.ed_dim,
                       w.ed_shape, ed_type)

    def run(s, n):
        t = time.perf_counter()
        if w.mode == "map":
            O.map_images(s, som0, imgs_host[:n])
        else:
            O.train(s, som0.copy(), imgs_host[:n], F)
        return time.perf_counter() - t

    def rate(s, form, nthreads, budget):
        O.set_distance_form(form)
        O.set_num_threads(nthreads)
        try:
            n_all = len(imgs_host)
            probe = run(s, 1)                              # warm-up, and roughly how long an image takes
            n, dt = 1, probe
            if probe < budget / 2:
                # (the first image also wakes the thread pool: a second, warm probe sizes the sample)
                n = int(max(1, min(n_all, 0.1 * budget / max(probe, 1e-6))))
                dt = run(s, n)
                n = int(max(1, min(n_all, budget / max(dt / n, 1e-6))))
                dt = run(s, n)
        finally:
            O.set_num_threads(threads)
            O.set_distance_form(O.LANES)
        return n / dt, n, dt

    v, n, dt = rate(shape(capi.FLOAT), O.REFERENCE_LOOP, threads, budget_s)
    out = {"value": round(v, 3), "unit": "images/s", "cores": threads, "kind": "port",
           "sample": "%d images of %s, %.1f s" % (n, w.name, dt),
           "structure": "the oracle with the reference's own loop (generate_euclidean_distance_matrix.h:45-56): omp parallel "
                        "for over the rotations of one neuron, a call through a function pointer and an omp critical section "
                        "per pair; float32, the arithmetic of the reference's CPU path whatever the distance type"}
    vp, np_, dtp = rate(shape(w.ed_type), O.LANES, threads, budget_s / 3)
    out["port"] = {"value": round(vp, 3), "cores": threads, "dtype": DTYPE_NAME[w.ed_type],
                   "sample": "%d images, %.1f s" % (np_, dtp),
                   "what": "the oracle's own evaluation in the workload's distance type: sixteen variants side by side in "
                           "vector registers, threads over neurons and variant blocks; same results, leaner than the reference"}
    if not quick:
        v1, n1, dt1 = rate(shape(capi.FLOAT), O.REFERENCE_LOOP, 1, budget_s / 3)
        out["one_thread"] = {"value": round(v1, 3), "sample": "%d images, %.1f s" % (n1, dt1)}
    return out


def run_workload(name, steps, warmup, n_images, kernel, cpu_budget_s, host_inclusive, quick_cpu, calibrate_copy=0):
    import torch
    from pink_amd import capi, synthetic

    dev = torch.device("cuda:0")
    w = synthetic.WORKLOADS[name]
    kernel_choice = {"auto": capi.KERNEL_AUTO, "valu": capi.KERNEL_VALU, "mfma": capi.KERNEL_MFMA,
                     "mfma_sym": capi.KERNEL_MFMA_SYM, "mfma_gemm": capi.KERNEL_MFMA_GEMM,
                     "mfma_f32": capi.KERNEL_MFMA_F32}[kernel]
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
    d_heat = torch.empty((n_images, w.som_size), dtype=torch.float32, device=dev) if w.mode == "map" else None
    d_best = torch.empty((n_images, w.som_size), dtype=torch.int32, device=dev) if w.mode == "map" else None
    d_bmu = torch.empty((n_images,), dtype=torch.int32, device=dev)
    som_host = np.empty_like(som0)
    torch.cuda.synchronize()
    if calibrate_copy:
        src = torch.empty(calibrate_copy << 20, dtype=torch.uint8, device=dev)
        dst = torch.empty_like(src)
        dst.copy_(src)            # reads and writes exactly calibrate_copy MiB each
        torch.cuda.synchronize()
        del src, dst

    def step():
        if w.mode == "map":
            ctx.map_device(d_imgs.data_ptr(), n_images, d_heat.data_ptr(), d_best.data_ptr())
        else:
            ctx.train_device(d_imgs.data_ptr(), n_images, d_bmu.data_ptr())
            ctx.get_som(out=som_host)              # Trainer::update_som(): the weights back on the host

    for _ in range(warmup):
        if w.mode == "train":
            ctx.set_som(som0)
        step()
    ctx.synchronize()

    # ---- timed region: exactly `steps` steps, nothing but the path's own launches on the stream.
    # A training step starts from the weights the step before left (a further epoch): resetting them
    # would put an upload into the clock that the path does not have.
    ctx.set_profiling(False)
    torch.cuda.synchronize()
    ctx.synchronize()
    t_start = time.perf_counter()
    for _ in range(steps):
        step()
    ctx.synchronize()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t_start
    # ---- per-kernel durations: HIP events around every launch, on the context's stream, in a pass of
    # the same step right after the timed ones (the event records cost a mapper several per cent of its
    # throughput and a trainer, with tens of thousands of launches per second, much more)
    ctx.set_profiling(True)
    prof_steps = steps if w.mode == "map" else 1
    for _ in range(prof_steps):
        step()
    prof_images = n_images * prof_steps
    measured = "%d step(s) repeated right after the timed ones with per-launch HIP events" % prof_steps
    times = ctx.kernel_times()
    ctx.set_profiling(False)

    value = n_images * steps / elapsed
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
    second_peak = None
    if dominant == "distance" and path == capi.KERNEL_MFMA_F32:
        bound, unit, peak = "mfma", "TFLOP/s", FP32_PEAK_TFLOPS
        achieved = alg["distance"]["ops"] * per_s / 1e12
        notes = ("float32 MFMA recast |a|^2 + |b|^2 - 2 a.b, requested with --kernel mfma_f32: not the CPU's summation "
                 "order (distances to a relative tolerance only); never the default")
    elif dominant == "distance" and w.ed_type == capi.FLOAT:
        # direct float32 form on the vector ALU: subtract + fma per pair element, counted as 2 ops
        bound, unit, peak = "valu", "TFLOP/s", FP32_PEAK_TFLOPS
        achieved = alg["distance"]["ops"] * per_s / 1e12
        second_peak = ("non-packed vector-ALU stream measured on this pool (subtract + fma, eight waves per SIMD)",
                       MEASURED_VALU_LANE_OPS_T)
        notes = ("compute bound on the vector ALU: bit-faithful sequential fma per (neuron, rotation), one subtract + "
                 "one fma per pair element (counted as 2 operations); non-packed instructions (packed FP32 is disabled in "
                 "this build) issue at 3.15 clocks per wave at best, measured: %.0f T operations/s = about a third of the "
                 "published 157.3 TFLOP/s is this form's ceiling" % MEASURED_VALU_LANE_OPS_T)
        if w.mode == "train" and 0 < times["update"][0] < times["distance"][0]:
            notes += ("; a small float32 trainer: the distance launch of an image also applies the update of the image "
                      "before it to the SOM operand (per chunk of 64 elements 8 instructions next to the 128 of the "
                      "distances, not counted as operations), so the launch priced here is the whole step of an image "
                      "but for one launch per group that brings the neurons' full images up to date")
    elif dominant == "distance" and path in (capi.KERNEL_MFMA_SYM, capi.KERNEL_MFMA_GEMM, capi.KERNEL_MFMA):
        bound, unit, peak = "mfma", "TOP/s", MFMA_INT8_PEAK_TOPS
        achieved = alg["distance"]["ops"] * per_s / 1e12
        second_peak = ("int8 MFMA stream measured on this pool (all SIMDs issuing)", MEASURED_INT8_MFMA_TOPS)
        notes = "int8 MFMA; measured MFMA peak on this pool %.0f TOP/s" % MEASURED_INT8_MFMA_TOPS
        if w.ed_type == capi.UINT16:
            notes += "; uint16 runs four byte-plane products per pair element, counted once"
    else:
        bound, unit, peak = "hbm", "GB/s", HBM_PEAK_GBS
        achieved = alg[dominant]["bytes"] * per_s / 1e9
        if dominant == "rotate" and path != capi.KERNEL_VALU:
            notes = ("vector-ALU bound (exact bilinear arithmetic per operand byte), far from HBM: "
                     "algorithmic bytes = image read + packed operand written")
        if dominant == "update" and times["distance"][0] == 0:
            notes = ("a small uint8 trainer: distances, best match and update of a whole group of images in one resident "
                     "launch (class 'update'), one block per neuron; per image the blocks exchange one 64-bit word each "
                     "through memory (store, then polls: about 0.9 us) around about 1 us of lone-wave instruction issue; "
                     "bound by that chain, not by HBM: no roofline claimed")
    traffic = COUNTER_TRAFFIC_PER_IMAGE.get((name, dominant))
    roofline = {
        "kernel": dominant, "bound": bound, "achieved": round(achieved, 3), "peak": peak, "unit": unit,
        "frac": round(achieved / peak, 5),
        "traffic": round(traffic[0] * imgs_per_launch) if traffic else None,
        "algorithmic_bytes_per_launch": round(alg[dominant]["bytes"] * imgs_per_launch),
        "avg_launch_ms": round(avg_ms, 6), "launches": launches, "images_per_launch": imgs_per_launch,
        "measured": measured,
        "share_of_kernel_time": round(ms / total_ms, 4),
        "kernel_ms": {k: round(v[1], 4) for k, v in times.items()},
        "kernel_us_per_image": {k: round(v[1] * 1e3 / prof_images, 4) for k, v in times.items()},
        "distance_path": distance_path_name(w, path, times),
    }
    if second_peak:
        roofline["measured_ceiling"] = {"what": second_peak[0], "peak": second_peak[1], "unit": unit,
                                        "frac": round(achieved / second_peak[1], 5)}
    if traffic:
        roofline["traffic_source"] = traffic[1] + " (rocprofv3 counters of an earlier run of this command, not of this run)"
    if notes:
        roofline["note"] = notes
    # the HBM-bound kernels by their algorithmic bytes
    for cls, key in (("rotate", "rotate_kernel"), ("update", "update_kernel")):
        c_launches, c_ms = times[cls]
        if c_launches:
            c_per_s = prof_images / (c_ms * 1e-3)
            roofline[key] = {"share_of_kernel_time": round(c_ms / total_ms, 4),
                             "hbm_frac_algorithmic_bytes": round(alg[cls]["bytes"] * c_per_s / 1e9 / HBM_PEAK_GBS, 5),
                             "us_per_image": round(c_ms * 1e3 / prof_images, 4)}
    d_launches, d_ms = times["distance"]
    if d_launches and dominant != "distance":
        d_per_s = prof_images / (d_ms * 1e-3)
        peak_ops = FP32_PEAK_TFLOPS if w.ed_type == capi.FLOAT else MFMA_INT8_PEAK_TOPS
        roofline["distance_kernel"] = {"share_of_kernel_time": round(d_ms / total_ms, 4),
                                       "frac": round(alg["distance"]["ops"] * d_per_s / 1e12 / peak_ops, 5),
                                       "us_per_image": round(d_ms * 1e3 / prof_images, 4)}

    host = None
    if host_inclusive:
        # the same step through the host-pointer entry points, as the reference's own loop hands images over
        # (Pink/main_generic.h:87-89): H2D of the images, D2H of the results, the final SOM for a trainer
        # (timed on the second call: the first one allocates the library's staging buffers and copy stream)
        for timed in (False, True):
            if w.mode == "train":
                ctx.set_som(som0)
            ctx.synchronize()
            t = time.perf_counter()
            if w.mode == "map":
                ctx.map(imgs_host)
            else:
                ctx.train(imgs_host)
                ctx.get_som(out=som_host)
            dt = time.perf_counter() - t
        host = {"value": round(n_images / dt, 2), "unit": "images/s",
                "what": "one step through pink_hip_%s with pageable host buffers, after one untimed step of the same "
                        "kind: H2D of the images and D2H of the results (a trainer: best matches and the final SOM) "
                        "inside the clock" % w.mode}

    cpu = cpu_baseline(w, som0, imgs_host, cpu_budget_s, quick=quick_cpu) if cpu_budget_s > 0 else None
    ctx.close()
    del d_imgs, d_heat, d_best, d_bmu
    torch.cuda.empty_cache()
    return {
        "metric": ("map" if w.mode == "map" else "train") + " images/sec @%d rot x flip" % w.R,
        "value": round(value, 2), "device_resident": round(value, 2), "unit": "images/s", "steps": steps, "warmup": warmup,
        "ms_per_step": round(elapsed / steps * 1e3, 4), "dtype": DTYPE_NAME[w.ed_type],
        "config": {"workload": w.name, "mode": w.mode, "images_per_step": n_images, "images_in_config": w.n_images,
                   "som_size": w.som_size, "neuron": [w.channels, w.neuron_dim, w.neuron_dim],
                   "image": [w.channels, w.image_dim, w.image_dim], "variants": w.R, "region_elements": E,
                   "distance_kernel": kernel,
                   "som": "cfg0 trained 1 epoch on the GPU" if w.mode == "map" else "mt19937(1234) U[0,1)"},
        "roofline": roofline, "cpu_baseline": cpu, "host_inclusive": host, "setup_s": round(setup_s, 2),
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=None,
                    help="timed steps of the headline workload (default: 10 for training, 30 for the mapping workload, "
                         "whose step takes a few ms)")
    ap.add_argument("--warmup", type=int, default=None, help="untimed steps before them (default: 2 training, 10 mapping)")
    ap.add_argument("--workload", default="cfg0", choices=["cfg0", "cfg1", "cfg2", "cfg3", "cfg4"])
    ap.add_argument("--images", type=int, default=0, help="override the number of images per step")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-all-configs", action="store_true", help="only the headline workload")
    ap.add_argument("--no-host-inclusive", action="store_true")
    ap.add_argument("--kernel", default="auto", choices=["auto", "valu", "mfma", "mfma_sym", "mfma_gemm", "mfma_f32"])
    ap.add_argument("--calibrate-copy", type=int, default=0, metavar="MIB",
                    help="also run one plain device-to-device copy of this many MiB (a kernel of known "
                         "traffic, to scale rocprofv3 FETCH_SIZE / WRITE_SIZE readings)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU; --gpus %d is not supported (every figure is a "
              "single-MI355X figure)" % args.gpus, file=sys.stderr)
        sys.exit(2)

    import torch
    from pink_amd import synthetic

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(3)
    w = synthetic.WORKLOADS[args.workload]
    # a mapping step is a few milliseconds of GPU time: enough of them that the clocks have settled
    if args.steps is None:
        args.steps = 30 if w.mode == "map" else 10
    if args.warmup is None:
        args.warmup = 10 if w.mode == "map" else 2
    cpu_budget = 0.0 if args.no_cpu_baseline else 10.0
    head = run_workload(args.workload, args.steps, args.warmup, args.images or w.n_images, args.kernel, cpu_budget,
                        not args.no_host_inclusive, False, args.calibrate_copy)
    out = {
        "metric": head["metric"], "value": head["value"], "unit": head["unit"], "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": head["ms_per_step"], "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": head["dtype"], "data": "synthetic", "config": head["config"],
        "value_is": "device_resident: images in HBM when the clock starts, the trainer's final SOM copied back inside it; "
                    "host_inclusive.value is the same step through the host-pointer entry points (H2D and D2H inside the clock)",
        "device_resident": head["value"],
        "roofline": head["roofline"], "cpu_baseline": head["cpu_baseline"], "host_inclusive": head["host_inclusive"],
        "setup_s": head["setup_s"],
    }
    if not args.no_all_configs:
        side = {}
        for name in ("cfg0", "cfg1", "cfg2", "cfg3", "cfg4"):
            if name == args.workload:
                continue
            wu, st = SIDE_STEPS[name]
            r = run_workload(name, st, wu, min(SIDE_IMAGES[name], synthetic.WORKLOADS[name].n_images), "auto",
                             0.0 if args.no_cpu_baseline else 5.0, not args.no_host_inclusive, True)
            side[name] = {k: r[k] for k in ("metric", "value", "device_resident", "unit", "steps", "warmup", "ms_per_step", "dtype", "config",
                                            "roofline", "cpu_baseline", "host_inclusive")}
        out["all_configs"] = side
    print(json.dumps(out))


if __name__ == "__main__":
    main()
