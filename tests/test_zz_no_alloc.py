"""pink_hip_map_device_static: the mapping entry point that allocates nothing (its per-group buffers
come from a static device array) against pink_hip_map_device on the same inputs, through the C ABI.
Bar: identical bits (heatmaps and best rotations), on two calls in a row, the second with fewer images,
and with contexts of different shapes taking turns on the one array.  Collected last on purpose.
"""
import ctypes as C
import sys

import numpy as np
import pytest

from pink_amd import capi

pytestmark = pytest.mark.gpu


class Hip:
    """Device buffers for the test straight from the HIP runtime that the library itself runs on (the
    one already in the process once the library is loaded), so that the test depends on nothing else."""

    def __init__(self):
        capi.lib()
        self.rt = C.CDLL("libamdhip64.so.7")
        self.rt.hipMalloc.argtypes = [C.POINTER(C.c_void_p), C.c_size_t]
        self.rt.hipMemcpy.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t, C.c_int]
        self.rt.hipMemset.argtypes = [C.c_void_p, C.c_int, C.c_size_t]
        self.rt.hipFree.argtypes = [C.c_void_p]
        self.rt.hipMemGetInfo.argtypes = [C.POINTER(C.c_size_t), C.POINTER(C.c_size_t)]
        self.held = []

    def ok(self, rc):
        assert rc == 0, "HIP error %d" % rc

    def alloc(self, nbytes, fill=0xff):
        p = C.c_void_p()
        self.ok(self.rt.hipMalloc(C.byref(p), max(nbytes, 16)))
        self.ok(self.rt.hipMemset(p, fill, max(nbytes, 16)))
        self.held.append(p)
        return p

    def upload(self, a):
        a = np.ascontiguousarray(a)
        p = self.alloc(a.nbytes)
        self.ok(self.rt.hipMemcpy(p, a.ctypes.data_as(C.c_void_p), a.nbytes, 1))      # host to device
        return p

    def download(self, p, shape, dtype):
        out = np.empty(shape, dtype)
        self.ok(self.rt.hipMemcpy(out.ctypes.data_as(C.c_void_p), p, out.nbytes, 2))   # device to host
        return out

    def free_bytes(self):
        free, total = C.c_size_t(), C.c_size_t()
        self.ok(self.rt.hipMemGetInfo(C.byref(free), C.byref(total)))
        return free.value

    def release(self):
        for p in self.held:
            self.rt.hipFree(p)
        self.held = []


def say(*a):
    print(*a, flush=True)
    sys.stdout.flush()


# N, C, I, D, nrot, flip, ed, shape, ed_type, kernel, images
SHAPES = [
    (100, 1, 64, 44, 360, True, 32, capi.QUADRATIC, capi.UINT8, capi.KERNEL_AUTO, 700),      # cfg 1: resident-SOM MFMA kernel, several groups
    (37, 1, 40, 29, 16, True, 21, capi.CIRCULAR, capi.UINT8, capi.KERNEL_MFMA, 33),
    (37, 1, 40, 29, 16, True, 21, capi.CIRCULAR, capi.UINT8, capi.KERNEL_MFMA_GEMM, 33),
    (70, 1, 40, 29, 16, True, 21, capi.CIRCULAR, capi.UINT16, capi.KERNEL_AUTO, 19),         # GEMM, two byte planes
    (9, 2, 17, 24, 8, True, 13, capi.QUADRATIC, capi.UINT8, capi.KERNEL_VALU, 11),           # float variants + a packing kernel
    (50, 1, 64, 44, 360, True, 32, capi.QUADRATIC, capi.FLOAT, capi.KERNEL_AUTO, 13),        # float32 rows out of the rotation kernel
    (5, 1, 290, 205, 8, True, 40, capi.CIRCULAR, capi.FLOAT, capi.KERNEL_AUTO, 3),           # nothing in LDS: two stored symmetries + packing kernels
]


def _run(ctx, fn, d_imgs, n, d_heat, d_best, hip):
    # outputs are filled with ones before every call (the buffers are the caller's, allocated beforehand)
    hip.ok(hip.rt.hipMemset(d_heat, 0xff, n * ctx.N * 4))
    hip.ok(hip.rt.hipMemset(d_best, 0xff, n * ctx.N * 4))
    fn(d_imgs, n, d_heat, d_best)
    ctx.synchronize()
    return hip.download(d_heat, (n, ctx.N), np.uint32), hip.download(d_best, (n, ctx.N), np.uint32)


def test_static_scratch_matches_the_allocating_entry_point():
    hip = Hip()
    rng = np.random.default_rng(2024)
    made = []
    try:
        for (N, C_, I, D, nrot, flip, ed, shape_, ed_type, choice, n) in SHAPES:
            ctx = capi.Context(N, C_, I, D, nrot, flip, ed, shape_, ed_type, kernel_choice=choice)
            ctx.set_som(rng.random((N, C_ * D * D), dtype=np.float32))
            imgs = hip.upload(rng.random((n, C_, I, I), dtype=np.float32))
            made.append((ctx, imgs, n, hip.alloc(n * N * 4), hip.alloc(n * N * 4)))
        want = [(_run(ctx, ctx.map_device, imgs, n, dh, db, hip), _run(ctx, ctx.map_device, imgs, max(1, n // 3), dh, db, hip))
                for ctx, imgs, n, dh, db in made]
        free_before = hip.free_bytes()
        # two rounds over all contexts: every call finds the array as a context of another shape left it
        for rnd in range(2):
            for (ctx, imgs, n, dh, db), (full, part) in zip(made, want):
                say("static scratch, round", rnd, "kernel", ctx.distance_kernel, "N", ctx.N, "images", n)
                got = _run(ctx, ctx.map_device_static, imgs, n, dh, db, hip)
                assert np.array_equal(got[0], full[0]) and np.array_equal(got[1], full[1])
                m = max(1, n // 3)
                got = _run(ctx, ctx.map_device_static, imgs, m, dh, db, hip)         # second call, fewer images
                assert np.array_equal(got[0], part[0]) and np.array_equal(got[1], part[1])
        # nothing was allocated on the device by the static calls (tolerance: what the runtime itself may
        # take for kernel arguments and signals)
        assert free_before - hip.free_bytes() <= 4 << 20
        # the allocating entry point still gives what it gave
        for (ctx, imgs, n, dh, db), (full, part) in zip(made, want):
            again = _run(ctx, ctx.map_device, imgs, n, dh, db, hip)
            assert np.array_equal(again[0], full[0]) and np.array_equal(again[1], full[1])
    finally:
        for m in made:
            m[0].close()
        hip.release()


def test_static_scratch_refusals():
    hip = Hip()
    try:
        imgs = hip.alloc(150 * 150 * 4, fill=0)
        heat = hip.alloc(16 * 4)
        # one image needs 200 x 200 region elements x 768 variant rows x 4 bytes = 123 MB: beyond the array
        with capi.Context(2, 1, 150, 200, 360, True, 200, capi.QUADRATIC, capi.FLOAT) as ctx:
            ctx.set_som(np.zeros((2, 200 * 200), np.float32))
            with pytest.raises(capi.PinkError) as e:
                ctx.map_device_static(imgs, 1, heat)
            assert e.value.status == -1 and "bytes of scratch" in str(e.value)
        F = capi.make_update_factors(capi.CARTESIAN, [2, 2], capi.GAUSSIAN, 1.0, 0.5)
        with capi.Context(4, 1, 16, 12, 8, True, 8, capi.QUADRATIC, capi.UINT8, F) as tr:
            with pytest.raises(capi.PinkError) as e:
                tr.map_device_static(imgs, 1, heat)
            assert e.value.status == -4 and "pink_hip_map_device_static" in str(e.value)
        # the float32 matrix-core kernel choice (measurement only) keeps its operands in the context's own buffers
        with capi.Context(4, 1, 16, 12, 8, True, 8, capi.QUADRATIC, capi.FLOAT, kernel_choice=capi.KERNEL_MFMA_F32) as mf:
            with pytest.raises(capi.PinkError) as e:
                mf.map_device_static(imgs, 1, heat)
            assert e.value.status == -4 and "float32 matrix-core" in str(e.value)
        with capi.Context(4, 1, 16, 12, 8, True, 8, capi.QUADRATIC, capi.UINT8) as mp:
            mp.set_profiling(True)
            with pytest.raises(capi.PinkError) as e:
                mp.map_device_static(imgs, 1, heat)
            assert e.value.status == -4
            mp.set_profiling(False)
            mp.map_device_static(imgs, 0, heat)          # no images: nothing to do
    finally:
        hip.release()
