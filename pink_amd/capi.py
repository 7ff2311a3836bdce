"""ctypes binding of the C ABI in include/pink_hip.h.

Loads pink_amd/lib/libpink_hip.so (built by `python -m pink_amd.build`) and raises
if it is missing: there is no CPU fallback.  Errors returned by the library become
`PinkError`, the counterpart of the reference's pink::exception
(src/UtilitiesLib/pink_exception.h:8-13).
"""
import ctypes as C
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "lib", "libpink_hip.so")

FLOAT, UINT16, UINT8 = 0, 1, 2
QUADRATIC, CIRCULAR = 0, 1
NEAREST_NEIGHBOR, BILINEAR = 0, 1
KERNEL_AUTO, KERNEL_VALU, KERNEL_MFMA, KERNEL_MFMA_SYM, KERNEL_MFMA_GEMM, KERNEL_MFMA_F32 = 0, 1, 2, 3, 4, 5
CARTESIAN, HEXAGONAL = 0, 1
STEP, GAUSSIAN, UNITY_GAUSSIAN, MEXICAN_HAT = 0, 1, 2, 3
NUM_KERNEL_CLASSES = 5
KERNEL_CLASS_NAMES = ("rotate", "pack", "distance", "update", "finalize")

EXPORTS = (
    "pink_hip_abi_version", "pink_hip_create", "pink_hip_destroy", "pink_hip_last_error",
    "pink_hip_set_som", "pink_hip_get_som", "pink_hip_train", "pink_hip_train_device",
    "pink_hip_map", "pink_hip_map_device", "pink_hip_synchronize", "pink_hip_rotate",
    "pink_hip_distance", "pink_hip_region_size", "pink_hip_distance_kernel", "pink_hip_set_profiling",
    "pink_hip_kernel_times", "pink_hip_device_info", "pink_hip_som_size",
    "pink_hip_make_update_factors", "pink_hip_layout_distances", "pink_hip_shuffled_order",
    "pink_hip_fill_random_uniform", "pink_hip_update_counts", "pink_hip_check_config",
    "pink_hip_map_device_static",
)


class PinkError(RuntimeError):
    def __init__(self, status, message):
        super().__init__(message)
        self.status = status


class Config(C.Structure):
    _fields_ = [
        ("som_size", C.c_uint32), ("channels", C.c_uint32), ("image_dim", C.c_uint32),
        ("neuron_dim", C.c_uint32), ("num_rot", C.c_uint32), ("use_flip", C.c_uint32),
        ("interpolation", C.c_uint32), ("ed_dim", C.c_uint32), ("ed_shape", C.c_uint32),
        ("ed_type", C.c_uint32), ("update_factors", C.POINTER(C.c_float)), ("device", C.c_int32),
        ("max_batch", C.c_uint32), ("kernel_choice", C.c_uint32),
    ]


_lib = None


def lib():
    """The loaded library.  Raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise PinkError(-3, "%s is missing: run `python -m pink_amd.build` (there is no CPU fallback)" % LIB_PATH)
        # PyTorch ships a HIP runtime of its own; this library runs on the system's.  Both can live in one
        # process, but PyTorch's must initialise first: once this library has touched the GPU, a PyTorch that
        # initialises afterwards finds no devices.  So where PyTorch is already imported, bring it up now.
        torch = sys.modules.get("torch")
        if torch is not None:
            try:
                if torch.cuda.is_available():
                    torch.cuda.init()
            except Exception:       # a PyTorch without a GPU build, or no GPU: nothing to order
                pass
        L = C.CDLL(LIB_PATH)
        vp, u32, f32p, u32p = C.c_void_p, C.c_uint32, C.POINTER(C.c_float), C.POINTER(C.c_uint32)
        L.pink_hip_abi_version.restype = C.c_int
        L.pink_hip_create.argtypes = [C.POINTER(vp), C.POINTER(Config)]
        L.pink_hip_check_config.argtypes = [C.POINTER(Config)]
        L.pink_hip_destroy.argtypes = [vp]
        L.pink_hip_destroy.restype = None
        L.pink_hip_last_error.argtypes = [vp]
        L.pink_hip_last_error.restype = C.c_char_p
        L.pink_hip_set_som.argtypes = [vp, f32p]
        L.pink_hip_get_som.argtypes = [vp, f32p]
        L.pink_hip_train.argtypes = [vp, f32p, u32, u32p]
        L.pink_hip_update_counts.argtypes = [vp, u32p]
        L.pink_hip_train_device.argtypes = [vp, vp, u32, vp]
        L.pink_hip_map.argtypes = [vp, f32p, u32, f32p, u32p]
        L.pink_hip_map_device.argtypes = [vp, vp, u32, vp, vp]
        L.pink_hip_map_device_static.argtypes = [vp, vp, u32, vp, vp]
        L.pink_hip_synchronize.argtypes = [vp]
        L.pink_hip_rotate.argtypes = [vp, f32p, f32p]
        L.pink_hip_distance.argtypes = [vp, f32p, f32p, C.POINTER(C.c_int64), u32p]
        L.pink_hip_region_size.argtypes = [vp]
        L.pink_hip_region_size.restype = u32
        L.pink_hip_distance_kernel.argtypes = [vp]
        L.pink_hip_distance_kernel.restype = u32
        L.pink_hip_set_profiling.argtypes = [vp, C.c_int]
        L.pink_hip_kernel_times.argtypes = [vp, C.POINTER(C.c_uint64), C.POINTER(C.c_double)]
        L.pink_hip_device_info.argtypes = [C.c_char_p, C.c_size_t]
        L.pink_hip_som_size.argtypes = [u32, u32p, u32]
        L.pink_hip_som_size.restype = u32
        L.pink_hip_make_update_factors.argtypes = [u32, u32p, u32, u32, C.c_float, C.c_float, C.c_float, f32p]
        L.pink_hip_layout_distances.argtypes = [u32, u32p, u32, f32p]
        L.pink_hip_shuffled_order.argtypes = [C.c_uint64, u32, u32p]
        L.pink_hip_fill_random_uniform.argtypes = [f32p, C.c_size_t, u32]
        _lib = L
    return _lib


def _f32(a):
    return a.ctypes.data_as(C.POINTER(C.c_float))


def _u32(a):
    return a.ctypes.data_as(C.POINTER(C.c_uint32))


def device_info():
    buf = C.create_string_buffer(4096)
    n = lib().pink_hip_device_info(buf, len(buf))
    if n < 0:
        raise PinkError(n, lib().pink_hip_last_error(None).decode())
    return n, buf.value.decode()


def som_size(layout, dims):
    dims = np.asarray(dims, np.uint32)
    return int(lib().pink_hip_som_size(layout, _u32(dims), len(dims)))


def make_update_factors(layout, dims, functor, sigma, damping=0.0, max_update_distance=-1.0):
    """The N x N matrix of TrainerCommon (Trainer.h:69-76), row = BMU."""
    dims = np.ascontiguousarray(dims, np.uint32)
    n = som_size(layout, dims)
    if n == 0:
        raise PinkError(-1, "invalid SOM layout dimensions")
    out = np.empty((n, n), np.float32)
    rc = lib().pink_hip_make_update_factors(layout, _u32(dims), len(dims), functor, sigma, damping,
                                            max_update_distance, _f32(out))
    if rc != 0:
        raise PinkError(rc, "pink_hip_make_update_factors: invalid argument")
    return out


def layout_distances(layout, dims):
    """SOMLayout::get_distance for all neuron pairs, (N, N) float32."""
    dims = np.ascontiguousarray(dims, np.uint32)
    n = som_size(layout, dims)
    if n == 0:
        raise PinkError(-1, "invalid SOM layout dimensions")
    out = np.empty((n, n), np.float32)
    rc = lib().pink_hip_layout_distances(layout, _u32(dims), len(dims), _f32(out))
    if rc != 0:
        raise PinkError(rc, "pink_hip_layout_distances: invalid argument")
    return out


def shuffled_order(seed, n):
    """The order in which the reference's shuffled iterator visits n entries (DataIteratorShuffled.h:62-69)."""
    out = np.empty(n, np.uint32)
    rc = lib().pink_hip_shuffled_order(int(seed), n, _u32(out))
    if rc != 0:
        raise PinkError(rc, "pink_hip_shuffled_order: invalid argument")
    return out


def fill_random_uniform(length, seed):
    """fill_random_uniform (UtilitiesLib/Filler.h:16-25): `length` float32 in [0, 1) from std::mt19937(seed)."""
    out = np.empty(length, np.float32)
    rc = lib().pink_hip_fill_random_uniform(_f32(out), length, int(seed))
    if rc != 0:
        raise PinkError(rc, "pink_hip_fill_random_uniform: invalid argument")
    return out


def check_config(som_size, channels, image_dim, neuron_dim, num_rot, use_flip, ed_dim, ed_shape=QUADRATIC,
                 ed_type=FLOAT, interpolation=BILINEAR):
    """The argument checks of a context's creation without touching a device; raises PinkError as
    the creation would."""
    cfg = Config(som_size, channels, image_dim, neuron_dim, num_rot, int(bool(use_flip)), interpolation,
                 ed_dim, ed_shape, ed_type, None, 0, 0, KERNEL_AUTO)
    rc = lib().pink_hip_check_config(C.byref(cfg))
    if rc != 0:
        raise PinkError(rc, lib().pink_hip_last_error(None).decode())


class Context:
    """One device context: a trainer when `update_factors` is given, else a mapper."""

    def __init__(self, som_size, channels, image_dim, neuron_dim, num_rot, use_flip, ed_dim,
                 ed_shape=QUADRATIC, ed_type=FLOAT, update_factors=None, interpolation=BILINEAR,
                 device=0, max_batch=0, kernel_choice=KERNEL_AUTO):
        self._h = C.c_void_p()
        self._L = lib()
        cfg = Config(som_size, channels, image_dim, neuron_dim, num_rot, int(bool(use_flip)), interpolation,
                     ed_dim, ed_shape, ed_type, None, device, max_batch, kernel_choice)
        if update_factors is not None:
            uf = np.ascontiguousarray(update_factors, np.float32)
            if uf.size != som_size * som_size:
                raise PinkError(-1, "update_factors must hold som_size * som_size floats")
            cfg.update_factors = _f32(uf)
        rc = self._L.pink_hip_create(C.byref(self._h), C.byref(cfg))
        if rc != 0:
            self._h = C.c_void_p()
            raise PinkError(rc, self._L.pink_hip_last_error(None).decode())
        self.N, self.C, self.I, self.D = som_size, channels, image_dim, neuron_dim
        self.R = num_rot * (2 if use_flip else 1)
        self.S = channels * neuron_dim * neuron_dim
        self.image_size = channels * image_dim * image_dim
        self.ed_type = ed_type

    def _check(self, rc):
        if rc != 0:
            raise PinkError(rc, self._L.pink_hip_last_error(self._h).decode())

    def close(self):
        if self._h:
            self._L.pink_hip_destroy(self._h)
            self._h = C.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def __enter__(self):
        return self

    def __exit__(self, *a):
        self.close()

    @property
    def region_size(self):
        return int(self._L.pink_hip_region_size(self._h))

    @property
    def distance_kernel(self):
        """KERNEL_VALU, KERNEL_MFMA or KERNEL_MFMA_SYM: the distance kernel this context runs."""
        return int(self._L.pink_hip_distance_kernel(self._h))

    def set_som(self, som):
        som = np.ascontiguousarray(som, np.float32)
        assert som.size == self.N * self.S
        self._check(self._L.pink_hip_set_som(self._h, _f32(som)))

    def get_som(self, out=None):
        if out is None:
            out = np.empty((self.N, self.S), np.float32)
        assert out.dtype == np.float32 and out.flags.c_contiguous and out.size == self.N * self.S
        self._check(self._L.pink_hip_get_som(self._h, _f32(out)))
        return out

    def train(self, images, want_bmu=True):
        """Train on the images in order.  want_bmu=False returns nothing and, for up to 128 KiB of
        images, only copies them: they are trained in order a launch group at a time, when the group is full or
        another call on the context follows (update_counts / synchronize / get_som wait for the result)."""
        images = np.ascontiguousarray(images, np.float32)
        n = images.size // self.image_size
        assert n * self.image_size == images.size
        if not want_bmu:
            self._check(self._L.pink_hip_train(self._h, _f32(images), n, None))
            return None
        bmu = np.empty(n, np.uint32)
        self._check(self._L.pink_hip_train(self._h, _f32(images), n, _u32(bmu)))
        return bmu

    def update_counts(self):
        """How often each neuron was the best match so far (the reference's update info)."""
        counts = np.empty(self.N, np.uint32)
        self._check(self._L.pink_hip_update_counts(self._h, _u32(counts)))
        return counts

    def train_device(self, dev_images_ptr, n, dev_bmu_ptr=None):
        self._check(self._L.pink_hip_train_device(self._h, dev_images_ptr, n, dev_bmu_ptr))

    def map(self, images):
        images = np.ascontiguousarray(images, np.float32)
        n = images.size // self.image_size
        assert n * self.image_size == images.size
        heat = np.empty((n, self.N), np.float32)
        best = np.empty((n, self.N), np.uint32)
        self._check(self._L.pink_hip_map(self._h, _f32(images), n, _f32(heat), _u32(best)))
        return heat, best

    def map_device(self, dev_images_ptr, n, dev_heat_ptr, dev_best_ptr=None):
        self._check(self._L.pink_hip_map_device(self._h, dev_images_ptr, n, dev_heat_ptr, dev_best_ptr))

    def map_device_static(self, dev_images_ptr, n, dev_heat_ptr, dev_best_ptr=None):
        """map_device out of the library's static scratch array: allocates nothing."""
        self._check(self._L.pink_hip_map_device_static(self._h, dev_images_ptr, n, dev_heat_ptr, dev_best_ptr))

    def synchronize(self):
        self._check(self._L.pink_hip_synchronize(self._h))

    def rotate(self, image):
        image = np.ascontiguousarray(image, np.float32)
        assert image.size == self.image_size
        out = np.empty((self.R, self.C, self.D, self.D), np.float32)
        self._check(self._L.pink_hip_rotate(self._h, _f32(image), _f32(out)))
        return out

    def distance(self, image):
        image = np.ascontiguousarray(image, np.float32)
        assert image.size == self.image_size
        d = np.empty(self.N, np.float32)
        ssd = np.zeros(self.N, np.int64)
        best = np.empty(self.N, np.uint32)
        self._check(self._L.pink_hip_distance(self._h, _f32(image), _f32(d),
                                              ssd.ctypes.data_as(C.POINTER(C.c_int64)), _u32(best)))
        return d, ssd, best

    def set_profiling(self, enable):
        self._check(self._L.pink_hip_set_profiling(self._h, int(bool(enable))))

    def kernel_times(self):
        """{class name: (launches, total ms)} since profiling was last switched on."""
        n = (C.c_uint64 * NUM_KERNEL_CLASSES)()
        ms = (C.c_double * NUM_KERNEL_CLASSES)()
        self._check(self._L.pink_hip_kernel_times(self._h, n, ms))
        return {KERNEL_CLASS_NAMES[i]: (int(n[i]), float(ms[i])) for i in range(NUM_KERNEL_CLASSES)}
