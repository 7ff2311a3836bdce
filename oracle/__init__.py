"""ctypes bindings of the CPU oracle -- TEST INFRASTRUCTURE ONLY.

`oracle.lib()` loads oracle/libpink_oracle.so (the C restatement of the reference
CPU path, oracle/pink_oracle.c); `oracle.ref()` loads oracle/_ref/libpink_ref.so (the
real reference headers behind extern "C", oracle/ref_shim.cpp) when it has been
built.  Only tests, the smoke check and the benchmark's cpu_baseline leg import
this module; the shipped library never does.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = None
_REF = None

FLOAT, UINT16, UINT8 = 0, 1, 2
QUADRATIC, CIRCULAR = 0, 1
CARTESIAN, HEXAGONAL = 0, 1
STEP, GAUSSIAN, UNITY_GAUSSIAN, MEXICAN_HAT = 0, 1, 2, 3

_f32p = np.ctypeslib.ndpointer(np.float32, flags="C_CONTIGUOUS")
_u32p = np.ctypeslib.ndpointer(np.uint32, flags="C_CONTIGUOUS")
_i32p = np.ctypeslib.ndpointer(np.int32, flags="C_CONTIGUOUS")
_i64p = np.ctypeslib.ndpointer(np.int64, flags="C_CONTIGUOUS")


class Shape(C.Structure):
    _fields_ = [(n, C.c_uint32) for n in (
        "som_size", "channels", "image_dim", "neuron_dim", "num_rot", "use_flip",
        "ed_dim", "ed_shape", "ed_type")]

    @property
    def R(self):
        return self.num_rot * (2 if self.use_flip else 1)

    @property
    def neuron_size(self):
        return self.channels * self.neuron_dim * self.neuron_dim

    @property
    def image_size(self):
        return self.channels * self.image_dim * self.image_dim


def build():
    """(Re)build the oracle and, if the reference tree is present, oracle/_ref."""
    subprocess.check_call(["make", "-s", "-C", _HERE])


def lib():
    global _LIB
    if _LIB is None:
        path = os.path.join(_HERE, "libpink_oracle.so")
        if not os.path.exists(path):
            build()
        L = C.CDLL(path)
        L.pink_oracle_region.restype = C.c_uint32
        L.pink_oracle_ssd_f32.restype = C.c_float
        L.pink_oracle_ssd_int.restype = C.c_int64
        L.pink_oracle_quantise.restype = C.c_int32
        L.pink_oracle_quantise.argtypes = [C.c_float, C.c_uint32]
        L.pink_oracle_hex_size.restype = C.c_uint32
        L.pink_oracle_cartesian_distance.restype = C.c_float
        L.pink_oracle_hex_distance.restype = C.c_float
        L.pink_oracle_functor.restype = C.c_float
        L.pink_oracle_functor.argtypes = [C.c_uint32, C.c_float, C.c_float, C.c_float]
        L.pink_oracle_bmu.restype = C.c_uint32
        _LIB = L
    return _LIB


def ref():
    """The real-reference shim, or None when oracle/_ref has not been built."""
    global _REF
    if _REF is None:
        path = os.path.join(_HERE, "_ref", "libpink_ref.so")
        if not os.path.exists(path):
            return None
        L = C.CDLL(path)
        L.ref_ssd_f32.restype = C.c_float
        L.ref_ssd_i32.restype = C.c_int32
        L.ref_ssd_i64.restype = C.c_int64
        L.ref_cartesian_distance.restype = C.c_float
        L.ref_hex_distance.restype = C.c_float
        L.ref_hex_size.restype = C.c_uint32
        L.ref_functor.restype = C.c_float
        L.ref_functor.argtypes = [C.c_uint32, C.c_float, C.c_float, C.c_float]
        _REF = L
    return _REF


def _p(a, t):
    return a.ctypes.data_as(C.POINTER(t))


def shape(som_size, channels, image_dim, neuron_dim, num_rot, use_flip, ed_dim,
          ed_shape=QUADRATIC, ed_type=FLOAT):
    return Shape(som_size, channels, image_dim, neuron_dim, num_rot, int(bool(use_flip)),
                 ed_dim, ed_shape, ed_type)


# ---- oracle wrappers --------------------------------------------------------
def rotated_images(image, channels, image_dim, neuron_dim, num_rot, use_flip):
    image = np.ascontiguousarray(image, np.float32)
    R = num_rot * (2 if use_flip else 1)
    out = np.empty((R, channels, neuron_dim, neuron_dim), np.float32)
    lib().pink_oracle_rotated_images(_p(image, C.c_float), C.c_uint32(channels), C.c_uint32(image_dim),
                                     C.c_uint32(neuron_dim), C.c_uint32(num_rot), C.c_int(int(use_flip)),
                                     _p(out, C.c_float))
    return out


def rotate_bilinear(src, dst_dim, alpha):
    src = np.ascontiguousarray(src, np.float32)
    dst = np.empty((dst_dim, dst_dim), np.float32)
    lib().pink_oracle_rotate_bilinear(_p(src, C.c_float), _p(dst, C.c_float), C.c_uint32(src.shape[0]),
                                      C.c_uint32(src.shape[1]), C.c_uint32(dst_dim), C.c_uint32(dst_dim),
                                      C.c_float(alpha))
    return dst


def region(channels, neuron_dim, ed_dim, ed_shape):
    n = lib().pink_oracle_region(C.c_uint32(channels), C.c_uint32(neuron_dim), C.c_uint32(ed_dim),
                                 C.c_uint32(ed_shape), None)
    off = np.empty(max(n, 1), np.uint32)
    lib().pink_oracle_region(C.c_uint32(channels), C.c_uint32(neuron_dim), C.c_uint32(ed_dim),
                             C.c_uint32(ed_shape), _p(off, C.c_uint32))
    return off[:n]


def ssd_f32(a, b, channels, neuron_dim, ed_dim, ed_shape):
    a = np.ascontiguousarray(a, np.float32)
    b = np.ascontiguousarray(b, np.float32)
    return float(lib().pink_oracle_ssd_f32(_p(a, C.c_float), _p(b, C.c_float), C.c_uint32(channels),
                                           C.c_uint32(neuron_dim), C.c_uint32(ed_dim), C.c_uint32(ed_shape)))


def ssd_int(a, b, channels, neuron_dim, ed_dim, ed_shape):
    a = np.ascontiguousarray(a, np.int32)
    b = np.ascontiguousarray(b, np.int32)
    return int(lib().pink_oracle_ssd_int(_p(a, C.c_int32), _p(b, C.c_int32), C.c_uint32(channels),
                                         C.c_uint32(neuron_dim), C.c_uint32(ed_dim), C.c_uint32(ed_shape)))


def quantise(x, ed_type):
    return np.array([lib().pink_oracle_quantise(float(v), ed_type) for v in np.ravel(x)],
                    np.int32).reshape(np.shape(x))


def distance_matrix(s, som, rotated):
    som = np.ascontiguousarray(som, np.float32)
    rotated = np.ascontiguousarray(rotated, np.float32)
    d = np.empty(s.som_size, np.float32)
    ssd = np.zeros(s.som_size, np.int64)
    best = np.zeros(s.som_size, np.uint32)
    lib().pink_oracle_distance_matrix(C.byref(s), _p(som, C.c_float), _p(rotated, C.c_float),
                                      _p(d, C.c_float), _p(ssd, C.c_int64), _p(best, C.c_uint32))
    return d, ssd, best


def distance_matrix_pairwise(s, som, rotated):
    """The same matrix with one functor call per pair (what distance_matrix is checked against)."""
    som = np.ascontiguousarray(som, np.float32)
    rotated = np.ascontiguousarray(rotated, np.float32)
    d = np.empty(s.som_size, np.float32)
    ssd = np.zeros(s.som_size, np.int64)
    best = np.zeros(s.som_size, np.uint32)
    lib().pink_oracle_distance_matrix_pairwise(C.byref(s), _p(som, C.c_float), _p(rotated, C.c_float),
                                               _p(d, C.c_float), _p(ssd, C.c_int64), _p(best, C.c_uint32))
    return d, ssd, best


def distance_matrix_reference_loop(s, som, rotated):
    """Float mode with the reference's own OpenMP structure (a parallel loop over rotations per neuron,
    a call through a pointer and a critical section per pair)."""
    som = np.ascontiguousarray(som, np.float32)
    rotated = np.ascontiguousarray(rotated, np.float32)
    d = np.empty(s.som_size, np.float32)
    best = np.zeros(s.som_size, np.uint32)
    lib().pink_oracle_distance_matrix_reference_loop(C.byref(s), _p(som, C.c_float), _p(rotated, C.c_float),
                                                     _p(d, C.c_float), _p(best, C.c_uint32))
    return d, best


def update_factors(layout, dims, functor, sigma, damping, max_update_distance=-1.0):
    dims = np.asarray(dims, np.uint32)
    N = int(lib().pink_oracle_hex_size(C.c_uint32(int(dims[0])))) if layout == HEXAGONAL else int(np.prod(dims))
    F = np.empty((N, N), np.float32)
    lib().pink_oracle_update_factors(C.c_uint32(layout), _p(dims, C.c_uint32), C.c_uint32(len(dims)),
                                     C.c_uint32(functor), C.c_float(sigma), C.c_float(damping),
                                     C.c_float(max_update_distance), _p(F, C.c_float))
    return F


def bmu(s, dist, ssd=None):
    dist = np.ascontiguousarray(dist, np.float32)
    ssd_p = _p(np.ascontiguousarray(ssd, np.int64), C.c_int64) if ssd is not None else None
    return int(lib().pink_oracle_bmu(C.byref(s), _p(dist, C.c_float), ssd_p))


def update(som, rotated, best_rot, bmu_idx, factors):
    """In-place neuron update of `som` (N, neuron_size)."""
    assert som.dtype == np.float32 and som.flags.c_contiguous
    rotated = np.ascontiguousarray(rotated, np.float32)
    best_rot = np.ascontiguousarray(best_rot, np.uint32)
    factors = np.ascontiguousarray(factors, np.float32)
    N = factors.shape[0]
    lib().pink_oracle_update(_p(som, C.c_float), C.c_uint32(N), C.c_uint32(som.size // N),
                             _p(rotated, C.c_float), _p(best_rot, C.c_uint32), C.c_uint32(bmu_idx),
                             _p(factors, C.c_float))


def train_step(s, som, image, factors):
    """One Trainer call; `som` updated in place.  Returns (bmu, dist, best_rot)."""
    assert som.dtype == np.float32 and som.flags.c_contiguous
    image = np.ascontiguousarray(image, np.float32)
    factors = np.ascontiguousarray(factors, np.float32)
    b = C.c_uint32(0)
    d = np.empty(s.som_size, np.float32)
    best = np.empty(s.som_size, np.uint32)
    rc = lib().pink_oracle_train_step(C.byref(s), _p(som, C.c_float), _p(image, C.c_float),
                                      _p(factors, C.c_float), None, C.byref(b), _p(d, C.c_float),
                                      _p(best, C.c_uint32))
    assert rc == 0
    return b.value, d, best


def train(s, som, images, factors):
    assert som.dtype == np.float32 and som.flags.c_contiguous
    images = np.ascontiguousarray(images, np.float32)
    factors = np.ascontiguousarray(factors, np.float32)
    n = images.size // s.image_size
    bmus = np.empty(n, np.uint32)
    rc = lib().pink_oracle_train(C.byref(s), _p(som, C.c_float), _p(images, C.c_float), C.c_uint32(n),
                                 _p(factors, C.c_float), _p(bmus, C.c_uint32))
    assert rc == 0
    return bmus


def map_images(s, som, images):
    som = np.ascontiguousarray(som, np.float32)
    images = np.ascontiguousarray(images, np.float32)
    n = images.size // s.image_size
    heat = np.empty((n, s.som_size), np.float32)
    best = np.empty((n, s.som_size), np.uint32)
    rc = lib().pink_oracle_map(C.byref(s), _p(som, C.c_float), _p(images, C.c_float), C.c_uint32(n),
                               _p(heat, C.c_float), _p(best, C.c_uint32))
    assert rc == 0
    return heat, best


LANES, PAIRWISE, REFERENCE_LOOP = 0, 1, 2


def set_distance_form(form):
    """Which evaluation of the distance matrix train() and map_images() use (LANES by default)."""
    assert lib().pink_oracle_set_distance_form(C.c_int(form)) == 0


def num_threads():
    return int(lib().pink_oracle_num_threads())


def set_num_threads(n):
    lib().pink_oracle_set_num_threads(C.c_int(int(n)))


def fill_random_uniform(n, seed):
    a = np.empty(n, np.float32)
    lib().pink_oracle_fill_random_uniform(_p(a, C.c_float), C.c_size_t(n), C.c_uint32(seed))
    return a


def shuffled_order(seed, n):
    a = np.empty(n, np.uint32)
    lib().pink_oracle_shuffled_order(C.c_uint64(seed), C.c_uint32(n), _p(a, C.c_uint32))
    return a


def ref_shuffled_order(seed, n, shuffle=True):
    a = np.empty(n, np.uint32)
    ref().ref_shuffled_order(C.c_uint64(seed), C.c_uint32(n), C.c_int(int(shuffle)), _p(a, C.c_uint32))
    return a


def ref_progress_ticks(total, max_prints):
    a = np.empty(total, np.int32)
    k = ref().ref_progress_ticks(C.c_int(total), C.c_int(max_prints), _p(a, C.c_int32))
    return a[:k].tolist()


def mt19937_raw(seed, n):
    a = np.empty(n, np.uint32)
    lib().pink_oracle_mt19937_raw(C.c_uint32(seed), _p(a, C.c_uint32), C.c_size_t(n))
    return a


# ---- real-reference wrappers (None-safe callers check ref() first) -----------
def ref_rotated_images(image, channels, image_dim, neuron_dim, num_rot, use_flip, data_dims=None):
    image = np.ascontiguousarray(image, np.float32)
    data_dims = data_dims or (2 if channels == 1 else 3)
    R = num_rot * (2 if use_flip else 1)
    out = np.empty((R, channels, neuron_dim, neuron_dim), np.float32)
    n = ref().ref_rotated_images(_p(image, C.c_float), C.c_uint32(channels), C.c_uint32(image_dim),
                                 C.c_uint32(neuron_dim), C.c_uint32(num_rot), C.c_int(int(use_flip)),
                                 C.c_uint32(data_dims), _p(out, C.c_float))
    assert n == out.size
    return out


def ref_rotate_bilinear(src, dst_dim, alpha):
    src = np.ascontiguousarray(src, np.float32)
    dst = np.empty((dst_dim, dst_dim), np.float32)
    ref().ref_rotate_bilinear(_p(src, C.c_float), _p(dst, C.c_float), C.c_uint32(src.shape[0]),
                              C.c_uint32(src.shape[1]), C.c_uint32(dst_dim), C.c_uint32(dst_dim),
                              C.c_float(alpha))
    return dst


def ref_ssd_f32(a, b, channels, neuron_dim, ed_dim, ed_shape, data_dims=None):
    a = np.ascontiguousarray(a, np.float32)
    b = np.ascontiguousarray(b, np.float32)
    data_dims = data_dims or (2 if channels == 1 else 3)
    return float(ref().ref_ssd_f32(_p(a, C.c_float), _p(b, C.c_float), C.c_uint32(channels),
                                   C.c_uint32(neuron_dim), C.c_uint32(ed_dim), C.c_uint32(ed_shape),
                                   C.c_uint32(data_dims)))


def ref_ssd_i64(a, b, channels, neuron_dim, ed_dim, ed_shape, data_dims=None):
    a = np.ascontiguousarray(a, np.int64)
    b = np.ascontiguousarray(b, np.int64)
    data_dims = data_dims or (2 if channels == 1 else 3)
    return int(ref().ref_ssd_i64(_p(a, C.c_int64), _p(b, C.c_int64), C.c_uint32(channels),
                                 C.c_uint32(neuron_dim), C.c_uint32(ed_dim), C.c_uint32(ed_shape),
                                 C.c_uint32(data_dims)))
