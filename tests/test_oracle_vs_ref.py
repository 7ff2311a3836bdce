"""Differential test: the C oracle against the REAL reference headers.

oracle/_ref/libpink_ref.so is the reference's own templates (ImageProcessingLib,
generate_rotated_images.h, layouts, functors, filler) compiled where they lie by
oracle/Makefile.  Every comparison is bit-for-bit.  Skipped when the library has
not been built (no reference tree on this machine).
"""
import ctypes as C

import numpy as np
import pytest

ROT_SHAPES = [
    # C, I, D, num_rot, flip        (the benchmark configurations, then the odd ones of
    #                                test/CudaTest/compare_trainer_cpu.cu:81-98)
    (1, 64, 44, 360, True),         # cfg 0 / 1
    (1, 150, 106, 360, True),       # cfg 2
    (3, 100, 70, 180, True),        # cfg 3
    (1, 28, 28, 4, True),           # cfg 4
    (1, 64, 45, 360, True),
    (1, 64, 100, 360, True),        # image smaller than the neuron: padded
    (1, 124, 91, 360, True),
    (2, 17, 24, 16, False),
    (1, 2, 4, 1, False),
    (1, 4, 2, 8, True),
    (1, 5, 3, 360, False),
    (3, 9, 9, 1, True),
]


@pytest.mark.parametrize("C_,I,D,nrot,flip", ROT_SHAPES)
def test_rotated_images_bit_exact(ref_mod, C_, I, D, nrot, flip):
    O = ref_mod
    rng = np.random.default_rng(1000 + I * D + nrot)
    img = rng.random((C_, I, I), dtype=np.float32)
    got = O.rotated_images(img, C_, I, D, nrot, flip)
    want = O.ref_rotated_images(img, C_, I, D, nrot, flip)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    if C_ == 1:   # 3-D layout with depth 1 is the same bytes as 2-D
        want3 = O.ref_rotated_images(img, C_, I, D, nrot, flip, data_dims=3)
        assert np.array_equal(got.view(np.uint32), want3.view(np.uint32))


def test_rotate_bilinear_many_angles(ref_mod):
    O = ref_mod
    rng = np.random.default_rng(5)
    for I, D in ((64, 44), (31, 40), (8, 8)):
        img = rng.random((I, I), dtype=np.float32) - 0.25
        for alpha in rng.uniform(0, 2 * np.pi, 25).astype(np.float32):
            got = O.rotate_bilinear(img, D, float(alpha))
            want = O.ref_rotate_bilinear(img, D, float(alpha))
            assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


SSD_SHAPES = [
    # C, D, e, shape
    (1, 44, 32, 0), (1, 106, 75, 1), (3, 70, 50, 0), (1, 28, 28, 0),
    (1, 45, 45, 0), (1, 91, 64, 0), (1, 100, 45, 0), (1, 44, 32, 1), (1, 45, 31, 1),
    (2, 24, 13, 0), (2, 24, 13, 1), (3, 70, 50, 1), (1, 300, 200, 1), (1, 7, 6, 1),
]


@pytest.mark.parametrize("C_,D,e,shape_", SSD_SHAPES)
def test_ssd_f32_bit_exact(ref_mod, C_, D, e, shape_):
    O = ref_mod
    rng = np.random.default_rng(2000 + D * e + shape_)
    for trial in range(12):
        a = rng.random(C_ * D * D, dtype=np.float32)
        b = rng.random(C_ * D * D, dtype=np.float32)
        if trial % 3 == 1:
            b = (a + rng.normal(0, 1e-3, a.shape)).astype(np.float32)   # near match
        if trial % 3 == 2:
            b *= np.float32(0.01)                                         # neuron-dominated
        got = np.float32(O.ssd_f32(a, b, C_, D, e, shape_))
        want = np.float32(O.ref_ssd_f32(a, b, C_, D, e, shape_))
        assert got.view(np.uint32) == want.view(np.uint32)


@pytest.mark.parametrize("C_,D,e,shape_", SSD_SHAPES)
def test_ssd_integer_exact(ref_mod, C_, D, e, shape_):
    O = ref_mod
    rng = np.random.default_rng(3000 + D * e + shape_)
    for hi in (256, 65536):
        a = rng.integers(0, hi, C_ * D * D)
        b = rng.integers(0, hi, C_ * D * D)
        got = O.ssd_int(a, b, C_, D, e, shape_)
        assert got == O.ref_ssd_i64(a, b, C_, D, e, shape_)
        off = O.region(C_, D, e, shape_)
        assert got == int(((a[off] - b[off]) ** 2).sum())


def test_layout_distances(ref_mod):
    O = ref_mod
    L, Rf = O.lib(), O.ref()
    for dims in ([10, 10], [40, 40], [8, 8], [3, 5], [7], [2, 3, 4]):
        d = (C.c_uint32 * len(dims))(*dims)
        n = int(np.prod(dims))
        idx = np.random.default_rng(n).integers(0, n, (200, 2))
        for i, j in idx:
            assert L.pink_oracle_cartesian_distance(d, len(dims), int(i), int(j)) == \
                Rf.ref_cartesian_distance(d, len(dims), int(i), int(j))
    for dim in (3, 5, 21):
        n = Rf.ref_hex_size(dim)
        assert n == L.pink_oracle_hex_size(dim)
        for i in range(0, n, max(1, n // 40)):
            for j in range(n):
                assert L.pink_oracle_hex_distance(dim, i, j) == Rf.ref_hex_distance(dim, i, j)


def test_functors_bit_exact(ref_mod):
    O = ref_mod
    L, Rf = O.lib(), O.ref()
    dists = np.concatenate([np.arange(0, 60, dtype=np.float32),
                            np.sqrt(np.arange(0, 400, dtype=np.float32))])
    for kind in range(4):
        for sigma, damping in ((1.1, 0.2), (1.5, 0.1), (2.0, 0.05), (1.0, 0.3), (10.0, 1.0)):
            for x in dists:
                a = np.float32(L.pink_oracle_functor(kind, sigma, damping, float(x)))
                b = np.float32(Rf.ref_functor(kind, sigma, damping, float(x)))
                assert a.view(np.uint32) == b.view(np.uint32), (kind, sigma, damping, x)


def test_filler_bit_exact(ref_mod):
    O = ref_mod
    for seed in (1234, 5489, 0, 42):
        n = 100000
        want = np.empty(n, np.float32)
        O.ref().ref_fill_random_uniform(want.ctypes.data_as(C.POINTER(C.c_float)), C.c_size_t(n), C.c_uint32(seed))
        assert np.array_equal(O.fill_random_uniform(n, seed).view(np.uint32), want.view(np.uint32))


def test_shuffled_order_matches_the_reference_iterator(ref_mod):
    O = ref_mod
    # both branches of std::shuffle (two positions per draw up to 65536 entries, one beyond), odd and even
    # lengths, a seed beyond 32 bits, the seeds 0 and 2^31 - 1 that the first engine maps to 1
    for seed, n in ((2, 2), (1234, 10), (1234, 2001), (0, 7), (2147483647, 100), (2 ** 40 + 3, 1000),
                    (99, 65536), (99, 65537), (5, 70001), (7, 1), (3, 3)):
        assert np.array_equal(O.shuffled_order(seed, n), O.ref_shuffled_order(seed, n)), (seed, n)
    assert O.ref_shuffled_order(5, 6, False).tolist() == [0, 1, 2, 3, 4, 5]


def test_intermediate_storage_ticks_match_the_reference_progress_bar(ref_mod):
    from pink_amd import fileio
    for total, prints in ((100, 10), (3, 2), (1, 10), (7, 3), (8, 3), (24, 10), (2000, 10), (2001, 7), (69, 70), (500, 70)):
        assert fileio.progress_ticks(total, prints) == ref_mod.ref_progress_ticks(total, prints), (total, prints)

