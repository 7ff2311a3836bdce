"""The CPU oracle against the reference's own test vectors and closed forms.

Each case cites the reference test it restates (paths relative to the reference
tree).  These pin the oracle without running any reference code.
"""
import math

import numpy as np
import pytest

import oracle as O


def test_rotated_images_2d_golden():
    # test/SelfOrganizingMapTest/generate_rotated_images.cpp:15-27
    img = np.array([1, 2, 3, 4], np.float32)
    out = O.rotated_images(img, 1, 2, 2, 4, False)
    assert out.ravel().tolist() == [1, 2, 3, 4, 3, 1, 4, 2, 4, 3, 2, 1, 2, 4, 1, 3]


def test_rotated_images_3d_golden():
    # test/SelfOrganizingMapTest/generate_rotated_images.cpp:29-41
    img = np.arange(1, 9, dtype=np.float32)
    out = O.rotated_images(img, 2, 2, 2, 4, False)
    assert out.ravel().tolist() == [1, 2, 3, 4, 5, 6, 7, 8, 3, 1, 4, 2, 7, 5, 8, 6,
                                    4, 3, 2, 1, 8, 7, 6, 5, 2, 4, 1, 3, 6, 8, 5, 7]


def test_rot90_list_golden():
    # test/CudaTest/rotate_90_degrees_list.cu:16-29 : {1,2,3,4} -> {3,1,4,2}
    out = O.rotated_images(np.array([1, 2, 3, 4], np.float32), 1, 2, 2, 4, False)
    assert out[1].ravel().tolist() == [3, 1, 4, 2]


def test_resize_golden():
    # test/CudaTest/resize.cu:16-37 (crop 4x4 -> 2x2 = {5,6,9,10}); ImageProcessingTest/resize.cpp
    img = np.arange(16, dtype=np.float32)
    out = O.rotated_images(img, 1, 4, 2, 1, False)
    assert out.ravel().tolist() == [5, 6, 9, 10]
    # enlarge 2x2 -> 4x4: centred, zero border
    out = O.rotated_images(np.array([1, 2, 3, 4], np.float32), 1, 2, 4, 1, False)
    assert out.ravel().tolist() == [0, 0, 0, 0, 0, 1, 2, 0, 0, 3, 4, 0, 0, 0, 0, 0]


def test_rotate_bilinear_45deg_of_ones():
    # test/ImageProcessingTest/rotate.cpp:24-62 : 45 degrees of all-ones keeps
    # only pixels whose source position stays inside the image.
    one = O.rotate_bilinear(np.ones((1, 1), np.float32), 1, math.pi / 4)
    assert one.tolist() == [[1.0]]
    two = O.rotate_bilinear(np.ones((2, 2), np.float32), 2, math.pi / 4)
    # each corner maps 0.707 away from the centre along an axis: outside [0,1] on one side
    assert float(two.sum()) == 0.0 or np.all((two == 0) | (np.abs(two - 1) < 1e-6))


def test_rotate_zero_is_centre_crop():
    rng = np.random.default_rng(0)
    img = rng.random((9, 9), dtype=np.float32)
    out = O.rotate_bilinear(img, 5, 0.0)
    assert np.array_equal(out, img[2:7, 2:7])


@pytest.mark.parametrize("a,b,chan,dim,ed,expect", [
    # test/SelfOrganizingMapTest/euclidean_distance.cpp:16-69
    ([0, 0, 0, 0], [1, 0, 0, 0], 1, 2, 2, 1),
    ([0] * 9, [0, 0, 1, 0, 0, 1, 1, 1, 1], 1, 3, 2, 0),
    ([0] * 16, [1, 1, 1, 1, 1, 0, 0, 1, 1, 0, 0, 1, 1, 1, 1, 1], 1, 4, 2, 0),
    ([0] * 8, [1, 1, 1, 1, 1, 0, 0, 1], 2, 2, 2, 6),
    ([0] * 32, [0, 0, 0, 0, 0, 1, 1, 0, 0, 1, 1, 0, 0, 0, 0, 0] * 2, 2, 4, 2, 8),
])
def test_ssd_known_answers(a, b, chan, dim, ed, expect):
    assert O.ssd_int(a, b, chan, dim, ed, O.QUADRATIC) == expect
    assert O.ssd_f32(a, b, chan, dim, ed, O.QUADRATIC) == float(expect)


def test_circular_count_31428():
    # test/SelfOrganizingMapTest/euclidean_distance.cpp:71-89
    dim, ed = 300, 200
    a = np.zeros((dim, dim), np.int32)
    b = np.zeros((dim, dim), np.int32)
    b[50:50 + ed, 50:50 + ed] = 1
    assert O.ssd_int(a, b, 1, dim, ed, O.CIRCULAR) == 31428
    assert len(O.region(1, dim, ed, O.CIRCULAR)) == 31428


def test_circular_odd_diameter_last_row_empty():
    # circular_euclidean_distance.h:51-57 : row e-1 of an odd diameter has a
    # negative radicand -> NaN -> no columns.
    off = O.region(1, 106, 75, O.CIRCULAR)
    rows = np.unique(off // 106)
    assert rows.min() == 15 and rows.max() == 88     # row 89 (i = 74) is empty
    assert len(off) == 4304
    # brute force of the same rule in float64
    n = 0
    for i in range(75):
        rad = 2 * 37 * (i + 0.5) - (i + 0.5) ** 2
        if rad < 0:
            continue
        d = math.sqrt(rad)
        lo, hi = math.floor(53 - d + 0.5), math.floor(53 + d + 0.5)
        n += hi - lo
    assert n == 4304


def test_mapper_known_answers():
    # test/SelfOrganizingMapTest/Mapper.cpp:80-100 (+ test/CudaTest/mapper.cu:115-119 for u8/u16)
    cases = [(1, 2, 2, 2, 1, False, 0.0, 1.0, 2.0), (1, 3, 3, 2, 1, False, 0.0, 1.0, 2.0),
             (1, 3, 5, 2, 360, False, 0.0, 1.0, 2.0), (2, 3, 5, 2, 360, False, 0.0, 1.0, 2.0),
             (2, 3, 5, 2, 360, True, 0.0, 1.0, 2.0), (1, 2, 2, 2, 1, False, 1.0, 0.0, 2.0),
             (2, 3, 5, 2, 360, True, 1.0, 0.0, 2.0), (1, 2, 2, 2, 1, False, 0.0, 0.5, 1.0),
             (1, 2, 2, 2, 1, False, 0.5, 0.0, 1.0), (1, 2, 2, 2, 1, False, 0.5, 0.5, 0.0),
             (2, 2, 2, 2, 1, False, 0.0, 0.5, 1.0), (1, 3, 3, 2, 360, False, 1.0, 0.0, 2.0)]
    for som_dim, nd, idim, ed, nrot, flip, nv, iv, expect in cases:
        N = som_dim * som_dim
        for ed_type in (O.FLOAT, O.UINT8, O.UINT16):
            if ed_type != O.FLOAT and (iv != 0.0 or nv != 1.0):
                continue   # mapper.cu:55-120 runs the integer modes on a zero image only
            s = O.shape(N, 1, idim, nd, nrot, flip, ed, O.QUADRATIC, ed_type)
            heat, _ = O.map_images(s, np.full((N, nd, nd), nv, np.float32), np.full((idim, idim), iv, np.float32))
            assert heat.ravel().tolist() == [expect] * N, (som_dim, nd, idim, ed, nrot, flip, ed_type)


def test_circular_mapper_known_answer():
    # test/SelfOrganizingMapTest/circular_ed.cpp:23-53
    image = np.zeros(16, np.float32)
    image[4] = 1.0
    som = np.zeros(64, np.float32)
    som[4], som[18], som[43], som[61] = 1.0, 0.5, 0.8, 0.3
    s = O.shape(4, 1, 4, 4, 4, False, 4, O.CIRCULAR, O.FLOAT)
    heat, best = O.map_images(s, som, image)
    assert np.allclose(heat.ravel(), [0.0, 0.5, 0.2, 0.7], atol=0.01)
    assert best.ravel().tolist() == [0, 1, 2, 3]


def test_trainer_known_answers():
    # test/SelfOrganizingMapTest/Trainer.cpp:49-69 : one image {1000..4000}, zero SOM 2x2 of 2x2,
    # Gaussian(1.1, 0.2), num_rot 1 -> neuron(0,0)[1,1] = int(290.1) = 290
    F = O.update_factors(O.CARTESIAN, [2, 2], O.GAUSSIAN, 1.1, 0.2, 0.0)
    som = np.zeros((4, 4), np.float32)
    s = O.shape(4, 1, 2, 2, 1, False, 2)
    O.train_step(s, som, np.array([1000, 2000, 3000, 4000], np.float32), F)
    assert int(som[0, 3]) == 290
    # :71-94 : StepFunctor(10) pulls the single neuron fully onto the centre crop {6,7,10,11}
    F = O.update_factors(O.CARTESIAN, [1, 1], O.STEP, 10.0, 0.0, 0.0)
    som = np.zeros((1, 4), np.float32)
    s = O.shape(1, 1, 4, 2, 1, False, 2)
    O.train_step(s, som, np.arange(1, 17, dtype=np.float32), F)
    assert som.ravel().tolist() == [6, 7, 10, 11]
    # :96-124 : 3-D, neuron 1 equals the 180-degree variant -> BMU 1, unchanged, best rotation 2
    F = O.update_factors(O.CARTESIAN, [2, 2], O.STEP, 0.0, 0.0, 0.0)
    som = np.zeros((4, 8), np.float32)
    som[1] = [4, 3, 2, 1, 8, 7, 6, 5]
    s = O.shape(4, 2, 2, 2, 4, False, 2)
    bmu, d, best = O.train_step(s, som, np.arange(1, 9, dtype=np.float32), F)
    assert bmu == 1 and best[1] == 2 and d[1] == 0.0
    assert som[1].tolist() == [4, 3, 2, 1, 8, 7, 6, 5]
    # :126-151 : 3-D 2x4x4, zero SOM, Step(0): BMU is neuron 0, neuron 1 stays zero
    som = np.zeros((4, 32), np.float32)
    s = O.shape(4, 2, 4, 4, 4, False, 4)
    bmu, _, _ = O.train_step(s, som, np.arange(1, 33, dtype=np.float32), F)
    assert bmu == 0 and not som[1].any() and som[0].any()


def test_update_kernel_known_answer():
    # test/CudaTest/update_neurons.cu:16-41
    som = np.zeros((4, 4), np.float32)
    rot = np.arange(1, 9, dtype=np.float32)
    d = np.array([2, 1, 3, 4], np.float32)
    s = O.shape(4, 1, 2, 2, 1, False, 2)
    b = O.bmu(s, d)
    assert b == 1
    O.update(som, rot, np.array([0, 1, 0, 0], np.uint32), b, np.eye(4, dtype=np.float32))
    assert som.ravel().tolist() == [0, 0, 0, 0, 5, 6, 7, 8, 0, 0, 0, 0, 0, 0, 0, 0]


def test_functor_closed_forms():
    # test/UtilitiesTest/DistributionFunctorTest.cpp:28-79
    L = O.lib()
    for sigma, damping in [(1.0, 1.0), (1.1, 0.2), (2.0, 0.05), (1.5, 0.1)]:
        for x in (0.0, 0.5, 1.0, 2.0, 3.7):
            g = damping / (sigma * math.sqrt(2 * math.pi)) * math.exp(-0.5 * (x / sigma) ** 2)
            assert abs(L.pink_oracle_functor(O.GAUSSIAN, sigma, damping, x) - g) < 1e-6
            u = damping * math.exp(-0.5 * (x / sigma) ** 2)
            assert abs(L.pink_oracle_functor(O.UNITY_GAUSSIAN, sigma, damping, x) - u) < 1e-6
            m = (2 * damping / (math.sqrt(3 * sigma) * math.pi ** 0.25) * (1 - x * x / sigma ** 2)
                 * math.exp(-x * x / (2 * sigma ** 2)))
            assert abs(L.pink_oracle_functor(O.MEXICAN_HAT, sigma, damping, x) - m) < 1e-6
    assert L.pink_oracle_functor(O.STEP, 1.0, 0.0, 1.0) == 1.0
    assert L.pink_oracle_functor(O.STEP, 1.0, 0.0, 1.5) == 0.0


def test_hex_layout():
    # test/SelfOrganizingMapTest/Hexagonal.cpp:15-53 : dim 3 -> 7 cells; dim 21 -> 331
    L = O.lib()
    assert L.pink_oracle_hex_size(3) == 7 and L.pink_oracle_hex_size(21) == 331
    # dim 3 cells: (1,0)(2,0) / (0,1)(1,1)(2,1) / (0,2)(1,2); cube metric
    assert L.pink_oracle_hex_distance(3, 0, 0) == 0.0
    assert L.pink_oracle_hex_distance(3, 0, 1) == 1.0
    assert L.pink_oracle_hex_distance(3, 0, 6) == 2.0
    assert L.pink_oracle_hex_distance(3, 3, 5) == 1.0 or L.pink_oracle_hex_distance(3, 3, 4) == 1.0
    assert all(L.pink_oracle_hex_distance(3, 3, j) == 1.0 for j in (0, 1, 2, 4, 5, 6))


def test_mt19937_and_filler():
    # C++ standard [rand.predef]: the 10000th output of default-seeded mt19937 is 4123659995
    raw = O.mt19937_raw(5489, 10000)
    assert int(raw[-1]) == 4123659995
    # numpy's legacy seeding is the same init_genrand
    rs = np.random.RandomState(1234)
    assert np.array_equal(O.mt19937_raw(1234, 64), rs._bit_generator.random_raw(64).astype(np.uint32))
    # Filler.h with seed 1234 (libstdc++: one word per float)
    f = O.fill_random_uniform(4, 1234)
    assert np.allclose(f, [0.191519, 0.497664, 0.622109, 0.817838], atol=1e-6)
    assert f.max() < 1.0 and f.min() >= 0.0


def test_quantise_contract():
    # tools 255^2 = 65025 (test/UtilitiesTest/ipowTest.cpp:13-23)
    assert O.lib().pink_oracle_quant_factor(O.UINT8) ** 2 == 65025
    assert O.quantise([0.0, 1.0, 0.5, 0.999, -0.2, 1.7], O.UINT8).tolist() == [0, 255, 127, 254, 0, 255]
    assert O.quantise([0.0, 1.0, 0.5, -1.0, 2.0], O.UINT16).tolist() == [0, 65535, 32767, 0, 65535]


def test_integer_distance_brute_force():
    rng = np.random.default_rng(7)
    N, C, I, D, e = 5, 1, 12, 9, 6
    for ed_type, factor in ((O.UINT8, 255), (O.UINT16, 65535)):
        for shape_ in (O.QUADRATIC, O.CIRCULAR):
            s = O.shape(N, C, I, D, 8, True, e, shape_, ed_type)
            som = rng.random((N, C * D * D), dtype=np.float32)
            img = rng.random(C * I * I, dtype=np.float32)
            rot = O.rotated_images(img, C, I, D, 8, True).reshape(16, -1)
            d, ssd, best = O.distance_matrix(s, som, rot)
            off = O.region(C, D, e, shape_)
            qs = np.trunc(som.astype(np.float32) * np.float32(factor)).astype(np.int64)[:, off]
            qr = np.trunc(rot * np.float32(factor)).astype(np.int64)[:, off]
            full = ((qs[:, None, :] - qr[None, :, :]) ** 2).sum(-1)
            assert np.array_equal(ssd, full.min(1))
            assert np.array_equal(best, full.argmin(1))
            assert np.array_equal(d, (full.min(1) / float(factor * factor)).astype(np.float32))


def test_float_distance_close_to_float64():
    rng = np.random.default_rng(3)
    N, C, I, D, e = 6, 2, 16, 11, 8
    s = O.shape(N, C, I, D, 12, True, e)
    som = rng.random((N, C * D * D), dtype=np.float32)
    rot = O.rotated_images(rng.random(C * I * I, dtype=np.float32), C, I, D, 12, True).reshape(24, -1)
    d, _, best = O.distance_matrix(s, som, rot)
    off = O.region(C, D, e, O.QUADRATIC)
    full = ((som[:, None, off].astype(np.float64) - rot[None, :, off]) ** 2).sum(-1)
    assert np.allclose(d, full.min(1), rtol=1e-5)
    assert np.array_equal(best, full.argmin(1))


def test_variant_invariants():
    rng = np.random.default_rng(11)
    C, I, D, nrot = 2, 20, 14, 16
    img = rng.random((C, I, I), dtype=np.float32)
    out = O.rotated_images(img, C, I, D, nrot, True)
    nrr = nrot // 4
    for k in range(nrot - nrr):
        # variant k + nrr is the clockwise quarter turn of variant k
        assert np.array_equal(out[k + nrr], np.rot90(out[k], k=-1, axes=(1, 2)))
    for k in range(nrot):
        assert np.array_equal(out[k + nrot], out[k][:, ::-1, :])


@pytest.mark.parametrize("ed_type", [O.FLOAT, O.UINT8, O.UINT16])
@pytest.mark.parametrize("N,C,I,D,e,shape_,nrot,flip", [
    (7, 1, 20, 14, 9, O.QUADRATIC, 12, True),       # 24 variants: one full block of 16 and half a block
    (5, 3, 12, 9, 6, O.QUADRATIC, 36, True),        # 72 variants: an odd number of blocks
    (9, 1, 24, 17, 11, O.CIRCULAR, 8, False),       # 8 variants: less than one block; odd diameter
    (4, 1, 10, 10, 10, O.QUADRATIC, 4, True),       # permutations only
    (3, 2, 16, 12, 8, O.CIRCULAR, 20, True),        # 3-D circular: channel 0 counted twice
])
def test_distance_matrix_forms_agree_bit_for_bit(ed_type, N, C, I, D, e, shape_, nrot, flip):
    """The sixteen-variants-at-a-time evaluation against the definition: one functor call per pair."""
    rng = np.random.default_rng(1000 * ed_type + N)
    R = nrot * (2 if flip else 1)
    s = O.shape(N, C, I, D, nrot, flip, e, shape_, ed_type)
    for trial in range(3):
        som = rng.random((N, C * D * D), dtype=np.float32)
        img = rng.random(C * I * I, dtype=np.float32)
        if trial == 1:                                  # few levels: equal distances between variants
            som = np.round(som * 3) / np.float32(3)
            img = np.round(img * 2) / np.float32(2)
        if trial == 2:                                  # a neuron that is a variant: distance 0 late in the list
            som[N - 1] = O.rotated_images(img, C, I, D, nrot, flip).reshape(R, -1)[R - 1]
        rot = O.rotated_images(img, C, I, D, nrot, flip).reshape(R, -1)
        d0, ssd0, best0 = O.distance_matrix_pairwise(s, som, rot)
        d1, ssd1, best1 = O.distance_matrix(s, som, rot)
        assert np.array_equal(d0.view(np.uint32), d1.view(np.uint32))
        assert np.array_equal(ssd0, ssd1)
        assert np.array_equal(best0, best1)


def test_distance_matrix_reference_loop_one_thread():
    """The reference's own loop structure gives the one-thread answer when run on one thread (with more,
    equal distances go to whichever thread comes first, as in the reference)."""
    rng = np.random.default_rng(5)
    N, C, I, D, e, nrot = 6, 1, 20, 14, 9, 24
    s = O.shape(N, C, I, D, nrot, True, e)
    som = rng.random((N, C * D * D), dtype=np.float32)
    rot = O.rotated_images(rng.random(C * I * I, dtype=np.float32), C, I, D, nrot, True).reshape(2 * nrot, -1)
    d0, _, best0 = O.distance_matrix_pairwise(s, som, rot)
    before = O.num_threads()
    O.set_num_threads(1)
    try:
        d1, best1 = O.distance_matrix_reference_loop(s, som, rot)
    finally:
        O.set_num_threads(before)
    assert np.array_equal(d0.view(np.uint32), d1.view(np.uint32))
    assert np.array_equal(best0, best1)
    d2, best2 = O.distance_matrix_reference_loop(s, som, rot)     # all threads: same distances
    assert np.array_equal(d0.view(np.uint32), d2.view(np.uint32))
