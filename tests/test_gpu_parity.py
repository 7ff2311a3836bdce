"""GPU parity: the HIP path through the C ABI against the CPU oracle.

Bars (stated where checked): rotated pixels bit-exact; float32 distances bit-exact
with the oracle (stricter than the 1e-5 relative gate) and best rotation / BMU
identical; integer sums, best rotations and BMUs bit-exact; trained weights
bit-exact after several sequential images (gate: 1e-4 absolute).
"""
import sys

import numpy as np
import pytest

import oracle as O
from pink_amd import capi, synthetic

pytestmark = pytest.mark.gpu


def say(*a):
    print(*a, flush=True)
    sys.stdout.flush()


def bits(a):
    return np.ascontiguousarray(a, np.float32).view(np.uint32)


ROT_SHAPES = [
    # C, I, D, num_rot, flip
    (1, 64, 44, 360, True), (1, 150, 106, 360, True), (3, 100, 70, 180, True), (1, 28, 28, 4, True),
    (1, 64, 45, 360, True), (1, 64, 100, 360, True), (1, 124, 91, 360, True), (2, 17, 24, 16, False),
    (1, 2, 4, 1, False), (1, 4, 2, 8, True), (1, 5, 3, 360, False), (3, 9, 9, 1, True),
    (1, 200, 141, 8, True),     # a base rotation of 78 KiB in LDS
    (1, 290, 205, 8, True),     # 205*205*4 B > 158 KiB and so is the image: nothing in LDS
    (1, 150, 205, 16, True),    # the image in LDS instead of the base rotation
    (2, 160, 226, 8, False),
    (1, 210, 260, 8, True),     # nothing in LDS, neurons larger than the image
]


@pytest.mark.parametrize("C_,I,D,nrot,flip", ROT_SHAPES)
def test_rotate_bit_exact(C_, I, D, nrot, flip):
    say("rotate", C_, I, D, nrot, flip)
    rng = np.random.default_rng(I * 1000 + D + nrot)
    img = rng.random((C_, I, I), dtype=np.float32)
    with capi.Context(3, C_, I, D, nrot, flip, min(D, 2)) as ctx:
        got = ctx.rotate(img)
    want = O.rotated_images(img, C_, I, D, nrot, flip)
    assert np.array_equal(bits(got), bits(want))


@pytest.mark.parametrize("ed_type", [capi.UINT8, capi.UINT16])
def test_rotate_tap_on_integer_contexts_with_channels(ed_type):
    # integer contexts keep the base rotations of all channels in one block of the rotation kernel
    C_, I, D, nrot, flip = 3, 20, 14, 8, True
    say("rotate tap, integer, channels", ed_type)
    rng = np.random.default_rng(ed_type)
    img = rng.random((C_, I, I), dtype=np.float32)
    want = O.rotated_images(img, C_, I, D, nrot, flip)
    F = capi.make_update_factors(capi.CARTESIAN, [3], capi.GAUSSIAN, 1.0, 0.5)
    for factors in (None, F):
        with capi.Context(3, C_, I, D, nrot, flip, 9, capi.QUADRATIC, ed_type, factors) as ctx:
            assert np.array_equal(bits(ctx.rotate(img)), bits(want))


def test_rotate_reference_golden():
    # test/SelfOrganizingMapTest/generate_rotated_images.cpp:15-41
    with capi.Context(1, 1, 2, 2, 4, False, 2) as ctx:
        out = ctx.rotate(np.array([1, 2, 3, 4], np.float32))
    assert out.ravel().tolist() == [1, 2, 3, 4, 3, 1, 4, 2, 4, 3, 2, 1, 2, 4, 1, 3]
    with capi.Context(1, 2, 2, 2, 4, False, 2) as ctx:
        out = ctx.rotate(np.arange(1, 9, dtype=np.float32))
    assert out.ravel().tolist() == [1, 2, 3, 4, 5, 6, 7, 8, 3, 1, 4, 2, 7, 5, 8, 6,
                                    4, 3, 2, 1, 8, 7, 6, 5, 2, 4, 1, 3, 6, 8, 5, 7]


DIST_SHAPES = [
    # N, C, I, D, nrot, flip, ed, shape
    (100, 1, 64, 44, 360, True, 32, capi.QUADRATIC),      # cfg 0 / 1
    (64, 1, 28, 28, 4, True, 28, capi.QUADRATIC),         # cfg 4
    (37, 1, 40, 29, 16, True, 21, capi.CIRCULAR),
    (9, 2, 17, 24, 8, False, 13, capi.QUADRATIC),
    (9, 2, 17, 24, 8, True, 13, capi.CIRCULAR),           # 3-D circular: channel 0 counted twice (CPU rule)
    (4, 1, 8, 8, 1, False, 8, capi.QUADRATIC),
    (5, 1, 8, 8, 1, True, 5, capi.QUADRATIC),
    (331, 1, 150, 106, 360, True, 75, capi.CIRCULAR),     # cfg 2
    (1600, 3, 100, 70, 180, True, 50, capi.QUADRATIC),    # cfg 3
    (7, 1, 40, 28, 720, True, 20, capi.QUADRATIC),        # 1440 variants: six row tiles of base rotations
    (3, 1, 30, 20, 1024, False, 15, capi.CIRCULAR),       # eight
    (5, 1, 160, 226, 8, True, 113, capi.QUADRATIC),       # neurons too large for an LDS tile: the image in LDS
    (5, 1, 290, 205, 8, True, 40, capi.CIRCULAR),         # ... nothing in LDS
    (4, 1, 210, 297, 12, True, 148, capi.QUADRATIC),      # ... and neurons larger than the image
    (5, 1, 128, 181, 16, True, 90, capi.QUADRATIC),       # a 128 KiB base rotation in LDS
]


def _som_and_image(N, C_, I, D, seed):
    rng = np.random.default_rng(seed)
    som = rng.random((N, C_ * D * D), dtype=np.float32)
    img = rng.random((C_, I, I), dtype=np.float32)
    return som, img


@pytest.mark.parametrize("ed_type", [capi.FLOAT, capi.UINT8, capi.UINT16])
@pytest.mark.parametrize("N,C_,I,D,nrot,flip,ed,shape_", DIST_SHAPES)
def test_distance_parity(N, C_, I, D, nrot, flip, ed, shape_, ed_type):
    say("distance", N, C_, I, D, nrot, flip, ed, shape_, ed_type)
    som, img = _som_and_image(N, C_, I, D, N + D + ed)
    if N < 331:
        som[1] = O.rotated_images(img, C_, I, D, nrot, flip)[min(3, nrot - 1)].ravel()   # an exact match
        som[2] = som[1] * np.float32(0.5)
    s = O.shape(N, C_, I, D, nrot, flip, ed, shape_, ed_type)
    rot = O.rotated_images(img, C_, I, D, nrot, flip)
    od, ossd, obest = O.distance_matrix(s, som, rot)
    # a uint8 mapper runs on the matrix cores where a kernel applies: check every kernel
    choices = [capi.KERNEL_AUTO]
    if ed_type == capi.UINT8:
        choices += [capi.KERNEL_VALU, capi.KERNEL_MFMA, capi.KERNEL_MFMA_SYM, capi.KERNEL_MFMA_GEMM]
    if ed_type == capi.UINT16:
        choices += [capi.KERNEL_VALU, capi.KERNEL_MFMA_GEMM]
    ran = 0
    for choice in choices:
        try:
            ctx = capi.Context(N, C_, I, D, nrot, flip, ed, shape_, ed_type, kernel_choice=choice)
        except capi.PinkError:
            assert choice in (capi.KERNEL_MFMA, capi.KERNEL_MFMA_SYM)    # refused: shape outside that kernel
            continue
        ran += 1
        with ctx:
            ctx.set_som(som)
            assert ctx.region_size == len(O.region(C_, D, ed, shape_))
            d, ssd, best = ctx.distance(img)
        if ed_type == capi.FLOAT:
            # gate: 1e-5 relative, argmin identical up to ties; achieved and asserted: bit-exact
            assert np.array_equal(bits(d), bits(od))
        else:
            assert np.array_equal(ssd, ossd), choice
            assert np.array_equal(bits(d), bits(od)), choice
        assert np.array_equal(best, obest), choice


# The float32 distance kernel has two forms chosen by the amount of work per launch: neuron values by DPP
# broadcast (blocks of one neuron per wave, while they are all resident at once) and neuron values as scalar
# operands with two or four neurons per wave.  Same chains, same order: every form is bit-equal to the oracle.
@pytest.mark.parametrize("N,C_,I,D,nrot,flip,ed,shape_,n_map", [
    (397, 1, 64, 44, 360, True, 32, capi.QUADRATIC, 0),      # one image: scalar operands, two neurons per wave
    (1597, 1, 64, 44, 360, True, 32, capi.QUADRATIC, 0),     # one image: four neurons per wave
    (70, 1, 20, 14, 32, True, 9, capi.CIRCULAR, 300),        # a launch group of small images: four neurons per wave, two stages
    (37, 1, 40, 29, 16, True, 21, capi.CIRCULAR, 150),       # ... two neurons per wave, neuron count not a multiple of 8
])
def test_float32_distance_forms(N, C_, I, D, nrot, flip, ed, shape_, n_map):
    say("float32 distance forms", N, C_, I, D, nrot, flip, ed, shape_, n_map)
    rng = np.random.default_rng(N * 31 + n_map)
    som = rng.random((N, C_ * D * D), dtype=np.float32)
    s = O.shape(N, C_, I, D, nrot, flip, ed, shape_, capi.FLOAT)
    with capi.Context(N, C_, I, D, nrot, flip, ed, shape_, capi.FLOAT) as ctx:
        ctx.set_som(som)
        if n_map == 0:
            img = rng.random((C_, I, I), dtype=np.float32)
            som[N // 2] = O.rotated_images(img, C_, I, D, nrot, flip)[min(5, nrot - 1)].ravel()   # an exact match
            ctx.set_som(som)
            od, _, obest = O.distance_matrix(s, som, O.rotated_images(img, C_, I, D, nrot, flip))
            d, _, best = ctx.distance(img)
            assert np.array_equal(bits(d), bits(od))
            assert np.array_equal(best, obest)
        else:
            imgs = rng.random((n_map, C_, I, I), dtype=np.float32)
            heat, best = ctx.map(imgs)
            oheat, obest = O.map_images(s, som, imgs)
            assert np.array_equal(bits(heat), bits(oheat))
            assert np.array_equal(best, obest)


TRAIN_CASES = [
    # workload, images, ed_type override, distance kernel
    ("cfg0", 6, None, capi.KERNEL_AUTO), ("cfg4", 40, None, capi.KERNEL_AUTO), ("cfg4", 10, None, capi.KERNEL_VALU),
    ("cfg0", 4, capi.UINT8, capi.KERNEL_AUTO), ("cfg0", 3, capi.UINT8, capi.KERNEL_VALU),
    ("cfg0", 3, capi.UINT16, capi.KERNEL_AUTO), ("cfg2", 3, None, capi.KERNEL_AUTO), ("cfg2", 1, None, capi.KERNEL_VALU),
    ("cfg3", 1, None, capi.KERNEL_AUTO),
]


@pytest.mark.parametrize("name,n,ed_type,choice", TRAIN_CASES)
def test_train_parity(name, n, ed_type, choice):
    w = synthetic.WORKLOADS[name]
    ed_type = w.ed_type if ed_type is None else ed_type
    say("train", name, n, ed_type, choice)
    imgs = synthetic.images(w, n)
    som0 = synthetic.initial_som(w)
    F = synthetic.update_factors(w)
    with capi.Context(w.som_size, w.channels, w.image_dim, w.neuron_dim, w.num_rot, w.use_flip, w.ed_dim,
                      w.ed_shape, ed_type, F, kernel_choice=choice) as ctx:
        ctx.set_som(som0)
        bmu = ctx.train(imgs)
        got = ctx.get_som()
    s = O.shape(w.som_size, w.channels, w.image_dim, w.neuron_dim, w.num_rot, w.use_flip, w.ed_dim,
                w.ed_shape, ed_type)
    want = som0.copy()
    obmu = O.train(s, want, imgs, F)
    assert np.array_equal(bmu, obmu)
    # gate: 1e-4 absolute (test/CudaTest/compare_trainer_cpu.cu:76); asserted: bit-exact
    assert np.abs(got - want).max() <= 1e-4
    assert np.array_equal(bits(got), bits(want))


def test_train_one_call_per_image_equals_batched_call():
    w = synthetic.WORKLOADS["cfg4"]
    imgs = synthetic.images(w, 12)
    som0 = synthetic.initial_som(w)
    with synthetic.make_context(w) as a, synthetic.make_context(w) as b:
        a.set_som(som0)
        b.set_som(som0)
        bm_a = a.train(imgs)
        bm_b = np.concatenate([b.train(imgs[i]) for i in range(len(imgs))])
        assert np.array_equal(bm_a, bm_b)
        assert np.array_equal(bits(a.get_som()), bits(b.get_som()))


@pytest.mark.parametrize("name,n", [("cfg0", 150), ("cfg4", 200)])
def test_calls_without_a_result_train_in_order_whatever_comes_between(name, n):
    """Calls that hand nothing back (the reference's Trainer::operator()) are collected into launch groups;
    every other call on the context first trains what is pending.  Weights, best matches and counts are those of
    one call over all images, and of the CPU."""
    w = synthetic.WORKLOADS[name]
    imgs = synthetic.images(w, n)
    som0 = synthetic.initial_som(w)
    F = synthetic.update_factors(w)
    s = O.shape(w.som_size, w.channels, w.image_dim, w.neuron_dim, w.num_rot, w.use_flip, w.ed_dim, w.ed_shape, w.ed_type)
    with synthetic.make_context(w) as ctx:
        ctx.set_som(som0)
        bmu_mid = None
        for i in range(n):
            if i == 70:
                d_mid = ctx.distance(imgs[0])[0]          # sees the SOM after 70 images
            if i == 100:
                bmu_mid = ctx.train(imgs[100:103])         # a call with a result, in the middle of pending ones
                continue
            if i in (101, 102):
                continue
            if i == 120:
                ctx.rotate(imgs[5])                        # the debug tap shares buffers with the trainer
            ctx.train(imgs[i], want_bmu=False)             # three of them in one call further down
        counts = ctx.update_counts()
        got = ctx.get_som()
    want = som0.copy()
    obmu = O.train(s, want, imgs, F)
    assert np.array_equal(bits(got), bits(want))
    assert np.array_equal(bmu_mid, obmu[100:103])
    assert np.array_equal(counts, np.bincount(obmu, minlength=w.som_size))
    mid = som0.copy()
    O.train(s, mid, imgs[:70], F)
    od = O.distance_matrix(s, mid, O.rotated_images(imgs[0], w.channels, w.image_dim, w.neuron_dim, w.num_rot, w.use_flip))[0]
    assert np.array_equal(bits(d_mid), bits(od))


@pytest.mark.parametrize("name", ["cfg4", "cfg0"])
def test_rotation_tap_between_training_calls(name):
    # a trainer keeps two of a base rotation's eight symmetries; the tap asks for all of them in between
    w = synthetic.WORKLOADS[name]
    say("tap between training calls", name)
    imgs = synthetic.images(w, 6)
    som0 = synthetic.initial_som(w)
    with synthetic.make_context(w) as a, synthetic.make_context(w) as b:
        a.set_som(som0)
        b.set_som(som0)
        bm_a = a.train(imgs)
        first = b.train(imgs[:3])
        variants = b.rotate(imgs[5])
        second = b.train(imgs[3:])
        want = O.rotated_images(imgs[5], w.channels, w.image_dim, w.neuron_dim, w.num_rot, w.use_flip)
        assert np.array_equal(bits(variants), bits(want))
        assert np.array_equal(bm_a, np.concatenate([first, second]))
        assert np.array_equal(bits(a.get_som()), bits(b.get_som()))


def test_reference_trainer_known_answers():
    # test/SelfOrganizingMapTest/Trainer.cpp:49-94 and test/CudaTest/update_neurons.cu:16-41
    F = capi.make_update_factors(capi.CARTESIAN, [2, 2], capi.GAUSSIAN, 1.1, 0.2, 0.0)
    with capi.Context(4, 1, 2, 2, 1, False, 2, update_factors=F) as ctx:
        ctx.set_som(np.zeros((4, 4), np.float32))
        ctx.train(np.array([1000, 2000, 3000, 4000], np.float32))
        assert int(ctx.get_som()[0, 3]) == 290
    F = capi.make_update_factors(capi.CARTESIAN, [1, 1], capi.STEP, 10.0)
    with capi.Context(1, 1, 4, 2, 1, False, 2, update_factors=F) as ctx:
        ctx.set_som(np.zeros((1, 4), np.float32))
        ctx.train(np.arange(1, 17, dtype=np.float32))
        assert ctx.get_som().ravel().tolist() == [6, 7, 10, 11]
    F = capi.make_update_factors(capi.CARTESIAN, [2, 2], capi.STEP, 0.0)
    with capi.Context(4, 2, 2, 2, 4, False, 2, update_factors=F) as ctx:
        som = np.zeros((4, 8), np.float32)
        som[1] = [4, 3, 2, 1, 8, 7, 6, 5]
        ctx.set_som(som)
        bmu = ctx.train(np.arange(1, 9, dtype=np.float32))
        assert bmu.tolist() == [1] and np.array_equal(ctx.get_som(), som)


MAP_CASES = [("cfg1", 24, None, capi.KERNEL_AUTO), ("cfg1", 9, None, capi.KERNEL_VALU),
             ("cfg1", 13, None, capi.KERNEL_MFMA), ("cfg1", 40, None, capi.KERNEL_MFMA_SYM),
             ("cfg0", 5, capi.FLOAT, capi.KERNEL_AUTO),
             ("cfg4", 300, None, capi.KERNEL_AUTO), ("cfg4", 50, None, capi.KERNEL_VALU),
             ("cfg2", 2, None, capi.KERNEL_AUTO)]


@pytest.mark.parametrize("name,n,ed_type,choice", MAP_CASES)
def test_map_parity(name, n, ed_type, choice):
    w = synthetic.WORKLOADS[name]
    ed_type = w.ed_type if ed_type is None else ed_type
    say("map", name, n, ed_type, choice)
    imgs = synthetic.images(w, n)
    som = synthetic.initial_som(w)
    som[3] = O.rotated_images(imgs[1], w.channels, w.image_dim, w.neuron_dim, w.num_rot, w.use_flip)[5 % w.R].ravel()
    with capi.Context(w.som_size, w.channels, w.image_dim, w.neuron_dim, w.num_rot, w.use_flip, w.ed_dim,
                      w.ed_shape, ed_type, None, max_batch=7, kernel_choice=choice) as ctx:
        ctx.set_som(som)
        heat, best = ctx.map(imgs)
    s = O.shape(w.som_size, w.channels, w.image_dim, w.neuron_dim, w.num_rot, w.use_flip, w.ed_dim,
                w.ed_shape, ed_type)
    oheat, obest = O.map_images(s, som, imgs)
    assert np.array_equal(bits(heat), bits(oheat))
    assert np.array_equal(best, obest)


SYM_SHAPES = [
    # N, C, I, D, nrot, flip, ed, shape, images   -- each exercises another corner of the resident-SOM kernels
    (3, 1, 24, 18, 40, True, 16, capi.QUADRATIC, 5),       # 8 k-steps, one unit per image, one column tile, batch not a multiple of 4
    (70, 1, 32, 24, 160, True, 22, capi.QUADRATIC, 9),     # 16 k-steps, two units per image, three SOM slices
    (150, 1, 45, 32, 360, True, 27, capi.QUADRATIC, 3),    # 24 k-steps, three units, five slices, image edge not a multiple of 4
    (33, 1, 40, 44, 360, False, 32, capi.QUADRATIC, 37),   # 32 k-steps, padded neurons (I < D), no flip, more images than one group
    (20, 2, 20, 16, 8, True, 10, capi.QUADRATIC, 6),       # two channels, two base rotations
    (12, 1, 16, 12, 4, True, 12, capi.QUADRATIC, 4),       # quarter turns only
    (12, 1, 16, 12, 1, True, 12, capi.QUADRATIC, 4),       # flip only
    (25, 1, 40, 29, 16, True, 21, capi.CIRCULAR, 7),       # circular region, odd diameter
    (1, 1, 28, 28, 360, True, 28, capi.QUADRATIC, 1),      # a single neuron, a single image
    (3, 2, 6, 7, 360, True, 1, capi.QUADRATIC, 3),         # a one-pixel region: equal distances all over, the first variant wins
    (37, 1, 64, 91, 360, True, 45, capi.QUADRATIC, 9),     # 2025 elements: the wide form (64 k-steps, one column tile per wave)
    (130, 1, 64, 64, 360, True, 44, capi.CIRCULAR, 2),     # wide form, 48 k-steps, nine slices
    (9, 1, 52, 42, 360, True, 38, capi.QUADRATIC, 40),     # wide form, several images per group
    (20, 2, 40, 30, 360, False, 30, capi.QUADRATIC, 4),    # wide form, two channels, no flip
    (40, 1, 24, 18, 40, True, 16, capi.QUADRATIC, 600),    # ten column tiles: a whole block and two tiles for the kernel that splits k, more images than its blocks
    (100, 1, 45, 32, 72, True, 27, capi.QUADRATIC, 5),     # 25 column tiles at 24 k-steps: three blocks and one tile
]


@pytest.mark.parametrize("N,C_,I,D,nrot,flip,ed,shape_,n", SYM_SHAPES)
def test_map_uint8_kernels_over_shapes(N, C_, I, D, nrot, flip, ed, shape_, n):
    say("map u8 shapes", N, C_, I, D, nrot, flip, ed, shape_, n)
    rng = np.random.default_rng(N * 7 + I + nrot)
    som = rng.random((N, C_ * D * D), dtype=np.float32)
    imgs = rng.random((n, C_, I, I), dtype=np.float32)
    R = nrot * (2 if flip else 1)
    som[N // 2] = O.rotated_images(imgs[0], C_, I, D, nrot, flip)[R - 1].ravel()       # an exact match at the last variant
    s = O.shape(N, C_, I, D, nrot, flip, ed, shape_, capi.UINT8)
    oheat, obest = O.map_images(s, som, imgs)
    ran = []
    for choice in (capi.KERNEL_AUTO, capi.KERNEL_MFMA_SYM, capi.KERNEL_MFMA, capi.KERNEL_MFMA_GEMM):
        try:
            ctx = capi.Context(N, C_, I, D, nrot, flip, ed, shape_, capi.UINT8, None, max_batch=16, kernel_choice=choice)
        except capi.PinkError:
            assert choice in (capi.KERNEL_MFMA, capi.KERNEL_MFMA_SYM)
            continue
        with ctx:
            ran.append(ctx.distance_kernel)
            ctx.set_som(som)
            heat, best = ctx.map(imgs)
            heat_again, best_again = ctx.map(imgs[:1])        # a second, shorter call on the same context
        assert np.array_equal(bits(heat), bits(oheat)), choice
        assert np.array_equal(best, obest), choice
        assert np.array_equal(bits(heat_again), bits(oheat[:1])) and np.array_equal(best_again, obest[:1]), choice
    say("   kernels that ran:", ran)
    assert capi.KERNEL_MFMA_GEMM in ran and capi.KERNEL_MFMA_SYM in ran


@pytest.mark.parametrize("ed_type", [capi.FLOAT, capi.UINT8, capi.UINT16])
def test_equal_distances_go_to_the_first_variant(ed_type):
    """A constant image has 720 identical quantised variants: every kernel must report variant 0 for every neuron
    (strict `<` over ascending variants, generate_euclidean_distance_matrix.h:43-50), also where the
    equal distances sit in different tiles of rotations."""
    N, C_, I, D, nrot, flip, ed = 9, 1, 32, 22, 360, True, 16
    rng = np.random.default_rng(17)
    som = rng.random((N, D * D), dtype=np.float32)
    imgs = np.full((2, C_, I, I), 0.5, np.float32)
    imgs[1, 0, 8:24, 8:24] = 0.25                     # constant inside every rotated region, not outside
    s = O.shape(N, C_, I, D, nrot, flip, ed, O.QUADRATIC, ed_type)
    oheat, obest = O.map_images(s, som, imgs)
    if ed_type != capi.FLOAT:                          # (in float32 the interpolation weights do not sum to exactly 1)
        assert (obest[0] == 0).all()
    choices = [capi.KERNEL_AUTO] if ed_type == capi.FLOAT else [capi.KERNEL_AUTO, capi.KERNEL_VALU, capi.KERNEL_MFMA_GEMM]
    if ed_type == capi.UINT8:
        choices += [capi.KERNEL_MFMA, capi.KERNEL_MFMA_SYM]
    for choice in choices:
        say("ties", ed_type, choice)
        with capi.Context(N, C_, I, D, nrot, flip, ed, capi.QUADRATIC, ed_type, kernel_choice=choice) as ctx:
            ctx.set_som(som)
            heat, best = ctx.map(imgs)
        assert np.array_equal(best, obest), choice
        assert np.array_equal(bits(heat), bits(oheat)), choice


@pytest.mark.parametrize("ed", [32, 45])
def test_largest_distances_do_not_lose_to_padding(ed):
    """Neurons of zeros against images of ones (and the reverse) give the largest distances a region
    allows: they must still beat the padded rows and columns of every integer kernel (ed = 45, 2025
    elements, takes the wide form of the symmetric kernel)."""
    N, C_, I, D, nrot, flip = 6, 1, 64, (44 if ed == 32 else 91), 360, True
    rng = np.random.default_rng(ed)
    som = rng.random((N, D * D), dtype=np.float32)
    som[0] = 0.0
    som[1] = 1.0
    imgs = rng.random((4, C_, I, I), dtype=np.float32)
    imgs[0] = 1.0
    imgs[1] = 0.0
    for ed_type in (capi.UINT8, capi.UINT16):
        s = O.shape(N, C_, I, D, nrot, flip, ed, O.QUADRATIC, ed_type)
        oheat, obest = O.map_images(s, som, imgs)
        choices = [capi.KERNEL_AUTO, capi.KERNEL_MFMA_GEMM] + ([capi.KERNEL_MFMA_SYM, capi.KERNEL_MFMA] if ed_type == capi.UINT8 else [])
        for choice in choices:
            say("extremes", ed, ed_type, choice)
            try:
                ctx = capi.Context(N, C_, I, D, nrot, flip, ed, capi.QUADRATIC, ed_type, kernel_choice=choice)
            except capi.PinkError:
                assert choice == capi.KERNEL_MFMA
                continue
            with ctx:
                ctx.set_som(som)
                heat, best = ctx.map(imgs)
            assert np.array_equal(bits(heat), bits(oheat)), (ed_type, choice)
            assert np.array_equal(best, obest), (ed_type, choice)


FUSED_TRAIN_SHAPES = [
    # N, C, I, D, nrot, flip, ed, shape, ed_type, images  -- operand packing inside the rotation and update kernels
    (10, 1, 20, 16, 24, True, 11, capi.CIRCULAR, capi.UINT16, 5),
    (70, 1, 20, 14, 8, False, 14, capi.QUADRATIC, capi.UINT8, 6),     # two column tiles, no flip
    (6, 3, 12, 10, 8, True, 6, capi.QUADRATIC, capi.UINT8, 4),        # three channels: their base rotations side by side in LDS, byte planes packed by the rotation kernel
    (6, 3, 12, 10, 8, True, 6, capi.QUADRATIC, capi.FLOAT, 4),        # three channels, float32 rows from the rotation kernel
    (5, 2, 9, 8, 4, True, 7, capi.CIRCULAR, capi.FLOAT, 3),           # region repeats channel 0 (CPU rule): no inverse table
    (5, 2, 9, 8, 4, True, 7, capi.CIRCULAR, capi.UINT16, 3),
    (4, 1, 200, 150, 8, True, 100, capi.CIRCULAR, capi.UINT8, 2),     # a large LDS tile in the rotation kernel
    (3, 1, 160, 129, 4, True, 128, capi.QUADRATIC, capi.FLOAT, 2),
    (4, 1, 290, 205, 8, True, 100, capi.CIRCULAR, capi.UINT8, 2),     # neurons too large for the rotation kernel's LDS tile
    (3, 1, 280, 201, 4, True, 128, capi.QUADRATIC, capi.FLOAT, 2),
    (4, 1, 160, 226, 8, True, 113, capi.QUADRATIC, capi.UINT8, 2),    # ... but the image fits: interpolated out of LDS
    (3, 1, 160, 226, 8, True, 113, capi.CIRCULAR, capi.UINT16, 2),
    (3, 1, 150, 201, 8, True, 100, capi.QUADRATIC, capi.FLOAT, 2),
    (3, 1, 210, 260, 8, True, 130, capi.QUADRATIC, capi.UINT8, 2),    # nothing in LDS and neurons larger than the image:
    (3, 1, 210, 297, 16, True, 148, capi.CIRCULAR, capi.FLOAT, 2),    # tiles of the base rotation that lie beyond the image
    (2, 2, 204, 230, 4, False, 100, capi.QUADRATIC, capi.UINT16, 2),
    (3, 1, 150, 200, 4, True, 200, capi.QUADRATIC, capi.UINT8, 2),    # 40 000 region elements: uint8 sums beyond 31 bits
    (2, 1, 150, 200, 4, False, 190, capi.QUADRATIC, capi.UINT16, 2),
    (2, 1, 100, 257, 4, False, 257, capi.QUADRATIC, capi.UINT8, 2),   # 66 049: beyond the matrix-core path's row length
    (2, 1, 100, 256, 4, False, 256, capi.QUADRATIC, capi.UINT16, 2),  # 65 536 (uint16 sums reach 2^48 just above that)
    (12, 1, 64, 44, 360, True, 32, capi.QUADRATIC, capi.UINT16, 2),   # 720 variants, uint16 planes out of the rotation kernel
    (70, 1, 40, 48, 36, True, 44, capi.QUADRATIC, capi.UINT16, 3),    # long rows, few tiles: 32 x 32 tiles (3 x 3 real ones among 16), each finished by its block
    (70, 1, 40, 52, 36, True, 48, capi.QUADRATIC, capi.UINT8, 3),     # the same for uint8 (72 k-steps)
    # small uint8 trainers: distance, best match and update of an image in one launch
    (33, 1, 44, 40, 4, True, 40, capi.QUADRATIC, capi.UINT8, 5),      # 1600 elements per neuron, 50 k-steps (two batches of operand loads), a second column tile of one neuron
    (64, 1, 30, 28, 16, True, 20, capi.CIRCULAR, capi.UINT8, 5),      # 32 variants (a full row tile), eight stored variants staged in LDS
    (5, 2, 14, 12, 1, True, 9, capi.QUADRATIC, capi.UINT8, 4),        # one rotation and its flip, two channels
    (7, 1, 14, 12, 1, False, 9, capi.QUADRATIC, capi.UINT8, 3),       # a single variant
    (40, 1, 20, 20, 8, True, 20, capi.QUADRATIC, capi.UINT8, 7),      # an odd number of images: the SOM operand ends in its second buffer
    # small float32 trainers: the distance launch of an image applies the update of the image before it
    (70, 1, 20, 14, 32, True, 9, capi.CIRCULAR, capi.FLOAT, 5),       # three chunks of 64 elements, neurons not a multiple of four
    (9, 1, 12, 8, 16, True, 8, capi.QUADRATIC, capi.FLOAT, 4),        # a single chunk
    (130, 2, 16, 11, 4, True, 11, capi.QUADRATIC, capi.FLOAT, 3),     # two channels, three keys per lane in the search
    (256, 1, 14, 10, 8, False, 10, capi.QUADRATIC, capi.FLOAT, 3),    # the most neurons that train this way
    (257, 1, 14, 10, 8, False, 10, capi.QUADRATIC, capi.FLOAT, 3),    # ... and one more
    (103, 1, 20, 14, 360, True, 12, capi.QUADRATIC, capi.FLOAT, 3),   # 12 x 26 blocks of four neurons are more than the CUs: five per block, the last block three
    (110, 1, 20, 14, 360, True, 9, capi.CIRCULAR, capi.FLOAT, 3),     # ... six per block
    (131, 1, 20, 14, 360, True, 9, capi.QUADRATIC, capi.FLOAT, 3),    # ... seven, three keys per lane in the search
    (165, 1, 20, 14, 360, True, 12, capi.QUADRATIC, capi.FLOAT, 4),   # ... eight, the last block five
]


@pytest.mark.parametrize("N,C_,I,D,nrot,flip,ed,shape_,ed_type,n", FUSED_TRAIN_SHAPES)
def test_train_over_shapes(N, C_, I, D, nrot, flip, ed, shape_, ed_type, n):
    say("train shapes", N, C_, I, D, nrot, flip, ed, shape_, ed_type, n)
    rng = np.random.default_rng(N + I * 3 + nrot)
    som0 = rng.random((N, C_ * D * D), dtype=np.float32)
    imgs = rng.random((n, C_, I, I), dtype=np.float32)
    F = capi.make_update_factors(capi.CARTESIAN, [N], capi.GAUSSIAN, 1.0, 0.5)
    F[F < 0.01] = 0.0                                        # some neurons are skipped by the update
    s = O.shape(N, C_, I, D, nrot, flip, ed, shape_, ed_type)
    want = som0.copy()
    obmu = O.train(s, want, imgs, F)
    with capi.Context(N, C_, I, D, nrot, flip, ed, shape_, ed_type, F, max_batch=2) as ctx:
        ctx.set_som(som0)
        bmu = np.concatenate([ctx.train(imgs[:1]), ctx.train(imgs[1:])])      # two calls, groups of two images
        som = ctx.get_som()
        # the packed operand the update kernel maintains must match a fresh pack of the same weights
        d1, ssd1, best1 = ctx.distance(imgs[0])
        ctx.set_som(som)
        d2, ssd2, best2 = ctx.distance(imgs[0])
    assert np.array_equal(bmu, obmu)
    assert np.array_equal(bits(som), bits(want))             # gate 1e-4; achieved and asserted: bit-exact
    assert np.array_equal(bits(d1), bits(d2)) and np.array_equal(ssd1, ssd2) and np.array_equal(best1, best2)


SMALL_UINT8_SHAPES = [s for s in FUSED_TRAIN_SHAPES if s[8] == capi.UINT8 and s[0] <= 64 and s[4] * (2 if s[5] else 1) <= 32
                      and s[1] * s[3] * s[3] <= 2048] + [
    (64, 1, 28, 28, 4, True, 28, capi.QUADRATIC, capi.UINT8, 40),     # the 8 x 8 MNIST-sized trainer of the benchmark set
    (1, 1, 16, 16, 4, True, 12, capi.QUADRATIC, capi.UINT8, 9),       # one neuron: an exchange with itself
    (64, 1, 45, 45, 4, False, 45, capi.QUADRATIC, capi.UINT8, 6),     # 2025 elements: four per thread, 64 k-steps
]


@pytest.mark.parametrize("form", ["resident", "gives up", "off", "tags wrap"])
@pytest.mark.parametrize("N,C_,I,D,nrot,flip,ed,shape_,ed_type,n", SMALL_UINT8_SHAPES)
def test_small_uint8_trainer_forms(monkeypatch, N, C_, I, D, nrot, flip, ed, shape_, ed_type, n, form):
    """Small uint8 trainers run a whole launch group in one resident launch whose blocks exchange a word per image;
    when a block gives up waiting for the others (forced here by a wait limit of zero polls: every kernel still
    ends by itself) nothing of the context has changed and the group is trained again with one launch per image,
    as it is with the resident form switched off.  All against the oracle, bit for bit."""
    say("small uint8 trainer", form, N, C_, I, D, nrot, flip, ed, shape_, n)
    if form == "gives up":
        monkeypatch.setenv("PINK_HIP_RESIDENT_SPIN_LIMIT", "0")
    if form == "off":
        monkeypatch.setenv("PINK_HIP_RESIDENT_TRAINER", "0")
    if form == "tags wrap":
        # the exchange tags every image with a running 32-bit number; start it where the second call passes the end
        monkeypatch.setenv("PINK_HIP_RESIDENT_FIRST_TAG", str(0xfffffff0 - n + 1))
    rng = np.random.default_rng(N * 7 + I + nrot)
    som0 = rng.random((N, C_ * D * D), dtype=np.float32)
    imgs = rng.random((n, C_, I, I), dtype=np.float32)
    F = capi.make_update_factors(capi.CARTESIAN, [N], capi.GAUSSIAN, 1.0, 0.5)
    F[F < 0.01] = 0.0
    s = O.shape(N, C_, I, D, nrot, flip, ed, shape_, ed_type)
    want = som0.copy()
    obmu = O.train(s, want, imgs, F)
    for max_batch in (0, 3):                                 # the whole call in one group; groups of three images
        with capi.Context(N, C_, I, D, nrot, flip, ed, shape_, ed_type, F, max_batch=max_batch) as ctx:
            ctx.set_som(som0)
            bmu = np.concatenate([ctx.train(imgs[:2]), ctx.train(imgs[2:])])
            som = ctx.get_som()
            counts = ctx.update_counts()
            d1, ssd1, best1 = ctx.distance(imgs[0])          # the operand and norms the trainer left behind
            ctx.set_som(som)
            d2, ssd2, best2 = ctx.distance(imgs[0])
        assert np.array_equal(bmu, obmu), max_batch
        assert np.array_equal(bits(som), bits(want)), max_batch
        assert np.array_equal(counts, np.bincount(obmu, minlength=N)), max_batch
        assert np.array_equal(bits(d1), bits(d2)) and np.array_equal(ssd1, ssd2) and np.array_equal(best1, best2)


@pytest.mark.parametrize("N,ed_type", [(9, capi.FLOAT), (9, capi.UINT8), (530, capi.UINT8)])
def test_train_with_any_factor_matrix(N, ed_type):
    # the C interface takes any N x N matrix, not only the symmetric ones that a distance functor gives
    say("train, factor matrix", N, ed_type)
    C_, I, D, nrot, flip, ed, n = 1, 12, 8, 4, True, 6, 3
    rng = np.random.default_rng(N + ed_type)
    som0 = rng.random((N, C_ * D * D), dtype=np.float32)
    imgs = rng.random((n, C_, I, I), dtype=np.float32)
    F = rng.random((N, N), dtype=np.float32) * np.float32(0.5)
    F[rng.random((N, N)) < 0.3] = 0.0
    assert not np.array_equal(F, F.T)
    s = O.shape(N, C_, I, D, nrot, flip, ed, capi.QUADRATIC, ed_type)
    want = som0.copy()
    obmu = O.train(s, want, imgs, F)
    with capi.Context(N, C_, I, D, nrot, flip, ed, capi.QUADRATIC, ed_type, F) as ctx:
        ctx.set_som(som0)
        bmu = ctx.train(imgs)
        som = ctx.get_som()
    assert np.array_equal(bmu, obmu)
    assert np.array_equal(bits(som), bits(want))


def test_contexts_of_different_sizes_side_by_side():
    # LDS limits are set per kernel, not per context: a context created later with smaller images must
    # not take away what an earlier one needs (uint8 mappers of 150 and 100 pixels, trainers of 181 and 44)
    say("contexts side by side")
    rng = np.random.default_rng(77)
    made = []
    for (I, D, ed, et, F) in ((150, 30, 20, capi.UINT8, None), (100, 30, 20, capi.UINT8, None),
                              (128, 181, 90, capi.UINT16, capi.make_update_factors(capi.CARTESIAN, [4], capi.GAUSSIAN, 1.0, 0.5)),
                              (64, 44, 32, capi.UINT16, capi.make_update_factors(capi.CARTESIAN, [4], capi.GAUSSIAN, 1.0, 0.5))):
        ctx = capi.Context(4, 1, I, D, 8, True, ed, capi.QUADRATIC, et, F)
        som = rng.random((4, D * D), dtype=np.float32)
        img = rng.random((1, I, I), dtype=np.float32)
        ctx.set_som(som)
        made.append((ctx, som, img, I, D, ed, et))
    try:
        for ctx, som, img, I, D, ed, et in made:          # the first contexts run after the last was created
            s = O.shape(4, 1, I, D, 8, True, ed, capi.QUADRATIC, et)
            od, ossd, obest = O.distance_matrix(s, som, O.rotated_images(img, 1, I, D, 8, True))
            d, ssd, best = ctx.distance(img)
            assert np.array_equal(ssd, ossd) and np.array_equal(best, obest)
    finally:
        for m in made:
            m[0].close()


@pytest.mark.parametrize("ed_type,factor", [(capi.UINT8, 255), (capi.UINT16, 65535)])
def test_largest_matrix_core_region_with_extreme_data(ed_type, factor):
    # 65 025 region elements, all of them at one end of the range in both operands: the byte-plane dot
    # products are as large as they get (closed form: 0, and factor^2 * elements)
    say("largest region on the matrix cores", ed_type)
    D = 255
    som = np.zeros((2, D * D), np.float32)
    som[1] = 1.0
    with capi.Context(2, 1, D, D, 1, False, D, capi.QUADRATIC, ed_type) as ctx:
        assert ctx.distance_kernel == capi.KERNEL_MFMA_GEMM
        ctx.set_som(som)
        for value in (0.0, 1.0):
            d, ssd, best = ctx.distance(np.full((1, D, D), value, np.float32))
            want = [0, factor * factor * D * D] if value == 0.0 else [factor * factor * D * D, 0]
            assert ssd.tolist() == want and best.tolist() == [0, 0]


def test_reference_mapper_known_answers():
    # test/CudaTest/mapper.cu:115-119 in float, uint8 and uint16; circular_ed.cu:23-53
    for som_dim, nd, idim, ed, nrot, flip in [(1, 2, 2, 2, 1, False), (1, 3, 3, 2, 1, False), (1, 3, 3, 2, 360, False),
                                              (2, 3, 3, 2, 360, False), (2, 3, 3, 2, 360, True)]:
        N = som_dim * som_dim
        for ed_type in (capi.FLOAT, capi.UINT8, capi.UINT16):
            with capi.Context(N, 1, idim, nd, nrot, flip, ed, capi.QUADRATIC, ed_type) as ctx:
                ctx.set_som(np.ones((N, nd * nd), np.float32))
                heat, _ = ctx.map(np.zeros((idim, idim), np.float32))
            assert heat.ravel().tolist() == [2.0] * N
    image = np.zeros(16, np.float32)
    image[4] = 1.0
    som = np.zeros(64, np.float32)
    som[4], som[18], som[43], som[61] = 1.0, 0.5, 0.8, 0.3
    with capi.Context(4, 1, 4, 4, 4, False, 4, capi.CIRCULAR, capi.FLOAT) as ctx:
        ctx.set_som(som)
        heat, best = ctx.map(image)
    assert np.allclose(heat.ravel(), [0.0, 0.5, 0.2, 0.7], atol=0.01)
    assert best.ravel().tolist() == [0, 1, 2, 3]


def test_map_full_size_properties():
    """cfg 1 at a size the oracle does not cover: properties that hold at any size."""
    w = synthetic.WORKLOADS["cfg1"]
    n = 2000
    imgs = synthetic.images(w, n)
    som = synthetic.initial_som(w)
    with synthetic.make_context(w) as ctx:
        ctx.set_som(som)
        heat, best = ctx.map(imgs)
        heat2, best2 = ctx.map(imgs[::-1])
        # rotating an image by a quarter turn permutes its variants: same heatmap, shifted index
        turned = np.ascontiguousarray(np.rot90(imgs[:50], k=-1, axes=(2, 3)))
        heat3, best3 = ctx.map(turned)
    assert np.array_equal(bits(heat2[::-1]), bits(heat)) and np.array_equal(best2[::-1], best)   # order-independent
    assert (heat >= 0).all() and np.isfinite(heat).all() and (best < w.R).all()
    assert np.array_equal(bits(heat3), bits(heat[:50]))


def test_host_buffers_in_pieces_match_smaller_calls():
    """Inputs beyond 64 MB go to the device piece by piece while the kernels of the piece before run, a mapper's
    inputs from 32 MB on through two pinned buffers that several host threads fill side by side (147 MB here: pieces
    that are no multiple of the 8 MB buffers): the results are those of calls small enough to go in one plain copy
    (1500 images, 25 MB)."""
    w = synthetic.WORKLOADS["cfg1"]
    n = 9000                                                   # 147 MB of images: three pieces
    imgs = synthetic.images(w, n)
    say("pieces: map", n)
    with synthetic.make_context(w) as ctx:
        ctx.set_som(synthetic.initial_som(w))
        heat, best = ctx.map(imgs)
        parts = [ctx.map(imgs[i:i + 1500]) for i in range(0, n, 1500)]
    assert np.array_equal(bits(heat), bits(np.concatenate([p[0] for p in parts])))
    assert np.array_equal(best, np.concatenate([p[1] for p in parts]))
    w = synthetic.WORKLOADS["cfg3"]
    n = 1200                                                   # 144 MB of three-channel images: three pieces
    imgs = synthetic.images(w, n)
    tiny = dict(N=16, dims=[4, 4])
    F = capi.make_update_factors(capi.CARTESIAN, tiny["dims"], capi.GAUSSIAN, 1.1, 0.2)
    som0 = synthetic.mt19937_uniform(tiny["N"] * w.channels * 40 * 40, 7).reshape(tiny["N"], -1)
    say("pieces: train", n)
    results = []
    for step in (n, 200):
        with capi.Context(tiny["N"], w.channels, w.image_dim, 40, 8, True, 30, capi.QUADRATIC, capi.UINT8, F) as ctx:
            ctx.set_som(som0)
            bmu = np.concatenate([ctx.train(imgs[i:i + step]) for i in range(0, n, step)])
            results.append((bmu, ctx.get_som(), ctx.update_counts()))
    assert np.array_equal(results[0][0], results[1][0]) and np.array_equal(bits(results[0][1]), bits(results[1][1]))
    assert np.array_equal(results[0][2], np.bincount(results[0][0], minlength=tiny["N"]))


def test_empty_inputs_are_no_ops():
    w = synthetic.WORKLOADS["cfg4"]
    som = synthetic.initial_som(w)
    none = np.empty((0, w.channels, w.image_dim, w.image_dim), np.float32)
    with synthetic.make_context(w) as ctx:
        ctx.set_som(som)
        assert ctx.train(none).shape == (0,)
        assert np.array_equal(bits(ctx.get_som()), bits(som))
    with capi.Context(w.som_size, w.channels, w.image_dim, w.neuron_dim, w.num_rot, w.use_flip, w.ed_dim,
                      w.ed_shape, w.ed_type) as ctx:
        ctx.set_som(som)
        heat, best = ctx.map(none)
        assert heat.shape == (0, w.som_size) and best.shape == (0, w.som_size)


@pytest.mark.parametrize("ed_type", [capi.UINT8, capi.UINT16])
def test_out_of_range_pixels_saturate_like_the_oracle(ed_type):
    """Values outside [0, 1] (undefined in the reference) quantise to the ends of the range on every
    integer path, 1.0 exactly to the top value."""
    N, C_, I, D, nrot, flip, ed = 20, 1, 24, 18, 40, True, 16
    rng = np.random.default_rng(5)
    som = (rng.random((N, D * D), dtype=np.float32) * 2 - 0.5).astype(np.float32)
    imgs = (rng.random((6, C_, I, I), dtype=np.float32) * 2 - 0.5).astype(np.float32)
    imgs[0, 0, :4, :4] = 1.0
    som[0, :9] = [1.0, 0.0, -0.0, 2.0, -3.0, 1.0000001, 0.99999994, 0.5, 1e-9]
    s = O.shape(N, C_, I, D, nrot, flip, ed, O.QUADRATIC, ed_type)
    oheat, obest = O.map_images(s, som, imgs)
    for choice in (capi.KERNEL_AUTO, capi.KERNEL_VALU, capi.KERNEL_MFMA_GEMM):
        with capi.Context(N, C_, I, D, nrot, flip, ed, capi.QUADRATIC, ed_type, kernel_choice=choice) as ctx:
            ctx.set_som(som)
            heat, best = ctx.map(imgs)
        assert np.array_equal(bits(heat), bits(oheat)) and np.array_equal(best, obest), choice


def test_train_full_size_is_deterministic_and_counts_every_image():
    """cfg 4 at its full size (60 000 images), where the oracle is not run: two runs agree bit for
    bit, every image gets a best-matching neuron, and a second epoch moves the map less than the first."""
    w = synthetic.WORKLOADS["cfg4"]
    imgs = synthetic.images(w)
    som0 = synthetic.initial_som(w)
    runs = []
    for _ in range(2):
        with synthetic.make_context(w) as ctx:
            ctx.set_som(som0)
            bmu = ctx.train(imgs)
            som1 = ctx.get_som()
            ctx.train(imgs)
            som2 = ctx.get_som()
        runs.append((bmu, som1, som2))
    assert np.array_equal(runs[0][0], runs[1][0]) and np.array_equal(bits(runs[0][1]), bits(runs[1][1]))
    bmu, som1, som2 = runs[0]
    assert bmu.shape == (w.n_images,) and bmu.max() < w.som_size
    assert np.bincount(bmu, minlength=w.som_size).sum() == w.n_images
    assert np.isfinite(som2).all()
    assert np.abs(som2 - som1).mean() < np.abs(som1 - som0).mean()


def test_mfma_kernel_refused_where_it_does_not_apply():
    with pytest.raises(capi.PinkError):
        capi.Context(200, 1, 16, 12, 8, True, 8, capi.QUADRATIC, capi.UINT8, kernel_choice=capi.KERNEL_MFMA)
    with pytest.raises(capi.PinkError):
        capi.Context(16, 1, 16, 12, 8, True, 8, capi.QUADRATIC, capi.FLOAT, kernel_choice=capi.KERNEL_MFMA)


@pytest.mark.parametrize("name,choice,distance_launches,update_launches", [
    # a small float32 trainer: a distance launch applies the update of the image before it; the group ends with one
    # launch for the neurons' full images and the last image's update
    ("cfg0", capi.KERNEL_AUTO, 5, 2),
    ("cfg4", capi.KERNEL_MFMA_GEMM, 5, 5),
    ("cfg4", capi.KERNEL_AUTO, 0, 1),       # a small uint8 trainer: one resident launch for the group
])
def test_profiling_counts_launches(name, choice, distance_launches, update_launches):
    w = synthetic.WORKLOADS[name]
    with synthetic.make_context(w, kernel_choice=choice) as ctx:
        ctx.set_som(synthetic.initial_som(w))
        ctx.set_profiling(True)
        ctx.train(synthetic.images(w, 5))
        t = ctx.kernel_times()
        ctx.set_profiling(False)
    # variants are prepared for a group of images per launch; distance and update run per image
    assert t["rotate"][0] == 1 and t["distance"][0] == distance_launches and t["update"][0] == update_launches
    assert all(ms >= 0 for _, ms in t.values())
