"""Seeded random shapes through the trainer and the mapper, against the CPU oracle, bit for bit.

The fixed lists elsewhere in tests/ follow the reference's own cases and the benchmark configurations; this
file draws shapes the lists do not hold (odd image and neuron sizes, regions from 2 x 2 to the whole neuron,
1 to 360 rotations, 1 to 400 neurons, 1 to 3 channels, both region shapes, all three distance types, small
launch groups, update factors with and without exact zeros), so that every distance kernel, every rotation
form and every update form is reached with sizes its tiling was not chosen for.
"""
import sys

import numpy as np
import pytest

import oracle as O
from pink_amd import capi

pytestmark = pytest.mark.gpu

CASES_PER_SEED = 60


def say(*a):
    print(*a, flush=True)
    sys.stdout.flush()


def bits(a):
    return np.ascontiguousarray(a, np.float32).view(np.uint32)


def draw(rng):
    while True:
        channels = int(rng.choice([1, 1, 1, 2, 3]))
        image_dim = int(rng.integers(8, 150))
        neuron_dim = int(rng.integers(6, min(160, int(image_dim * 1.5) + 2)))
        ed_dim = int(rng.integers(2, neuron_dim + 1))
        ed_shape = int(rng.choice([capi.QUADRATIC, capi.CIRCULAR]))
        ed_type = int(rng.choice([capi.FLOAT, capi.UINT8, capi.UINT16]))
        num_rot = int(rng.choice([1, 4, 8, 12, 36, 64, 120, 360]))
        use_flip = bool(rng.integers(0, 2))
        som_size = int(rng.choice([1, 3, 9, 33, 64, 65, 100, 130, 257, 331, 400]))
        n_images = int(rng.integers(2, 30))
        max_batch = int(rng.choice([0, 0, 2, 5]))
        sigma, damping = float(rng.uniform(0.5, 3)), float(rng.uniform(0.05, 0.9))
        cut = bool(rng.integers(0, 2))
        region = len(O.region(channels, neuron_dim, ed_dim, ed_shape))
        if region and som_size * num_rot * (2 if use_flip else 1) * region <= 6e9:   # seconds for the oracle
            return (som_size, channels, image_dim, neuron_dim, num_rot, use_flip, ed_dim, ed_shape, ed_type,
                    n_images, max_batch, sigma, damping, cut)


@pytest.mark.parametrize("seed", [11, 12, 13, 14])
def test_random_shapes_train_then_map(seed):
    rng = np.random.default_rng(seed)
    for k in range(CASES_PER_SEED):
        (N, C, I, D, nrot, flip, ed, shp, ty, n, mb, sigma, damping, cut) = case = draw(rng)
        say("seed", seed, "case", k, case)
        som0 = rng.random((N, C * D * D), dtype=np.float32)
        imgs = rng.random((n, C, I, I), dtype=np.float32)
        F = capi.make_update_factors(capi.CARTESIAN, [N], capi.GAUSSIAN, sigma, damping)
        if cut:
            F[F < 0.01] = 0.0
        s = O.shape(N, C, I, D, nrot, flip, ed, shp, ty)
        want = som0.copy()
        obmu = O.train(s, want, imgs, F)
        with capi.Context(N, C, I, D, nrot, flip, ed, shp, ty, F, max_batch=mb) as ctx:
            ctx.set_som(som0)
            bmu = ctx.train(imgs)
            got = ctx.get_som()
        assert np.array_equal(bmu, obmu), case
        assert np.array_equal(bits(got), bits(want)), case
        with capi.Context(N, C, I, D, nrot, flip, ed, shp, ty, max_batch=mb) as mapper:
            mapper.set_som(want)
            heat, best = mapper.map(imgs)
        oheat, obest = O.map_images(s, want, imgs)
        assert np.array_equal(bits(heat), bits(oheat)), case
        assert np.array_equal(best, obest), case
