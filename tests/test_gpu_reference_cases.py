"""The reference's own differential trainer cases, replayed through the HIP trainer.

The reference compares its CPU trainer with its GPU trainer on these shapes, one image, gate 1e-4 on the
weights: test/CudaTest/compare_trainer_cpu.cu:81-98 (2-D), compare_trainer_3d_cpu.cu:83-102 (two channels)
and compare_trainer_mixed.cu:78-93 (float against uint8 distances).  Same set-up here: a 2 x 2 cartesian
SOM, GaussianFunctor(1.1, 0.2), bilinear interpolation, the image and the SOM both filled by
fill_random_uniform with its default seed (UtilitiesLib/Filler.h:17-25: std::mt19937::default_seed = 5489,
so the image repeats the first values of the SOM).  The CPU side is the oracle; the HIP side goes through
the C ABI.  Beyond the reference's gate the tests assert what this build achieves: equal best matches and
bit-equal weights.
"""
import sys

import numpy as np
import pytest

import oracle as O
from pink_amd import capi

pytestmark = pytest.mark.gpu

# som_dim, image_dim, neuron_dim, euclidean_distance_dim, num_rot, use_flip  (compare_trainer_cpu.cu:81-98)
CASES_2D = [
    (2, 2, 2, 2, 1, False), (2, 2, 2, 2, 4, False), (2, 2, 2, 2, 8, False),
    (2, 2, 2, 2, 1, True), (2, 2, 2, 2, 4, True), (2, 2, 2, 2, 8, True),
    (2, 4, 4, 4, 1, False), (2, 2, 4, 4, 1, False),
    (2, 64, 45, 45, 360, True), (2, 64, 100, 100, 360, True), (2, 64, 100, 45, 360, True),
    (2, 124, 91, 64, 360, True),
    (2, 4, 2, 2, 1, False), (2, 4, 2, 2, 8, False), (2, 4, 2, 2, 1, True), (2, 4, 2, 2, 8, True),
]
# the same sixteen with an image depth of 2 (compare_trainer_3d_cpu.cu:83-102)
CASES_3D = [(s, i, 2, d, e, r, f) for (s, i, d, e, r, f) in CASES_2D]
# compare_trainer_mixed.cu:78-93: the first eleven, max_update_distance 0.0 (no limit, like -1)
CASES_MIXED = CASES_2D[:11]

DEFAULT_SEED = 5489


def say(*a):
    print(*a, flush=True)
    sys.stdout.flush()


def bits(a):
    return np.ascontiguousarray(a, np.float32).view(np.uint32)


def _case(som_dim, image_dim, depth, neuron_dim, ed_dim, num_rot, use_flip, ed_type, max_update_distance=-1.0):
    N = som_dim * som_dim
    image = O.fill_random_uniform(depth * image_dim * image_dim, DEFAULT_SEED).reshape(1, depth, image_dim, image_dim)
    som0 = O.fill_random_uniform(N * depth * neuron_dim * neuron_dim, DEFAULT_SEED).reshape(N, -1)
    F = capi.make_update_factors(capi.CARTESIAN, [som_dim, som_dim], capi.GAUSSIAN, 1.1, 0.2, max_update_distance)
    s = O.shape(N, depth, image_dim, neuron_dim, num_rot, use_flip, ed_dim, O.QUADRATIC, ed_type)
    want = som0.copy()
    obmu = O.train(s, want, image, F)
    with capi.Context(N, depth, image_dim, neuron_dim, num_rot, use_flip, ed_dim, capi.QUADRATIC, ed_type, F) as ctx:
        ctx.set_som(som0)
        bmu = ctx.train(image)
        got = ctx.get_som()                                  # the reference's update_som()
    return som0, want, obmu, got, bmu


@pytest.mark.parametrize("som_dim,image_dim,neuron_dim,ed_dim,num_rot,use_flip", CASES_2D)
def test_compare_trainer_cpu_cartesian_2d_float(som_dim, image_dim, neuron_dim, ed_dim, num_rot, use_flip):
    say("compare_trainer_cpu", som_dim, image_dim, neuron_dim, ed_dim, num_rot, use_flip)
    som0, want, obmu, got, bmu = _case(som_dim, image_dim, 1, neuron_dim, ed_dim, num_rot, use_flip, capi.FLOAT)
    assert np.abs(got - want).max() <= 1e-4                  # the reference's gate (compare_trainer_cpu.cu:76)
    assert not np.array_equal(want, som0)                    # the image did move the SOM
    assert np.array_equal(bmu, obmu)
    assert np.array_equal(bits(got), bits(want))


@pytest.mark.parametrize("som_dim,image_dim,depth,neuron_dim,ed_dim,num_rot,use_flip", CASES_3D)
def test_compare_trainer_3d_cpu_cartesian_3d_float(som_dim, image_dim, depth, neuron_dim, ed_dim, num_rot, use_flip):
    say("compare_trainer_3d_cpu", som_dim, image_dim, depth, neuron_dim, ed_dim, num_rot, use_flip)
    som0, want, obmu, got, bmu = _case(som_dim, image_dim, depth, neuron_dim, ed_dim, num_rot, use_flip, capi.FLOAT)
    assert np.abs(got - want).max() <= 1e-4                  # compare_trainer_3d_cpu.cu:78
    assert np.array_equal(bmu, obmu)
    assert np.array_equal(bits(got), bits(want))


@pytest.mark.parametrize("ed_type", [capi.UINT8, capi.UINT16])
@pytest.mark.parametrize("som_dim,image_dim,neuron_dim,ed_dim,num_rot,use_flip", CASES_MIXED)
def test_compare_trainer_mixed(som_dim, image_dim, neuron_dim, ed_dim, num_rot, use_flip, ed_type):
    """The reference trains one SOM with float and one with uint8 distances and expects the same weights
    within 1e-4 (the update never sees the distance type; the two agree when they pick the same best match
    and rotations).  Here: the integer trainer against the oracle in the same integer mode, bit for bit,
    and the reference's own comparison, float against integer, on the HIP side."""
    say("compare_trainer_mixed", som_dim, image_dim, neuron_dim, ed_dim, num_rot, use_flip, ed_type)
    som0, want, obmu, got, bmu = _case(som_dim, image_dim, 1, neuron_dim, ed_dim, num_rot, use_flip, ed_type, 0.0)
    assert np.array_equal(bmu, obmu)
    assert np.array_equal(bits(got), bits(want))
    _, fwant, _, fgot, fbmu = _case(som_dim, image_dim, 1, neuron_dim, ed_dim, num_rot, use_flip, capi.FLOAT, 0.0)
    assert np.array_equal(bits(fgot), bits(fwant))
    # the reference's own assertion (compare_trainer_mixed.cu:73): float against integer distances
    say("   float against integer distances: max weight difference %.3g" % np.abs(fgot - got).max())
    assert np.abs(fgot - got).max() <= 1e-4
