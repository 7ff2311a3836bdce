"""The float32 matrix-core recast (kernel_choice KERNEL_MFMA_F32, never the default) against the CPU
oracle: what it keeps and what it gives up.

The recast computes |a|^2 + |b|^2 - 2 a.b with float32 MFMA dot products, so it does not follow the
CPU's summation order.  Gates of the path (float32 distances within 1e-5 relative, best rotation equal
except where the CPU's candidates are that close, weights within 1e-4 after an epoch) are measured here
at the cfg0 and cfg3 shapes, at SOM initialisation and on a trained SOM; each assertion states the bound
this mode does meet, and the printed line gives the measured values.
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


def _shape(w):
    return O.shape(w.som_size, w.channels, w.image_dim, w.neuron_dim, w.num_rot, w.use_flip, w.ed_dim, w.ed_shape, capi.FLOAT)


def _compare_distances(w, som, imgs):
    """Recast distances and best rotations of `imgs` against the oracle's.  Returns the largest relative
    distance error, the share of (image, neuron) pairs with another best rotation, and the largest relative
    gap, in the CPU's own arithmetic, between the CPU's minimum and its distance at the rotation the recast chose."""
    s = _shape(w)
    worst_rel, mismatches, pairs, worst_gap = 0.0, 0, 0, 0.0
    with synthetic.make_context(w, trainer=False, ed_type=capi.FLOAT, kernel_choice=capi.KERNEL_MFMA_F32) as ctx:
        assert ctx.distance_kernel == capi.KERNEL_MFMA_F32
        ctx.set_som(som)
        for img in imgs:
            d, _, best = ctx.distance(img)
            rot = O.rotated_images(img, w.channels, w.image_dim, w.neuron_dim, w.num_rot, w.use_flip)
            od, _, obest = O.distance_matrix(s, som, rot)
            worst_rel = max(worst_rel, float((np.abs(d.astype(np.float64) - od) / np.maximum(od, 1e-30)).max()))
            pairs += len(od)
            for n in np.nonzero(best != obest)[0]:
                mismatches += 1
                at_choice = O.ssd_f32(som[n], rot[best[n]].ravel(), w.channels, w.neuron_dim, w.ed_dim, w.ed_shape)
                worst_gap = max(worst_gap, (float(at_choice) - float(od[n])) / max(float(od[n]), 1e-30))
    return worst_rel, mismatches / pairs, worst_gap


@pytest.fixture(scope="module")
def trained_cfg0():
    w0 = synthetic.WORKLOADS["cfg0"]
    with synthetic.make_context(w0) as tr:
        tr.set_som(synthetic.initial_som(w0))
        tr.train(synthetic.images(w0))
        return tr.get_som()


def test_cfg0_distances_at_initialisation():
    w = synthetic.WORKLOADS["cfg0"]
    rel, share, gap = _compare_distances(w, synthetic.initial_som(w), synthetic.images(w, 6))
    say("recast cfg0, initial SOM: max relative distance error %.3g, best rotation differs in %.2f %% of pairs, "
        "largest CPU-side gap at the chosen rotation %.3g" % (rel, 100 * share, gap))
    assert rel <= 1e-5                      # the distance gate holds on noise-like neurons
    assert gap <= 1e-5                      # and every different choice is a tie within it


def test_cfg0_distances_on_the_trained_som(trained_cfg0):
    w = synthetic.WORKLOADS["cfg0"]
    rel, share, gap = _compare_distances(w, trained_cfg0, synthetic.images(w, 6, seed=99))
    say("recast cfg0, SOM after one epoch: max relative distance error %.3g, best rotation differs in %.2f %% of pairs, "
        "largest CPU-side gap at the chosen rotation %.3g" % (rel, 100 * share, gap))
    assert rel <= 1e-4
    assert gap <= 1e-4


def test_cfg3_distances_at_initialisation():
    w = synthetic.WORKLOADS["cfg3"]
    rel, share, gap = _compare_distances(w, synthetic.initial_som(w), synthetic.images(w, 1))
    say("recast cfg3, initial SOM: max relative distance error %.3g, best rotation differs in %.2f %% of pairs, "
        "largest CPU-side gap at the chosen rotation %.3g" % (rel, 100 * share, gap))
    assert rel <= 1e-5
    assert gap <= 1e-5


def test_cfg0_weights_after_training_with_the_recast():
    """Free-running training: a different best rotation pulls a neuron toward another variant, so the
    weights leave the CPU's trajectory; reported, with the bound that holds."""
    w = synthetic.WORKLOADS["cfg0"]
    n = 300
    imgs = synthetic.images(w, n)
    som0 = synthetic.initial_som(w)
    F = synthetic.update_factors(w)
    with synthetic.make_context(w, kernel_choice=capi.KERNEL_MFMA_F32) as ctx:
        ctx.set_som(som0)
        bmu = ctx.train(imgs)
        got = ctx.get_som()
    want = som0.copy()
    obmu = O.train(_shape(w), want, imgs, F)
    drift = float(np.abs(got - want).max())
    say("recast cfg0, %d images trained: best-matching neuron equal for %.1f %% of the images, max weight difference %.3g "
        "(gate of the exact path: 1e-4)" % (n, 100 * float((bmu == obmu).mean()), drift))
    assert np.isfinite(got).all()
    assert drift <= 0.2                      # weights stay within the images' own range of each other, no more
