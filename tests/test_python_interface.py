"""The Python interface pink_amd.pink mirrors the reference's pybind11 module (src/pink/pink.cpp).

Host-side behaviour runs everywhere; the scenarios of the reference's own Python and C++ binding
tests (python/tests/test_dynamic.py, test/PythonBindingTest) run on the GPU against the oracle.
"""
import math

import numpy as np
import pytest

import oracle as O
from pink_amd import capi, pink


def test_module_surface():
    # python/tests/test_pink_pybind11.py:4-7 and the names bound in src/pink/pink.cpp:25-153
    assert pink.doc() == "PINK python interface"
    assert pink.__version__.startswith("2.5")
    assert int(pink.Interpolation.BILINEAR) == 1 and pink.NEAREST_NEIGHBOR == 0
    assert (int(pink.DataType.FLOAT), int(pink.DataType.UINT16), int(pink.DataType.UINT8)) == (0, 1, 2)
    assert (int(pink.Layout.CARTESIAN), int(pink.Layout.HEXAGONAL)) == (0, 1)
    assert (int(pink.EuclideanDistanceShape.QUADRATIC), int(pink.CIRCULAR)) == (0, 1)
    for name in ("Data", "SOM", "Trainer", "Mapper", "GaussianFunctor"):
        assert hasattr(pink, name)


def test_gaussian_functor_closed_form():
    # test/UtilitiesTest/DistributionFunctorTest.cpp:28-40
    f = pink.GaussianFunctor(1.1, 0.2)
    for d in (0.0, 1.0, 2.5):
        want = 0.2 / (1.1 * math.sqrt(2 * math.pi)) * math.exp(-0.5 * (d / 1.1) ** 2)
        assert f(d) == pytest.approx(want, rel=1e-6)
    assert pink.GaussianFunctor().sigma == pytest.approx(1.1) and pink.GaussianFunctor().damping == pytest.approx(0.2)


def test_data_and_som_hold_copies_with_the_buffer_protocol():
    a = np.arange(6, dtype=np.float32).reshape(2, 3)
    with pytest.raises(pink.exception):
        pink.Data(a, layout="cartesian-3d")
    img = np.arange(16, dtype=np.float32).reshape(4, 4)
    d = pink.Data(img)
    img[0, 0] = 99.0
    assert np.array(d, copy=False)[0, 0] == 0.0 and d.shape == (4, 4)        # a copy, like the std::vector
    with pytest.raises(TypeError):
        pink.Data(np.zeros((4, 4), np.float64))
    with pytest.raises(pink.exception):
        pink.Data(img, data_type="float64")
    s = pink.SOM(np.zeros((3, 2, 4, 4), np.float32))
    assert s.get_som_layout() == "cartesian-2d" and s.number_of_neurons == 6 and s.neuron_shape == (4, 4)
    assert np.array(s, copy=False).shape == (3, 2, 4, 4)
    h = pink.SOM(np.zeros((19, 4, 4), np.float32), som_layout="hexagonal-2d")
    assert h.number_of_neurons == 19 and h._dims == [5]
    with pytest.raises(pink.exception):
        pink.SOM(np.zeros((18, 4, 4), np.float32), som_layout="hexagonal-2d")
    with pytest.raises(pink.exception):
        pink.SOM(np.zeros((2, 2, 4, 4), np.float32), som_layout="cartesian-3d")
    c3 = pink.SOM(np.zeros((2, 2, 3, 4, 4), np.float32), neuron_layout="cartesian-3d")
    assert c3.neuron_shape == (3, 4, 4)


def test_update_factors_from_python_callables_match_the_library():
    som = pink.SOM(np.zeros((4, 3, 4, 4), np.float32))
    lib = pink.Trainer._update_factors(som, pink.GaussianFunctor(1.3, 0.4), -1.0)

    class SameGaussian(pink.GaussianFunctor):       # a subclass takes the generic path: evaluated in Python
        pass

    py = pink.Trainer._update_factors(som, SameGaussian(1.3, 0.4), -1.0)
    assert lib.shape == (12, 12) and np.allclose(lib, py, rtol=2e-7, atol=0)
    step = pink.Trainer._update_factors(som, lambda d: 1.0 if d <= 1.0 else 0.0, -1.0)
    assert np.array_equal(step, capi.make_update_factors(capi.CARTESIAN, [4, 3], capi.STEP, 1.0))
    limited = pink.Trainer._update_factors(som, lambda d: 1.0, 1.5)           # Trainer.h:72: strictly below the limit
    dist = capi.layout_distances(capi.CARTESIAN, [4, 3])
    assert np.array_equal(limited != 0, dist < 1.5)
    hexa = pink.SOM(np.zeros((7, 4, 4), np.float32), som_layout="hexagonal-2d")
    want = capi.make_update_factors(capi.HEXAGONAL, [3], capi.GAUSSIAN, 1.1, 0.2)
    assert np.array_equal(pink.Trainer._update_factors(hexa, pink.GaussianFunctor(), -1.0), want)


def test_argument_errors_at_construction():
    som = pink.SOM(np.zeros((2, 2, 4, 4), np.float32))
    with pytest.raises(TypeError):
        pink.Trainer(som)                                                   # euclidean_distance_dim has no default
    with pytest.raises(pink.exception):
        pink.Trainer(som, euclidean_distance_dim=2, use_gpu=False)
    with pytest.raises(pink.exception):
        pink.Trainer(som, number_of_rotations=7, euclidean_distance_dim=2)  # Trainer.h:66-67
    with pytest.raises(pink.exception):
        pink.Mapper(som, number_of_rotations=7, euclidean_distance_dim=2)
    one_d = pink.SOM(np.zeros((2, 2, 4), np.float32), neuron_layout="cartesian-1d")
    with pytest.raises(pink.exception):
        pink.Trainer(one_d, euclidean_distance_dim=2)                       # generate_rotated_images.h:36-46


@pytest.mark.gpu
def test_reference_dynamic_scenario():
    # python/tests/test_dynamic.py:33-49 (with the distance dimension its constructor needs)
    np_data = np.array([[1, 2], [3, 4]], np.float32)
    data = pink.Data(np_data, data_type="float32", layout="cartesian-2d")
    np_som = np.zeros((2, 2, 2, 2)).astype(np.float32)
    som = pink.SOM(np_som, data_type="float32", som_layout="cartesian-2d", neuron_layout="cartesian-2d")
    fn = pink.GaussianFunctor(sigma=1.1, damping=1.0)
    trainer = pink.Trainer(som, fn, number_of_rotations=1, use_flip=False, use_gpu=True, euclidean_distance_dim=2,
                           euclidean_distance_type=pink.DataType.FLOAT)
    trainer(data)
    trainer.update_som()
    got = np.array(som, copy=False)
    F = capi.make_update_factors(capi.CARTESIAN, [2, 2], capi.GAUSSIAN, 1.1, 1.0)
    want = np.zeros((4, 4), np.float32)
    s = O.shape(4, 1, 2, 2, 1, False, 2, O.QUADRATIC, capi.FLOAT)
    O.train(s, want, np_data[None, None], F)
    assert np.array_equal(got.reshape(4, 4).view(np.uint32), want.view(np.uint32))
    assert trainer.get_update_info().sum() == 1


@pytest.mark.gpu
@pytest.mark.parametrize("ed_type", [pink.DataType.FLOAT, pink.DataType.UINT8, pink.DataType.UINT16])
def test_trainer_and_mapper_against_the_oracle(ed_type):
    rng = np.random.default_rng(11)
    np_som = rng.random((3, 3, 12, 12), dtype=np.float32)
    images = rng.random((5, 16, 16), dtype=np.float32)
    som = pink.SOM(np_som.copy())
    trainer = pink.Trainer(som, pink.GaussianFunctor(1.1, 0.2), number_of_rotations=8, use_flip=True,
                           euclidean_distance_dim=8, euclidean_distance_type=ed_type)
    for img in images[:2]:
        trainer(pink.Data(img))                       # per image, as the reference is driven
    trainer.train(images[2:])                         # and the rest in one call
    trainer.update_som()
    F = capi.make_update_factors(capi.CARTESIAN, [3, 3], capi.GAUSSIAN, 1.1, 0.2)
    want = np_som.reshape(9, -1).copy()
    s = O.shape(9, 1, 16, 12, 8, True, 8, O.QUADRATIC, int(ed_type))
    obmu = O.train(s, want, images[:, None], F)
    assert np.array_equal(np.array(som, copy=False).reshape(9, -1).view(np.uint32), want.view(np.uint32))
    assert np.array_equal(trainer.get_update_info(), np.bincount(obmu, minlength=9))
    mapper = pink.Mapper(som, number_of_rotations=8, use_flip=True, euclidean_distance_dim=8,
                         euclidean_distance_type=ed_type)
    heat, best = mapper(pink.Data(images[0]))
    assert isinstance(heat, list) and isinstance(best, list) and len(heat) == 9
    oheat, obest = O.map_images(s, want, images[:1, None])
    assert np.array_equal(np.float32(heat).view(np.uint32), oheat[0].view(np.uint32)) and best == obest[0].tolist()
    heat_all, best_all = mapper.map(images)
    oheat, obest = O.map_images(s, want, images[:, None])
    assert np.array_equal(heat_all.view(np.uint32), oheat.view(np.uint32)) and np.array_equal(best_all, obest)


@pytest.mark.gpu
def test_hexagonal_som_with_three_channels():
    rng = np.random.default_rng(3)
    np_som = rng.random((7, 2, 10, 10), dtype=np.float32)          # hexagonal edge 3, neurons of 2 channels
    images = rng.random((3, 2, 14, 14), dtype=np.float32)
    som = pink.SOM(np_som.copy(), som_layout="hexagonal-2d", neuron_layout="cartesian-3d")
    trainer = pink.Trainer(som, lambda d: 0.3 if d < 1.5 else 0.0, number_of_rotations=4, euclidean_distance_dim=6,
                           euclidean_distance_type=pink.DataType.FLOAT)
    for img in images:
        trainer(pink.Data(img, layout="cartesian-3d"))
    trainer.update_som()
    F = trainer.update_factors
    want = np_som.reshape(7, -1).copy()
    s = O.shape(7, 2, 14, 10, 4, True, 6, O.QUADRATIC, capi.FLOAT)
    O.train(s, want, images, F)
    assert np.array_equal(np.array(som, copy=False).reshape(7, -1).view(np.uint32), want.view(np.uint32))


@pytest.mark.gpu
def test_per_image_calls_are_queued_and_counted_on_the_device():
    # 40 operator() calls in a row (more than the ring of staging slots holds), a call that hands the
    # best-matching neurons back in between, an image of another size (a new device context), and the
    # update counts over all of it
    rng = np.random.default_rng(3)
    np_som = rng.random((3, 3, 10, 10), dtype=np.float32)
    images = rng.random((45, 14, 14), dtype=np.float32)
    som = pink.SOM(np_som.copy())
    trainer = pink.Trainer(som, pink.GaussianFunctor(1.1, 0.2), number_of_rotations=4, use_flip=True,
                           euclidean_distance_dim=6, euclidean_distance_type=pink.DataType.UINT8)
    assert trainer.get_update_info().sum() == 0
    for img in images[:20]:
        trainer(pink.Data(img))
    bmu_mid = trainer.train(images[20:25])
    for img in images[25:]:
        trainer(pink.Data(img))
    F = capi.make_update_factors(capi.CARTESIAN, [3, 3], capi.GAUSSIAN, 1.1, 0.2)
    want = np_som.reshape(9, -1).copy()
    s = O.shape(9, 1, 14, 10, 4, True, 6, O.QUADRATIC, capi.UINT8)
    obmu = O.train(s, want, images[:, None], F)
    assert np.array_equal(bmu_mid, obmu[20:25])
    assert np.array_equal(trainer.get_update_info(), np.bincount(obmu, minlength=9))
    trainer.update_som()
    assert np.array_equal(np.array(som, copy=False).reshape(9, -1).view(np.uint32), want.view(np.uint32))
    # a larger image: the weights and the counts carry over into the new context
    big = rng.random((1, 18, 18), dtype=np.float32)
    trainer(pink.Data(big[0]))
    s2 = O.shape(9, 1, 18, 10, 4, True, 6, O.QUADRATIC, capi.UINT8)
    obmu2 = O.train(s2, want, big[:, None], F)
    assert np.array_equal(trainer.get_update_info(), np.bincount(np.concatenate([obmu, obmu2]), minlength=9))
    trainer.update_som()
    assert np.array_equal(np.array(som, copy=False).reshape(9, -1).view(np.uint32), want.view(np.uint32))
