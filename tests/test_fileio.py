"""Binary file formats of the reference (FILE_FORMATS.md:53-85) in pink_amd.fileio.

The expected bytes are written out field by field from the reference's own writers and test
fixtures (cited per test), not produced by the module under test.
"""
import json
import math
import os
import struct
import zlib

import numpy as np
import pytest

import oracle as O
from pink_amd import capi, fileio, pink


def ints(*v):
    return struct.pack("<%di" % len(v), *v)


IMAGES = np.array([[[1, 2], [3, 4]], [[5, 6], [7, 8]]], np.float32)
# test/SelfOrganizingMapTest/DataIterator.cpp:20-44: version 2, type 0, float32, 2 entries, cartesian, 2-d, 2 x 2
DATA_BYTES = ints(2, 0, 0, 2, 0, 2, 2, 2) + IMAGES.tobytes()


@pytest.mark.parametrize("header", [b"", b"# test header\n# END OF HEADER\n"])
def test_data_file_fixture_of_the_reference_iterator_tests(tmp_path, header):
    # DataIterator.cpp:48-86 (without and with header)
    p = tmp_path / "data.bin"
    p.write_bytes(header + DATA_BYTES)
    d = fileio.DataFile(p)
    assert d.header == header and len(d) == 2 and d.dimensions == [2, 2] and d.layout == 0
    assert [img.ravel().tolist() for img in d] == [[1, 2, 3, 4], [5, 6, 7, 8]]
    q = tmp_path / "out.bin"
    fileio.write_data_file(q, IMAGES, header)
    assert q.read_bytes() == header + DATA_BYTES


def test_header_parser_follows_get_file_header(tmp_path):
    # UtilitiesLib/get_file_header.cpp:10-30: '#' lines until "# END OF HEADER"; without the end marker
    # every leading '#' line belongs to the header; a file without '#' lines has none
    p = tmp_path / "h.bin"
    p.write_bytes(b"# a\n# b\n" + DATA_BYTES)
    assert fileio.DataFile(p).header == b"# a\n# b\n"
    p.write_bytes(b"# a\n# END OF HEADER\n" + DATA_BYTES)
    with open(p, "rb") as f:
        assert fileio.read_header(f) == b"# a\n# END OF HEADER\n" and f.tell() == 20
    p.write_bytes(DATA_BYTES)
    with open(p, "rb") as f:
        assert fileio.read_header(f) == b"" and f.tell() == 0


def test_data_file_errors(tmp_path):
    p = tmp_path / "bad.bin"
    p.write_bytes(ints(1, 0, 0, 2, 0, 2, 2, 2) + IMAGES.tobytes())
    with pytest.raises(fileio.FormatError):
        fileio.DataFile(p)                       # version
    p.write_bytes(ints(2, 1, 0, 2, 0, 2, 2, 2) + IMAGES.tobytes())
    with pytest.raises(fileio.FormatError):
        fileio.DataFile(p)                       # a SOM file is not a data file
    p.write_bytes(ints(2, 0, 1, 2, 0, 2, 2, 2) + IMAGES.tobytes())
    with pytest.raises(fileio.FormatError):
        fileio.DataFile(p)                       # float64
    p.write_bytes(DATA_BYTES[:-4])
    with pytest.raises(fileio.FormatError):
        fileio.DataFile(p)                       # truncated
    p.write_bytes(ints(2, 0, 0))
    with pytest.raises(fileio.FormatError):
        fileio.DataFile(p)


def test_som_file_field_order(tmp_path):
    # SelfOrganizingMapLib/FileIO.h:28-48: header text, then 2 1 0 | 0 <som dimensionality> dims | 0 <neuron
    # dimensionality> dims | data; the layout indices are written as 0 for every layout
    w = np.arange(2 * 3 * 4 * 4, dtype=np.float32)
    p = tmp_path / "som.bin"
    fileio.write_som_file(p, w, "cartesian-2d", (2, 3), (4, 4), b"# made by a test\n# END OF HEADER\n")
    want = b"# made by a test\n# END OF HEADER\n" + ints(2, 1, 0, 0, 2, 2, 3, 0, 2, 4, 4) + w.tobytes()
    assert p.read_bytes() == want
    header, som_dims, neuron_dims, data = fileio.read_som_file(p)
    assert header.startswith(b"# made") and som_dims == [2, 3] and neuron_dims == [4, 4]
    assert data.shape == (6, 16) and np.array_equal(data.ravel(), w)
    # a hexagonal SOM of edge 3 (7 neurons) is written as (3, 3) with layout index 0, FileIO.h:34,40
    h = np.arange(7 * 4, dtype=np.float32)
    fileio.write_som_file(p, h, "hexagonal-2d", (3,), (2, 2))
    assert p.read_bytes() == ints(2, 1, 0, 0, 2, 3, 3, 0, 2, 2, 2) + h.tobytes()
    assert fileio.read_som_file(p)[3].shape == (7, 4)
    # 3-d neurons (channels, edge, edge)
    fileio.write_som_file(p, np.zeros(2 * 2 * 3 * 4 * 4, np.float32), "cartesian-2d", (2, 2), (3, 4, 4))
    assert p.read_bytes()[:48] == ints(2, 1, 0, 0, 2, 2, 2, 0, 3, 3, 4, 4)
    # size of the file: FILE_FORMATS.md:67-71
    assert p.stat().st_size == 4 * 12 + 4 * 2 * 2 * 3 * 4 * 4


def test_mapping_and_rot_flip_files(tmp_path):
    # Pink/main_generic.h:132-145 (mapping header), :147-161 (rot/flip header), :185-195 (records)
    heat = np.arange(3 * 4, dtype=np.float32).reshape(3, 4) / 7
    p = tmp_path / "map.bin"
    fileio.write_mapping_file(p, heat, "cartesian-2d", (2, 2))
    assert p.read_bytes() == ints(2, 2, 0, 3, 0, 2, 2, 2) + heat.tobytes()
    som_dims, got = fileio.read_mapping_file(p)
    assert som_dims == [2, 2] and np.array_equal(got, heat)
    nrot = 360
    best = np.array([[0, 1, 359, 360], [361, 719, 90, 450]], np.uint32)
    q = tmp_path / "rot.bin"
    fileio.write_rot_flip_file(q, best, nrot, "cartesian-2d", (2, 2))
    raw = q.read_bytes()
    assert raw[:28] == ints(2, 3, 2, 0, 2, 2, 2) and len(raw) == 28 + 2 * 4 * 5         # char + float per neuron
    step = np.float32(2.0 * math.pi) / np.float32(nrot)
    off = 28
    for b in best.ravel():
        flip, angle = struct.unpack_from("<bf", raw, off)
        assert flip == int(b) // nrot and angle == np.float32(int(b) % nrot) * step
        off += 5
    _, flips, angles = fileio.read_rot_flip_file(q)
    assert flips.tolist() == [[0, 0, 0, 1], [1, 1, 0, 1]] and angles.shape == (2, 4)


def _shuffle_vectors():
    with open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "shuffle_orders.json")) as f:
        return json.load(f)


@pytest.mark.parametrize("make", [capi.shuffled_order, O.shuffled_order], ids=["library", "oracle"])
def test_shuffled_order_against_the_reference_vectors(make):
    # tests/golden/shuffle_orders.json holds orders taken from the reference's own iterator
    for v in _shuffle_vectors():
        order = make(v["seed"], v["n"])
        assert sorted(order.tolist()) == list(range(v["n"]))
        assert order[:len(v.get("order", v.get("head")))].tolist() == v.get("order", v.get("head")), v
        assert zlib.crc32(order.astype("<u4").tobytes()) == v["crc32"], v
    # test/SelfOrganizingMapTest/DataIteratorShuffled.cpp:19-35: seed 2 leaves two entries in file order
    assert make(2, 2).tolist() == [0, 1]
    assert make(7, 0).size == 0
    # the training loop reseeds with seed + iteration (main_generic.h:83-84): the passes differ
    assert not np.array_equal(make(1234, 50), make(1235, 50))


def test_initial_som_kinds(tmp_path):
    # SOM.h:77-96
    z = fileio.initial_som("cartesian-2d", (3, 2), (4, 4), "zero")
    assert z.shape == (6, 16) and not z.any()
    r = fileio.initial_som("hexagonal-2d", (5,), (2, 4, 4), "random", seed=77)
    assert r.shape == (19, 32)
    assert np.array_equal(r.ravel(), O.fill_random_uniform(19 * 32, 77))
    # Filler probe of the reference with seed 1234
    assert np.allclose(fileio.initial_som("cartesian-2d", (1, 1), (2, 2), "random")[0],
                       [0.191519, 0.497664, 0.622109, 0.817838], atol=1e-6)
    d = fileio.initial_som("cartesian-2d", (2, 2), (3, 3), "random_with_preferred_direction", seed=5)
    plain = O.fill_random_uniform(4 * 9, 5).reshape(4, 9)
    assert np.array_equal(d[:, [0, 4, 8]], np.ones((4, 3), np.float32))
    assert np.array_equal(np.delete(d, [0, 4, 8], axis=1), np.delete(plain, [0, 4, 8], axis=1))
    # three channels: the reference's flat index n * d*d + i*d + i (SOM.h:83-86) has no channel factor, so the
    # diagonals of the first <number of neurons> planes are set, wherever they fall
    d3 = fileio.initial_som("cartesian-2d", (2, 2), (3, 2, 2), "random_with_preferred_direction", seed=5)
    want = O.fill_random_uniform(4 * 12, 5)
    for n_ in range(4):
        for i_ in range(2):
            want[n_ * 4 + i_ * 2 + i_] = 1.0
    assert np.array_equal(d3.ravel(), want)
    # "file": weights behind the header and 9 + <SOM dimensionality> integers
    w = np.arange(4 * 9, dtype=np.float32).reshape(4, 9)
    fileio.write_som_file(tmp_path / "init.bin", w, "cartesian-2d", (2, 2), (3, 3), b"# x\n# END OF HEADER\n")
    assert np.array_equal(fileio.initial_som("cartesian-2d", (2, 2), (3, 3), "file", som_file=tmp_path / "init.bin"), w)
    (tmp_path / "short.bin").write_bytes(b"")
    with pytest.raises(fileio.FormatError):
        fileio.initial_som("cartesian-2d", (2, 2), (3, 3), "file", som_file=tmp_path / "short.bin")
    with pytest.raises(fileio.FormatError):
        fileio.initial_som("cartesian-2d", (2, 2), (3, 3), "spiral")


def test_progress_ticks_of_the_reference_progress_bar():
    # test/UtilitiesTest/ProgressBarTest.cpp:15-26: 100 ticks, 10 prints: valid after 10 increments, not before
    assert fileio.progress_ticks(100, 10) == list(range(10, 100, 10))
    # ProgressBarTest.cpp:52-64: 3 ticks, 2 prints: prints after the second and third increment; the loop
    # checks before the increment, so only tick 2 is seen
    assert fileio.progress_ticks(3, 2) == [2]
    # ProgressBarTest.cpp:39-50: a single tick prints once, after the loop's check
    assert fileio.progress_ticks(1, 10) == []
    # ProgressBarTest.cpp:28-37
    for bad in ((0, 10, 70), (10, 0, 70), (100, 10, 9)):
        with pytest.raises(ValueError):
            fileio.progress_ticks(*bad)


@pytest.mark.gpu
def test_intermediate_storage_writes_the_som_at_the_progress_ticks(tmp_path):
    rng = np.random.default_rng(5)
    images = rng.random((7, 12, 12), dtype=np.float32)
    np_som = rng.random((2, 2, 8, 8), dtype=np.float32)
    fileio.write_data_file(tmp_path / "data.bin", images)
    F = capi.make_update_factors(capi.CARTESIAN, [2, 2], capi.GAUSSIAN, 1.1, 0.2)
    s = O.shape(4, 1, 12, 8, 8, True, 6, O.QUADRATIC, capi.FLOAT)
    order = np.concatenate([O.shuffled_order(9 + i, 7) for i in range(2)])        # 14 ticks, 3 prints: after 5 and 9
    ticks = fileio.progress_ticks(14, 3)
    assert ticks == [5, 9, 13]
    for kind in ("keep", "overwrite"):
        som = pink.SOM(np_som.copy())
        trainer = pink.Trainer(som, pink.GaussianFunctor(1.1, 0.2), number_of_rotations=8, euclidean_distance_dim=6,
                               euclidean_distance_type=pink.FLOAT)
        fileio.train_file(trainer, tmp_path / "data.bin", som, tmp_path / (kind + ".bin"), 2, seed=9,
                          intermediate_storage=kind, max_number_of_progress_prints=3)
        want = np_som.reshape(4, -1).copy()
        done = 0
        for k, t in enumerate(ticks):
            O.train(s, want, images[order[done:t + 1]][:, None], F)
            done = t + 1
            if kind == "keep":
                got = fileio.read_som_file(tmp_path / ("keep_%d.bin" % k))[3]
                assert np.allclose(got, want, rtol=1e-4, atol=1e-6), (k, t)        # float32 weights: 1e-4 relative
        O.train(s, want, images[order[done:]][:, None], F)
        assert np.allclose(fileio.read_som_file(tmp_path / (kind + ".bin"))[3], want, rtol=1e-4, atol=1e-6)
    assert not (tmp_path / "overwrite_0.bin").exists() and not (tmp_path / "keep_3.bin").exists()


@pytest.mark.gpu
def test_train_and_map_from_files_against_the_oracle(tmp_path):
    rng = np.random.default_rng(21)
    images = rng.random((12, 20, 20), dtype=np.float32)
    np_som = rng.random((19, 14, 14), dtype=np.float32)                 # hexagonal, edge 5
    fileio.write_data_file(tmp_path / "data.bin", images, b"# synthetic\n# END OF HEADER\n")
    som = pink.SOM(np_som.copy(), som_layout="hexagonal-2d")
    trainer = pink.Trainer(som, pink.GaussianFunctor(1.1, 0.2), number_of_rotations=16, euclidean_distance_dim=10,
                           euclidean_distance_shape=pink.CIRCULAR, euclidean_distance_type=pink.UINT16)
    counts = fileio.train_file(trainer, tmp_path / "data.bin", som, tmp_path / "som.bin", number_of_iterations=2,
                               shuffle=False)
    # the same two epochs with the oracle
    F = capi.make_update_factors(capi.HEXAGONAL, [5], capi.GAUSSIAN, 1.1, 0.2)
    s = O.shape(19, 1, 20, 14, 16, True, 10, O.CIRCULAR, capi.UINT16)
    want = np_som.reshape(19, -1).copy()
    bmu = np.concatenate([O.train(s, want, images[:, None], F), O.train(s, want, images[:, None], F)])
    # and two shuffled epochs (the default, seed 1234): pass i in the oracle's order for seed + i
    som_s = pink.SOM(np_som.copy(), som_layout="hexagonal-2d")
    trainer_s = pink.Trainer(som_s, pink.GaussianFunctor(1.1, 0.2), number_of_rotations=16, euclidean_distance_dim=10,
                             euclidean_distance_shape=pink.CIRCULAR, euclidean_distance_type=pink.UINT16)
    counts_s = fileio.train_file(trainer_s, tmp_path / "data.bin", som_s, tmp_path / "som_shuffled.bin", 2)
    want_s = np_som.reshape(19, -1).copy()
    bmu_s = np.concatenate([O.train(s, want_s, images[O.shuffled_order(1234 + i, 12)][:, None], F) for i in range(2)])
    assert np.array_equal(counts_s, np.bincount(bmu_s, minlength=19))
    assert np.array_equal(fileio.read_som_file(tmp_path / "som_shuffled.bin")[3].view(np.uint32), want_s.view(np.uint32))
    assert not np.array_equal(want_s, want)
    assert np.array_equal(counts, np.bincount(bmu, minlength=19))
    header, som_dims, neuron_dims, got = fileio.read_som_file(tmp_path / "som.bin")
    assert som_dims == [5, 5] and neuron_dims == [14, 14]
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    # map with the trained SOM read back from its file
    som2 = pink.SOM(got.reshape(19, 14, 14), som_layout="hexagonal-2d")
    mapper = pink.Mapper(som2, number_of_rotations=16, euclidean_distance_dim=10, euclidean_distance_shape=pink.CIRCULAR,
                         euclidean_distance_type=pink.UINT16)
    fileio.map_file(mapper, tmp_path / "data.bin", som2, tmp_path / "map.bin", tmp_path / "rot.bin", 16)
    oheat, obest = O.map_images(s, want, images[:, None])
    _, heat = fileio.read_mapping_file(tmp_path / "map.bin")
    assert np.array_equal(heat.view(np.uint32), oheat.view(np.uint32))
    _, flips, angles = fileio.read_rot_flip_file(tmp_path / "rot.bin")
    assert np.array_equal(flips, obest // 16)
    assert np.array_equal(angles, (obest % 16).astype(np.float32) * (np.float32(2.0 * math.pi) / np.float32(16)))
    assert (tmp_path / "map.bin").stat().st_size == 4 * 8 + 4 * 12 * 19                 # FILE_FORMATS.md:73-77
