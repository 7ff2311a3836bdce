"""python -m pink_amd.cli: the reference's command line (UtilitiesLib/InputData.cpp:84-497) over this
package's file loops."""
import numpy as np
import pytest

import oracle as O
from pink_amd import capi, cli, fileio, pink


def _data(tmp_path, n=6, edge=64, channels=0, seed=1):
    rng = np.random.default_rng(seed)
    shape = (n, edge, edge) if channels == 0 else (n, channels, edge, edge)
    images = rng.random(shape, dtype=np.float32)
    fileio.write_data_file(tmp_path / "data.bin", images)
    return images


def test_defaults_and_derived_sizes(tmp_path):
    _data(tmp_path)
    c = cli.InputData().parse(["--train", str(tmp_path / "data.bin"), str(tmp_path / "som.bin")]).finish()
    # InputData.cpp:46-82 and :452-476: 10 x 10 cartesian, 360 rotations with flip, uint8 distances,
    # neuron edge 2 * 64 / sqrt(2) + 1 = 91, distance edge 64 * sqrt(2) / 2 = 45
    assert (c.som_width, c.som_height, c.som_size, c.layout) == (10, 10, 100, "cartesian")
    assert (c.number_of_rotations, c.use_flip, c.seed, c.init) == (360, True, 1234, "zero")
    assert c.euclidean_distance_type == pink.DataType.UINT8 and c.shuffle_data_input
    assert c.neuron_dim == 91 and c.neuron_dimension == [91, 91] and c.euclidean_distance_dim == 45
    assert (c.sigma, c.damping, c.distribution_function) == (1.1, 0.2, "gaussian")
    # no rotations: the neuron is the image; circular regions keep the image edge
    c = cli.InputData().parse(["--train", str(tmp_path / "data.bin"), "x.bin", "-n", "1"]).finish()
    assert c.neuron_dim == 64 and c.euclidean_distance_dim == 64
    c = cli.InputData().parse(["--train", str(tmp_path / "data.bin"), "x.bin", "--euclidean-distance-shape",
                               "circular"]).finish()
    assert c.neuron_dim == 91 and c.euclidean_distance_dim == 64


def test_options(tmp_path):
    _data(tmp_path, channels=3, edge=20)
    argv = ["--som-width", "5", "--som-height=5", "--layout", "hexagonal", "-d", "14", "--euclidean-distance-dimension", "8",
            "-n", "8", "--flip-off", "-s", "7", "-x", "random", "--num-iter", "3", "-p", "4", "--inter-store", "keep",
            "--dist-func", "mexicanhat", "2.0", "0.05", "--max-update-distance", "2.5", "--euclidean-distance-type",
            "uint16", "--input-shuffle-off", "--numthreads", "3", "--b1", "128", "--verbose",
            "--map", str(tmp_path / "data.bin"), "map.bin", "som.bin", "--store-rot-flip", "rot.bin"]
    c = cli.InputData().parse(argv).finish()
    assert (c.layout, c.som_size, c.som_dims(), c.som_layout()) == ("hexagonal", 19, (5,), "hexagonal-2d")
    assert c.neuron_dimension == [3, 14, 14] and c.neuron_layout() == "cartesian-3d" and c.euclidean_distance_dim == 8
    assert (c.number_of_rotations, c.use_flip, c.seed, c.number_of_iterations) == (8, False, 7, 3)
    assert (c.max_number_of_progress_prints, c.intermediate_storage) == (4, "keep")
    assert (c.distribution_function, c.sigma, c.damping, c.max_update_distance) == ("mexicanhat", 2.0, 0.05, 2.5)
    assert c.euclidean_distance_type == pink.DataType.UINT16 and not c.shuffle_data_input and c.verbose
    assert (c.execution_path, c.result_filename, c.som_filename) == ("map", "map.bin", "som.bin")
    assert c.init == "file" and c.write_rot_flip and c.rot_flip_filename == "rot.bin"      # --map forces FILEINIT
    f = c.distribution()
    assert (f.kind, f.sigma, f.damping) == (capi.MEXICAN_HAT, 2.0, 0.05)
    # --progress goes through std::atoi (InputData.cpp:181): leading digits count, anything else is 0
    for text, want in (("12abc", 12), ("abc", 0), (" 7", 7), ("2.9", 2)):
        c = cli.InputData().parse(["--train", str(tmp_path / "data.bin"), "x.bin", "--progress", text])
        assert c.max_number_of_progress_prints == want


def test_som_dimensionality_follows_height_and_depth(tmp_path):
    """InputData.cpp:429-430 counts a SOM dimension for the width, one for a height above 1 and one for a depth
    above 1; the SOM takes that many of (width, height, depth) (SOM.h:25-43)."""
    _data(tmp_path)
    base = ["--train", str(tmp_path / "data.bin"), "x.bin"]
    c = cli.InputData().parse(base + ["--som-width", "4", "--som-height", "3", "--som-depth", "2"]).finish()
    assert (c.som_size, c.som_layout(), c.som_dims()) == (24, "cartesian-3d", (4, 3, 2))
    c = cli.InputData().parse(base + ["--som-width", "7", "--som-height", "1"]).finish()
    assert (c.som_size, c.som_layout(), c.som_dims()) == (7, "cartesian-1d", (7,))
    # a height of 1 with a depth above 1 is two-dimensional to the reference: width x 1
    c = cli.InputData().parse(base + ["--som-width", "5", "--som-height", "1", "--som-depth", "3"]).finish()
    assert (c.som_layout(), c.som_dims()) == ("cartesian-2d", (5, 1))
    with pytest.raises(cli.UsageError) as e:
        cli.InputData().parse(base + ["-l", "hexagonal", "--som-width", "5", "--som-height", "5", "--som-depth", "2"]).finish()
    assert "For hexagonal layout som-depth must be equal to 1." in str(e.value)


@pytest.mark.parametrize("argv,text", [
    ([], "Unknown execution path."),
    (["--train", "DATA"], "Missing arguments for --train option."),
    (["--map", "DATA", "a.bin", "--verbose"], "Missing arguments for --map option."),
    (["--train", "DATA", "a.bin", "-n", "6"], "Number of rotations must be 1 or a multiple of 4"),
    (["--train", "DATA", "a.bin", "--num-iter", "0"], "Number of iterations must be larger than 0"),
    (["--train", "DATA", "a.bin", "-l", "ring"], "Unknown layout option RING"),
    (["--train", "DATA", "a.bin", "-l", "hexagonal", "--som-width", "4", "--som-height", "4"],
     "For hexagonal layout only odd dimension supported."),
    (["--train", "DATA", "a.bin", "-l", "hexagonal", "--som-width", "5", "--som-height", "3"],
     "For hexagonal layout som-width must be equal to som-height."),
    (["--train", "DATA", "a.bin", "--som-width", "1"], "som-width must be > 1."),
    (["--train", "DATA", "a.bin", "--max-update-distance", "0"], "max-update-distance must be positive."),
    (["--train", "DATA", "a.bin", "--dist-func", "gaussian", "1.0"], "Missing arguments for --dist-func option."),
    (["--train", "DATA", "a.bin", "-d", "20", "--euclidean-distance-dimension", "21"],
     "euclidean distance dimension must be equal or smaller than neuron dimension."),
    (["--train", "DATA", "a.bin", "--pbc"], "Periodic boundary conditions are not supported in version 2."),
    (["--train", "DATA", "a.bin", "-e", "8"], "Unknown option -e"),          # the short-option string has no 'e'
    (["--train", "DATA", "a.bin", "--cuda-off"], "no CPU path"),
    (["--train", "missing.bin", "a.bin"], "Error opening"),
])
def test_errors(tmp_path, argv, text):
    _data(tmp_path)
    argv = [str(tmp_path / "data.bin") if a == "DATA" else a for a in argv]
    with pytest.raises(cli.UsageError) as e:
        cli.InputData().parse(argv).finish()
    assert text in str(e.value)


@pytest.mark.gpu
def test_train_then_map_from_the_command_line(tmp_path):
    images = _data(tmp_path, n=9, edge=16, seed=4)
    data, som_file = str(tmp_path / "data.bin"), str(tmp_path / "som.bin")
    assert cli.main(["--train", data, som_file, "--som-width", "3", "--som-height", "3", "-n", "8", "-x", "random",
                     "-s", "11", "--num-iter", "2", "--euclidean-distance-type", "uint16", "--dist-func",
                     "unitygaussian", "1.3", "0.4"]) == 0
    # the same run with the oracle: neuron 2 * 16 / sqrt(2) + 1 = 23, region 16 * sqrt(2) / 2 = 11
    F = capi.make_update_factors(capi.CARTESIAN, [3, 3], capi.UNITY_GAUSSIAN, 1.3, 0.4)
    s = O.shape(9, 1, 16, 23, 8, True, 11, O.QUADRATIC, capi.UINT16)
    want = O.fill_random_uniform(9 * 23 * 23, 11).reshape(9, -1)
    for i in range(2):
        O.train(s, want, images[O.shuffled_order(11 + i, 9)][:, None], F)
    _, som_dims, neuron_dims, got = fileio.read_som_file(som_file)
    assert som_dims == [3, 3] and neuron_dims == [23, 23]
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    assert cli.main(["--map", data, str(tmp_path / "map.bin"), som_file, "--som-width", "3", "--som-height", "3",
                     "-n", "8", "--euclidean-distance-type", "uint16", "--store-rot-flip", str(tmp_path / "rot.bin")]) == 0
    oheat, obest = O.map_images(s, want, images[:, None])
    _, heat = fileio.read_mapping_file(tmp_path / "map.bin")
    assert np.array_equal(heat.view(np.uint32), oheat.view(np.uint32))
    _, flips, _ = fileio.read_rot_flip_file(tmp_path / "rot.bin")
    assert np.array_equal(flips, obest // 8)
    assert cli.main(["--map", data, str(tmp_path / "map.bin")]) == 1          # reports, does not raise


@pytest.mark.gpu
@pytest.mark.parametrize("dims", [(3, 2, 2), (5,)])
def test_train_then_map_one_and_three_dimensional_soms(tmp_path, dims):
    """--som-depth above 1 and --som-height 1: the reference's command line builds CartesianLayout<3> and <1>
    SOMs (CudaLib/main_gpu.cu:19-25); the layout only enters through the neurons' distances
    (CartesianLayout.h:84-123) and the file headers."""
    images = _data(tmp_path, n=7, edge=12, seed=9)
    data, som_file = str(tmp_path / "data.bin"), str(tmp_path / "som.bin")
    whd = list(dims) + [1] * (3 - len(dims))
    size = ["--som-width", str(whd[0]), "--som-height", str(whd[1]), "--som-depth", str(whd[2])]
    assert cli.main(["--train", data, som_file] + size + ["-n", "4", "-x", "random", "-s", "3", "--input-shuffle-off",
                                                          "--euclidean-distance-type", "float"]) == 0
    n = int(np.prod(dims))
    F = capi.make_update_factors(capi.CARTESIAN, list(dims), capi.GAUSSIAN, 1.1, 0.2)
    # the distances behind F are the reference's: sqrt of the summed squared position differences, positions
    # as CartesianLayout<N>::get_position gives them
    D = capi.layout_distances(capi.CARTESIAN, list(dims))
    if len(dims) == 3:
        def pos(i):
            z = i // dims[0] // dims[1]
            return (i % dims[1], (i - z * dims[0] * dims[1]) // dims[1], z)
    else:
        def pos(i):
            return (i,)
    want_D = np.array([[np.sqrt(np.float32(sum((a - b) ** 2 for a, b in zip(pos(i), pos(j))))) for j in range(n)]
                       for i in range(n)], np.float32)
    assert np.array_equal(D.reshape(n, n), want_D)
    s = O.shape(n, 1, 12, 17, 4, True, 8, O.QUADRATIC, capi.FLOAT)      # neuron 2 * 12 / sqrt(2) + 1 = 17, region 8
    want = O.fill_random_uniform(n * 17 * 17, 3).reshape(n, -1)
    O.train(s, want, images[:, None], F)
    _, som_dims, neuron_dims, got = fileio.read_som_file(som_file)
    assert som_dims == list(dims) and neuron_dims == [17, 17]
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    assert cli.main(["--map", data, str(tmp_path / "map.bin"), som_file] + size + ["-n", "4", "--euclidean-distance-type",
                                                                                  "float"]) == 0
    oheat, _ = O.map_images(s, want, images[:, None])
    map_dims, heat = fileio.read_mapping_file(tmp_path / "map.bin")
    assert map_dims == list(dims)
    assert np.array_equal(heat.view(np.uint32), oheat.view(np.uint32))
