"""`Pink --train / --map` with the reference's options (UtilitiesLib/InputData.cpp:84-497), run
through this package:

    python -m pink_amd.cli --train <data> <result> [options]
    python -m pink_amd.cli --map <data> <result> <som> [options]

The option names, defaults, derived sizes and error texts follow InputData.cpp; the loops are
pink_amd.fileio.train_file / map_file (Pink/main_generic.h:57-198).  What differs: there is no CPU
path here (--cuda-off is refused), and --numthreads / --b1 are accepted and ignored.
"""
import math
import sys

from . import capi, fileio, pink


class UsageError(Exception):
    """pink::exception of the argument parser."""


LONG_OPTIONS = {   # name -> takes an argument (InputData.cpp:84-115)
    "neuron-dimension": True, "euclidean-distance-dimension": True, "layout": True, "seed": True, "numrot": True,
    "numthreads": True, "init": True, "progress": True, "version": False, "help": False, "dist-func": True,
    "som-width": True, "num-iter": True, "flip-off": False, "cuda-off": False, "verbose": False,
    "interpolation": True, "train": True, "map": True, "inter-store": True, "b1": True,
    "max-update-distance": True, "som-height": True, "som-depth": True, "pbc": False, "store-rot-flip": True,
    "euclidean-distance-type": True, "input-shuffle-off": False, "euclidean-distance-shape": True,
}
# the short-option string of the reference, "vd:l:s:n:t:x:p:a:hf:" (InputData.cpp:121): it has no 'e',
# so the distance dimension can only be given by its long name
SHORT_OPTIONS = {"v": ("version", False), "d": ("neuron-dimension", True), "l": ("layout", True), "s": ("seed", True),
                 "n": ("numrot", True), "t": ("numthreads", True), "x": ("init", True), "p": ("progress", True),
                 "h": ("help", False), "f": ("dist-func", True)}


def _atoi(text):
    """std::atoi: optional sign and leading digits, 0 when there are none."""
    import re
    m = re.match(r"\s*([+-]?\d+)", text)
    return int(m.group(1)) if m else 0


def _uint32(text):
    try:
        value = int(text)
    except ValueError:
        raise UsageError("Invalid unsigned integer " + repr(text))
    if not 0 <= value < 2 ** 32:
        raise UsageError("Invalid unsigned integer " + repr(text))
    return value


class InputData:
    """The fields of the reference's InputData that the train and map paths use, with its defaults
    (InputData.cpp:46-82)."""

    def __init__(self):
        self.verbose = False
        self.som_width, self.som_height, self.som_depth = 10, 10, 1
        self.neuron_dim = 0
        self.euclidean_distance_dim = 0
        self.layout = "cartesian"
        self.seed = 1234
        self.number_of_rotations = 360
        self.init = "zero"
        self.som_filename = None
        self.number_of_iterations = 1
        self.max_number_of_progress_prints = 10
        self.use_flip = True
        self.use_gpu = True
        self.interpolation = pink.Interpolation.BILINEAR
        self.execution_path = None
        self.data_filename = self.result_filename = None
        self.intermediate_storage = "off"
        self.distribution_function = "gaussian"
        self.sigma, self.damping = 1.1, 0.2
        self.max_update_distance = -1.0
        self.use_pbc = False
        self.write_rot_flip = False
        self.rot_flip_filename = None
        self.euclidean_distance_type = pink.DataType.UINT8
        self.shuffle_data_input = True
        self.euclidean_distance_shape = pink.EuclideanDistanceShape.QUADRATIC
        # derived from the data file
        self.number_of_data_entries = 0
        self.data_dimension = None
        self.neuron_dimension = None
        self.som_size = 0

    # -- the option loop ---------------------------------------------------------------------
    def parse(self, argv):
        args = list(argv)
        i = 0

        def following(count, option):
            # the file names of --train / --map and the two numbers of --dist-func are plain words
            # after the option's own argument; one that is missing or starts with '-' is an error
            nonlocal i
            words = []
            for _ in range(count):
                if i >= len(args) or args[i].startswith("-"):
                    raise UsageError("Missing arguments for --%s option." % option)
                words.append(args[i])
                i += 1
            return words

        while i < len(args):
            word = args[i]
            i += 1
            if word.startswith("--"):
                name, eq, value = word[2:].partition("=")
                if name not in LONG_OPTIONS:
                    raise UsageError("Unknown option " + word)
                takes = LONG_OPTIONS[name]
            elif word.startswith("-") and len(word) > 1:
                if word[1] not in SHORT_OPTIONS:
                    raise UsageError("Unknown option " + word)
                name, takes = SHORT_OPTIONS[word[1]]
                eq, value = ("=", word[2:]) if len(word) > 2 else ("", "")
            else:
                continue                                   # getopt_long skips words that are not options
            if takes and not eq:
                if i >= len(args):
                    raise UsageError("Missing arguments for --%s option." % name)
                value = args[i]
                i += 1
            self._apply(name, value, following)
        return self

    def _apply(self, name, value, following):
        upper = value.upper() if isinstance(value, str) else value
        if name == "neuron-dimension":
            self.neuron_dim = _uint32(value)
        elif name == "euclidean-distance-dimension":
            self.euclidean_distance_dim = _uint32(value)
        elif name == "som-width":
            self.som_width = _uint32(value)
        elif name == "som-height":
            self.som_height = _uint32(value)
        elif name == "som-depth":
            self.som_depth = _uint32(value)
        elif name == "num-iter":
            self.number_of_iterations = _uint32(value)
            if self.number_of_iterations == 0:
                raise UsageError("Number of iterations must be larger than 0")
        elif name == "layout":
            if upper not in ("CARTESIAN", "HEXAGONAL"):
                raise UsageError("Unknown layout option " + upper)
            self.layout = upper.lower()
        elif name == "seed":
            self.seed = _uint32(value)
        elif name == "progress":
            self.max_number_of_progress_prints = _atoi(value)      # std::atoi (InputData.cpp:181)
        elif name == "numrot":
            self.number_of_rotations = _uint32(value)
            if self.number_of_rotations == 0 or (self.number_of_rotations != 1 and self.number_of_rotations % 4):
                raise UsageError("Number of rotations must be 1 or a multiple of 4")
        elif name in ("numthreads", "b1"):
            pass                                           # host threads / CUDA block size: nothing to set here
        elif name == "init":
            if upper in ("ZERO", "RANDOM", "RANDOM_WITH_PREFERRED_DIRECTION"):
                self.init = upper.lower()
            else:
                self.init, self.som_filename = "file", value
        elif name == "flip-off":
            self.use_flip = False
        elif name == "cuda-off":
            self.use_gpu = False
        elif name == "verbose":
            self.verbose = True
        elif name == "interpolation":
            if upper == "NEAREST_NEIGHBOR":
                self.interpolation = pink.Interpolation.NEAREST_NEIGHBOR
            elif upper == "BILINEAR":
                self.interpolation = pink.Interpolation.BILINEAR
            else:
                raise UsageError("Unknown interpolation option " + upper)
        elif name == "train":
            self.execution_path = "train"
            self.data_filename = value
            if value.startswith("-"):
                raise UsageError("Missing arguments for --train option.")
            (self.result_filename,) = following(1, "train")
        elif name == "map":
            self.execution_path = "map"
            self.data_filename = value
            if value.startswith("-"):
                raise UsageError("Missing arguments for --map option.")
            self.result_filename, self.som_filename = following(2, "map")
        elif name == "inter-store":
            if upper not in ("OFF", "OVERWRITE", "KEEP"):
                raise UsageError("Unknown intermediate storage option " + upper)
            self.intermediate_storage = upper.lower()
        elif name == "max-update-distance":
            self.max_update_distance = float(value)
            if self.max_update_distance <= 0.0:
                raise UsageError("max-update-distance must be positive.")
        elif name == "pbc":
            self.use_pbc = True
        elif name == "store-rot-flip":
            self.write_rot_flip, self.rot_flip_filename = True, value
        elif name == "euclidean-distance-type":
            if upper not in ("FLOAT", "UINT16", "UINT8"):
                raise UsageError("Unknown intermediate storage option " + upper)      # the reference's text
            self.euclidean_distance_type = getattr(pink.DataType, upper)
        elif name == "input-shuffle-off":
            self.shuffle_data_input = False
        elif name == "euclidean-distance-shape":
            if upper not in ("QUADRATIC", "CIRCULAR"):
                raise UsageError("Unknown euclidean distance shape " + upper)
            self.euclidean_distance_shape = getattr(pink.EuclideanDistanceShape, upper)
        elif name == "dist-func":
            if upper not in ("GAUSSIAN", "UNITYGAUSSIAN", "MEXICANHAT"):
                raise UsageError("Unknown intermediate storage option " + upper)      # the reference's text
            self.distribution_function = upper.lower()
            sigma, damping = following(2, "dist-func")
            self.sigma, self.damping = float(sigma), float(damping)
        elif name == "version":
            print("pink_amd, C ABI version %d" % capi.lib().pink_hip_abi_version())
            raise SystemExit(0)
        elif name == "help":
            print(__doc__)
            raise SystemExit(0)

    # -- what follows the option loop (InputData.cpp:394-497) -----------------------------------
    def finish(self):
        if self.execution_path == "map":
            self.init = "file"
        elif self.execution_path is None:
            raise UsageError("Unknown execution path.")
        if self.layout == "hexagonal":
            if self.use_pbc:
                raise UsageError("Periodic boundary conditions are not supported for hexagonal layout.")
            if (self.som_width - 1) % 2:
                raise UsageError("For hexagonal layout only odd dimension supported.")
            if self.som_width != self.som_height:
                raise UsageError("For hexagonal layout som-width must be equal to som-height.")
            if self.som_depth != 1:
                raise UsageError("For hexagonal layout som-depth must be equal to 1.")
            self.som_size = capi.som_size(capi.HEXAGONAL, [self.som_width, self.som_height])
        else:
            self.som_size = self.som_width * self.som_height * self.som_depth
        if self.som_width < 2:
            raise UsageError("som-width must be > 1.")
        if self.som_height < 1:
            raise UsageError("som-height must be > 0.")
        if self.som_depth < 1:
            raise UsageError("som-depth must be > 0.")
        try:
            data = fileio.DataFile(self.data_filename)
        except OSError:
            raise UsageError("Error opening " + str(self.data_filename))
        self.number_of_data_entries = len(data)
        self.data_dimension = list(data.dimensions)
        edge = self.data_dimension[1] if len(self.data_dimension) > 1 else self.data_dimension[0]
        if self.neuron_dim == 0:
            self.neuron_dim = edge
            if self.number_of_rotations != 1:
                self.neuron_dim = int(2 * edge / math.sqrt(2.0) + 1)
        self.neuron_dimension = list(self.data_dimension)
        if len(self.neuron_dimension) == 2:
            self.neuron_dimension = [self.neuron_dim, self.neuron_dim]
        elif len(self.neuron_dimension) == 3:
            self.neuron_dimension[1] = self.neuron_dimension[2] = self.neuron_dim
        if self.euclidean_distance_dim == 0:
            self.euclidean_distance_dim = edge
            if self.number_of_rotations != 1 and self.euclidean_distance_shape == pink.EuclideanDistanceShape.QUADRATIC:
                self.euclidean_distance_dim = int(self.euclidean_distance_dim * math.sqrt(2.0) / 2)
        if self.number_of_data_entries == 0:
            raise UsageError("Number of data entries must be larger than 0.")
        if self.euclidean_distance_dim > self.neuron_dim:
            raise UsageError("euclidean distance dimension must be equal or smaller than neuron dimension.")
        if self.use_pbc:
            raise UsageError("Periodic boundary conditions are not supported in version 2.")
        if not self.use_gpu:
            raise UsageError("this build has no CPU path: --cuda-off is not supported")
        return self

    # -- objects of the path ------------------------------------------------------------------------
    def som_dimensionality(self):
        """InputData.cpp:429-430: one, plus one for a height above 1, plus one for a depth above 1; the SOM
        then takes that many of (width, height, depth) in this order (SOM.h:25-43,71-72), so a height of 1
        with a depth above 1 gives a width x 1 SOM, as in the reference."""
        return 1 + (self.som_height > 1) + (self.som_depth > 1)

    def som_layout(self):
        return "hexagonal-2d" if self.layout == "hexagonal" else "cartesian-%dd" % self.som_dimensionality()

    def som_dims(self):
        if self.layout == "hexagonal":
            return (self.som_width,)
        return (self.som_width, self.som_height, self.som_depth)[:self.som_dimensionality()]

    def neuron_layout(self):
        return "cartesian-3d" if len(self.neuron_dimension) == 3 else "cartesian-2d"

    def distribution(self):
        """get_distribution_function (InputData.cpp:657-669): the functor named by --dist-func."""
        kind = {"gaussian": capi.GAUSSIAN, "unitygaussian": capi.UNITY_GAUSSIAN, "mexicanhat": capi.MEXICAN_HAT}
        if self.distribution_function == "mexicanhat" and self.sigma <= 0:
            raise UsageError("MexicanHatFunctor: sigma <= 0 not defined.")     # DistributionFunctor.cpp:50
        return pink.LibraryFunctor(kind[self.distribution_function], self.sigma, self.damping)


def run(argv):
    """Parse, then train or map; returns the InputData."""
    import numpy as np
    cfg = InputData().parse(argv).finish()
    header = b""
    if cfg.init == "file":
        with open(cfg.som_filename, "rb") as f:
            header = fileio.read_header(f)
    weights = fileio.initial_som(cfg.som_layout(), cfg.som_dims(), cfg.neuron_dimension, cfg.init, cfg.seed,
                                 cfg.som_filename)
    shape = ((cfg.som_size,) if cfg.layout == "hexagonal" else cfg.som_dims()) + tuple(cfg.neuron_dimension)
    som = pink.SOM(np.ascontiguousarray(weights).reshape(shape), som_layout=cfg.som_layout(),
                   neuron_layout=cfg.neuron_layout(), _command_line=True)
    common = dict(verbosity=int(cfg.verbose), number_of_rotations=cfg.number_of_rotations, use_flip=cfg.use_flip,
                  interpolation=cfg.interpolation, euclidean_distance_dim=cfg.euclidean_distance_dim,
                  euclidean_distance_shape=cfg.euclidean_distance_shape,
                  euclidean_distance_type=cfg.euclidean_distance_type)
    if cfg.execution_path == "train":
        trainer = pink.Trainer(som, cfg.distribution(), max_update_distance=cfg.max_update_distance, **common)
        counts = fileio.train_file(trainer, cfg.data_filename, som, cfg.result_filename, cfg.number_of_iterations,
                                   header, cfg.shuffle_data_input, cfg.seed, cfg.intermediate_storage,
                                   cfg.max_number_of_progress_prints)
        if cfg.verbose:
            print("\n  Number of updates of each neuron:\n\n%s\n" % counts)
    else:
        mapper = pink.Mapper(som, **common)
        fileio.map_file(mapper, cfg.data_filename, som, cfg.result_filename,
                        cfg.rot_flip_filename if cfg.write_rot_flip else None, cfg.number_of_rotations)
    return cfg


def main(argv=None):
    try:
        run(sys.argv[1:] if argv is None else argv)
    except (UsageError, pink.exception, fileio.FormatError) as e:
        print("PINK exception: %s" % e, file=sys.stderr)
        return 1
    return 0


if __name__ == "__main__":
    sys.exit(main())
