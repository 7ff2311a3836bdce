"""Python interface with the names, keyword arguments and defaults of the reference's
pybind11 module `pink` (src/pink/pink.cpp:25-153), over the C ABI of include/pink_hip.h.

    from pink_amd import pink

    som = pink.SOM(np_som, som_layout="cartesian-2d", neuron_layout="cartesian-2d")
    trainer = pink.Trainer(som, pink.GaussianFunctor(1.1, 0.2), number_of_rotations=360,
                           euclidean_distance_dim=32)
    trainer(pink.Data(np_image))
    trainer.update_som()
    heatmap, best_rotations = pink.Mapper(som, euclidean_distance_dim=32)(pink.Data(np_image))

What differs from the reference module:
  * `use_gpu=False` raises: this build has no CPU path (the reference's CPU classes are its own);
  * `Trainer.train(images)` / `Mapper.map(images)` take a whole array of images per call (the
    per-image `__call__` costs one host round trip per image, as in the reference);
  * SOM layouts: "cartesian-2d" and "hexagonal-2d" as in the reference's module (src/pink/DynamicSOM.cpp:22-42);
    "cartesian-1d" and "cartesian-3d" only for this package's command line (`_command_line=True`), whose
    counterpart in the reference builds such SOMs directly (CudaLib/main_gpu.cu:19-25);
  * neuron layouts: "cartesian-2d" (edge, edge) and "cartesian-3d" (channels, edge, edge); the
    reference's spatial transformer throws for "cartesian-1d"
    (SelfOrganizingMapLib/generate_rotated_images.h:36-46), so does this module.
"""
import enum
import math

import numpy as np

from . import capi

__version__ = "2.5 revision pink_amd"


def doc():
    return "PINK python interface"


class Interpolation(enum.IntEnum):
    NEAREST_NEIGHBOR = 0
    BILINEAR = 1


class DataType(enum.IntEnum):
    FLOAT = 0
    UINT16 = 1
    UINT8 = 2


class Layout(enum.IntEnum):
    CARTESIAN = 0
    HEXAGONAL = 1


class EuclideanDistanceShape(enum.IntEnum):
    QUADRATIC = 0
    CIRCULAR = 1


# pybind11's export_values(): the enumerators are module attributes too
NEAREST_NEIGHBOR, BILINEAR = Interpolation.NEAREST_NEIGHBOR, Interpolation.BILINEAR
FLOAT, UINT16, UINT8 = DataType.FLOAT, DataType.UINT16, DataType.UINT8
CARTESIAN, HEXAGONAL = Layout.CARTESIAN, Layout.HEXAGONAL
QUADRATIC, CIRCULAR = EuclideanDistanceShape.QUADRATIC, EuclideanDistanceShape.CIRCULAR

exception = capi.PinkError


class GaussianFunctor:
    """UtilitiesLib/DistributionFunctor.cpp:29-37 (float arithmetic)."""

    def __init__(self, sigma=1.1, damping=0.2):
        self.sigma = float(sigma)
        self.damping = float(damping)

    def __call__(self, distance):
        s, d = np.float32(self.sigma), np.float32(self.damping)
        x = np.float32(distance) / s
        return float(d / (s * np.sqrt(np.float32(2.0) * np.float32(math.pi))) * np.exp(np.float32(-0.5) * x * x))


class LibraryFunctor:
    """A neighbourhood function of UtilitiesLib/DistributionFunctor.cpp:19-59 by kind (capi.STEP, GAUSSIAN,
    UNITY_GAUSSIAN, MEXICAN_HAT): the library evaluates it with the reference's float arithmetic.  Not in
    the reference's Python module (which exports GaussianFunctor only); the command line selects them."""

    def __init__(self, kind, sigma, damping):
        self.kind, self.sigma, self.damping = int(kind), float(sigma), float(damping)


def _as_float32_copy(buffer, what):
    a = np.asarray(buffer)
    if a.dtype != np.float32:
        raise TypeError("%s must be a float32 buffer" % what)     # py::arg().noconvert()
    return np.array(a, dtype=np.float32, order="C", copy=True)     # the reference copies into a std::vector


class Data:
    """pink.Data (src/pink/DynamicData.cpp:15-41): one image, copied from a float32 buffer."""

    def __init__(self, buffer, data_type="float32", layout="cartesian-2d"):
        if data_type != "float32":
            raise exception(-1, "data-type not supported")
        ndim = {"cartesian-1d": 1, "cartesian-2d": 2, "cartesian-3d": 3}.get(layout)
        if ndim is None:
            raise exception(-1, "layout " + layout + " is not supported")
        self._a = _as_float32_copy(buffer, "data")
        if self._a.ndim != ndim:
            raise exception(-1, "data shape does not match layout " + layout)
        self.data_type, self.layout = data_type, layout

    def __array__(self, dtype=None, copy=None):
        return self._a if dtype in (None, np.float32) else self._a.astype(dtype)

    @property
    def shape(self):
        return self._a.shape


def _image_geometry(shape, layout, what):
    """(channels, edge) of a cartesian-2d (edge, edge) or cartesian-3d (channels, edge, edge) shape."""
    if layout == "cartesian-2d" and len(shape) == 2:
        channels, h, w = 1, shape[0], shape[1]
    elif layout == "cartesian-3d" and len(shape) == 3:
        channels, h, w = shape
    elif layout == "cartesian-1d":
        raise exception(-1, "Not implemented yet.")     # generate_rotated_images.h:36-46
    else:
        raise exception(-1, what + " shape does not match layout " + layout)
    if h != w:
        raise exception(-1, what + " must be quadratic")
    return int(channels), int(h)


class SOM:
    """pink.SOM (src/pink/DynamicSOM.cpp:12-44): shape = SOM dimensions followed by the neuron
    shape; "hexagonal-2d" takes the number of neurons as its one SOM dimension."""

    def __init__(self, buffer, data_type="float32", som_layout="cartesian-2d", neuron_layout="cartesian-2d",
                 _command_line=False):
        if data_type != "float32":
            raise exception(-1, "data-type not supported")
        self._a = _as_float32_copy(buffer, "som")
        shape = self._a.shape
        if som_layout == "cartesian-2d" or (_command_line and som_layout in ("cartesian-1d", "cartesian-3d")):
            rank = int(som_layout[10])
            if len(shape) < rank + 1:
                raise exception(-1, "som shape does not match layout " + som_layout)
            self._layout, self._dims, neuron_shape = capi.CARTESIAN, list(shape[:rank]), shape[rank:]
        elif som_layout == "hexagonal-2d":
            if len(shape) < 2:
                raise exception(-1, "som shape does not match layout " + som_layout)
            dim = self.hexagonal_dim_from_size(shape[0])
            self._layout, self._dims, neuron_shape = capi.HEXAGONAL, [dim], shape[1:]
        else:
            raise exception(-1, "SOM layout " + som_layout + " is not supported")
        if neuron_layout not in ("cartesian-1d", "cartesian-2d", "cartesian-3d"):
            raise exception(-1, "neuron layout " + neuron_layout + " is not supported")
        self.data_type, self.som_layout, self.neuron_layout = data_type, som_layout, neuron_layout
        self.neuron_shape = tuple(int(v) for v in neuron_shape)
        self.number_of_neurons = capi.som_size(self._layout, self._dims)
        if self.number_of_neurons * int(np.prod(self.neuron_shape)) != self._a.size:
            raise exception(-1, "som shape does not match its layouts")

    @staticmethod
    def hexagonal_dim_from_size(size):
        """HexagonalLayout::get_dim_from_size: the odd edge length d with d*d - r*(r+1) = size, r = (d-1)/2."""
        d = 1
        while d * d - ((d - 1) // 2) * ((d - 1) // 2 + 1) < size:
            d += 2
        if d * d - ((d - 1) // 2) * ((d - 1) // 2 + 1) != size:
            raise exception(-1, "number of neurons does not fit a hexagonal layout")
        return d

    def get_som_layout(self):
        return self.som_layout

    def __array__(self, dtype=None, copy=None):
        return self._a if dtype in (None, np.float32) else self._a.astype(dtype)

    @property
    def shape(self):
        return self._a.shape

    def _rows(self):
        return self._a.reshape(self.number_of_neurons, -1)


class _Device:
    """The context behind a Trainer or Mapper; created at the first image, whose size the
    constructors do not know (as the C++ classes of pink_amd/host do)."""

    def __init__(self, som, number_of_rotations, use_flip, interpolation, use_gpu, euclidean_distance_dim,
                 euclidean_distance_shape, euclidean_distance_type, update_factors):
        if not use_gpu:
            raise exception(-4, "this build has no CPU path: use_gpu=False is not supported")
        if euclidean_distance_dim is None:
            raise TypeError("missing required argument: euclidean_distance_dim")
        self.som = som
        self.channels, self.neuron_dim = _image_geometry(som.neuron_shape, som.neuron_layout, "neuron")
        self.args = dict(num_rot=int(number_of_rotations), use_flip=bool(use_flip), ed_dim=int(euclidean_distance_dim),
                         ed_shape=int(euclidean_distance_shape), ed_type=int(euclidean_distance_type),
                         interpolation=int(interpolation), update_factors=update_factors)
        self.ctx = None
        self.image_dim = None
        self.update_factors = update_factors
        self.counts_base = None
        # argument errors surface at construction, as in the reference; the image size is not known
        # yet and takes no part in these checks, so the neuron size stands in for it
        a = self.args
        capi.check_config(som.number_of_neurons, self.channels, self.neuron_dim, self.neuron_dim, a["num_rot"],
                          a["use_flip"], a["ed_dim"], a["ed_shape"], a["ed_type"], a["interpolation"])

    def _context(self, image_dim):
        return capi.Context(self.som.number_of_neurons, self.channels, image_dim, self.neuron_dim, **self.args)

    def update_counts(self):
        """How often each neuron was the best match, over every context this object has had."""
        counts = np.zeros(self.som.number_of_neurons, np.uint32) if self.ctx is None else self.ctx.update_counts()
        return counts if self.counts_base is None else counts + self.counts_base

    def for_images(self, images, layout):
        images = np.ascontiguousarray(images, np.float32)
        per_image_ndim = 3 if self.channels > 1 or layout == "cartesian-3d" else 2
        shape = images.shape[-per_image_ndim:]
        channels, image_dim = _image_geometry(shape, "cartesian-3d" if per_image_ndim == 3 else "cartesian-2d", "image")
        if channels != self.channels:
            raise exception(-1, "image and neuron channel counts differ")
        if self.ctx is None or image_dim != self.image_dim:
            weights = self.ctx.get_som() if self.ctx is not None else self.som._rows()
            if self.ctx is not None:
                if self.update_factors is not None:           # the counts of the context that goes away
                    self.counts_base = self.update_counts()
                self.ctx.close()
            self.ctx = self._context(image_dim)
            self.ctx.set_som(weights)
            self.image_dim = image_dim
        return images.reshape(-1, channels, image_dim, image_dim)


class Trainer:
    """pink.Trainer (src/pink/pink.cpp:113-135, SelfOrganizingMapLib/Trainer.h:201-335)."""

    def __init__(self, som, distribution_function=None, verbosity=0, number_of_rotations=360, use_flip=True,
                 max_update_distance=-1.0, interpolation=Interpolation.BILINEAR, use_gpu=True,
                 euclidean_distance_dim=None, euclidean_distance_shape=EuclideanDistanceShape.QUADRATIC,
                 euclidean_distance_type=DataType.UINT8):
        if distribution_function is None:
            distribution_function = GaussianFunctor(1.1, 0.2)
        self.update_factors = self._update_factors(som, distribution_function, float(max_update_distance))
        self._dev = _Device(som, number_of_rotations, use_flip, interpolation, use_gpu, euclidean_distance_dim,
                            euclidean_distance_shape, euclidean_distance_type, self.update_factors)
        self._som = som
        self.verbosity = verbosity

    @staticmethod
    def _update_factors(som, function, max_update_distance):
        """TrainerCommon's constructor loop (Trainer.h:69-76): f(distance) where the distance is
        below max_update_distance (or that is not positive), else 0."""
        if type(function) in (GaussianFunctor, LibraryFunctor):
            # the library evaluates these functors itself, with the reference's float arithmetic
            kind = capi.GAUSSIAN if type(function) is GaussianFunctor else function.kind
            return capi.make_update_factors(som._layout, som._dims, kind, function.sigma, function.damping,
                                            max_update_distance)
        dist = capi.layout_distances(som._layout, som._dims)
        values = {float(d): np.float32(function(float(d))) for d in np.unique(dist)}
        factors = np.vectorize(lambda d: values[float(d)], otypes=[np.float32])(dist)
        if max_update_distance > 0:
            factors[~(dist < np.float32(max_update_distance))] = 0.0
        return np.ascontiguousarray(factors, np.float32)

    def __call__(self, data):
        """One image (Trainer.h:263-304).  Returns nothing, like the reference, and does not wait for
        the GPU: the image is copied, and images are trained in order a launch group at a time (when the group
        is full, or when update_som() or get_update_info() follows); those two wait for the result."""
        images = self._dev.for_images(np.asarray(data)[None], getattr(data, "layout", "cartesian-2d"))
        self._dev.ctx.train(images, want_bmu=False)

    def train(self, images, layout="cartesian-2d"):
        """Many images in order, one call: image k+1 sees the weights left by image k.  Returns the
        best-matching neuron of every image."""
        images = self._dev.for_images(images, layout)
        return self._dev.ctx.train(images)

    def update_som(self):
        """Device weights -> the SOM object (Trainer.h:306-309)."""
        if self._dev.ctx is not None:
            self._som._rows()[...] = self._dev.ctx.get_som()

    @property
    def update_info(self):
        """TrainerCommon::m_update_info: how often each neuron was the best match (counted on the device)."""
        return self._dev.update_counts()

    def get_update_info(self):
        return self.update_info


class Mapper:
    """pink.Mapper (src/pink/pink.cpp:137-152, SelfOrganizingMapLib/Mapper.h:129-230): snapshots the
    SOM at construction."""

    def __init__(self, som, verbosity=0, number_of_rotations=360, use_flip=True, interpolation=Interpolation.BILINEAR,
                 use_gpu=True, euclidean_distance_dim=None, euclidean_distance_shape=EuclideanDistanceShape.QUADRATIC,
                 euclidean_distance_type=DataType.UINT8):
        if som.neuron_layout != "cartesian-2d" and som.neuron_layout != "cartesian-3d":
            raise exception(-1, "neuron layout " + som.neuron_layout + " is not supported")
        snapshot = SOM(np.asarray(som), som.data_type, som.som_layout, som.neuron_layout, _command_line=True)
        self._dev = _Device(snapshot, number_of_rotations, use_flip, interpolation, use_gpu, euclidean_distance_dim,
                            euclidean_distance_shape, euclidean_distance_type, None)
        self.verbosity = verbosity

    def __call__(self, data):
        """One image: (heatmap, best rotation per neuron) as two lists, like the bound
        std::tuple<std::vector<float>, std::vector<uint32_t>> (Mapper.h:181-208)."""
        heat, best = self.map(np.asarray(data)[None], getattr(data, "layout", "cartesian-2d"))
        return heat[0].tolist(), best[0].tolist()

    def map(self, images, layout="cartesian-2d"):
        """Many images, one call: (n, N) float32 heatmaps (square-rooted) and (n, N) uint32 best rotations."""
        images = self._dev.for_images(images, layout)
        return self._dev.ctx.map(images)
