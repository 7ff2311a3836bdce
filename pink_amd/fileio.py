"""The reference's binary file formats (FILE_FORMATS.md:53-85): the data on either side of the
train / map path.

  data file     <header> 2 0 <data-type> <entries> <layout> <dimensionality> <dims...> <float32 data>
  SOM file      <header> 2 1 <data-type> <som layout> <dimensionality> <dims...>
                         <neuron layout> <dimensionality> <dims...> <float32 data>
  mapping file  2 2 <data-type> <entries> <som layout> <dimensionality> <dims...> <float32 N per entry>
  rot/flip file 2 3 <entries> <som layout> <dimensionality> <dims...> <(char flip, float32 angle) N per entry>

All header fields are 32-bit integers.  An optional text header of lines starting with '#' ends
with the line "# END OF HEADER" (UtilitiesLib/get_file_header.cpp:10-30).  Writers follow the
reference's own writers field by field (SelfOrganizingMapLib/FileIO.h:20-49,
Pink/main_generic.h:132-161,185-195), including that they write layout index 0 for every SOM
layout (FileIO.h:34, main_generic.h:135) and give a hexagonal SOM as (d, d).
"""
import math
import struct

import numpy as np

VERSION = 2
FILE_DATA, FILE_SOM, FILE_MAPPING, FILE_ROT_FLIP = 0, 1, 2, 3
END_OF_HEADER = b"# END OF HEADER"


class FormatError(ValueError):
    pass


def read_header(f):
    """get_file_header: the leading '#' lines up to and including "# END OF HEADER"; the stream is
    left behind them (or where it was when there are none)."""
    header = b""
    pos = f.tell()
    while True:
        line = f.readline()
        if not line or not line.startswith(b"#"):
            break
        pos = f.tell()
        header += line.rstrip(b"\n") + b"\n"
        if line.rstrip(b"\n") == END_OF_HEADER:
            break
    f.seek(pos)
    return header


def _ints(f, n):
    raw = f.read(4 * n)
    if len(raw) != 4 * n:
        raise FormatError("file ends inside its header")
    return list(struct.unpack("<%di" % n, raw))


def _layout(f):
    layout, dimensionality = _ints(f, 2)
    if not 1 <= dimensionality <= 3:
        raise FormatError("dimensionality %d is not supported" % dimensionality)
    return layout, _ints(f, dimensionality)


def _check(version, file_type, want_type, data_type=0):
    if version != VERSION:
        raise FormatError("file format version %d is not supported (expected %d)" % (version, VERSION))
    if file_type != want_type:
        raise FormatError("file type %d where %d was expected" % (file_type, want_type))
    if data_type != 0:
        raise FormatError("data type %d is not supported (only 0, float32)" % data_type)


class DataFile:
    """A data file for training or mapping, memory-mapped: `images` has shape (entries, *dims)
    (the reference reads it entry by entry, SelfOrganizingMapLib/DataIterator.h)."""

    def __init__(self, path):
        with open(path, "rb") as f:
            self.header = read_header(f)
            version, file_type, data_type, self.number_of_entries = _ints(f, 4)
            _check(version, file_type, FILE_DATA, data_type)
            self.layout, self.dimensions = _layout(f)
            offset = f.tell()
            f.seek(0, 2)
            size = f.tell()
        per_entry = int(np.prod(self.dimensions))
        if size - offset < 4 * per_entry * self.number_of_entries:
            raise FormatError("data file is shorter than its header announces")
        self.images = np.memmap(path, np.float32, "r", offset, (self.number_of_entries, *self.dimensions))

    def __len__(self):
        return self.number_of_entries

    def __iter__(self):
        return iter(self.images)


def write_data_file(path, images, header=b""):
    """images: (entries, edge, edge) or (entries, channels, edge, edge) float32."""
    images = np.ascontiguousarray(images, np.float32)
    if images.ndim not in (2, 3, 4):
        raise FormatError("images must have 1 to 3 dimensions per entry")
    with open(path, "wb") as f:
        f.write(header)
        dims = images.shape[1:]
        f.write(struct.pack("<%di" % (6 + len(dims)), VERSION, FILE_DATA, 0, images.shape[0], 0, len(dims), *dims))
        f.write(images.tobytes())


def _som_dims(som_layout, number_of_neurons_or_dims):
    if som_layout == "hexagonal-2d":
        d = number_of_neurons_or_dims[0]
        return [d, d]
    return list(number_of_neurons_or_dims)


def write_som_file(path, weights, som_layout, som_dims, neuron_dims, header=b""):
    """write(SOM, filename), FileIO.h:20-49.  som_dims: (w, h) or (w, h, d) for "cartesian-*d", the
    edge length (d,) for "hexagonal-2d"; weights: number_of_neurons * prod(neuron_dims) floats."""
    weights = np.ascontiguousarray(weights, np.float32)
    sd, nd = _som_dims(som_layout, list(som_dims)), list(neuron_dims)
    with open(path, "wb") as f:
        f.write(header)
        f.write(struct.pack("<%di" % (7 + len(sd) + len(nd)), VERSION, FILE_SOM, 0, 0, len(sd), *sd, 0, len(nd), *nd))
        f.write(weights.tobytes())


def read_som_file(path):
    """-> (header, som_dims, neuron_dims, weights (number_of_neurons, prod(neuron_dims))).  The number of
    neurons is what is left of the file, so files of hexagonal SOMs (written as (d, d)) read too."""
    with open(path, "rb") as f:
        header = read_header(f)
        version, file_type, data_type = _ints(f, 3)
        _check(version, file_type, FILE_SOM, data_type)
        _, som_dims = _layout(f)
        _, neuron_dims = _layout(f)
        data = np.frombuffer(f.read(), np.float32)
    per_neuron = int(np.prod(neuron_dims))
    if per_neuron == 0 or data.size % per_neuron:
        raise FormatError("SOM file does not hold whole neurons")
    return header, som_dims, neuron_dims, data.reshape(-1, per_neuron).copy()


def write_mapping_file(path, heatmaps, som_layout, som_dims):
    """main_generic.h:132-145,185-187: the (entries, N) heatmaps of Mapper::operator()."""
    heatmaps = np.ascontiguousarray(heatmaps, np.float32)
    sd = _som_dims(som_layout, list(som_dims))
    with open(path, "wb") as f:
        f.write(struct.pack("<%di" % (6 + len(sd)), VERSION, FILE_MAPPING, 0, heatmaps.shape[0], 0, len(sd), *sd))
        f.write(heatmaps.tobytes())


def read_mapping_file(path):
    with open(path, "rb") as f:
        version, file_type, data_type, entries = _ints(f, 4)
        _check(version, file_type, FILE_MAPPING, data_type)
        _, som_dims = _layout(f)
        data = np.frombuffer(f.read(), np.float32)
    if entries == 0 or data.size % entries:
        raise FormatError("mapping file does not hold whole entries")
    return som_dims, data.reshape(entries, -1).copy()


ROT_FLIP_RECORD = np.dtype([("flip", np.int8), ("angle", "<f4")])       # packed: 5 bytes per neuron


def write_rot_flip_file(path, best_rotations, number_of_rotations, som_layout, som_dims):
    """main_generic.h:147-161,189-195: per neuron a char `flipped` and the float32 angle
    (best % num_rot) * float(2 pi) / num_rot of the best variant index."""
    best = np.ascontiguousarray(best_rotations, np.uint32)
    sd = _som_dims(som_layout, list(som_dims))
    step = np.float32(2.0 * math.pi) / np.float32(number_of_rotations)
    rec = np.empty(best.shape, ROT_FLIP_RECORD)
    rec["flip"] = (best // number_of_rotations).astype(np.int8)
    rec["angle"] = (best % number_of_rotations).astype(np.float32) * step
    with open(path, "wb") as f:
        f.write(struct.pack("<%di" % (5 + len(sd)), VERSION, FILE_ROT_FLIP, best.shape[0], 0, len(sd), *sd))
        f.write(rec.tobytes())


def read_rot_flip_file(path):
    with open(path, "rb") as f:
        version, file_type, entries = _ints(f, 3)
        _check(version, file_type, FILE_ROT_FLIP)
        _, som_dims = _layout(f)
        rec = np.frombuffer(f.read(), ROT_FLIP_RECORD)
    if entries == 0 or rec.size % entries:
        raise FormatError("rot/flip file does not hold whole entries")
    rec = rec.reshape(entries, -1)
    return som_dims, rec["flip"].copy(), rec["angle"].copy()


def initial_som(som_layout, som_dims, neuron_dims, init="zero", seed=1234, som_file=None):
    """The SOM the reference starts training from (SOM.h:69-98), as (number_of_neurons, prod(neuron_dims))
    float32: "zero"; "random" = fill_random_uniform(seed); "random_with_preferred_direction" = the same with
    the diagonals of the first <number of neurons> planes of neuron_dims[-1] x neuron_dims[-1] set to 1
    (one per neuron for single-channel neurons); "file" = the
    weights of `som_file`, found as the reference finds them: behind the text header and 9 +
    <SOM dimensionality> integers (SOM.h:94, which assumes two neuron dimensions)."""
    from . import capi
    layout = capi.HEXAGONAL if som_layout == "hexagonal-2d" else capi.CARTESIAN
    n = capi.som_size(layout, np.asarray(list(som_dims), np.uint32))
    if n == 0:
        raise FormatError("invalid SOM dimensions")
    per_neuron = int(np.prod(neuron_dims))
    if init == "zero":
        return np.zeros((n, per_neuron), np.float32)
    if init in ("random", "random_with_preferred_direction"):
        som = capi.fill_random_uniform(n * per_neuron, seed).reshape(n, per_neuron)
        if init == "random_with_preferred_direction":
            # SOM.h:83-86 indexes the flat weights as n * d*d + i * d + i for n < number of neurons, without
            # the channel count: for C channels that is the diagonal of the first n planes of d x d, not one
            # plane per neuron
            d = int(neuron_dims[-1])
            flat = som.reshape(-1)
            i = np.arange(d)
            flat[(np.arange(n)[:, None] * (d * d) + i * d + i).ravel()] = 1.0
        return som
    if init == "file":
        with open(som_file, "rb") as f:
            read_header(f)
            f.seek(4 * (9 + len(_som_dims(som_layout, list(som_dims)))), 1)
            data = np.frombuffer(f.read(4 * n * per_neuron), np.float32)
        if data.size != n * per_neuron:
            raise FormatError("SOM file is shorter than the SOM")
        return data.reshape(n, per_neuron).copy()
    raise FormatError("unknown SOM initialisation " + repr(init))


def progress_ticks(number_of_ticks, max_number_of_progress_prints=10, width=70):
    """The ticks t (images trained before, counted over all passes) at which the training loop finds
    ProgressBar::valid() true after training image t, i.e. where it writes an intermediate SOM
    (main_generic.h:78,86-90 with UtilitiesLib/ProgressBar.h:21-52,72-75)."""
    if number_of_ticks < 1:
        raise ValueError("ProgressBar: number_of_iterations must be larger than 0")
    if max_number_of_progress_prints < 1:
        raise ValueError("ProgressBar: max number of progress prints must be larger than 0")
    prints = min(number_of_ticks, max_number_of_progress_prints)
    if width < prints:
        raise ValueError("ProgressBar: width must be equal or larger than number of progress prints")
    section = number_of_ticks // prints
    next_valid = section + (1 if number_of_ticks % prints else 0)
    out = []
    for tick in range(number_of_ticks):          # `tick` increments have happened when image `tick` is trained
        if tick == next_valid:
            out.append(tick)
            next_valid += section
    return out


def train_file(trainer, data_path, som, result_path, number_of_iterations=1, header=b"", shuffle=True, seed=1234,
               intermediate_storage="off", max_number_of_progress_prints=10):
    """The training loop of Pink --train (main_generic.h:75-110): `number_of_iterations` passes over the
    data file, pass i in the order of DataIteratorShuffled(seed + i) -- or in file order with
    shuffle=False (--input-shuffle-off) -- then the SOM file.  intermediate_storage "overwrite" or "keep"
    also writes the SOM at the progress ticks of the reference, into the result file or into
    <result>_<count>.<ext> (main_generic.h:88-104).  `trainer` and `som` are pink_amd.pink objects."""
    from . import capi
    if intermediate_storage not in ("off", "overwrite", "keep"):
        raise ValueError("unknown intermediate storage type " + repr(intermediate_storage))
    data = DataFile(data_path)
    n = len(data)
    layout = "cartesian-3d" if len(data.dimensions) == 3 else "cartesian-2d"
    step = max(1, (1 << 28) // max(1, 4 * int(np.prod(data.dimensions))))      # images gathered per call
    stops = progress_ticks(n * number_of_iterations, max_number_of_progress_prints) if intermediate_storage != "off" and n else []
    result_path = str(result_path)
    count = 0

    def store_intermediate():
        nonlocal count
        name = result_path
        if intermediate_storage == "keep":
            dot = name.rfind(".")            # std::string::insert at find_last_of("."): npos throws in the reference
            if dot < 0:
                raise ValueError("result file name has no '.' to put the count in front of")
            name = name[:dot] + "_%d" % count + name[dot:]
            count += 1
        trainer.update_som()
        write_som_file(name, np.asarray(som), som.som_layout, som._dims, som.neuron_shape, header)

    for i in range(number_of_iterations):
        order = capi.shuffled_order(seed + i, n) if shuffle else None
        # the pass is cut after every image that is followed by an intermediate SOM, and into calls of `step` images
        cuts = sorted({t - i * n + 1 for t in stops if i * n <= t < (i + 1) * n} | {n})
        begin = 0
        for cut in cuts:
            while begin < cut:
                end = min(cut, begin + step)
                trainer.train(data.images[begin:end] if order is None else data.images[order[begin:end]], layout)
                begin = end
            if cut - 1 + i * n in stops:
                store_intermediate()
    trainer.update_som()
    write_som_file(result_path, np.asarray(som), som.som_layout, som._dims, som.neuron_shape, header)
    return trainer.get_update_info()


def map_file(mapper, data_path, som, result_path, rot_flip_path=None, number_of_rotations=360):
    """The mapping loop of Pink --map (main_generic.h:122-197): the heatmap of every image, and
    optionally the best rotation / flip per neuron."""
    data = DataFile(data_path)
    layout = "cartesian-3d" if len(data.dimensions) == 3 else "cartesian-2d"
    heat, best = mapper.map(data.images, layout)
    write_mapping_file(result_path, heat, som.som_layout, som._dims)
    if rot_flip_path:
        write_rot_flip_file(rot_flip_path, best, number_of_rotations, som.som_layout, som._dims)
    return heat, best
