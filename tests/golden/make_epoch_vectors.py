"""Writes tests/golden/epoch_<cfg>.npz: what one whole epoch of a training workload leaves behind when the
CPU oracle (oracle/pink_oracle.c, the restatement of Trainer.h:133-186 over the loop of
main_generic.h:80-89) trains it, image after image with free-running weights.

    python tests/golden/make_epoch_vectors.py cfg2 [threads]      # about an hour on 8 cores
    python tests/golden/make_epoch_vectors.py cfg3 [threads]

The oracle takes minutes to hours for these epochs, so it runs once, here, and the GPU test
(tests/test_gpu_epoch.py) trains the same epoch on the device and compares with what this file holds:

    bmu            best-matching neuron of every image, in order
    som_sha256     SHA-256 of the final weights (bit-equality)
    checkpoints    SHA-256 of the weights after every `piece` images (to say where a run departs)
    neuron_sums    float64 sum of every neuron's final weights
    slice_index, slice_values   every `stride`-th final weight (the 1e-4 gate is applied to these and the sums)
    images_sha256, factors_sha256, som0_sha256   the inputs, so that a host whose libm or numpy builds other
                   inputs is told apart from a device that computes other outputs

Nothing of the reference is read or run here; the inputs are pink_amd.synthetic's.
"""
import hashlib
import os
import sys
import time

import numpy as np

sys.path.insert(0, os.path.join(os.path.dirname(os.path.abspath(__file__)), "..", ".."))
import oracle as O                      # noqa: E402
from pink_amd import synthetic          # noqa: E402

PIECE = 250
STRIDE = 997                            # a prime: the slice walks through all rows and columns


def sha(a):
    return hashlib.sha256(np.ascontiguousarray(a).tobytes()).hexdigest()


def main():
    name = sys.argv[1]
    if len(sys.argv) > 2:
        O.set_num_threads(int(sys.argv[2]))
    w = synthetic.WORKLOADS[name]
    n = int(os.environ.get("EPOCH_IMAGES", w.n_images))
    imgs = synthetic.images(w, n)
    som = synthetic.initial_som(w)
    F = synthetic.update_factors(w)
    s = O.shape(w.som_size, w.channels, w.image_dim, w.neuron_dim, w.num_rot, w.use_flip, w.ed_dim,
                w.ed_shape, w.ed_type)
    meta = dict(images_sha256=sha(imgs), factors_sha256=sha(F), som0_sha256=sha(som))
    bmu, checkpoints = [], []
    t0 = time.time()
    for i in range(0, n, PIECE):
        bmu.append(O.train(s, som, imgs[i:i + PIECE], F))
        checkpoints.append(sha(som))
        print("%s: %d of %d images, %.0f s" % (name, min(i + PIECE, n), n, time.time() - t0), flush=True)
    flat = som.reshape(-1)
    idx = np.arange(0, flat.size, STRIDE, dtype=np.int64)
    out = os.path.join(os.path.dirname(os.path.abspath(__file__)), "epoch_%s.npz" % name)
    np.savez_compressed(out, workload=w.name, n_images=n, piece=PIECE, bmu=np.concatenate(bmu).astype(np.uint16),
                        som_sha256=sha(som), checkpoints=np.array(checkpoints),
                        neuron_sums=som.astype(np.float64).sum(1), slice_index=idx, slice_values=flat[idx],
                        **meta)
    print("wrote", out, os.path.getsize(out), "bytes")


if __name__ == "__main__":
    main()
