"""The five synthetic workloads the benchmark and the parity tests run.

Each workload fixes the SOM geometry, the distance region and type, the rotation
count, the neighbourhood function and a deterministic image generator.  Images are
float32 in [0, 1]; SOMs start as the reference's `--init random` does: a
std::mt19937 seeded stream mapped to U[0,1) floats
(src/UtilitiesLib/Filler.h:17-25, src/SelfOrganizingMapLib/SOM.h:79-80).
"""
from dataclasses import dataclass

import numpy as np

from . import capi


@dataclass(frozen=True)
class Workload:
    name: str
    mode: str               # "train" | "map"
    layout: int             # capi.CARTESIAN | capi.HEXAGONAL
    som_dims: tuple
    channels: int
    image_dim: int
    neuron_dim: int
    ed_dim: int
    ed_shape: int
    ed_type: int
    num_rot: int
    use_flip: bool
    functor: int
    sigma: float
    damping: float
    n_images: int
    seed: int

    @property
    def som_size(self):
        if self.layout == capi.HEXAGONAL:
            d = self.som_dims[0]
            r = (d - 1) // 2
            return d * d - r * (r + 1)
        return int(np.prod(self.som_dims))

    @property
    def R(self):
        return self.num_rot * (2 if self.use_flip else 1)

    @property
    def neuron_size(self):
        return self.channels * self.neuron_dim ** 2

    @property
    def image_size(self):
        return self.channels * self.image_dim ** 2


WORKLOADS = {
    "cfg0": Workload("cfg0_train_f32_10x10", "train", capi.CARTESIAN, (10, 10), 1, 64, 44, 32, capi.QUADRATIC,
                     capi.FLOAT, 360, True, capi.GAUSSIAN, 1.1, 0.2, 2000, 20260),
    "cfg1": Workload("cfg1_map_u8_10x10", "map", capi.CARTESIAN, (10, 10), 1, 64, 44, 32, capi.QUADRATIC,
                     capi.UINT8, 360, True, capi.GAUSSIAN, 1.1, 0.2, 20000, 20261),
    "cfg2": Workload("cfg2_train_u16_hex21", "train", capi.HEXAGONAL, (21, 21), 1, 150, 106, 75, capi.CIRCULAR,
                     capi.UINT16, 360, True, capi.GAUSSIAN, 1.5, 0.1, 10000, 20262),
    "cfg3": Workload("cfg3_train_f32_40x40_3ch", "train", capi.CARTESIAN, (40, 40), 3, 100, 70, 50, capi.QUADRATIC,
                     capi.FLOAT, 180, True, capi.MEXICAN_HAT, 2.0, 0.05, 5000, 20263),
    "cfg4": Workload("cfg4_train_u8_8x8_28px", "train", capi.CARTESIAN, (8, 8), 1, 28, 28, 28, capi.QUADRATIC,
                     capi.UINT8, 4, True, capi.GAUSSIAN, 1.0, 0.3, 60000, 20264),
}


def mt19937_uniform(n, seed):
    """n floats of std::uniform_real_distribution<float>(0,1) over std::mt19937(seed) (libstdc++:
    one 32-bit word per float, float(word) / 2^32, a value rounding to 1 replaced by the float below 1)."""
    raw = np.random.RandomState(seed)._bit_generator.random_raw(n).astype(np.uint32)
    v = raw.astype(np.float32) / np.float32(4294967296.0)
    v[v >= 1.0] = np.nextafter(np.float32(1.0), np.float32(0.0))
    return v


def initial_som(w, seed=1234):
    return mt19937_uniform(w.som_size * w.neuron_size, seed).reshape(w.som_size, w.neuron_size)


def _blob_fields(rng, n, dim, kmin, kmax, amp, axes=(2.0, 12.0)):
    """n fields of kmin..kmax elliptical Gaussian blobs with random centre, orientation and axes."""
    yy, xx = np.meshgrid(np.arange(dim, dtype=np.float32), np.arange(dim, dtype=np.float32), indexing="ij")
    out = np.zeros((n, dim, dim), np.float32)
    count = rng.integers(kmin, kmax + 1, n)
    for b in range(kmax):
        on = (count > b).astype(np.float32)[:, None, None]
        cx = rng.uniform(0.2 * dim, 0.8 * dim, n).astype(np.float32)[:, None, None]
        cy = rng.uniform(0.2 * dim, 0.8 * dim, n).astype(np.float32)[:, None, None]
        th = rng.uniform(0, np.pi, n).astype(np.float32)[:, None, None]
        sa = rng.uniform(axes[0], axes[1], n).astype(np.float32)[:, None, None] * np.float32(dim / 64.0)
        sb = rng.uniform(axes[0], axes[1], n).astype(np.float32)[:, None, None] * np.float32(dim / 64.0)
        a = amp(rng, n).astype(np.float32)[:, None, None]
        dx, dy = xx[None] - cx, yy[None] - cy
        u = dx * np.cos(th) + dy * np.sin(th)
        v = -dx * np.sin(th) + dy * np.cos(th)
        out += on * a * np.exp(-0.5 * ((u / sa) ** 2 + (v / sb) ** 2))
    return out


def _uniform_amp(rng, n):
    return rng.uniform(0.3, 1.0, n)


def _lognormal_amp(rng, n):
    return rng.lognormal(-1.0, 0.8, n)


def images(w, n=None, seed=None, chunk=2048):
    """n images of workload w, shape (n, C, I, I), float32 in [0, 1]."""
    n = w.n_images if n is None else n
    rng = np.random.default_rng(w.seed if seed is None else seed)
    out = np.empty((n, w.channels, w.image_dim, w.image_dim), np.float32)
    for s in range(0, n, chunk):
        m = min(chunk, n - s)
        key = w.name[:4]
        if key in ("cfg0", "cfg1"):
            f = _blob_fields(rng, m, w.image_dim, 1, 3, _uniform_amp)
            f += rng.normal(0, 0.02, f.shape).astype(np.float32)
            f = np.clip(f, 0, 1)
            f /= np.sqrt((f.astype(np.float64) ** 2).sum((1, 2), keepdims=True)).astype(np.float32) + np.float32(1e-12)
            out[s:s + m, 0] = f
        elif key == "cfg2":
            f = _blob_fields(rng, m, w.image_dim, 1, 4, _lognormal_amp)
            f = np.clip(f, 0, None)
            f /= f.max((1, 2), keepdims=True) + np.float32(1e-12)     # peak-normalised: uses the uint16 range
            out[s:s + m, 0] = f
        elif key == "cfg3":
            common = _blob_fields(rng, m, w.image_dim, 1, 3, _uniform_amp)
            for c in range(w.channels):
                own = _blob_fields(rng, m, w.image_dim, 1, 3, _uniform_amp)
                out[s:s + m, c] = np.clip(np.float32(np.sqrt(0.7)) * common + np.float32(np.sqrt(0.3)) * own, 0, 1)
        else:  # cfg4: strokes and blobs with uint8-valued pixels
            f = _blob_fields(rng, m, w.image_dim, 0, 2, _uniform_amp, axes=(1.5, 5.0))
            for _ in range(2):       # straight strokes
                x0, y0 = rng.uniform(4, 24, (2, m))
                ang = rng.uniform(0, np.pi, m)
                ln = rng.uniform(4, 12, m)
                tt = np.linspace(-0.5, 0.5, 24, dtype=np.float32)
                px = np.clip(np.rint(x0[:, None] + ln[:, None] * tt * np.cos(ang)[:, None]), 0, w.image_dim - 1).astype(int)
                py = np.clip(np.rint(y0[:, None] + ln[:, None] * tt * np.sin(ang)[:, None]), 0, w.image_dim - 1).astype(int)
                f[np.arange(m)[:, None], py, px] = 1.0
            f = np.clip(f, 0, 1)
            out[s:s + m, 0] = np.floor(f * 255.0) / np.float32(255.0)
    return out


def update_factors(w):
    return capi.make_update_factors(w.layout, w.som_dims, w.functor, w.sigma, w.damping, -1.0)


def make_context(w, trainer=None, ed_type=None, **kw):
    """A device context shaped for workload w (a trainer for "train" workloads), optionally with
    another distance type."""
    trainer = (w.mode == "train") if trainer is None else trainer
    return capi.Context(w.som_size, w.channels, w.image_dim, w.neuron_dim, w.num_rot, w.use_flip, w.ed_dim,
                        w.ed_shape, w.ed_type if ed_type is None else ed_type,
                        update_factors(w) if trainer else None, **kw)
