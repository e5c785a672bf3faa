"""Seeded synthetic inputs for tests and benchmarks (no datasets are available).

The delta-mask generator follows the structurally sparse generator of the
reference benchmark (benchmark/input_handlers.py:69-86: a random field, a
neighbourhood pooling and a threshold) in the form the benchmark
configurations specify: a uniform random field, Gaussian blur with sigma =
4 px (reflect padding), thresholded so that exactly round(p * H * W) pixels
are active; the mask is shared by all channels.
"""
import numpy as np
import torch
from scipy.ndimage import gaussian_filter


def blob_mask(h: int, w: int, density: float, seed: int, sigma: float = 4.0) -> np.ndarray:
    """uint8 (H, W) mask with exactly round(density * H * W) active pixels in smooth blobs."""
    g = torch.Generator().manual_seed(int(seed))
    u = torch.rand((h, w), generator=g, dtype=torch.float64).numpy()
    f = gaussian_filter(u, sigma=sigma, mode="reflect")
    k = int(round(density * h * w))
    mask = np.zeros(h * w, dtype=np.uint8)
    if k > 0:
        idx = np.argpartition(-f.reshape(-1), k - 1)[:k]
        mask[idx] = 1
    return mask.reshape(h, w)


def gaussian_delta(n, c, h, w, density, std, seed) -> "tuple[torch.Tensor, torch.Tensor]":
    """Delta ~ N(0, std) on a blob mask, 0 elsewhere.  Returns (delta NCHW fp32, mask uint8 (N,1,H,W))."""
    g = torch.Generator().manual_seed(int(seed) + 7919)
    masks = np.stack([blob_mask(h, w, density, seed * 131 + b) for b in range(n)])
    m = torch.from_numpy(masks).view(n, 1, h, w)
    d = torch.randn((n, c, h, w), generator=g) * std
    return d * m.float(), m


def event_voxel_delta(n, bins, h, w, density, seed) -> "tuple[torch.Tensor, torch.Tensor]":
    """Delta voxel grid of an event camera step: on a blob mask each bin gets
    Poisson(lambda=2) event counts with random polarity, scaled by 0.1."""
    g = torch.Generator().manual_seed(int(seed) + 104729)
    masks = np.stack([blob_mask(h, w, density, seed * 131 + b) for b in range(n)])
    m = torch.from_numpy(masks).view(n, 1, h, w)
    counts = torch.poisson(torch.full((n, bins, h, w), 2.0), generator=g)
    sign = torch.randint(0, 2, (n, bins, h, w), generator=g).float() * 2.0 - 1.0
    return counts * sign * 0.1 * m.float(), m


class MovingEdges:
    """Moving-edge event generator: random line segments that translate 1-3 px per step; the
    pixels a segment sweeps in a step fire events.  Yields (delta NCHW fp32, mask uint8) per
    step for a 4-channel event image: positive / negative counts and their latest timestamps."""

    def __init__(self, h, w, segments=17, seed=0, thickness=1):
        self.h, self.w, self.thickness = h, w, thickness
        self.rng = np.random.default_rng(seed)
        r = self.rng
        self.p0 = np.stack([r.uniform(0, h, segments), r.uniform(0, w, segments)], 1)
        ang = r.uniform(0, 2 * np.pi, segments)
        length = r.uniform(0.15, 0.5, segments) * min(h, w)
        self.d = np.stack([np.sin(ang), np.cos(ang)], 1) * length[:, None]
        vang = r.uniform(0, 2 * np.pi, segments)
        speed = r.uniform(1.0, 3.0, segments)
        self.v = np.stack([np.sin(vang), np.cos(vang)], 1) * speed[:, None]
        self.pol = r.integers(0, 2, segments)
        self.t = 0

    def _raster(self):
        m = np.zeros((self.h, self.w), dtype=np.int8)
        pol = np.zeros((self.h, self.w), dtype=np.int8)
        for p0, d, pl in zip(self.p0, self.d, self.pol):
            npts = int(np.hypot(*d)) * 2 + 2
            ts = np.linspace(0.0, 1.0, npts)
            ys = np.round(p0[0] + ts * d[0]).astype(int) % self.h
            xs = np.round(p0[1] + ts * d[1]).astype(int) % self.w
            for dy in range(self.thickness):
                m[(ys + dy) % self.h, xs] = 1
                pol[(ys + dy) % self.h, xs] = pl
        return m, pol

    def step(self):
        before, _ = self._raster()
        self.p0 = self.p0 + self.v
        self.t += 1
        after, pol = self._raster()
        fired = ((after == 1) & (before == 0)) | ((after == 0) & (before == 1))
        counts = self.rng.poisson(2.0, size=(self.h, self.w)).astype(np.float32) + 1.0
        d = np.zeros((1, 4, self.h, self.w), dtype=np.float32)
        d[0, 0] = fired * (pol == 1) * counts
        d[0, 1] = fired * (pol == 0) * counts
        d[0, 2] = fired * (pol == 1) * 0.1 * self.t
        d[0, 3] = fired * (pol == 0) * 0.1 * self.t
        mask = fired.astype(np.uint8)[None, None]
        return torch.from_numpy(d) * 0.1, torch.from_numpy(mask)


def random_events(n_events: int, width: int, height: int, t0: float, t1: float, seed: int,
                  density: float = 0.05, polarity=(0.0, 1.0), t_unit: float = 1e9) -> np.ndarray:
    """(n, 4) float64 rows (t, x, y, p) sorted by time, the row layout of the reference's event
    files: stamps uniform in [t0, t1] seconds, stored in 1/t_unit seconds (nanoseconds by default);
    pixels drawn from a smooth blob mask of the given density; polarity from `polarity`."""
    rng = np.random.default_rng(seed)
    ys, xs = np.nonzero(blob_mask(height, width, density, seed))
    pick = rng.integers(0, ys.size, size=n_events)
    t = np.sort(rng.uniform(t0, t1, size=n_events)) * t_unit
    p = rng.choice(np.asarray(polarity, dtype=np.float64), size=n_events)
    return np.stack([t, xs[pick].astype(np.float64), ys[pick].astype(np.float64), p], axis=1)


def he_normal_conv_weight(cout, cin, k, seed) -> torch.Tensor:
    """He-normal (std sqrt(2 / (cin * k * k))) conv weight, OIHW."""
    g = torch.Generator().manual_seed(int(seed))
    return torch.randn((cout, cin, k, k), generator=g) * (2.0 / (cin * k * k)) ** 0.5


def seed_module_(module: torch.nn.Module, seed: int, bias_std: float = 0.05):
    """Deterministic random init of every conv weight (He-normal) and bias of a module."""
    g = torch.Generator().manual_seed(int(seed))
    with torch.no_grad():
        for name, p in sorted(module.named_parameters()):
            if p.dim() == 4:
                fan_in = p.shape[1] * p.shape[2] * p.shape[3]
                p.copy_(torch.randn(p.shape, generator=g) * (2.0 / fan_in) ** 0.5)
            else:
                p.copy_(torch.randn(p.shape, generator=g) * bias_std)
    return module
