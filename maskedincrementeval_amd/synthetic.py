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
