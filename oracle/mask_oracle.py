"""CPU oracle for pixel masks, footprints and active-tile lists (numpy, integer exact).

TEST INFRASTRUCTURE ONLY: imported by tests/, __graft_entry__.smoke() and the
cpu_baseline leg of bench.py as the checker; never by the product package.

The reference holds no mask propagation to compare with (every module returns
None in the mask slot, incr_modules/mask_incr_modules.py:41,103,178); its only
mask definitions are max-pool dilations of abs(x) against a threshold:
  incr_modules/utils.py:22-25              compute_mask  (field 5, thr 1e-4, .le)
  utils/str_sparse_utils.py:10-11          get_mask      (field 3, thr 1e-4, .ge)
  metrics/structural_sparsity.py:11-14     field_channel_sparsity
  benchmark/input_handlers.py:77-85        neighbourhood mask of a random field
`maxpool_mask` restates that definition; `pixel_mask` + `footprint_conv` is the
same thing split into "which pixels carry a delta" and "which outputs can a
k x k op reach from them", reduced over channels.  Pinned by
tests/test_oracle_pinning.py against brute force and torch max_pool2d.
"""
import numpy as np

TILE = 8


def pixel_mask(delta: np.ndarray, threshold: float = 0.0) -> np.ndarray:
    """delta (N,C,H,W) -> uint8 (N,H,W): any_c(|delta| > threshold)."""
    return (np.abs(delta) > threshold).any(axis=1).astype(np.uint8)


def maxpool_mask(x: np.ndarray, field_size: int, threshold: float) -> np.ndarray:
    """Per-element mask maxpool_{f x f, stride 1, pad (f-1)//2}(|x|) >= threshold
    (utils/str_sparse_utils.py:10-11); x (N,C,H,W) -> uint8 (N,C,H,W)."""
    n, c, h, w = x.shape
    p = (field_size - 1) // 2
    a = np.full((n, c, h + 2 * p, w + 2 * p), -np.inf, dtype=np.float64)
    a[:, :, p:p + h, p:p + w] = np.abs(x)
    out = np.full((n, c, h, w), -np.inf)
    for dy in range(field_size):
        for dx in range(field_size):
            out = np.maximum(out, a[:, :, dy:dy + h, dx:dx + w])
    return (out >= threshold).astype(np.uint8)


def conv_out_size(h, w, k, stride, pad):
    """ext/pointops/pointops_functional.py:25-26."""
    return (h + 2 * pad - k) // stride + 1, (w + 2 * pad - k) // stride + 1


def footprint_conv(mask: np.ndarray, k: int, stride: int, pad: int) -> np.ndarray:
    """Output pixels a k x k / stride / pad conv can reach from the active input pixels.
    mask uint8 (N,H,W) -> uint8 (N,Ho,Wo)."""
    n, h, w = mask.shape
    ho, wo = conv_out_size(h, w, k, stride, pad)
    padded = np.zeros((n, h + 2 * pad + k, w + 2 * pad + k), dtype=np.uint8)
    padded[:, pad:pad + h, pad:pad + w] = mask
    out = np.zeros((n, ho, wo), dtype=np.uint8)
    for ky in range(k):
        for kx in range(k):
            out |= padded[:, ky:ky + (ho - 1) * stride + 1:stride, kx:kx + (wo - 1) * stride + 1:stride]
    return out


def _up2x_sources(o: int, size: int):
    """Source indices with non-zero bilinear weight of output index o
    (scale 2, align_corners=False: src = max(0, (o + 0.5) / 2 - 0.5))."""
    j = o // 2
    if o % 2 == 1:
        return {j, min(j + 1, size - 1)}
    if j == 0:
        return {0}
    return {j - 1, j}


def footprint_up2x(mask: np.ndarray) -> np.ndarray:
    n, h, w = mask.shape
    out = np.zeros((n, 2 * h, 2 * w), dtype=np.uint8)
    rows = [sorted(_up2x_sources(o, h)) for o in range(2 * h)]
    cols = [sorted(_up2x_sources(o, w)) for o in range(2 * w)]
    rowred = np.zeros((n, 2 * h, w), dtype=np.uint8)
    for oy, rs in enumerate(rows):
        for r in rs:
            rowred[:, oy, :] |= mask[:, r, :]
    for ox, cs in enumerate(cols):
        for c in cs:
            out[:, :, ox] |= rowred[:, :, c]
    return out


def footprint_tconv(mask: np.ndarray, k: int, stride: int, pad: int, ho: int, wo: int) -> np.ndarray:
    """Output pixels of a transposed conv reached from active inputs: oy = iy*s - p + ky."""
    n, h, w = mask.shape
    out = np.zeros((n, ho, wo), dtype=np.uint8)
    ys, xs = np.arange(h) * stride - pad, np.arange(w) * stride - pad
    for ky in range(k):
        oy = ys + ky
        vy = (oy >= 0) & (oy < ho)
        for kx in range(k):
            ox = xs + kx
            vx = (ox >= 0) & (ox < wo)
            out[:, oy[vy][:, None], ox[vx][None, :]] |= mask[:, vy][:, :, vx]
    return out


def tile_grid(h, w):
    return (h + TILE - 1) // TILE, (w + TILE - 1) // TILE


def tile_list(mask: np.ndarray) -> np.ndarray:
    """Ascending ids (n*tiles_y + ty)*tiles_x + tx of the 8x8 tiles with an active pixel."""
    n, h, w = mask.shape
    ty, tx = tile_grid(h, w)
    padded = np.zeros((n, ty * TILE, tx * TILE), dtype=np.uint8)
    padded[:, :h, :w] = mask
    flags = padded.reshape(n, ty, TILE, tx, TILE).any(axis=(2, 4))
    return np.flatnonzero(flags.reshape(-1)).astype(np.int32)


def stale_list(prev_tiles: np.ndarray, cur_tiles: np.ndarray) -> np.ndarray:
    """Tiles active in the previous step and not now, ascending."""
    return np.setdiff1d(prev_tiles, cur_tiles).astype(np.int32)


def tiles_to_pixels(tiles: np.ndarray, n, h, w) -> np.ndarray:
    """uint8 (N,H,W) with 1 on every pixel of the listed tiles."""
    ty, tx = tile_grid(h, w)
    flags = np.zeros(n * ty * tx, dtype=np.uint8)
    flags[tiles] = 1
    full = np.repeat(np.repeat(flags.reshape(n, ty, tx), TILE, axis=1), TILE, axis=2)
    return full[:, :h, :w]
