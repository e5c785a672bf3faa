"""TEST INFRASTRUCTURE ONLY - CPU restatement of the reference's event front end.

numpy restatement of data_fetchers/utils/util.py:62-107 (event_histogram,
events_to_voxel_grid_absT) plus the reflection padding of
run_e2depth_continuous_dataset.py:49 and the frame difference of :66.  Only tests/,
__graft_entry__.smoke() and bench.py's cpu_baseline may import this file; the shipped
package never does.

Pinned by tests/test_oracle_pinning.py: closed forms (an event on a bin boundary puts its
whole polarity into that bin; the two weights of an event sum to its polarity; weights are
linear in time), counts against numpy.bincount, padding against torch.nn.ReflectionPad2d.
Deliberate differences from the reference, which gets pre-sliced events: window membership
is decided here (start < t < start + delta_t), events off the sensor are dropped, and the
input array is not modified in place (util.py:90,94 overwrite their argument).
"""
import numpy as np


def _in_window(ev, t_scale, start, delta_t, width, height):
    t = ev[:, 0] * t_scale
    ok = (t > start) & (t < start + delta_t)
    ok &= (ev[:, 1] >= 0) & (ev[:, 1] < width) & (ev[:, 2] >= 0) & (ev[:, 2] < height)
    return ok


def voxel_grid_abst(events, num_bins, height, width, delta_t, start, t_scale=1e-9):
    """events_to_voxel_grid_absT (util.py:78-107): (num_bins, height, width) float32, and the
    (height, width) uint8 mask of pixels that received an event."""
    ev = np.asarray(events, dtype=np.float64).reshape(-1, 4)
    ev = ev[_in_window(ev, t_scale, start, delta_t, width, height)]
    grid = np.zeros((num_bins, height, width), np.float32).ravel()
    mask = np.zeros((height, width), np.uint8)
    if ev.shape[0] == 0:
        return grid.reshape(num_bins, height, width), mask
    ts = (num_bins - 1) * (ev[:, 0] * t_scale - start) / delta_t
    xs, ys = ev[:, 1].astype(int), ev[:, 2].astype(int)
    pols = ev[:, 3].copy()
    pols[pols == 0] = -1
    tis = ts.astype(int)
    dts = ts - tis
    left, right = pols * (1.0 - dts), pols * dts
    ok = tis < num_bins
    np.add.at(grid, xs[ok] + ys[ok] * width + tis[ok] * width * height, left[ok])
    ok = (tis + 1) < num_bins
    np.add.at(grid, xs[ok] + ys[ok] * width + (tis[ok] + 1) * width * height, right[ok])
    mask[ys, xs] = 1
    return grid.reshape(num_bins, height, width), mask


def histogram(events, height, width, delta_t, start, t_scale=1e-9):
    """event_histogram (util.py:62-75) as (2, height, width): channel 0 = p == -1, 1 = p == +1."""
    ev = np.asarray(events, dtype=np.float64).reshape(-1, 4)
    ev = ev[_in_window(ev, t_scale, start, delta_t, width, height)]
    x, y, p = ev[:, 1].astype(int), ev[:, 2].astype(int), ev[:, 3]
    pos = np.zeros(height * width, np.float32)
    neg = np.zeros(height * width, np.float32)
    np.add.at(pos, x[p == 1] + width * y[p == 1], 1)
    np.add.at(neg, x[p == -1] + width * y[p == -1], 1)
    mask = np.zeros((height, width), np.uint8)
    counted = (p == 1) | (p == -1)
    mask[y[counted], x[counted]] = 1
    return np.stack([neg, pos]).reshape(2, height, width), mask


def reflect_pad(a, pad):
    """ReflectionPad2d((left, right, top, bottom)) on the last two axes."""
    l, r, t, b = pad
    width = [(0, 0)] * (a.ndim - 2) + [(t, b), (l, r)]
    return np.pad(a, width, mode="reflect")


def frame(events, kind, num_bins, height, width, delta_t, start, t_scale=1e-9, pad=(0, 0, 0, 0)):
    if kind == "voxelgrid":
        g, m = voxel_grid_abst(events, num_bins, height, width, delta_t, start, t_scale)
    else:
        g, m = histogram(events, height, width, delta_t, start, t_scale)
    return reflect_pad(g, pad), reflect_pad(m, pad)


def frame_delta(events, kind, num_bins, height, width, delta_t, start_old, start_new, t_scale=1e-9,
                pad=(0, 0, 0, 0)):
    """frame(start_new) - frame(start_old) (run_e2depth_continuous_dataset.py:66) and the union of
    the two touched-pixel masks."""
    g1, m1 = frame(events, kind, num_bins, height, width, delta_t, start_new, t_scale, pad)
    g0, m0 = frame(events, kind, num_bins, height, width, delta_t, start_old, t_scale, pad)
    return g1 - g0, m0 | m1
