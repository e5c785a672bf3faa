"""Event front end on the GPU: raw events -> the frames and frame deltas the incremental
networks consume.

The reference forms each input on the host (numpy scatter, data_fetchers/utils/util.py:62-107),
pads it (ReflectionPad2d((3, 3, 2, 2)), run_e2depth_continuous_dataset.py:49), copies it to the
device and subtracts the previous frame densely (:66).  `EventFrames` keeps the events of a sliding
window on the device and produces

  frame(start)              the dense frame for forward_refresh_reservoirs, and
  delta(start_old, start)   [delta NHWC, pixel mask] for the incremental forward,

the delta straight from the events of the two windows (one scatter kernel, no dense subtraction,
no any-over-channels mask pass).
"""
from typing import Sequence, Tuple

import numpy as np
import torch

from . import _lib, ops
from ._lib import check, lib


class EventFrames:
    """kind 'voxelgrid' (events_to_voxel_grid_absT, util.py:78-107) or 'histogram'
    (event_histogram, :62-75), as ContinuousEventsDataset.evframe_type
    (data_fetchers/continuous_event_datasets.py:86-93).

    window_size: window length in seconds (the reference's 0.05); t_scale converts the
    event stamps to seconds (1e-9 for the nanosecond stamps of the reference's .npy files);
    pad = (left, right, top, bottom) reflection padding.
    dtype: element type of the frames handed out -- torch.float32, or torch.bfloat16 for the networks that run
    on bf16 deltas (the fp32 sums are rounded in the same stream, mie_events_to_frame_bf16).
    """

    def __init__(self, width: int, height: int, num_bins: int = 5, evframe_type: str = "voxelgrid",
                 window_size: float = 0.05, t_scale: float = 1e-9, pad: Sequence[int] = (3, 3, 2, 2),
                 device="cuda:0", dtype=torch.float32):
        if evframe_type not in ("voxelgrid", "histogram"):
            raise NotImplementedError(evframe_type)
        self.kind = _lib.EVENTS_VOXEL if evframe_type == "voxelgrid" else _lib.EVENTS_HISTOGRAM
        self.channels = num_bins if evframe_type == "voxelgrid" else 2
        self.width, self.height, self.num_bins = int(width), int(height), int(num_bins)
        self.window_size, self.t_scale = float(window_size), float(t_scale)
        self.pad = tuple(int(v) for v in pad)
        self.device = torch.device(device)
        self.out_h = self.height + self.pad[2] + self.pad[3]
        self.out_w = self.width + self.pad[0] + self.pad[1]
        if dtype not in (torch.float32, torch.bfloat16):
            raise NotImplementedError("EventFrames: frames are float32 or bfloat16, not %s" % (dtype,))
        self.dtype = dtype
        self._events = None
        self._n = 0
        self._frame = ops.new_nhwc(1, self.channels, self.out_h, self.out_w, self.device, dtype)
        self._delta = ops.new_nhwc(1, self.channels, self.out_h, self.out_w, self.device, dtype)
        # bf16 frames: the fp32 sums the scatter accumulates (float atomics), kept beside the rounded frame
        self._sums = ops.new_nhwc(1, self.channels, self.out_h, self.out_w, self.device) if dtype != torch.float32 else None
        self._mask = torch.zeros((1, 1, self.out_h, self.out_w), dtype=torch.uint8, device=self.device)
        self._fmask = torch.zeros_like(self._mask)

    def set_events(self, events) -> int:
        """events: (n, 4) array-like of (t, x, y, p), float64, covering every window asked for
        until the next call.  Copied to the device once."""
        ev = torch.as_tensor(np.ascontiguousarray(events, dtype=np.float64) if not torch.is_tensor(events) else events)
        if ev.dim() != 2 or ev.shape[1] != 4 or ev.dtype != torch.float64:
            raise ValueError("events must be float64 of shape (n, 4), got %s %s" % (tuple(ev.shape), ev.dtype))
        self._events = ev.contiguous().to(self.device)
        self._n = int(ev.shape[0])
        return self._n

    def _run(self, start_old, start_new, delta, out, mask):
        if self._events is None:
            raise RuntimeError("EventFrames: call set_events first")
        stream = torch.cuda.current_stream(self.device).cuda_stream
        head = (self._events.data_ptr() if self._n else None, self._n, self.kind, self.num_bins, self.height,
                self.width, self.pad[0], self.pad[1], self.pad[2], self.pad[3], self.t_scale, float(start_old),
                float(start_new), self.window_size, 1 if delta else 0)
        if self._sums is None:
            check(lib().mie_events_to_frame(*head, ops.nhwc_ptr(out, "out"), mask.data_ptr(), stream))
        else:
            check(lib().mie_events_to_frame_bf16(*head, ops.nhwc_ptr(self._sums, "sums"), ops.nhwc_ptr(out, "out", dtype=self.dtype),
                                                 mask.data_ptr(), stream))

    def frame(self, start: float) -> torch.Tensor:
        """Dense (1, C, H', W') channels_last frame of the window (start, start + window_size)."""
        self._run(0.0, start, False, self._frame, self._fmask)
        return self._frame

    def delta(self, start_old: float, start_new: float) -> Tuple[torch.Tensor, torch.Tensor]:
        """[frame(start_new) - frame(start_old), pixel mask of the touched pixels]."""
        self._run(start_old, start_new, True, self._delta, self._mask)
        return [self._delta, self._mask]
