"""Type vocabulary of the incremental modules.

Mirrors incr_modules/masked_types.py:4-14 of the reference (names `_device`,
`Sp`, `DenseT`, `SpOrDense`, `Masked`).  In the reference `Masked` is an alias
of torch.Tensor, but every call site treats it as a 2-element sequence
`[values, mask]` (e.g. incr_modules/mask_incr_functional.py:60-61); the mask
slot is always None there.  Here the mask slot carries a `TileMask` (pixel
mask + ordered active-tile list kept in device memory); None still means
"every pixel active", and a plain bool/uint8/int tensor of shape (N,C,H,W) or
(N,1,H,W) is accepted and reduced over channels.
"""
import ctypes
from typing import List, Optional, Sequence, Union

import torch

from . import _lib

_device = "cuda" if torch.cuda.is_available() else "cpu"

Sp = torch.Tensor            # sparse COO tensors are not used by this path
DenseT = torch.Tensor
SpOrDense = Union[Sp, DenseT]
Masked = Sequence            # [delta: DenseT (N,C,H,W) channels_last, mask: TileMask | None]


class TileMask:
    """Pixel mask and ordered active-tile list of a delta at resolution (n, h, w).

    pixmask : uint8 (n, 1, h, w), 1 = pixel carries a delta
    tiles   : int32 [capacity], ids of active 8x8 tiles, ascending; first
              counts[0] entries valid
    stale   : int32 [capacity], tiles active in the previous step and inactive
              now (their deltas get zeroed by the next producer kernel)
    counts  : int32 [4] = (active, stale, ticket, reserved)
    A view made by `with_pixmask` shares tiles/stale/counts with its parent
    and differs in the pixel mask only (refined mask after an activation).
    """

    def __init__(self, n: int, h: int, w: int, device, _parent: "Optional[TileMask]" = None,
                 _pixmask: Optional[torch.Tensor] = None):
        self.n, self.h, self.w = int(n), int(h), int(w)
        self.device = torch.device(device)
        self.capacity = _lib.tile_capacity(self.n, self.h, self.w)
        if _parent is None:
            self.pixmask = torch.zeros((n, 1, h, w), dtype=torch.uint8, device=device)
            self.tiles = torch.zeros(self.capacity, dtype=torch.int32, device=device)
            self.stale = torch.zeros(self.capacity, dtype=torch.int32, device=device)
            self.counts = torch.zeros(_lib.CNT_WORDS, dtype=torch.int32, device=device)
            self.flags = torch.zeros(self.capacity, dtype=torch.int32, device=device)
        else:
            self.pixmask = _pixmask
            self.tiles, self.stale = _parent.tiles, _parent.stale
            self.counts, self.flags = _parent.counts, _parent.flags
        self.parent = _parent
        self.ready = None      # event of the latest build when it ran on the mask-planning stream
        self.c_struct = _lib.MieTileSet(
            self.n, self.h, self.w, self.pixmask.data_ptr(), self.tiles.data_ptr(),
            self.stale.data_ptr(), self.counts.data_ptr(), self.flags.data_ptr())

    def with_pixmask(self, pixmask: torch.Tensor) -> "TileMask":
        assert pixmask.shape == (self.n, 1, self.h, self.w) and pixmask.dtype == torch.uint8
        return TileMask(self.n, self.h, self.w, self.device, _parent=self, _pixmask=pixmask)

    def shares_tiles_with(self, other) -> bool:
        return isinstance(other, TileMask) and other.tiles.data_ptr() == self.tiles.data_ptr()

    @property
    def ref(self):
        return ctypes.byref(self.c_struct)

    def reset(self):
        """Forget the previous step (use together with zeroing the deltas written under it)."""
        self.pixmask.zero_()
        self.counts.zero_()
        self.flags.zero_()

    # -- host-side readers (synchronise; for tests and diagnostics only) ------
    def active_tiles(self) -> torch.Tensor:
        n = int(self.counts[_lib.CNT_ACTIVE].item())
        return self.tiles[:n].clone()

    def stale_tiles(self) -> torch.Tensor:
        n = int(self.counts[_lib.CNT_STALE].item())
        return self.stale[:n].clone()

    def density(self) -> float:
        return float(self.pixmask.float().mean().item())


MaskLike = Union[None, TileMask, torch.Tensor]
