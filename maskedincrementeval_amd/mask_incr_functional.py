"""Reservoir state and functional incremental ops.

Drop-in for incr_modules/mask_incr_functional.py of the reference: same names
and call conventions (`IncrementReserve`, `AccumStreamManager`,
`IncrPointwiseMultiply`, `conv2d_from_module`, `transposed_conv2d_from_module`,
`bn2d_from_module`, `interpolate_from_module`), but the linear ops run as
masked HIP kernels over active tiles and return a real `TileMask` in the mask
slot instead of None.  The functional forms are stateless: each call owns a
fresh output and tile set (the nn.Module forms in mask_incr_modules.py keep
persistent buffers and are the ones to use in a loop).
"""
import torch
import torch.nn as nn

from . import _lib, ops
from .masked_types import DenseT, Masked, TileMask


class AccumStreamManager:
    """Kept for API compatibility (reference: mask_incr_functional.py:9-21).

    The reference creates a side CUDA stream meant for off-critical-path
    accumulation and never uses it.  Here the accumulation is fused into the
    kernel that produces the delta, so `get_stream` hands back the current
    stream and no extra stream is created.
    """
    instance = None

    @classmethod
    def createAccumStream(cls):
        if cls.instance is None:
            cls.instance = cls()
        return cls.instance

    def get_stream(self):
        return torch.cuda.current_stream()


class IncrementReserve:
    """Dense cached activation ("reservoir"), channels_last for 4-D tensors.

    Reference: mask_incr_functional.py:26-48.  `update_reservoir` copies into
    the existing buffer when the shape is unchanged, so device pointers stay
    stable across refreshes (needed for HIP-graph replay).
    """

    def __init__(self, x_init=None):
        self.accum_stream = AccumStreamManager.createAccumStream()
        self.reservoir = None
        if x_init is not None:
            self.update_reservoir(x_init)

    def _adjust_mem_format(self):
        if self.reservoir is not None and self.reservoir.dim() == 4:
            self.reservoir = ops.as_nhwc(self.reservoir)

    def accumulate(self, incr: Masked):
        # stand-alone form; the incremental modules update reservoirs inside their kernels
        self.reservoir.add_(incr[0])

    def update_reservoir(self, x: DenseT):
        x = x.detach()
        if x.dtype == torch.bfloat16:       # reservoirs stay fp32 when the deltas are bf16
            x = x.float()
        if (self.reservoir is not None and self.reservoir.shape == x.shape
                and self.reservoir.device == x.device and self.reservoir.dtype == x.dtype):
            self.reservoir.copy_(x)
        else:
            self.reservoir = x.clone()
            self._adjust_mem_format()


def _unpack(x_incr: Masked):
    """(delta as NHWC fp32, pixel mask tensor | None, TileMask | None)."""
    delta = ops.as_nhwc(x_incr[0])
    mask = x_incr[1] if len(x_incr) > 1 else None
    pix = ops.pixel_mask_of(mask, delta)
    return delta, pix, (mask if isinstance(mask, TileMask) else None)


def tileset_for(x_incr: Masked, cache=None) -> TileMask:
    """Tile set covering the delta of a Masked pair at its own resolution.

    A TileMask in the mask slot is used as is; None / plain tensors get a tile
    set built with the identity footprint (into `cache` when given).
    """
    delta, pix, tm = _unpack(x_incr)
    if tm is not None:
        return tm
    n, _, h, w = delta.shape
    ts = cache if cache is not None else TileMask(n, h, w, delta.device)
    ops.build_mask_tiles(pix, None, n, h, w, _lib.FOOT_CONV, 1, 1, 0, ts)
    return ts


def IncrPointwiseMultiply(x1_incr: Masked, x1: IncrementReserve, x2_incr: Masked,
                          x2: IncrementReserve) -> Masked:
    """(dx2 + R2) * dx1 + R1 * dx2, reservoirs untouched (reference :52-54)."""
    d1, p1, t1 = _unpack(x1_incr)
    d2, p2, t2 = _unpack(x2_incr)
    n, c, h, w = d1.shape
    # two refined views of one parent share the tile list but not the pixel mask: the kernel gates on ONE pixel
    # mask, so the operands' own tile set serves only when it is the same mask; else the union is built
    if t1 is not None and t1.shares_tiles_with(t2) and t1.pixmask.data_ptr() == t2.pixmask.data_ptr():
        ts = t1
    else:
        ts = TileMask(n, h, w, d1.device)
        ops.build_mask_tiles(p1, p2, n, h, w, _lib.FOOT_CONV, 1, 1, 0, ts)
    out = ops.new_nhwc(n, c, h, w, d1.device, d1.dtype)
    ops.mul_incr(d1, p1, x1.reservoir, d2, p2, x2.reservoir, out, ts, keep_reservoir=True)
    return [out, ts]


def _square(v, what):
    if isinstance(v, (tuple, list)):
        if len(v) != 2 or v[0] != v[1]:
            raise NotImplementedError("%s must be square, got %s" % (what, (v,)))
        return int(v[0])
    return int(v)


def conv2d_from_module(x: Masked, conv_weights, stride=(1, 1), padding=(1, 1)) -> Masked:
    """Masked conv of a delta with a [Cin,K,K,Cout] filter (reference :60-61)."""
    delta, pix, _ = _unpack(x)
    n, _, h, w = delta.shape
    k = conv_weights.shape[1]
    s, p = _square(stride, "stride"), _square(padding, "padding")
    if k not in (1, 3, 5, 7) or conv_weights.shape[2] != k:
        raise NotImplementedError("not Implemented convolution for these dimensions!")
    ho, wo = ops.conv_out_size(h, w, k, s, p)
    ts = TileMask(n, ho, wo, delta.device)
    ops.build_mask_tiles(pix, None, n, h, w, _lib.FOOT_CONV, k, s, p, ts)
    out = ops.new_nhwc(n, conv_weights.shape[3], ho, wo, delta.device, delta.dtype)
    ops.conv_masked(delta, pix, None, None, conv_weights, k, s, p, ts, out)
    return [out, ts]


def transposed_conv2d_from_module(x: Masked, gates: nn.ConvTranspose2d, bias=True) -> Masked:
    """Masked conv_transpose2d of a delta, bias dropped (reference :64-66)."""
    delta, pix, _ = _unpack(x)
    n, _, h, w = delta.shape
    k = _square(gates.kernel_size, "kernel_size")
    s, p = _square(gates.stride, "stride"), _square(gates.padding, "padding")
    op = _square(gates.output_padding, "output_padding")
    if _square(gates.dilation, "dilation") != 1 or gates.groups != 1:
        raise NotImplementedError("transposed conv with dilation / groups")
    ho, wo = (h - 1) * s - 2 * p + k + op, (w - 1) * s - 2 * p + k + op
    filt = gates.weight.detach().permute(0, 2, 3, 1).contiguous()   # [Cin,K,K,Cout]
    ts = TileMask(n, ho, wo, delta.device)
    ops.build_mask_tiles(pix, None, n, h, w, _lib.FOOT_TCONV, k, s, p, ts)
    out = ops.new_nhwc(n, filt.shape[3], ho, wo, delta.device, delta.dtype)
    ops.tconv_masked(delta, pix, filt, k, s, p, ts, out)
    return [out, ts]


def bn_scale(bnm: nn.BatchNorm2d) -> torch.Tensor:
    """gamma / sqrt(running_var + eps) as contiguous fp32 [C]."""
    scale = torch.rsqrt(bnm.running_var.detach().float() + bnm.eps)
    if bnm.weight is not None:
        scale = scale * bnm.weight.detach().float()
    return scale.contiguous()


def bn2d_from_module(x: Masked, bnm: nn.BatchNorm2d) -> Masked:
    """Linear part of eval-mode batch norm on a delta: dx * gamma / sqrt(var + eps).

    Reference :69-73 (F.batch_norm with zero mean and no bias).  A per-channel
    scale keeps zeros zero, so the mask passes through.
    """
    delta, pix, tm = _unpack(x)
    n, c, h, w = delta.shape
    if not isinstance(tm, TileMask):
        tm = TileMask(n, h, w, delta.device)
        ops.build_mask_tiles(pix, None, n, h, w, _lib.FOOT_CONV, 1, 1, 0, tm)
    out = ops.new_nhwc(n, c, h, w, delta.device, delta.dtype)
    ops.scale_incr(delta, bn_scale(bnm), out, tm)
    return [out, tm]


def interpolate_from_module(x: Masked) -> Masked:
    """Bilinear x2 (align_corners=False) of a delta (reference :76-78)."""
    delta, pix, _ = _unpack(x)
    n, c, h, w = delta.shape
    ts = TileMask(n, 2 * h, 2 * w, delta.device)
    ops.build_mask_tiles(pix, None, n, h, w, _lib.FOOT_UP2X, 0, 0, 0, ts)
    out = ops.new_nhwc(n, c, 2 * h, 2 * w, delta.device, delta.dtype)
    ops.upsample2x_incr(delta, pix, None, None, ts, out)
    return [out, ts]
