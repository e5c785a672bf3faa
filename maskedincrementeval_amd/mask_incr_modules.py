"""nn.Module surface of the incremental layers.

Drop-in for incr_modules/mask_incr_modules.py of the reference: same class
names, constructor signatures and the two-forward protocol

    forward(x_incr: Masked) -> Masked          incremental step on [delta, mask]
    forward_refresh_reservoirs(x) -> dense     dense pass that (re)fills reservoirs

(reference :13-17).  The incremental forwards run the masked HIP kernels of
libmie_hip.so on persistent per-module buffers; the mask slot of the result
is a `TileMask`.  The dense refresh of the convolutions runs through the same
kernels with every tile active (bias and the reservoir fill fused in); the
cheap point-wise parts of the refresh are torch ops on the device.
"""
import functools
from typing import Optional, Tuple

import torch
import torch.nn as nn
import torch.nn.functional as F

from . import _lib, ops
from .masked_types import DenseT, Masked, TileMask
from .mask_incr_functional import (IncrPointwiseMultiply, IncrementReserve, _square, _unpack,
                                   bn2d_from_module, bn_scale, conv2d_from_module)


class _IncrBuffers:
    """Persistent per-module device buffers of the incremental path.

    Deltas written by the kernels live in fixed buffers (stable pointers, zero
    outside the active tiles); `_reset_incr` returns them to the all-zero state
    a dense refresh implies.  Delta buffers, tile sets and pixel masks exist once per
    `ops.buffer_parity` (0 unless a network is run with its next step planned ahead,
    ops.pipelined_step).
    """

    def _ib(self):
        d = self.__dict__.get("_incr_bufs")
        if d is None:
            d = {}
            self.__dict__["_incr_bufs"] = d
        return d

    def _delta_buf(self, name, shape, device, dtype=torch.float32) -> torch.Tensor:
        key = ("d", name, tuple(shape), str(device), dtype, ops.buffer_parity)
        b = self._ib().get(key)
        if b is None:
            b = ops.new_nhwc(*shape, device, dtype)
            self._ib()[key] = b
        return b

    def _tile_set(self, name, n, h, w, device) -> TileMask:
        key = ("t", name, (n, h, w), str(device), ops.buffer_parity)
        b = self._ib().get(key)
        if b is None:
            b = TileMask(n, h, w, device)
            self._ib()[key] = b
        return b

    def _pix_buf(self, name, n, h, w, device) -> torch.Tensor:
        key = ("p", name, (n, h, w), str(device), ops.buffer_parity)
        b = self._ib().get(key)
        if b is None:
            b = torch.zeros((n, 1, h, w), dtype=torch.uint8, device=device)
            self._ib()[key] = b
        return b

    def _view(self, name, parent: TileMask, pix: torch.Tensor) -> TileMask:
        key = ("v", name, parent.tiles.data_ptr(), pix.data_ptr())
        b = self._ib().get(key)
        if b is None:
            b = parent.with_pixmask(pix)
            self._ib()[key] = b
        return b

    def _dense_tile_set(self, n, h, w, device) -> TileMask:
        """Tile set with every tile active (built once; survives `_reset_incr`)."""
        key = ("T", "dense", (n, h, w), str(device))
        b = self._ib().get(key)
        if b is None:
            b = TileMask(n, h, w, device)
            ops.build_mask_tiles(None, None, n, h, w, _lib.FOOT_CONV, 1, 1, 0, b)
            self._ib()[key] = b
        return b

    def _dense_buf(self, name, shape, device, dtype=torch.float32) -> torch.Tensor:
        """Persistent dense output of the refresh pass (not touched by `_reset_incr`)."""
        key = ("D", name, tuple(shape), str(device), dtype)
        b = self._ib().get(key)
        if b is None:
            b = ops.new_nhwc(*shape, device, dtype)
            self._ib()[key] = b
        return b

    def _reset_incr(self):
        """Called by every dense refresh; leaves the incremental buffers alone.  They need no reset: a
        delta buffer is zero outside the active tiles of the step that last wrote it, and the first step
        after the refresh finds those tiles in its stale list and zeroes them, exactly as between two
        incremental steps.  (Zero-filling every delta buffer and tile set here cost about as many fill
        launches per refresh as the refresh has convs.)"""
        return

    def _zero_incr(self):
        """Force the all-zero state: delta buffers, pixel masks, tile sets (for callers that rewrite
        these buffers by hand)."""
        for key, b in self._ib().items():
            if key[0] in ("d", "p"):
                b.zero_()
            elif key[0] == "t":
                b.reset()


# input output increments: interface for incremental modules
class IncrementMaskModule(nn.Module, _IncrBuffers):

    def forward_refresh_reservoirs(self, x: DenseT) -> DenseT:
        return x


class KFencedMaskModule(IncrementMaskModule):
    """Delta quantiser: lets multiples of k through, carries the rest (reference :21-47).

    T = Rd + d;  f = k * floor(0.5 + T / k);  Rd = T - f;  returns [f, mask of f != 0].
    One kernel over the active tiles of the input (where d = 0 the carry Rd stays
    within [-k/2, k/2] and the dense expression emits 0 as well); the refined pixel
    mask it emits is what makes the layers behind it sparse again.  k is `tp` until
    a refresh sets it to tp * ||x||_2 (:45), kept in a 1-element device tensor whose
    address survives later refreshes.  The reference instantiates the module in
    every nnConvIncr but never calls its forward (:166).
    """

    def __init__(self, tp: float = .1, norm: str = "l2"):
        super().__init__()
        self.delta = IncrementReserve()
        self.tp = tp
        self.k = tp
        # "l2": k = tp * ||x||_2 over the whole tensor, the reference's rule (:45), which grows with the
        # square root of the tensor size; "rms": k = tp * ||x||_2 / sqrt(numel), a step relative to the
        # typical magnitude of an element
        self.norm = norm

    def floor_by_k(self, T):
        return self.k * torch.floor(0.5 + T / self.k)

    def forward(self, incr: Masked) -> Masked:
        d, _, _ = _unpack(incr)
        n, c, h, w = d.shape
        if self.delta.reservoir is None or self.delta.reservoir.shape != d.shape:
            self.delta.update_reservoir(ops.new_nhwc(n, c, h, w, d.device))
        mask = incr[1] if len(incr) > 1 else None
        if isinstance(mask, TileMask):
            ts = mask
        else:
            ts = self._tile_set("own", n, h, w, d.device)
            ops.build_mask_tiles(ops.pixel_mask_of(mask, d), None, n, h, w, _lib.FOOT_CONV, 1, 1, 0, ts)
        out = self._delta_buf("out", (n, c, h, w), d.device, d.dtype)
        pix = self._pix_buf("refined", n, h, w, d.device)
        ops.kfence_incr(d, self.delta.reservoir, self.k, out, ts, pix)
        return [out, self._view("refined", ts, pix)]

    def forward_refresh_reservoirs(self, x: DenseT) -> DenseT:
        k = (self.tp * torch.norm(x.detach().float())).reshape(1)
        if self.norm == "rms":
            k = k / float(x.numel()) ** 0.5
        elif self.norm != "l2":
            raise ValueError("KFencedMaskModule.norm must be 'l2' or 'rms', got %r" % (self.norm,))
        if isinstance(self.k, torch.Tensor) and self.k.device == k.device:
            self.k.copy_(k)
        else:
            self.k = k
        if self.delta.reservoir is not None and self.delta.reservoir.shape == x.shape:
            self.delta.reservoir.zero_()
        else:
            self.delta.update_reservoir(torch.zeros_like(x, dtype=torch.float32))
        self._reset_incr()
        return x


class PointwiseMultiplyIncr(IncrementMaskModule):
    """Product rule on cached operands, reservoirs owned elsewhere (reference :51-64)."""

    def __init__(self, x1res_module: IncrementReserve, x2res_module: IncrementReserve):
        super().__init__()
        self.x1_res: IncrementReserve = x1res_module
        self.x2_res: IncrementReserve = x2res_module

    def forward(self, x1_incr: Masked, x2_incr: Masked) -> Masked:
        return IncrPointwiseMultiply(x1_incr, self.x1_res, x2_incr, self.x2_res)

    def forward_refresh_reservoirs(self, x1: DenseT, x2: DenseT) -> DenseT:
        return x1 * x2


class nnReservedMultiplication(PointwiseMultiplyIncr):
    """Product rule + accumulation of both operands, one kernel (reference :67-81)."""

    def __init__(self):
        super().__init__(IncrementReserve(), IncrementReserve())

    def forward(self, x1_incr: Masked, x2_incr: Masked) -> Masked:
        d1, p1, t1 = _unpack(x1_incr)
        d2, p2, t2 = _unpack(x2_incr)
        if self.x1_res.reservoir is None or self.x2_res.reservoir is None:
            raise RuntimeError("nnReservedMultiplication: call forward_refresh_reservoirs first")
        n, c, h, w = d1.shape
        if t1 is not None and t1.shares_tiles_with(t2) and t1.pixmask.data_ptr() == t2.pixmask.data_ptr():
            ts = t1
        else:
            ts = self._tile_set("union", n, h, w, d1.device)
            ops.build_mask_tiles(p1, p2, n, h, w, _lib.FOOT_CONV, 1, 1, 0, ts)
        out = self._delta_buf("out", (n, c, h, w), d1.device, d1.dtype)
        ops.mul_incr(d1, p1, self.x1_res.reservoir, d2, p2, self.x2_res.reservoir, out, ts)
        return [out, ts]

    def forward_refresh_reservoirs(self, x1: DenseT, x2: DenseT) -> DenseT:
        out = PointwiseMultiplyIncr.forward_refresh_reservoirs(self, x1, x2)
        self.x1_res.update_reservoir(x1)
        self.x2_res.update_reservoir(x2)
        self._reset_incr()
        return out


def activation_kind(op) -> Tuple[int, float]:
    """Map a unary torch callable onto a kernel activation (kind, negative slope)."""
    if isinstance(op, functools.partial):
        kind, slope = activation_kind(op.func)
        if kind == _lib.ACT_LEAKY_RELU:
            slope = op.keywords.get("negative_slope", op.args[0] if op.args else slope)
        return kind, float(slope)
    if isinstance(op, nn.LeakyReLU):
        return _lib.ACT_LEAKY_RELU, float(op.negative_slope)
    if isinstance(op, nn.ReLU) or op in (torch.relu, F.relu, torch.relu_):
        return _lib.ACT_RELU, 0.0
    if isinstance(op, nn.Sigmoid) or op in (torch.sigmoid, F.sigmoid):
        return _lib.ACT_SIGMOID, 0.0
    if isinstance(op, nn.Tanh) or op in (torch.tanh, F.tanh):
        return _lib.ACT_TANH, 0.0
    if op is F.leaky_relu:
        return _lib.ACT_LEAKY_RELU, 0.01
    slope = getattr(op, "negative_slope", None)
    if slope is not None:
        return _lib.ACT_LEAKY_RELU, float(slope)
    raise NotImplementedError(
        "incremental activation for %r has no kernel (supported: relu, leaky_relu, sigmoid, tanh)" % (op,))


_ACTIVATION_OPS = {"relu": torch.relu, "sigmoid": torch.sigmoid, "tanh": torch.tanh}


def activation_op(name: str):
    """Unary torch callable for an activation named in a layer constructor ('relu', 'sigmoid', 'tanh',
    'leaky_relu').  The reference looks the name up with getattr(torch, name, 'relu')
    (incr_modules/e2depth_incr.py:19), which turns an unknown name into the *string* 'relu' and fails at the
    first forward; here an unknown name raises at construction."""
    if name == "leaky_relu":
        return leaky_relu_op()
    try:
        return _ACTIVATION_OPS[name]
    except KeyError:
        raise ValueError("unknown activation %r (known: %s, leaky_relu)" % (name, ", ".join(sorted(_ACTIVATION_OPS)))) from None


def leaky_relu_op(negative_slope: float = 0.01):
    """Unary callable for nnReservedActivation(op=...) that the kernels recognise."""
    return functools.partial(F.leaky_relu, negative_slope=negative_slope)


class NonlinearPointOpIncr(IncrementMaskModule):
    """out = op(R + d) - op(R); the reservoir is owned by the caller (reference :86-103)."""

    def __init__(self, res_in: IncrementReserve, op=torch.tanh, refine_mask: bool = True):
        super().__init__()
        self.reservoir_in = res_in
        self.op = op
        self.refine_mask = refine_mask

    def forward(self, x_incr: Masked) -> Masked:
        return self._nonlin(x_incr, keep_reservoir=True)

    def forward_refresh_reservoirs(self, x: DenseT):
        return self.op(x)

    def _nonlin(self, x_incr: Masked, keep_reservoir: bool):
        kind, slope = activation_kind(self.op)
        d, _, _ = _unpack(x_incr)
        res = self.reservoir_in.reservoir
        if res is None:
            raise RuntimeError("incremental activation: call forward_refresh_reservoirs first")
        n, c, h, w = d.shape
        mask = x_incr[1] if len(x_incr) > 1 else None
        if isinstance(mask, TileMask):
            ts = mask
        else:
            ts = self._tile_set("own", n, h, w, d.device)
            ops.build_mask_tiles(ops.pixel_mask_of(mask, d), None, n, h, w, _lib.FOOT_CONV, 1, 1, 0, ts)
        out = self._delta_buf("out", (n, c, h, w), d.device, d.dtype)
        if self.refine_mask:
            pix = self._pix_buf("refined", n, h, w, d.device)
            ops.act_incr(kind, slope, d, res, out, ts, pix, keep_reservoir=keep_reservoir)
            return [out, self._view("refined", ts, pix)]
        ops.act_incr(kind, slope, d, res, out, ts, None, keep_reservoir=keep_reservoir)
        return [out, ts]


class nnLinearIncr(nn.Linear):
    """Fully connected layer on a delta: bias dropped (reference :106-116).  One kernel that reads only
    the weight rows of the features whose delta is non-zero; the transposed weight copy it walks is
    rebuilt when the weight changes."""

    def _weight_t(self) -> torch.Tensor:
        w = self.weight
        key = (w.data_ptr(), w._version, w.device)
        cached = self.__dict__.get("_wt")
        if cached is None or cached[0] != key:
            cached = (key, w.detach().float().t().contiguous())
            self.__dict__["_wt"] = cached
        return cached[1]

    def forward(self, x_incr: Masked) -> Masked:
        d = x_incr[0]
        lead = d.shape[:-1]
        d2 = d.reshape(-1, d.shape[-1]).contiguous()
        out = torch.empty((d2.shape[0], self.out_features), dtype=d2.dtype, device=d2.device)
        ops.linear_incr(d2, self._weight_t(), out)
        return [out.reshape(*lead, self.out_features), None]

    def forward_refresh_reservoirs(self, x: DenseT) -> DenseT:
        return super().forward(x)


class _ConvIncrMixin(_IncrBuffers):
    """Shared body of nnConvIncrBase / nnConvIncr."""

    def _geometry(self):
        k = _square(self.kernel_size, "kernel_size")
        s = _square(self.stride, "stride")
        p = _square(self.padding, "padding")
        if _square(self.dilation, "dilation") != 1 or self.groups != 1:
            raise NotImplementedError("incremental conv with dilation / groups")
        if k not in (1, 3, 5, 7) or s not in (1, 2):
            raise NotImplementedError("not Implemented convolution for these dimensions!")
        return k, s, p

    @property
    def conv2d_weights(self) -> "ops.ConvFilter":
        """Filter in the kernel layouts ([Cin, K, K, Cout] and its matrix-core copy), rebuilt when
        the weight changes."""
        w = self.weight
        tag = (w.data_ptr(), w._version, str(w.device))
        cached = self.__dict__.get("_filt_cache")
        if cached is None or cached[0] != tag:
            cached = (tag, ops.ConvFilter(w.detach().permute(1, 2, 3, 0).contiguous().float()))
            self.__dict__["_filt_cache"] = cached
        return cached[1]

    def _incr_forward(self, x_incr: Masked, x2_incr: Masked = None, reservoir=None,
                      act=_lib.ACT_NONE, slope=0.0, path=_lib.PATH_AUTO, out_name="out",
                      addend_incr: Masked = None, filt=None) -> Masked:
        """addend_incr: delta added to the conv result before the epilogue; the caller
        guarantees that its active pixels are covered by the conv's output mask.
        filt: a row slice of conv2d_weights when only part of the input channels is fed."""
        k, s, p = self._geometry()
        x, pix, _ = _unpack(x_incr)
        x2 = pix2 = None
        if x2_incr is not None:
            x2, pix2, _ = _unpack(x2_incr)
        n, _, h, w = x.shape
        ho, wo = ops.conv_out_size(h, w, k, s, p)
        out = self._delta_buf(out_name, (n, self.out_channels, ho, wo), x.device, x.dtype)
        in_tm = x_incr[1] if len(x_incr) > 1 else None
        if k == 1 and s == 1 and p == 0 and x2 is None and isinstance(in_tm, TileMask):
            ts = in_tm            # a 1x1 conv reaches exactly the pixels of its input: same tile set
        else:
            ts = self._conv_tile_set(out_name, x, pix, x2, pix2, k, s, p)
        addend = None if addend_incr is None else ops.as_nhwc(addend_incr[0])
        ops.conv_masked(x, pix, x2, pix2, self.conv2d_weights if filt is None else filt, k, s, p, ts,
                        out, reservoir, act, slope, path, addend)
        return [out, ts]


    def _upconv_forward(self, up: "nnUpsample2xIncr", x_incr: Masked, skip_incr: Masked, reservoir, act, slope,
                        out_name="out_act") -> Masked:
        """conv over up2x(x + skip) without forming the up-sampled delta (ops.upconv_masked)."""
        k, s, p = self._geometry()
        a, pa, b, pb, ts_up = up.plan(x_incr, skip_incr)
        n, _, h, w = a.shape
        ts = self._tile_set(out_name, n, 2 * h, 2 * w, a.device)
        ops.build_mask_tiles(ts_up, None, n, 2 * h, 2 * w, _lib.FOOT_CONV, k, s, p, ts)
        out = self._delta_buf(out_name, (n, self.out_channels, 2 * h, 2 * w), a.device, a.dtype)
        ops.upconv_masked(a, pa, b, pb, self.conv2d_weights, k, p, ts, out, reservoir, act, slope)
        return [out, ts]

    def _conv_tile_set(self, name, x, pix, x2, pix2, k, s, p) -> TileMask:
        """Tile set of the conv output for the (one or two) masked inputs, built for this step."""
        n, _, h, w = x.shape
        ho, wo = ops.conv_out_size(h, w, k, s, p)
        ts = self._tile_set(name, n, ho, wo, x.device)
        if x2 is None:
            m1, m2 = pix, None
        elif pix is None or pix2 is None:      # one input dense -> every tile active
            m1 = m2 = None
        else:
            m1, m2 = pix, pix2
        ops.build_mask_tiles(m1, m2, n, h, w, _lib.FOOT_CONV, k, s, p, ts)
        return ts

    def _refresh_forward(self, x: DenseT, x2: DenseT = None, activation=None, out=None,
                         path=_lib.PATH_AUTO, addend: DenseT = None, reserve=None, filt=None,
                         bias=None) -> DenseT:
        """Dense pass: conv2d(cat(x, x2), W, b) through the same kernels with every tile
        active.  With `activation` (an nnReservedActivation) the pre-activation goes straight
        into its reservoir and the activated tensor is returned; with `reserve` (an
        IncrementReserve) the fp32 result is also written into that reservoir.  `out` overrides
        the result buffer.  CPU tensors are refused: this package has no CPU path.
        """
        self._reset_incr()
        ops._require_gpu(x, "x")
        k, s, p = self._geometry()
        x = ops.as_nhwc(x)
        x2 = None if x2 is None else ops.as_nhwc(x2)
        n, _, h, w = x.shape
        ho, wo = ops.conv_out_size(h, w, k, s, p)
        ts = self._dense_tile_set(n, ho, wo, x.device)
        shape = (n, self.out_channels, ho, wo)
        if out is None:
            out = self._dense_buf("refresh_out", shape, x.device, x.dtype)
        res, kind, slope = None, _lib.ACT_NONE, 0.0
        if activation is not None:
            kind, slope = activation_kind(activation.op)
            r = activation.in_res.reservoir
            if r is None or tuple(r.shape) != shape or r.device != x.device:
                activation.in_res.reservoir = ops.new_nhwc(*shape, x.device)
            res = activation.in_res.reservoir
            activation._reset_incr()
        elif reserve is not None:
            r = reserve.reservoir
            if r is None or tuple(r.shape) != shape or r.device != x.device:
                reserve.reservoir = ops.new_nhwc(*shape, x.device)
            res = reserve.reservoir
        if filt is None:     # else: filter and bias in another column order, given together
            filt = self.conv2d_weights
            bias = None if self.bias is None else self.bias.detach()
        ops.conv_refresh(x, x2, filt, bias, k, s, p, ts, out, res, kind, slope, path,
                         None if addend is None else ops.as_nhwc(addend))
        return out


class nnConvIncrBase(nn.Conv2d, _ConvIncrMixin):
    """Reference :122-142."""

    def forward(self, x_incr):
        return self._incr_forward(x_incr)

    def forward_refresh_reservoirs(self, x):
        return self._refresh_forward(x)


class nnConvIncr(nn.Conv2d, _ConvIncrMixin):
    """Incremental conv: forward([d, m]) = [conv2d(d, W, bias=None), tile mask].

    Reference :146-196, where forward always falls back to a dense F.conv2d on
    the delta (:175-178); here only the active output tiles are computed.
    `path` selects the kernel (auto / VALU / MFMA), for tests and benchmarks.
    """

    def __init__(self, in_channels: int, out_channels: int, kernel_size, stride=1, padding=0,
                 bias=True):
        nn.Conv2d.__init__(self, in_channels, out_channels, kernel_size, stride, padding, bias=bias)
        self.kf = KFencedMaskModule(0.3)
        self.use_kf = False          # the reference leaves the quantiser switched off (:166)
        # Lossy input mask: pixels whose delta stays within +-in_threshold in every channel are dropped from
        # the input mask (the reference's mask definition, maxpool(abs(x)) >= thr with field 1,
        # incr_modules/utils.py:22-25); None = exact masks.  What is dropped is lost (no carry).
        self.in_threshold = None
        self.path = _lib.PATH_AUTO

    def load_state_dict(self, state_dict, strict: bool = True):
        ret = nn.Conv2d.load_state_dict(self, state_dict, strict=strict)
        self.__dict__.pop("_filt_cache", None)
        return ret

    @property
    def lossy(self) -> bool:
        return self.use_kf or self.in_threshold is not None

    def lossy_input(self, x_incr):
        """The delta quantiser and / or the threshold mask in front of the conv (both off by default)."""
        if self.use_kf:
            x_incr = self.kf(x_incr)
        if self.in_threshold is not None:
            x = ops.as_nhwc(x_incr[0])
            n, _, h, w = x.shape
            pix = ops.threshold_mask_lazy(x, float(self.in_threshold), self._pix_buf("thr_in", n, h, w, x.device))
            x_incr = [x, pix]
        return x_incr

    def forward(self, x_incr, x2_incr=None):
        return self._incr_forward(self.lossy_input(x_incr), x2_incr, path=self.path)

    def forward_fused(self, x_incr, activation: "nnReservedActivation", x2_incr=None,
                      addend_incr=None, filt=None):
        """conv (+ addend) + activation increment in one kernel; updates activation.in_res in place."""
        x_incr = self.lossy_input(x_incr)
        kind, slope = activation_kind(activation.op)
        res = activation.in_res.reservoir
        if res is None:
            raise RuntimeError("fused conv+activation: call forward_refresh_reservoirs first")
        return self._incr_forward(x_incr, x2_incr, reservoir=res, act=kind, slope=slope,
                                  path=self.path, out_name="out_act", addend_incr=addend_incr, filt=filt)

    def forward_fused_upsampled(self, up: "nnUpsample2xIncr", x_incr, skip_incr, activation: "nnReservedActivation"):
        """bilinear x2 of (x + skip) + conv + activation increment; one kernel when the shape allows it,
        else the up-sampling kernel followed by forward_fused."""
        k, s, p = self._geometry()
        x = x_incr[0]
        # Measured on MI355X.  bf16: the one-kernel form wins at every size (264x352 frame -3 %, 8x480x640
        # step -6 %).  fp32 on the fp32 matrix-core instruction: on planes of up to a few thousand tiles the step
        # is bound by launches and the one-kernel form wins (1.5 % of a 264x352 frame) unless the layer has more
        # than 4 staged chunks (256 channels: the per-chunk blend then costs what the saved launch gains); on
        # large planes the separate up-sampling kernel is cheaper (8x480x640 step +2 % with the one-kernel form).
        # fp32 in the three-term form: the one-kernel form wins at every size and depth (264x352 frame -0.4 %,
        # 8x480x640 step -1.8 %).
        dt = ops.delta_torch_dtype(x)
        tiles = x.shape[0] * ((2 * x.shape[2] + 7) // 8) * ((2 * x.shape[3] + 7) // 8)
        chunks = x.shape[1] // ops.mfma_chunk(dt)
        three_term = dt == torch.float32 and ops.f32x3_takes(k, s, x.shape[1], 0, self.out_channels)
        small = (dt == torch.bfloat16 or three_term
                 or (tiles <= ops.upconv_max_tiles and chunks <= ops.upconv_max_chunks))
        if self.lossy or not small or not ops.upconv_takes(x.shape[1], self.out_channels, k, s, p,
                                                            self.conv2d_weights, dt):
            return self.forward_fused(up(x_incr, skip_incr), activation)
        kind, slope = activation_kind(activation.op)
        res = activation.in_res.reservoir
        if res is None:
            raise RuntimeError("fused conv+activation: call forward_refresh_reservoirs first")
        return self._upconv_forward(up, x_incr, skip_incr, res, kind, slope)

    def forward_refresh_reservoirs(self, x):
        # The reference refreshes self.kf here unconditionally (:193): a norm and a zero clone
        # that nothing reads while kf.forward is not called (:166); done only when it is in use.
        if self.use_kf:
            self.kf.forward_refresh_reservoirs(x)
        return self._refresh_forward(x, path=self.path)

    def forward_refresh_fused(self, x, activation: "nnReservedActivation", x2=None, addend=None):
        """Dense conv + bias (+ addend) + activation, pre-activation written into activation.in_res."""
        if self.use_kf:
            self.kf.forward_refresh_reservoirs(x)
        return self._refresh_forward(x, x2, activation, path=self.path, addend=addend)


def set_kfence(net: nn.Module, tp: Optional[float], norm: str = "l2") -> int:
    """Switch the delta quantiser of every nnConvIncr in `net` on (threshold factor tp; at the next refresh
    k = tp*||x||_2, or tp*||x||_2/sqrt(numel) with norm="rms") or off (tp None).  Returns the number of convs
    touched; refresh afterwards."""
    count = 0
    for m in net.modules():
        if isinstance(m, nnConvIncr):
            m.use_kf = tp is not None
            if tp is not None:
                m.kf.tp = float(tp)
                m.kf.norm = norm
            count += 1
    return count


def set_input_threshold(net: nn.Module, thr: Optional[float]) -> int:
    """Threshold mask in front of every nnConvIncr of `net` (None: exact masks).  Returns the number of convs."""
    count = 0
    for m in net.modules():
        if isinstance(m, nnConvIncr):
            m.in_threshold = None if thr is None else float(thr)
            count += 1
    return count


class nnConvTranspose2dIncr(nn.ConvTranspose2d, _IncrBuffers):
    """Incremental transposed conv (named but not defined by the reference,
    incr_modules/e2depth_incr.py:248; semantics of transposed_conv2d_from_module,
    mask_incr_functional.py:64-66).  The decoder case -- stride 2, kernel 3 or 5, padding k // 2,
    output_padding 1, channel counts in whole staging chunks -- runs on the matrix cores
    (ops.tconv2x_masked: four sub-pixel phases, one or two inputs, optional addend); every other
    shape takes the gather kernel (ops.tconv_masked)."""

    def _filter(self) -> "ops.ConvFilter":
        w = self.weight
        tag = (w.data_ptr(), w._version, str(w.device))
        cached = self.__dict__.get("_filt_cache")
        if cached is None or cached[0] != tag:
            cached = (tag, ops.ConvFilter(w.detach().permute(0, 2, 3, 1).contiguous().float()))
            self.__dict__["_filt_cache"] = cached
        return cached[1]

    def _geometry(self):
        k = _square(self.kernel_size, "kernel_size")
        s, p = _square(self.stride, "stride"), _square(self.padding, "padding")
        op = _square(self.output_padding, "output_padding")
        if _square(self.dilation, "dilation") != 1 or self.groups != 1:
            raise NotImplementedError("transposed conv with dilation / groups")
        return k, s, p, op

    def forward(self, x_incr: Masked, reservoir=None, act=_lib.ACT_NONE, slope=0.0, x2_incr: Masked = None,
                addend_incr: Masked = None, filt=None, out_name="out") -> Masked:
        """x2_incr: second input (the conv runs over the channel concat of the two without forming it);
        addend_incr: delta added before the epilogue, covered by the output mask; filt: a row slice of
        self._filter() when only part of the input channels is fed.  Two inputs and the addend need the
        matrix-core form."""
        k, s, p, op = self._geometry()
        x, pix, _ = _unpack(x_incr)
        x2 = pix2 = None
        if x2_incr is not None:
            x2, pix2, _ = _unpack(x2_incr)
        n, c1, h, w = x.shape
        c2 = 0 if x2 is None else x2.shape[1]
        ho, wo = (h - 1) * s - 2 * p + k + op, (w - 1) * s - 2 * p + k + op
        ts = self._tile_set(out_name, n, ho, wo, x.device)
        out = self._delta_buf(out_name, (n, self.out_channels, ho, wo), x.device, x.dtype)
        if x2 is not None and (pix is None or pix2 is None):
            m1 = m2 = None
        else:
            m1, m2 = pix, pix2
        ops.build_mask_tiles(m1, m2, n, h, w, _lib.FOOT_TCONV, k, s, p, ts)
        filt = self._filter() if filt is None else filt
        if ops.tconv2x_takes(c1, c2, self.out_channels, k, s, p, op, filt, ops.delta_torch_dtype(x)):
            blocks = self._tile_set(out_name + "_blocks", n, h, w, x.device)
            ops.build_mask_tiles(ts, None, n, ho, wo, _lib.FOOT_CONV, 2, 2, 0, blocks)
            addend = None if addend_incr is None else ops.as_nhwc(addend_incr[0])
            ops.tconv2x_masked(x, pix, x2, pix2, filt, k, ts, blocks, out, reservoir, act, slope, addend)
            return [out, ts]
        if x2 is not None or addend_incr is not None:
            raise NotImplementedError("transposed conv over two inputs / with an addend needs the matrix-core form "
                                      "(stride 2, k in {3, 5}, padding k // 2, output_padding 1, channels in whole chunks)")
        ops.tconv_masked(x, pix, filt, k, s, p, ts, out, reservoir, act, slope)
        return [out, ts]

    def forward_refresh_reservoirs(self, x, x2=None, addend=None, filt=None, bias=None, reservoir=None,
                                   act=_lib.ACT_NONE, slope=0.0, out_name="refresh_out"):
        """conv_transpose2d(cat(x, x2), W, b) (+ addend) through the same kernels with every tile active."""
        self._reset_incr()
        ops._require_gpu(x, "x")
        k, s, p, op = self._geometry()
        x = ops.as_nhwc(x)
        x2 = None if x2 is None else ops.as_nhwc(x2)
        n, c1, h, w = x.shape
        c2 = 0 if x2 is None else x2.shape[1]
        ho, wo = (h - 1) * s - 2 * p + k + op, (w - 1) * s - 2 * p + k + op
        ts = self._dense_tile_set(n, ho, wo, x.device)
        out = self._dense_buf(out_name, (n, self.out_channels, ho, wo), x.device, x.dtype)
        if filt is None:
            filt = self._filter()
            bias = None if self.bias is None else self.bias.detach()
        if ops.tconv2x_takes(c1, c2, self.out_channels, k, s, p, op, filt, ops.delta_torch_dtype(x)):
            blocks = self._dense_tile_set(n, h, w, x.device)
            return ops.tconv2x_refresh(x, x2, filt, bias, k, ts, blocks, out, reservoir, act, slope,
                                       None if addend is None else ops.as_nhwc(addend))
        if x2 is not None or addend is not None:
            raise NotImplementedError("transposed conv over two inputs / with an addend needs the matrix-core form")
        return ops.tconv_refresh(x, filt, bias, k, s, p, ts, out, reservoir, act, slope)


class nnBatchNorm2dIncr(nn.BatchNorm2d, _IncrBuffers):
    """Reference :200-207: the linear part of the eval-mode batch norm on a delta, one masked kernel into a
    buffer the module keeps."""

    def forward(self, x_incr):
        delta, pix, tm = _unpack(x_incr)
        n, c, h, w = delta.shape
        if not isinstance(tm, TileMask):
            tm = self._tile_set("in", n, h, w, delta.device)
            ops.build_mask_tiles(pix, None, n, h, w, _lib.FOOT_CONV, 1, 1, 0, tm)
        out = self._delta_buf("out", (n, c, h, w), delta.device, delta.dtype)
        ops.scale_incr(delta, bn_scale(self), out, tm)
        return [out, tm]

    def forward_refresh_reservoirs(self, x):
        return super().forward(x)


class nnMaxPool2dIncr(nn.MaxPool2d, _IncrBuffers):
    """pool(R + d) - pool(R), then R += d (reference :210-224): one kernel over the active output
    tiles and a masked accumulate of the reservoir (square windows, no dilation, floor mode)."""

    def __init__(self, kernel_size, stride=None, padding=0):
        nn.MaxPool2d.__init__(self, kernel_size=kernel_size, stride=stride, padding=padding)
        self.functional = lambda x: F.max_pool2d(x, kernel_size=self.kernel_size,
                                                 stride=self.stride, padding=self.padding)
        self.mp_res = IncrementReserve()

    def forward(self, x_incr: Masked) -> Masked:
        if self.mp_res.reservoir is None:
            raise RuntimeError("nnMaxPool2dIncr: call forward_refresh_reservoirs first")
        if _square(self.dilation, "dilation") != 1 or self.ceil_mode or self.return_indices:
            raise NotImplementedError("incremental max pooling with dilation / ceil_mode / indices")
        k = _square(self.kernel_size, "kernel_size")
        s, p = _square(self.stride, "stride"), _square(self.padding, "padding")
        x, pix, _ = _unpack(x_incr)
        n, c, h, w = x.shape
        ho, wo = ops.conv_out_size(h, w, k, s, p)
        ts = self._tile_set("out", n, ho, wo, x.device)
        ops.build_mask_tiles(pix, None, n, h, w, _lib.FOOT_CONV, k, s, p, ts)
        out = self._delta_buf("out", (n, c, ho, wo), x.device, x.dtype)
        ops.maxpool_incr(x, pix, self.mp_res.reservoir, k, s, p, ts, out)
        in_tm = x_incr[1] if len(x_incr) > 1 else None
        if not isinstance(in_tm, TileMask):
            in_tm = self._tile_set("in", n, h, w, x.device)
            ops.build_mask_tiles(pix, None, n, h, w, _lib.FOOT_CONV, 1, 1, 0, in_tm)
        ops.accumulate(x, self.mp_res.reservoir, in_tm)
        return [out, ts]

    def forward_refresh_reservoirs(self, x: DenseT) -> DenseT:
        self._reset_incr()
        self.mp_res.update_reservoir(x)
        return super().forward(x)


class nnAdaptiveAvgPool2dIncr(nn.AdaptiveAvgPool2d):
    """Reference :228-233: adaptive average pooling of a delta; inactive pixels are not read.  The pooled
    delta is small and dense, so it carries no mask."""

    def forward(self, x_incr):
        delta, pix, _ = _unpack(x_incr)
        n, c, h, w = delta.shape
        size = self.output_size if isinstance(self.output_size, (tuple, list)) else (self.output_size,) * 2
        ho, wo = (h if size[0] is None else int(size[0])), (w if size[1] is None else int(size[1]))
        out = ops.new_nhwc(n, c, ho, wo, delta.device, delta.dtype)
        ops.avgpool_incr(delta, pix, out)
        return [out, None]

    def forward_refresh_reservoirs(self, x):
        return super().forward(x)


class nnSequentialIncr(nn.Sequential):
    """Reference :236-240."""

    def forward_refresh_reservoirs(self, x):
        for module in self:
            x = module.forward_refresh_reservoirs(x)
        return x


class nnReservedActivation(NonlinearPointOpIncr):
    """Activation increment with its own reservoir, updated in the same kernel
    (reference :243-256)."""

    def __init__(self, op=torch.relu, refine_mask: bool = True):
        nn.Module.__init__(self)
        self.in_res = IncrementReserve()
        NonlinearPointOpIncr.__init__(self, self.in_res, op, refine_mask)

    def forward(self, x_incr: Masked):
        return self._nonlin(x_incr, keep_reservoir=False)

    def forward_refresh_reservoirs(self, x: DenseT):
        out = NonlinearPointOpIncr.forward_refresh_reservoirs(self, x)
        self.in_res.update_reservoir(x)
        self._reset_incr()
        return out


class nnReluIncr(nnReservedActivation):
    def __init__(self):
        nnReservedActivation.__init__(self, torch.relu)


class nnSigmoidIncr(nnReservedActivation):
    def __init__(self):
        nnReservedActivation.__init__(self, torch.sigmoid)


class nnTanhIncr(nnReservedActivation):
    def __init__(self):
        nnReservedActivation.__init__(self, torch.tanh)


class nnAddIncr(IncrementMaskModule):
    """Sum of two deltas with the union of their masks (the skip / residual sum the
    reference writes as a tensor add, incr_modules/e2depth_incr.py:220,333)."""

    def forward(self, a_incr: Masked, b_incr: Masked, a_covers_b: bool = False) -> Masked:
        """a_covers_b: the caller knows that every active pixel of b is active in a (e.g. a is
        a same-padding conv chain applied to b); a's tile set is then used as is."""
        a, pa, ta = _unpack(a_incr)
        b, pb, _ = _unpack(b_incr)
        n, c, h, w = a.shape
        if a_covers_b and ta is not None:
            ts = ta
        else:
            ts = self._tile_set("union", n, h, w, a.device)
            ops.build_mask_tiles(pa, pb, n, h, w, _lib.FOOT_CONV, 1, 1, 0, ts)
        out = self._delta_buf("out", (n, c, h, w), a.device, a.dtype)
        ops.add_incr(a, pa, b, pb, out, ts)
        return [out, ts]

    def forward_refresh_reservoirs(self, a: DenseT, b: DenseT) -> DenseT:
        self._reset_incr()
        return a + b


class nnUpsample2xIncr(IncrementMaskModule):
    """Bilinear x2 of a delta (optionally of the sum of two deltas) on persistent
    buffers; module form of interpolate_from_module (mask_incr_functional.py:76-78)."""

    def forward(self, x_incr: Masked, skip_incr: Masked = None) -> Masked:
        a, pa, _ = _unpack(x_incr)
        b = pb = None
        if skip_incr is not None:
            b, pb, _ = _unpack(skip_incr)
        n, c, h, w = a.shape
        ts = self._tile_set("out", n, 2 * h, 2 * w, a.device)
        if skip_incr is not None and (pa is None or pb is None):
            m1 = m2 = None
        else:
            m1, m2 = pa, pb
        ops.build_mask_tiles(m1, m2, n, h, w, _lib.FOOT_UP2X, 0, 0, 0, ts)
        out = self._delta_buf("out", (n, c, 2 * h, 2 * w), a.device, a.dtype)
        ops.upsample2x_incr(a, pa, b, pb, ts, out)
        return [out, ts]

    def plan(self, x_incr: Masked, skip_incr: Masked = None):
        """Only the tile set of the up-sampled delta (for a consumer that up-samples on the fly):
        returns (a, mask a, b, mask b, tile set at twice the resolution)."""
        a, pa, _ = _unpack(x_incr)
        b = pb = None
        if skip_incr is not None:
            b, pb, _ = _unpack(skip_incr)
        n, c, h, w = a.shape
        ts = self._tile_set("out", n, 2 * h, 2 * w, a.device)
        if skip_incr is not None and (pa is None or pb is None):
            m1 = m2 = None
        else:
            m1, m2 = pa, pb
        ops.build_mask_tiles(m1, m2, n, h, w, _lib.FOOT_UP2X, 0, 0, 0, ts)
        return a, pa, b, pb, ts

    def forward_refresh_reservoirs(self, x: DenseT, skip: DenseT = None) -> DenseT:
        """up2x(x + skip) of dense tensors through the same kernel with every pixel and tile active."""
        self._reset_incr()
        ops._require_gpu(x, "x")
        a = ops.as_nhwc(x)
        b = None if skip is None else ops.as_nhwc(skip)
        n, c, h, w = a.shape
        ts = self._dense_tile_set(n, 2 * h, 2 * w, a.device)
        out = self._dense_buf("refresh_out", (n, c, 2 * h, 2 * w), a.device, a.dtype)
        ops.upsample2x_incr(a, None, b, None, ts, out)
        return out
