"""E2Depth / E2VID recurrent UNet in incremental form.

Restates incr_modules/e2depth_incr.py of the reference on the masked kernels:
same class names, constructor arguments, sub-module names (so state_dict keys
match) and the forward / forward_refresh_reservoirs pair.  Differences that
are deliberate:

* conv + activation run as one kernel (`fuse=True`), the ConvLSTM gate chain
  as one kernel (`fused=True`); the un-fused chains of the reference remain
  available and are what the fused ones are tested against;
* skip connections are mask-aware: the skip sum is folded into the bilinear
  up-sampling kernel (reference :333,429-431 add the tensors);
* three slips of the reference are not reproduced: `m1(...) + m2(...)`
  concatenates two lists and drops the m2 term (:113), `self.norm ==
  ['BN','IN']` is never true (:35), and the per-stage `print_sparsity` calls
  (:404-437) synchronise with the host inside the hot loop.
* `BaseE2VID` (an un-vendored dependency of the reference, :4) is replaced
  by a plain config dict on `E2VIDRecurrentIncr`.
"""
import contextlib

import torch
import torch.nn as nn
import torch.nn.functional as F

from . import _lib, ops
from .masked_types import DenseT, Masked, TileMask
from .mask_incr_functional import IncrementReserve, _unpack
from .mask_incr_modules import (_IncrBuffers, nnAddIncr, nnBatchNorm2dIncr, nnConvIncr,
                                nnConvTranspose2dIncr, nnReluIncr, nnReservedActivation,
                                nnReservedMultiplication, nnSigmoidIncr, nnTanhIncr,
                                nnUpsample2xIncr, activation_kind, activation_op)


def _mask_of(x_incr):
    return x_incr[1] if len(x_incr) > 1 else None


def _same_mask(a, b) -> bool:
    """Whether two mask slots name the same pixel mask in memory (None = all active on both sides)."""
    if a is None or b is None:
        return a is None and b is None
    pa = a.pixmask if isinstance(a, TileMask) else a
    pb = b.pixmask if isinstance(b, TileMask) else b
    return pa.data_ptr() == pb.data_ptr() and pa.shape == pb.shape and pa.dtype == pb.dtype


class ConvLayerIncr(nn.Module):
    """conv -> [BN] -> activation (reference :12-51)."""

    def __init__(self, in_channels, out_channels, kernel_size, stride=1, padding=0,
                 activation='relu', norm=None, fuse=True):
        super().__init__()
        bias = False if norm == 'BN' else True
        self.conv2d = nnConvIncr(in_channels, out_channels, kernel_size, stride, padding, bias=bias)
        if activation is not None:
            op = activation_op(activation)
            self.activation = nnReservedActivation(op)
        else:
            self.activation = None
        self.norm = norm
        if norm == 'BN':
            self.norm_layer = nnBatchNorm2dIncr(out_channels)
        elif norm == 'IN':
            raise NotImplementedError
        self.fuse = fuse

    def forward(self, x_incr: Masked, x2_incr: Masked = None) -> Masked:
        if self.fuse and self.activation is not None and self.norm not in ['BN', 'IN']:
            return self.conv2d.forward_fused(x_incr, self.activation, x2_incr)
        out_incr = self.conv2d(x_incr, x2_incr)
        if self.norm in ['BN', 'IN']:
            out_incr = self.norm_layer(out_incr)
        if self.activation is not None:
            out_incr = self.activation(out_incr)
        return out_incr

    def forward_refresh_reservoirs(self, x: DenseT):
        if self.fuse and self.activation is not None and self.norm not in ['BN', 'IN']:
            return self.conv2d.forward_refresh_fused(x, self.activation)
        out = self.conv2d.forward_refresh_reservoirs(x)
        if self.norm in ['BN', 'IN']:
            out = self.norm_layer.forward_refresh_reservoirs(out)
        if self.activation is not None:
            out = self.activation.forward_refresh_reservoirs(out)
        return out


class ConvLSTMIncr(nn.Module, _IncrBuffers):
    """Incremental ConvLSTM cell (reference :54-166).

    fused=True keeps three reservoirs -- gate pre-activations (4*hid channels),
    previous cell state, new cell state -- and runs the whole gate chain in
    one kernel after the gates conv; the concat of (input, previous hidden) is
    never formed (two-pointer conv input, and the hidden half is skipped when
    no previous-state delta is given).  fused=False runs the reference chain
    sigmoid1..3 / tanh1 / m1 / m2 / tanh2 / m3 module by module.
    """

    def __init__(self, input_size: int, hidden_size: int, kernel_size: int,
                 prev_c_res: IncrementReserve = None, fused: bool = True):
        super().__init__()
        self.input_size = input_size
        self.hidden_size = hidden_size
        self.kernel_size = kernel_size
        pad = kernel_size // 2
        self.zero_tensors = {}
        self.fused = fused
        self.Gates = nnConvIncr(input_size + hidden_size, 4 * hidden_size, kernel_size, padding=pad)
        self.m1 = nnReservedMultiplication()
        self.m2 = nnReservedMultiplication()
        self.m3 = nnReservedMultiplication()
        self.sigmoid1 = nnSigmoidIncr()
        self.sigmoid2 = nnSigmoidIncr()
        self.sigmoid3 = nnSigmoidIncr()
        self.tanh1 = nnTanhIncr()
        self.tanh2 = nnTanhIncr()
        self.add_cell = nnAddIncr()
        # reservoirs of the fused chain
        self.gates_res = IncrementReserve()
        self.cprev_res = IncrementReserve()
        self.cell_res = IncrementReserve()

    def forward(self, input_incr: Masked, prev_state_incr):
        prev_h_incr = prev_c_incr = None
        if prev_state_incr is not None:
            prev_h_incr, prev_c_incr = prev_state_incr
        if self.fused:
            return self._forward_fused(input_incr, prev_h_incr, prev_c_incr)
        return self._forward_chain(input_incr, prev_h_incr, prev_c_incr)

    # -- state buffers ---------------------------------------------------------------------------
    # The fused forms return the state deltas in buffers this module owns ([dh, ts], [dc, ts]).  A caller
    # may feed them back as the next step's previous state, and that step reads them (with a 3x3 halo, and
    # their pixel mask for the tile-set build) while it writes its own state: it must write elsewhere.  Two
    # sets of (dh, dc, tile set) are kept and a step takes the one its inputs do not live in.  Each set
    # has its own stale list, relative to the last step that wrote it, so every buffer stays a clean delta.
    @staticmethod
    def _ptrs_of(*state_incrs):
        used = set()
        for s_ in state_incrs:
            if s_ is None:
                continue
            used.add(s_[0].data_ptr())
            m = _mask_of(s_)
            if isinstance(m, TileMask):
                used.update((m.tiles.data_ptr(), m.pixmask.data_ptr()))
            elif torch.is_tensor(m):
                used.add(m.data_ptr())
        return used

    def _state_slot(self, prev_h_incr, prev_c_incr) -> int:
        used = self._ptrs_of(prev_h_incr, prev_c_incr)
        owned = self.__dict__.setdefault("_slot_ptrs", {})
        for slot in (0, 1):
            if not (owned.get(slot, set()) & used):
                return slot
        raise RuntimeError("ConvLSTMIncr: the previous state mixes buffers of both of this cell's state sets")

    def _own_slot(self, slot, dh, dc, ts):
        self.__dict__.setdefault("_slot_ptrs", {})[slot] = {
            dh.data_ptr(), dc.data_ptr(), ts.tiles.data_ptr(), ts.pixmask.data_ptr()}

    def _cover_prev_c(self, prev_h_incr, prev_c_incr):
        """The tile set of the gates conv is built from the masks of its two inputs; it must also cover the
        active pixels of the previous-cell delta.  Returns the mask to build with in place of the hidden
        one: the hidden mask itself when the cell delta has the same one (the usual case: both come from
        one earlier step), else the union of the two (all active if either is unmasked)."""
        if prev_c_incr is None:
            return None if prev_h_incr is None else _mask_of(prev_h_incr)
        mh = None if prev_h_incr is None else _mask_of(prev_h_incr)
        mc = _mask_of(prev_c_incr)
        if prev_h_incr is not None and _same_mask(mh, mc):
            return mh
        if mc is None or (prev_h_incr is not None and mh is None):
            return None
        c = ops.as_nhwc(prev_c_incr[0])
        pc = ops.pixel_mask_of(mc, c)
        if prev_h_incr is None:
            return pc
        n, _, h, w = c.shape
        ph = ops.pixel_mask_of(mh, c)
        union = self._tile_set("prev_union", n, h, w, c.device)
        ops.build_mask_tiles(ph, pc, n, h, w, _lib.FOOT_CONV, 1, 1, 0, union)
        return union

    # -- gates conv and gate chain in one kernel ------------------------------------------------
    def _gates_filter(self):
        """(ConvFilter, bias) of the gates conv in the gate-interleaved column order."""
        w = self.Gates.weight
        tag = (w.data_ptr(), w._version, str(w.device))
        cached = self.__dict__.get("_gates_filt_cache")
        if cached is None or cached[0] != tag:
            perm = ops.gate_interleave_index(self.hidden_size, w.device)
            filt = ops.ConvFilter(w.detach().permute(1, 2, 3, 0)[..., perm].contiguous().float())
            bias = None if self.Gates.bias is None else self.Gates.bias.detach()[perm].contiguous().float()
            cached = (tag, filt, bias)
            self.__dict__["_gates_filt_cache"] = cached
        return cached[1], cached[2]

    def _one_kernel_ok(self, x, hidden_present: bool) -> bool:
        """Whether the conv + gate chain kernel takes this cell: matrix-core shapes only."""
        chunk = ops.mfma_chunk(x.dtype)
        return (x.is_cuda and self.kernel_size == 3 and self.hidden_size % 8 == 0
                and self.input_size % chunk == 0 and (not hidden_present or self.hidden_size % chunk == 0)
                and self.Gates.path != _lib.PATH_VALU)

    def _gates_tile_set(self, name, x, pix, prev_h_incr, prev_c_incr, pix2):
        """Tile set of the gates conv for this step: footprint of the input mask and of the previous-state
        masks (the hidden delta is read through its OWN mask pix2; the build may use a wider one)."""
        cover = self._cover_prev_c(prev_h_incr, prev_c_incr)
        n, _, h, w = x.shape
        ts = self.Gates._tile_set(name, n, h, w, x.device)
        if prev_h_incr is None and prev_c_incr is None:
            m1, m2 = pix, None
        elif pix is None or cover is None:
            m1 = m2 = None
        else:
            m1, m2 = pix, ops.pixel_mask_of(cover, x)
        k = self.kernel_size
        ops.build_mask_tiles(m1, m2, n, h, w, _lib.FOOT_CONV, k, 1, k // 2, ts)
        return ts

    def _forward_one_kernel(self, input_incr, prev_h_incr, prev_c_incr):
        input_incr = self.Gates.lossy_input(input_incr)
        x, pix, _ = _unpack(input_incr)
        x2 = pix2 = None
        if prev_h_incr is not None:
            x2, pix2, _ = _unpack(prev_h_incr)
        n, _, h, w = x.shape
        hid = self.hidden_size
        slot = self._state_slot(prev_h_incr, prev_c_incr)
        sfx = "" if slot == 0 else "_b"
        ts = self._gates_tile_set("gates" + sfx, x, pix, prev_h_incr, prev_c_incr, pix2)
        dh = self._delta_buf("h" + sfx, (n, hid, h, w), x.device, x.dtype)
        dc = self._delta_buf("c" + sfx, (n, hid, h, w), x.device, x.dtype)
        self._own_slot(slot, dh, dc, ts)
        cp = cpm = None
        if prev_c_incr is not None:
            cp, cpm, _ = _unpack(prev_c_incr)
        filt, _ = self._gates_filter()
        ops.conv_gates_incr(x, pix, x2, pix2, filt, ts, self.gates_res.reservoir, cp, cpm,
                            self.cprev_res.reservoir, self.cell_res.reservoir, dh, dc)
        return [dh, ts], [dc, ts]

    def _forward_fused(self, input_incr, prev_h_incr, prev_c_incr):
        if self.gates_res.reservoir is None:
            raise RuntimeError("ConvLSTMIncr: call forward_refresh_reservoirs first")
        if self.__dict__.get("_gates_interleaved", False):
            if not self._one_kernel_ok(ops.as_nhwc(input_incr[0]), prev_h_incr is not None):
                raise RuntimeError("ConvLSTMIncr: the reservoirs were refreshed for the one-kernel form, which "
                                   "does not take this input (dtype / previous hidden state); refresh again")
            return self._forward_one_kernel(input_incr, prev_h_incr, prev_c_incr)
        slot = self._state_slot(prev_h_incr, prev_c_incr)
        sfx = "" if slot == 0 else "_b"
        input_incr = self.Gates.lossy_input(input_incr)
        x, pix, _ = _unpack(input_incr)
        x2 = pix2 = None
        if prev_h_incr is not None:
            x2, pix2, _ = _unpack(prev_h_incr)
        n, _, h, w = x.shape
        hid = self.hidden_size
        ts = self._gates_tile_set("out" + sfx, x, pix, prev_h_incr, prev_c_incr, pix2)
        gates = self.Gates._delta_buf("out", (n, 4 * hid, h, w), x.device, x.dtype)
        k = self.kernel_size
        ops.conv_masked(x, pix, x2, pix2, self.Gates.conv2d_weights, k, 1, k // 2, ts, gates, path=self.Gates.path)
        dh = self._delta_buf("h" + sfx, (n, hid, h, w), gates.device, gates.dtype)
        dc = self._delta_buf("c" + sfx, (n, hid, h, w), gates.device, gates.dtype)
        self._own_slot(slot, dh, dc, ts)
        cp = cpm = None
        if prev_c_incr is not None:
            cp, cpm, _ = _unpack(prev_c_incr)
        ops.convlstm_gates_incr(gates, self.gates_res.reservoir, cp, cpm, self.cprev_res.reservoir,
                                self.cell_res.reservoir, dh, dc, ts)
        return [dh, ts], [dc, ts]

    def _forward_chain(self, input_incr, prev_h_incr, prev_c_incr):
        gates_incr = self.Gates(input_incr, prev_h_incr)
        ts = gates_incr[1]
        in_gate, remember_gate, out_gate, cell_gate = gates_incr[0].chunk(4, 1)
        in_gate = self.sigmoid1([in_gate, ts])
        remember_gate = self.sigmoid2([remember_gate, ts])
        out_gate = self.sigmoid3([out_gate, ts])
        cell_gate = self.tanh1([cell_gate, ts])
        cell = self.m1(in_gate, cell_gate)
        if prev_c_incr is None:
            # d(f * c_prev) with dc_prev = 0 is df * c_prev: the product rule with a zero delta
            zero = self._delta_buf("zero_c", tuple(cell[0].shape), cell[0].device, cell[0].dtype)
            prev_c_incr = [zero, remember_gate[1]]
        cell = self.add_cell(cell, self.m2(remember_gate, prev_c_incr))
        cell_tanh = self.tanh2(cell)
        hidden = self.m3(out_gate, cell_tanh)
        return hidden, cell

    def _refresh_state(self, input_, prev_c, interleaved):
        """Dense (hidden, cell) from the gate pre-activations the conv refresh left in gates_res, and the
        cell reservoirs of the gate chain, in one kernel."""
        n, _, h, w = input_.shape
        dev, hid = input_.device, self.hidden_size
        for res in (self.cprev_res, self.cell_res):
            r = res.reservoir
            if r is None or tuple(r.shape) != (n, hid, h, w) or r.device != dev:
                res.reservoir = ops.new_nhwc(n, hid, h, w, dev)
        dt = ops.delta_torch_dtype(input_)
        hidden = self._dense_buf("h_refresh", (n, hid, h, w), dev, dt)
        cell = self._dense_buf("c_refresh", (n, hid, h, w), dev, dt)
        if prev_c is not None:
            prev_c = ops.as_nhwc(prev_c.to(dt))      # may be `cell` itself (the last refresh's state fed back)
        ops.convlstm_gates_refresh(self.gates_res.reservoir, interleaved, prev_c, self.cprev_res.reservoir,
                                   self.cell_res.reservoir, hidden, cell)
        return hidden, cell

    def forward_refresh_reservoirs(self, input_, prev_state):
        """Dense (hidden, cell).  With fused=True both are views of buffers this module owns and the next refresh
        overwrites them in place (the reference returns fresh tensors): clone what must outlive it."""
        batch_size = input_.data.size()[0]
        spatial_size = input_.data.size()[2:]
        if prev_state is None:
            state_size = tuple([batch_size, self.hidden_size] + list(spatial_size))
            zkey = state_size + (input_.dtype,)
            if zkey not in self.zero_tensors:
                self.zero_tensors[zkey] = tuple(
                    torch.zeros(state_size, device=input_.device, dtype=input_.dtype).to(memory_format=torch.channels_last)
                    for _ in range(2))
            prev_state = self.zero_tensors[zkey]
        zero_state = prev_state is self.zero_tensors.get(
            tuple([batch_size, self.hidden_size] + list(spatial_size)) + (input_.dtype,))
        prev_h, prev_c = prev_state
        self._reset_incr()
        # buffer ownership of the two state sets is told by raw addresses: forget them here, so that an address the
        # allocator has reused since (a shape or device change frees the old buffers) cannot be mistaken for one
        self.__dict__.pop("_slot_ptrs", None)
        if self.Gates.use_kf:
            self.Gates.kf.forward_refresh_reservoirs(input_)
        # the concat is never formed: two-pointer conv input, hidden half skipped when it is zero
        if self.fused:
            # the fp32 gate pre-activations go straight into their reservoir; the state is
            # computed from them in fp32 and handed on in the dtype of the input
            one_kernel = self._one_kernel_ok(input_, True)
            self.__dict__["_gates_interleaved"] = one_kernel
            if one_kernel:
                # reservoir in the gate-interleaved column order of the conv + gate chain kernel
                filt, bias = self._gates_filter()
                self.Gates._refresh_forward(input_, None if zero_state else prev_h, path=self.Gates.path,
                                            reserve=self.gates_res, filt=filt, bias=bias)
            else:
                self.Gates._refresh_forward(input_, None if zero_state else prev_h, path=self.Gates.path,
                                            reserve=self.gates_res)
            return self._refresh_state(input_, None if zero_state else prev_c, one_kernel)
        gates = self.Gates._refresh_forward(input_, None if zero_state else prev_h, path=self.Gates.path)
        in_gate, remember_gate, out_gate, cell_gate = gates.chunk(4, 1)
        in_gate = self.sigmoid1.forward_refresh_reservoirs(in_gate)
        remember_gate = self.sigmoid2.forward_refresh_reservoirs(remember_gate)
        out_gate = self.sigmoid3.forward_refresh_reservoirs(out_gate)
        cell_gate = self.tanh1.forward_refresh_reservoirs(cell_gate)
        cell = self.m1.forward_refresh_reservoirs(in_gate, cell_gate) + \
            self.m2.forward_refresh_reservoirs(remember_gate, prev_c)
        self.add_cell.forward_refresh_reservoirs(cell, cell)
        cell_tanh = self.tanh2.forward_refresh_reservoirs(cell)
        hidden = self.m3.forward_refresh_reservoirs(out_gate, cell_tanh)
        return hidden, cell


class RecurrentConvLayerIncr(nn.Module):
    """Reference :169-186."""

    def __init__(self, in_channels, out_channels, kernel_size=3, stride=1, padding=0,
                 recurrent_block_type='convlstm', activation='relu', norm=None, fuse=True):
        super().__init__()
        assert recurrent_block_type == 'convlstm'
        self.conv = ConvLayerIncr(in_channels, out_channels, kernel_size, stride, padding,
                                  activation, norm, fuse=fuse)
        self.recurrent_block = ConvLSTMIncr(input_size=out_channels, hidden_size=out_channels,
                                            kernel_size=3, fused=fuse)

    def forward(self, x_incr, prev_state_incr):
        x_incr = self.conv(x_incr)
        state_incr = self.recurrent_block(x_incr, prev_state_incr)
        x_incr = state_incr[0]
        return x_incr, state_incr

    def forward_refresh_reservoirs(self, x: DenseT, prev_state):
        x = self.conv.forward_refresh_reservoirs(x)
        state = self.recurrent_block.forward_refresh_reservoirs(x, prev_state)
        x = state[0]
        return x, state


class ResidualBlockIncr(nn.Module):
    """conv-relu-conv, + residual, relu (reference :189-240)."""

    def __init__(self, in_channels, out_channels, stride=1, downsample=None, norm=None, fuse=True):
        super().__init__()
        bias = False if norm == 'BN' else True
        self.conv1 = nnConvIncr(in_channels, out_channels, kernel_size=3, stride=stride, padding=1, bias=bias)
        self.norm = norm
        if norm == 'BN':
            self.bn1 = nnBatchNorm2dIncr(out_channels)
            self.bn2 = nnBatchNorm2dIncr(out_channels)
        elif norm == 'IN':
            raise NotImplementedError
        self.relu1 = nnReluIncr()
        self.conv2 = nnConvIncr(out_channels, out_channels, kernel_size=3, stride=1, padding=1, bias=bias)
        self.relu2 = nnReluIncr()
        self.relu2.refine_mask = not fuse     # the structural mask is passed through when fused
        self.downsample = downsample
        self.add = nnAddIncr()
        self.fuse = fuse

    def forward(self, x_incr: Masked) -> Masked:
        residual_incr = x_incr
        if self.fuse and self.norm not in ['BN', 'IN']:
            out_incr = self.conv1.forward_fused(x_incr, self.relu1)
        else:
            out_incr = self.conv1(x_incr)
            if self.norm in ['BN', 'IN']:
                out_incr = self.bn1(out_incr)
            out_incr = self.relu1(out_incr)
        if self.fuse and self.norm not in ['BN', 'IN'] and not self.downsample:
            # conv2 + residual + relu2 in one kernel: conv2(relu(conv1(x))) reaches every active
            # pixel of x (two same-padding 3x3), so the residual delta rides in as the addend
            return self.conv2.forward_fused(out_incr, self.relu2, addend_incr=residual_incr)
        out_incr = self.conv2(out_incr)
        if self.norm in ['BN', 'IN']:
            out_incr = self.bn2(out_incr)
        if self.downsample:
            residual_incr = self.downsample(x_incr)
        out_incr = self.add(out_incr, residual_incr, a_covers_b=not self.downsample)
        out_incr = self.relu2(out_incr)
        return out_incr

    def forward_refresh_reservoirs(self, x):
        residual = x
        if self.fuse and self.norm not in ['BN', 'IN']:
            out = self.conv1.forward_refresh_fused(x, self.relu1)
        else:
            out = self.conv1.forward_refresh_reservoirs(x)
            if self.norm in ['BN', 'IN']:
                out = self.bn1.forward_refresh_reservoirs(out)
            out = self.relu1.forward_refresh_reservoirs(out)
        if self.fuse and self.norm not in ['BN', 'IN'] and not self.downsample:
            return self.conv2.forward_refresh_fused(out, self.relu2, addend=residual)
        out = self.conv2.forward_refresh_reservoirs(out)
        if self.norm in ['BN', 'IN']:
            out = self.bn2.forward_refresh_reservoirs(out)
        if self.downsample:
            residual = self.downsample.forward_refresh_reservoirs(x)
        out = self.add.forward_refresh_reservoirs(out, residual)
        out = self.relu2.forward_refresh_reservoirs(out)
        return out


class TransposedConvLayerIncr(nn.Module):
    """Transposed conv (stride 2, output_padding 1) -> activation (reference :243-282)."""

    def __init__(self, in_channels, out_channels, kernel_size, stride=1, padding=0,
                 activation='relu', norm=None, fuse=True):
        super().__init__()
        bias = False if norm == 'BN' else True
        self.transposed_conv2d = nnConvTranspose2dIncr(
            in_channels, out_channels, kernel_size, stride=2, padding=padding, output_padding=1, bias=bias)
        self.activation = None
        if activation is not None:
            op = activation_op(activation)
            self.activation = nnReservedActivation(op)
        self.norm = norm
        if norm == 'BN':
            self.norm_layer = nnBatchNorm2dIncr(out_channels)
        elif norm == 'IN':
            raise NotImplementedError
        self.add = nnAddIncr()
        self.fuse = fuse

    def forward(self, x_incr: Masked, skip_incr: Masked = None) -> Masked:
        if skip_incr is not None:
            x_incr = self.add(x_incr, skip_incr)
        if self.fuse and self.activation is not None and self.norm not in ['BN', 'IN']:
            kind, slope = activation_kind(self.activation.op)
            return self.transposed_conv2d(x_incr, self.activation.in_res.reservoir, kind, slope)
        out_incr = self.transposed_conv2d(x_incr)
        if self.norm in ['BN', 'IN']:
            out_incr = self.norm_layer(out_incr)
        if self.activation is not None:
            out_incr = self.activation(out_incr)
        return out_incr

    def forward_refresh_reservoirs(self, x, skip=None):
        if skip is not None:
            x = self.add.forward_refresh_reservoirs(x, skip)
        out = self.transposed_conv2d.forward_refresh_reservoirs(x)
        if self.norm in ['BN', 'IN']:
            out = self.norm_layer.forward_refresh_reservoirs(out)
        if self.activation is not None:
            out = self.activation.forward_refresh_reservoirs(out)
        return out


class UpsampleConvLayerIncr(nn.Module):
    """bilinear x2 -> conv -> activation (reference :284-322); the skip sum of the
    UNet is taken inside the up-sampling kernel."""

    def __init__(self, in_channels, out_channels, kernel_size, stride=1, padding=0,
                 activation='relu', norm=None, fuse=True):
        super().__init__()
        bias = False if norm == 'BN' else True
        self.conv2d = nnConvIncr(in_channels, out_channels, kernel_size, stride, padding, bias=bias)
        if activation is not None:
            op = activation_op(activation)
            self.activation = nnReservedActivation(op)
        else:
            self.activation = None
        self.norm = norm
        if norm == 'BN':
            self.norm_layer = nnBatchNorm2dIncr(out_channels)
        elif norm == 'IN':
            raise NotImplementedError
        self.upsample = nnUpsample2xIncr()
        self.fuse = fuse

    def forward(self, x_incr: Masked, skip_incr: Masked = None) -> Masked:
        if self.fuse and self.activation is not None and self.norm not in ['BN', 'IN']:
            # up-sampling, skip sum, conv and activation in one kernel where the shape allows it
            return self.conv2d.forward_fused_upsampled(self.upsample, x_incr, skip_incr, self.activation)
        x_upsampled_incr = self.upsample(x_incr, skip_incr)
        out_incr = self.conv2d(x_upsampled_incr)
        if self.norm in ['BN', 'IN']:
            out_incr = self.norm_layer(out_incr)
        if self.activation is not None:
            out_incr = self.activation(out_incr)
        return out_incr

    def forward_refresh_reservoirs(self, x, skip=None):
        x_upsampled = self.upsample.forward_refresh_reservoirs(x, skip)
        if self.fuse and self.activation is not None and self.norm not in ['BN', 'IN']:
            return self.conv2d.forward_refresh_fused(x_upsampled, self.activation)
        out = self.conv2d.forward_refresh_reservoirs(x_upsampled)
        if self.norm in ['BN', 'IN']:
            out = self.norm_layer.forward_refresh_reservoirs(out)
        if self.activation is not None:
            out = self.activation.forward_refresh_reservoirs(out)
        return out


class BaseUNetIncr(nn.Module):
    """Reference :325-377."""

    def __init__(self, num_input_channels, num_output_channels=1, skip_type='sum', activation='sigmoid',
                 num_encoders=4, base_num_channels=32, num_residual_blocks=2, norm=None,
                 use_upsample_conv=True, fuse=True):
        super().__init__()
        self.num_input_channels = num_input_channels
        self.num_output_channels = num_output_channels
        self.skip_type = skip_type
        if skip_type != 'sum':
            raise NotImplementedError("E2Depth-incr is built with skip_type='sum'")
        self.norm = norm
        self.fuse = fuse
        self.UpsampleLayer = UpsampleConvLayerIncr if use_upsample_conv else TransposedConvLayerIncr
        self.num_encoders = num_encoders
        self.base_num_channels = base_num_channels
        self.num_residual_blocks = num_residual_blocks
        self.max_num_channels = self.base_num_channels * pow(2, self.num_encoders)
        assert self.num_input_channels > 0
        assert self.num_output_channels > 0
        self.encoder_input_sizes = [self.base_num_channels * pow(2, i) for i in range(self.num_encoders)]
        self.encoder_output_sizes = [self.base_num_channels * pow(2, i + 1) for i in range(self.num_encoders)]
        op = activation_op(activation)
        self.activation = nnReservedActivation(op, refine_mask=not fuse)

    def build_resblocks(self):
        self.resblocks = nn.ModuleList()
        for _ in range(self.num_residual_blocks):
            self.resblocks.append(ResidualBlockIncr(self.max_num_channels, self.max_num_channels,
                                                    norm=self.norm, fuse=self.fuse))

    def build_decoders(self):
        decoder_input_sizes = list(reversed([self.base_num_channels * pow(2, i + 1)
                                             for i in range(self.num_encoders)]))
        self.decoders = nn.ModuleList()
        for input_size in decoder_input_sizes:
            self.decoders.append(self.UpsampleLayer(input_size, input_size // 2, kernel_size=5,
                                                    padding=2, norm=self.norm, fuse=self.fuse))

    def build_prediction_layer(self):
        self.pred = ConvLayerIncr(self.base_num_channels, self.num_output_channels, 1,
                                  activation=None, norm=self.norm, fuse=self.fuse)
        self.pred_add = nnAddIncr()


class UNetRecurrentIncr(BaseUNetIncr):
    """Recurrent UNet: head, stride-2 conv + ConvLSTM encoders, residual blocks,
    up-sampling decoders with skip sums, 1x1 prediction + sigmoid (reference :380-468)."""

    def __init__(self, num_input_channels, num_output_channels=1, skip_type='sum',
                 recurrent_block_type='convlstm', activation='sigmoid', num_encoders=4,
                 base_num_channels=32, num_residual_blocks=2, norm=None, use_upsample_conv=True,
                 fuse=True):
        super().__init__(num_input_channels, num_output_channels, skip_type, activation,
                         num_encoders, base_num_channels, num_residual_blocks, norm,
                         use_upsample_conv, fuse)
        self.head = ConvLayerIncr(self.num_input_channels, self.base_num_channels,
                                  kernel_size=5, stride=1, padding=2, fuse=fuse)
        self.encoders = nn.ModuleList()
        for input_size, output_size in zip(self.encoder_input_sizes, self.encoder_output_sizes):
            self.encoders.append(RecurrentConvLayerIncr(input_size, output_size, kernel_size=5,
                                                        stride=2, padding=2,
                                                        recurrent_block_type=recurrent_block_type,
                                                        norm=self.norm, fuse=fuse))
        self.build_resblocks()
        self.build_decoders()
        self.build_prediction_layer()

    def forward(self, x_incr: Masked, prev_states_incr):
        x_incr = self.head(x_incr)
        head = x_incr
        if prev_states_incr is None:
            prev_states_incr = [None] * self.num_encoders
        blocks = []
        states_incr = []
        for i, encoder in enumerate(self.encoders):
            x_incr, state_incr = encoder(x_incr, prev_states_incr[i])
            blocks.append(x_incr)
            states_incr.append(state_incr)
        for resblock in self.resblocks:
            x_incr = resblock(x_incr)
        for i, decoder in enumerate(self.decoders):
            if i == self.num_encoders - 1 and self._tail_is_fusable(decoder, x_incr, head):
                # last decoder, skip sum, prediction conv and output activation in one kernel
                return self._fused_tail(decoder, x_incr, blocks[0], head), states_incr
            x_incr = decoder(x_incr, blocks[self.num_encoders - i - 1])
        if self.fuse and self.norm not in ['BN', 'IN']:
            # skip sum, 1x1 conv and output activation in one kernel: the conv is linear, so
            # pred(x + head) is the conv of the two tensors side by side with the filter rows repeated
            # (the pre-activation reservoir is the activation's)
            pred_incr = self.pred.conv2d.forward_fused(x_incr, self.activation, x2_incr=head,
                                                       filt=self._pred_sum_filter())
        else:
            pred_incr = self.activation(self.pred(self.pred_add(x_incr, head)))
        return pred_incr, states_incr

    def _tail_is_fusable(self, decoder, x_incr, head) -> bool:
        """The shape ops.upconv_pred_masked takes: up-sampling decoder 64 -> 32 with a ReLU-kind activation on bf16
        deltas, exact masks, one prediction channel, a plane of at least 2048 tiles."""
        if not (self.fuse and self.norm not in ['BN', 'IN'] and isinstance(decoder, UpsampleConvLayerIncr)
                and decoder.activation is not None and self.num_output_channels == 1):
            return False
        conv, pconv = decoder.conv2d, self.pred.conv2d
        if conv.lossy or pconv.lossy or not isinstance(head[1] if len(head) > 1 else None, TileMask):
            return False
        x = x_incr[0]
        k, s, p = conv._geometry()
        tiles = x.shape[0] * ((2 * x.shape[2] + 7) // 8) * ((2 * x.shape[3] + 7) // 8)
        try:
            kind, _ = activation_kind(decoder.activation.op)
        except NotImplementedError:
            return False
        return ops.upconv_pred_takes(x.shape[1], conv.out_channels, k, s, p, conv.conv2d_weights,
                                     ops.delta_torch_dtype(x), tiles, kind)

    def _fused_tail(self, decoder, x_incr, skip_incr, head):
        conv, pconv, up = decoder.conv2d, self.pred.conv2d, decoder.upsample
        k, s, p = conv._geometry()
        a, pa, b, pb, ts_up = up.plan(x_incr, skip_incr)
        n, _, h, w = a.shape
        H, W = 2 * h, 2 * w
        ts_dec = conv._tile_set("out_act", n, H, W, a.device)           # the decoder's own output set ...
        ops.build_mask_tiles(ts_up, None, n, H, W, _lib.FOOT_CONV, k, s, p, ts_dec)
        ts_pred = pconv._tile_set("out_act", n, H, W, a.device)          # ... and the prediction's: its union with the head's
        ops.build_mask_tiles(ts_dec, head[1], n, H, W, _lib.FOOT_CONV, 1, 1, 0, ts_pred)
        res, pres = decoder.activation.in_res.reservoir, self.activation.in_res.reservoir
        if res is None or pres is None:
            raise RuntimeError("fused tail: call forward_refresh_reservoirs first")
        kind, slope = activation_kind(decoder.activation.op)
        pkind, pslope = activation_kind(self.activation.op)
        out = pconv._delta_buf("out_act", (n, 1, H, W), a.device, a.dtype)
        ops.upconv_pred_masked(a, pa, b, pb, conv.conv2d_weights, ts_pred, res, kind, slope, ops.as_nhwc(head[0]), head[1],
                               self._pred_tail_weights(), pres, pkind, pslope, out)
        return [out, ts_pred]

    def _pred_tail_weights(self):
        base = self.pred.conv2d.conv2d_weights
        cached = self.__dict__.get("_pred_tail_w")
        if cached is None or cached[0] is not base:
            # [Cin, 1, 1, 1] -> (1, Cin), rounded to bf16 like every weight a bf16 network multiplies
            row = base.for_dtype(torch.bfloat16)[0].reshape(1, -1).float()
            cached = (base, torch.cat((row, row), 0).contiguous())
            self.__dict__["_pred_tail_w"] = cached
        return cached[1]

    def _pred_sum_filter(self):
        base = self.pred.conv2d.conv2d_weights
        cached = self.__dict__.get("_pred_sum_filt")
        if cached is None or cached[0] is not base:
            cached = (base, ops.ConvFilter(torch.cat((base.plain, base.plain), 0).contiguous()))
            self.__dict__["_pred_sum_filt"] = cached
        return cached[1]

    def forward_refresh_reservoirs(self, x: DenseT, prev_states):
        x = self.head.forward_refresh_reservoirs(x)
        head = x
        if prev_states is None:
            prev_states = [None] * self.num_encoders
        blocks = []
        states = []
        for i, encoder in enumerate(self.encoders):
            x, state = encoder.forward_refresh_reservoirs(x, prev_states[i])
            blocks.append(x)
            states.append(state)
        for resblock in self.resblocks:
            x = resblock.forward_refresh_reservoirs(x)
        for i, decoder in enumerate(self.decoders):
            x = decoder.forward_refresh_reservoirs(x, blocks[self.num_encoders - i - 1])
        if self.fuse and self.norm not in ['BN', 'IN'] and not self.pred.conv2d.use_kf:
            # as in forward: pred(x + head) as the conv of the two tensors side by side
            conv = self.pred.conv2d
            pred = conv._refresh_forward(x, head, self.activation, path=conv.path, filt=self._pred_sum_filter(),
                                         bias=None if conv.bias is None else conv.bias.detach())
        else:
            summed = self.pred_add.forward_refresh_reservoirs(x, head)
            pred = self.activation.forward_refresh_reservoirs(self.pred.forward_refresh_reservoirs(summed))
        return pred, states


E2DEPTH_DEFAULT_CONFIG = dict(num_bins=5, skip_type='sum', num_encoders=3, base_num_channels=32,
                              num_residual_blocks=2, norm=None, use_upsample_conv=True,
                              recurrent_block_type='convlstm')


class E2VIDRecurrentIncr(nn.Module, _IncrBuffers):
    """E2Depth-incr / E2VID-incr (reference :471-498).

    `config` is a dict (keys of E2DEPTH_DEFAULT_CONFIG; missing keys take the
    defaults, which give the network traced in the reference's todo.txt:34-57).
    When the input pair carries no mask (the reference drivers pass
    `(x_t - x_{t-1}, None)`), the pixel mask is derived on the device as
    any_c(|delta| > mask_threshold).
    """

    def __init__(self, config=None, fuse=True, mask_threshold: float = 0.0, derive_input_mask=True,
                 async_masks=False, plan_first=False):
        super().__init__()
        self.async_masks = async_masks     # build the tile sets on a second stream, ahead of the convs
        # with async_masks: walk the network twice per step, first launching only the mask builds, then
        # only the other kernels (needs masks that depend on the input mask alone: no refined masks, no
        # delta quantisers)
        self.plan_first = plan_first
        cfg = dict(E2DEPTH_DEFAULT_CONFIG)
        cfg.update(config or {})
        self.num_bins = int(cfg['num_bins'])
        self.skip_type = str(cfg['skip_type'])
        self.num_encoders = int(cfg['num_encoders'])
        self.base_num_channels = int(cfg['base_num_channels'])
        self.num_residual_blocks = int(cfg['num_residual_blocks'])
        self.norm = cfg['norm']
        self.use_upsample_conv = bool(cfg['use_upsample_conv'])
        self.recurrent_block_type = str(cfg['recurrent_block_type'])
        self.mask_threshold = float(mask_threshold)
        self.derive_input_mask = derive_input_mask
        self.unetrecurrent = UNetRecurrentIncr(num_input_channels=self.num_bins,
                                               num_output_channels=1,
                                               skip_type=self.skip_type,
                                               recurrent_block_type=self.recurrent_block_type,
                                               activation='sigmoid',
                                               num_encoders=self.num_encoders,
                                               base_num_channels=self.base_num_channels,
                                               num_residual_blocks=self.num_residual_blocks,
                                               norm=self.norm,
                                               use_upsample_conv=self.use_upsample_conv,
                                               fuse=fuse)

    def input_mask(self, delta: torch.Tensor) -> torch.Tensor:
        n, _, h, w = delta.shape
        pix = self._pix_buf("input", n, h, w, delta.device)
        return ops.mask_from_delta(delta, self.mask_threshold, pix)

    def forward(self, event_tensor: Masked, prev_states):
        ops.require_no_lookahead(self)
        delta = ops.as_nhwc(event_tensor[0])
        mask = _mask_of(event_tensor)
        if not self.async_masks and not self.plan_first:
            if mask is None and self.derive_input_mask:
                mask = self.input_mask(delta)
            return self.unetrecurrent.forward([delta, mask], prev_states)
        # (plan_first without async_masks: the planning pass runs on the compute stream, ahead of the compute pass)
        with (ops.mask_planner(delta.device) if self.async_masks else contextlib.nullcontext()):
            if mask is None and self.derive_input_mask:
                mask = self.input_mask(delta)
            if self.plan_first:
                with ops.network_pass("plan"):
                    self.unetrecurrent.forward([delta, mask], prev_states)
                with ops.network_pass("compute"):
                    img_pred, states = self.unetrecurrent.forward([delta, mask], prev_states)
            else:
                img_pred, states = self.unetrecurrent.forward([delta, mask], prev_states)
        return img_pred, states

    def _lookahead_parts(self, delta):
        n, _, h, w = delta.shape

        def make_mask(d):
            return self.input_mask(d) if self.derive_input_mask else None

        def mask_buffer(d):
            return self._pix_buf("input", n, h, w, d.device) if self.derive_input_mask else None
        return (self.__dict__.setdefault("_pipe", {}), make_mask, mask_buffer,
                lambda d, m: self.unetrecurrent.forward([d, m], None))

    def forward_pipelined(self, event_tensor: Masked, next_event_tensor: Masked, parity: int):
        """forward(event_tensor, None) with the tile sets of the NEXT step -- whose delta, next_event_tensor, must
        already hold its values -- planned on a second stream while this step computes (ops.pipelined_step: the
        plan, 7 % of a 264x352 step, leaves the critical path).  parity alternates 0 / 1 from call to call; the
        next call must be for the delta announced here.  None as next_event_tensor: no look-ahead (last step).
        Exact masks only (no delta quantiser, no thresholds), previous states None."""
        delta = ops.as_nhwc(event_tensor[0])
        nxt = None if next_event_tensor is None else ops.as_nhwc(next_event_tensor[0])
        state, make_mask, mask_buffer, walk = self._lookahead_parts(delta)
        return ops.pipelined_step(state, parity, delta, nxt, make_mask, mask_buffer, walk)

    def plan_ahead(self, event_tensor: Masked, parity: int) -> None:
        """The planning half of forward_pipelined, on the current stream: input mask and every tile set of the step
        that will take event_tensor with this parity (ops.plan_step_ahead has the ordering the caller owes)."""
        delta = ops.as_nhwc(event_tensor[0])
        state, make_mask, _, walk = self._lookahead_parts(delta)
        ops.plan_step_ahead(state, parity, delta, make_mask, walk)

    def forward_planned(self, event_tensor: Masked, parity: int):
        """The compute half: forward(event_tensor, None) over the tile sets plan_ahead built for this parity."""
        delta = ops.as_nhwc(event_tensor[0])
        state, make_mask, mask_buffer, walk = self._lookahead_parts(delta)
        return ops.run_planned_step(state, parity, delta, make_mask, mask_buffer, walk)

    def forward_refresh_reservoirs(self, event_tensor: DenseT, prev_states):
        ops.drop_lookahead(self)
        img_pred, states = self.unetrecurrent.forward_refresh_reservoirs(event_tensor, prev_states)
        return img_pred, states
