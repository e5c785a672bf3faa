"""Recurrent multi-resolution EV-FlowNet (ConvGRU) in incremental form.

Restates incr_modules/evflownet_incr.py of the reference on the masked kernels:
same class names, constructor arguments and sub-module names, the forward /
forward_refresh_reservoirs pair, stride-2 3x3 encoders each followed by a
ConvGRU, two residual blocks, decoders with concatenated skips and a 2-channel
tanh flow head per scale whose prediction is fed to the next decoder.

What differs on purpose:
* The concat of (previous flow, x, skip) in front of a decoder is never formed
  for the up-sampling decoders: bilinear x2 is per channel and a conv over a
  concat is the sum of convs over its parts, so the two wide parts go through
  the matrix-core conv as two input pointers and the 2-channel flow part through
  a small conv whose result rides in as the addend of the wide one.
* `ResidualBlockIncr` of the reference applies ONE activation module (one
  reservoir) to two different tensors and adds the residual with `+=` on
  lists (:252-263); here each use has its own reservoir and the residual is a
  tensor sum, as the dense twin (:285) defines.
* `ConvGRUIncr.forward` of the reference ignores the reset gate (:58-66).  That
  is exact when the recurrent state held at refresh time is zero (the drivers
  pass no state); it is restated as is.
* Constructor arguments replace the literals of the reference class
  (`num_bins`, `base_num_channels`, decoder kind), defaults = the reference's.
"""
import contextlib

import torch
import torch.nn as nn
import torch.nn.functional as F

from . import _lib, ops
from .masked_types import DenseT, Masked, TileMask
from .mask_incr_functional import _unpack
from .mask_incr_modules import (_IncrBuffers, nnAddIncr, nnBatchNorm2dIncr, nnConvIncr,
                                nnConvTranspose2dIncr, nnReservedActivation, nnReservedMultiplication,
                                nnSigmoidIncr, nnTanhIncr, nnUpsample2xIncr, activation_kind, activation_op)


def skip_concat(x1, x2):
    """Reference :9-14 (dense tensors; zero-pads x1 to the size of x2)."""
    diffY = x2.size()[2] - x1.size()[2]
    diffX = x2.size()[3] - x1.size()[3]
    padding = nn.ZeroPad2d((diffX // 2, diffX - diffX // 2, diffY // 2, diffY - diffY // 2))
    x1 = padding(x1)
    return torch.cat([x1, x2], dim=1)


def _mask_of(x_incr):
    return x_incr[1] if len(x_incr) > 1 else None


class nnCatIncr(nn.Module, _IncrBuffers):
    """Channel concat of deltas with the union of their masks (torch.cat on the clean delta
    buffers; used where a kernel takes one input pointer only)."""

    def forward(self, parts):
        if ops._planner is not None:
            # torch.cat / torch.maximum below run on the compute stream and would read pixel masks that the
            # planning stream is still writing
            raise NotImplementedError("nnCatIncr under asynchronous mask planning; use async_masks=False")
        deltas = [ops.as_nhwc(p[0]) for p in parts]
        n, _, h, w = deltas[0].shape
        pix = [ops.pixel_mask_of(_mask_of(p), d) for p, d in zip(parts, deltas)]
        out = ops.as_nhwc(torch.cat(deltas, dim=1))
        if any(m is None for m in pix):
            return [out, None]
        ts = self._tile_set("union", n, h, w, out.device)
        acc = pix[0]
        for m in pix[1:-1]:
            acc = torch.maximum(acc, m)
        ops.build_mask_tiles(acc, pix[-1] if len(pix) > 1 else None, n, h, w, _lib.FOOT_CONV, 1, 1, 0, ts)
        return [out, ts]


class ConvGRUIncr(nn.Module, _IncrBuffers):
    """Incremental ConvGRU (reference :18-96)."""

    def __init__(self, input_size, hidden_size, kernel_size, activation=None, fuse=True, stacked=True):
        super().__init__()
        self.stacked = stacked          # with fuse: both gate convs as one conv + the gate-math kernel
        padding = kernel_size // 2
        self.input_size = input_size
        self.hidden_size = hidden_size
        self.reset_gate = nnConvIncr(input_size + hidden_size, hidden_size, kernel_size, padding=padding)
        self.update_gate = nnConvIncr(input_size + hidden_size, hidden_size, kernel_size, padding=padding)
        self.out_gate = nnConvIncr(input_size + hidden_size, hidden_size, kernel_size, padding=padding)
        assert activation is None, "ConvGRU activation cannot be set (just for compatibility)"
        nn.init.orthogonal_(self.reset_gate.weight)
        nn.init.orthogonal_(self.update_gate.weight)
        nn.init.orthogonal_(self.out_gate.weight)
        nn.init.constant_(self.reset_gate.bias, 0.0)
        nn.init.constant_(self.update_gate.bias, 0.0)
        nn.init.constant_(self.out_gate.bias, 0.0)
        self.sigmoid1 = nnSigmoidIncr()
        self.sigmoid2 = nnSigmoidIncr()
        self.tanh = nnTanhIncr()
        self.mult = nnReservedMultiplication()
        self.add_state = nnAddIncr()
        self.fuse = fuse
        if fuse:                       # structural masks are passed through the fused epilogues
            self.sigmoid1.refine_mask = self.tanh.refine_mask = False

    def _gate(self, conv, act, x_incr, h_incr):
        if self.fuse:
            return conv.forward_fused(x_incr, act, h_incr)
        return act(conv(x_incr, h_incr))

    # -- one conv for both gates + one gate-math kernel (state reset each step) -------------------
    def _stacked_filter(self):
        """ConvFilter of the update-gate and out-gate filters side by side: columns [0, hid) | [hid, 2*hid)."""
        wu, wo = self.update_gate.weight, self.out_gate.weight
        tag = (wu.data_ptr(), wu._version, wo.data_ptr(), wo._version, str(wu.device))
        cached = self.__dict__.get("_stacked_filt_cache")
        if cached is None or cached[0] != tag:
            both = torch.cat((wu.detach(), wo.detach()), 0)                    # [2*hid, cin, k, k]
            cached = (tag, ops.ConvFilter(both.permute(1, 2, 3, 0).contiguous().float()))
            self.__dict__["_stacked_filt_cache"] = cached
        return cached[1]

    def _forward_stacked(self, input_incr):
        """update and candidate deltas from ONE conv (the two gate convs read the same input), then sigmoid /
        tanh increments and the incremental product in one kernel (mie_convgru_gates_incr).  The operands of the
        product are recomputed from the pre-activation reservoirs, so self.mult's own reservoirs are not
        maintained on this path (as with the fused ConvLSTM cell): switch paths only at a refresh."""
        conv = self.update_gate
        k, s, p = conv._geometry()
        x, pix, _ = _unpack(input_incr)
        n, _, h, w = x.shape
        ts = conv._conv_tile_set("out_act", x, pix, None, None, k, s, p)
        gates = self._delta_buf("gru_gates", (n, 2 * self.hidden_size, h, w), x.device, x.dtype)
        ops.conv_masked(x, pix, None, None, self._stacked_filter(), k, s, p, ts, gates)
        new_state = self._delta_buf("gru_state", (n, self.hidden_size, h, w), x.device, x.dtype)
        ops.convgru_gates_incr(gates, self.sigmoid1.in_res.reservoir, self.tanh.in_res.reservoir, new_state, ts)
        return [new_state, ts]

    def forward(self, input_incr, prev_state):
        """new_state = prev_state + mult(out - prev_state, update)  (reference :47-69)."""
        if (self.fuse and self.stacked and prev_state is None and not self.update_gate.lossy
                and not self.out_gate.lossy and self.sigmoid1.in_res.reservoir is not None):
            new_state = self._forward_stacked(input_incr)
            self.__dict__["_mult_stale"] = True       # self.mult's reservoirs have missed this step
            return new_state, new_state
        if self.__dict__.get("_mult_stale", False):
            raise RuntimeError("ConvGRUIncr: steps since the last refresh ran the one-conv form (no previous "
                               "state), which does not maintain the reservoirs of the module-by-module form; "
                               "refresh before switching to it")
        update = self._gate(self.update_gate, self.sigmoid1, input_incr, prev_state)
        out_inputs = self._gate(self.out_gate, self.tanh, input_incr, prev_state)
        if prev_state is None:
            new_state = self.mult(out_inputs, update)
        else:
            diff = [ops.as_nhwc(out_inputs[0] - prev_state[0]), None]
            new_state = self.add_state(prev_state, self.mult(diff, update))
        return new_state, new_state

    def forward_refresh_reservoirs(self, x, prev_state):
        self._reset_incr()
        self.__dict__["_mult_stale"] = False
        zero_state = prev_state is None
        h_in = None if zero_state else ops.as_nhwc(prev_state)
        update = self.update_gate.forward_refresh_fused(x, self.sigmoid1, h_in)
        if zero_state:
            # prev_state * reset is zero whatever the reset gate says: its conv is skipped
            out_inputs = self.out_gate.forward_refresh_fused(x, self.tanh, None)
        else:
            reset = self.reset_gate.forward_refresh_fused(x, self.sigmoid2, h_in)
            gated = ops.mul_dense(h_in, reset, self._dense_buf("reset_state", tuple(h_in.shape), h_in.device, h_in.dtype))
            out_inputs = self.out_gate.forward_refresh_fused(x, self.tanh, gated)
        # new_state = prev_state + (out - prev_state) * update and the cached operands of self.mult, one kernel
        n, _, h, w = update.shape
        shape = (n, self.hidden_size, h, w)
        for res in (self.mult.x1_res, self.mult.x2_res):
            r = res.reservoir
            if r is None or tuple(r.shape) != shape or r.device != update.device:
                res.reservoir = ops.new_nhwc(*shape, update.device)
        self.mult._reset_incr()
        new_state = self._dense_buf("state_refresh", shape, update.device, update.dtype)
        ops.convgru_gates_refresh(update, out_inputs, h_in, self.mult.x1_res.reservoir, self.mult.x2_res.reservoir,
                                  new_state)
        self.add_state._reset_incr()
        return new_state, new_state


class ConvLayerIncr(nn.Module):
    """conv -> [BN] -> activation (reference :99-156)."""

    def __init__(self, in_channels, out_channels, kernel_size, stride=1, activation="relu", norm=None,
                 BN_momentum=0.1, w_scale=None, padding=None, fuse=True):
        super().__init__()
        bias = False if norm == "BN" else True
        if padding is None:
            padding = kernel_size // 2
        self.conv2d = nnConvIncr(in_channels, out_channels, kernel_size, stride, padding, bias=bias)
        if w_scale is not None:
            nn.init.uniform_(self.conv2d.weight, -w_scale, w_scale)
            nn.init.zeros_(self.conv2d.bias)
        self.activation = None
        if activation is not None:
            self.activation = nnReservedActivation(activation_op(activation), refine_mask=not fuse)
        self.norm = norm
        if norm == "BN":
            self.norm_layer = nnBatchNorm2dIncr(out_channels, momentum=BN_momentum)
        elif norm == "IN":
            raise NotImplementedError
        self.fuse = fuse

    def forward(self, x):
        if self.fuse and self.activation is not None and self.norm not in ["BN", "IN"]:
            return self.conv2d.forward_fused(x, self.activation)
        out = self.conv2d(x)
        if self.norm in ["BN", "IN"]:
            out = self.norm_layer(out)
        if self.activation is not None:
            out = self.activation(out)
        return out

    def forward_refresh_reservoirs(self, x):
        if self.fuse and self.activation is not None and self.norm not in ["BN", "IN"]:
            return self.conv2d.forward_refresh_fused(x, self.activation)
        out = self.conv2d.forward_refresh_reservoirs(x)
        if self.norm in ["BN", "IN"]:
            out = self.norm_layer.forward_refresh_reservoirs(out)
        if self.activation is not None:
            out = self.activation.forward_refresh_reservoirs(out)
        return out


class RecurrentConvLayerIncr(nn.Module):
    """Reference :160-195."""

    def __init__(self, in_channels, out_channels, kernel_size=3, stride=1, activation_ff="relu",
                 activation_rec=None, norm=None, BN_momentum=0.1, fuse=True):
        super().__init__()
        self.conv = ConvLayerIncr(in_channels, out_channels, kernel_size, stride, activation_ff, norm,
                                  BN_momentum=BN_momentum, fuse=fuse)
        self.recurrent_block = ConvGRUIncr(input_size=out_channels, hidden_size=out_channels,
                                           kernel_size=3, activation=activation_rec, fuse=fuse)

    def forward(self, x, prev_state):
        x = self.conv(x)
        x, state = self.recurrent_block(x, prev_state)
        return x, state

    def forward_refresh_reservoirs(self, x, prev_state):
        x = self.conv.forward_refresh_reservoirs(x)
        x, state = self.recurrent_block.forward_refresh_reservoirs(x, prev_state)
        return x, state


class ResidualBlockIncr(nn.Module):
    """conv - act - conv, + residual, act; returns (out2, out1) (reference :198-289)."""

    def __init__(self, in_channels, out_channels, stride=1, activation="relu", downsample=None,
                 norm=None, BN_momentum=0.1, fuse=True):
        super().__init__()
        bias = False if norm == "BN" else True
        self.conv1 = nnConvIncr(in_channels, out_channels, kernel_size=3, stride=stride, padding=1, bias=bias)
        self.activation = self.activation2 = None
        if activation is not None:
            self.activation = nnReservedActivation(activation_op(activation), refine_mask=not fuse)
            self.activation2 = nnReservedActivation(activation_op(activation), refine_mask=not fuse)
        self.norm = norm
        if norm == "BN":
            self.bn1 = nnBatchNorm2dIncr(out_channels, momentum=BN_momentum)
            self.bn2 = nnBatchNorm2dIncr(out_channels, momentum=BN_momentum)
        elif norm == "IN":
            raise NotImplementedError
        self.conv2 = nnConvIncr(out_channels, out_channels, kernel_size=3, stride=1, padding=1, bias=bias)
        self.downsample = downsample
        self.add = nnAddIncr()
        self.fuse = fuse

    def _fusable(self):
        return self.fuse and self.activation is not None and self.norm not in ["BN", "IN"] and not self.downsample

    def forward(self, x):
        residual = x
        if self._fusable():
            out1 = self.conv1.forward_fused(x, self.activation)
            return self.conv2.forward_fused(out1, self.activation2, addend_incr=residual), out1
        out1 = self.conv1(x)
        if self.norm in ["BN", "IN"]:
            out1 = self.bn1(out1)
        if self.activation is not None:
            out1 = self.activation(out1)
        out2 = self.conv2(out1)
        if self.norm in ["BN", "IN"]:
            out2 = self.bn2(out2)
        if self.downsample:
            residual = self.downsample(x)
        out2 = self.add(out2, residual, a_covers_b=not self.downsample)
        if self.activation2 is not None:
            out2 = self.activation2(out2)
        return out2, out1

    def forward_refresh_reservoirs(self, x):
        residual = x
        if self._fusable():
            out1 = self.conv1.forward_refresh_fused(x, self.activation)
            return self.conv2.forward_refresh_fused(out1, self.activation2, addend=residual), out1
        out1 = self.conv1.forward_refresh_reservoirs(x)
        if self.norm in ["BN", "IN"]:
            out1 = self.bn1.forward_refresh_reservoirs(out1)
        if self.activation is not None:
            out1 = self.activation.forward_refresh_reservoirs(out1)
        out2 = self.conv2.forward_refresh_reservoirs(out1)
        if self.norm in ["BN", "IN"]:
            out2 = self.bn2.forward_refresh_reservoirs(out2)
        if self.downsample:
            residual = self.downsample.forward_refresh_reservoirs(x)
        out2 = self.add.forward_refresh_reservoirs(out2, residual)
        if self.activation2 is not None:
            out2 = self.activation2.forward_refresh_reservoirs(out2)
        return out2, out1


class UpsampleConvLayerIncr(nn.Module):
    """bilinear x2 -> conv -> activation over the parts of a concat (reference :294-343).

    forward / forward_refresh_reservoirs take the list of parts in concat order
    [previous flow (2 ch, optional), x, skip]; in_channels is the channel count of the concat.
    """

    def __init__(self, in_channels, out_channels, kernel_size, stride=1, activation="relu",
                 padding=None, norm=None, fuse=True):
        super().__init__()
        bias = False if norm == "BN" else True
        if padding is None:
            padding = kernel_size // 2
        self.conv2d = nnConvIncr(in_channels, out_channels, kernel_size, stride, padding, bias=bias)
        self.activation = None
        if activation is not None:
            self.activation = nnReservedActivation(activation_op(activation), refine_mask=not fuse)
        self.norm = norm
        if norm == "BN":
            self.norm_layer = nnBatchNorm2dIncr(out_channels)
        elif norm == "IN":
            raise NotImplementedError
        self.up = nn.ModuleList([nnUpsample2xIncr() for _ in range(3)])
        self.cat = nnCatIncr()
        # buffers of the conv over the narrow leading part of the concat (it shares conv2d's filter)
        self.__dict__["_lead"] = _IncrBuffers()
        self.fuse = fuse

    def _split_ok(self, parts):
        wide = parts[-2:]
        return (self.fuse and self.activation is not None and self.norm not in ["BN", "IN"]
                and len(parts) in (2, 3) and all(p[0].shape[2:] == parts[0][0].shape[2:] for p in parts)
                and _mask_of(wide[0]) is not None and _mask_of(wide[1]) is not None)

    def forward(self, parts):
        k, s, p = self.conv2d._geometry()
        # the narrow leading part (the flow estimate) is up-sampled inside its conv when the shape allows it
        lead_fused = (len(parts) == 3 and self._split_ok(parts) and _mask_of(parts[0]) is not None
                      and ops.upconv_few_takes(parts[0][0].shape[1], self.conv2d.out_channels, k, s, p))
        ups = [None] * len(parts)
        if self._split_ok(parts) and parts[-2][0].shape == parts[-1][0].shape and parts[-2][0].dtype == parts[-1][0].dtype:
            ups[-2], ups[-1] = self._up_pair(len(parts) - 2, parts[-2], parts[-1])      # the two wide parts in one launch
        for i, p_ in enumerate(parts):
            if ups[i] is None and not (lead_fused and i == 0):
                ups[i] = self.up[i](p_)
        if not self._split_ok(parts):
            out = self.conv2d(self.cat(ups))
            if self.norm in ["BN", "IN"]:
                out = self.norm_layer(out)
            return out if self.activation is None else self.activation(out)
        filt = self.conv2d.conv2d_weights
        lead_c = 0
        addend = None
        if len(ups) == 3:
            lead_c = parts[0][0].shape[1]
            # the flow estimate of the previous scale shares the mask of x (it is a 1x1 conv + tanh of
            # it), so the wide conv's output mask covers this partial result
            if lead_fused:
                addend = self._lead_upconv(parts[0], filt.rows(0, lead_c))
            else:
                addend = self._lead_conv(ups[0], filt.rows(0, lead_c))
        return self.conv2d.forward_fused(ups[-2], self.activation, ups[-1], addend_incr=addend,
                                         filt=filt.rows(lead_c, filt.shape[0]))

    def _up_pair(self, i, x_incr, y_incr):
        """self.up[i](x), self.up[i + 1](y) as one launch (ops.upsample2x_pair_incr)."""
        a, pa, _, _, ts_a = self.up[i].plan(x_incr, None)
        b, pb, _, _, ts_b = self.up[i + 1].plan(y_incr, None)
        n, c, h, w = a.shape
        out_a = self.up[i]._delta_buf("out", (n, c, 2 * h, 2 * w), a.device, a.dtype)
        out_b = self.up[i + 1]._delta_buf("out", (n, c, 2 * h, 2 * w), b.device, b.dtype)
        ops.upsample2x_pair_incr(a, pa, ts_a, out_a, b, pb, ts_b, out_b)
        return [out_a, ts_a], [out_b, ts_b]

    def _lead_upconv(self, x_incr, filt):
        """conv over up2x(x) of the narrow leading part in one kernel (ops.upconv_masked, few-channel form)."""
        k, s, p = self.conv2d._geometry()
        a, pa, _, _, ts_up = self.up[0].plan(x_incr, None)
        n, _, h, w = a.shape
        ts = self._lead._tile_set("lead", n, 2 * h, 2 * w, a.device)
        ops.build_mask_tiles(ts_up, None, n, 2 * h, 2 * w, _lib.FOOT_CONV, k, s, p, ts)
        out = self._lead._delta_buf("lead", (n, self.conv2d.out_channels, 2 * h, 2 * w), a.device, a.dtype)
        ops.upconv_masked(a, pa, None, None, filt, k, p, ts, out)
        return [out, ts]

    def _lead_conv(self, x_incr, filt):
        k, s, p = self.conv2d._geometry()
        x, pix, _ = _unpack(x_incr)
        n, _, h, w = x.shape
        ho, wo = ops.conv_out_size(h, w, k, s, p)
        ts = self._lead._tile_set("lead", n, ho, wo, x.device)
        out = self._lead._delta_buf("lead", (n, self.conv2d.out_channels, ho, wo), x.device, x.dtype)
        ops.build_mask_tiles(pix, None, n, h, w, _lib.FOOT_CONV, k, s, p, ts)
        ops.conv_masked(x, pix, None, None, filt, k, s, p, ts, out)
        return [out, ts]

    def forward_refresh_reservoirs(self, parts):
        for m in list(self.up) + [self.cat, self._lead]:
            m._reset_incr()
        ups = [self.up[i].forward_refresh_reservoirs(p) for i, p in enumerate(parts)]
        fused = self.fuse and self.activation is not None and self.norm not in ["BN", "IN"]
        if fused and len(ups) in (2, 3) and not self.conv2d.use_kf:
            # as in forward: the two wide parts side by side through the two-pointer conv (matrix-core shapes
            # stay on the matrix cores instead of a VALU conv over the odd channel count of the concat), the
            # narrow leading part (the 2-channel flow) as a conv of its own whose result rides in as the addend
            filt = self.conv2d.conv2d_weights
            lead_c, addend = 0, None
            if len(ups) == 3:
                lead_c = ups[0].shape[1]
                k, s, p = self.conv2d._geometry()
                lead = ops.as_nhwc(ups[0])
                n, _, h, w = lead.shape
                ho, wo = ops.conv_out_size(h, w, k, s, p)
                ts = self.conv2d._dense_tile_set(n, ho, wo, lead.device)
                addend = self._lead._dense_buf("lead_refresh", (n, self.conv2d.out_channels, ho, wo), lead.device, lead.dtype)
                ops.conv_refresh(lead, None, filt.rows(0, lead_c), None, k, s, p, ts, addend)
            return self.conv2d._refresh_forward(ups[-2], ups[-1], self.activation, path=self.conv2d.path, addend=addend,
                                                filt=filt.rows(lead_c, filt.shape[0]),
                                                bias=None if self.conv2d.bias is None else self.conv2d.bias.detach())
        x = torch.cat(ups, 1)
        if fused:
            return self.conv2d.forward_refresh_fused(x, self.activation)
        out = self.conv2d.forward_refresh_reservoirs(x)
        if self.norm in ["BN", "IN"]:
            out = self.norm_layer.forward_refresh_reservoirs(out)
        if self.activation is not None:
            out = self.activation.forward_refresh_reservoirs(out)
        return out


class TransposedConvLayerIncr(nn.Module):
    """Transposed conv (stride 2, output_padding 1) -> activation over the concat of the parts:
    the decoder kind the benchmark configuration of this network names.  As in the up-sampling
    decoder the concat [previous flow (2 ch, optional), x, skip] is never formed: the two wide parts
    are the two input pointers of the matrix-core transposed conv, the narrow leading part goes
    through the gather kernel and rides in as the addend."""

    def __init__(self, in_channels, out_channels, kernel_size, activation="relu", padding=None, norm=None,
                 fuse=True):
        super().__init__()
        if padding is None:
            padding = kernel_size // 2
        self.transposed_conv2d = nnConvTranspose2dIncr(in_channels, out_channels, kernel_size, stride=2,
                                                       padding=padding, output_padding=1, bias=True)
        self.activation = None
        if activation is not None:
            self.activation = nnReservedActivation(activation_op(activation), refine_mask=not fuse)
        self.cat = nnCatIncr()
        self.fuse = fuse

    def _split_ok(self, shapes, dtype, masked=True):
        """Whether the parts (channel counts in `shapes`) run as lead + two-pointer transposed conv."""
        tc = self.transposed_conv2d
        k, s, p, op = tc._geometry()
        lead_c = shapes[0] if len(shapes) == 3 else 0
        filt = tc._filter()
        return (self.fuse and self.activation is not None and len(shapes) in (2, 3) and masked
                and ops.tconv2x_takes(shapes[-2], shapes[-1], tc.out_channels, k, s, p, op,
                                      filt.rows(lead_c, filt.shape[0]), dtype))

    def forward(self, parts):
        tc = self.transposed_conv2d
        chans = [p_[0].shape[1] for p_ in parts]
        same = all(p_[0].shape[2:] == parts[0][0].shape[2:] for p_ in parts)
        masked = all(_mask_of(p_) is not None for p_ in parts)
        if same and self._split_ok(chans, ops.delta_torch_dtype(parts[0][0]), masked):
            filt = tc._filter()
            lead_c, addend = 0, None
            if len(parts) == 3:
                # the flow estimate of the previous scale shares the mask of x (a 1x1 conv + tanh of it), so the
                # wide conv's output mask covers this partial result
                lead_c = chans[0]
                addend = tc.forward(parts[0], filt=filt.rows(0, lead_c), out_name="lead")
            kind, slope = activation_kind(self.activation.op)
            return tc.forward(parts[-2], self.activation.in_res.reservoir, kind, slope, x2_incr=parts[-1],
                              addend_incr=addend, filt=filt.rows(lead_c, filt.shape[0]))
        x = self.cat(parts)
        if self.fuse and self.activation is not None:
            kind, slope = activation_kind(self.activation.op)
            return tc(x, self.activation.in_res.reservoir, kind, slope)
        out = tc(x)
        return out if self.activation is None else self.activation(out)

    def forward_refresh_reservoirs(self, parts):
        self.cat._reset_incr()
        tc = self.transposed_conv2d
        parts = list(parts)
        chans = [p_.shape[1] for p_ in parts]
        if all(p_.shape[2:] == parts[0].shape[2:] for p_ in parts) and self._split_ok(chans, ops.delta_torch_dtype(parts[0])):
            filt = tc._filter()
            lead_c, addend = 0, None
            if len(parts) == 3:
                lead_c = chans[0]
                addend = tc.forward_refresh_reservoirs(parts[0], filt=filt.rows(0, lead_c), bias=None,
                                                       out_name="lead_refresh")
            kind, slope = activation_kind(self.activation.op)
            n, _, h, w = parts[-1].shape
            shape = (n, tc.out_channels, 2 * h, 2 * w)
            r = self.activation.in_res.reservoir
            if r is None or tuple(r.shape) != shape or r.device != parts[-1].device:
                self.activation.in_res.reservoir = ops.new_nhwc(*shape, parts[-1].device)
            self.activation._reset_incr()
            return tc.forward_refresh_reservoirs(parts[-2], parts[-1], addend, filt=filt.rows(lead_c, filt.shape[0]),
                                                 bias=None if tc.bias is None else tc.bias.detach(),
                                                 reservoir=self.activation.in_res.reservoir, act=kind, slope=slope)
        out = tc.forward_refresh_reservoirs(torch.cat(parts, 1))
        if self.activation is not None:
            out = self.activation.forward_refresh_reservoirs(out)
        return out


class MultiResUNetRecurrentIncr(nn.Module, _IncrBuffers):
    """EVFlowNet-incr (reference :346-495).  Defaults are the reference's literals
    (2 input bins, base 32, 4 encoders 64/128/256/512, 2 residual blocks, up-sampling
    decoders, tanh flow heads); `decoder="transposed"` swaps in transposed-conv decoders."""

    def __init__(self, num_bins=2, base_num_channels=32, num_encoders=4, num_residual_blocks=2,
                 decoder="upsample", fuse=True, mask_threshold=0.0, derive_input_mask=True,
                 async_masks=False, plan_first=False):
        super().__init__()
        # async_masks: build the tile sets on a second stream; plan_first: walk the network twice per step,
        # mask builds first (the masks of this network depend on the input mask only)
        self.async_masks, self.plan_first = async_masks, plan_first
        self.final_activation = 'tanh'
        self.w_scale_pred = None
        self.num_encoders = num_encoders
        self.num_residual_blocks = num_residual_blocks
        self.ff_act, self.rec_act = ['relu', None]
        self.skip_ftn = skip_concat
        self.kernel_size = 3
        self.num_bins = num_bins
        self.norm = None
        self.base_num_channels = base_num_channels
        self.channel_multiplier = 2
        self.num_output_channels = 2
        self.decoder_kind = decoder
        self.fuse = fuse
        self.mask_threshold = float(mask_threshold)
        self.derive_input_mask = derive_input_mask
        self.encoder_input_sizes = [int(self.base_num_channels * pow(self.channel_multiplier, i))
                                    for i in range(self.num_encoders)]
        self.encoder_output_sizes = [int(self.base_num_channels * pow(self.channel_multiplier, i + 1))
                                     for i in range(self.num_encoders)]
        self.max_num_channels = self.encoder_output_sizes[-1]
        self.encoders = self.build_recurrent_encoders()
        self.resblocks = self.build_resblocks()
        self.decoders = self.build_multires_prediction_decoders()
        self.preds = self.build_multires_prediction_layer()
        self.num_states = self.num_encoders
        self.states = [None] * self.num_states

    def build_recurrent_encoders(self):
        encoders = nn.ModuleList()
        for i, (input_size, output_size) in enumerate(zip(self.encoder_input_sizes, self.encoder_output_sizes)):
            if i == 0:
                input_size = self.num_bins
            encoders.append(RecurrentConvLayerIncr(input_size, output_size, kernel_size=self.kernel_size,
                                                   stride=2, activation_ff=self.ff_act,
                                                   activation_rec=self.rec_act, norm=self.norm, fuse=self.fuse))
        return encoders

    def build_resblocks(self):
        resblocks = nn.ModuleList()
        for _ in range(self.num_residual_blocks):
            resblocks.append(ResidualBlockIncr(self.max_num_channels, self.max_num_channels,
                                               activation=self.ff_act, norm=self.norm, fuse=self.fuse))
        return resblocks

    def build_multires_prediction_layer(self):
        preds = nn.ModuleList()
        for output_size in reversed(self.encoder_input_sizes):
            preds.append(ConvLayerIncr(output_size, self.num_output_channels, 1,
                                       activation=self.final_activation, norm=self.norm, fuse=self.fuse))
        return preds

    def build_multires_prediction_decoders(self):
        decoders = nn.ModuleList()
        sizes = zip(reversed(self.encoder_output_sizes), reversed(self.encoder_input_sizes))
        for i, (input_size, output_size) in enumerate(sizes):
            prediction_channels = 0 if i == 0 else self.num_output_channels
            cin = 2 * input_size + prediction_channels
            if self.decoder_kind == "transposed":
                decoders.append(TransposedConvLayerIncr(cin, output_size, kernel_size=self.kernel_size,
                                                        activation=self.ff_act, fuse=self.fuse))
            else:
                decoders.append(UpsampleConvLayerIncr(cin, output_size, kernel_size=self.kernel_size,
                                                      activation=self.ff_act, norm=self.norm, fuse=self.fuse))
        return decoders

    def forward(self, x_incr):
        ops.require_no_lookahead(self)
        delta = ops.as_nhwc(x_incr[0])
        mask = _mask_of(x_incr)
        if not self.async_masks and not self.plan_first:
            return self._forward(delta, mask)
        # (plan_first without async_masks: the planning pass runs on the compute stream, ahead of the compute pass)
        with (ops.mask_planner(delta.device) if self.async_masks else contextlib.nullcontext()):
            if mask is None and self.derive_input_mask:
                n, _, h, w = delta.shape
                mask = ops.mask_from_delta(delta, self.mask_threshold, self._pix_buf("input", n, h, w, delta.device))
            if self.plan_first:
                with ops.network_pass("plan"):
                    self._forward(delta, mask)
                with ops.network_pass("compute"):
                    return self._forward(delta, mask)
            return self._forward(delta, mask)

    def _forward(self, delta, mask):
        if mask is None and self.derive_input_mask:
            n, _, h, w = delta.shape
            mask = ops.mask_from_delta(delta, self.mask_threshold, self._pix_buf("input", n, h, w, delta.device))
        x_incr = [delta, mask]
        states_incr = [None] * self.num_states
        blocks = []
        for i, encoder in enumerate(self.encoders):
            x_incr, state = encoder(x_incr, states_incr[i])
            blocks.append(x_incr)
            states_incr[i] = state
        for resblock in self.resblocks:
            x_incr, _ = resblock(x_incr)
        predictions = []
        for i, (decoder, pred) in enumerate(zip(self.decoders, self.preds)):
            parts = [x_incr, blocks[self.num_encoders - i - 1]]
            if i > 0:
                parts = [predictions[-1]] + parts
            x_incr = decoder(parts)
            predictions.append(pred(x_incr))
        return predictions

    def _lookahead_parts(self, delta):
        n, _, h, w = delta.shape

        def make_mask(d):
            if not self.derive_input_mask:
                return None
            return ops.mask_from_delta(d, self.mask_threshold, self._pix_buf("input", n, h, w, d.device))

        def mask_buffer(d):
            return self._pix_buf("input", n, h, w, d.device) if self.derive_input_mask else None
        return self.__dict__.setdefault("_pipe", {}), make_mask, mask_buffer, self._forward

    def forward_pipelined(self, x_incr, next_x_incr, parity: int):
        """forward(x_incr) with the tile sets of the NEXT step -- whose delta, next_x_incr[0], must already hold its
        values -- planned on a second stream while this step computes (ops.pipelined_step).  parity alternates
        0 / 1 from call to call; the next call must be for the delta announced here; None: no look-ahead."""
        delta = ops.as_nhwc(x_incr[0])
        nxt = None if next_x_incr is None else ops.as_nhwc(next_x_incr[0])
        state, make_mask, mask_buffer, walk = self._lookahead_parts(delta)
        return ops.pipelined_step(state, parity, delta, nxt, make_mask, mask_buffer, walk)

    def plan_ahead(self, x_incr, parity: int) -> None:
        """The planning half of forward_pipelined, on the current stream: input mask and every tile set of the step
        that will take x_incr with this parity (ops.plan_step_ahead has the ordering the caller owes)."""
        delta = ops.as_nhwc(x_incr[0])
        state, make_mask, _, walk = self._lookahead_parts(delta)
        ops.plan_step_ahead(state, parity, delta, make_mask, walk)

    def forward_planned(self, x_incr, parity: int):
        """The compute half: forward(x_incr) over the tile sets plan_ahead built for this parity."""
        delta = ops.as_nhwc(x_incr[0])
        state, make_mask, mask_buffer, walk = self._lookahead_parts(delta)
        return ops.run_planned_step(state, parity, delta, make_mask, mask_buffer, walk)

    def forward_refresh_reservoirs(self, x):
        ops.drop_lookahead(self)
        self._reset_incr()
        blocks = []
        for i, encoder in enumerate(self.encoders):
            x, state = encoder.forward_refresh_reservoirs(x, self.states[i])
            blocks.append(x)
            self.states[i] = state
        for resblock in self.resblocks:
            x, _ = resblock.forward_refresh_reservoirs(x)
        predictions = []
        for i, (decoder, pred) in enumerate(zip(self.decoders, self.preds)):
            parts = [x, blocks[self.num_encoders - i - 1]]
            if i > 0:
                parts = [predictions[-1]] + parts
            x = decoder.forward_refresh_reservoirs(parts)
            predictions.append(pred.forward_refresh_reservoirs(x))
        return predictions
