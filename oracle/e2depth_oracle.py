"""CPU oracle of E2Depth-incr: the reference network executed the way the reference
executes it today -- every conv as a dense F.conv2d on the delta, every
activation as op(R + d) - op(R) with a dense reservoir add, ConvLSTM through
the module chain -- in torch-CPU fp32.

TEST INFRASTRUCTURE ONLY (checker in tests/ and smoke(), timed baseline in
bench.py's cpu_baseline leg); never imported by the product package.

Follows incr_modules/e2depth_incr.py: ConvLayerIncr :32-51, ConvLSTMIncr
:79-166, RecurrentConvLayerIncr :176-186, ResidualBlockIncr :206-240,
UpsampleConvLayerIncr :303-322, UNetRecurrentIncr :402-468, with the layer
shapes of todo.txt:34-57 (head 5x5; encoders 5x5 stride 2 + ConvLSTM 3x3;
residual blocks 3x3; decoders bilinear x2 + 5x5 with skip sum; 1x1 prediction
+ sigmoid).  Parameters come as a dict with the state_dict keys of the
reference's module tree (`unetrecurrent.head.conv2d.weight`, ...).  The skip
"sum" is the tensor sum of the dense twin (:333,:459), not the list
concatenation the incremental forward performs by accident.
"""
import torch

from . import incr_oracle as io


class _ConvAct:
    def __init__(self, params, prefix, stride, padding, op):
        self.w = params[prefix + ".weight"]
        self.b = params.get(prefix + ".bias")
        self.stride, self.padding, self.op = stride, padding, op
        self.res = io.Reserve()

    def refresh(self, x):
        out = io.conv_refresh(x, self.w, self.b, self.stride, self.padding)
        if self.op is None:
            return out
        self.res.update_reservoir(out)
        return self.op(out)

    def incr(self, dx):
        out = io.conv_incr(dx, self.w, self.stride, self.padding)
        if self.op is None:
            return out
        return io.act_incr(self.op, self.res, out)


class _ResBlock:
    def __init__(self, params, prefix):
        self.c1 = _ConvAct(params, prefix + ".conv1", 1, 1, torch.relu)
        self.c2 = _ConvAct(params, prefix + ".conv2", 1, 1, None)
        self.res2 = io.Reserve()

    def refresh(self, x):
        out = self.c2.refresh(self.c1.refresh(x)) + x
        self.res2.update_reservoir(out)
        return torch.relu(out)

    def incr(self, dx):
        out = self.c2.incr(self.c1.incr(dx)) + dx
        return io.act_incr(torch.relu, self.res2, out)


class E2DepthOracle:
    def __init__(self, params, num_encoders=3, num_residual_blocks=2, base=32):
        p = {k: v.detach().clone().float().cpu() for k, v in params.items()}
        u = "unetrecurrent."
        self.head = _ConvAct(p, u + "head.conv2d", 1, 2, torch.relu)
        self.enc, self.lstm = [], []
        for i in range(num_encoders):
            self.enc.append(_ConvAct(p, u + "encoders.%d.conv.conv2d" % i, 2, 2, torch.relu))
            hid = base * 2 ** (i + 1)
            self.lstm.append(io.ConvLSTMOracle(p[u + "encoders.%d.recurrent_block.Gates.weight" % i],
                                               p[u + "encoders.%d.recurrent_block.Gates.bias" % i], hid))
        self.resblocks = [_ResBlock(p, u + "resblocks.%d" % i) for i in range(num_residual_blocks)]
        self.dec = [_ConvAct(p, u + "decoders.%d.conv2d" % i, 1, 2, torch.relu)
                    for i in range(num_encoders)]
        self.pred = _ConvAct(p, u + "pred.conv2d", 1, 0, torch.sigmoid)
        self.n_enc = num_encoders

    def refresh(self, x):
        """UNetRecurrentIncr.forward_refresh_reservoirs with prev_states=None (:442-468)."""
        x = self.head.refresh(x)
        head = x
        blocks = []
        for conv, lstm in zip(self.enc, self.lstm):
            x = conv.refresh(x)
            x, _ = lstm.refresh(x, None)
            blocks.append(x)
        for rb in self.resblocks:
            x = rb.refresh(x)
        for i, dec in enumerate(self.dec):
            x = dec.refresh(io.interp_incr(x + blocks[self.n_enc - i - 1]))
        return self.pred.refresh(x + head)

    def incr(self, dx):
        """UNetRecurrentIncr.forward with prev_states_incr=None (:402-439)."""
        dx = self.head.incr(dx)
        head = dx
        blocks = []
        for conv, lstm in zip(self.enc, self.lstm):
            dx = conv.incr(dx)
            dx, _ = lstm.incr(dx, None)
            blocks.append(dx)
        for rb in self.resblocks:
            dx = rb.incr(dx)
        for i, dec in enumerate(self.dec):
            dx = dec.incr(io.interp_incr(dx + blocks[self.n_enc - i - 1]))
        return self.pred.incr(dx + head)
