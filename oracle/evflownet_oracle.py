"""CPU oracle of EVFlowNet-incr: the reference network executed the way the reference executes
it (dense convs on the delta, reservoir non-linearities) in torch-CPU fp32.

TEST INFRASTRUCTURE ONLY (checker in tests/); never imported by the product package.

Follows incr_modules/evflownet_incr.py: ConvGRUIncr :47-96 (the incremental forward leaves the
reset gate out, :58-66), ConvLayerIncr :143-167, RecurrentConvLayerIncr :186-195,
ResidualBlockIncr :245-289, UpsampleConvLayerIncr :324-343, MultiResUNetRecurrentIncr :447-495.
Where the incremental forward of the reference trips over Python lists (`out2 += residual`,
one activation reservoir used for two tensors, :252-263) the dense twin (:267-289) is the
specification: tensor sum, one reservoir per use.  Parameters come as a dict with the
state_dict keys of the reference's module tree.
"""
import torch
import torch.nn.functional as F

from . import incr_oracle as io


class _ConvAct:
    def __init__(self, p, prefix, stride, padding, op):
        self.w, self.b = p[prefix + ".weight"], p.get(prefix + ".bias")
        self.stride, self.padding, self.op = stride, padding, op
        self.res = io.Reserve()

    def refresh(self, x):
        out = io.conv_refresh(x, self.w, self.b, self.stride, self.padding)
        self.res.update_reservoir(out)
        return self.op(out)

    def incr(self, dx):
        return io.act_incr(self.op, self.res, io.conv_incr(dx, self.w, self.stride, self.padding))


class _TConvAct(_ConvAct):
    def refresh(self, x):
        out = F.conv_transpose2d(x, self.w, self.b, stride=2, padding=self.padding, output_padding=1)
        self.res.update_reservoir(out)
        return self.op(out)

    def incr(self, dx):
        return io.act_incr(self.op, self.res, io.tconv_incr(dx, self.w, 2, self.padding, 1))


class _ConvGRU:
    def __init__(self, p, prefix, hid):
        self.hid = hid
        self.update = _ConvAct(p, prefix + ".update_gate", 1, 1, torch.sigmoid)
        self.reset = _ConvAct(p, prefix + ".reset_gate", 1, 1, torch.sigmoid)
        self.out = _ConvAct(p, prefix + ".out_gate", 1, 1, torch.tanh)
        self.m1, self.m2 = io.Reserve(), io.Reserve()

    def refresh(self, x, prev):
        if prev is None:
            prev = torch.zeros(x.shape[0], self.hid, *x.shape[2:])
        stacked = torch.cat([x, prev], 1)
        update = self.update.refresh(stacked)
        reset = self.reset.refresh(stacked)
        out = self.out.refresh(torch.cat([x, prev * reset], 1))
        self.m1.update_reservoir(out - prev)
        self.m2.update_reservoir(update)
        return prev + (out - prev) * update

    def incr(self, dx, dprev=None):
        if dprev is None:
            dprev = torch.zeros(dx.shape[0], self.hid, *dx.shape[2:])
        stacked = torch.cat([dx, dprev], 1)
        update = self.update.incr(stacked)
        out = self.out.incr(stacked)
        return dprev + io.mul_incr(out - dprev, self.m1, update, self.m2)


class _ResBlock:
    def __init__(self, p, prefix):
        self.c1 = _ConvAct(p, prefix + ".conv1", 1, 1, torch.relu)
        self.w2, self.b2 = p[prefix + ".conv2.weight"], p[prefix + ".conv2.bias"]
        self.res2 = io.Reserve()

    def refresh(self, x):
        out2 = io.conv_refresh(self.c1.refresh(x), self.w2, self.b2, 1, 1) + x
        self.res2.update_reservoir(out2)
        return torch.relu(out2)

    def incr(self, dx):
        out2 = io.conv_incr(self.c1.incr(dx), self.w2, 1, 1) + dx
        return io.act_incr(torch.relu, self.res2, out2)


class EVFlowNetOracle:
    def __init__(self, params, num_encoders=4, num_residual_blocks=2, base=32, decoder="upsample"):
        p = {k: v.detach().clone().float().cpu() for k, v in params.items()}
        self.n_enc = num_encoders
        self.decoder = decoder
        self.enc = [_ConvAct(p, "encoders.%d.conv.conv2d" % i, 2, 1, torch.relu) for i in range(num_encoders)]
        self.gru = [_ConvGRU(p, "encoders.%d.recurrent_block" % i, base * 2 ** (i + 1)) for i in range(num_encoders)]
        self.resblocks = [_ResBlock(p, "resblocks.%d" % i) for i in range(num_residual_blocks)]
        if decoder == "transposed":
            self.dec = [_TConvAct(p, "decoders.%d.transposed_conv2d" % i, 2, 1, torch.relu) for i in range(num_encoders)]
        else:
            self.dec = [_ConvAct(p, "decoders.%d.conv2d" % i, 1, 1, torch.relu) for i in range(num_encoders)]
        self.preds = [_ConvAct(p, "preds.%d.conv2d" % i, 1, 0, torch.tanh) for i in range(num_encoders)]
        self.states = [None] * num_encoders

    def _decode(self, x, blocks, refresh):
        preds = []
        for i, (dec, pred) in enumerate(zip(self.dec, self.preds)):
            x = torch.cat([x, blocks[self.n_enc - i - 1]], 1)
            if i > 0:
                x = torch.cat([preds[-1], x], 1)
            if self.decoder != "transposed":
                x = io.interp_incr(x)
            x = dec.refresh(x) if refresh else dec.incr(x)
            preds.append(pred.refresh(x) if refresh else pred.incr(x))
        return preds

    def refresh(self, x):
        """forward_refresh_reservoirs (:475-495); the recurrent states persist across refreshes."""
        blocks = []
        for i in range(self.n_enc):
            x = self.gru[i].refresh(self.enc[i].refresh(x), self.states[i])
            self.states[i] = x
            blocks.append(x)
        for rb in self.resblocks:
            x = rb.refresh(x)
        return self._decode(x, blocks, True)

    def incr(self, dx):
        """forward (:447-472): no recurrent-state deltas."""
        blocks = []
        for i in range(self.n_enc):
            dx = self.gru[i].incr(self.enc[i].incr(dx), None)
            blocks.append(dx)
        for rb in self.resblocks:
            dx = rb.incr(dx)
        return self._decode(dx, blocks, False)
