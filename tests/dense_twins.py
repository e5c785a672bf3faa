"""Independent dense twins of the two networks, written from their published topology with plain
torch.nn modules only (nn.Conv2d, nn.ConvTranspose2d, F.interpolate) -- no code shared with oracle/ or
with the package.  Their module trees carry the reference's state_dict keys
(`unetrecurrent.head.conv2d.weight`, `encoders.0.recurrent_block.update_gate.weight`, ...), so loading an
incremental network's state_dict with strict=True already checks every parameter name and shape.

E2Depth: todo.txt:34-57 of the reference lists every conv of one 1x5x264x352 forward (input shape, filter
shape, stride, padding); E2DEPTH_CONV_TRACE restates that list as data and `conv_trace` records the same
from a twin's forward.  Topology: incr_modules/e2depth_incr.py:126-166 (ConvLSTM, gate order in, remember,
out, cell), :325-377, :442-468 (UNet with skip sums, sigmoid head).  EVFlowNet: incr_modules/
evflownet_incr.py:71-96 (ConvGRU), :346-495 (concat skips, flow heads fed forward).
"""
import torch
import torch.nn as nn
import torch.nn.functional as F

# (input shape, filter shape [Cout, Cin, K, K], stride, padding) of every conv, in execution order
E2DEPTH_CONV_TRACE = [
    ((1, 5, 264, 352), (32, 5, 5, 5), 1, 2),
    ((1, 32, 264, 352), (64, 32, 5, 5), 2, 2), ((1, 128, 132, 176), (256, 128, 3, 3), 1, 1),
    ((1, 64, 132, 176), (128, 64, 5, 5), 2, 2), ((1, 256, 66, 88), (512, 256, 3, 3), 1, 1),
    ((1, 128, 66, 88), (256, 128, 5, 5), 2, 2), ((1, 512, 33, 44), (1024, 512, 3, 3), 1, 1),
    ((1, 256, 33, 44), (256, 256, 3, 3), 1, 1), ((1, 256, 33, 44), (256, 256, 3, 3), 1, 1),
    ((1, 256, 33, 44), (256, 256, 3, 3), 1, 1), ((1, 256, 33, 44), (256, 256, 3, 3), 1, 1),
    ((1, 256, 66, 88), (128, 256, 5, 5), 1, 2),
    ((1, 128, 132, 176), (64, 128, 5, 5), 1, 2),
    ((1, 64, 264, 352), (32, 64, 5, 5), 1, 2),
    ((1, 32, 264, 352), (1, 32, 1, 1), 1, 0),
]


def _holder(**mods):
    m = nn.Module()
    for k, v in mods.items():
        setattr(m, k, v)
    return m


class E2DepthTwin(nn.Module):
    def __init__(self, bins=5, base=32, num_encoders=3, num_residual_blocks=2):
        super().__init__()
        u = nn.Module()
        u.head = _holder(conv2d=nn.Conv2d(bins, base, 5, 1, 2))
        u.encoders = nn.ModuleList()
        for i in range(num_encoders):
            cin, cout = base * 2 ** i, base * 2 ** (i + 1)
            u.encoders.append(_holder(conv=_holder(conv2d=nn.Conv2d(cin, cout, 5, 2, 2)),
                                      recurrent_block=_holder(Gates=nn.Conv2d(2 * cout, 4 * cout, 3, 1, 1))))
        top = base * 2 ** num_encoders
        u.resblocks = nn.ModuleList(_holder(conv1=nn.Conv2d(top, top, 3, 1, 1), conv2=nn.Conv2d(top, top, 3, 1, 1))
                                    for _ in range(num_residual_blocks))
        u.decoders = nn.ModuleList(_holder(conv2d=nn.Conv2d(top // 2 ** i, top // 2 ** (i + 1), 5, 1, 2))
                                   for i in range(num_encoders))
        u.pred = _holder(conv2d=nn.Conv2d(base, 1, 1))
        self.unetrecurrent = u

    def forward(self, x):
        """One dense frame from a zero recurrent state."""
        u = self.unetrecurrent
        x = torch.relu(u.head.conv2d(x))
        head, skips = x, []
        for enc in u.encoders:
            x = torch.relu(enc.conv.conv2d(x))
            h0 = torch.zeros_like(x)
            gates = enc.recurrent_block.Gates(torch.cat([x, h0], 1))
            i, f, o, g = gates.chunk(4, 1)
            cell = torch.sigmoid(f) * torch.zeros_like(x) + torch.sigmoid(i) * torch.tanh(g)
            x = torch.sigmoid(o) * torch.tanh(cell)
            skips.append(x)
        for rb in u.resblocks:
            x = torch.relu(rb.conv2(torch.relu(rb.conv1(x))) + x)
        for k, dec in enumerate(u.decoders):
            x = x + skips[len(skips) - 1 - k]
            x = torch.relu(dec.conv2d(F.interpolate(x, scale_factor=2, mode="bilinear", align_corners=False)))
        return torch.sigmoid(u.pred.conv2d(x + head))


class EVFlowNetTwin(nn.Module):
    def __init__(self, bins=4, base=32, num_encoders=4, num_residual_blocks=2, decoder="upsample"):
        super().__init__()
        self.decoder = decoder
        ins = [base * 2 ** i for i in range(num_encoders)]
        outs = [base * 2 ** (i + 1) for i in range(num_encoders)]
        self.encoders = nn.ModuleList()
        for i, (cin, cout) in enumerate(zip(ins, outs)):
            gru = _holder(**{g: nn.Conv2d(2 * cout, cout, 3, 1, 1) for g in ("reset_gate", "update_gate", "out_gate")})
            self.encoders.append(_holder(conv=_holder(conv2d=nn.Conv2d(bins if i == 0 else cin, cout, 3, 2, 1)),
                                         recurrent_block=gru))
        top = outs[-1]
        self.resblocks = nn.ModuleList(_holder(conv1=nn.Conv2d(top, top, 3, 1, 1), conv2=nn.Conv2d(top, top, 3, 1, 1))
                                       for _ in range(num_residual_blocks))
        self.decoders, self.preds = nn.ModuleList(), nn.ModuleList()
        for k, (cin, cout) in enumerate(zip(reversed(outs), reversed(ins))):
            c = 2 * cin + (0 if k == 0 else 2)
            if decoder == "transposed":
                self.decoders.append(_holder(transposed_conv2d=nn.ConvTranspose2d(c, cout, 3, 2, 1, output_padding=1)))
            else:
                self.decoders.append(_holder(conv2d=nn.Conv2d(c, cout, 3, 1, 1)))
            self.preds.append(_holder(conv2d=nn.Conv2d(cout, 2, 1)))

    def forward(self, x):
        """Flow at every scale (coarse to fine) from a zero recurrent state."""
        skips = []
        for enc in self.encoders:
            x = torch.relu(enc.conv.conv2d(x))
            g, h0 = enc.recurrent_block, torch.zeros_like(x)
            xh = torch.cat([x, h0], 1)
            update, reset = torch.sigmoid(g.update_gate(xh)), torch.sigmoid(g.reset_gate(xh))
            cand = torch.tanh(g.out_gate(torch.cat([x, h0 * reset], 1)))
            x = h0 * (1 - update) + cand * update
            skips.append(x)
        for rb in self.resblocks:
            x = torch.relu(rb.conv2(torch.relu(rb.conv1(x))) + x)
        flows = []
        for k, (dec, pred) in enumerate(zip(self.decoders, self.preds)):
            parts = [x, skips[len(skips) - 1 - k]]
            if k > 0:
                parts = [flows[-1]] + parts
            x = torch.cat(parts, 1)
            if self.decoder == "transposed":
                x = torch.relu(dec.transposed_conv2d(x))
            else:
                x = torch.relu(dec.conv2d(F.interpolate(x, scale_factor=2, mode="bilinear", align_corners=False)))
            flows.append(torch.tanh(pred.conv2d(x)))
        return flows


def conv_trace(net, x):
    """[(input shape, filter shape, stride, padding)] of every nn.Conv2d call of net(x), in execution order."""
    trace, hooks = [], []

    def hook(m, inp, out):
        trace.append((tuple(inp[0].shape), tuple(m.weight.shape), m.stride[0], m.padding[0]))
    for m in net.modules():
        if isinstance(m, nn.Conv2d):
            hooks.append(m.register_forward_hook(hook))
    with torch.no_grad():
        net(x)
    for h in hooks:
        h.remove()
    return trace
