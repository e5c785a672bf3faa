"""CPU oracle of the incremental ops: a restatement of the reference algorithm in
torch-CPU fp32 (dense-on-delta linear ops + reservoir non-linearities).

TEST INFRASTRUCTURE ONLY: imported by tests/, __graft_entry__.smoke() and the
cpu_baseline leg of bench.py as the checker / timed baseline; never by the
product package.

The reference's own Python cannot be imported (it needs a CUDA-only compiled
extension, a GPU and an empty git submodule), and it holds no golden vectors;
each function below cites the reference lines it follows and is pinned in
tests/test_oracle_pinning.py by the identities the reference's own tests
assert (tests/test_pointops.py:17-22,31-35; tests/test_network.py:24-31),
brute-force loops on tiny inputs and closed forms.
"""
import torch
import torch.nn.functional as F


# ---- reservoir -------------------------------------------------------------------------
class Reserve:
    """incr_modules/mask_incr_functional.py:26-48 (IncrementReserve)."""

    def __init__(self, x_init=None):
        self.reservoir = None if x_init is None else x_init.clone().detach()

    def accumulate(self, incr):
        self.reservoir.add_(incr)          # :41-42

    def update_reservoir(self, x):
        self.reservoir = x.clone().detach()  # :46-48


# ---- linear ops on deltas -----------------------------------------------------------------
def conv_incr(delta, weight, stride=1, padding=0):
    """nnConvIncr.forward: F.conv2d(delta, W, bias=None, padding, stride)
    (incr_modules/mask_incr_modules.py:175-178)."""
    return F.conv2d(delta, weight, bias=None, stride=stride, padding=padding)


def conv_refresh(x, weight, bias, stride=1, padding=0):
    """nnConvIncr.forward_refresh_reservoirs -> nn.Conv2d.forward (:182-196)."""
    return F.conv2d(x, weight, bias=bias, stride=stride, padding=padding)


def tconv_incr(delta, weight, stride, padding, output_padding):
    """transposed_conv2d_from_module (incr_modules/mask_incr_functional.py:64-66)."""
    return F.conv_transpose2d(delta, weight, bias=None, stride=stride, padding=padding,
                              output_padding=output_padding)


def interp_incr(delta):
    """interpolate_from_module (mask_incr_functional.py:76-78)."""
    return F.interpolate(delta, scale_factor=2, mode='bilinear', align_corners=False)


def bn_incr(delta, running_var, weight, eps):
    """bn2d_from_module (mask_incr_functional.py:69-73): batch norm with zero mean, no bias."""
    return F.batch_norm(delta, running_mean=torch.zeros_like(running_var), running_var=running_var,
                        weight=weight, training=False, eps=eps)


def linear_incr(delta, weight):
    """nnLinearIncr.forward (mask_incr_modules.py:112)."""
    return F.linear(delta, weight, bias=None)


def avgpool_incr(delta, output_size):
    """nnAdaptiveAvgPool2dIncr.forward (mask_incr_modules.py:228-233): the pooling is linear, so it
    applies to the delta as it is."""
    return F.adaptive_avg_pool2d(delta, output_size)


# ---- point-wise ops ----------------------------------------------------------------------------
def act_incr(op, res: Reserve, delta):
    """nnReservedActivation.forward: op(R + d) - op(R), then R += d
    (mask_incr_modules.py:101-103,248-251; native twin pointop_cuda.cu:44-51)."""
    out = op(res.reservoir + delta) - op(res.reservoir)
    res.accumulate(delta)
    return out


def mul_incr(d1, r1: Reserve, d2, r2: Reserve):
    """nnReservedMultiplication.forward: (d2 + R2) * d1 + R1 * d2, then R1 += d1, R2 += d2
    (mask_incr_functional.py:54; mask_incr_modules.py:71-75)."""
    out = (d2 + r2.reservoir) * d1 + r1.reservoir * d2
    r1.accumulate(d1)
    r2.accumulate(d2)
    return out


def kfenced(res: Reserve, k, delta):
    """KFencedMaskModule.forward (mask_incr_modules.py:36-42)."""
    t1 = res.reservoir + delta
    f = k * torch.floor(0.5 + t1 / k)
    res.update_reservoir(t1 - f)
    return f


def maxpool_incr(res: Reserve, delta, kernel_size, stride, padding):
    """nnMaxPool2dIncr.forward (mask_incr_modules.py:217-220)."""
    fn = lambda t: F.max_pool2d(t, kernel_size=kernel_size, stride=stride, padding=padding)
    out = fn(res.reservoir + delta) - fn(res.reservoir)
    res.accumulate(delta)
    return out


def leaky_relu(t, slope=0.01):
    return F.leaky_relu(t, slope)


# ---- ConvLSTM ------------------------------------------------------------------------------------
class ConvLSTMOracle:
    """ConvLSTMIncr (incr_modules/e2depth_incr.py:54-166) with the reservoirs the
    reference keeps: pre-activations of the four gates and of tanh2, and both
    operands of m1, m2, m3 (post-activation values, accumulated).  `m1 + m2` is
    taken as the tensor sum the dense twin defines (:161), not the list
    concatenation of :113."""

    def __init__(self, weight, bias, hidden):
        self.w, self.b, self.hid = weight, bias, hidden
        self.pad = weight.shape[2] // 2
        names = ("sig1", "sig2", "sig3", "tanh1", "tanh2", "m1a", "m1b", "m2a", "m2b", "m3a", "m3b")
        self.r = {k: Reserve() for k in names}

    def refresh(self, x, prev_state=None):
        """forward_refresh_reservoirs (:126-166)."""
        n, _, h, w = x.shape
        if prev_state is None:
            prev_state = (torch.zeros(n, self.hid, h, w), torch.zeros(n, self.hid, h, w))
        prev_h, prev_c = prev_state
        gates = F.conv2d(torch.cat((x, prev_h), 1), self.w, self.b, padding=self.pad)
        i, f, o, g = gates.chunk(4, 1)
        r = self.r
        r["sig1"].update_reservoir(i); r["sig2"].update_reservoir(f)
        r["sig3"].update_reservoir(o); r["tanh1"].update_reservoir(g)
        i, f, o, g = torch.sigmoid(i), torch.sigmoid(f), torch.sigmoid(o), torch.tanh(g)
        r["m1a"].update_reservoir(i); r["m1b"].update_reservoir(g)
        r["m2a"].update_reservoir(f); r["m2b"].update_reservoir(prev_c)
        cell = i * g + f * prev_c
        r["tanh2"].update_reservoir(cell)
        ct = torch.tanh(cell)
        r["m3a"].update_reservoir(o); r["m3b"].update_reservoir(ct)
        return o * ct, cell

    def incr(self, dx, prev_state_incr=None):
        """forward (:79-120)."""
        n, _, h, w = dx.shape
        if prev_state_incr is None:
            prev_state_incr = (torch.zeros(n, self.hid, h, w), torch.zeros(n, self.hid, h, w))
        dh_prev, dc_prev = prev_state_incr
        gates = conv_incr(torch.cat((dx, dh_prev), 1), self.w, 1, self.pad)
        di, df, do, dg = gates.chunk(4, 1)
        r = self.r
        di = act_incr(torch.sigmoid, r["sig1"], di)
        df = act_incr(torch.sigmoid, r["sig2"], df)
        do = act_incr(torch.sigmoid, r["sig3"], do)
        dg = act_incr(torch.tanh, r["tanh1"], dg)
        dcell = mul_incr(di, r["m1a"], dg, r["m1b"]) + mul_incr(df, r["m2a"], dc_prev, r["m2b"])
        dct = act_incr(torch.tanh, r["tanh2"], dcell)
        dhid = mul_incr(do, r["m3a"], dct, r["m3b"])
        return dhid, dcell


# ---- brute force (tiny inputs only) -----------------------------------------------------------------
def conv2d_bruteforce(x, weight, stride, padding):
    """Seven nested loops, float64 accumulation; x (N,C,H,W), weight (O,C,K,K)."""
    n, c, h, w = x.shape
    o, _, k, _ = weight.shape
    ho, wo = (h + 2 * padding - k) // stride + 1, (w + 2 * padding - k) // stride + 1
    out = torch.zeros(n, o, ho, wo, dtype=torch.float64)
    xd, wd = x.double(), weight.double()
    for b in range(n):
        for oc in range(o):
            for oy in range(ho):
                for ox in range(wo):
                    acc = 0.0
                    for ic in range(c):
                        for ky in range(k):
                            iy = oy * stride - padding + ky
                            if iy < 0 or iy >= h:
                                continue
                            for kx in range(k):
                                ix = ox * stride - padding + kx
                                if 0 <= ix < w:
                                    acc += float(xd[b, ic, iy, ix]) * float(wd[oc, ic, ky, kx])
                    out[b, oc, oy, ox] = acc
    return out


def tconv2d_bruteforce(x, weight, stride, padding, output_padding):
    """Scatter form of the transposed conv; weight (C_in, C_out, K, K)."""
    n, c, h, w = x.shape
    _, o, k, _ = weight.shape
    ho = (h - 1) * stride - 2 * padding + k + output_padding
    wo = (w - 1) * stride - 2 * padding + k + output_padding
    out = torch.zeros(n, o, ho, wo, dtype=torch.float64)
    xd, wd = x.double(), weight.double()
    for b in range(n):
        for ic in range(c):
            for iy in range(h):
                for ix in range(w):
                    v = float(xd[b, ic, iy, ix])
                    if v == 0.0:
                        continue
                    for ky in range(k):
                        oy = iy * stride - padding + ky
                        if oy < 0 or oy >= ho:
                            continue
                        for kx in range(k):
                            ox = ix * stride - padding + kx
                            if 0 <= ox < wo:
                                out[b, :, oy, ox] += v * wd[ic, :, ky, kx]
    return out


def up2x_bruteforce(x):
    """Bilinear x2, align_corners=False, from the definition src = (o + .5)/2 - .5 clamped at 0."""
    n, c, h, w = x.shape
    out = torch.zeros(n, c, 2 * h, 2 * w, dtype=torch.float64)
    xd = x.double()

    def coef(o, size):
        src = max(0.0, (o + 0.5) / 2.0 - 0.5)
        i0 = int(src)
        i1 = min(i0 + 1, size - 1)
        lam = src - i0
        return i0, i1, 1.0 - lam, lam

    for oy in range(2 * h):
        r0, r1, a0, a1 = coef(oy, h)
        for ox in range(2 * w):
            c0, c1, b0, b1 = coef(ox, w)
            out[:, :, oy, ox] = a0 * (b0 * xd[:, :, r0, c0] + b1 * xd[:, :, r0, c1]) + \
                a1 * (b0 * xd[:, :, r1, c0] + b1 * xd[:, :, r1, c1])
    return out
