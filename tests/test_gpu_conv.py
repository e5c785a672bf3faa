"""GPU parity of the masked convolutions (VALU, MFMA, small-Cout, transposed) against
the CPU oracle, through the C ABI.  fp32 tolerance: rtol 1e-4, atol 1e-5."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

from maskedincrementeval_amd import _lib, ops
from maskedincrementeval_amd.masked_types import TileMask
from maskedincrementeval_amd.synthetic import blob_mask, gaussian_delta, he_normal_conv_weight
from oracle import incr_oracle as io
from oracle import mask_oracle as mo
from tolerances import BF16_RTOL, bf16_atol

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
RTOL, ATOL = 1e-4, 1e-5


def _dev(t):
    return ops.as_nhwc(t.to(DEV).contiguous(memory_format=torch.channels_last))


def _filt(w_oihw):
    return ops.ConvFilter(w_oihw.permute(1, 2, 3, 0).contiguous().to(DEV))


def _close(got, ref, what=""):
    got = got.cpu()
    err = (got - ref).abs().max().item()
    assert torch.allclose(got, ref, rtol=RTOL, atol=ATOL), "%s max|diff| = %.3e" % (what, err)


class _Conv:
    """One masked conv on persistent buffers, as a module would hold them."""

    def __init__(self, n, cin, cout, h, w, k, s, p, seed, path):
        self.k, self.s, self.p, self.path = k, s, p, path
        self.w = he_normal_conv_weight(cout, cin, k, seed)
        self.filt = _filt(self.w)
        self.ho, self.wo = mo.conv_out_size(h, w, k, s, p)
        self.ts = TileMask(n, self.ho, self.wo, DEV)
        self.out = ops.new_nhwc(n, cout, self.ho, self.wo, DEV)
        self.n, self.h, self.w_in = n, h, w

    def run(self, delta, mask, reservoir=None, act=_lib.ACT_NONE, slope=0.0, x2=None, m2=None):
        dm = None if mask is None else mask.to(DEV)
        dm2 = None if m2 is None else m2.to(DEV)
        both = dm if x2 is None else (None if (dm is None or dm2 is None) else dm)
        ops.build_mask_tiles(both, dm2 if both is not None else None, self.n, self.h, self.w_in,
                             _lib.FOOT_CONV, self.k, self.s, self.p, self.ts)
        ops.conv_masked(_dev(delta), dm, None if x2 is None else _dev(x2), dm2, self.filt, self.k,
                        self.s, self.p, self.ts, self.out, reservoir, act, slope, self.path)
        torch.cuda.synchronize()
        return self.out


PATHS = [("valu", _lib.PATH_VALU), ("mfma", _lib.PATH_MFMA)]


def _mfma_takes(k, s, cin, cout):
    """Shapes the matrix-core path takes (fp32): whole staging chunks of input channels (32, or 16
    for 7x7; stride 2 may fall back to half of that) and whole output slabs for the wave splits
    the chunk depth allows (32 / 64 / 128 for 4 / 2 / 1 sub-chunks of 8 channels)."""
    for half in ((False, True) if s == 2 else (False,)):
        cc = (32 if k <= 5 else 16) // (2 if half else 1)
        cmul = {4: 32, 2: 64, 1: 128}[cc // 8]
        if cin % cc == 0 and cout % cmul == 0:
            return True
    return False


@pytest.mark.parametrize("pname,path", PATHS)
@pytest.mark.parametrize("k,s,p", [(1, 1, 0), (3, 1, 1), (3, 2, 1), (5, 1, 2), (5, 2, 2), (7, 1, 3), (7, 2, 3)])
@pytest.mark.parametrize("cin,cout", [(32, 32), (32, 64), (64, 128)])
@pytest.mark.parametrize("f32mode", ["bf16x3", "native"])
def test_conv_paths_match_oracle(pname, path, k, s, p, cin, cout, f32mode):
    if path == _lib.PATH_MFMA and not _mfma_takes(k, s, cin, cout):
        pytest.skip("shape not taken by the matrix-core path (falls to the VALU path)")
    n, h, w = 2, 37, 45      # ragged: not multiples of the 8x8 tile
    d, m = gaussian_delta(n, cin, h, w, 0.06, 0.5, seed=k * 100 + s * 10 + cin)
    conv = _Conv(n, cin, cout, h, w, k, s, p, seed=3, path=path)
    got = conv.run(d, m)
    _close(got, io.conv_incr(d, conv.w, s, p), "%s k%d s%d" % (pname, k, s))


@pytest.mark.parametrize("cin,cout,k,s,p", [(5, 32, 5, 1, 2), (3, 5, 3, 1, 1), (7, 70, 3, 2, 1), (32, 1, 1, 1, 0),
                                            (32, 2, 3, 1, 1), (4, 3, 5, 2, 2), (20, 33, 1, 2, 0), (64, 2, 1, 1, 0), (12, 4, 1, 1, 0),
                                            (6, 3, 1, 1, 0)])
def test_odd_channel_counts_auto_path(cin, cout, k, s, p):
    # head (Cin=5), prediction (Cout=1), flow heads (Cout=2) and other shapes the MFMA path cannot take
    n, h, w = 1, 41, 29
    d, m = gaussian_delta(n, cin, h, w, 0.1, 0.5, seed=cin + cout)
    conv = _Conv(n, cin, cout, h, w, k, s, p, seed=4, path=_lib.PATH_AUTO)
    _close(conv.run(d, m), io.conv_incr(d, conv.w, s, p))


@pytest.mark.parametrize("pname,path", PATHS)
def test_all_ones_mask_equals_dense_conv(pname, path):
    # reference tests/test_pointops.py:25-35, at a shape both paths take
    n, cin, cout, h, w = 1, 32, 32, 25, 25
    x = torch.randn(n, cin, h, w, generator=torch.Generator().manual_seed(0))
    conv = _Conv(n, cin, cout, h, w, 3, 1, 1, seed=5, path=path)
    ref = io.conv_refresh(x, conv.w, None, 1, 1)
    _close(conv.run(x, torch.ones(n, 1, h, w, dtype=torch.uint8)), ref)
    _close(conv.run(x, None), ref)        # mask None = all active


@pytest.mark.parametrize("pname,path", PATHS)
def test_inactive_pixels_are_never_read_and_output_is_clean(pname, path):
    n, cin, cout, h, w = 1, 32, 32, 64, 72
    conv = _Conv(n, cin, cout, h, w, 3, 1, 1, seed=6, path=path)
    for step, dens in enumerate((0.08, 0.02, 0.15, 0.0)):   # fresh masks: tiles go stale, last one empty
        d, m = gaussian_delta(n, cin, h, w, dens, 0.3, seed=40 + step)
        poisoned = torch.where(m.bool().expand_as(d), d, torch.full_like(d, float("nan")))
        got = conv.run(poisoned, m).cpu()
        ref = io.conv_incr(d, conv.w, 1, 1)
        assert torch.isfinite(got).all()
        _close(got, ref, "step %d" % step)
        # exactly zero outside the footprint of the mask (clean-delta invariant)
        fp = torch.from_numpy(mo.footprint_conv(m[:, 0].numpy(), 3, 1, 1)).bool().unsqueeze(1)
        assert torch.count_nonzero(got * (~fp)) == 0


@pytest.mark.parametrize("pname,path", PATHS)
@pytest.mark.parametrize("f32mode", ["bf16x3", "native"])
def test_two_pointer_input_equals_concat(pname, path, f32mode):
    # ConvLSTM gates: conv over cat(x, h) without forming the concat (e2depth_incr.py:100-101)
    n, c1, c2, cout, h, w = 1, 32, 32, 128, 33, 44
    dx, mx = gaussian_delta(n, c1, h, w, 0.05, 0.3, seed=60)
    dh, mh = gaussian_delta(n, c2, h, w, 0.03, 0.3, seed=61)
    conv = _Conv(n, c1 + c2, cout, h, w, 3, 1, 1, seed=7, path=path)
    ref = io.conv_incr(torch.cat((dx, dh), 1), conv.w, 1, 1)
    _close(conv.run(dx, mx, x2=dh, m2=mh), ref, "x ++ h")
    # hidden half absent: only the first c1 filter channels are used
    ref0 = io.conv_incr(torch.cat((dx, torch.zeros_like(dh)), 1), conv.w, 1, 1)
    _close(conv.run(dx, mx), ref0, "x only")


@pytest.mark.parametrize("pname,path", PATHS)
@pytest.mark.parametrize("act,slope,op", [(_lib.ACT_RELU, 0.0, torch.relu),
                                          (_lib.ACT_LEAKY_RELU, 0.01, io.leaky_relu),
                                          (_lib.ACT_SIGMOID, 0.0, torch.sigmoid),
                                          (_lib.ACT_TANH, 0.0, torch.tanh)])
@pytest.mark.parametrize("f32mode", ["bf16x3", "native"])
def test_fused_conv_activation_epilogue(pname, path, act, slope, op, f32mode):
    n, cin, cout, h, w = 1, 32, 32, 40, 48
    conv = _Conv(n, cin, cout, h, w, 3, 1, 1, seed=8, path=path)
    r0 = torch.randn(n, cout, h, w, generator=torch.Generator().manual_seed(1))
    res_gpu = _dev(r0.clone())
    res_cpu = io.Reserve(r0)
    for step in range(3):
        d, m = gaussian_delta(n, cin, h, w, 0.1, 0.5, seed=70 + step)
        got = conv.run(d, m, reservoir=res_gpu, act=act, slope=slope)
        ref = io.act_incr(op, res_cpu, io.conv_incr(d, conv.w, 1, 1))
        _close(got, ref, "delta step %d" % step)
        _close(res_gpu, res_cpu.reservoir, "reservoir step %d" % step)


def test_config1_cached_output_plus_increment_is_dense_conv():
    # benchmark configuration 1: 1x32x264x352 -> 32, 3x3 s1 p1, He-normal weights, x_prev ~ N(0,1),
    # 5 % smoothed-threshold mask, delta ~ N(0, 0.1)
    n, c, h, w = 1, 32, 264, 352
    g = torch.Generator().manual_seed(0)
    x_prev = torch.randn(n, c, h, w, generator=g)
    d, m = gaussian_delta(n, c, h, w, 0.05, 0.1, seed=1000)
    assert int(m.sum()) == round(0.05 * h * w)
    for path in (_lib.PATH_VALU, _lib.PATH_MFMA):
        conv = _Conv(n, c, 32, h, w, 3, 1, 1, seed=0, path=path)
        cached = io.conv_refresh(x_prev, conv.w, None, 1, 1)
        got = conv.run(d, m).cpu()
        dense = io.conv_refresh(x_prev + d, conv.w, None, 1, 1)
        assert torch.allclose(cached + got, dense, rtol=RTOL, atol=ATOL)
        tiles = conv.ts.active_tiles().cpu().numpy()
        assert np.array_equal(tiles, mo.tile_list(mo.footprint_conv(m[:, 0].numpy(), 3, 1, 1)))
        assert 0 < tiles.size < conv.ts.capacity // 2


@pytest.mark.parametrize("k,s,p,op", [(3, 2, 1, 1), (4, 2, 1, 0), (5, 2, 2, 1), (2, 2, 0, 0)])
def test_tconv_matches_oracle(k, s, p, op):
    n, cin, cout, h, w = 2, 12, 20, 19, 23
    d, m = gaussian_delta(n, cin, h, w, 0.08, 0.5, seed=k)
    wt = torch.randn(cin, cout, k, k, generator=torch.Generator().manual_seed(k)) * 0.2
    ho, wo = (h - 1) * s - 2 * p + k + op, (w - 1) * s - 2 * p + k + op
    ts = TileMask(n, ho, wo, DEV)
    out = ops.new_nhwc(n, cout, ho, wo, DEV)
    filt = wt.permute(0, 2, 3, 1).contiguous().to(DEV)
    ref = io.tconv_incr(d, wt, s, p, op)
    for step in range(2):
        ops.build_mask_tiles(m.to(DEV), None, n, h, w, _lib.FOOT_TCONV, k, s, p, ts)
        ops.tconv_masked(_dev(d), m.to(DEV), filt, k, s, p, ts, out)
        torch.cuda.synchronize()
        _close(out, ref, "tconv k%d" % k)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("cin,cout,h,w", [(2, 32, 16, 16), (2, 64, 13, 21), (8, 20, 7, 9), (1, 4, 33, 5)])
def test_tconv2x_few_channel_form(cin, cout, h, w, dtype):
    """The decoder geometry over very few input channels (the flow lead of an EVFlowNet decoder) takes a kernel
    of its own: against the oracle, over three steps with moving masks (stale tiles are zeroed), ragged planes."""
    n, k, s, p, op = 2, 3, 2, 1, 1
    wt = torch.randn(cin, cout, k, k, generator=torch.Generator().manual_seed(cin + cout)) * 0.3
    if dtype == torch.bfloat16:
        wt = wt.to(dtype).float()
    ho, wo = 2 * h, 2 * w
    ts = TileMask(n, ho, wo, DEV)
    out = ops.new_nhwc(n, cout, ho, wo, DEV, dtype)
    filt = wt.permute(0, 2, 3, 1).contiguous().to(DEV)
    for step in range(3):
        d, m = gaussian_delta(n, cin, h, w, 0.06, 0.5, seed=10 * step + cin)
        if dtype == torch.bfloat16:
            d = d.to(dtype).float()
        ref = io.tconv_incr(d, wt, s, p, op)
        ops.build_mask_tiles(m.to(DEV), None, n, h, w, _lib.FOOT_TCONV, k, s, p, ts)
        ops.tconv_masked(_dev(d).to(dtype), m.to(DEV), filt, k, s, p, ts, out)
        torch.cuda.synchronize()
        if dtype == torch.bfloat16:
            assert torch.allclose(out.float().cpu(), ref, rtol=2.0 ** -7, atol=bf16_atol(ref, 1)), "step %d" % step
        else:
            _close(out, ref, "tconv2x few-channel step %d" % step)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("c1,c2,cout,h,w,k", [
    (64, 0, 32, 13, 17, 3),        # one input, ragged plane
    (64, 64, 64, 16, 16, 3),       # two inputs (the concat-free decoder form), 2 chunks: not split
    (256, 256, 64, 16, 16, 3),     # 4 blocks x 2 slabs, 16 chunks: the contraction is split over workgroups
    (64, 0, 128, 40, 48, 5),       # 5x5 (the depth network's decoder kind): halo on all sides
    (128, 128, 32, 9, 20, 5)])
@pytest.mark.parametrize("f32mode", ["bf16x3", "native"])
def test_tconv2x_matrix_core_form(c1, c2, cout, h, w, k, dtype, f32mode):
    # stride-2 transposed conv as four sub-pixel phases on the matrix cores, against F.conv_transpose2d of the
    # concat; three steps with fresh masks (stale blocks), reservoir + ReLU epilogue and an addend
    if dtype == torch.bfloat16 and (c1 % 64 or c2 % 64):
        pytest.skip("bf16 chunks hold 64 channels")
    n, p = 2, k // 2
    cin = c1 + c2
    wt = torch.randn(cin, cout, k, k, generator=torch.Generator().manual_seed(k + cin)) * (2.0 / (cin * k * k)) ** 0.5
    rnd = (lambda t: t.to(dtype).float())
    wt = rnd(wt)
    filt = ops.ConvFilter(wt.permute(0, 2, 3, 1).contiguous().to(DEV))
    ho, wo = 2 * h, 2 * w
    ts, blocks = TileMask(n, ho, wo, DEV), TileMask(n, h, w, DEV)
    out = ops.new_nhwc(n, cout, ho, wo, DEV, dtype)
    r0 = torch.randn(n, cout, ho, wo, generator=torch.Generator().manual_seed(5))
    res_gpu, res_cpu = _dev(r0.clone()), io.Reserve(r0.clone())
    tc_tol = dict(rtol=RTOL, atol=ATOL) if dtype == torch.float32 else dict(rtol=2 ** -7, atol=2 ** -7)
    for step, dens in enumerate((0.10, 0.03, 0.25)):
        d1, m1 = gaussian_delta(n, c1, h, w, dens, 0.5, seed=900 + step)
        d1 = rnd(d1)
        nan = float("nan")
        x1 = torch.where(m1.bool().expand_as(d1), d1, torch.full_like(d1, nan))      # inactive pixels are never read
        x2 = m2 = d2 = None
        full, mask = d1, m1
        if c2:
            d2, m2 = gaussian_delta(n, c2, h, w, dens / 2, 0.5, seed=950 + step)
            d2 = rnd(d2)
            x2 = torch.where(m2.bool().expand_as(d2), d2, torch.full_like(d2, nan))
            full, mask = torch.cat((d1, d2), 1), m1 | m2
        ops.build_mask_tiles(m1.to(DEV), None if m2 is None else m2.to(DEV), n, h, w, _lib.FOOT_TCONV, k, 2, p, ts)
        ops.build_mask_tiles(ts, None, n, ho, wo, _lib.FOOT_CONV, 2, 2, 0, blocks)
        want_mask = mo.footprint_tconv(mask[:, 0].numpy(), k, 2, p, ho, wo)
        assert np.array_equal(ts.pixmask[:, 0].cpu().numpy(), want_mask)
        add = rnd(torch.randn(n, cout, ho, wo, generator=torch.Generator().manual_seed(70 + step)) * 0.1
                  * torch.from_numpy(want_mask).unsqueeze(1).float())
        ops.tconv2x_masked(_dev(x1.to(dtype)), m1.to(DEV), None if x2 is None else _dev(x2.to(dtype)),
                           None if m2 is None else m2.to(DEV), filt, k, ts, blocks, out, res_gpu, _lib.ACT_RELU, 0.0,
                           _dev(add.to(dtype)))
        torch.cuda.synchronize()
        ref = io.act_incr(torch.relu, res_cpu, io.tconv_incr(full, wt, 2, p, 1) + add)
        got = out.float().cpu()
        assert torch.isfinite(got).all()
        assert torch.allclose(got, ref, **tc_tol), "step %d max|diff| %.3e" % (step, (got - ref).abs().max())
        assert torch.allclose(res_gpu.cpu(), res_cpu.reservoir, rtol=RTOL, atol=ATOL if dtype == torch.float32 else 1e-4)
        outside = ~torch.from_numpy(want_mask).bool().unsqueeze(1)
        assert torch.count_nonzero(got * outside) == 0          # clean delta, stale blocks zeroed
    # dense refresh twin: bias + activation + reservoir fill
    dts, dbl = TileMask(n, ho, wo, DEV), TileMask(n, h, w, DEV)
    ops.build_mask_tiles(None, None, n, ho, wo, _lib.FOOT_CONV, 1, 1, 0, dts)
    ops.build_mask_tiles(None, None, n, h, w, _lib.FOOT_CONV, 1, 1, 0, dbl)
    xa = rnd(torch.randn(n, c1, h, w, generator=torch.Generator().manual_seed(80)))
    xb = rnd(torch.randn(n, c2, h, w, generator=torch.Generator().manual_seed(81))) if c2 else None
    bias = torch.randn(cout, generator=torch.Generator().manual_seed(82)) * 0.1
    dense = ops.new_nhwc(n, cout, ho, wo, DEV, dtype)
    ops.tconv2x_refresh(_dev(xa.to(dtype)), None if xb is None else _dev(xb.to(dtype)), filt, bias.to(DEV), k, dts, dbl,
                        dense, res_gpu, _lib.ACT_RELU, 0.0)
    torch.cuda.synchronize()
    pre = F.conv_transpose2d(xa if xb is None else torch.cat((xa, xb), 1), wt, bias, stride=2, padding=p, output_padding=1)
    rt = dict(rtol=RTOL, atol=ATOL) if dtype == torch.float32 else dict(rtol=2 ** -7, atol=2 ** -7)
    assert torch.allclose(res_gpu.cpu(), pre, rtol=1e-4, atol=1e-5 if dtype == torch.float32 else 1e-4)
    assert torch.allclose(dense.float().cpu(), torch.relu(pre), **rt)


@pytest.mark.parametrize("f32mode", ["bf16x3", "native"])
def test_large_channel_mfma_bottleneck_shapes(f32mode):
    # 256 -> 256 3x3 at 33x44 (residual blocks) and 512 -> 1024 gates: K = 2304 / 4608 contractions
    n, h, w = 1, 33, 44
    for cin, cout in ((256, 256), (512, 1024)):
        d, m = gaussian_delta(n, cin, h, w, 0.2, 0.2, seed=cin)
        conv = _Conv(n, cin, cout, h, w, 3, 1, 1, seed=9, path=_lib.PATH_MFMA)
        _close(conv.run(d, m), io.conv_incr(d, conv.w, 1, 1), "%d->%d" % (cin, cout))


@pytest.mark.parametrize("pname,path", PATHS)
@pytest.mark.parametrize("f32mode", ["bf16x3", "native"])
def test_addend_rides_into_the_epilogue(pname, path, f32mode):
    # residual block tail: relu2(conv2(d) + residual) with the residual delta as the conv's addend
    n, c, h, w = 1, 32, 40, 56
    conv = _Conv(n, c, c, h, w, 3, 1, 1, seed=10, path=path)
    r0 = torch.randn(n, c, h, w, generator=torch.Generator().manual_seed(3))
    res_gpu, res_cpu = _dev(r0.clone()), io.Reserve(r0)
    for step in range(3):
        d, m = gaussian_delta(n, c, h, w, 0.08, 0.5, seed=90 + step)
        resid = d * 0.5                                   # lives on m, which the 3x3 footprint covers
        dm = m.to(DEV)
        ops.build_mask_tiles(dm, None, n, h, w, _lib.FOOT_CONV, 3, 1, 1, conv.ts)
        ops.conv_masked(_dev(d), dm, None, None, conv.filt, 3, 1, 1, conv.ts, conv.out, res_gpu,
                        _lib.ACT_RELU, 0.0, path, _dev(resid))
        torch.cuda.synchronize()
        ref = io.act_incr(torch.relu, res_cpu, io.conv_incr(d, conv.w, 1, 1) + resid)
        _close(conv.out, ref, "step %d" % step)
        _close(res_gpu, res_cpu.reservoir, "reservoir %d" % step)


@pytest.mark.parametrize("f32mode", ["bf16x3", "native"])
def test_refresh_conv_matches_dense_conv_with_bias(f32mode):
    n, cin, cout, h, w = 2, 32, 64, 37, 45
    g = torch.Generator().manual_seed(5)
    x, x2 = torch.randn(n, cin, h, w, generator=g), torch.randn(n, cin, h, w, generator=g)
    wt = he_normal_conv_weight(cout, 2 * cin, 3, 11)
    bias = torch.randn(cout, generator=g)
    ts = TileMask(n, h, w, DEV)
    ops.build_mask_tiles(None, None, n, h, w, _lib.FOOT_CONV, 1, 1, 0, ts)
    out, res = ops.new_nhwc(n, cout, h, w, DEV), ops.new_nhwc(n, cout, h, w, DEV)
    for path in (_lib.PATH_VALU, _lib.PATH_MFMA):
        ops.conv_refresh(_dev(x), _dev(x2), _filt(wt), bias.to(DEV), 3, 1, 1, ts, out, res, _lib.ACT_TANH, 0.0, path)
        torch.cuda.synchronize()
        pre = io.conv_refresh(torch.cat((x, x2), 1), wt, bias, 1, 1)
        _close(res, pre, "reservoir = pre-activation")
        _close(out, torch.tanh(pre), "activated output")


def test_pack_filter_layout_and_row_views():
    cin, k, cout = 24, 3, 40
    f = torch.arange(cin * k * k * cout, dtype=torch.float32).reshape(cin, k, k, cout).to(DEV)
    p = ops.pack_filter(f)
    torch.cuda.synchronize()
    want = f.reshape(cin // 8, 2, 4, k * k, cout).permute(0, 3, 1, 4, 2).contiguous()    # [b,t,h,co,j]
    assert torch.equal(p, want)
    cf = ops.ConvFilter(f)
    sub = cf.rows(8, 24)
    assert sub.mc.data_ptr() == cf.mc[1:].data_ptr() and torch.equal(sub.mc, ops.pack_filter(f[8:24].contiguous()))
    assert cf.rows(8, 24) is sub
    odd = cf.rows(4, 20)                 # not on an 8-row boundary: a packed copy of its own
    assert torch.equal(odd.mc, ops.pack_filter(f[4:20].contiguous()))
    assert ops.ConvFilter(f[:12].contiguous()).mc is None


# 5x5 conv over up2x(a + b) in one kernel (the decoder layers): against interpolate + conv of the oracle,
# for the three workgroup organisations (32 / 64 / 128 output channels per slab), ragged sizes whose
# borders exercise the clamped bilinear taps and the conv's zero padding, fresh masks per step (stale
# tiles), with and without the second input, plain and reservoir + activation epilogue.
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("c,cout,h,w", [(64, 32, 13, 17), (64, 64, 70, 90), (128, 128, 88, 80), (64, 96, 9, 40)])
@pytest.mark.parametrize("f32mode", ["bf16x3", "native"])
def test_upsampled_conv_in_one_kernel(c, cout, h, w, dtype, f32mode):
    bf = dtype == torch.bfloat16
    tol = (lambda ref: dict(rtol=BF16_RTOL, atol=bf16_atol(ref, 2.0))) if bf else (lambda ref: dict(rtol=RTOL, atol=ATOL))
    q = (lambda t: t.to(torch.bfloat16).float()) if bf else (lambda t: t)
    wt = q(he_normal_conv_weight(cout, c, 5, 9))
    filt = _filt(wt)
    assert ops.upconv_takes(c, cout, 5, 1, 2, filt, dtype)
    ts_up, ts = TileMask(1, 2 * h, 2 * w, DEV), TileMask(1, 2 * h, 2 * w, DEV)
    out = ops.new_nhwc(1, cout, 2 * h, 2 * w, DEV, dtype)
    r0 = gaussian_delta(1, cout, 2 * h, 2 * w, 1.0, 1.0, seed=3)[0]
    for step, (da, db, two, with_res) in enumerate([(0.2, 0.1, True, False), (0.03, 0.05, True, False),
                                                    (0.1, 0.0, False, False), (0.3, 0.2, True, True)]):
        a, ma = gaussian_delta(1, c, h, w, da, 0.5, seed=100 + step)
        b, mb = gaussian_delta(1, c, h, w, db, 0.5, seed=200 + step)
        a, b = q(a), q(b)
        up = io.interp_incr(a + b if two else a)
        if bf:
            up = q(up)            # the staged tile is rounded to bf16, like the up-sampled delta would be
        ref = io.conv_incr(up, wt, 1, 2)
        dma, dmb = ma.to(DEV), mb.to(DEV)
        ops.build_mask_tiles(dma, dmb if two else None, 1, h, w, _lib.FOOT_UP2X, 0, 0, 0, ts_up)
        ops.build_mask_tiles(ts_up, None, 1, 2 * h, 2 * w, _lib.FOOT_CONV, 5, 1, 2, ts)
        poison = lambda t, m: torch.where(m.bool().expand_as(t), t, torch.full_like(t, float("nan")))
        res = _dev(r0).clone() if with_res else None
        ops.upconv_masked(_dev(poison(a, ma)).to(dtype), dma, _dev(poison(b, mb)).to(dtype) if two else None,
                          dmb if two else None, filt, 5, 2, ts, out, res,
                          _lib.ACT_RELU if with_res else _lib.ACT_NONE)
        torch.cuda.synchronize()
        got = out.float().cpu()
        assert torch.isfinite(got).all()
        want = torch.relu(r0 + ref) - torch.relu(r0) if with_res else ref
        assert torch.allclose(got, want, **tol(want)), "step %d max|diff| = %.3e" % (step, (got - want).abs().max())
        if with_res:
            assert torch.allclose(res.cpu(), r0 + ref, rtol=RTOL, atol=bf16_atol(ref, 2.0) if bf else ATOL)


# Up-sampling decoder convs on planes of few tiles: the contraction is split over workgroups through a workspace
# (mie_upconv_masked_ws) and a second kernel runs the epilogue.  Against the oracle and against the unsplit launch;
# three steps with fresh masks (stale tiles), reservoir + activation on the last two.
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("c,cout,h,w,two", [(256, 128, 16, 16, True), (128, 64, 12, 20, True), (256, 32, 9, 7, False)])
@pytest.mark.parametrize("f32mode", ["bf16x3", "native"])
def test_small_upsampled_planes_split_the_contraction(c, cout, h, w, two, dtype, f32mode):
    bf = dtype == torch.bfloat16
    if bf and c // 64 < 4:
        pytest.skip("fewer than 4 staged chunks of 64 bf16 channels: not split")
    tol = (lambda ref: dict(rtol=BF16_RTOL, atol=bf16_atol(ref, 2.0))) if bf else (lambda ref: dict(rtol=RTOL, atol=ATOL))
    q = (lambda t: t.to(torch.bfloat16).float()) if bf else (lambda t: t)
    wt = q(he_normal_conv_weight(cout, c, 5, 19))
    filt = _filt(wt)
    ho, wo = 2 * h, 2 * w
    ts_up, ts = TileMask(1, ho, wo, DEV), TileMask(1, ho, wo, DEV)
    assert ts.capacity * (cout // 32) <= 128
    out, out_plain = ops.new_nhwc(1, cout, ho, wo, DEV, dtype), ops.new_nhwc(1, cout, ho, wo, DEV, dtype)
    ws = torch.full((ops.SPLIT_WORKSPACE_BYTES // 4,), float("nan"), device=DEV)
    r0 = gaussian_delta(1, cout, ho, wo, 1.0, 1.0, seed=7)[0]
    res, res_plain, res_ref = _dev(r0).clone(), _dev(r0).clone(), r0.clone()
    for step, (da, db, with_res) in enumerate([(0.3, 0.2, False), (0.05, 0.02, True), (0.5, 0.4, True)]):
        a, ma = gaussian_delta(1, c, h, w, da, 0.5, seed=500 + step)
        b, mb = gaussian_delta(1, c, h, w, db, 0.5, seed=600 + step)
        a, b = q(a), q(b)
        up = io.interp_incr(a + b if two else a)
        if bf:
            up = q(up)
        ref = io.conv_incr(up, wt, 1, 2)
        dma, dmb = ma.to(DEV), mb.to(DEV)
        ops.build_mask_tiles(dma, dmb if two else None, 1, h, w, _lib.FOOT_UP2X, 0, 0, 0, ts_up)
        ops.build_mask_tiles(ts_up, None, 1, ho, wo, _lib.FOOT_CONV, 5, 1, 2, ts)
        poison = lambda t, m: torch.where(m.bool().expand_as(t), t, torch.full_like(t, float("nan")))
        xa, xb = _dev(poison(a, ma)).to(dtype), (_dev(poison(b, mb)).to(dtype) if two else None)
        for o, r, wsp in ((out, res, ws), (out_plain, res_plain, False)):
            ops.upconv_masked(xa, dma, xb, dmb if two else None, filt, 5, 2, ts, o, r if with_res else None,
                              _lib.ACT_RELU if with_res else _lib.ACT_NONE, workspace=wsp)
        torch.cuda.synchronize()
        got, plain = out.float().cpu(), out_plain.float().cpu()
        assert torch.isfinite(got).all()
        want = torch.relu(res_ref + ref) - torch.relu(res_ref) if with_res else ref
        if with_res:
            res_ref = res_ref + ref
        assert torch.allclose(got, want, **tol(want)), "step %d max|diff| = %.3e" % (step, (got - want).abs().max())
        assert torch.allclose(got, plain, **tol(plain)), "step %d split vs unsplit %.3e" % (step, (got - plain).abs().max())
        if with_res:
            assert torch.allclose(res.cpu(), res_ref, rtol=RTOL, atol=bf16_atol(ref, 2.0) if bf else ATOL)
    plane = ho * wo * cout
    assert torch.isfinite(ws[:plane]).any() and torch.isfinite(ws[plane:2 * plane]).any()      # the split form ran


# The same for a single input of very few channels (the flow estimate in front of an EVFlowNet decoder): 3x3 and 5x5.
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("c,cout,k,h,w", [(2, 64, 3, 13, 17), (2, 32, 3, 32, 32), (5, 96, 5, 9, 40), (8, 32, 3, 21, 11)])
def test_upsampled_conv_few_channels(c, cout, k, h, w, dtype):
    bf = dtype == torch.bfloat16
    tol = (lambda ref: dict(rtol=BF16_RTOL, atol=bf16_atol(ref, 2.0))) if bf else (lambda ref: dict(rtol=RTOL, atol=ATOL))
    q = (lambda t: t.to(torch.bfloat16).float()) if bf else (lambda t: t)
    n, p = 2, k // 2
    wt = q(he_normal_conv_weight(cout, c, k, 19))
    filt = _filt(wt)
    assert ops.upconv_few_takes(c, cout, k, 1, p)
    ts_up, ts = TileMask(n, 2 * h, 2 * w, DEV), TileMask(n, 2 * h, 2 * w, DEV)
    out = ops.new_nhwc(n, cout, 2 * h, 2 * w, DEV, dtype)
    for step, dens in enumerate((0.3, 0.05, 1.0)):
        a, ma = gaussian_delta(n, c, h, w, dens, 0.5, seed=700 + step)
        a = q(a)
        ref = io.conv_incr(io.interp_incr(a), wt, 1, p)          # the staged tile stays fp32: no rounding in between
        dma = ma.to(DEV)
        ops.build_mask_tiles(dma, None, n, h, w, _lib.FOOT_UP2X, 0, 0, 0, ts_up)
        ops.build_mask_tiles(ts_up, None, n, 2 * h, 2 * w, _lib.FOOT_CONV, k, 1, p, ts)
        poisoned = torch.where(ma.bool().expand_as(a), a, torch.full_like(a, float("nan")))
        ops.upconv_masked(_dev(poisoned).to(dtype), dma, None, None, filt, k, p, ts, out)
        torch.cuda.synchronize()
        got = out.float().cpu()
        assert torch.isfinite(got).all()
        assert torch.allclose(got, ref, **tol(ref)), "step %d max|diff| = %.3e" % (step, (got - ref).abs().max())


def _random_cases(count, seed):
    rng = np.random.RandomState(seed)
    cases = []
    for i in range(count):
        k = int(rng.choice([1, 3, 5, 7]))
        s = int(rng.choice([1, 2]))
        cin = int(rng.choice([3, 8, 16, 24, 32, 48, 64, 96, 128]))
        cout = int(rng.choice([1, 2, 5, 16, 32, 40, 64, 96, 128, 160]))
        h, w = int(rng.randint(k, 70)), int(rng.randint(k, 90))
        n = int(rng.choice([1, 1, 2, 3]))
        dens = float(rng.choice([0.0, 0.02, 0.1, 0.4, 1.0]))
        pad = int(rng.choice([0, k // 2]))
        cases.append((i, k, s, pad, cin, cout, n, h, w, dens))
    return cases


# A seeded sweep over shapes nobody picked by hand: kernel size, stride, padding (none / same), channel
# counts on and off the matrix-core path, ragged planes down to the kernel size, batch, density from empty
# to dense; two steps per case so that tiles go stale.  Auto path, fp32 and bf16.
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("case", _random_cases(36, seed=2024), ids=lambda c: "k%ds%dp%d_%dto%d_n%d_%dx%d_d%g" % c[1:])
def test_seeded_random_shapes(case, dtype):
    i, k, s, pad, cin, cout, n, h, w, dens = case
    bf = dtype == torch.bfloat16
    tol = (lambda ref: dict(rtol=BF16_RTOL, atol=bf16_atol(ref, 2.0))) if bf else (lambda ref: dict(rtol=RTOL, atol=ATOL))
    q = (lambda t: t.to(torch.bfloat16).float()) if bf else (lambda t: t)
    wt = q(he_normal_conv_weight(cout, cin, k, 50 + i))
    filt = _filt(wt)
    ho, wo = mo.conv_out_size(h, w, k, s, pad)
    ts = TileMask(n, ho, wo, DEV)
    out = ops.new_nhwc(n, cout, ho, wo, DEV, dtype)
    for step, dd in enumerate((dens, dens * 0.5)):
        d, m = gaussian_delta(n, cin, h, w, dd, 0.5, seed=7000 + 10 * i + step)
        d = q(d)
        ref = io.conv_incr(d, wt, s, pad)
        dm = m.to(DEV)
        ops.build_mask_tiles(dm, None, n, h, w, _lib.FOOT_CONV, k, s, pad, ts)
        ops.conv_masked(_dev(d).to(dtype), dm, None, None, filt, k, s, pad, ts, out)
        torch.cuda.synchronize()
        got = out.float().cpu()
        assert torch.allclose(got, ref, **tol(ref)), "step %d max|diff| = %.3e" % (step, (got - ref).abs().max())
        foot = torch.from_numpy(mo.footprint_conv(m[:, 0].numpy(), k, s, pad)).bool().unsqueeze(1)
        assert torch.count_nonzero(got * (~foot)) == 0


# Planes of very few tiles: with a workspace the matrix-core path splits the contraction of every
# (tile, slab) over several workgroups and a second kernel adds the partial sums and runs the epilogue.
# Three steps with fresh masks (stale tiles), the last two with reservoir + activation and an addend;
# checked against the oracle and against the unsplit launch, and the workspace must have been written.
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("k", [3, 5])
@pytest.mark.parametrize("c1,c2,cout,h,w,s", [(512, 0, 512, 16, 16, 1), (256, 0, 512, 32, 32, 2), (128, 0, 96, 13, 11, 1),
                                              (128, 64, 64, 20, 9, 1), (256, 128, 160, 8, 8, 1), (128, 0, 32, 31, 29, 2),
                                              (256, 0, 256, 32, 32, 1)])
@pytest.mark.parametrize("f32mode", ["bf16x3", "native"])
def test_small_planes_split_the_contraction(c1, c2, cout, h, w, s, dtype, k, f32mode):
    bf = dtype == torch.bfloat16
    if bf and (c1 % 64 or c2 % 64 or (c1 + c2) // 64 < 4):
        pytest.skip("fewer than 4 staged chunks of 64 bf16 channels: not split")
    tol = (lambda ref: dict(rtol=BF16_RTOL, atol=bf16_atol(ref, 2.0))) if bf else (lambda ref: dict(rtol=RTOL, atol=ATOL))
    q = (lambda t: t.to(torch.bfloat16).float()) if bf else (lambda t: t)
    n, cin = 1, c1 + c2
    wt = q(he_normal_conv_weight(cout, cin, k, 21))
    filt = _filt(wt)
    ho, wo = mo.conv_out_size(h, w, k, s, k // 2)
    ts = TileMask(n, ho, wo, DEV)
    assert ts.capacity * (cout // 32) <= 128
    out, out_plain = ops.new_nhwc(n, cout, ho, wo, DEV, dtype), ops.new_nhwc(n, cout, ho, wo, DEV, dtype)
    ws = torch.full((ops.SPLIT_WORKSPACE_BYTES // 4,), float("nan"), device=DEV)
    r0 = gaussian_delta(n, cout, ho, wo, 1.0, 1.0, seed=5)[0]
    res, res_plain, res_ref = _dev(r0).clone(), _dev(r0).clone(), r0.clone()
    for step, (dens, with_res) in enumerate([(0.3, False), (0.05, True), (0.6, True)]):
        d, m = gaussian_delta(n, cin, h, w, dens, 0.5, seed=300 + step)
        d = q(d)
        foot = torch.from_numpy(mo.footprint_conv(m[:, 0].numpy(), k, s, k // 2)).bool().unsqueeze(1)
        # an addend is a clean delta on pixels of the output mask
        add = q(gaussian_delta(n, cout, ho, wo, 1.0, 0.3, seed=400 + step)[0]) * foot if with_res else None
        ref = io.conv_incr(d, wt, s, k // 2)
        dm = m.to(DEV)
        ops.build_mask_tiles(dm, None, n, h, w, _lib.FOOT_CONV, k, s, k // 2, ts)
        dx = _dev(d).to(dtype)
        x1, x2 = (dx, None) if c2 == 0 else (ops.as_nhwc(dx[:, :c1].contiguous(memory_format=torch.channels_last)),
                                             ops.as_nhwc(dx[:, c1:].contiguous(memory_format=torch.channels_last)))
        dadd = None if add is None else _dev(add).to(dtype)
        for o, r, wsp in ((out, res, ws), (out_plain, res_plain, False)):
            ops.conv_masked(x1, dm, x2, None if x2 is None else dm, filt, k, s, k // 2, ts, o, r if with_res else None,
                            _lib.ACT_RELU if with_res else _lib.ACT_NONE, 0.0, _lib.PATH_MFMA, dadd, workspace=wsp)
        torch.cuda.synchronize()
        got, plain = out.float().cpu(), out_plain.float().cpu()
        if with_res:
            acc = ref + add
            want = torch.relu(res_ref + acc) - torch.relu(res_ref)
            res_ref = res_ref + acc
        else:
            want = ref
        assert torch.allclose(got, want, **tol(want)), "step %d max|diff| = %.3e" % (step, (got - want).abs().max())
        assert torch.allclose(got, plain, **tol(plain)), "step %d split vs unsplit %.3e" % (step, (got - plain).abs().max())
        if with_res:
            assert torch.allclose(res.cpu(), res_ref, rtol=RTOL, atol=bf16_atol(ref, 2.0) if bf else ATOL)
    # the split form ran: its partial sums replaced the NaN fill of the first planes
    plane = n * ho * wo * cout
    assert torch.isfinite(ws[:plane]).any() and torch.isfinite(ws[plane:2 * plane]).any()


# Layers of at most 8 input channels (the network heads) have a matrix-core kernel of their own on the
# automatic path: against the oracle and against the VALU kernel, every channel count, both kernel sizes and
# strides, ragged plane, two steps (stale tiles), plain and with reservoir + activation.
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("k,s", [(3, 1), (3, 2), (5, 1), (5, 2)])
@pytest.mark.parametrize("cin,cout", [(1, 32), (2, 64), (4, 64), (5, 32), (7, 96), (8, 32)])
def test_few_input_channels_matrix_core_kernel(cin, cout, k, s, dtype):
    bf = dtype == torch.bfloat16
    tol = (lambda ref: dict(rtol=BF16_RTOL, atol=bf16_atol(ref, 2.0))) if bf else (lambda ref: dict(rtol=RTOL, atol=ATOL))
    q = (lambda t: t.to(torch.bfloat16).float()) if bf else (lambda t: t)
    n, h, w, p = 2, 29, 43, k // 2
    wt = q(he_normal_conv_weight(cout, cin, k, 60 + cin))
    filt = _filt(wt)
    ho, wo = mo.conv_out_size(h, w, k, s, p)
    ts = TileMask(n, ho, wo, DEV)
    out, out_valu = ops.new_nhwc(n, cout, ho, wo, DEV, dtype), ops.new_nhwc(n, cout, ho, wo, DEV, dtype)
    r0 = gaussian_delta(n, cout, ho, wo, 1.0, 1.0, seed=8)[0]
    res, res_valu, res_ref = _dev(r0).clone(), _dev(r0).clone(), r0.clone()
    for step, (dens, with_res) in enumerate([(0.2, False), (0.07, True)]):
        d, m = gaussian_delta(n, cin, h, w, dens, 0.5, seed=900 + 10 * cin + step)
        d = q(d)
        ref = io.conv_incr(d, wt, s, p)
        dm = m.to(DEV)
        ops.build_mask_tiles(dm, None, n, h, w, _lib.FOOT_CONV, k, s, p, ts)
        x = _dev(torch.where(m.bool().expand_as(d), d, torch.full_like(d, float("nan")))).to(dtype)   # inactive pixels are never read
        for o, r, path in ((out, res, _lib.PATH_AUTO), (out_valu, res_valu, _lib.PATH_VALU)):
            ops.conv_masked(x, dm, None, None, filt, k, s, p, ts, o, r if with_res else None,
                            _lib.ACT_RELU if with_res else _lib.ACT_NONE, 0.0, path)
        torch.cuda.synchronize()
        got, valu = out.float().cpu(), out_valu.float().cpu()
        want = torch.relu(res_ref + ref) - torch.relu(res_ref) if with_res else ref
        if with_res:
            res_ref = res_ref + ref
        assert torch.isfinite(got).all()
        assert torch.allclose(got, want, **tol(want)), "step %d max|diff| = %.3e" % (step, (got - want).abs().max())
        assert torch.allclose(got, valu, **tol(valu)), "step %d vs VALU %.3e" % (step, (got - valu).abs().max())
        foot = torch.from_numpy(mo.footprint_conv(m[:, 0].numpy(), k, s, p)).bool().unsqueeze(1)
        assert torch.count_nonzero(got * (~foot)) == 0
    assert torch.allclose(res.cpu(), res_ref, rtol=RTOL, atol=bf16_atol(ref, 2.0) if bf else ATOL)


# The persistent form of the 64 -> 32 bf16 up-sampling conv (the last decoder of the batched network) takes planes of
# at least 2048 tiles.  Same inputs once as a batch of three ragged frames (2250 tiles: the persistent kernel) and once
# frame by frame (750 tiles each: one workgroup per tile) must agree bit for bit -- deltas and reservoirs -- over three
# steps with fresh masks (stale tiles, an empty step), one and two inputs, with and without the reservoir epilogue;
# and both match the oracle.
def test_persistent_upsampled_conv_agrees_with_the_one_tile_kernel():
    bf = torch.bfloat16
    n, c, cout, h, w = 3, 64, 32, 100, 118                   # output 200 x 236: 25 x 30 tiles per frame, ragged right edge
    q = lambda t: t.to(bf).float()
    wt = q(he_normal_conv_weight(cout, c, 5, 9))
    filt = _filt(wt)
    assert _lib.tile_capacity(n, 2 * h, 2 * w) >= 2048 > _lib.tile_capacity(1, 2 * h, 2 * w)
    big = dict(up=TileMask(n, 2 * h, 2 * w, DEV), ts=TileMask(n, 2 * h, 2 * w, DEV), out=ops.new_nhwc(n, cout, 2 * h, 2 * w, DEV, bf))
    one = [dict(up=TileMask(1, 2 * h, 2 * w, DEV), ts=TileMask(1, 2 * h, 2 * w, DEV), out=ops.new_nhwc(1, cout, 2 * h, 2 * w, DEV, bf))
           for _ in range(n)]
    r0 = gaussian_delta(n, cout, 2 * h, 2 * w, 1.0, 1.0, seed=3)[0]
    res_big = _dev(r0).clone()
    res_one = [_dev(r0[i:i + 1]).clone() for i in range(n)]
    res_ref = r0.clone()
    for step, (da, db, two, with_res) in enumerate([(0.2, 0.1, True, True), (0.0, 0.0, True, False), (0.05, 0.0, False, True),
                                                    (0.3, 0.2, True, False)]):
        a, ma = gaussian_delta(n, c, h, w, da, 0.5, seed=100 + step) if da > 0 else (torch.zeros(n, c, h, w), torch.zeros(n, 1, h, w, dtype=torch.uint8))
        b, mb = gaussian_delta(n, c, h, w, db, 0.5, seed=200 + step) if db > 0 else (torch.zeros(n, c, h, w), torch.zeros(n, 1, h, w, dtype=torch.uint8))
        a, b = q(a), q(b)
        ref = io.conv_incr(q(io.interp_incr(a + b if two else a)), wt, 1, 2)
        act = _lib.ACT_RELU if with_res else _lib.ACT_NONE

        def run(sets, ad, am, bd, bm, res):
            nn = ad.shape[0]
            ops.build_mask_tiles(am, bm if two else None, nn, h, w, _lib.FOOT_UP2X, 0, 0, 0, sets["up"])
            ops.build_mask_tiles(sets["up"], None, nn, 2 * h, 2 * w, _lib.FOOT_CONV, 5, 1, 2, sets["ts"])
            ops.upconv_masked(ad, am, bd if two else None, bm if two else None, filt, 5, 2, sets["ts"], sets["out"],
                              res if with_res else None, act)
        ad, bd, am, bm = _dev(a).to(bf), _dev(b).to(bf), ma.to(DEV), mb.to(DEV)
        run(big, ad, am, bd, bm, res_big)
        for i in range(n):
            run(one[i], ad[i:i + 1].contiguous(memory_format=torch.channels_last), am[i:i + 1].contiguous(),
                bd[i:i + 1].contiguous(memory_format=torch.channels_last), bm[i:i + 1].contiguous(), res_one[i])
        torch.cuda.synchronize()
        for i in range(n):
            assert torch.equal(big["out"][i:i + 1], one[i]["out"]), "step %d frame %d: delta" % (step, i)
            assert torch.equal(res_big[i:i + 1], res_one[i]), "step %d frame %d: reservoir" % (step, i)
        got = big["out"].float().cpu()
        want = torch.relu(res_ref + ref) - torch.relu(res_ref) if with_res else ref
        assert torch.allclose(got, want, rtol=BF16_RTOL, atol=bf16_atol(want, 2.0)), "step %d max|diff| = %.3e" % (step, (got - want).abs().max())
        if with_res:
            res_ref = res_ref + ref
            assert torch.allclose(res_big.cpu(), res_ref, rtol=RTOL, atol=bf16_atol(ref, 2.0))
        # clean delta: zero outside the active pixels of the tile set
        assert torch.count_nonzero(big["out"].float() * (1 - big["ts"].pixmask.float())) == 0


def test_fused_tail_equals_decoder_then_prediction():
    # mie_upconv_pred_masked: last decoder + 1x1 prediction over (its increment + a second delta) + sigmoid increment in
    # one kernel, against the two launches it replaces (same decoder arithmetic: the decoder's reservoir must come out
    # bit-equal; the prediction's 64-term sum is regrouped, fp32) and against a CPU restatement.  Four steps with
    # fresh masks: stale tiles of the prediction's set, an empty step, one input only.
    bf = torch.bfloat16
    n, c, cout, h, w = 3, 64, 32, 100, 118
    H, W = 2 * h, 2 * w
    q = lambda t: t.to(bf).float()
    wt = q(he_normal_conv_weight(cout, c, 5, 9))
    filt = _filt(wt)
    pw = q(torch.randn(cout, generator=torch.Generator().manual_seed(4)) * 0.3)      # bf16 networks carry bf16 weights
    pred_filt = _filt(torch.cat((pw, pw)).reshape(1, 2 * cout, 1, 1))                  # [1, 64, 1, 1] -> rows repeated
    pred_w = torch.stack((pw, pw)).contiguous().to(DEV)
    assert ops.upconv_pred_takes(c, cout, 5, 1, 2, filt, bf, _lib.tile_capacity(n, H, W), _lib.ACT_RELU)
    sets = [dict(up=TileMask(n, H, W, DEV), dec=TileMask(n, H, W, DEV), pred=TileMask(n, H, W, DEV)) for _ in range(2)]
    y_buf = ops.new_nhwc(n, cout, H, W, DEV, bf)
    outs = [ops.new_nhwc(n, 1, H, W, DEV, bf) for _ in range(2)]
    r0 = gaussian_delta(n, cout, H, W, 1.0, 1.0, seed=3)[0]
    p0 = gaussian_delta(n, 1, H, W, 1.0, 1.0, seed=5)[0]
    res = [_dev(r0).clone() for _ in range(2)]
    pres = [_dev(p0).clone() for _ in range(2)]
    res_ref, pres_ref = r0.clone(), p0.clone()
    for step, (da, db, ds, two) in enumerate([(0.2, 0.1, 0.1, True), (0.0, 0.0, 0.0, True), (0.05, 0.0, 0.3, False), (0.3, 0.2, 0.02, True)]):
        zeros = lambda ch, hh, ww: (torch.zeros(n, ch, hh, ww), torch.zeros(n, 1, hh, ww, dtype=torch.uint8))
        a, ma = gaussian_delta(n, c, h, w, da, 0.5, seed=100 + step) if da > 0 else zeros(c, h, w)
        b, mb = gaussian_delta(n, c, h, w, db, 0.5, seed=200 + step) if db > 0 else zeros(c, h, w)
        sk, ms = gaussian_delta(n, cout, H, W, ds, 0.5, seed=300 + step) if ds > 0 else zeros(cout, H, W)
        a, b, sk = q(a), q(b), q(sk)
        ad, bd, am, bm = _dev(a).to(bf), _dev(b).to(bf), ma.to(DEV), mb.to(DEV)
        skd, msd = _dev(sk).to(bf), ms.to(DEV)
        for s_ in sets:
            ops.build_mask_tiles(am, bm if two else None, n, h, w, _lib.FOOT_UP2X, 0, 0, 0, s_["up"])
            ops.build_mask_tiles(s_["up"], None, n, H, W, _lib.FOOT_CONV, 5, 1, 2, s_["dec"])
            ops.build_mask_tiles(s_["dec"], msd, n, H, W, _lib.FOOT_CONV, 1, 1, 0, s_["pred"])
        # the two launches
        ops.upconv_masked(ad, am, bd if two else None, bm if two else None, filt, 5, 2, sets[0]["dec"], y_buf, res[0], _lib.ACT_RELU)
        ops.conv_masked(y_buf, sets[0]["dec"], skd, msd, pred_filt, 1, 1, 0, sets[0]["pred"], outs[0], pres[0], _lib.ACT_SIGMOID)
        # the one
        ops.upconv_pred_masked(ad, am, bd if two else None, bm if two else None, filt, sets[1]["pred"], res[1], _lib.ACT_RELU, 0.0,
                               skd, msd, pred_w, pres[1], _lib.ACT_SIGMOID, 0.0, outs[1])
        torch.cuda.synchronize()
        # CPU restatement
        conv = io.conv_incr(q(io.interp_incr(a + b if two else a)), wt, 1, 2)
        y = q(torch.relu(res_ref + conv) - torch.relu(res_ref))
        res_ref = res_ref + conv
        z = ((y + sk) * pw.view(1, -1, 1, 1)).sum(1, keepdim=True)
        want = torch.sigmoid(pres_ref + z) - torch.sigmoid(pres_ref)
        pres_ref = pres_ref + z
        assert torch.equal(res[0], res[1]), "step %d: decoder reservoir" % step
        assert torch.allclose(pres[0], pres[1], rtol=1e-5, atol=1e-5), "step %d: prediction reservoir %.3e" % (step, (pres[0] - pres[1]).abs().max())
        assert torch.allclose(outs[0].float(), outs[1].float(), rtol=2 ** -7, atol=2 ** -9), "step %d: prediction delta %.3e" % (
            step, (outs[0].float() - outs[1].float()).abs().max())
        # (the GPU's y differs from the CPU's by a bf16 rounding step where the conv sums differ in their last bits: a few
        # 1e-4 per step on a reservoir of order 1, carried over the steps)
        assert torch.allclose(pres[1].cpu(), pres_ref, rtol=1e-3, atol=4e-3), "step %d: reservoir vs CPU %.3e" % (
            step, (pres[1].cpu() - pres_ref).abs().max())
        assert torch.allclose(outs[1].float().cpu(), want, rtol=BF16_RTOL, atol=2e-3), "step %d: delta vs CPU %.3e" % (
            step, (outs[1].float().cpu() - want).abs().max())
        # clean delta: zero outside the pixels of the prediction's tile set
        assert torch.count_nonzero(outs[1].float() * (1 - sets[1]["pred"].pixmask.float())) == 0
