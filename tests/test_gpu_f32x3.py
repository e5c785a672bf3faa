"""The three-term bf16 form of the fp32 matrix-core convs (MIE_DTYPE_F32_BF16X3): filter copy, accuracy against an
fp64 reference next to the fp32 instruction's, agreement of the two forms in every kernel family, error paths.
No counterpart in the reference, whose convs have one arithmetic (cuDNN fp32)."""
import ctypes

import pytest
import torch
import torch.nn.functional as F

from maskedincrementeval_amd import _lib, ops
from maskedincrementeval_amd.masked_types import TileMask
from maskedincrementeval_amd.synthetic import blob_mask, he_normal_conv_weight

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _dev(t):
    return ops.as_nhwc(t.to(DEV).contiguous(memory_format=torch.channels_last))


def _filt(w_oihw):
    return ops.ConvFilter(w_oihw.permute(1, 2, 3, 0).contiguous().to(DEV))


def _err():
    msg = _lib.lib().mie_last_error_string()
    return msg.decode("utf-8", "replace") if msg else ""


def test_three_term_filter_copy_sums_to_the_weights_exactly():
    cin, k, cout = 32, 3, 40
    w = torch.randn(cin, k, k, cout) * torch.logspace(-6, 3, cout)          # a wide range of magnitudes
    packed = ops.pack_filter(w.contiguous().to(DEV), x3=True).cpu()          # [cin/16, k*k, 3, 2, cout, 8] bf16
    assert packed.dtype == torch.bfloat16 and tuple(packed.shape) == (cin // 16, k * k, 3, 2, cout, 8)
    # term planes back in [cin, k, k, cout] order
    terms = packed.permute(2, 0, 3, 5, 1, 4).reshape(3, cin, k * k, cout).reshape(3, cin, k, k, cout).double()
    assert torch.equal(terms.sum(0), w.double()), "hi + mid + lo must be the fp32 weight, bit for bit"
    hi = w.to(torch.bfloat16).double()
    assert torch.equal(terms[0], hi), "the first term is the weight rounded to bf16"
    assert (terms[1].abs() <= w.double().abs() * 2.0 ** -8 + 1e-300).all()
    assert (terms[2].abs() <= w.double().abs() * 2.0 ** -16 + 1e-300).all()


@pytest.mark.parametrize("cin,cout,k,h,w,density", [(64, 64, 3, 40, 40, 1.0), (64, 32, 5, 33, 47, 0.3), (256, 256, 3, 33, 44, 1.0),
                                                      (256, 128, 5, 34, 42, 1.0), (128, 96, 3, 20, 28, 0.5)])
def test_error_against_fp64_beside_the_fp32_instructions(cin, cout, k, h, w, density):
    p = k // 2
    torch.manual_seed(cin + cout + k)
    x = torch.randn(1, cin, h, w)
    mask = None
    if density < 1.0:
        mask = torch.from_numpy(blob_mask(h, w, density, seed=3)).view(1, 1, h, w)
        x = x * mask
    wt = he_normal_conv_weight(cout, cin, k, 7)
    ref = F.conv2d(x.double(), wt.double(), padding=p)
    bound = F.conv2d(x.double().abs(), wt.double().abs(), padding=p)            # sum of |x||w| per output
    ts = TileMask(1, h, w, DEV)
    dm = None if mask is None else mask.to(DEV)
    ops.build_mask_tiles(dm, None, 1, h, w, _lib.FOOT_CONV, k, 1, p, ts)
    active = torch.ones(1, 1, h, w, dtype=torch.bool) if mask is None else \
        F.max_pool2d(mask.float(), k, 1, p) > 0
    err = {}
    old = ops.f32_matmul
    try:
        for mode in ("native", "bf16x3"):
            ops.f32_matmul = mode
            out = ops.new_nhwc(1, cout, h, w, DEV)
            ops.conv_masked(_dev(x), dm, None, None, _filt(wt), k, 1, p, ts, out, path=_lib.PATH_MFMA, workspace=False)
            torch.cuda.synchronize()
            e = ((out.cpu().double() - ref).abs() * active)
            err[mode] = (e.max().item(), (e / bound.clamp_min(1e-30)).max().item())
    finally:
        ops.f32_matmul = old
    # relative to sum |x||w| both stay within a few fp32 rounding steps, and the three-term form within a quarter of the
    # fp32 instruction's error (it is the smaller one where both kernels split the contraction the same way)
    assert err["bf16x3"][1] < 4e-7 and err["native"][1] < 4e-7, err
    assert err["bf16x3"][0] <= 1.25 * err["native"][0] + 1e-7, err


def test_library_says_which_shapes_take_the_three_term_form():
    L = _lib.lib()
    assert L.mie_conv_f32x3_takes(3, 1, 64, 64, 256) == 1
    assert L.mie_conv_f32x3_takes(5, 1, 256, 0, 128) == 1
    assert L.mie_conv_f32x3_takes(5, 2, 64, 0, 128) == 1
    assert L.mie_conv_f32x3_takes(5, 2, 48, 16, 64) == 1          # stride 2: chunks of 16 channels
    assert L.mie_conv_f32x3_takes(3, 2, 64, 0, 64) == 0           # 3x3 stride 2 stays on the fp32 instruction
    assert L.mie_conv_f32x3_takes(7, 2, 64, 0, 64) == 0
    assert L.mie_conv_f32x3_takes(3, 1, 48, 0, 64) == 0           # 48 input channels: not whole chunks
    assert L.mie_conv_f32x3_takes(1, 1, 64, 0, 64) == 0
    old = ops.f32_matmul
    try:
        ops.f32_matmul = "native"
        assert not ops.f32x3_takes(3, 1, 64, 0, 64)
        ops.f32_matmul = "bf16x3"
        assert ops.f32x3_takes(3, 1, 64, 0, 64)
        ops.f32_matmul = "fp16"
        with pytest.raises(ValueError):
            ops.f32x3_takes(3, 1, 64, 0, 64)
    finally:
        ops.f32_matmul = old


def test_three_term_dtype_is_refused_where_it_has_no_kernel():
    L = _lib.lib()
    n, c, h, w, k = 1, 64, 16, 16, 3
    x = _dev(torch.randn(n, c, h, w))
    filt = _filt(he_normal_conv_weight(c, c, k, 1))
    plain, mc3 = filt.for_dtype(torch.float32, x3=True)
    ts = TileMask(n, h, w, DEV)
    ops.build_mask_tiles(None, None, n, h, w, _lib.FOOT_CONV, k, 1, 1, ts)
    out = ops.new_nhwc(n, c, h, w, DEV)
    def call(path, stride, pad, ts_):
        return L.mie_conv_masked(ops.nhwc_ptr(x, "x"), None, c, None, None, 0, h, w, plain.data_ptr(), mc3.data_ptr(), c, k, stride,
                                 pad, c, ts_.ref, ops.nhwc_ptr(out, "out"), None, None, _lib.ACT_NONE, 0.0, path,
                                 _lib.DTYPE_F32_BF16X3, None)
    assert call(_lib.PATH_MFMA, 1, 1, ts) == 0
    assert call(_lib.PATH_AUTO, 1, 1, ts) == 0
    rc = call(_lib.PATH_VALU, 1, 1, ts)
    assert rc != 0 and "matrix-core" in _err()
    # a 1x1 conv has no three-term kernel
    w1 = _filt(he_normal_conv_weight(c, c, 1, 2))
    plain1, mc1 = w1.for_dtype(torch.float32, x3=True)
    rc = L.mie_conv_masked(ops.nhwc_ptr(x, "x"), None, c, None, None, 0, h, w, plain1.data_ptr(), mc1.data_ptr(), c, 1, 1, 0, c,
                           ts.ref, ops.nhwc_ptr(out, "out"), None, None, _lib.ACT_NONE, 0.0, _lib.PATH_AUTO,
                           _lib.DTYPE_F32_BF16X3, None)
    assert rc != 0 and "mie_conv_f32x3_takes" in _err()
    # the pointwise entry points know two delta types only
    rc = L.mie_mask_from_delta(ops.nhwc_ptr(x, "x"), n, h, w, c, 0.0, ts.pixmask.data_ptr(), _lib.DTYPE_F32_BF16X3, None)
    assert rc != 0


def _conv_both_modes(x, wt, k, modes=("native", "bf16x3")):
    n, cin, h, w = x.shape
    cout, p = wt.shape[0], k // 2
    ts = TileMask(n, h, w, DEV)
    ops.build_mask_tiles(None, None, n, h, w, _lib.FOOT_CONV, k, 1, p, ts)
    outs = {}
    old = ops.f32_matmul
    try:
        for mode in modes:
            ops.f32_matmul = mode
            out = ops.new_nhwc(n, cout, h, w, DEV)
            ops.conv_masked(_dev(x), None, None, None, _filt(wt), k, 1, p, ts, out, path=_lib.PATH_MFMA, workspace=False)
            torch.cuda.synchronize()
            outs[mode] = out.cpu()
    finally:
        ops.f32_matmul = old
    return outs


@pytest.mark.parametrize("lo_exp,hi_exp", [(-12, 12), (-30, 30), (-36, -30)])
def test_error_bound_holds_over_many_decades_of_magnitude(lo_exp, hi_exp):
    # Inputs and weights whose magnitudes span many decades -- per input channel a scale 10^e on the delta and,
    # in the first two cases, 10^-e on the weights, so that every channel contributes O(1) products from operands
    # between 1e-30 and 1e+30; in the last case all operands are tiny (1e-36 .. 1e-30): the second and third bf16
    # terms of such values (2^-9 and 2^-18 of them) reach the subnormal range.  The error against fp64 must stay
    # within a few fp32 rounding steps of sum |x||w| for the three-term form exactly as for the fp32 instruction.
    cin, cout, k, h, w = 64, 64, 3, 24, 24
    g = torch.Generator().manual_seed(11)
    exps = torch.linspace(lo_exp, hi_exp, cin, dtype=torch.float64)
    sx = (10.0 ** exps).view(1, cin, 1, 1)
    x = (torch.randn(1, cin, h, w, generator=g, dtype=torch.float64) * sx).float()
    wt = torch.randn(cout, cin, k, k, generator=g, dtype=torch.float64)
    if hi_exp > 0:
        wt = wt / sx.view(1, cin, 1, 1)
    wt = wt.float()
    assert torch.isfinite(x).all() and torch.isfinite(wt).all()
    ref = F.conv2d(x.double(), wt.double(), padding=k // 2)
    bound = F.conv2d(x.double().abs(), wt.double().abs(), padding=k // 2)
    outs = _conv_both_modes(x, wt, k)
    rel = {m: ((o.double() - ref).abs() / bound.clamp_min(1e-300)).max().item() for m, o in outs.items()}
    # (fp32 results below the normal range lose bits in any arithmetic: the tiny case is compared where |ref| is normal)
    assert rel["native"] < 4e-7 and rel["bf16x3"] < 4e-7, rel
    assert torch.isfinite(outs["bf16x3"]).all()


def test_non_finite_deltas_never_come_out_as_finite_numbers():
    # The three-term split does not carry non-finite values (inf - inf is NaN), and a value of 3.39e38 or more rounds to
    # an infinite first term.  What the library guarantees, and this test pins: an output whose window holds such a
    # value is non-finite in BOTH arithmetic forms (never a finite wrong number), outputs whose windows hold none
    # are unaffected, and with f32_matmul = "native" the result is what an IEEE fp32 conv gives (inf stays inf).
    cin, cout, k, h, w = 32, 32, 3, 24, 24
    g = torch.Generator().manual_seed(12)
    x = torch.randn(1, cin, h, w, generator=g)
    wt = torch.randn(cout, cin, k, k, generator=g).abs() + 0.1          # positive weights: inf * w = inf, no cancellation
    clean = _conv_both_modes(x, wt, k)
    bad = x.clone()
    bad[0, 3, 5, 7] = float("inf")
    bad[0, 9, 17, 4] = float("-inf")
    bad[0, 20, 11, 19] = float("nan")
    bad[0, 1, 20, 20] = 3.4e38                                            # finite, rounds to an infinite bf16 term
    touched = torch.zeros(1, 1, h, w)
    for (y, x_) in ((5, 7), (17, 4), (11, 19), (20, 20)):
        touched[0, 0, y, x_] = 1
    touched = (F.max_pool2d(touched, k, 1, k // 2) > 0).expand(1, cout, h, w)
    outs = _conv_both_modes(bad, wt, k)
    ieee = F.conv2d(bad, wt, padding=k // 2)
    for mode in ("native", "bf16x3"):
        o = outs[mode]
        assert torch.equal(o[~touched], clean[mode][~touched]), mode + ": outputs away from the non-finite values changed"
    # native: IEEE propagation, as torch's fp32 conv has it (inf where it has inf, nan where it has nan)
    nat = outs["native"]
    assert torch.equal(torch.isnan(nat), torch.isnan(ieee)) and torch.equal(torch.isinf(nat), torch.isinf(ieee))
    assert torch.equal(nat[torch.isinf(ieee)], ieee[torch.isinf(ieee)])
    # three-term form: every output the IEEE conv makes non-finite is non-finite (NaN in place of inf is allowed) ...
    x3 = outs["bf16x3"]
    assert (~torch.isfinite(x3[~torch.isfinite(ieee)])).all()
    # ... and so is every output whose window holds the 3.4e38 value, which the fp32 conv still carries
    near_big = torch.zeros(1, 1, h, w)
    near_big[0, 0, 20, 20] = 1
    near_big = (F.max_pool2d(near_big, k, 1, k // 2) > 0).expand(1, cout, h, w)
    assert (~torch.isfinite(x3[near_big])).all()
