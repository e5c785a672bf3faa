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
