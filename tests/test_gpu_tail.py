"""GPU parity of the classifier-tail ops on deltas (per-channel scale, adaptive average pooling, fully
connected layer) and of the modules built on them, against the CPU oracle, through the C ABI.
fp32 tolerance rtol 1e-4 / atol 1e-5; bf16 deltas rtol 2e-2."""
import pytest
import torch

from maskedincrementeval_amd import _lib, ops
from maskedincrementeval_amd import mask_incr_modules as mm
from maskedincrementeval_amd.masked_types import TileMask
from maskedincrementeval_amd.synthetic import gaussian_delta
from oracle import incr_oracle as io

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _cl(t):
    return ops.as_nhwc(t.to(DEV).contiguous(memory_format=torch.channels_last))


def _tol(dtype):
    return dict(rtol=2e-2, atol=2e-2) if dtype == torch.bfloat16 else dict(rtol=1e-4, atol=1e-5)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("c", [5, 16, 70])
def test_scale_incr_matches_batch_norm_on_a_delta(c, dtype):
    n, h, w = 2, 19, 27
    d, m = gaussian_delta(n, c, h, w, 0.2, 0.5, seed=c)
    if dtype == torch.bfloat16:
        d = d.to(dtype).float()
    var, gamma = torch.rand(c) + 0.5, torch.randn(c)
    ref = io.bn_incr(d, var, gamma, 1e-5)
    scale = (gamma / torch.sqrt(var + 1e-5)).to(DEV)
    ts = TileMask(n, h, w, DEV)
    ops.build_mask_tiles(m.to(DEV), None, n, h, w, _lib.FOOT_CONV, 1, 1, 0, ts)
    poisoned = torch.where(m.bool().expand_as(d), d, torch.full_like(d, float("nan")))
    out = ops.new_nhwc(n, c, h, w, DEV, dtype)
    ops.scale_incr(_cl(poisoned).to(dtype), scale, out, ts)
    torch.cuda.synchronize()
    got = out.float().cpu()
    assert torch.isfinite(got).all()                   # inactive pixels are not read
    assert torch.allclose(got, ref, **_tol(dtype)), (got - ref).abs().max()
    assert torch.count_nonzero(got * (1 - m.float())) == 0


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("h,w,size", [(7, 7, 1), (10, 13, (3, 4)), (5, 6, (7, 9)), (16, 24, (None, 5))])
def test_avgpool_incr_matches_oracle(h, w, size, dtype):
    n, c = 2, 300
    d, m = gaussian_delta(n, c, h, w, 0.4, 0.5, seed=h * w)
    if dtype == torch.bfloat16:
        d = d.to(dtype).float()
    ref = io.avgpool_incr(d, size)
    pool = mm.nnAdaptiveAvgPool2dIncr(size)
    poisoned = torch.where(m.bool().expand_as(d), d, torch.full_like(d, float("nan")))
    out, mask = pool([_cl(poisoned).to(dtype), m.to(DEV)])
    torch.cuda.synchronize()
    assert mask is None and out.shape == ref.shape
    got = out.float().cpu()
    assert torch.isfinite(got).all()
    assert torch.allclose(got, ref, **_tol(dtype)), (got - ref).abs().max()
    # without a mask every pixel counts
    out2, _ = pool([_cl(d).to(dtype), None])
    assert torch.allclose(out2.float().cpu(), ref, **_tol(dtype))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("n,f_in,f_out", [(1, 512, 1000), (3, 100, 37), (2, 64, 64), (4, 700, 130)])
def test_linear_incr_matches_oracle_and_skips_zero_features(n, f_in, f_out, dtype):
    g = torch.Generator().manual_seed(f_in + f_out)
    w = torch.randn(f_out, f_in, generator=g) / f_in ** 0.5
    d = torch.randn(n, f_in, generator=g)
    dead = torch.rand(f_in, generator=g) < 0.7          # features no sample touches
    d[:, dead] = 0.0
    if dtype == torch.bfloat16:
        d = d.to(dtype).float()
    ref = io.linear_incr(d, w)
    wt = w.t().contiguous().to(DEV)
    wt[dead.to(DEV)] = float("nan")                      # rows that must not be read
    out = torch.empty(n, f_out, dtype=dtype, device=DEV)
    ops.linear_incr(d.to(DEV).to(dtype), wt, out)
    torch.cuda.synchronize()
    got = out.float().cpu()
    assert torch.isfinite(got).all()
    assert torch.allclose(got, ref, **_tol(dtype)), (got - ref).abs().max()
    # the module: transposed weight copy follows weight updates
    lin = mm.nnLinearIncr(f_in, f_out).to(DEV)
    with torch.no_grad():
        lin.weight.copy_(w)
        y1, _ = lin([d.to(DEV).to(dtype), None])
        lin.weight.mul_(2.0)
        y2, _ = lin([d.to(DEV).to(dtype), None])
    assert torch.allclose(y1.float().cpu(), ref, **_tol(dtype))
    assert torch.allclose(y2.float().cpu(), 2 * ref, **_tol(dtype))


def test_classifier_tail_accumulates_to_the_dense_result():
    # conv -> batch norm -> relu -> max pool -> global average pool -> linear: refresh + sum of
    # increments equals the dense net on the accumulated input (reference tests/test_network.py:24-31)
    torch.manual_seed(5)
    n, cin, h, w, classes = 2, 8, 24, 32, 10
    body = mm.nnSequentialIncr(mm.nnConvIncr(cin, 16, 3, 1, 1), mm.nnBatchNorm2dIncr(16), mm.nnReluIncr(),
                               mm.nnMaxPool2dIncr(2, 2), mm.nnAdaptiveAvgPool2dIncr(1)).to(DEV).eval()
    fc = mm.nnLinearIncr(16, classes).to(DEV).eval()
    bn = body[1]
    with torch.no_grad():
        bn.running_mean.normal_(0, 0.2)
        bn.running_var.uniform_(0.5, 1.5)
        bn.weight.normal_(1.0, 0.2)
        bn.bias.normal_(0, 0.2)

    def dense(x):
        conv = body[0]
        y = torch.nn.functional.conv2d(x, conv.weight.detach().cpu(), conv.bias.detach().cpu(), 1, 1)
        y = torch.nn.functional.batch_norm(y, bn.running_mean.cpu(), bn.running_var.cpu(), bn.weight.detach().cpu(),
                                           bn.bias.detach().cpu(), False, 0.0, bn.eps)
        y = torch.nn.functional.max_pool2d(torch.relu(y), 2, 2)
        y = torch.nn.functional.adaptive_avg_pool2d(y, 1).flatten(1)
        return torch.nn.functional.linear(y, fc.weight.detach().cpu(), fc.bias.detach().cpu())

    x = torch.randn(n, cin, h, w)
    with torch.no_grad():
        acc = fc.forward_refresh_reservoirs(body.forward_refresh_reservoirs(_cl(x)).flatten(1)).cpu().clone()
    assert torch.allclose(acc, dense(x), rtol=1e-4, atol=1e-5)
    for step in range(5):
        d, m = gaussian_delta(n, cin, h, w, 0.1, 0.3, seed=900 + step)
        with torch.no_grad():
            pooled, _ = body([_cl(d), m.to(DEV)])
            out, _ = fc([pooled.flatten(1), None])
        torch.cuda.synchronize()
        acc += out.cpu()
        x = x + d
        assert torch.allclose(acc, dense(x), rtol=1e-4, atol=1e-5), (step, (acc - dense(x)).abs().max())
