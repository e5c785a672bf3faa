"""GPU parity of the point-wise incremental kernels against the CPU oracle, through the
C ABI: activation increments (ReLU / LeakyReLU bit-exact, sigmoid / tanh within
rtol 1e-4 / atol 1e-5), product rule, sum, bilinear x2, fused ConvLSTM gates."""
import numpy as np
import pytest
import torch

from maskedincrementeval_amd import _lib, ops
from maskedincrementeval_amd.masked_types import TileMask
from maskedincrementeval_amd.synthetic import gaussian_delta
from oracle import incr_oracle as io
from oracle import mask_oracle as mo

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
RTOL, ATOL = 1e-4, 1e-5


def _dev(t):
    return ops.as_nhwc(t.to(DEV).contiguous(memory_format=torch.channels_last))


def _close(got, ref, what=""):
    got = got.cpu()
    err = (got - ref).abs().max().item()
    assert torch.allclose(got, ref, rtol=RTOL, atol=ATOL), "%s max|diff| = %.3e" % (what, err)


def _identity_ts(ts, mask, n, h, w):
    ops.build_mask_tiles(None if mask is None else mask.to(DEV), None, n, h, w, _lib.FOOT_CONV, 1, 1, 0, ts)
    return ts


def _randn(*shape, seed):
    return torch.randn(shape, generator=torch.Generator().manual_seed(seed))


@pytest.mark.parametrize("kind,slope,op,exact", [
    (_lib.ACT_RELU, 0.0, torch.relu, True),
    (_lib.ACT_LEAKY_RELU, 0.01, io.leaky_relu, True),
    (_lib.ACT_SIGMOID, 0.0, torch.sigmoid, False),
    (_lib.ACT_TANH, 0.0, torch.tanh, False)])
@pytest.mark.parametrize("n,c,h,w", [(1, 32, 45, 61), (2, 5, 19, 23), (1, 1, 16, 24)])
def test_activation_increment(kind, slope, op, exact, n, c, h, w):
    r0 = _randn(n, c, h, w, seed=c)
    res_cpu, res_gpu = io.Reserve(r0), _dev(r0.clone())
    ts = TileMask(n, h, w, DEV)
    out = ops.new_nhwc(n, c, h, w, DEV)
    refined = torch.zeros((n, 1, h, w), dtype=torch.uint8, device=DEV)
    for step in range(4):
        d, m = gaussian_delta(n, c, h, w, 0.1, 0.7, seed=100 + step + h)
        _identity_ts(ts, m, n, h, w)
        r_old = res_gpu.cpu().clone()
        ops.act_incr(kind, slope, _dev(d), res_gpu, out, ts, refined)
        torch.cuda.synchronize()
        ref = io.act_incr(op, res_cpu, d)
        if exact:
            # reference tests/test_pointops.py:17-22: zero differing elements, reservoir == X + d
            assert torch.count_nonzero(out.cpu() - ref) == 0
            assert torch.count_nonzero(res_gpu.cpu() - res_cpu.reservoir) == 0
        else:
            _close(out, ref, "delta")
            _close(res_gpu, res_cpu.reservoir, "reservoir")
        # emitted mask, staged on the GPU-produced reservoir pair: exact integer function
        r_new = res_gpu.cpu()
        want = ((op(r_new) - op(r_old)) != 0).any(dim=1, keepdim=True) & m.bool()
        if exact:
            assert np.array_equal(refined.cpu().numpy(), want.to(torch.uint8).numpy())
        assert np.array_equal(refined.cpu().numpy(),
                              (out.cpu() != 0).any(dim=1, keepdim=True).to(torch.uint8).numpy())


def test_activation_zero_delta_and_keep_reservoir():
    n, c, h, w = 1, 16, 24, 24
    r0 = _randn(n, c, h, w, seed=1)
    res = _dev(r0.clone())
    ts = _identity_ts(TileMask(n, h, w, DEV), None, n, h, w)
    out = ops.new_nhwc(n, c, h, w, DEV)
    ops.act_incr(_lib.ACT_TANH, 0.0, _dev(torch.zeros(n, c, h, w)), res, out, ts)
    assert torch.count_nonzero(out) == 0 and torch.equal(res.cpu(), r0)
    d = _randn(n, c, h, w, seed=2)
    ops.act_incr(_lib.ACT_RELU, 0.0, _dev(d), res, out, ts, keep_reservoir=True)
    assert torch.equal(res.cpu(), r0)                       # NonlinearPointOpIncr.forward: no accumulate
    assert torch.equal(out.cpu(), torch.relu(r0 + d) - torch.relu(r0))


@pytest.mark.parametrize("n,c,h,w", [(1, 64, 33, 44), (2, 3, 17, 9)])
def test_product_rule(n, c, h, w):
    r1, r2 = _randn(n, c, h, w, seed=3), _randn(n, c, h, w, seed=4)
    R1, R2 = io.Reserve(r1), io.Reserve(r2)
    g1, g2 = _dev(r1.clone()), _dev(r2.clone())
    ts = TileMask(n, h, w, DEV)
    out = ops.new_nhwc(n, c, h, w, DEV)
    for step in range(3):
        d1, m1 = gaussian_delta(n, c, h, w, 0.08, 0.3, seed=200 + step)
        d2, m2 = gaussian_delta(n, c, h, w, 0.05, 0.3, seed=300 + step)
        ops.build_mask_tiles(m1.to(DEV), m2.to(DEV), n, h, w, _lib.FOOT_CONV, 1, 1, 0, ts)
        ops.mul_incr(_dev(d1), m1.to(DEV), g1, _dev(d2), m2.to(DEV), g2, out, ts)
        torch.cuda.synchronize()
        _close(out, io.mul_incr(d1, R1, d2, R2), "product")
        _close(g1, R1.reservoir), _close(g2, R2.reservoir)
        union = (m1 | m2).bool()
        assert torch.count_nonzero(out.cpu() * (~union)) == 0
    # bare IncrPointwiseMultiply: reservoirs untouched
    before = g1.cpu().clone()
    ops.mul_incr(_dev(d1), m1.to(DEV), g1, _dev(d2), m2.to(DEV), g2, out, ts, keep_reservoir=True)
    assert torch.equal(g1.cpu(), before)


@pytest.mark.parametrize("form", ["functional", "module"])
def test_product_of_two_refined_views_of_one_tile_set(form):
    # Two activations applied under ONE tile set each emit a refined pixel mask of their own (a view that
    # shares the tile list).  The product must cover the union of the two masks: a pixel active in the
    # second operand only contributes R1 * d2.
    from maskedincrementeval_amd import mask_incr_functional as mf
    from maskedincrementeval_amd import mask_incr_modules as mm
    n, c, h, w = 1, 8, 24, 40
    parent = TileMask(n, h, w, DEV)
    base = torch.zeros(n, 1, h, w, dtype=torch.uint8)
    base[:, :, 2:20, 3:33] = 1
    ops.build_mask_tiles(base.to(DEV), None, n, h, w, _lib.FOOT_CONV, 1, 1, 0, parent)
    m1, m2 = torch.zeros_like(base), torch.zeros_like(base)
    m1[:, :, 2:10, 3:20] = 1            # view 1: upper left part
    m2[:, :, 6:20, 12:33] = 1           # view 2: lower right part, overlapping view 1
    v1, v2 = parent.with_pixmask(m1.to(DEV)), parent.with_pixmask(m2.to(DEV))
    assert v1.shares_tiles_with(v2)
    d1 = _randn(n, c, h, w, seed=31) * m1.float()
    d2 = _randn(n, c, h, w, seed=32) * m2.float()
    r1, r2 = _randn(n, c, h, w, seed=33), _randn(n, c, h, w, seed=34)
    want = (d2 + r2) * d1 + r1 * d2
    if form == "functional":
        R1, R2 = mf.IncrementReserve(_dev(r1)), mf.IncrementReserve(_dev(r2))
        out, ts = mf.IncrPointwiseMultiply([_dev(d1), v1], R1, [_dev(d2), v2], R2)
    else:
        mod = mm.nnReservedMultiplication()
        mod.forward_refresh_reservoirs(_dev(r1), _dev(r2))
        out, ts = mod([_dev(d1), v1], [_dev(d2), v2])
    torch.cuda.synchronize()
    _close(out, want, "product under the union of two refined masks")
    only2 = (m2.bool() & ~m1.bool()).expand_as(d1)
    assert torch.count_nonzero(out.cpu()[only2]) > 0            # the R1 * d2 term is there
    assert torch.equal(ts.pixmask.cpu(), m1 | m2)


def test_sum_of_deltas():
    n, c, h, w = 2, 32, 21, 35
    ts = TileMask(n, h, w, DEV)
    out = ops.new_nhwc(n, c, h, w, DEV)
    for step in range(3):
        a, ma = gaussian_delta(n, c, h, w, 0.07, 1.0, seed=400 + step)
        b, mb = gaussian_delta(n, c, h, w, 0.04, 1.0, seed=500 + step)
        ops.build_mask_tiles(ma.to(DEV), mb.to(DEV), n, h, w, _lib.FOOT_CONV, 1, 1, 0, ts)
        nan = float("nan")
        pa = torch.where(ma.bool().expand_as(a), a, torch.full_like(a, nan))
        ops.add_incr(_dev(pa), ma.to(DEV), _dev(b), mb.to(DEV), out, ts)
        torch.cuda.synchronize()
        assert torch.equal(out.cpu(), a + b)


@pytest.mark.parametrize("n,c,h,w", [(1, 64, 33, 44), (2, 5, 7, 5), (1, 8, 1, 1)])
def test_bilinear_up2x_with_skip_sum(n, c, h, w):
    ts = TileMask(n, 2 * h, 2 * w, DEV)
    out = ops.new_nhwc(n, c, 2 * h, 2 * w, DEV)
    for step in range(3):
        a, ma = gaussian_delta(n, c, h, w, 0.15, 1.0, seed=600 + step)
        b, mb = gaussian_delta(n, c, h, w, 0.10, 1.0, seed=700 + step)
        ops.build_mask_tiles(ma.to(DEV), mb.to(DEV), n, h, w, _lib.FOOT_UP2X, 0, 0, 0, ts)
        ops.upsample2x_incr(_dev(a), ma.to(DEV), _dev(b), mb.to(DEV), ts, out)
        torch.cuda.synchronize()
        _close(out, io.interp_incr(a + b), "up2x(a+b)")
        fp = torch.from_numpy(mo.footprint_up2x((ma | mb)[:, 0].numpy())).bool().unsqueeze(1)
        assert torch.count_nonzero(out.cpu() * (~fp)) == 0
    ops.build_mask_tiles(ma.to(DEV), None, n, h, w, _lib.FOOT_UP2X, 0, 0, 0, ts)
    ops.upsample2x_incr(_dev(a), ma.to(DEV), None, None, ts, out)
    torch.cuda.synchronize()
    _close(out, io.interp_incr(a), "up2x(a)")


@pytest.mark.parametrize("hid,h,w,with_prev", [(64, 33, 44, False), (16, 19, 27, True), (3, 9, 9, True)])
@pytest.mark.parametrize("f32mode", ["bf16x3", "native"])
def test_fused_convlstm_gates_match_module_chain(hid, h, w, with_prev, f32mode):
    """Gate chain of ConvLSTMIncr.forward (e2depth_incr.py:103-117) in one kernel vs the
    oracle's module-by-module chain; reservoirs are set up from a dense refresh."""
    n = 1
    cin = hid
    wgt = _randn(4 * hid, cin + hid, 3, 3, seed=5) * (0.5 / (cin * 9) ** 0.5)
    bias = _randn(4 * hid, seed=6) * 0.1
    cell = io.ConvLSTMOracle(wgt, bias, hid)
    x0, h0, c0 = _randn(n, cin, h, w, seed=7), _randn(n, hid, h, w, seed=8), _randn(n, hid, h, w, seed=9)
    cell.refresh(x0, (h0, c0))
    gates_res = _dev(torch.cat([cell.r[k].reservoir for k in ("sig1", "sig2", "sig3", "tanh1")], 1))
    cprev_res = _dev(cell.r["m2b"].reservoir.clone())
    cell_res = _dev(cell.r["tanh2"].reservoir.clone())
    ts = TileMask(n, h, w, DEV)
    dh = ops.new_nhwc(n, hid, h, w, DEV)
    dc = ops.new_nhwc(n, hid, h, w, DEV)
    acc_h, acc_h_ref = torch.zeros(n, hid, h, w), torch.zeros(n, hid, h, w)
    for step in range(5):
        dx, mx = gaussian_delta(n, cin, h, w, 0.1, 0.3, seed=800 + step)
        prev = None
        if with_prev:
            dhp, mh = gaussian_delta(n, hid, h, w, 0.05, 0.2, seed=900 + step)
            dcp, _ = gaussian_delta(n, hid, h, w, 0.05, 0.2, seed=900 + step)   # same mask as dhp
            dcp = dcp * 0.5
            prev = (dhp, dcp)
        gates_delta = io.conv_incr(torch.cat((dx, prev[0] if prev else torch.zeros(n, hid, h, w)), 1), wgt, 1, 1)
        gmask = torch.from_numpy(mo.footprint_conv(((mx | mh) if with_prev else mx)[:, 0].numpy(), 3, 1, 1)).unsqueeze(1)
        _identity_ts(ts, gmask, n, h, w)
        ops.convlstm_gates_incr(_dev(gates_delta), gates_res, _dev(prev[1]) if prev else None,
                                mh.to(DEV) if prev else None, cprev_res, cell_res, dh, dc, ts)
        torch.cuda.synchronize()
        dh_ref, dc_ref = cell.incr(dx, prev)
        _close(dh, dh_ref, "dh step %d" % step)
        _close(dc, dc_ref, "dc step %d" % step)
        acc_h += dh.cpu()
        acc_h_ref += dh_ref
    _close(acc_h, acc_h_ref, "accumulated hidden")
    _close(cell_res, cell.r["tanh2"].reservoir, "cell reservoir")
    _close(gates_res[:, :hid], cell.r["sig1"].reservoir, "in-gate reservoir")


@pytest.mark.parametrize("n,c,h,w,k_on_device", [(1, 32, 45, 61, True), (2, 5, 19, 23, False), (1, 1, 16, 24, True)])
def test_kfence_quantiser_is_bit_exact(n, c, h, w, k_on_device):
    # KFencedMaskModule.forward (incr_modules/mask_incr_modules.py:36-42): f = k*floor(0.5 + T/k),
    # carry = T - f.  Every op is IEEE fp32, so delta, carry and emitted mask must equal the oracle's
    kval = 0.173
    k = torch.tensor([kval], dtype=torch.float32, device=DEV) if k_on_device else kval
    carry_cpu = io.Reserve(torch.zeros(n, c, h, w))
    carry_gpu = ops.new_nhwc(n, c, h, w, DEV)
    ts = TileMask(n, h, w, DEV)
    out = ops.new_nhwc(n, c, h, w, DEV)
    refined = torch.zeros((n, 1, h, w), dtype=torch.uint8, device=DEV)
    total = torch.zeros(n, c, h, w)
    for step in range(6):
        d, m = gaussian_delta(n, c, h, w, 0.15, 0.1, seed=300 + step + c)
        _identity_ts(ts, m, n, h, w)
        ops.kfence_incr(_dev(d), carry_gpu, k, out, ts, refined)
        torch.cuda.synchronize()
        ref = io.kfenced(carry_cpu, torch.tensor(kval), d)
        total += d
        assert torch.equal(out.cpu(), ref), "quantised delta differs at step %d" % step
        assert torch.equal(carry_gpu.cpu(), carry_cpu.reservoir), "carry differs at step %d" % step
        assert np.array_equal(refined.cpu().numpy(), (ref != 0).any(dim=1, keepdim=True).to(torch.uint8).numpy())
        # what went through is a multiple of k, and nothing is lost: sum(f) + carry = sum(d)
        q = out.cpu() / kval
        assert torch.allclose(q, q.round(), atol=1e-4)
    assert carry_gpu.abs().max().item() <= 0.5 * kval * (1 + 1e-6)


def test_kfence_in_place_and_switched_off():
    n, c, h, w = 1, 8, 16, 24
    d, m = gaussian_delta(n, c, h, w, 0.3, 1.0, seed=5)
    ts = _identity_ts(TileMask(n, h, w, DEV), m, n, h, w)
    carry = ops.new_nhwc(n, c, h, w, DEV)
    x = _dev(d.clone())
    ops.kfence_incr(x, carry, 0.5, x, ts)                       # out aliases in
    ref = io.kfenced(io.Reserve(torch.zeros(n, c, h, w)), torch.tensor(0.5), d)
    assert torch.equal(x.cpu(), ref)
    # a k that is not positive (device scalar): the delta passes, the carry empties
    kz = torch.zeros(1, device=DEV)
    out = ops.new_nhwc(n, c, h, w, DEV)
    carry2 = ops.new_nhwc(n, c, h, w, DEV)
    ops.kfence_incr(_dev(d), carry2, kz, out, ts)
    assert torch.equal(out.cpu(), d) and torch.count_nonzero(carry2) == 0
    with pytest.raises(RuntimeError, match="positive and finite"):
        ops.kfence_incr(_dev(d), carry2, 0.0, out, ts)
    with pytest.raises(RuntimeError, match="alias"):
        ops.kfence_incr(x, x, 0.5, out, ts)


@pytest.mark.parametrize("k,s,p", [(2, 2, 0), (3, 2, 1), (3, 1, 1)])
@pytest.mark.parametrize("n,c,h,w", [(1, 16, 37, 45), (2, 3, 16, 24)])
def test_maxpool_increment_and_masked_accumulate(k, s, p, n, c, h, w):
    # nnMaxPool2dIncr.forward (incr_modules/mask_incr_modules.py:217-219): pool(R + d) - pool(R), R += d.
    # max and one subtraction of identical fp32 operands: bit-exact against torch's max_pool2d
    from maskedincrementeval_amd import mask_incr_modules as mm
    pool = mm.nnMaxPool2dIncr(k, s, p)
    r0 = _randn(n, c, h, w, seed=k + c)
    res_cpu = io.Reserve(r0.clone())
    with torch.no_grad():
        y0 = pool.forward_refresh_reservoirs(_dev(r0.clone()))
    assert torch.equal(y0.cpu(), torch.nn.functional.max_pool2d(r0, k, s, p))
    for step in range(3):
        d, m = gaussian_delta(n, c, h, w, 0.1, 0.8, seed=500 + step + h)
        x = _dev(d)
        x[~m.to(DEV).bool().expand_as(x)] = float("nan")          # inactive pixels are never read
        out, ts = pool([x, m.to(DEV) if step < 2 else m.expand(n, c, h, w).to(DEV)])
        torch.cuda.synchronize()
        want = io.maxpool_incr(res_cpu, d, k, s, p)
        assert torch.equal(out.cpu(), want), "step %d" % step
        assert torch.equal(pool.mp_res.reservoir.cpu(), res_cpu.reservoir)
        assert np.array_equal(ts.pixmask[:, 0].cpu().numpy(), mo.footprint_conv(m[:, 0].numpy(), k, s, p))
    # dense delta (mask None)
    d = _randn(n, c, h, w, seed=77) * 0.3
    out, _ = pool([_dev(d), None])
    assert torch.equal(out.cpu(), io.maxpool_incr(res_cpu, d, k, s, p))
    assert torch.equal(pool.mp_res.reservoir.cpu(), res_cpu.reservoir)


@pytest.mark.parametrize("argv", [["--op", "act"], ["--op", "mul"], ["--op", "add"], ["--op", "up2x"], ["--op", "gates"],
                                  ["--cin", "32", "--cout", "32", "--k", "3"],
                                  ["--cin", "64", "--cout", "32", "--k", "5", "--up2x"], ["--copy-mb", "1"]])
@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_kernel_bench_modes_run_and_report(argv, dtype, monkeypatch, capsys):
    # the single-kernel benchmark the rocprofv3 counter runs use: every mode launches and prints one JSON line
    # with a positive duration and the algorithmic bytes of its op
    import json
    from maskedincrementeval_amd import kernel_bench
    small = ["--h", "24", "--w", "40", "--n", "2", "--iters", "2", "--warmup", "1", "--density", "0.3", "--dtype", dtype]
    if "--cin" not in argv:
        small += ["--cin", "16"]
    monkeypatch.setattr("sys.argv", ["kernel_bench"] + argv + small)
    kernel_bench.main()
    line = json.loads(capsys.readouterr().out.strip().splitlines()[-1])
    assert line["us"] > 0
    assert line.get("algorithmic_bytes", line.get("bytes_read", 0)) > 0


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("c,h,w", [(64, 13, 17), (8, 16, 16), (6, 9, 30)])
def test_upsample_pair_equals_two_single_launches(c, h, w, dtype):
    # two up-samplings of the same geometry in one launch: bit-identical to the two separate calls, over
    # three steps with fresh masks (stale tiles), inactive inputs poisoned
    from maskedincrementeval_amd.masked_types import TileMask
    n = 2
    ts = [TileMask(n, 2 * h, 2 * w, DEV) for _ in range(4)]
    outs = [ops.new_nhwc(n, c, 2 * h, 2 * w, DEV, dtype) for _ in range(4)]
    for step in range(3):
        ins = []
        for j in range(2):
            d, m = gaussian_delta(n, c, h, w, (0.3, 0.05, 0.6)[step] * (1 + j) / 2, 0.5, seed=880 + 10 * step + j)
            x = _dev(torch.where(m.bool().expand_as(d), d, torch.full_like(d, float("nan")))).to(dtype)
            ins.append((x, m.to(DEV)))
        for j in range(2):
            for t in (ts[j], ts[2 + j]):
                ops.build_mask_tiles(ins[j][1], None, n, h, w, _lib.FOOT_UP2X, 0, 0, 0, t)
            ops.upsample2x_incr(ins[j][0], ins[j][1], None, None, ts[j], outs[j])
        ops.upsample2x_pair_incr(ins[0][0], ins[0][1], ts[2], outs[2], ins[1][0], ins[1][1], ts[3], outs[3])
        torch.cuda.synchronize()
        for j in range(2):
            assert torch.isfinite(outs[2 + j].float()).all()
            assert torch.equal(outs[j], outs[2 + j]), "step %d input %d" % (step, j)
