"""GPU parity of the drop-in module surface (mask_incr_modules / mask_incr_functional)
and of E2Depth-incr against the CPU oracle.  The first two tests mirror the
reference's own tests/test_pointops.py."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

from maskedincrementeval_amd import _lib, ops
from maskedincrementeval_amd import mask_incr_functional as mf
from maskedincrementeval_amd import mask_incr_modules as mm
from maskedincrementeval_amd.e2depth_incr import ConvLSTMIncr, E2VIDRecurrentIncr
from maskedincrementeval_amd.masked_types import TileMask
from maskedincrementeval_amd.synthetic import (event_voxel_delta, gaussian_delta, he_normal_conv_weight,
                                               seed_module_)
from oracle import incr_oracle as io
from oracle import mask_oracle as mo
from oracle.e2depth_oracle import E2DepthOracle
import mask_chain

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
RTOL, ATOL = 1e-4, 1e-5


def _cl(t):
    return t.to(DEV).contiguous(memory_format=torch.channels_last)


def _close(got, ref, what="", rtol=RTOL, atol=ATOL):
    got = got.detach().cpu()
    err = (got - ref).abs().max().item()
    assert torch.allclose(got, ref, rtol=rtol, atol=atol), "%s max|diff| = %.3e" % (what, err)


def test_accumulate_incr_like_reference():
    # tests/test_pointops.py:11-22, as a 4-D tensor (1, 1, 40, 80)
    shape = (1, 1, 40, 80)
    X = torch.randn(shape, generator=torch.Generator().manual_seed(0))
    incr = torch.randn(shape, generator=torch.Generator().manual_seed(1))
    zz = torch.relu(X + incr) - torch.relu(X)
    act = mm.nnReluIncr()
    act.forward_refresh_reservoirs(_cl(X))
    out = act([_cl(incr), None])
    torch.cuda.synchronize()
    assert torch.count_nonzero(out[0].cpu() - zz) == 0, "output check"
    assert torch.count_nonzero(X + incr - act.in_res.reservoir.cpu()) == 0, "incremented_input"
    assert isinstance(out[1], TileMask)


def test_convkxkincr_functional_like_reference():
    # tests/test_pointops.py:25-35: nnConvIncr(3,5,3,1,1,bias=False), 1x3x25x25, all-ones mask
    c = mm.nnConvIncr(3, 5, 3, 1, 1, bias=False).to(device=DEV).eval()
    x = _cl(torch.randn([1, 3, 25, 25], generator=torch.Generator().manual_seed(2)))
    with torch.no_grad():
        out_base = c.forward_refresh_reservoirs(x.contiguous())
        out = c((x, torch.ones_like(x, dtype=bool)))
    torch.cuda.synchronize()
    # the reference asserts bit equality against cuDNN; two different summation orders can only
    # be held to fp32 round-off
    _close(out[0], out_base.cpu(), "output check", rtol=1e-5, atol=1e-6)
    _close(out[0], io.conv_incr(x.cpu(), c.weight.detach().cpu(), 1, 1), "vs oracle", rtol=1e-5, atol=1e-6)


def test_kfenced_conv_restores_sparsity_and_matches_oracle():
    # nnConvIncr with its quantiser switched on (the reference's commented-out `x_incr = self.kf(x_incr)`,
    # incr_modules/mask_incr_modules.py:166): k = tp*||x0|| from the refresh (:45), conv of the
    # quantised delta, carry kept across steps
    n, cin, cout, h, w = 1, 16, 32, 40, 56
    conv = mm.nnConvIncr(cin, cout, 3, 1, 1).to(DEV).eval()
    conv.use_kf, conv.kf.tp = True, 2e-3
    x0 = torch.randn(n, cin, h, w, generator=torch.Generator().manual_seed(11))
    with torch.no_grad():
        conv.forward_refresh_reservoirs(_cl(x0))
    k_ref = (conv.kf.tp * torch.norm(x0)).float()
    assert torch.allclose(conv.kf.k.cpu(), k_ref.reshape(1), rtol=1e-6)
    k_cpu = conv.kf.k.cpu()[0]                       # the value the kernel reads
    k_ptr = conv.kf.k.data_ptr()
    carry = io.Reserve(torch.zeros(n, cin, h, w))
    wt = conv.weight.detach().cpu()
    for step in range(5):
        d, m = gaussian_delta(n, cin, h, w, 0.2, 0.08, seed=40 + step)
        with torch.no_grad():
            out = conv([_cl(d), m.to(DEV)])
        torch.cuda.synchronize()
        f = io.kfenced(carry, k_cpu, d)
        assert torch.equal(conv.kf.delta.reservoir.cpu(), carry.reservoir)
        fmask = (f != 0).any(dim=1).to(torch.uint8).numpy()
        assert 0 < fmask.sum() < m.sum().item()         # the fence removed pixels, not all of them
        assert np.array_equal(out[1].pixmask[:, 0].cpu().numpy(), mo.footprint_conv(fmask, 3, 1, 1))
        assert np.array_equal(out[1].active_tiles().cpu().numpy(), mo.tile_list(mo.footprint_conv(fmask, 3, 1, 1)))
        _close(out[0], io.conv_incr(f, wt, 1, 1), "conv of the quantised delta, step %d" % step)
    with torch.no_grad():
        conv.forward_refresh_reservoirs(_cl(2 * x0))        # k follows the refresh in place
    assert conv.kf.k.data_ptr() == k_ptr and torch.allclose(conv.kf.k.cpu(), 2 * k_ref.reshape(1), rtol=1e-6)
    assert torch.count_nonzero(conv.kf.delta.reservoir) == 0


def test_functional_ops_match_oracle():
    n, c, h, w = 1, 16, 30, 38
    d, m = gaussian_delta(n, c, h, w, 0.1, 0.5, seed=3)
    wt = he_normal_conv_weight(32, c, 3, seed=4)
    filt = wt.permute(1, 2, 3, 0).contiguous().to(DEV)
    out = mf.conv2d_from_module([_cl(d), _cl(m.float()).to(torch.uint8)], filt, stride=(2, 2), padding=(1, 1))
    _close(out[0], io.conv_incr(d, wt, 2, 1), "conv2d_from_module")
    assert np.array_equal(out[1].pixmask[:, 0].cpu().numpy(), mo.footprint_conv(m[:, 0].numpy(), 3, 2, 1))
    up = mf.interpolate_from_module([_cl(d), m.to(DEV)])
    _close(up[0], io.interp_incr(d), "interpolate_from_module")
    tc = torch.nn.ConvTranspose2d(c, 8, 3, stride=2, padding=1, output_padding=1).to(DEV)
    tout = mf.transposed_conv2d_from_module([_cl(d), m.to(DEV)], tc)
    _close(tout[0], io.tconv_incr(d, tc.weight.detach().cpu(), 2, 1, 1), "transposed_conv2d_from_module")
    bn = torch.nn.BatchNorm2d(c).to(DEV).eval()
    bn.running_var.uniform_(0.5, 2.0)
    bn.weight.data.normal_()
    bout = mf.bn2d_from_module([_cl(d), None], bn)
    _close(bout[0], io.bn_incr(d, bn.running_var.cpu(), bn.weight.detach().cpu(), bn.eps), "bn2d_from_module")
    r1, r2 = mf.IncrementReserve(_cl(torch.randn(n, c, h, w))), mf.IncrementReserve(_cl(torch.randn(n, c, h, w)))
    d2, m2 = gaussian_delta(n, c, h, w, 0.05, 0.5, seed=5)
    keep = r1.reservoir.clone()
    pm = mf.IncrPointwiseMultiply([_cl(d), m.to(DEV)], r1, [_cl(d2), m2.to(DEV)], r2)
    ref = (d2 + r2.reservoir.cpu()) * d + r1.reservoir.cpu() * d2
    _close(pm[0], ref, "IncrPointwiseMultiply")
    assert torch.equal(keep, r1.reservoir)


@pytest.mark.parametrize("density", [0.01, 0.05, 0.20])
def test_config2_activation_chain_50_steps(density):
    """Benchmark configuration 2: 1x64x132x176, conv3x3 64->64 -> incremental LeakyReLU(0.01)
    -> incremental ReLU, 50 steps with a fresh mask each step: emitted masks exact (staged on
    the GPU reservoirs), drift against a dense recompute at steps 1 and 50."""
    n, c, h, w = 1, 64, 132, 176
    conv = mm.nnConvIncr(c, c, 3, 1, 1).to(DEV).eval()
    seed_module_(conv, 11)
    leaky = mm.nnReservedActivation(mm.leaky_relu_op(0.01))
    relu = mm.nnReservedActivation(torch.relu)
    x = torch.randn(n, c, h, w, generator=torch.Generator().manual_seed(12))
    wt, b = conv.weight.detach().cpu(), conv.bias.detach().cpu()
    with torch.no_grad():
        y = relu.forward_refresh_reservoirs(leaky.forward_refresh_reservoirs(conv.forward_refresh_reservoirs(_cl(x))))
    acc = y.clone()
    o_leaky, o_relu = io.Reserve(io.conv_refresh(x, wt, b, 1, 1)), io.Reserve(None)
    o_relu.update_reservoir(io.leaky_relu(o_leaky.reservoir))
    acc_ref = torch.relu(o_relu.reservoir)
    _close(acc, acc_ref, "refresh")
    for step in range(50):
        d, m = gaussian_delta(n, c, h, w, density, 0.2, seed=2000 + step)
        r_leaky_old = leaky.in_res.reservoir.clone()
        r_relu_old = relu.in_res.reservoir.clone()
        with torch.no_grad():
            a = conv([_cl(d), m.to(DEV)])
            bq = leaky(a)
            out = relu(bq)
        torch.cuda.synchronize()
        ref = io.act_incr(torch.relu, o_relu, io.act_incr(io.leaky_relu, o_leaky, io.conv_incr(d, wt, 1, 1)))
        x = x + d
        acc += out[0]
        acc_ref += ref
        if step in (0, 49):
            _close(out[0], ref, "step %d delta" % step)
            dense = torch.relu(io.leaky_relu(io.conv_refresh(x, wt, b, 1, 1)))
            _close(acc, dense, "step %d accumulated vs dense recompute" % step)
            _close(leaky.in_res.reservoir, o_leaky.reservoir, "step %d reservoir" % step)
        # structural mask of the conv: exact
        assert np.array_equal(a[1].pixmask[:, 0].cpu().numpy(), mo.footprint_conv(m[:, 0].numpy(), 3, 1, 1))
        assert np.array_equal(a[1].active_tiles().cpu().numpy(), mo.tile_list(a[1].pixmask[:, 0].cpu().numpy()))
        # emitted masks, staged on the GPU-produced reservoir pairs: exact
        lk = lambda t: F.leaky_relu(t, 0.01)
        want1 = ((lk(leaky.in_res.reservoir) - lk(r_leaky_old)) != 0).any(1, keepdim=True) & a[1].pixmask.bool()
        assert torch.equal(bq[1].pixmask.bool(), want1)
        want2 = ((torch.relu(relu.in_res.reservoir) - torch.relu(r_relu_old)) != 0).any(1, keepdim=True) & want1
        assert torch.equal(out[1].pixmask.bool(), want2)
    _close(acc, acc_ref, "accumulated after 50 steps")


@pytest.mark.parametrize("fused", [True, False])
@pytest.mark.parametrize("cin,hid", [(16, 16), (32, 32), (64, 32)])
@pytest.mark.parametrize("f32mode", ["bf16x3", "native"])
def test_convlstm_module_matches_oracle(fused, cin, hid, f32mode):
    # (32, 32) and (64, 32) take the conv + gate chain kernel when fused, (16, 16) the two-kernel form
    n, h, w = 1, 26, 34
    cell = ConvLSTMIncr(cin, hid, 3, fused=fused).to(DEV).eval()
    seed_module_(cell, 21)
    ref = io.ConvLSTMOracle(cell.Gates.weight.detach().cpu(), cell.Gates.bias.detach().cpu(), hid)
    x0 = torch.randn(n, cin, h, w, generator=torch.Generator().manual_seed(22))
    with torch.no_grad():
        h_d, c_d = cell.forward_refresh_reservoirs(_cl(x0), None)
    h_r, c_r = ref.refresh(x0)
    _close(h_d, h_r, "refresh h"), _close(c_d, c_r, "refresh c")
    assert cell.__dict__.get("_gates_interleaved", False) == (fused and cin % 32 == 0)
    for step in range(4):
        d, m = gaussian_delta(n, cin, h, w, 0.08, 0.3, seed=2300 + step)
        with torch.no_grad():
            dh, dc = cell([_cl(d), m.to(DEV)], None)
        torch.cuda.synchronize()
        dh_r, dc_r = ref.incr(d)
        _close(dh[0], dh_r, "dh %d" % step), _close(dc[0], dc_r, "dc %d" % step)


def _run_e2depth(h, w, steps, density, fuse, seed=31):
    model = seed_module_(E2VIDRecurrentIncr(fuse=fuse), seed=seed).to(DEV).eval()
    oracle = E2DepthOracle(model.state_dict())
    x0 = torch.randn(1, 5, h, w, generator=torch.Generator().manual_seed(seed + 1)) * 0.5
    with torch.no_grad():
        acc = model.forward_refresh_reservoirs(_cl(x0), None)[0].clone()
    acc_ref = oracle.refresh(x0)
    _close(acc, acc_ref, "refresh")
    x = x0.clone()
    prev_lists, sets_checked = {}, 0
    for step in range(steps):
        d, m = event_voxel_delta(1, 5, h, w, density, seed=3000 + step)
        with torch.no_grad(), mask_chain.BuildRecorder() as rec:
            out, states = model([_cl(d), None], None)      # the reference drivers pass mask None
        torch.cuda.synchronize()
        ref = oracle.incr(d)
        _close(out[0], ref, "step %d" % step)
        acc += out[0]
        acc_ref += ref
        x += d
        # input mask and head tile list: exact against the oracle definitions
        pm = mo.pixel_mask(d.numpy(), 0.0)
        assert np.all(pm <= m[:, 0].numpy())     # (an event pixel whose five bins all drew 0 carries no delta)
        head_ts = model.unetrecurrent.head.conv2d._tile_set("out_act" if fuse else "out", 1, h, w, torch.device(DEV))
        assert np.array_equal(head_ts.active_tiles().cpu().numpy(), mo.tile_list(mo.footprint_conv(pm, 5, 1, 2)))
        if fuse:
            # every tile set of the step, in situ: pixel mask, ascending tile list and stale list of each build against
            # the chained footprints of the input pixel mask, and the named layers against the chain written down
            # from the network definition (structural masks only: the un-fused chain refines masks from values)
            seeds = {model._pix_buf("input", 1, h, w, torch.device(DEV)).data_ptr(): pm}
            sets_checked += mask_chain.check_recorded_builds(rec.calls, seeds, prev_lists, "step %d" % step)
            sets_checked += mask_chain.check_e2depth_layers(model, pm, "step %d" % step)
    assert not fuse or sets_checked >= 30 * steps
    _close(acc, acc_ref, "accumulated")
    return model, acc, x


class _AtenLog(torch.utils._python_dispatch.TorchDispatchMode):
    """Names of the ATen ops dispatched inside the block (views included)."""

    def __init__(self):
        super().__init__()
        self.ops = []

    def __torch_dispatch__(self, func, types, args=(), kwargs=None):
        self.ops.append(str(func))
        return func(*args, **(kwargs or {}))


# ATen ops that launch nothing: views and metadata
_VIEW_OPS = ("aten.detach", "aten.permute", "aten.view", "aten._unsafe_view", "aten.reshape", "aten.alias",
             "aten.as_strided", "aten.slice", "aten.select", "aten.expand", "aten.t.", "aten.transpose",
             "aten.unsqueeze", "aten.squeeze", "aten.chunk", "aten.split", "aten.narrow", "aten.sym_",
             "aten.is_", "aten._to_copy.default_noop")


def _kernel_ops(log):
    return [o for o in log.ops if not any(o.startswith(v) for v in _VIEW_OPS)]


def test_e2depth_refresh_runs_on_the_library_kernels_and_replays_as_a_graph():
    # The dense refresh (incr_modules/e2depth_incr.py:442-468): convs, bilinear x2, ConvLSTM state math and the
    # skip sums all go through libmie_hip; once the buffers exist a refresh dispatches no ATen kernel, so it can
    # be captured in a HIP graph.  A refresh in the middle of a stream must leave the incremental state
    # consistent (no buffer is zero-filled: the next step's stale lists clean up).
    h, w = 72, 104
    model = seed_module_(E2VIDRecurrentIncr(), seed=31).to(DEV).eval()
    oracle = E2DepthOracle(model.state_dict())
    g = torch.Generator().manual_seed(33)
    x0, x1 = (torch.randn(1, 5, h, w, generator=g) * 0.5 for _ in range(2))
    static_x = _cl(x0)
    with torch.no_grad():
        model.forward_refresh_reservoirs(static_x, None)            # allocates every buffer
        for step in range(2):
            d, _ = event_voxel_delta(1, 5, h, w, 0.05, seed=3300 + step)
            model([_cl(d), None], None)
        torch.cuda.synchronize()
        with _AtenLog() as log:
            pred = model.forward_refresh_reservoirs(static_x, None)[0]
        assert _kernel_ops(log) == [], "ATen kernels in the refresh: %s" % sorted(set(_kernel_ops(log)))
        _close(pred, oracle.refresh(x0), "eager refresh")
        # captured: replay on another input, then incremental steps on top of it
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            model.forward_refresh_reservoirs(static_x, None)
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            pred_g = model.forward_refresh_reservoirs(static_x, None)[0]
        for x in (x1, x0, x1):
            static_x.copy_(_cl(x))
            graph.replay()
            torch.cuda.synchronize()
            ref = oracle.refresh(x)
            _close(pred_g, ref, "graph replay of the refresh")
        acc, acc_ref = pred_g.clone(), ref.clone()
        for step in range(3):
            d, _ = event_voxel_delta(1, 5, h, w, 0.05, seed=3400 + step)
            out, _ = model([_cl(d), None], None)
            torch.cuda.synchronize()
            ref_d = oracle.incr(d)
            _close(out[0], ref_d, "step %d after the replayed refresh" % step)
            acc += out[0]
            acc_ref += ref_d
        _close(acc, acc_ref, "accumulated after the replayed refresh")


@pytest.mark.parametrize("fuse", [True, False])
@pytest.mark.parametrize("f32mode", ["bf16x3", "native"])
def test_e2depth_incr_small_matches_oracle(fuse, f32mode):
    _run_e2depth(72, 104, steps=4, density=0.05, fuse=fuse)


def test_e2depth_incr_full_size_matches_oracle_and_dense():
    # benchmark configuration 3 at its real size (264x352, 5 %): per-step parity for a few steps,
    # then refresh + sum of increments == dense forward on the last input (tests/test_network.py:24-31)
    model, acc, x = _run_e2depth(264, 352, steps=3, density=0.05, fuse=True)
    fresh = seed_module_(E2VIDRecurrentIncr(), seed=31).to(DEV).eval()
    with torch.no_grad():
        dense = fresh.forward_refresh_reservoirs(_cl(x), None)[0]
    _close(acc, dense.cpu(), "refresh + increments vs dense")


def test_e2depth_incr_50_steps_of_accumulation():
    # 50 successive delta accumulations into the same reservoirs (the reference drivers refresh every 20-100
    # frames, run_e2depth_continuous_dataset.py:61): parity per step and of the accumulated prediction, and
    # refresh + 50 increments == dense forward on x0 + the 50 deltas.  Reduced frame (72x104) so that the CPU
    # oracle takes seconds; at this size the bottleneck planes are 9x13, i.e. the split form of the conv runs too.
    model, acc, x = _run_e2depth(72, 104, steps=50, density=0.05, fuse=True)
    fresh = seed_module_(E2VIDRecurrentIncr(), seed=31).to(DEV).eval()
    with torch.no_grad():
        dense = fresh.forward_refresh_reservoirs(_cl(x), None)[0]
    _close(acc, dense.cpu(), "refresh + 50 increments vs dense")


def test_e2depth_incr_full_size_100_steps_of_accumulation():
    # benchmark configuration 3 at its real size for the 100 steps it names (the reference driver refreshes every
    # 100 frames, run_e2depth_continuous_dataset.py:61): every step against the CPU oracle, every tile set of every
    # step against the mask oracle, the accumulated prediction against the oracle's, and refresh + 100 increments
    # == dense refresh of a fresh network on x0 + the 100 deltas (tests/test_network.py:24-31) -- all at
    # rtol 1e-4 / atol 1e-5
    model, acc, x = _run_e2depth(264, 352, steps=100, density=0.05, fuse=True)
    fresh = seed_module_(E2VIDRecurrentIncr(), seed=31).to(DEV).eval()
    with torch.no_grad():
        dense = fresh.forward_refresh_reservoirs(_cl(x), None)[0]
    _close(acc, dense.cpu(), "refresh + 100 increments vs dense at 264x352")


def test_e2depth_incr_empty_frames_between_active_ones():
    # a frame without any event: every tile list is empty, every output exactly zero, reservoirs
    # untouched; the frame after it clears the stale tiles of the frame before (clean-delta invariant)
    h, w = 72, 104
    model = seed_module_(E2VIDRecurrentIncr(), seed=31).to(DEV).eval()
    oracle = E2DepthOracle(model.state_dict())
    x0 = torch.randn(1, 5, h, w, generator=torch.Generator().manual_seed(32)) * 0.5
    with torch.no_grad():
        model.forward_refresh_reservoirs(_cl(x0), None)
    oracle.refresh(x0)
    zero = torch.zeros(1, 5, h, w)
    frames = [event_voxel_delta(1, 5, h, w, 0.05, seed=1)[0], zero, zero, event_voxel_delta(1, 5, h, w, 0.02, seed=2)[0]]
    for i, d in enumerate(frames):
        with torch.no_grad():
            out, _ = model([_cl(d), None], None)
        torch.cuda.synchronize()
        ref = oracle.incr(d)
        _close(out[0], ref, "frame %d" % i)
        if not d.any():
            assert torch.count_nonzero(out[0]) == 0 and out[1].active_tiles().numel() == 0
            assert torch.count_nonzero(ref) == 0
    # every persistent delta buffer is zero outside the active pixels of its tile set after the last frame
    head = model.unetrecurrent.head.conv2d
    buf = head._delta_buf("out_act", (1, 32, h, w), torch.device(DEV))
    ts = head._tile_set("out_act", 1, h, w, torch.device(DEV))
    assert torch.count_nonzero(buf * (1 - ts.pixmask.float())) == 0


@pytest.mark.parametrize("cin,hid,h,w", [(128, 128, 16, 8), (64, 64, 12, 20), (256, 256, 8, 8)])
@pytest.mark.parametrize("f32mode", ["bf16x3", "native"])
def test_convlstm_on_a_small_plane_splits_the_gates_conv(cin, hid, h, w, f32mode):
    # planes of few tiles: the gates conv runs as a split contraction (partial sums in the workspace) and the gate
    # chain in a second kernel (mie_conv_gates_masked_ws).  Against the oracle, and against a twin cell whose launches
    # are not split; previous-state deltas from the second step on (two-input contraction, previous-cell term).
    n = 1
    cells = [seed_module_(ConvLSTMIncr(cin, hid, 3, fused=True), 81).to(DEV).eval() for _ in range(2)]
    ref = io.ConvLSTMOracle(cells[0].Gates.weight.detach().cpu(), cells[0].Gates.bias.detach().cpu(), hid)
    x0 = torch.randn(n, cin, h, w, generator=torch.Generator().manual_seed(82)) * 0.5
    with torch.no_grad():
        for cell in cells:
            h_d, c_d = cell.forward_refresh_reservoirs(_cl(x0), None)
    h_r, c_r = ref.refresh(x0)
    _close(h_d, h_r, "refresh h"), _close(c_d, c_r, "refresh c")
    ws = ops.split_workspace(torch.device(DEV))
    ws.fill_(float("nan"))
    for step in range(4):
        d, m = gaussian_delta(n, cin, h, w, (0.4, 0.05, 0.7, 0.2)[step], 0.3, seed=8300 + step)
        prev, prev_ref = None, None
        if step >= 1:
            dhp, mh = gaussian_delta(n, hid, h, w, 0.2, 0.2, seed=8400 + step)
            dcp, mc = gaussian_delta(n, hid, h, w, 0.1, 0.2, seed=8500 + step)
            prev = lambda: ([_cl(dhp), mh.to(DEV)], [_cl(dcp), mc.to(DEV)])
            prev_ref = (dhp, dcp)
        outs = []
        for cell, split in zip(cells, (True, False)):
            ops.split_enabled = split
            try:
                with torch.no_grad():
                    outs.append(cell([_cl(d), m.to(DEV)], None if prev is None else prev()))
            finally:
                ops.split_enabled = True
        torch.cuda.synchronize()
        dh_r, dc_r = ref.incr(d, prev_ref) if prev_ref is not None else ref.incr(d)
        for (dh, dc), what in zip(outs, ("split", "one launch")):
            assert torch.isfinite(dh[0]).all() and torch.isfinite(dc[0]).all()
            _close(dh[0], dh_r, "%s dh %d" % (what, step)), _close(dc[0], dc_r, "%s dc %d" % (what, step))
    plane = n * h * w * 4 * hid
    assert torch.isfinite(ws[:plane]).any() and torch.isfinite(ws[plane:2 * plane]).any()      # the split form ran


@pytest.mark.parametrize("cin,hid", [(16, 16), (32, 32)])
def test_convlstm_with_previous_state_deltas(cin, hid):
    # non-zero refresh state and non-zero deltas of the previous hidden / cell state (the module
    # signature allows them, incr_modules/e2depth_incr.py:79,98): two-pointer conv input + m2 term
    n, h, w = 1, 24, 32
    cell = seed_module_(ConvLSTMIncr(cin, hid, 3, fused=True), 61).to(DEV).eval()
    ref = io.ConvLSTMOracle(cell.Gates.weight.detach().cpu(), cell.Gates.bias.detach().cpu(), hid)
    g = torch.Generator().manual_seed(62)
    x0, h0, c0 = (torch.randn(n, c, h, w, generator=g) * 0.5 for c in (cin, hid, hid))
    with torch.no_grad():
        h_d, c_d = cell.forward_refresh_reservoirs(_cl(x0), (_cl(h0), _cl(c0)))
    h_r, c_r = ref.refresh(x0, (h0, c0))
    _close(h_d, h_r, "refresh h"), _close(c_d, c_r, "refresh c")
    for step in range(4):
        d, m = gaussian_delta(n, cin, h, w, 0.08, 0.3, seed=6300 + step)
        dhp, mh = gaussian_delta(n, hid, h, w, 0.05, 0.2, seed=6400 + step)
        if step < 2:
            # hidden and cell deltas under ONE mask (one device tensor, or two equal copies: the cell then
            # builds their union): the masked previous-hidden path, pix2 + union tile set
            dcp, _ = gaussian_delta(n, hid, h, w, 0.05, 0.2, seed=6400 + step)
            mh_dev = mh.to(DEV)
            mc_dev = mh_dev if step == 0 else mh.to(DEV)
            mc = mh
        else:
            # different masks for the two: the tile set must cover the union, each delta is read under its own
            dcp, mc = gaussian_delta(n, hid, h, w, 0.04, 0.2, seed=6500 + step)
            mh_dev, mc_dev = mh.to(DEV), mc.to(DEV)
        # inactive pixels of the previous-state deltas are never read
        nan = float("nan")
        dhp_dev = _cl(torch.where(mh.bool().expand_as(dhp), dhp, torch.full_like(dhp, nan)))
        dcp_dev = _cl(torch.where(mc.bool().expand_as(dcp), dcp, torch.full_like(dcp, nan)))
        if step == 3:      # tile masks in the mask slots
            tmh, tmc = TileMask(n, h, w, DEV), TileMask(n, h, w, DEV)
            ops.build_mask_tiles(mh_dev, None, n, h, w, _lib.FOOT_CONV, 1, 1, 0, tmh)
            ops.build_mask_tiles(mc_dev, None, n, h, w, _lib.FOOT_CONV, 1, 1, 0, tmc)
            mh_dev, mc_dev = tmh, tmc
        with torch.no_grad():
            dh, dc = cell([_cl(d), m.to(DEV)], ([dhp_dev, mh_dev], [dcp_dev, mc_dev]))
        torch.cuda.synchronize()
        dh_r, dc_r = ref.incr(d, (dhp, dcp))
        assert torch.isfinite(dh[0]).all() and torch.isfinite(dc[0]).all()
        _close(dh[0], dh_r, "dh %d" % step), _close(dc[0], dc_r, "dc %d" % step)
        if step >= 2:      # the tile set is sparse (not "every tile") and covers the cell delta's pixels
            assert int(dh[1].counts[0].item()) < dh[1].capacity
            assert torch.all(dh[1].pixmask.cpu() >= mc)


@pytest.mark.parametrize("cin,hid", [(16, 16), (32, 32)])
def test_convlstm_state_deltas_fed_back(cin, hid):
    # the returned [dh, ts], [dc, ts] go straight back in as the next step's previous state
    # (forward(x, prev_states) of the reference, incr_modules/e2depth_incr.py:79,98): the cell must not
    # write the buffers and the tile set it is reading
    n, h, w = 1, 40, 48
    cell = seed_module_(ConvLSTMIncr(cin, hid, 3, fused=True), 71).to(DEV).eval()
    ref = io.ConvLSTMOracle(cell.Gates.weight.detach().cpu(), cell.Gates.bias.detach().cpu(), hid)
    g = torch.Generator().manual_seed(72)
    x0 = torch.randn(n, cin, h, w, generator=g) * 0.5
    with torch.no_grad():
        cell.forward_refresh_reservoirs(_cl(x0), None)
    ref.refresh(x0, None)
    state, state_r = None, None
    for step in range(6):
        d, m = gaussian_delta(n, cin, h, w, 0.04, 0.3, seed=7300 + step)
        with torch.no_grad():
            state = cell([_cl(d), m.to(DEV)], state)
        torch.cuda.synchronize()
        state_r = ref.incr(d, state_r)
        _close(state[0][0], state_r[0], "dh %d" % step), _close(state[1][0], state_r[1], "dc %d" % step)
        # clean delta: zero outside the active pixels of the tile set it is returned with
        for dlt, ts in state:
            assert torch.count_nonzero(dlt * (1 - ts.pixmask.float())) == 0
        if step > 0:
            assert state[0][0].data_ptr() != prev_ptr      # the two state sets alternate
        prev_ptr = state[0][0].data_ptr()


@pytest.mark.parametrize("plan_first", [False, True])
@pytest.mark.parametrize("graph", [False, True])
def test_async_mask_planning_gives_the_same_frames_as_inline_planning(graph, plan_first):
    # Tile sets built on the planning stream (eagerly and as edges of a replayed HIP graph) must be the
    # ones inline planning builds: the same kernels then run over the same tiles, so the predictions
    # agree bit for bit.  Every step has a fresh mask, so a build that read a mask of the previous
    # step (or raced with the kernel that writes it) shows up as a difference.
    h, w, steps = 72, 104, 8
    a = seed_module_(E2VIDRecurrentIncr(async_masks=True, plan_first=plan_first), seed=31).to(DEV).eval()
    s = seed_module_(E2VIDRecurrentIncr(async_masks=False), seed=31).to(DEV).eval()
    x0 = torch.randn(1, 5, h, w, generator=torch.Generator().manual_seed(32)) * 0.5
    deltas = [_cl(event_voxel_delta(1, 5, h, w, 0.03 + 0.02 * (i % 3), seed=4100 + i)[0]) for i in range(steps)]
    static_in = _cl(torch.zeros(1, 5, h, w))
    with torch.no_grad():
        a.forward_refresh_reservoirs(_cl(x0), None)
        s.forward_refresh_reservoirs(_cl(x0), None)
        refs = [s([d, None], None)[0][0].clone() for d in deltas]
        got = []
        g, g_out = None, None
        for i, d in enumerate(deltas):
            static_in.copy_(d)
            if graph and i == 2:       # two eager steps first: they allocate every persistent buffer
                torch.cuda.synchronize()
                g = torch.cuda.CUDAGraph()
                with torch.cuda.graph(g):
                    g_out = a([static_in, None], None)[0][0]
            if g is not None:
                g.replay()
                got.append(g_out.clone())
            else:
                got.append(a([static_in, None], None)[0][0].clone())
        torch.cuda.synchronize()
    for i in range(steps):
        assert torch.equal(got[i], refs[i]), "step %d max|diff| = %.3e" % (i, (got[i] - refs[i]).abs().max().item())


def test_planning_pass_refuses_masks_that_depend_on_values():
    # a delta quantiser emits a refined mask from the values it lets through: nothing downstream of it
    # can be planned before the compute pass has run
    h, w = 40, 56
    m = seed_module_(E2VIDRecurrentIncr(async_masks=True, plan_first=True), seed=33).to(DEV).eval()
    mm.set_kfence(m, 1e-3)
    x0 = torch.randn(1, 5, h, w, generator=torch.Generator().manual_seed(34))
    with torch.no_grad():
        m.forward_refresh_reservoirs(_cl(x0), None)
        with pytest.raises(RuntimeError, match="cannot be planned ahead"):
            m([_cl(event_voxel_delta(1, 5, h, w, 0.05, seed=35)[0]), None], None)
    assert ops._phase is None and ops._planner is None      # both context managers unwound


@pytest.mark.parametrize("knob", ["threshold", "kfence"])
def test_value_dependent_masks_replay_from_a_graph(knob):
    # A network whose masks depend on the values (threshold masks in front of every conv, incr_modules/utils.py:22-25; the
    # delta quantiser, incr_modules/mask_incr_modules.py:21-47) cannot be planned ahead, but it can be captured: every
    # mask build is a launch on the compute stream and no launch reads device data on the host.  Eight steps with fresh
    # inputs replayed from ONE captured graph must reproduce the eager network bit for bit (predictions and, for the
    # thresholded network, the number of tiles every step left active in the last decoder), with the program's own
    # work between the replays.
    h, w, steps = 72, 104, 8
    nets = []
    for _ in range(2):
        m = seed_module_(E2VIDRecurrentIncr(), seed=31).to(DEV).eval()
        if knob == "threshold":
            mm.set_input_threshold(m, 3e-3)
        else:
            mm.set_kfence(m, 0.05, norm="rms")
        nets.append(m)
    eager, captured = nets
    x0 = torch.randn(1, 5, h, w, generator=torch.Generator().manual_seed(32)) * 0.5
    deltas = [_cl(event_voxel_delta(1, 5, h, w, 0.03 + 0.02 * (i % 3), seed=4300 + i)[0]) for i in range(steps)]
    static_in = _cl(torch.zeros(1, 5, h, w))
    last = lambda m: m.unetrecurrent.decoders[2].conv2d
    with torch.no_grad():
        eager.forward_refresh_reservoirs(_cl(x0), None)
        captured.forward_refresh_reservoirs(_cl(x0), None)
        refs, ref_tiles = [], []
        for d in deltas:
            refs.append(eager([d, None], None)[0][0].clone())
            ref_tiles.append([int(b.counts[0].item()) for k_, b in last(eager)._ib().items() if k_[0] == "t"])
        got, got_tiles = [], []
        g = g_out = None
        for i, d in enumerate(deltas):
            static_in.copy_(d)
            if i == 2:                # two eager steps first: they allocate every persistent buffer
                torch.cuda.synchronize()
                g = torch.cuda.CUDAGraph()
                with torch.cuda.graph(g):
                    g_out = captured([static_in, None], None)[0][0]
            if g is not None:
                g.replay()
                got.append(g_out.clone())
            else:
                got.append(captured([static_in, None], None)[0][0].clone())
            got_tiles.append([int(b.counts[0].item()) for k_, b in last(captured)._ib().items() if k_[0] == "t"])
    torch.cuda.synchronize()
    for i in range(steps):
        assert torch.equal(got[i], refs[i]), "step %d max|diff| = %.3e" % (i, (got[i] - refs[i]).abs().max().item())
        assert got_tiles[i] == ref_tiles[i], "step %d: active tiles %s vs %s" % (i, got_tiles[i], ref_tiles[i])
    if knob == "threshold":
        # the masks did depend on the values: the thresholded network runs fewer tiles than the plane holds
        cap = max(b.capacity for k_, b in last(captured)._ib().items() if k_[0] == "t")
        assert min(max(t) for t in got_tiles) < cap


def test_thresholded_network_with_one_launch_builds_equals_the_separate_launches():
    # Threshold masks in front of every conv: with ops.fused_threshold_build the threshold test, the footprint and the
    # tile lists of a conv go out as one launch (mie_build_mask_tiles_thresholded) instead of mie_mask_from_delta +
    # mie_build_mask_tiles.  Same predictions bit for bit over six steps, same thresholded input masks and tile lists
    # in every conv (the gates convs take a second mask, the decoders read up-sampled deltas, the head has 5 channels).
    h, w, steps = 72, 104, 6
    nets = []
    for _ in range(2):
        m = seed_module_(E2VIDRecurrentIncr(), seed=31).to(DEV).eval()
        mm.set_input_threshold(m, 3e-3)
        nets.append(m)
    fused, plain = nets
    x0 = torch.randn(1, 5, h, w, generator=torch.Generator().manual_seed(32)) * 0.5
    deltas = [_cl(event_voxel_delta(1, 5, h, w, 0.03 + 0.02 * (i % 3), seed=4400 + i)[0]) for i in range(steps)]
    keep = ops.fused_threshold_build
    try:
        with torch.no_grad():
            for m in nets:
                m.forward_refresh_reservoirs(_cl(x0), None)
            for i, d in enumerate(deltas):
                ops.fused_threshold_build = True
                a = fused([d, None], None)[0][0].clone()
                assert not ops._pending_thr, "a thresholded mask was never launched"
                ops.fused_threshold_build = False
                b = plain([d, None], None)[0][0].clone()
                assert torch.equal(a, b), "step %d max|diff| = %.3e" % (i, (a - b).abs().max().item())
                checked = 0
                for (na, ma), (nb_, mb) in zip(fused.named_modules(), plain.named_modules()):
                    if not isinstance(ma, mm.nnConvIncr):
                        continue
                    for key, ba in ma._ib().items():
                        bb = mb._ib()[key]
                        if key[0] == "p":                                   # pixel-mask buffers (thresholded inputs)
                            assert torch.equal(ba, bb), "step %d %s %s" % (i, na, key)
                            checked += 1
                        elif key[0] == "t":                                 # tile sets
                            assert torch.equal(ba.counts[:2], bb.counts[:2]), "step %d %s %s counts" % (i, na, key)
                            n_act = int(ba.counts[0].item())
                            assert torch.equal(ba.tiles[:n_act], bb.tiles[:n_act]) and torch.equal(ba.pixmask, bb.pixmask)
                            checked += 1
                assert checked >= 20
    finally:
        ops.fused_threshold_build = keep
    torch.cuda.synchronize()


@pytest.mark.parametrize("net", ["e2depth", "evflownet_transposed", "evflownet_upsample"])
def test_planning_one_step_ahead_reproduces_plain_steps(net):
    # forward_pipelined: the tile sets of step t + 1 are planned on a second stream while step t computes, in a second
    # generation of every tile set / delta buffer (ops.pipelined_step).  Against the same network stepped plainly, bit
    # for bit: 7 eager steps with fresh masks (stale tiles in both generations), a dense refresh with a plan still
    # pending (buffers are zeroed), then four resident inputs captured as four graphs -- each holds its step and the
    # plan of the next input -- and replayed cyclically three times over, with the program's own work in between.
    from maskedincrementeval_amd.evflownet_incr import MultiResUNetRecurrentIncr
    from maskedincrementeval_amd.synthetic import MovingEdges
    if net == "e2depth":
        h, w, c = 72, 104, 5
        make = lambda: seed_module_(E2VIDRecurrentIncr(), seed=31).to(DEV).eval()
        plain = lambda m, d: m([d, None], None)[0][0]
        piped = lambda m, d, nx, p: m.forward_pipelined([d, None], None if nx is None else [nx, None], p)[0][0]
        refresh = lambda m, x: m.forward_refresh_reservoirs(x, None)
        deltas = [_cl(event_voxel_delta(1, c, h, w, 0.02 + 0.03 * (i % 3), seed=5300 + i)[0]) for i in range(12)]
    else:
        h, w, c = 64, 96, 4
        kind = net.split("_")[1]
        make = lambda: seed_module_(MultiResUNetRecurrentIncr(num_bins=c, decoder=kind), seed=41).to(DEV).eval()
        plain = lambda m, d: m([d, None])[-1][0]
        piped = lambda m, d, nx, p: m.forward_pipelined([d, None], None if nx is None else [nx, None], p)[-1][0]
        refresh = lambda m, x: m.forward_refresh_reservoirs(x)
        gen = MovingEdges(h, w, seed=7)
        deltas = [_cl(gen.step()[0]) for _ in range(12)]
    a, b = make(), make()
    x0 = _cl(torch.randn(1, c, h, w, generator=torch.Generator().manual_seed(33)) * 0.5)
    with torch.no_grad():
        refresh(a, x0), refresh(b, x0)
        for i in range(7):
            want = plain(a, deltas[i]).clone()
            got = piped(b, deltas[i], deltas[i + 1], i % 2).clone()     # (after step 6 the plan of deltas[7] stays pending)
            assert torch.equal(got, want), "eager step %d: %.3e" % (i, (got - want).abs().max().item())
        # a step that is not the one announced is refused, loudly, and so is a plain step while a plan is pending
        with pytest.raises(RuntimeError, match="announced as next"):
            piped(b, deltas[9], None, 1)
        with pytest.raises(RuntimeError, match="planned ahead and has not run"):
            plain(b, deltas[7])
        refresh(a, x0), refresh(b, x0)
        res = deltas[8:12]
        for i in range(4):                                              # eager cycle: allocates nothing new, primes the graphs
            want = plain(a, res[i]).clone()
            got = piped(b, res[i], res[(i + 1) % 4], i % 2).clone()
            assert torch.equal(got, want), "first cycle, step %d" % i
        torch.cuda.synchronize()
        graphs, outs = [], []
        for i in range(4):
            g = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g):
                outs.append(piped(b, res[i], res[(i + 1) % 4], i % 2))
            graphs.append(g)
        for rnd in range(3):
            for i in range(4):
                want = plain(a, res[i]).clone()
                graphs[i].replay()
                got = outs[i].clone()
                assert torch.equal(got, want), "replay cycle %d step %d: %.3e" % (rnd, i, (got - want).abs().max().item())
    torch.cuda.synchronize()
    assert ops.buffer_parity == 0 and ops._phase is None


@pytest.mark.parametrize("host_ordered", [True, False])
@pytest.mark.parametrize("net", ["e2depth", "e2depth_264x352", "evflownet_transposed"])
def test_plan_and_compute_halves_on_two_streams_reproduce_plain_steps(net, host_ordered):
    # plan_ahead / forward_planned: the two halves of forward_pipelined on two streams (ops.LookaheadStepper).  The plan
    # of step k + 1 follows the event recorded after step k - 1 (same buffers as step k - 1), step k + 1 the event
    # recorded after that plan -- as waits on the GPU, or with the host waiting before it launches.  Eager for two cycles,
    # then each half captured as a graph of its own (no edge between streams inside any graph) and replayed three times.
    from maskedincrementeval_amd.evflownet_incr import MultiResUNetRecurrentIncr
    from maskedincrementeval_amd.synthetic import MovingEdges
    if net.startswith("e2depth"):
        h, w, c = (264, 352, 5) if net.endswith("264x352") else (72, 104, 5)      # (the headline frame size)
        make = lambda: seed_module_(E2VIDRecurrentIncr(), seed=31).to(DEV).eval()
        plain = lambda m, d: m([d, None], None)[0][0]
        out_of = lambda r: r[0][0]
        refresh = lambda m, x: m.forward_refresh_reservoirs(x, None)
        res = [_cl(event_voxel_delta(1, c, h, w, 0.02 + 0.03 * (i % 3), seed=5400 + i)[0]) for i in range(4)]
    else:
        h, w, c = 64, 96, 4
        make = lambda: seed_module_(MultiResUNetRecurrentIncr(num_bins=c, decoder="transposed"), seed=41).to(DEV).eval()
        plain = lambda m, d: m([d, None])[-1][0]
        out_of = lambda r: r[-1][0]
        refresh = lambda m, x: m.forward_refresh_reservoirs(x)
        gen = MovingEdges(h, w, seed=9)
        res = [_cl(gen.step()[0]) for _ in range(4)]
    a, b = make(), make()
    x0 = _cl(torch.randn(1, c, h, w, generator=torch.Generator().manual_seed(35)) * 0.5)
    stepper = ops.LookaheadStepper(DEV, host_ordered=host_ordered)

    def step(i, compute, plan):
        return stepper.step(i, lambda: compute(i), lambda: plan((i + 1) % 4))

    with torch.no_grad():
        refresh(a, x0), refresh(b, x0)
        torch.cuda.synchronize()
        for rnd in range(2):
            for i in range(4):
                want = plain(a, res[i]).clone()
                got = out_of(step(i, lambda j: b.forward_planned([res[j], None], j % 2),
                                  lambda j: b.plan_ahead([res[j], None], j % 2))).clone()
                assert torch.equal(got, want), "eager cycle %d step %d: %.3e" % (rnd, i, (got - want).abs().max().item())
        torch.cuda.synchronize()
        g_comp, g_plan, outs = [], [None] * 4, []
        for i in range(4):                                     # capture order = the order the state checks expect
            g = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g):
                outs.append(out_of(b.forward_planned([res[i], None], i % 2)))
            g_comp.append(g)
            g = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g):
                b.plan_ahead([res[(i + 1) % 4], None], (i + 1) % 2)
            g_plan[(i + 1) % 4] = g
        for rnd in range(3):
            for i in range(4):
                want = plain(a, res[i]).clone()
                step(i, lambda j: g_comp[j].replay(), lambda j: g_plan[j].replay())
                got = outs[i].clone()
                assert torch.equal(got, want), "replay cycle %d step %d: %.3e" % (rnd, i, (got - want).abs().max().item())
    torch.cuda.synchronize()
    assert ops.buffer_parity == 0 and ops._phase is None
