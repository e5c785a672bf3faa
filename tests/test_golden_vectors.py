"""Golden vectors (tests/golden/vectors.npz, written by tests/golden/make_golden.py).

CPU: the oracle still reproduces every stored vector (a change of the oracle shows up against
data).  GPU: the HIP path, through the C ABI, reproduces the stored expectations -- masks, tile
lists and the quantiser bit-exact, floating point within rtol 1e-4 / atol 1e-5.
"""
import os

import numpy as np
import pytest
import torch

from oracle import events_oracle as eo
from oracle import incr_oracle as io
from oracle import mask_oracle as mo

G = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "vectors.npz"))
RTOL, ATOL = 1e-4, 1e-5
DEV = "cuda:0"


def _t(name):
    return torch.from_numpy(G[name])


def _close(got, want, what):
    got = torch.as_tensor(got).detach().float().cpu()
    want = torch.as_tensor(want).float()
    assert torch.allclose(got, want, rtol=RTOL, atol=ATOL), "%s: max|diff| %.3e" % (what, (got - want).abs().max())


# ---- CPU: oracle against the stored vectors ---------------------------------------------------
def test_oracle_reproduces_mask_vectors():
    for k, s, p in ((3, 1, 1), (5, 2, 2)):
        tag = "k%ds%d" % (k, s)
        f0, f1 = mo.footprint_conv(G["mask_in0"], k, s, p), mo.footprint_conv(G["mask_in1"], k, s, p)
        assert np.array_equal(f0, G["foot0_" + tag]) and np.array_equal(f1, G["foot1_" + tag])
        assert np.array_equal(mo.tile_list(f0), G["tiles0_" + tag])
        assert np.array_equal(mo.stale_list(mo.tile_list(f0), mo.tile_list(f1)), G["stale1_" + tag])
    assert np.array_equal(mo.footprint_up2x(G["mask_in0"]), G["foot_up2x"])


def test_oracle_reproduces_float_vectors():
    res1, res2 = io.Reserve(_t("chain_r0").clone()), io.Reserve(io.leaky_relu(_t("chain_r0")).clone())
    for step in range(3):
        y = io.conv_incr(_t("chain_d%d" % step), _t("chain_w"), 1, 1)
        y = io.act_incr(torch.relu, res2, io.act_incr(io.leaky_relu, res1, y))
        _close(y, G["chain_out%d" % step], "chain step %d" % step)
    cell = io.ConvLSTMOracle(_t("lstm_w"), _t("lstm_b"), 8)
    h0, c0 = cell.refresh(_t("lstm_x0"), None)
    _close(h0, G["lstm_h0"], "lstm h0"), _close(c0, G["lstm_c0"], "lstm c0")
    for step in range(2):
        dh, dc = cell.incr(_t("lstm_d%d" % step))
        _close(dh, G["lstm_dh%d" % step], "lstm dh"), _close(dc, G["lstm_dc%d" % step], "lstm dc")
    carry = io.Reserve(torch.zeros(1, 4, 16, 16))
    for step in range(3):
        assert torch.equal(io.kfenced(carry, torch.tensor(0.125), _t("kf_d%d" % step)), _t("kf_f%d" % step))
    fr, fm = eo.frame(G["ev"], "voxelgrid", 5, 20, 30, 0.05, 0.01, pad=(3, 3, 2, 2))
    _close(fr, G["ev_frame"], "event frame")
    assert np.array_equal(fm, G["ev_frame_mask"])


# ---- GPU: the HIP path against the stored vectors ------------------------------------------------
def _dev(t):
    from maskedincrementeval_amd import ops
    return ops.as_nhwc(torch.as_tensor(t).to(DEV).contiguous(memory_format=torch.channels_last))


@pytest.mark.gpu
def test_gpu_masks_and_tile_lists_match_golden():
    from maskedincrementeval_amd import _lib, ops
    from maskedincrementeval_amd.masked_types import TileMask
    n, h, w = G["mask_in0"].shape
    for k, s, p in ((3, 1, 1), (5, 2, 2)):
        tag = "k%ds%d" % (k, s)
        ho, wo = mo.conv_out_size(h, w, k, s, p)
        ts = TileMask(n, ho, wo, DEV)
        for step in (0, 1):
            m = torch.from_numpy(G["mask_in%d" % step]).unsqueeze(1).contiguous().to(DEV)
            ops.build_mask_tiles(m, None, n, h, w, _lib.FOOT_CONV, k, s, p, ts)
            torch.cuda.synchronize()
            assert np.array_equal(ts.pixmask[:, 0].cpu().numpy(), G["foot%d_%s" % (step, tag)])
            assert np.array_equal(ts.active_tiles().cpu().numpy(), G["tiles%d_%s" % (step, tag)])
        assert np.array_equal(ts.stale_tiles().cpu().numpy(), G["stale1_" + tag])
    ts = TileMask(n, 2 * h, 2 * w, DEV)
    m = torch.from_numpy(G["mask_in0"]).unsqueeze(1).contiguous().to(DEV)
    ops.build_mask_tiles(m, None, n, h, w, _lib.FOOT_UP2X, 0, 0, 0, ts)
    assert np.array_equal(ts.pixmask[:, 0].cpu().numpy(), G["foot_up2x"])


@pytest.mark.gpu
def test_gpu_activation_chain_lstm_quantiser_events_match_golden():
    from maskedincrementeval_amd import mask_incr_modules as mm
    from maskedincrementeval_amd import ops
    from maskedincrementeval_amd.e2depth_incr import ConvLSTMIncr
    from maskedincrementeval_amd.event_frontend import EventFrames
    from maskedincrementeval_amd.masked_types import TileMask
    from maskedincrementeval_amd import _lib
    # conv3x3 -> LeakyReLU -> ReLU, module by module
    conv = mm.nnConvIncr(8, 8, 3, 1, 1, bias=False).to(DEV).eval()
    with torch.no_grad():
        conv.weight.copy_(_t("chain_w"))
    leaky, relu = mm.nnReservedActivation(mm.leaky_relu_op(0.01)), mm.nnReluIncr()
    leaky.forward_refresh_reservoirs(_dev(G["chain_r0"]))
    relu.forward_refresh_reservoirs(_dev(io.leaky_relu(_t("chain_r0"))))
    for step in range(3):
        with torch.no_grad():
            y = relu(leaky(conv([_dev(G["chain_d%d" % step]), _t("chain_m%d" % step).to(DEV)])))
        _close(y[0], G["chain_out%d" % step], "chain step %d" % step)
    _close(leaky.in_res.reservoir, G["chain_res_leaky"], "leaky reservoir")
    _close(relu.in_res.reservoir, G["chain_res_relu"], "relu reservoir")
    # ConvLSTM
    cell = ConvLSTMIncr(8, 8, 3).to(DEV).eval()
    with torch.no_grad():
        cell.Gates.weight.copy_(_t("lstm_w")), cell.Gates.bias.copy_(_t("lstm_b"))
        h0, c0 = cell.forward_refresh_reservoirs(_dev(G["lstm_x0"]), None)
        _close(h0, G["lstm_h0"], "lstm h0"), _close(c0, G["lstm_c0"], "lstm c0")
        for step in range(2):
            dh, dc = cell([_dev(G["lstm_d%d" % step]), _t("lstm_m%d" % step).to(DEV)], None)
            _close(dh[0], G["lstm_dh%d" % step], "lstm dh"), _close(dc[0], G["lstm_dc%d" % step], "lstm dc")
    # quantiser: bit-exact
    carry, out = ops.new_nhwc(1, 4, 16, 16, DEV), ops.new_nhwc(1, 4, 16, 16, DEV)
    ts = TileMask(1, 16, 16, DEV)
    for step in range(3):
        ops.build_mask_tiles(_t("kf_m%d" % step).to(DEV), None, 1, 16, 16, _lib.FOOT_CONV, 1, 1, 0, ts)
        ops.kfence_incr(_dev(G["kf_d%d" % step]), carry, 0.125, out, ts)
        assert torch.equal(out.cpu(), _t("kf_f%d" % step))
    assert torch.equal(carry.cpu(), _t("kf_carry"))
    # event front end
    fe = EventFrames(30, 20, pad=(3, 3, 2, 2), device=DEV)
    fe.set_events(G["ev"])
    _close(fe.frame(0.01)[0], G["ev_frame"], "event frame")
    d, m = fe.delta(0.01, 0.012)
    _close(d[0], G["ev_delta"], "event delta")
    assert np.array_equal(m[0, 0].cpu().numpy(), G["ev_delta_mask"])
    fh = EventFrames(30, 20, evframe_type="histogram", pad=(0, 0, 0, 0), device=DEV)
    ev = G["ev"].copy()
    ev[:, 3] = np.where(ev[:, 3] == 0, -1.0, ev[:, 3])
    fh.set_events(ev)
    assert np.array_equal(fh.frame(0.01)[0].cpu().numpy(), G["ev_hist"])
