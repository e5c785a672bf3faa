"""CPU-side checks: the C-ABI library loads and exports every symbol include/mie.h
declares, host-side argument validation returns status codes (no compute call
reaches a GPU here), and the host logic of the Python surface."""
import ctypes
import functools
import os
import re

import numpy as np
import pytest
import torch
import torch.nn as nn
import torch.nn.functional as F

from maskedincrementeval_amd import _lib
from maskedincrementeval_amd import masked_types as mt
from maskedincrementeval_amd import mask_incr_modules as mm
from maskedincrementeval_amd import synthetic

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "mie.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(mie_[a-z0-9_]+)\s*\(", text)))


def test_header_symbols_are_exported(mie_lib):
    declared = _declared_symbols()
    assert len(declared) >= 12
    assert sorted(_lib.EXPORTS) == declared
    for name in declared:
        assert hasattr(mie_lib, name), name
    assert mie_lib.mie_version() >= 100


def test_tile_capacity(mie_lib):
    assert mie_lib.mie_tile_capacity(1, 264, 352) == 33 * 44
    assert mie_lib.mie_tile_capacity(8, 480, 640) == 8 * 60 * 80
    assert mie_lib.mie_tile_capacity(1, 9, 9) == 4
    assert mie_lib.mie_tile_capacity(0, 8, 8) == 0
    assert _lib.tile_capacity(2, 19, 27) == mie_lib.mie_tile_capacity(2, 19, 27)


def _fake_tileset(n=1, h=16, w=16, null=None):
    """Tile set with non-NULL but never dereferenced host pointers (validation only)."""
    buf = ctypes.create_string_buffer(4096 + 16)
    p = (ctypes.addressof(buf) + 15) & ~15
    vals = dict(pixmask=p, tiles=p, stale=p, counts=p, flags=p)
    if null:
        vals[null] = None
    return _lib.MieTileSet(n, h, w, vals["pixmask"], vals["tiles"], vals["stale"], vals["counts"],
                           vals["flags"]), buf


def test_invalid_arguments_return_status_not_abort(mie_lib):
    # every call below is rejected by host-side validation: nothing is launched
    ts, keep = _fake_tileset()
    buf = ctypes.create_string_buffer(4096)
    p = (ctypes.addressof(buf) + 15) & ~15
    err = lambda: mie_lib.mie_last_error_string().decode()
    # NULL tile set
    assert mie_lib.mie_conv_masked(p, None, 16, None, None, 0, 16, 16, p, None, 16, 3, 1, 1, 32, None, p,
                                   None, None, 0, 0.0, 0, 0, None) == -1
    assert "tile set is NULL" in err()
    # NULL input pointer
    assert mie_lib.mie_conv_masked(None, None, 16, None, None, 0, 16, 16, p, None, 16, 3, 1, 1, 32,
                                   ctypes.byref(ts), p + 1024, None, None, 0, 0.0, 0, 0, None) == -1
    # unsupported kernel size and stride (the reference throws std::logic_error, ext_conv.cu:366)
    assert mie_lib.mie_conv_masked(p, None, 16, None, None, 0, 16, 16, p, None, 16, 4, 1, 1, 32,
                                   ctypes.byref(ts), p + 1024, None, None, 0, 0.0, 0, 0, None) == -2
    assert "kernel size 4" in err()
    assert mie_lib.mie_conv_masked(p, None, 16, None, None, 0, 16, 16, p, None, 16, 3, 3, 1, 32,
                                   ctypes.byref(ts), p + 1024, None, None, 0, 0.0, 0, 0, None) == -2
    # output geometry mismatch
    assert mie_lib.mie_conv_masked(p, None, 16, None, None, 0, 20, 16, p, None, 16, 3, 1, 1, 32,
                                   ctypes.byref(ts), p + 1024, None, None, 0, 0.0, 0, 0, None) == -1
    assert "tile set is" in err()
    # misaligned pointer
    assert mie_lib.mie_conv_masked(p + 4, None, 16, None, None, 0, 16, 16, p, None, 16, 3, 1, 1, 32,
                                   ctypes.byref(ts), p + 1024, None, None, 0, 0.0, 0, 0, None) == -1
    assert "aligned" in err()
    # MFMA path on a shape it cannot take
    assert mie_lib.mie_conv_masked(p, None, 24, None, None, 0, 16, 16, p, None, 24, 3, 1, 1, 32,
                                   ctypes.byref(ts), p + 1024, None, None, 0, 0.0, _lib.PATH_MFMA, 0, None) == -2
    # MFMA path without the matrix-core filter copy
    assert mie_lib.mie_conv_masked(p, None, 32, None, None, 0, 16, 16, p, None, 32, 3, 1, 1, 32,
                                   ctypes.byref(ts), p + 1024, None, None, 0, 0.0, _lib.PATH_MFMA, 0, None) == -2
    assert "mie_pack_filter" in err()
    # filter packing: cin must be a multiple of 8, buffers distinct
    assert mie_lib.mie_pack_filter(p, 12, 3, 32, p + 4096, 0, None) == -2
    assert mie_lib.mie_pack_filter(p, 16, 3, 32, p, 0, None) == -1
    assert mie_lib.mie_pack_filter(p, 16, 3, 32, None, 0, None) == -1
    assert mie_lib.mie_pack_filter(p, 24, 3, 32, p + 4096, 1, None) == -2      # bf16 blocks hold 16 channels
    assert mie_lib.mie_pack_filter(p, 16, 3, 32, p + 4096, 7, None) == -2      # unknown dtype
    # activation without a reservoir
    assert mie_lib.mie_conv_masked(p, None, 16, None, None, 0, 16, 16, p, None, 16, 3, 1, 1, 32,
                                   ctypes.byref(ts), p + 1024, None, None, _lib.ACT_RELU, 0.0, 0, 0, None) == -1
    # channels beyond the filter
    assert mie_lib.mie_conv_masked(p, None, 16, p, None, 16, 16, 16, p, None, 16, 3, 1, 1, 32,
                                   ctypes.byref(ts), p + 1024, None, None, 0, 0.0, 0, 0, None) == -1
    # aliasing that would make workgroups race: input == output for k > 1 (allowed for 1x1), an input mask that is
    # the output tile set's pixel mask, a mask build in place with a footprint wider than the pixel itself
    assert mie_lib.mie_conv_masked(p, None, 16, None, None, 0, 16, 16, p + 2048, None, 16, 3, 1, 1, 32,
                                   ctypes.byref(ts), p, None, None, 0, 0.0, 0, 0, None) == -1
    assert "alias" in err()
    assert mie_lib.mie_conv_masked(p + 512, None, 16, p, None, 16, 16, 16, p + 2048, None, 32, 3, 1, 1, 32,
                                   ctypes.byref(ts), p, None, None, 0, 0.0, 0, 0, None) == -1
    assert "alias" in err()
    assert mie_lib.mie_conv_masked(p, ts.pixmask, 16, None, None, 0, 16, 16, p + 2048, None, 16, 3, 1, 1, 32,
                                   ctypes.byref(ts), p + 1024, None, None, 0, 0.0, 0, 0, None) == -1
    assert "pixel mask" in err()
    assert mie_lib.mie_conv_gates_masked(p, None, 32, p + 512, None, 32, 16, 16, p + 2048, p + 2048, 64, 8,
                                         ctypes.byref(ts), p + 1024, None, None, p + 1024, p + 1024, p + 512,
                                         p + 1536, 0, None) == -1
    assert "h_delta" in err()
    assert mie_lib.mie_build_mask_tiles(ts.pixmask, None, 16, 16, _lib.FOOT_CONV, 3, 1, 1, ctypes.byref(ts), None) == -1
    assert "aliases" in err()
    assert mie_lib.mie_build_mask_tiles(p + 64, ts.pixmask, 16, 16, _lib.FOOT_CONV, 3, 1, 1, ctypes.byref(ts), None) == -1
    up, keep_up = _fake_tileset(h=32, w=32)
    assert mie_lib.mie_build_mask_tiles(up.pixmask, None, 16, 16, _lib.FOOT_UP2X, 0, 0, 0, ctypes.byref(up), None) == -1
    # workspace of the split form: misaligned, sized without a pointer, aliasing the output
    ws_call = lambda ws, nbytes: mie_lib.mie_conv_masked_ws(p, None, 16, None, None, 0, 16, 16, p + 2048, None, 16, 3, 1, 1, 32,
                                                            ctypes.byref(ts), p + 1024, None, None, 0, 0.0, 0, 0, ws, nbytes, None)
    assert ws_call(p + 512 + 4, 64) == -1 and "workspace" in err()
    assert ws_call(None, 64) == -1
    assert ws_call(p + 512, -1) == -1
    assert ws_call(p + 1024, 64) == -1 and "alias" in err()
    # ConvGRU gate math: NULL pointer, aliased reservoirs, unknown dtype
    assert mie_lib.mie_convgru_gates_incr(p, p + 256, None, p + 512, 8, ctypes.byref(ts), 0, None) == -1
    assert mie_lib.mie_convgru_gates_incr(p, p + 256, p + 256, p + 512, 8, ctypes.byref(ts), 0, None) == -1
    assert mie_lib.mie_convgru_gates_incr(p, p + 256, p + 1024, p + 512, 8, ctypes.byref(ts), 3, None) == -2
    # tile set with a NULL member / zero-sized geometry
    bad, keep2 = _fake_tileset(null="tiles")
    assert mie_lib.mie_act_incr(1, 0.0, p, p, p, 8, ctypes.byref(bad), None, 0, 0, None) == -1
    zero, keep3 = _fake_tileset(n=0)
    assert mie_lib.mie_act_incr(1, 0.0, p, p, p, 8, ctypes.byref(zero), None, 0, 0, None) == -1
    assert mie_lib.mie_act_incr(9, 0.0, p, p, p, 8, ctypes.byref(ts), None, 0, 0, None) == -2
    assert mie_lib.mie_act_incr(1, 0.0, p, p, p, 8, ctypes.byref(ts), None, 0, 5, None) == -2   # unknown dtype
    assert mie_lib.mie_build_mask_tiles(None, None, 16, 16, 7, 3, 1, 1, ctypes.byref(ts), None) == -2
    assert mie_lib.mie_build_mask_tiles(None, None, 9, 8, _lib.FOOT_UP2X, 0, 0, 0, ctypes.byref(ts), None) == -1
    assert mie_lib.mie_upsample2x_incr(p, None, None, None, 9, 8, 4, ctypes.byref(ts), p, 0, None) == -1
    assert mie_lib.mie_mask_from_delta(p, 1, 4, 4, 4, -1.0, p, 0, None) == -1
    assert mie_lib.mie_convlstm_gates_incr(p, p, None, p, p, p, p, p, 4, ctypes.byref(ts), 0, None) == -1
    assert mie_lib.mie_tconv_masked(p, None, 4, 9, 9, p, 3, 2, 1, 4, ctypes.byref(ts), p, None, 0, 0.0, 0, None) == -1


def test_mask_plan_rejects_what_it_cannot_run(mie_lib):
    # host-side validation of mie_build_mask_plan: every call below returns before anything is launched
    err = lambda: mie_lib.mie_last_error_string().decode()
    ts, keep = _fake_tileset()
    half, keep_h = _fake_tileset(h=8, w=8)
    two, keep_2 = _fake_tileset(n=2)
    buf = ctypes.create_string_buffer(4096)
    p = (ctypes.addressof(buf) + 15) & ~15

    def plan(*ops_):
        arr = (_lib.MiePlanOp * max(len(ops_), 1))()
        for o, (m1, m2, h, w, foot, k, s, pad, out) in zip(arr, ops_):
            o.in_mask, o.in_mask2, o.h_in, o.w_in, o.foot, o.k, o.stride, o.pad, o.out = m1, m2, h, w, foot, k, s, pad, out
        return mie_lib.mie_build_mask_plan(arr, len(ops_), None)
    conv = (p, None, 16, 16, _lib.FOOT_CONV, 3, 1, 1, ts)
    assert plan() == -1 and "no ops" in err()
    assert mie_lib.mie_build_mask_plan(None, 3, None) == -1
    one = (_lib.MiePlanOp * 1)()
    assert mie_lib.mie_build_mask_plan_wgs(one, 1, 0, None) == -1 and "max_workgroups" in err()
    assert mie_lib.mie_build_mask_plan_wgs(None, 1, 8, None) == -1 and "no ops" in err()
    assert plan(*([conv] * (_lib.PLAN_MAX_STEPS + 1))) == -3 and "at most" in err()
    assert plan((p, None, 16, 16, _lib.FOOT_CONV, 3, 3, 1, ts)) == -2 and "strides 1 and 2" in err()
    assert plan((p, None, 16, 16, _lib.FOOT_TCONV, 3, 1, 1, ts)) == -2 and "stride 2 only" in err()
    assert plan((p, None, 16, 16, 9, 3, 1, 1, ts)) == -2 and "unknown footprint" in err()
    assert plan((p, None, 20, 16, _lib.FOOT_CONV, 3, 1, 1, ts)) == -1 and "tile set is" in err()
    assert plan((p, None, 16, 16, _lib.FOOT_UP2X, 0, 0, 0, ts)) == -1 and "up2x" in err()
    assert plan((None, p, 16, 16, _lib.FOOT_CONV, 3, 1, 1, ts)) == -1 and "in_mask2 given without in_mask" in err()
    assert plan(conv, (p, None, 16, 16, _lib.FOOT_CONV, 3, 1, 1, two)) == -1 and "batch size" in err()
    assert plan((ts.pixmask, None, 16, 16, _lib.FOOT_CONV, 3, 1, 1, ts)) == -1 and "aliases" in err()
    # a mask of an earlier op read at another size than it was built with
    assert plan(conv, (ts.pixmask, None, 15, 15, _lib.FOOT_CONV, 3, 2, 1, half)) == -1 and "reads a mask of" in err()
    bad, keep_b = _fake_tileset(null="flags")
    assert plan((p, None, 16, 16, _lib.FOOT_CONV, 3, 1, 1, bad)) == -1


def test_newer_entry_points_reject_bad_arguments(mie_lib):
    # host-side validation of the fused tail, the workspace forms and the bf16 event frame: every call returns before
    # anything is launched
    err = lambda: mie_lib.mie_last_error_string().decode()
    big, keep = _fake_tileset(h=32, w=32)
    buf = ctypes.create_string_buffer(8192)
    p = (ctypes.addressof(buf) + 255) & ~255
    q = p + 1024
    BF16, F32 = 1, 0

    def pred(c=64, cout=32, dtype=BF16, act=1, h=16, w=16, skip=q, out=big, pdelta=p + 2048):
        return mie_lib.mie_upconv_pred_masked(p, None, None, None, c, h, w, p, p, c, cout, ctypes.byref(out), p + 512, act, 0.0,
                                              skip, None, p + 768, p + 1280, 3, 0.0, pdelta, dtype, None)
    assert pred(dtype=F32) == -2 and "bf16" in err()
    assert pred(c=128) == -2 and pred(cout=64) == -2
    assert pred(skip=None) == -1 and "NULL" in err()
    assert pred(h=15) == -1 and "twice the input" in err()
    assert pred(act=3) == -2 and "activation" in err()                # sigmoid on the decoder: the separate kernels
    assert pred(pdelta=q) == -1 and "alias" in err()

    # workspace forms: alignment, size without a pointer, aliasing
    up = lambda ws, nbytes: mie_lib.mie_upconv_masked_ws(p, None, None, None, 64, 16, 16, p, p, 64, 5, 2, 32, ctypes.byref(big),
                                                         p + 4096, None, None, 0, 0.0, F32, ws, nbytes, None)
    assert up(p + 5000 + 4, 1024) == -1 and "workspace" in err()
    assert up(None, 1024) == -1 and "workspace" in err()
    assert up(p + 4096, 1024) == -1 and "alias" in err()
    gates = lambda ws, nbytes: mie_lib.mie_conv_gates_masked_ws(p, None, 32, q, None, 32, 32, 32, p, p, 64, 32, ctypes.byref(big),
                                                                p + 512, None, None, p + 1024, p + 1536, p + 2048, p + 2560,
                                                                F32, ws, nbytes, None)
    assert gates(p + 2048, 4096) == -1 and "alias" in err()
    assert gates(p + 6000 + 4, 64) == -1 and "workspace" in err()

    # threshold mask + build in one launch: footprints it has no form for, aliasing, sizes
    half, keep_h = _fake_tileset(h=8, w=8)
    thr = lambda k=3, s=2, pad=1, mask=q, m2=None, t=0.1, c=4, dtype=F32, ts=half: mie_lib.mie_build_mask_tiles_thresholded(
        p, c, dtype, t, mask, m2, 16, 16, k, s, pad, ctypes.byref(ts), None)
    assert thr(k=1, s=2, pad=0) == -2 and "no one-launch form" in err()
    assert thr(k=11, s=2, pad=5) == -2
    assert thr(mask=None) == -1 and "NULL" in err()
    assert thr(t=-0.5) == -1 and "threshold" in err()
    assert thr(c=0) == -1 and thr(dtype=2) == -2
    assert thr(mask=half.pixmask) == -1 and "three buffers" in err()
    assert thr(m2=q) == -1 and "three buffers" in err()
    assert thr(k=3, s=1, pad=1) == -1 and "tile set is" in err()

    # bf16 event frame: the rounded frame is a buffer of its own
    ev = lambda out: mie_lib.mie_events_to_frame_bf16(None, 0, 0, 5, 8, 8, 0, 0, 0, 0, 1.0, 0.0, 0.0, -1.0, 0, p, out, q, None)
    assert ev(p + 4096) == -1 and "window length" in err()             # the base entry point's checks come first


def test_check_raises_runtime_error(mie_lib):
    rc = mie_lib.mie_mask_from_delta(None, 1, 4, 4, 4, 0.0, None, 0, None)
    with pytest.raises(RuntimeError, match="NULL pointer"):
        _lib.check(rc)
    assert issubclass(_lib.MieError, RuntimeError)


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", str(tmp_path / "nope.so"))
    with pytest.raises(RuntimeError, match="no fallback"):
        _lib.lib()


def test_ops_refuse_cpu_tensors():
    from maskedincrementeval_amd import ops
    ts = mt.TileMask(1, 16, 16, "cpu")
    x = torch.zeros(1, 8, 16, 16).contiguous(memory_format=torch.channels_last)
    with pytest.raises(RuntimeError, match="no CPU path"):
        ops.act_incr(_lib.ACT_RELU, 0.0, x, x.clone(), x.clone(), ts)


def test_activation_kind_mapping():
    assert mm.activation_kind(torch.relu) == (_lib.ACT_RELU, 0.0)
    assert mm.activation_kind(torch.sigmoid)[0] == _lib.ACT_SIGMOID
    assert mm.activation_kind(torch.tanh)[0] == _lib.ACT_TANH
    assert mm.activation_kind(F.leaky_relu) == (_lib.ACT_LEAKY_RELU, 0.01)
    assert mm.activation_kind(nn.LeakyReLU(0.2)) == (_lib.ACT_LEAKY_RELU, pytest.approx(0.2))
    assert mm.activation_kind(mm.leaky_relu_op(0.05)) == (_lib.ACT_LEAKY_RELU, pytest.approx(0.05))
    assert mm.activation_kind(functools.partial(F.leaky_relu, negative_slope=0.3))[1] == pytest.approx(0.3)
    with pytest.raises(NotImplementedError):
        mm.activation_kind(torch.exp)


def test_module_surface_matches_reference_names():
    # names the reference exports from incr_modules/mask_incr_modules.py and *_functional.py
    for name in ("IncrementMaskModule", "KFencedMaskModule", "PointwiseMultiplyIncr",
                 "nnReservedMultiplication", "NonlinearPointOpIncr", "nnLinearIncr", "nnConvIncrBase",
                 "nnConvIncr", "nnBatchNorm2dIncr", "nnMaxPool2dIncr", "nnAdaptiveAvgPool2dIncr",
                 "nnSequentialIncr", "nnReservedActivation", "nnReluIncr", "nnSigmoidIncr", "nnTanhIncr"):
        assert hasattr(mm, name), name
    from maskedincrementeval_amd import mask_incr_functional as mf
    for name in ("AccumStreamManager", "IncrementReserve", "IncrPointwiseMultiply", "conv2d_from_module",
                 "transposed_conv2d_from_module", "bn2d_from_module", "interpolate_from_module"):
        assert hasattr(mf, name), name
    for name in ("Sp", "DenseT", "SpOrDense", "Masked", "_device"):
        assert hasattr(mt, name), name
    c = mm.nnConvIncr(3, 5, 3, 1, 1, bias=False)
    assert set(c.state_dict().keys()) == {"weight"}               # nn.Conv2d keys, as in the reference
    assert tuple(c.conv2d_weights.shape) == (3, 3, 3, 5)          # [Cin, K, K, Cout]
    assert torch.equal(c.conv2d_weights.plain, c.weight.detach().permute(1, 2, 3, 0))
    with torch.no_grad():
        c.weight.mul_(2.0)
    assert torch.equal(c.conv2d_weights.plain, c.weight.detach().permute(1, 2, 3, 0))   # follows the weight
    with pytest.raises(NotImplementedError):
        mm.nnConvIncr(3, 5, 4)._geometry()
    with pytest.raises(NotImplementedError):
        mm.nnConvIncr(3, 5, 3, stride=3)._geometry()


def test_e2depth_module_tree_and_shapes():
    from maskedincrementeval_amd.e2depth_incr import E2VIDRecurrentIncr
    net = E2VIDRecurrentIncr()
    sd = net.state_dict()
    # layer shapes of the reference trace (todo.txt:34-57)
    u = "unetrecurrent."
    assert tuple(sd[u + "head.conv2d.weight"].shape) == (32, 5, 5, 5)
    assert tuple(sd[u + "encoders.0.conv.conv2d.weight"].shape) == (64, 32, 5, 5)
    assert tuple(sd[u + "encoders.0.recurrent_block.Gates.weight"].shape) == (256, 128, 3, 3)
    assert tuple(sd[u + "encoders.2.recurrent_block.Gates.weight"].shape) == (1024, 512, 3, 3)
    assert tuple(sd[u + "resblocks.1.conv2.weight"].shape) == (256, 256, 3, 3)
    assert tuple(sd[u + "decoders.0.conv2d.weight"].shape) == (128, 256, 5, 5)
    assert tuple(sd[u + "decoders.2.conv2d.weight"].shape) == (32, 64, 5, 5)
    assert tuple(sd[u + "pred.conv2d.weight"].shape) == (1, 32, 1, 1)
    # there is no CPU path: CPU tensors are refused loudly, by the refresh as by the incremental forward
    synthetic.seed_module_(net, 3)
    with torch.no_grad():
        with pytest.raises(RuntimeError, match="no CPU path"):
            net.forward_refresh_reservoirs(torch.randn(1, 5, 16, 24), None)
        with pytest.raises(RuntimeError, match="no CPU path"):
            net([torch.randn(1, 5, 16, 24), None], None)


def test_increment_reserve_keeps_pointer():
    from maskedincrementeval_amd.mask_incr_functional import IncrementReserve
    r = IncrementReserve(torch.randn(1, 4, 6, 6))
    assert r.reservoir.permute(0, 2, 3, 1).is_contiguous()       # channels_last, as the reference
    ptr = r.reservoir.data_ptr()
    x = torch.randn(1, 4, 6, 6)
    r.update_reservoir(x)
    assert r.reservoir.data_ptr() == ptr and torch.equal(r.reservoir, x)
    r.accumulate([torch.ones(1, 4, 6, 6), None])
    assert torch.equal(r.reservoir, x + 1)


def test_blob_mask_density_and_determinism():
    for p in (0.01, 0.05, 0.20):
        m = synthetic.blob_mask(264, 352, p, seed=11)
        assert m.sum() == round(p * 264 * 352)
        assert np.array_equal(m, synthetic.blob_mask(264, 352, p, seed=11))
    d, m = synthetic.gaussian_delta(1, 8, 32, 40, 0.1, 0.1, seed=2)
    assert (d[:, :, m[0, 0] == 0] == 0).all() and m.dtype == torch.uint8
    ev, m2 = synthetic.event_voxel_delta(1, 5, 32, 40, 0.05, seed=3)
    vals = torch.unique(ev * 10).round()
    assert (ev[:, :, m2[0, 0] == 0] == 0).all() and torch.allclose(ev * 10, (ev * 10).round(), atol=1e-5)
    assert vals.abs().max() >= 2


def test_single_hip_runtime_is_mapped(mie_lib):
    # libmie_hip.so must bind to the HIP runtime PyTorch-ROCm already loaded; two runtimes in one
    # process leave the second one without a device
    with open("/proc/self/maps") as f:
        paths = {line.split()[-1] for line in f if "libamdhip64" in line}
    assert len(paths) == 1, paths


def test_python_constants_mirror_the_header():
    """Every MIE_* code the Python side passes is the value include/mie.h defines (the dtype codes included: a
    mismatch would silently select another arithmetic)."""
    import re
    hdr = open(os.path.join(ROOT, "include", "mie.h")).read()
    defs = {m.group(1): int(m.group(2)) for m in re.finditer(r"#define\s+(MIE_[A-Z0-9_]+)\s+(-?\d+)\b", hdr)}
    pairs = [("MIE_DTYPE_F32", _lib.DTYPE_F32), ("MIE_DTYPE_BF16", _lib.DTYPE_BF16),
             ("MIE_DTYPE_F32_BF16X3", _lib.DTYPE_F32_BF16X3), ("MIE_PATH_AUTO", _lib.PATH_AUTO),
             ("MIE_PATH_VALU", _lib.PATH_VALU), ("MIE_PATH_MFMA", _lib.PATH_MFMA), ("MIE_FOOT_CONV", _lib.FOOT_CONV),
             ("MIE_FOOT_UP2X", _lib.FOOT_UP2X), ("MIE_FOOT_TCONV", _lib.FOOT_TCONV),
             ("MIE_PLAN_MAX_STEPS", _lib.PLAN_MAX_STEPS)]
    for name, value in pairs:
        assert defs[name] == value, name


def test_three_term_shape_query_needs_no_gpu(mie_lib):
    """mie_conv_f32x3_takes is host logic: which conv shapes run fp32 deltas in the three-term bf16 form."""
    takes = mie_lib.mie_conv_f32x3_takes
    assert takes(3, 1, 64, 64, 256) == 1 and takes(5, 1, 256, 0, 128) == 1 and takes(5, 2, 32, 0, 64) == 1
    assert takes(3, 2, 64, 0, 64) == 0 and takes(7, 1, 64, 0, 64) == 0 and takes(1, 1, 64, 0, 64) == 0
    assert takes(3, 1, 48, 0, 64) == 0 and takes(3, 1, 64, 0, 48) == 0 and takes(5, 2, 24, 0, 64) == 0
