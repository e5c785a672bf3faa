"""Test infrastructure: every tile set a network step builds, checked against the numpy mask oracle.

Every structural mask of the two networks is an integer function of the input pixel mask: a chain of
conv / bilinear / transposed-conv footprints (oracle/mask_oracle.py; definitions
incr_modules/utils.py:22-25, utils/str_sparse_utils.py:10-11 of the reference).  Two checks:

* `BuildRecorder` + `check_recorded_builds`: records every tile-set build of a step (which masks went in, which
  footprint, which set came out) and replays that wiring on the CPU **from the oracle's input pixel mask**; every
  set's pixel mask, ascending tile list and stale list (against the expected list of the step before) must
  match exactly.  This covers every set of a step, helper sets included.
* `e2depth_chain` / `evflownet_chain`: the chain written down independently from the network definitions
  (incr_modules/e2depth_incr.py:402-439, evflownet_incr.py:451-470), per named layer; `check_e2depth_layers` /
  `check_evflownet_layers` look the layers' tile sets up in the module tree and compare the lists.
"""
import numpy as np
import torch

from maskedincrementeval_amd import _lib, ops
from maskedincrementeval_amd.masked_types import TileMask
from oracle import mask_oracle as mo


class BuildRecorder:
    """`with BuildRecorder() as rec:` records the arguments of every ops.build_mask_tiles call."""

    def __enter__(self):
        self.calls = []
        self._orig = ops.build_mask_tiles

        def wrapped(in_mask, in_mask2, n, h_in, w_in, foot, k, stride, pad, out):
            self.calls.append((in_mask, in_mask2, n, h_in, w_in, foot, k, stride, pad, out))
            return self._orig(in_mask, in_mask2, n, h_in, w_in, foot, k, stride, pad, out)
        ops.build_mask_tiles = wrapped
        return self

    def __exit__(self, *exc):
        ops.build_mask_tiles = self._orig
        return False


def _pix_of(m):
    return None if m is None else (m.pixmask if isinstance(m, TileMask) else m)


def footprint(mask, foot, k, stride, pad, h_out, w_out):
    if foot == _lib.FOOT_CONV:
        return mo.footprint_conv(mask, k, stride, pad)
    if foot == _lib.FOOT_UP2X:
        return mo.footprint_up2x(mask)
    return mo.footprint_tconv(mask, k, stride, pad, h_out, w_out)


def check_recorded_builds(calls, seeds, prev_lists, what=""):
    """calls: BuildRecorder.calls of one step; seeds: {data_ptr of a pixel-mask tensor: numpy (N,H,W) oracle mask}
    for the masks that come from outside (the input mask); prev_lists: {data_ptr of a tile list: expected active
    list after the previous step}, updated in place.  Returns the number of sets checked."""
    known = dict(seeds)
    for idx, (m1, m2, n, h_in, w_in, foot, k, stride, pad, out) in enumerate(calls):
        p1, p2 = _pix_of(m1), _pix_of(m2)
        if p1 is None:
            src = np.ones((n, h_in, w_in), dtype=np.uint8)           # None = every pixel active
        else:
            assert p1.data_ptr() in known, "%s build %d reads a mask no earlier build or seed produced" % (what, idx)
            src = known[p1.data_ptr()]
            if p2 is not None:
                assert p2.data_ptr() in known, "%s build %d: second mask unknown" % (what, idx)
                src = src | known[p2.data_ptr()]
        want = footprint(src, foot, k, stride, pad, out.h, out.w)
        tag = "%s build %d (foot %d k %d s %d p %d -> %dx%d)" % (what, idx, foot, k, stride, pad, out.h, out.w)
        got = out.pixmask[:, 0].cpu().numpy()
        assert got.shape == want.shape and np.array_equal(got != 0, want != 0), tag + ": pixel mask"
        tiles = mo.tile_list(want)
        assert np.array_equal(out.active_tiles().cpu().numpy(), tiles), tag + ": active tile list"
        prev = prev_lists.get(out.tiles.data_ptr(), np.zeros(0, dtype=np.int32))
        assert np.array_equal(out.stale_tiles().cpu().numpy(), mo.stale_list(prev, tiles)), tag + ": stale list"
        prev_lists[out.tiles.data_ptr()] = tiles
        known[out.pixmask.data_ptr()] = want
    return len(calls)


def _tile_set(module, name, n, h, w):
    """The tile set `name` a module built at (n, h, w); fails if the module never made one."""
    hits = [b for key, b in module._ib().items() if key[0] == "t" and key[1] == name and key[2] == (n, h, w)]
    assert len(hits) == 1, "%s has no tile set %r at %s: %s" % (type(module).__name__, name, (n, h, w),
                                                                [k for k in module._ib() if k[0] == "t"])
    return hits[0]


def _check_layers(pairs, what):
    for name, ts, want in pairs:
        assert (ts.h, ts.w) == want.shape[1:], "%s %s: plane %s vs %s" % (what, name, (ts.h, ts.w), want.shape)
        assert np.array_equal(ts.active_tiles().cpu().numpy(), mo.tile_list(want)), "%s %s: active tile list" % (what, name)
        assert np.array_equal(ts.pixmask[:, 0].cpu().numpy() != 0, want != 0), "%s %s: pixel mask" % (what, name)
    return len(pairs)


def e2depth_chain(pm, num_encoders=3, num_res=2):
    """Layer name -> expected output pixel mask of E2Depth-incr for input pixel mask pm (N,H,W):
    head 5x5; per encoder a 5x5 stride-2 conv and the 3x3 gates conv of its ConvLSTM (state deltas zero);
    residual blocks of two 3x3 convs (the residual's pixels are covered); per decoder bilinear x2 of
    (x + skip) and a 5x5 conv; prediction 1x1 over (x + head)."""
    e = {}
    m = e["head"] = mo.footprint_conv(pm, 5, 1, 2)
    skips = []
    for i in range(num_encoders):
        m = e["enc%d.conv" % i] = mo.footprint_conv(m, 5, 2, 2)
        m = e["enc%d.gates" % i] = mo.footprint_conv(m, 3, 1, 1)
        skips.append(m)
    for j in range(num_res):
        m1 = e["res%d.conv1" % j] = mo.footprint_conv(m, 3, 1, 1)
        m = e["res%d.conv2" % j] = mo.footprint_conv(m1, 3, 1, 1)
    for i in range(num_encoders):
        u = e["dec%d.up" % i] = mo.footprint_up2x(m | skips[num_encoders - 1 - i])
        m = e["dec%d.conv" % i] = mo.footprint_conv(u, 5, 1, 2)
    e["pred"] = m | e["head"]
    return e


def check_e2depth_layers(model, pm, what=""):
    """Every layer's tile set of a fused E2VIDRecurrentIncr after a step against e2depth_chain(pm)."""
    net = model.unetrecurrent
    e = e2depth_chain(pm, net.num_encoders, net.num_residual_blocks)
    n = pm.shape[0]

    def ts(module, name, key):
        return _tile_set(module, name, n, *e[key].shape[1:])
    pairs = [("head", ts(net.head.conv2d, "out_act", "head"), e["head"])]
    for i, enc in enumerate(net.encoders):
        pairs.append(("enc%d.conv" % i, ts(enc.conv.conv2d, "out_act", "enc%d.conv" % i), e["enc%d.conv" % i]))
        gates = enc.recurrent_block
        name = "gates" if gates.__dict__.get("_gates_interleaved", False) else "out"
        pairs.append(("enc%d.gates" % i, ts(gates.Gates, name, "enc%d.gates" % i), e["enc%d.gates" % i]))
    for j, rb in enumerate(net.resblocks):
        pairs.append(("res%d.conv1" % j, ts(rb.conv1, "out_act", "res%d.conv1" % j), e["res%d.conv1" % j]))
        pairs.append(("res%d.conv2" % j, ts(rb.conv2, "out_act", "res%d.conv2" % j), e["res%d.conv2" % j]))
    for i, dec in enumerate(net.decoders):
        pairs.append(("dec%d.up" % i, ts(dec.upsample, "out", "dec%d.up" % i), e["dec%d.up" % i]))
        pairs.append(("dec%d.conv" % i, ts(dec.conv2d, "out_act", "dec%d.conv" % i), e["dec%d.conv" % i]))
    pairs.append(("pred", ts(net.pred.conv2d, "out_act", "pred"), e["pred"]))
    return _check_layers(pairs, what)


def evflownet_chain(pm, decoder, num_encoders=4, num_res=2):
    """Layer name -> expected output pixel mask of EVFlowNet-incr: per encoder a 3x3 stride-2 conv and the 3x3
    gate conv of its ConvGRU; residual blocks of two 3x3 convs; per decoder either bilinear x2 of every part and a
    3x3 conv over their concat, or a 3x3 stride-2 transposed conv (pad 1, output twice the input) over it; the flow
    head is a 1x1 conv (same pixels).  The flow estimate fed to the next decoder shares the mask of x."""
    e = {}
    m = pm
    skips = []
    for i in range(num_encoders):
        m = e["enc%d.conv" % i] = mo.footprint_conv(m, 3, 2, 1)
        m = e["enc%d.gru" % i] = mo.footprint_conv(m, 3, 1, 1)
        skips.append(m)
    for j in range(num_res):
        m1 = e["res%d.conv1" % j] = mo.footprint_conv(m, 3, 1, 1)
        m = e["res%d.conv2" % j] = mo.footprint_conv(m1, 3, 1, 1)
    for i in range(num_encoders):
        both = m | skips[num_encoders - 1 - i]
        n, h, w = both.shape
        if decoder == "transposed":
            m = mo.footprint_tconv(both, 3, 2, 1, 2 * h, 2 * w)
        else:
            m = mo.footprint_conv(mo.footprint_up2x(both), 3, 1, 1)
        e["dec%d" % i] = m
    return e


def check_evflownet_layers(model, pm, what=""):
    e = evflownet_chain(pm, model.decoder_kind, model.num_encoders, model.num_residual_blocks)
    n = pm.shape[0]
    pairs = []
    for i, enc in enumerate(model.encoders):
        key = "enc%d.conv" % i
        pairs.append((key, _tile_set(enc.conv.conv2d, "out_act", n, *e[key].shape[1:]), e[key]))
        key = "enc%d.gru" % i
        pairs.append((key, _tile_set(enc.recurrent_block.update_gate, "out_act", n, *e[key].shape[1:]), e[key]))
    for j, rb in enumerate(model.resblocks):
        for c in ("conv1", "conv2"):
            key = "res%d.%s" % (j, c)
            pairs.append((key, _tile_set(getattr(rb, c), "out_act", n, *e[key].shape[1:]), e[key]))
    for i, dec in enumerate(model.decoders):
        key = "dec%d" % i
        if model.decoder_kind == "transposed":
            ts = _tile_set(dec.transposed_conv2d, "out", n, *e[key].shape[1:])
        else:
            ts = _tile_set(dec.conv2d, "out_act", n, *e[key].shape[1:])
        pairs.append((key, ts, e[key]))
    return _check_layers(pairs, what)
