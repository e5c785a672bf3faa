"""GPU parity: pixel masks, footprints and ordered active-tile lists are bit-exact
against the numpy oracle (oracle/mask_oracle.py), through the C ABI."""
import numpy as np
import pytest
import torch

from maskedincrementeval_amd import _lib, ops
from maskedincrementeval_amd.masked_types import TileMask
from maskedincrementeval_amd.synthetic import blob_mask
from oracle import mask_oracle as mo

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _to_dev_mask(m: np.ndarray) -> torch.Tensor:
    return torch.from_numpy(m).unsqueeze(1).contiguous().to(DEV)


def _check_tileset(ts: TileMask, want_mask: np.ndarray, prev_tiles=None):
    torch.cuda.synchronize()
    got = ts.pixmask[:, 0].cpu().numpy()
    assert np.array_equal(got, want_mask), "pixel mask differs"
    tiles = ts.active_tiles().cpu().numpy()
    want_tiles = mo.tile_list(want_mask)
    assert np.array_equal(tiles, want_tiles), "tile list differs"
    assert int(ts.counts[_lib.CNT_TICKET].item()) == 0, "ticket counter not reset"
    if prev_tiles is not None:
        assert np.array_equal(ts.stale_tiles().cpu().numpy(), mo.stale_list(prev_tiles, want_tiles))
    return want_tiles


@pytest.mark.parametrize("dt", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("shape,c,thr", [((1, 264, 352), 5, 0.0), ((2, 37, 53), 3, 0.0),
                                         ((1, 33, 44), 64, 1e-4), ((1, 16, 16), 1, 0.5),
                                         ((3, 7, 9), 13, 0.0), ((1, 5, 13), 2, 0.5), ((2, 33, 41), 18, 0.0)])
def test_mask_from_delta(shape, c, thr, dt):
    # thread-per-pixel rows (multiples of 4 channels, many channels) and the contiguous-span form (few channels that
    # are no multiple of 4), pixel counts that are no multiple of 64, a delta whose last 16-byte load would run past
    # its end, one active channel per pixel
    n, h, w = shape
    g = torch.Generator().manual_seed(h * w + c)
    d = torch.randn((n, c, h, w), generator=g) * (torch.rand((n, 1, h, w), generator=g) < 0.07)
    d = d * (torch.rand((n, c, h, w), generator=g) < 0.4)         # most channels of an active pixel are zero
    d[0, :, 0, 0] = 0.0
    d[0, c - 1, h - 1, w - 1] = 2e-4 if thr < 1e-3 else 0.75    # only the last channel of the last pixel
    d[0, 0, 0, 1] = 0.25                                          # below the larger threshold
    d = d.to(dt).float()
    x = d.to(dt).to(DEV).contiguous(memory_format=torch.channels_last)
    x = ops.as_nhwc(x)
    out = torch.zeros((n, 1, h, w), dtype=torch.uint8, device=DEV)
    ops.mask_from_delta(x, thr, out)
    torch.cuda.synchronize()
    assert np.array_equal(out[:, 0].cpu().numpy(), mo.pixel_mask(d.numpy(), thr))


@pytest.mark.parametrize("k,s,p", [(1, 1, 0), (3, 1, 1), (3, 2, 1), (5, 1, 2), (5, 2, 2), (7, 1, 3), (7, 2, 3)])
@pytest.mark.parametrize("n,h,w,dens", [(1, 264, 352, 0.05), (2, 45, 61, 0.02), (1, 8, 8, 0.3)])
def test_conv_footprint_tiles_and_stale(k, s, p, n, h, w, dens):
    ho, wo = mo.conv_out_size(h, w, k, s, p)
    ts = TileMask(n, ho, wo, DEV)
    prev = np.zeros(0, np.int32)
    for step in range(3):       # fresh mask per step: exercises the stale list
        m = np.stack([blob_mask(h, w, dens, seed=1000 * step + 17 * b + k) for b in range(n)])
        ops.build_mask_tiles(_to_dev_mask(m), None, n, h, w, _lib.FOOT_CONV, k, s, p, ts)
        prev = _check_tileset(ts, mo.footprint_conv(m, k, s, p), prev)


@pytest.mark.parametrize("k,s,p", [(1, 1, 0), (3, 1, 1), (3, 2, 1), (5, 1, 2), (5, 2, 2), (7, 1, 3), (3, 1, 0), (5, 2, 1), (3, 1, 2)])
@pytest.mark.parametrize("n,h,w,c,dt,second", [(1, 33, 44, 256, torch.float32, False), (2, 45, 61, 5, torch.float32, True),
                                               (1, 132, 176, 64, torch.bfloat16, True), (4, 264, 352, 4, torch.float32, False),
                                               (1, 66, 88, 24, torch.bfloat16, False), (3, 9, 70, 2, torch.bfloat16, True)])
def test_threshold_mask_footprint_and_lists_in_one_launch(k, s, p, n, h, w, c, dt, second):
    # mie_build_mask_tiles_thresholded against the numpy oracle (threshold mask, union, conv footprint, tile and stale
    # lists) over three steps with fresh deltas: one lane per pixel (c not a multiple of 4) up to 16 lanes per pixel
    # (c = 256), both element types, a second mask OR-ed in, planes whose last tiles are partial, windows with and
    # without padding, 5808 tiles (lists by the separate ranking kernel) and fewer (ticket).  The thresholded input
    # mask comes out as mie_mask_from_delta writes it.
    thr = 0.05
    ho, wo = mo.conv_out_size(h, w, k, s, p)
    ts = TileMask(n, ho, wo, DEV)
    thr_mask = torch.full((n, 1, h, w), 7, dtype=torch.uint8, device=DEV)
    prev = np.zeros(0, np.int32)
    for step in range(3):
        g = torch.Generator().manual_seed(1000 * step + h + c + k)
        d = torch.randn((n, c, h, w), generator=g) * (torch.rand((n, 1, h, w), generator=g) < [0.03, 0.0, 0.3][step])
        d = d * (torch.rand((n, c, h, w), generator=g) < 0.5)              # most channels of an active pixel are zero
        d[0, c - 1, h - 1, w - 1] = 0.051                                   # last channel of the last pixel, just above
        d[0, 0, 0, 0] = 0.049                                               # just below
        d = d.to(dt).float()
        x = ops.as_nhwc(d.to(DEV).to(dt).contiguous(memory_format=torch.channels_last))
        m2 = np.stack([blob_mask(h, w, 0.02, seed=77 * step + b) for b in range(n)]) if second else None
        m2d = _to_dev_mask(m2) if second else None
        _lib.check(_lib.lib().mie_build_mask_tiles_thresholded(
            x.data_ptr(), c, ops.delta_dtype(x), thr, thr_mask.data_ptr(), None if m2d is None else m2d.data_ptr(),
            h, w, k, s, p, ts.ref, torch.cuda.current_stream().cuda_stream))
        torch.cuda.synchronize()
        want_in = mo.pixel_mask(d.numpy(), thr)
        assert np.array_equal(thr_mask[:, 0].cpu().numpy(), want_in), "step %d: thresholded input mask" % step
        src = want_in | m2 if second else want_in
        prev = _check_tileset(ts, mo.footprint_conv(src, k, s, p), prev)


def test_thresholded_build_refuses_footprints_without_a_one_launch_form():
    ts = TileMask(1, 8, 8, DEV)
    x = torch.zeros((1, 16, 16, 4), device=DEV)
    m = torch.zeros((1, 1, 16, 16), dtype=torch.uint8, device=DEV)
    lib = _lib.lib()
    st = torch.cuda.current_stream().cuda_stream
    assert lib.mie_build_mask_tiles_thresholded(x.data_ptr(), 4, _lib.DTYPE_F32, 0.1, m.data_ptr(), None, 16, 16, 1, 2, 0, ts.ref, st) == -2
    assert "no one-launch form" in lib.mie_last_error_string().decode()
    assert lib.mie_build_mask_tiles_thresholded(x.data_ptr(), 4, _lib.DTYPE_F32, 0.1, ts.pixmask.data_ptr(), None, 16, 16, 3, 2, 1, ts.ref, st) == -1
    assert lib.mie_build_mask_tiles_thresholded(x.data_ptr(), 4, _lib.DTYPE_F32, -1.0, m.data_ptr(), None, 16, 16, 3, 2, 1, ts.ref, st) == -1
    assert lib.mie_build_mask_tiles_thresholded(x.data_ptr(), 4, _lib.DTYPE_F32, 0.1, m.data_ptr(), None, 16, 16, 3, 1, 1, ts.ref, st) == -1   # output size
    torch.cuda.synchronize()


def test_all_active_empty_and_union():
    n, h, w = 2, 30, 41
    ts = TileMask(n, h, w, DEV)
    # NULL mask = every pixel active
    ops.build_mask_tiles(None, None, n, h, w, _lib.FOOT_CONV, 3, 1, 1, ts)
    prev = _check_tileset(ts, np.ones((n, h, w), np.uint8))
    assert prev.size == ts.capacity
    # empty mask: no tiles, everything stale
    ops.build_mask_tiles(_to_dev_mask(np.zeros((n, h, w), np.uint8)), None, n, h, w, _lib.FOOT_CONV, 3, 1, 1, ts)
    prev = _check_tileset(ts, np.zeros((n, h, w), np.uint8), prev)
    assert ts.stale_tiles().numel() == ts.capacity
    # union of two masks through a 3x3 footprint
    a = np.stack([blob_mask(h, w, 0.03, seed=5 + b) for b in range(n)])
    b = np.stack([blob_mask(h, w, 0.02, seed=50 + b) for b in range(n)])
    ops.build_mask_tiles(_to_dev_mask(a), _to_dev_mask(b), n, h, w, _lib.FOOT_CONV, 3, 1, 1, ts)
    _check_tileset(ts, mo.footprint_conv(a | b, 3, 1, 1), prev)
    # single pixels at the image corners
    c = np.zeros((n, h, w), np.uint8)
    c[0, 0, 0] = c[1, h - 1, w - 1] = c[0, h - 1, 0] = 1
    ops.build_mask_tiles(_to_dev_mask(c), None, n, h, w, _lib.FOOT_CONV, 1, 1, 0, ts)
    _check_tileset(ts, c)


@pytest.mark.parametrize("n,h,w", [(1, 33, 44), (2, 5, 7), (1, 1, 1)])
def test_up2x_footprint(n, h, w):
    ts = TileMask(n, 2 * h, 2 * w, DEV)
    prev = np.zeros(0, np.int32)
    for step in range(2):
        m = (np.random.default_rng(step + h).random((n, h, w)) < 0.1).astype(np.uint8)
        m[0, 0, 0] = 1
        m[-1, -1, -1] = step
        ops.build_mask_tiles(_to_dev_mask(m), None, n, h, w, _lib.FOOT_UP2X, 0, 0, 0, ts)
        prev = _check_tileset(ts, mo.footprint_up2x(m), prev)


@pytest.mark.parametrize("k,s,p,op", [(3, 2, 1, 1), (4, 2, 1, 0), (5, 2, 2, 1), (2, 2, 0, 0)])
def test_tconv_footprint(k, s, p, op):
    n, h, w = 2, 17, 23
    ho, wo = (h - 1) * s - 2 * p + k + op, (w - 1) * s - 2 * p + k + op
    ts = TileMask(n, ho, wo, DEV)
    m = np.stack([blob_mask(h, w, 0.05, seed=k + b) for b in range(n)])
    ops.build_mask_tiles(_to_dev_mask(m), None, n, h, w, _lib.FOOT_TCONV, k, s, p, ts)
    _check_tileset(ts, mo.footprint_tconv(m, k, s, p, ho, wo))


def test_large_batch_tile_compaction():
    # the batched high-resolution configuration: 8 streams of 480x640 -> 38400 tiles
    n, h, w = 8, 480, 640
    ts = TileMask(n, h, w, DEV)
    prev = np.zeros(0, np.int32)
    for step, dens in enumerate((0.01, 0.20)):
        m = np.stack([blob_mask(h, w, dens, seed=9000 + 10 * step + b) for b in range(n)])
        ops.build_mask_tiles(_to_dev_mask(m), None, n, h, w, _lib.FOOT_CONV, 3, 1, 1, ts)
        prev = _check_tileset(ts, mo.footprint_conv(m, 3, 1, 1), prev)


def test_repeated_builds_are_deterministic():
    n, h, w = 1, 264, 352
    m = blob_mask(h, w, 0.05, seed=77)[None]
    dm = _to_dev_mask(m)
    ts = TileMask(n, h, w, DEV)
    ref = None
    for _ in range(20):
        ops.build_mask_tiles(dm, None, n, h, w, _lib.FOOT_CONV, 5, 1, 2, ts)
        tiles = ts.active_tiles().cpu().numpy()
        if ref is None:
            ref = tiles
        assert np.array_equal(tiles, ref)
        assert ts.stale_tiles().numel() == 0


def test_planner_builds_fresh_tile_sets_after_their_zero_fill():
    # builds on the planning stream must be ordered after the zero-fill of a freshly allocated tile
    # set, and consumers after the build: many fresh tile sets, each used right away
    n, h, w = 1, 64, 96
    m = blob_mask(h, w, 0.1, seed=3)[None]
    dm = _to_dev_mask(m)
    want = mo.footprint_conv(m, 3, 1, 1)
    for rep in range(8):
        junk = torch.full((4096,), 0x7fffffff, dtype=torch.int32, device=DEV)   # recycled by the allocator
        del junk
        with ops.mask_planner(torch.device(DEV)):
            ts = TileMask(n, h, w, DEV)
            ops.build_mask_tiles(dm, None, n, h, w, _lib.FOOT_CONV, 3, 1, 1, ts)
            out = ops.new_nhwc(n, 8, h, w, DEV)
            res = ops.new_nhwc(n, 8, h, w, DEV)
            d = torch.ones(n, 8, h, w, device=DEV).contiguous(memory_format=torch.channels_last)
            ops.act_incr(_lib.ACT_RELU, 0.0, ops.as_nhwc(d), res, out, ts)
        torch.cuda.synchronize()
        _check_tileset(ts, want)
        assert np.array_equal((out[:, 0] != 0).cpu().numpy().astype(np.uint8), want)


def test_out_of_range_counts_are_ignored_by_kernels():
    # counts beyond the capacity (a tile set that was never built) make kernels skip, not read
    n, h, w = 1, 32, 32
    ts = TileMask(n, h, w, DEV)
    ts.counts[_lib.CNT_ACTIVE] = ts.capacity + 7
    ts.tiles.fill_(-1)
    out = torch.full((n, 4, h, w), 5.0, device=DEV).contiguous(memory_format=torch.channels_last)
    res = ops.new_nhwc(n, 4, h, w, DEV)
    ops.act_incr(_lib.ACT_RELU, 0.0, ops.as_nhwc(torch.ones_like(out)), res, ops.as_nhwc(out), ts)
    torch.cuda.synchronize()
    assert torch.count_nonzero(res) == 0
    # a build on top of it recovers a valid list
    ops.build_mask_tiles(None, None, n, h, w, _lib.FOOT_CONV, 1, 1, 0, ts)
    _check_tileset(ts, np.ones((n, h, w), np.uint8))


# ---- mie_build_mask_plan: a chain of builds as one launch ----------------------------------------------------
def _plan_chain(n, h, w):
    """(name, inputs, foot, k, s, p) of a chain that covers every footprint kind the plan has a bitmap form for: same-size
    and shrinking convs, strided convs, unions of two masks, an all-active input, bilinear x2, transposed convs of
    kernel 2 / 3 / 5 at stride 2, an identity footprint, and masks read again long after they were built."""
    c2 = lambda v, k, p: (v + 2 * p - k) // 2 + 1
    h2, w2 = c2(h, 5, 2), c2(w, 5, 2)
    h4, w4 = c2(h2, 3, 1), c2(w2, 3, 1)
    return [
        # name     inputs            foot            k  s  p   output plane
        ("a",      ("x",),           _lib.FOOT_CONV, 5, 1, 2, (h, w)),
        ("b",      ("a",),           _lib.FOOT_CONV, 5, 2, 2, (h2, w2)),
        ("c",      ("b",),           _lib.FOOT_CONV, 3, 1, 1, (h2, w2)),
        ("d",      ("c",),           _lib.FOOT_CONV, 3, 2, 1, (h4, w4)),
        ("e",      ("d", "y4"),      _lib.FOOT_CONV, 7, 1, 3, (h4, w4)),           # union with a mask from memory
        ("f",      ("e",),           _lib.FOOT_UP2X, 0, 0, 0, (2 * h4, 2 * w4)),
        ("g",      ("e",),           _lib.FOOT_TCONV, 3, 2, 1, (2 * h4, 2 * w4)),  # output_padding 1
        ("g5",     ("e",),           _lib.FOOT_TCONV, 5, 2, 2, (2 * h4 - 1, 2 * w4 - 1)),
        ("g2",     ("d",),           _lib.FOOT_TCONV, 2, 2, 0, (2 * h4, 2 * w4)),
        ("u",      ("f", "g"),       _lib.FOOT_CONV, 1, 1, 0, (2 * h4, 2 * w4)),   # union, identity footprint
        ("v",      ("u",),           _lib.FOOT_CONV, 3, 1, 0, (2 * h4 - 2, 2 * w4 - 2)),   # no padding: the plane shrinks
        ("blocks", ("u",),           _lib.FOOT_CONV, 2, 2, 0, (h4, w4)),           # even kernel (block sets of the tconv)
        ("all",    (None,),          _lib.FOOT_CONV, 3, 1, 1, (h, w)),             # NULL mask: every pixel active
        ("late",   ("a", "x"),       _lib.FOOT_CONV, 3, 1, 1, (h, w)),             # first mask of the chain, read last
    ]


def _plan_inputs(n, h, w, step):
    c2 = lambda v, k, p: (v + 2 * p - k) // 2 + 1
    h4, w4 = c2(c2(h, 5, 2), 3, 1), c2(c2(w, 5, 2), 3, 1)
    dens = [0.03, 0.0, 0.2][step % 3]                      # sparse, empty (everything stale), dense
    x = np.stack([blob_mask(h, w, dens, seed=100 * step + b) if dens > 0 else np.zeros((h, w), np.uint8) for b in range(n)])
    y4 = np.stack([blob_mask(h4, w4, 0.05, seed=900 + 100 * step + b) for b in range(n)])
    return {"x": x, "y4": y4}


def _run_chain(chain, sets, inputs_dev, n, planned, wgs=0):
    """Build the chain into `sets` (name -> TileMask): one mie_build_mask_plan call (wgs > 0: mie_build_mask_plan_wgs
    with that cap), or one build per set."""
    shape_of = {name: plane for name, _, _, _, _, _, plane in chain}
    batch = []
    for name, ins, foot, k, s, p, (ho, wo) in chain:
        srcs = [None if i is None else (inputs_dev[i] if i in inputs_dev else sets[i].pixmask) for i in ins]
        hi, wi = (ho, wo) if ins[0] is None else tuple(srcs[0].shape[2:])
        p1 = None if srcs[0] is None else srcs[0].data_ptr()
        p2 = srcs[1].data_ptr() if len(srcs) > 1 else None
        batch.append((p1, p2, hi, wi, foot, k, s, p, sets[name]))
    lib = _lib.lib()
    st = torch.cuda.current_stream().cuda_stream
    if planned:
        arr = ops._plan_ops(batch)
        if wgs:
            _lib.check(lib.mie_build_mask_plan_wgs(arr, len(batch), wgs, st))
        else:
            _lib.check(lib.mie_build_mask_plan(arr, len(batch), st))
    else:
        for p1, p2, hi, wi, foot, k, s, p, out in batch:
            _lib.check(lib.mie_build_mask_tiles(p1, p2, hi, wi, foot, k, s, p, out.ref, st))


@pytest.mark.parametrize("n,h,w", [(1, 264, 352), (1, 70, 94), (3, 37, 53), (2, 128, 160), (1, 33, 44)])
def test_mask_plan_equals_the_builds_it_replaces(n, h, w):
    # one launch for the whole chain against one mie_build_mask_tiles call per set, over three steps with fresh masks
    # (sparse, empty, dense: the stale lists see everything): every buffer of every tile set must match bit for bit,
    # and both match the numpy oracle.  Planes with rows that are multiples of 16 bytes, of 4 bytes and of neither;
    # one sample (lists ranked in the same launch) and several (second kernel).
    chain = _plan_chain(n, h, w)
    mk = lambda: {name: TileMask(n, plane[0], plane[1], DEV) for name, _, _, _, _, _, plane in chain}
    seq, plan = mk(), mk()
    prev = {}
    for step in range(3):
        inputs = _plan_inputs(n, h, w, step)
        dev = {k_: _to_dev_mask(v) for k_, v in inputs.items()}
        _run_chain(chain, seq, dev, n, planned=False)
        _run_chain(chain, plan, dev, n, planned=True)
        torch.cuda.synchronize()
        want = dict(inputs)
        for name, ins, foot, k, s, p, (ho, wo) in chain:
            a, b = seq[name], plan[name]
            na, ns = int(a.counts[0].item()), int(a.counts[1].item())
            tag = "step %d set %s" % (step, name)
            assert torch.equal(a.pixmask, b.pixmask), tag + ": pixel mask"
            assert torch.equal(a.counts, b.counts), tag + ": counts %s vs %s" % (a.counts.tolist(), b.counts.tolist())
            assert torch.equal(a.flags, b.flags), tag + ": flags"
            assert torch.equal(a.tiles[:na], b.tiles[:na]), tag + ": active list"
            assert torch.equal(a.stale[:ns], b.stale[:ns]), tag + ": stale list"
            # and the oracle (the chain restated with numpy)
            if ins[0] is None:
                src = np.ones((n, ho, wo), np.uint8)
            else:
                src = want[ins[0]] if len(ins) == 1 else (want[ins[0]] | want[ins[1]])
            if foot == _lib.FOOT_CONV:
                m = mo.footprint_conv(src, k, s, p)
            elif foot == _lib.FOOT_UP2X:
                m = mo.footprint_up2x(src)
            else:
                m = mo.footprint_tconv(src, k, s, p, ho, wo)
            want[name] = m
            prev[name] = _check_tileset(b, m, prev.get(name))


@pytest.mark.parametrize("n,h,w,wgs", [(1, 264, 352, 1), (1, 264, 352, 3), (4, 240, 320, 4), (4, 240, 320, 9),
                                       (3, 37, 53, 64), (2, 128, 160, 100000)])
def test_mask_plan_held_to_few_workgroups_builds_the_same_sets(n, h, w, wgs):
    # mie_build_mask_plan_wgs: the plan that runs beside other kernels, its first kernel capped at `wgs` workgroups --
    # one per sample, fewer than samples (the cap is then one per sample), an odd share count, and a cap above the
    # default.  Three steps with fresh masks; every buffer of every set bit-equal to the uncapped plan's.
    chain = _plan_chain(n, h, w)
    mk = lambda: {name: TileMask(n, plane[0], plane[1], DEV) for name, _, _, _, _, _, plane in chain}
    full, capped = mk(), mk()
    for step in range(3):
        dev = {k_: _to_dev_mask(v) for k_, v in _plan_inputs(n, h, w, step).items()}
        _run_chain(chain, full, dev, n, planned=True)
        _run_chain(chain, capped, dev, n, planned=True, wgs=wgs)
        torch.cuda.synchronize()
        for name, *_ in chain:
            a, b = full[name], capped[name]
            na, ns = int(a.counts[0].item()), int(a.counts[1].item())
            tag = "step %d set %s" % (step, name)
            assert torch.equal(a.pixmask, b.pixmask), tag + ": pixel mask"
            assert torch.equal(a.counts, b.counts), tag + ": counts"
            assert torch.equal(a.flags, b.flags), tag + ": flags"
            assert torch.equal(a.tiles[:na], b.tiles[:na]), tag + ": active list"
            assert torch.equal(a.stale[:ns], b.stale[:ns]), tag + ": stale list"


def test_mask_plan_of_a_large_plane_and_many_samples():
    # 8 samples of 480x640 (38 400 tiles per set: the lists are ranked by the second kernel, ten blocks per set) and a
    # chain whose masks need more than 64 KB of LDS at once; a device that offers less refuses the plan with
    # MIE_ERR_CAPACITY and launches nothing
    n, h, w = 8, 480, 640
    x = np.stack([blob_mask(h, w, 0.01, seed=7 + b) for b in range(n)])
    xd = _to_dev_mask(x)
    names = [("a", 5, 1, 2, (h, w)), ("b", 5, 2, 2, (240, 320)), ("c", 3, 1, 1, (240, 320))]
    sets = {nm: TileMask(n, pl[0], pl[1], DEV) for nm, _, _, _, pl in names}
    batch, src, hi, wi = [], xd, h, w
    for nm, k, s, p, pl in names:
        batch.append((src.data_ptr(), None, hi, wi, _lib.FOOT_CONV, k, s, p, sets[nm]))
        src, (hi, wi) = sets[nm].pixmask, pl
    batch.append((sets["a"].pixmask.data_ptr(), xd.data_ptr(), h, w, _lib.FOOT_CONV, 3, 1, 1, TileMask(n, h, w, DEV)))
    rc = _lib.lib().mie_build_mask_plan(ops._plan_ops(batch), len(batch), torch.cuda.current_stream().cuda_stream)
    if rc == -3:
        assert "LDS" in _lib.lib().mie_last_error_string().decode()
        pytest.skip("this device offers a workgroup less LDS than the plan needs")
    _lib.check(rc)
    m = x
    for nm, k, s, p, pl in names:
        m = mo.footprint_conv(m, k, s, p)
        _check_tileset(sets[nm], m)
    _check_tileset(batch[-1][-1], mo.footprint_conv(mo.footprint_conv(x, 5, 1, 2) | x, 3, 1, 1))


def test_mask_plan_holds_a_whole_unet_chain_at_full_resolution():
    # The 18 tile sets of E2Depth-incr at 8 x 480 x 640 in ONE plan: four full-resolution bitmaps of 38.4 KB live at
    # its end (head, the up-sampled mask, the last decoder's, their union), which fits a CU's 160 KB only with the LDS
    # slots packed from their lifetimes and the final union written in place over the head's bitmap.  Two steps with
    # different masks (stale lists); every set against the chained mask oracle.
    import mask_chain
    n, h, w = 8, 480, 640
    c2 = lambda v: (v + 4 - 5) // 2 + 1
    planes = [(h, w)]
    for _ in range(3):
        planes.append((c2(planes[-1][0]), c2(planes[-1][1])))
    S = lambda pl: TileMask(n, pl[0], pl[1], DEV)
    sets = {"head": S(planes[0])}
    ops_ = [("head", ("x", None), planes[0], _lib.FOOT_CONV, 5, 1, 2)]
    prev = "head"
    for i in range(3):
        sets["enc%d.conv" % i], sets["enc%d.gates" % i] = S(planes[i + 1]), S(planes[i + 1])
        ops_.append(("enc%d.conv" % i, (prev, None), planes[i], _lib.FOOT_CONV, 5, 2, 2))
        ops_.append(("enc%d.gates" % i, ("enc%d.conv" % i, None), planes[i + 1], _lib.FOOT_CONV, 3, 1, 1))
        prev = "enc%d.gates" % i
    for j in range(2):
        for c in ("conv1", "conv2"):
            name = "res%d.%s" % (j, c)
            sets[name] = S(planes[3])
            ops_.append((name, (prev, None), planes[3], _lib.FOOT_CONV, 3, 1, 1))
            prev = name
    for i in range(3):
        lo, hi = planes[3 - i], planes[2 - i]
        sets["dec%d.up" % i], sets["dec%d.conv" % i] = S(hi), S(hi)
        ops_.append(("dec%d.up" % i, (prev, "enc%d.gates" % (2 - i)), lo, _lib.FOOT_UP2X, 0, 0, 0))
        ops_.append(("dec%d.conv" % i, ("dec%d.up" % i, None), hi, _lib.FOOT_CONV, 5, 1, 2))
        prev = "dec%d.conv" % i
    sets["pred"] = S(planes[0])
    ops_.append(("pred", (prev, "head"), planes[0], _lib.FOOT_CONV, 1, 1, 0))
    assert len(ops_) == 18
    prev_lists = {}
    for step, dens in enumerate((0.01, 0.002)):
        x = np.stack([blob_mask(h, w, dens, seed=40 * step + b) for b in range(n)])
        xd = _to_dev_mask(x)
        ptr = lambda nm: None if nm is None else (xd.data_ptr() if nm == "x" else sets[nm].pixmask.data_ptr())
        batch = [(ptr(a), ptr(b), pl[0], pl[1], foot, k, s, p, sets[name]) for name, (a, b), pl, foot, k, s, p in ops_]
        rc = _lib.lib().mie_build_mask_plan(ops._plan_ops(batch), len(batch), torch.cuda.current_stream().cuda_stream)
        if rc == -3:
            assert "LDS" in _lib.lib().mie_last_error_string().decode()
            pytest.skip("this device offers a workgroup less LDS than the chain needs")
        _lib.check(rc)
        torch.cuda.synchronize()
        want = mask_chain.e2depth_chain(mo.footprint_conv(x, 1, 1, 0))
        for name in sets:
            _check_tileset(sets[name], want[name])
            tiles = mo.tile_list(want[name])
            assert np.array_equal(sets[name].stale_tiles().cpu().numpy(),
                                  mo.stale_list(prev_lists.get(name, np.zeros(0, dtype=np.int32)), tiles)), name
            prev_lists[name] = tiles
