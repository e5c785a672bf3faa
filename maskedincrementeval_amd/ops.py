"""Tensor-level wrappers over the C ABI of libmie_hip.so.

Each function checks shapes / layouts on the host, pulls raw device pointers
and the current HIP stream out of torch, and calls one entry point of
include/mie.h.  torch is used for memory and streams only.
"""
import os
from typing import Optional, Tuple

import torch

from . import _lib
from ._lib import check
from .masked_types import TileMask

# ---- planning pass / compute pass -----------------------------------------------------------------
# A network whose masks depend on the input mask only can be walked twice per step: a planning pass in
# which only the mask builds are launched (onto the planning stream), then a compute pass in which
# only the other kernels are.  All builds are then enqueued -- and, in a captured graph, ordered --
# ahead of the kernels that consume them.  `_phase` is None outside such a walk.
_phase = None
_BUILD_ENTRIES = ("mie_build_mask_tiles",)


class _PhaseLib:
    def __init__(self, real):
        self._real = real

    def __getattr__(self, name):
        fn = getattr(self._real, name)
        if name.startswith("mie_") and name not in ("mie_last_error_string", "mie_tile_capacity", "mie_version",
                                                     "mie_pack_filter"):
            runs = (name in _BUILD_ENTRIES) == (_phase == "plan")
            if not runs:
                return lambda *args: 0
        return fn


def lib():
    real = _lib.lib()
    return real if _phase is None else _PhaseLib(real)


# The builds of a planning pass are not launched one by one: they are collected and handed to the library as
# plans (mie_build_mask_plan: the whole chain of footprints on bitmaps in LDS, two kernels per plan).  A plan the
# library says is too long goes out in halves; a part the library does not take as a plan (a footprint it has no
# bitmap form for, masks too large for LDS) is built set by set as before.  `fused_plan = False` restores one
# mie_build_mask_tiles launch pair per set.  (Measured and not kept: the first one or two builds as a plan of their
# own with an event of their own, so that the first convs run beside the plan of the rest -- every extra dependency
# between the two streams costs 5-10 us of idle time in the replayed graph, more than the overlap wins.)
fused_plan = os.environ.get("MIE_FUSED_PLAN", "1") != "0"
_plan_batch = None       # [(p1, p2, h_in, w_in, foot, k, stride, pad, out TileMask)] while a planning pass collects
_plan_cache = {}         # signature of a batch -> [("plan", ctypes array, n) | ("single", index)] parts


class network_pass:
    """`with network_pass("plan")` / `with network_pass("compute")`: see above."""

    def __init__(self, phase):
        self.phase = phase

    def __enter__(self):
        global _phase, _plan_batch
        self.prev, _phase = _phase, self.phase
        if self.phase == "plan" and fused_plan:
            _plan_batch = []
        return self

    def __exit__(self, *exc):
        global _phase, _plan_batch
        batch, _plan_batch = _plan_batch, None
        try:
            if self.phase == "plan" and batch and exc[0] is None:
                _launch_plan(batch)
        finally:
            _phase = self.prev
        return False


def _plan_ops(batch):
    arr = (_lib.MiePlanOp * len(batch))()
    for op, (p1, p2, h_in, w_in, foot, k, stride, pad, out) in zip(arr, batch):
        op.in_mask, op.in_mask2, op.h_in, op.w_in = p1, p2, h_in, w_in
        op.foot, op.k, op.stride, op.pad = foot, k, stride, pad
        op.out = out.c_struct
    return arr


def _launch_plan(batch):
    """Enqueue the collected builds: on the planning stream when one is active (with the waits and events a
    single build would get), else on the current stream."""
    real = _lib.lib()
    dev = batch[0][-1].device
    side = _planner[0] if (_planner is not None and _planner[1] == dev) else None
    if side is not None:
        fresh = False
        for b in batch:
            root = b[-1].parent if b[-1].parent is not None else b[-1]
            if not root.__dict__.get("built_once"):
                root.built_once = fresh = True
        if fresh:       # freshly allocated tile sets are zero-filled on the compute stream
            ev0 = torch.cuda.Event()
            ev0.record(torch.cuda.current_stream(dev))
            side.wait_event(ev0)
        for b in batch:
            for ptr in b[:2]:
                ev = _pix_ready.get(ptr)
                if ev is not None:
                    side.wait_event(ev)
        stream = side.cuda_stream
    else:
        stream = torch.cuda.current_stream(dev).cuda_stream
    sig = tuple(b[:8] + (b[8].pixmask.data_ptr(), b[8].tiles.data_ptr()) for b in batch) + (_plan_wgs,)
    parts = _plan_cache.get(sig)
    if _plan_wgs:
        build_plan = lambda arr, n: real.mie_build_mask_plan_wgs(arr, n, _plan_wgs, stream)
    else:
        build_plan = lambda arr, n: real.mie_build_mask_plan(arr, n, stream)

    def single(b):
        p1, p2, h_in, w_in, foot, k, stride, pad, out = b
        check(real.mie_build_mask_tiles(p1, p2, h_in, w_in, foot, k, stride, pad, out.ref, stream))

    if parts is None:
        # first use of this batch: find parts the library takes (a refused plan launches nothing)
        parts = []
        todo = [(0, len(batch))]
        while todo:
            lo, hi = todo.pop(0)
            if lo >= hi:
                continue
            arr = _plan_ops(batch[lo:hi])
            rc = build_plan(arr, hi - lo)
            if rc == 0:
                parts.append(("plan", arr, hi - lo, lo))
            elif rc == -3 and hi - lo > 1:               # MIE_ERR_CAPACITY: too long or too much LDS -- halve it
                mid = (lo + hi) // 2
                todo = [(lo, mid), (mid, hi)] + todo
            elif rc in (-2, -3):                          # no bitmap form for this footprint / plane too large
                for i in range(lo, hi):
                    single(batch[i])
                    parts.append(("single", None, 1, i))
            else:
                check(rc)
        _plan_cache[sig] = parts
    else:
        for kind, arr, n_ops, lo in parts:
            if kind == "plan":
                check(build_plan(arr, n_ops))
            else:
                single(batch[lo])
    if side is not None:
        ev = torch.cuda.Event()
        ev.record(side)
        for b in batch:
            root = b[-1].parent if b[-1].parent is not None else b[-1]
            root.ready = ev


# ---- planning one step ahead ---------------------------------------------------------------------
# The tile sets of a step depend on that step's input mask alone, so where the next input is already there (a
# recorded sequence, a batch job, a front end that runs ahead) they can be built while the CURRENT step computes: the
# plan then leaves the critical path altogether.  Two generations of every tile set, pixel mask and delta buffer
# exist for that (`buffer_parity` is part of their keys in _IncrBuffers): the step of parity p reads the sets of
# parity p while the plan of the next step writes those of parity 1 - p.  Reservoirs are shared.  A delta buffer of
# parity p is next written two steps later, under a tile set whose previous build was the one it was last written
# under -- so stale lists stay right -- PROVIDED every plan is followed by its step: a set built twice with no
# compute pass between the builds forgets which tiles still hold data.  run_planned_step therefore refuses a delta that
# is not the one the plan of its parity was made for (same pointer and shape), and plan_step_ahead refuses sets whose
# last plan was never run.  (Under graph capture these checks see the capture order only: replay the captured steps in the
# cyclic order they were captured in.)
buffer_parity = 0
_lookahead_streams = {}
# A plan made ahead runs beside the convs of the step before it and nothing waits for it: it is held to this many
# workgroups (mie_build_mask_plan_wgs), so that the chip stays with the convs.  0: the library's own cap.
LOOKAHEAD_PLAN_WGS = int(os.environ.get("MIE_LOOKAHEAD_PLAN_WGS", "64"))      # tuning knob, read once
_plan_wgs = 0


def _delta_key(t):
    return (t.data_ptr(), tuple(t.shape), t.dtype)


def _check_lookahead_context(parity):
    if _phase is not None or _planner is not None:
        raise RuntimeError("planning one step ahead: not inside a planning pass or a mask_planner block")
    if parity not in (0, 1):
        raise ValueError("parity must be 0 or 1")


def plan_step_ahead(state: dict, parity: int, delta: torch.Tensor, make_mask, walk):
    """Build, on the CURRENT stream, the input mask and every tile set of the step that will run `delta` with
    `parity`.  It writes the buffers of that parity only, so it may run beside the step before it (other parity) --
    but not before the step two back (same parity) has finished, and the step it plans must wait for it: the caller
    orders that with events (pipelined_step does, with a fork and a join; with two streams of one's own, the planning
    stream waits for the event recorded after step k - 1 before planning step k + 1, and the compute stream waits for
    the event recorded after that plan before step k + 1).
    state: a dict the caller keeps per network instance; make_mask(delta) -> the input pixel mask (or None: every
    pixel), written into the parity's buffer; walk(delta, mask) -> one walk of the network."""
    global buffer_parity
    _check_lookahead_context(parity)
    pending = state.setdefault("planned", {})
    if pending.get(parity) is not None:
        raise RuntimeError("planning one step ahead: the step planned for parity %d was never run" % parity)
    global _plan_wgs
    try:
        buffer_parity, _plan_wgs = parity, LOOKAHEAD_PLAN_WGS
        mask = make_mask(delta)
        with network_pass("plan"):
            walk(delta, mask)
        pending[parity] = _delta_key(delta)
    finally:
        buffer_parity = _plan_wgs = 0


def run_planned_step(state: dict, parity: int, delta: torch.Tensor, make_mask, mask_buffer, walk):
    """The compute pass of the step plan_step_ahead planned for (parity, delta), on the current stream.  If nothing was
    planned for this parity (the first step of a sequence) the plan is made here first.  A plan for another delta
    (other pointer or shape) than the one passed is refused.  mask_buffer(delta) -> the parity's input-mask buffer
    without recomputing it."""
    global buffer_parity
    _check_lookahead_context(parity)
    pending = state.setdefault("planned", {})
    try:
        buffer_parity = parity
        if pending.get(parity) == _delta_key(delta):
            mask = mask_buffer(delta)
        elif pending.get(parity) is None:
            mask = make_mask(delta)
            with network_pass("plan"):
                walk(delta, mask)
        else:
            raise RuntimeError("planning one step ahead: the tile sets of parity %d were planned for another delta than "
                               "the one passed now; run the step that was announced as next" % parity)
        pending[parity] = None
        with network_pass("compute"):
            return walk(delta, mask)
    finally:
        buffer_parity = 0


def pipelined_step(state: dict, parity: int, delta: torch.Tensor, next_delta: Optional[torch.Tensor],
                   make_mask, mask_buffer, walk):
    """run_planned_step(parity, delta) with plan_step_ahead(1 - parity, next_delta) forked onto a second stream beside
    it and joined behind it -- one call, and one graph if captured.  (In a captured graph the fork and the join are
    edges between streams, and on this hardware they cost about half of what the overlap gains; two graphs on two
    streams of the caller's, ordered by events between the replays, keep all of it.)"""
    _check_lookahead_context(parity)
    dev = delta.device
    cur = torch.cuda.current_stream(dev)
    pending = state.setdefault("planned", {})
    fork = None
    if next_delta is not None:
        if pending.get(1 - parity) is not None:
            raise RuntimeError("planning one step ahead: the step planned for parity %d was never run" % (1 - parity))
        if pending.get(parity) not in (None, _delta_key(delta)):
            raise RuntimeError("planning one step ahead: the tile sets of parity %d were planned for another delta than "
                               "the one passed now; run the step that was announced as next" % parity)
        fork = torch.cuda.Event()
        fork.record(cur)
    # this step's kernels are enqueued first: the look-ahead depends on none of them
    out = run_planned_step(state, parity, delta, make_mask, mask_buffer, walk)
    if fork is not None:
        side = _lookahead_streams.get(dev)
        if side is None:
            side = _lookahead_streams[dev] = torch.cuda.Stream(dev)
        side.wait_event(fork)                          # fork (joins a graph capture, too)
        with torch.cuda.stream(side):
            plan_step_ahead(state, 1 - parity, next_delta, make_mask, walk)
        ev = torch.cuda.Event()
        ev.record(side)
        cur.wait_event(ev)                             # join
    return out


class LookaheadStepper:
    """The two halves of a planned-ahead step on two streams: step(i, compute, plan_next) runs compute() -- a network's
    forward_planned, or the replay of a graph of it -- on the current stream and plan_next() -- plan_ahead for step
    i + 1, or its graph -- on a planning stream of this object, and keeps the two orderings they need: a step starts
    after its plan has finished, and the plan of step i + 1 starts after step i - 1 has finished (it overwrites that
    step's generation of tile sets).
    host_ordered=True (default): the HOST waits for the two events before it launches -- the step's launch follows the
    plan's event, the plan's launch follows the event of the step before last -- so the GPU queues hold no wait on
    another queue.  The host then runs at most one step ahead of the GPU, which costs nothing while a step takes
    longer than its launch.  host_ordered=False: the same orderings as waits on the GPU (stream.wait_event); measured
    on MI355X such a wait in front of a step costs 10-20 us of idle time even when its event has long fired
    (264x352 frame: 0.533 ms plain, 0.514 with waits on the GPU, 0.503 with the host keeping the order)."""

    def __init__(self, device, host_ordered: bool = True):
        self.device = torch.device(device)
        self.host_ordered = host_ordered
        self.plan_stream = torch.cuda.Stream(self.device)
        self.planned = [torch.cuda.Event(), torch.cuda.Event()]      # by parity: the tile sets of that step are built
        self.computed = [torch.cuda.Event(), torch.cuda.Event()]     # by parity: that step has run

    def step(self, i: int, compute, plan_next=None):
        """Step number i (its parity is i % 2).  plan_next None: nothing is planned ahead (the last step)."""
        cur, p = torch.cuda.current_stream(self.device), i % 2
        if self.host_ordered:
            self.planned[p].synchronize()
        else:
            cur.wait_event(self.planned[p])
        out = compute()
        self.computed[p].record(cur)
        if plan_next is not None:
            if self.host_ordered:
                self.computed[1 - p].synchronize()
            with torch.cuda.stream(self.plan_stream):
                if not self.host_ordered:
                    self.plan_stream.wait_event(self.computed[1 - p])
                plan_next()
                self.planned[1 - p].record(self.plan_stream)
        return out


def require_no_lookahead(net):
    """Called by a network's plain forward: a step that was planned ahead must be run (forward_planned /
    forward_pipelined) or dropped by a refresh first -- a plain step would rebuild tile sets of that plan without a
    compute pass between the two builds, and their stale lists would no longer describe the delta buffers."""
    state = net.__dict__.get("_pipe")
    if state and any(v is not None for v in state.get("planned", {}).values()):
        raise RuntimeError("a step of this network was planned ahead and has not run: run it (forward_planned / "
                           "forward_pipelined) or refresh the reservoirs before stepping plainly")


def drop_lookahead(net):
    """Called by a network's dense refresh: the sequence starts anew.  If a step was planned ahead and never run, its
    tile sets were built without a compute pass behind them, and the next build would no longer know which tiles of
    their delta buffers hold data: every incremental buffer of the network is then put back to the all-zero state
    (pass None as the next delta of the last step before a refresh and nothing has to be zeroed)."""
    state = net.__dict__.pop("_pipe", None)
    if state and any(v is not None for v in state.get("planned", {}).values()):
        for m in net.modules():
            zero = getattr(m, "_zero_incr", None)
            if zero is not None:
                zero()


def _stream(t: torch.Tensor):
    return torch.cuda.current_stream(t.device).cuda_stream


# ---- mask planning on a side stream -------------------------------------------------------------
# The structural masks / tile lists of a network depend on the input mask only, never on the
# values, so their builds can run ahead of the convolutions.  Inside `mask_planner()` every
# mie_build_mask_tiles goes to a second stream (default priority); each tile set carries the
# event of its build and the first kernel that uses it makes the compute stream wait for it.
# Pixel masks written on the compute stream (input mask, refined masks) carry an event the
# other way.  Under HIP-graph capture these waits become edges of the graph.
_planner = None          # (side stream, device) while active
_side_streams = {}
_pix_ready = {}          # data_ptr of a pixel mask written on the compute stream -> event


class mask_planner:
    def __init__(self, device):
        self.device = torch.device(device)

    def __enter__(self):
        global _planner
        if _planner is not None or self.device.type != "cuda":
            self.nested = True
            return self
        self.nested = False
        side = _side_streams.get(self.device)
        if side is None:
            side = torch.cuda.Stream(self.device)
            _side_streams[self.device] = side
        ev = torch.cuda.Event()
        ev.record(torch.cuda.current_stream(self.device))
        side.wait_event(ev)          # forks from the compute stream (also joins a graph capture)
        _planner = (side, self.device)
        return self

    def __exit__(self, *exc):
        global _planner
        if self.nested:
            return False
        side, dev = _planner
        _planner = None
        _pix_ready.clear()
        ev = torch.cuda.Event()
        ev.record(side)
        torch.cuda.current_stream(dev).wait_event(ev)     # join
        return False


def _ready(ts: TileMask):
    """Make the compute stream wait for the build of `ts` (once)."""
    if _phase == "plan":
        return
    root = ts.parent if ts.parent is not None else ts
    ev = root.__dict__.get("ready")
    if ev is not None:
        torch.cuda.current_stream(ts.device).wait_event(ev)
        root.ready = None


def _mark_pix(t: Optional[torch.Tensor], from_values: bool = False):
    """A pixel mask was written on the compute stream: builds that read it must wait."""
    if t is not None and from_values and _phase is not None:
        raise RuntimeError("a mask that depends on values (a delta, refined or quantised deltas) cannot be "
                           "planned ahead: run this network without the planning pass")
    if _phase == "compute":
        return
    if _planner is not None and t is not None:
        ev = torch.cuda.Event()
        ev.record(torch.cuda.current_stream(t.device))
        _pix_ready[t.data_ptr()] = ev


def _require_gpu(t: torch.Tensor, name: str):
    if not t.is_cuda:
        raise RuntimeError("%s must live on the GPU (got %s); this package has no CPU path"
                           % (name, t.device))


_DTYPES = {torch.float32: _lib.DTYPE_F32, torch.bfloat16: _lib.DTYPE_BF16}


def delta_dtype(t: torch.Tensor) -> int:
    """MIE_DTYPE_* code of a delta tensor (fp32 or bf16; reservoirs are always fp32)."""
    try:
        return _DTYPES[t.dtype]
    except KeyError:
        raise ValueError("deltas must be float32 or bfloat16, got %s" % t.dtype) from None


def delta_torch_dtype(t: torch.Tensor):
    """torch dtype a delta travels in: bf16 stays bf16, everything else becomes fp32 (as_nhwc)."""
    return torch.bfloat16 if t.dtype == torch.bfloat16 else torch.float32


def nhwc_ptr(t: Optional[torch.Tensor], name: str, c: Optional[int] = None, dtype=torch.float32):
    """Device pointer of an (N,C,H,W) tensor of `dtype` stored channels_last; None -> NULL."""
    if t is None:
        return None
    _require_gpu(t, name)
    if t.dim() != 4 or t.dtype != dtype:
        raise ValueError("%s must be a 4-D %s tensor, got %s %s" % (name, dtype, tuple(t.shape), t.dtype))
    if not t.permute(0, 2, 3, 1).is_contiguous():
        raise ValueError("%s must be channels_last (NHWC in memory); strides %s" % (name, t.stride()))
    if c is not None and t.shape[1] != c:
        raise ValueError("%s has %d channels, expected %d" % (name, t.shape[1], c))
    return t.data_ptr()


def as_nhwc(t: torch.Tensor) -> torch.Tensor:
    """Return t as channels_last fp32 (bf16 stays bf16); copies only if the layout / dtype differs."""
    if t.dtype not in _DTYPES:
        t = t.float()
    if not t.permute(0, 2, 3, 1).is_contiguous():
        t = t.contiguous(memory_format=torch.channels_last)
        if not t.permute(0, 2, 3, 1).is_contiguous():   # C == 1 corner: force the strides
            t = t.permute(0, 2, 3, 1).contiguous().permute(0, 3, 1, 2)
    return t


def new_nhwc(n, c, h, w, device, dtype=torch.float32) -> torch.Tensor:
    """Zero-filled (N,C,H,W) tensor with NHWC storage."""
    return torch.zeros((n, h, w, c), dtype=dtype, device=device).permute(0, 3, 1, 2)


def pix_ptr(m, n, h, w, name):
    """Device pointer of a pixel mask: None | TileMask | uint8 (N,1,H,W) tensor."""
    if m is None:
        return None
    t = m.pixmask if isinstance(m, TileMask) else m
    if t.dtype != torch.uint8 or tuple(t.shape) != (n, 1, h, w) or not t.is_contiguous():
        raise ValueError("%s must be a contiguous uint8 (%d,1,%d,%d) mask, got %s %s"
                         % (name, n, h, w, tuple(t.shape), t.dtype))
    _require_gpu(t, name)
    if _pending_thr:
        _force_threshold_mask(t)
    return t.data_ptr()


def pixel_mask_of(mask, like: torch.Tensor) -> Optional[torch.Tensor]:
    """Normalise the mask slot of a Masked pair to a uint8 (N,1,H,W) tensor (None = dense)."""
    if mask is None:
        return None
    if isinstance(mask, TileMask):
        return mask.pixmask
    n, _, h, w = like.shape
    m = mask
    if m.dim() != 4 or m.shape[0] != n or m.shape[2] != h or m.shape[3] != w:
        raise ValueError("mask shape %s does not match delta %s" % (tuple(m.shape), tuple(like.shape)))
    # The kernels test mask bytes for non-zero, so a uint8 / bool (N,1,H,W) mask on the device is used
    # as it is: no copy, and the event of whoever wrote it on the compute stream still names it.
    if m.shape[1] == 1 and m.is_contiguous() and m.device == like.device:
        if m.dtype == torch.uint8:
            return m
        if m.dtype == torch.bool:
            return m.view(torch.uint8)
    if m.shape[1] != 1:
        m = m.ne(0).any(dim=1, keepdim=True)
    m = m.ne(0).to(torch.uint8).contiguous().to(like.device)
    _mark_pix(m)          # made on the compute stream: a build on the planning stream must wait for it
    return m


# ---- entry points ----------------------------------------------------------------
def mask_from_delta(delta: torch.Tensor, threshold: float, out: torch.Tensor):
    n, c, h, w = delta.shape
    check(lib().mie_mask_from_delta(nhwc_ptr(delta, "delta", dtype=delta.dtype), n, h, w, c, float(threshold),
                                    pix_ptr(out, n, h, w, "out"), delta_dtype(delta), _stream(delta)))
    _mark_pix(out, from_values=True)
    return out


# Thresholded masks whose kernel has not been launched yet: data pointer of the mask buffer -> (delta, threshold,
# buffer).  threshold_mask_lazy leaves the launch to the first reader of the buffer.  If that reader is the build of a
# conv's tile set, threshold test, footprint and lists go out as one launch (mie_build_mask_tiles_thresholded); any
# other reader (pix_ptr) launches mie_mask_from_delta first.
_pending_thr = {}
fused_threshold_build = os.environ.get("MIE_FUSED_THRESHOLD_BUILD", "1") != "0"      # tuning knob, read once


def threshold_mask_lazy(delta: torch.Tensor, threshold: float, out: torch.Tensor):
    """mask_from_delta(delta, threshold, out) whose launch waits for the first reader of `out` (delta must keep its
    values until then: call this right before the op that reads the mask)."""
    if not fused_threshold_build:
        return mask_from_delta(delta, threshold, out)
    _mark_pix(out, from_values=True)
    _pending_thr[out.data_ptr()] = (delta, float(threshold), out)
    return out


def _force_threshold_mask(t: torch.Tensor):
    ent = _pending_thr.pop(t.data_ptr(), None)
    if ent is not None:
        mask_from_delta(*ent)


def _thresholded_build(in_mask, in_mask2, n, h_in, w_in, foot, k, stride, pad, out: TileMask) -> bool:
    """The one-launch form of a pending threshold mask + the build that reads it, where the library has one."""
    t = in_mask.pixmask if isinstance(in_mask, TileMask) else in_mask
    ent = None if t is None else _pending_thr.get(t.data_ptr())
    if ent is None:
        return False
    delta, thr, buf = ent
    if (foot != _lib.FOOT_CONV or stride + pad > k or 7 * stride + k + max(0, stride - 1 - pad) > 24
            or _phase is not None or (_planner is not None and _planner[1] == out.device)
            or tuple(delta.shape) != (n, delta.shape[1], h_in, w_in)):
        return False
    del _pending_thr[t.data_ptr()]
    p2 = pix_ptr(in_mask2, n, h_in, w_in, "in_mask2")
    check(lib().mie_build_mask_tiles_thresholded(
        nhwc_ptr(delta, "delta", dtype=delta.dtype), delta.shape[1], delta_dtype(delta), thr,
        buf.data_ptr(), p2, h_in, w_in, k, stride, pad, out.ref, _stream(delta)))
    return True


def build_mask_tiles(in_mask, in_mask2, n, h_in, w_in, foot, k, stride, pad, out: TileMask):
    """in_mask / in_mask2: None | TileMask | uint8 (N,1,H,W)."""
    if _pending_thr and _thresholded_build(in_mask, in_mask2, n, h_in, w_in, foot, k, stride, pad, out):
        return out
    p1 = pix_ptr(in_mask, n, h_in, w_in, "in_mask")
    p2 = pix_ptr(in_mask2, n, h_in, w_in, "in_mask2")
    if p1 is None and p2 is not None:   # "all active" OR anything = all active
        p2 = None
    if _phase == "compute":             # built by the planning pass; its event is still attached
        return out
    if _phase == "plan" and _plan_batch is not None:
        _plan_batch.append((p1, p2, h_in, w_in, foot, k, stride, pad, out))
        return out
    if _planner is None or _planner[1] != out.device:
        st = torch.cuda.current_stream(out.device).cuda_stream
        check(lib().mie_build_mask_tiles(p1, p2, h_in, w_in, foot, k, stride, pad, out.ref, st))
        return out
    side = _planner[0]
    root = out.parent if out.parent is not None else out
    if not root.__dict__.get("built_once"):
        # a freshly allocated tile set is zero-filled on the compute stream: its first build
        # on the planning stream must come after that fill
        ev0 = torch.cuda.Event()
        ev0.record(torch.cuda.current_stream(out.device))
        side.wait_event(ev0)
        root.built_once = True
    for ptr in (p1, p2):
        ev = _pix_ready.get(ptr)
        if ev is not None:
            side.wait_event(ev)
    check(lib().mie_build_mask_tiles(p1, p2, h_in, w_in, foot, k, stride, pad, out.ref, side.cuda_stream))
    ev = torch.cuda.Event()
    ev.record(side)
    root.ready = ev
    return out


def pack_filter(filt: torch.Tensor, dtype=torch.float32, x3: bool = False) -> torch.Tensor:
    """Matrix-core copy of a contiguous fp32 [Cin,K,K,Cout] filter in `dtype`, shape
    [Cin/B, K*K, 2, Cout, B/2] with B = 8 (fp32) or 16 (bf16) input channels per block:
    element [b,t,h,co,j] is filt[B*b + (B/2)*h + j, t//K, t%K, co].
    x3=True: the three-term bf16 copy of an fp32 filter (MIE_DTYPE_F32_BF16X3), shape [Cin/16, K*K, 3, 2, Cout, 8]:
    [b,t,0] + [b,t,1] + [b,t,2] is the fp32 weight, each term rounded to bf16."""
    if filt.dim() != 4 or filt.shape[1] != filt.shape[2] or not filt.is_contiguous() or filt.dtype != torch.float32:
        raise ValueError("filter must be contiguous fp32 [Cin,K,K,Cout], got %s" % (tuple(filt.shape),))
    _require_gpu(filt, "filter")
    cin, k, _, cout = filt.shape
    if x3:
        packed = torch.empty((cin // 16, k * k, 3, 2, cout, 8), dtype=torch.bfloat16, device=filt.device)
        check(lib().mie_pack_filter(filt.data_ptr(), cin, k, cout, packed.data_ptr(), _lib.DTYPE_F32_BF16X3, _stream(filt)))
        return packed
    blk = 8 if dtype == torch.float32 else 16
    packed = torch.empty((cin // blk, k * k, 2, cout, blk // 2), dtype=dtype, device=filt.device)
    check(lib().mie_pack_filter(filt.data_ptr(), cin, k, cout, packed.data_ptr(), _DTYPES[dtype], _stream(filt)))
    return packed


# How the matrix-core kernels multiply fp32 deltas: "bf16x3" = every value as three bf16 terms, six term products
# per multiply on the bf16 matrix-core instruction (fp32 accuracy: the three dropped products are at most 2^-23 of
# |x * w|, typically 2^-26, and the measured error against fp64 is 0.6-1.1 times the fp32 instruction's; about twice
# its rate), where the library has that form (mie_conv_f32x3_takes: 3x3 / 5x5 at stride 1 with channel counts in
# multiples of 32, 5x5 at stride 2 in multiples of 16; the stride-2 transposed conv in multiples of 64);
# "native" = v_mfma_f32_32x32x2_f32 everywhere.  Environment variable MIE_F32_MATMUL.
f32_matmul = os.environ.get("MIE_F32_MATMUL", "bf16x3")


def f32x3_takes(k: int, stride: int, c1: int, c2: int, cout: int) -> bool:
    """Whether a conv of this shape on fp32 deltas runs in the three-term bf16 form under the current setting."""
    if f32_matmul != "bf16x3":
        if f32_matmul != "native":
            raise ValueError("ops.f32_matmul must be 'bf16x3' or 'native', not %r" % (f32_matmul,))
        return False
    return bool(lib().mie_conv_f32x3_takes(k, stride, c1, c2, cout))


class ConvFilter:
    """A conv filter as the kernels take it: `plain` [Cin,K,K,Cout] and, when Cin % 8 == 0, `mc`,
    its matrix-core copy (pack_filter).  For bf16 deltas `for_dtype(torch.bfloat16)` gives the
    weights rounded to bf16: as fp32 values for the VALU kernels and as the bf16 matrix-core copy
    (Cin % 16 == 0), both made on first use.  Make a new ConvFilter after every weight update."""

    def __init__(self, plain: torch.Tensor, mc: Optional[torch.Tensor] = None, _packed: bool = False):
        self.plain = plain
        self.mc = mc if _packed else (pack_filter(plain) if plain.is_cuda and plain.shape[0] % 8 == 0 else None)
        self._rows = {}
        self._bf16 = None
        self._x3 = None

    def for_dtype(self, dtype, x3: bool = False):
        """(plain fp32 tensor, matrix-core copy | None) for deltas of `dtype`; x3: the three-term copy for fp32
        deltas (Cin % 16 == 0), made on first use."""
        if dtype == torch.float32:
            if x3 and self.plain.is_cuda and self.plain.shape[0] % 16 == 0:
                if self._x3 is None:
                    self._x3 = pack_filter(self.plain.contiguous(), x3=True)
                return self.plain, self._x3
            return self.plain, self.mc
        if self._bf16 is None:
            rounded = self.plain.to(torch.bfloat16).float().contiguous()
            mc = pack_filter(rounded, torch.bfloat16) if rounded.is_cuda and rounded.shape[0] % 16 == 0 else None
            self._bf16 = (rounded, mc)
        return self._bf16

    @property
    def shape(self):
        return self.plain.shape

    def rows(self, lo: int, hi: int) -> "ConvFilter":
        """The filter of input channels lo..hi-1, made once per range (views of this filter when
        lo and hi are multiples of 8, else a packed copy of its own)."""
        sub = self._rows.get((lo, hi))
        if sub is None:
            plain = self.plain[lo:hi]
            if self.mc is not None and lo % 8 == 0 and hi % 8 == 0:
                sub = ConvFilter(plain, self.mc[lo // 8:hi // 8], _packed=True)
            else:
                sub = ConvFilter(plain)
            self._rows[(lo, hi)] = sub
        return sub


def _filter_args(filt, k, dtype=torch.float32, x3_shape=None, with_code=False):
    """(plain tensor, pointer of the matrix-core copy or None) of a Tensor or ConvFilter; with_code: a third value,
    the MIE_DTYPE_* code of the call.  x3_shape = (stride, c1, c2, cout): fp32 deltas take the three-term bf16 form
    (its filter copy, its code) where the setting (f32_matmul) and the library allow it."""
    mc = None
    code = _DTYPES.get(dtype)
    if isinstance(filt, ConvFilter):
        x3 = (x3_shape is not None and dtype == torch.float32 and filt.plain.shape[0] % 16 == 0
              and f32x3_takes(k, *x3_shape))
        filt, mc = filt.for_dtype(dtype, x3)
        if x3:
            code = _lib.DTYPE_F32_BF16X3
    if filt.dim() != 4 or filt.shape[1] != k or filt.shape[2] != k or not filt.is_contiguous() \
            or filt.dtype != torch.float32:
        raise ValueError("filter must be contiguous fp32 [Cin,%d,%d,Cout], got %s" % (k, k, tuple(filt.shape)))
    _require_gpu(filt, "filter")
    ptr = None if mc is None else mc.data_ptr()
    return (filt, ptr, code) if with_code else (filt, ptr)


# Workspace of the matrix-core conv for planes of very few tiles (a 16x16 plane is 4 tiles, 64 workgroups
# for 512 channels): the library then splits the contraction over up to 8 workgroups per (tile, slab) and
# needs room for their partial sums.  A launch is split only up to 128 workgroups, i.e. up to 4096
# tile-channels, so 8 planes of 4096 * 64 floats (8 MiB) cover every case.  One buffer per device: the
# convs of a device are taken to run on one stream at a time; callers that run convs concurrently on
# several streams pass buffers of their own (`workspace=`), or False for none.
SPLIT_WORKSPACE_BYTES = 8 * 4096 * 64 * 4
split_enabled = True
_split_ws = {}


def split_workspace(device):
    ws = _split_ws.get(device)
    if ws is None:
        ws = _split_ws[device] = torch.empty(SPLIT_WORKSPACE_BYTES // 4, dtype=torch.float32, device=device)
    return ws


def _workspace_args(workspace, small: bool, device):
    """(pointer, bytes) of the split form's workspace: None -> the device's shared buffer where the launch is small
    enough to be split, False -> none."""
    if workspace is None:
        workspace = split_workspace(device) if (split_enabled and small) else False
    if workspace is False:
        return None, 0
    if workspace.dtype != torch.float32 or not workspace.is_contiguous() or workspace.device != device:
        raise ValueError("workspace must be a contiguous fp32 tensor on the device of the operands")
    return workspace.data_ptr(), workspace.numel() * 4


def conv_masked(x, xmask, x2, x2mask, filt, k, stride, pad, out_ts: TileMask, out_delta,
                reservoir=None, act=_lib.ACT_NONE, slope=0.0, path=_lib.PATH_AUTO, addend=None, workspace=None):
    """filt: ConvFilter, or a contiguous fp32 [Cin_total, K, K, Cout] tensor (VALU kernels only).
    workspace: fp32 tensor for the split form of small launches (None: the device's shared one, False: none)."""
    n, c1, h, w = x.shape
    c2 = 0 if x2 is None else x2.shape[1]
    if x2 is not None and (x2.shape[0] != n or x2.shape[2:] != x.shape[2:]):
        raise ValueError("x2 shape %s incompatible with x %s" % (tuple(x2.shape), tuple(x.shape)))
    dt = x.dtype
    # launches the library would split over the contraction (k = 3 or 5, few tiles: see launch_split); at stride 2
    # only the fp32-instruction kernels have that form, and it is worth more there than the three-term arithmetic
    small = k in (3, 5) and out_ts.capacity * (filt.shape[3] // 32) <= 128
    want_split = small and split_enabled and workspace is not False
    x3_shape = (stride, c1, c2, filt.shape[3]) if (path != _lib.PATH_VALU and not (stride == 2 and want_split)) else None
    filt, mc_ptr, code = _filter_args(filt, k, dt, x3_shape, with_code=True)
    cin_total, cout = filt.shape[0], filt.shape[3]
    if tuple(out_delta.shape) != (n, cout, out_ts.h, out_ts.w) or out_ts.n != n:
        raise ValueError("out_delta shape %s, expected %s" % (tuple(out_delta.shape), (n, cout, out_ts.h, out_ts.w)))
    if reservoir is not None and reservoir.shape != out_delta.shape:
        raise ValueError("reservoir shape %s != output %s" % (tuple(reservoir.shape), tuple(out_delta.shape)))
    if addend is not None and addend.shape != out_delta.shape:
        raise ValueError("addend shape %s != output %s" % (tuple(addend.shape), tuple(out_delta.shape)))
    _ready(out_ts)
    # only launches the library would split get the shared buffer
    ws_ptr, ws_bytes = _workspace_args(workspace, small and mc_ptr is not None, x.device)
    check(lib().mie_conv_masked_ws(
        nhwc_ptr(x, "x", dtype=dt), pix_ptr(xmask, n, h, w, "xmask"), c1,
        nhwc_ptr(x2, "x2", dtype=dt), pix_ptr(x2mask, n, h, w, "x2mask"), c2, h, w,
        filt.data_ptr(), mc_ptr, cin_total, k, stride, pad, cout, out_ts.ref,
        nhwc_ptr(out_delta, "out_delta", dtype=dt), nhwc_ptr(addend, "addend", cout, dtype=dt),
        nhwc_ptr(reservoir, "reservoir"), act, float(slope), path, code, ws_ptr, ws_bytes, _stream(x)))
    return out_delta


# Up to which size fp32 decoder layers take the one-kernel form where they run on the fp32 matrix-core instruction
# (see nnConvIncr.forward_fused_upsampled; in the three-term form they always do).
upconv_max_tiles = 2048
upconv_max_chunks = 4


def upconv_takes(c: int, cout: int, k: int, stride: int, pad: int, filt, dtype) -> bool:
    """Whether upconv_masked has a kernel for the shape (else: upsample2x_incr + conv_masked)."""
    return (isinstance(filt, ConvFilter) and k == 5 and stride == 1 and pad == 2 and c % mfma_chunk(dtype) == 0
            and cout % 32 == 0 and filt.for_dtype(dtype)[1] is not None)


def upconv_few_takes(c: int, cout: int, k: int, stride: int, pad: int) -> bool:
    """Whether upconv_masked takes a SINGLE input of c channels through its few-channel kernel (3x3 or 5x5)."""
    return c <= 8 and k in (3, 5) and stride == 1 and pad == k // 2 and cout % 32 == 0


def upconv_masked(a, amask, b, bmask, filt, k, pad, out_ts: TileMask, out_delta, reservoir=None,
                  act=_lib.ACT_NONE, slope=0.0, addend=None, workspace=None):
    """conv over up2x(a + b) in one kernel; a, b at half the resolution of out_ts (b may be None): 5x5 for inputs in
    whole matrix-core chunks, 3x3 or 5x5 for a single input of at most 8 channels.  workspace: as in conv_masked."""
    n, c, h, w = a.shape
    dt = a.dtype
    if b is not None and (b.shape != a.shape or b.dtype != dt):
        raise ValueError("b %s %s does not match a %s %s" % (tuple(b.shape), b.dtype, tuple(a.shape), dt))
    plain, mc_ptr, code = _filter_args(filt, k, dt, (1, c, 0, filt.shape[3]) if (k == 5 and c > 8) else None,
                                       with_code=True)
    cin_total, cout = plain.shape[0], plain.shape[3]
    if tuple(out_delta.shape) != (n, cout, 2 * h, 2 * w) or out_ts.n != n:
        raise ValueError("out_delta shape %s, expected %s" % (tuple(out_delta.shape), (n, cout, 2 * h, 2 * w)))
    if reservoir is not None and reservoir.shape != out_delta.shape:
        raise ValueError("reservoir shape %s != output %s" % (tuple(reservoir.shape), tuple(out_delta.shape)))
    _ready(out_ts)
    ws_ptr, ws_bytes = _workspace_args(workspace, c > 8 and mc_ptr is not None and out_ts.capacity * (cout // 32) <= 128, a.device)
    check(lib().mie_upconv_masked_ws(
        nhwc_ptr(a, "a", dtype=dt), pix_ptr(amask, n, h, w, "amask"), nhwc_ptr(b, "b", dtype=dt),
        pix_ptr(bmask, n, h, w, "bmask"), c, h, w, plain.data_ptr(), mc_ptr, cin_total, k, pad, cout, out_ts.ref,
        nhwc_ptr(out_delta, "out_delta", dtype=dt), nhwc_ptr(addend, "addend", cout, dtype=dt),
        nhwc_ptr(reservoir, "reservoir"), act, float(slope), code, ws_ptr, ws_bytes, _stream(a)))
    return out_delta


# Planes the fused tail kernel takes (the persistent last-decoder kernel: tiles of the whole batch).
UPCONV_PRED_MIN_TILES, UPCONV_PRED_MAX_TILES = 2048, 1 << 20
upconv_pred_enabled = os.environ.get("MIE_UPCONV_PRED", "1") != "0"


def upconv_pred_takes(c: int, cout: int, k: int, stride: int, pad: int, filt, dtype, tiles: int, act: int) -> bool:
    """Whether upconv_pred_masked has a kernel for this last-decoder shape (else: upconv_masked + conv_masked)."""
    return (upconv_pred_enabled and dtype == torch.bfloat16 and c == 64 and cout == 32 and k == 5 and stride == 1
            and pad == 2 and UPCONV_PRED_MIN_TILES <= tiles <= UPCONV_PRED_MAX_TILES
            and act in (_lib.ACT_NONE, _lib.ACT_RELU, _lib.ACT_LEAKY_RELU)
            and isinstance(filt, ConvFilter) and filt.for_dtype(dtype)[1] is not None)


def upconv_pred_masked(a, amask, b, bmask, filt, out_ts: TileMask, reservoir, act, slope, skip, skip_mask, pred_w,
                       pred_res, pred_act, pred_slope, pred_out):
    """Last decoder (5x5 conv over up2x(a + b), 64 -> 32 bf16 channels, reservoir + activation) with the 1x1
    prediction conv over (its increment + skip), the prediction's reservoir and activation increment in its epilogue.
    out_ts: the prediction's tile set; pred_w: fp32 [2, 32] (weights of the increment, of skip); pred_res fp32 and
    pred_out bf16, both (N, 1, 2H, 2W)."""
    n, c, h, w = a.shape
    dt = a.dtype
    if b is not None and (b.shape != a.shape or b.dtype != dt):
        raise ValueError("b %s %s does not match a %s %s" % (tuple(b.shape), b.dtype, tuple(a.shape), dt))
    plain, mc_ptr, code = _filter_args(filt, 5, dt, None, with_code=True)
    cin_total, cout = plain.shape[0], plain.shape[3]
    full = (n, cout, 2 * h, 2 * w)
    if tuple(reservoir.shape) != full or tuple(skip.shape) != full or skip.dtype != dt:
        raise ValueError("reservoir %s / skip %s %s, expected %s %s" % (tuple(reservoir.shape), tuple(skip.shape), skip.dtype, full, dt))
    if tuple(pred_res.shape) != (n, 1, 2 * h, 2 * w) or tuple(pred_out.shape) != (n, 1, 2 * h, 2 * w) or pred_out.dtype != dt:
        raise ValueError("prediction buffers must be (%d, 1, %d, %d)" % (n, 2 * h, 2 * w))
    if pred_w.dtype != torch.float32 or tuple(pred_w.shape) != (2, cout) or not pred_w.is_contiguous():
        raise ValueError("pred_w must be contiguous fp32 (2, %d)" % cout)
    _require_gpu(pred_w, "pred_w")
    _ready(out_ts)
    check(lib().mie_upconv_pred_masked(
        nhwc_ptr(a, "a", dtype=dt), pix_ptr(amask, n, h, w, "amask"), nhwc_ptr(b, "b", dtype=dt),
        pix_ptr(bmask, n, h, w, "bmask"), c, h, w, plain.data_ptr(), mc_ptr, cin_total, cout, out_ts.ref,
        nhwc_ptr(reservoir, "reservoir"), act, float(slope), nhwc_ptr(skip, "skip", dtype=dt),
        pix_ptr(skip_mask, n, 2 * h, 2 * w, "skip_mask"), pred_w.data_ptr(), nhwc_ptr(pred_res, "pred_res"), pred_act,
        float(pred_slope), nhwc_ptr(pred_out, "pred_out", dtype=dt), code, _stream(a)))
    return pred_out


def conv_refresh(x, x2, filt, bias, k, stride, pad, out_ts: TileMask, out_dense, reservoir=None,
                 act=_lib.ACT_NONE, slope=0.0, path=_lib.PATH_AUTO, addend=None):
    """Dense conv + bias (+ activation, + reservoir fill) over the tiles of out_ts (all active)."""
    n, c1, h, w = x.shape
    c2 = 0 if x2 is None else x2.shape[1]
    dt = x.dtype
    filt, mc_ptr, code = _filter_args(filt, k, dt, (stride, c1, c2, filt.shape[3]) if path != _lib.PATH_VALU else None,
                                      with_code=True)
    cin_total, cout = filt.shape[0], filt.shape[3]
    if tuple(out_dense.shape) != (n, cout, out_ts.h, out_ts.w):
        raise ValueError("out_dense shape %s, expected %s" % (tuple(out_dense.shape), (n, cout, out_ts.h, out_ts.w)))
    if bias is not None and (bias.numel() != cout or bias.dtype != torch.float32 or not bias.is_contiguous()):
        raise ValueError("bias must be contiguous fp32 of %d elements" % cout)
    _ready(out_ts)
    check(lib().mie_conv_refresh(
        nhwc_ptr(x, "x", dtype=dt), c1, nhwc_ptr(x2, "x2", dtype=dt), c2, h, w, filt.data_ptr(), mc_ptr,
        cin_total, k, stride, pad, cout, None if bias is None else bias.data_ptr(), out_ts.ref,
        nhwc_ptr(out_dense, "out_dense", dtype=dt), nhwc_ptr(addend, "addend", cout, dtype=dt),
        nhwc_ptr(reservoir, "reservoir"), act, float(slope), path, code, _stream(x)))
    return out_dense


def tconv_masked(x, xmask, filt, k, stride, pad, out_ts: TileMask, out_delta, reservoir=None,
                 act=_lib.ACT_NONE, slope=0.0):
    """filt: ConvTranspose2d weight permuted to [Cin, K, K, Cout], contiguous fp32 (tensor or ConvFilter)."""
    n, cin, h, w = x.shape
    if isinstance(filt, ConvFilter):
        filt = filt.for_dtype(x.dtype)[0]
    if filt.dim() != 4 or filt.shape[0] != cin or filt.shape[1] != k or not filt.is_contiguous():
        raise ValueError("filter must be contiguous [Cin,%d,%d,Cout], got %s" % (k, k, tuple(filt.shape)))
    _require_gpu(filt, "filter")
    cout = filt.shape[3]
    if tuple(out_delta.shape) != (n, cout, out_ts.h, out_ts.w):
        raise ValueError("out_delta shape %s" % (tuple(out_delta.shape),))
    _ready(out_ts)
    check(lib().mie_tconv_masked(
        nhwc_ptr(x, "x", dtype=x.dtype), pix_ptr(xmask, n, h, w, "xmask"), cin, h, w, filt.data_ptr(), k, stride,
        pad, cout, out_ts.ref, nhwc_ptr(out_delta, "out_delta", dtype=x.dtype), nhwc_ptr(reservoir, "reservoir"),
        act, float(slope), delta_dtype(x), _stream(x)))
    return out_delta


def tconv_refresh(x, filt, bias, k, stride, pad, out_ts: TileMask, out_dense, reservoir=None,
                  act=_lib.ACT_NONE, slope=0.0):
    """Dense transposed conv + bias (+ activation, + reservoir fill) over the tiles of out_ts (all active)."""
    n, cin, h, w = x.shape
    if isinstance(filt, ConvFilter):
        filt = filt.for_dtype(x.dtype)[0]
    if filt.dim() != 4 or filt.shape[0] != cin or filt.shape[1] != k or not filt.is_contiguous():
        raise ValueError("filter must be contiguous [Cin,%d,%d,Cout], got %s" % (k, k, tuple(filt.shape)))
    _require_gpu(filt, "filter")
    cout = filt.shape[3]
    if tuple(out_dense.shape) != (n, cout, out_ts.h, out_ts.w):
        raise ValueError("out_dense shape %s" % (tuple(out_dense.shape),))
    if bias is not None and (bias.numel() != cout or bias.dtype != torch.float32 or not bias.is_contiguous()):
        raise ValueError("bias must be contiguous fp32 of %d elements" % cout)
    _ready(out_ts)
    check(lib().mie_tconv_refresh(
        nhwc_ptr(x, "x", dtype=x.dtype), cin, h, w, filt.data_ptr(), k, stride, pad, cout,
        None if bias is None else bias.data_ptr(), out_ts.ref, nhwc_ptr(out_dense, "out_dense", dtype=x.dtype),
        nhwc_ptr(reservoir, "reservoir"), act, float(slope), delta_dtype(x), _stream(x)))
    return out_dense


def tconv2x_takes(c1: int, c2: int, cout: int, k: int, stride: int, pad: int, out_pad: int, filt, dtype) -> bool:
    """Whether tconv2x_masked has a kernel for the layer: stride 2, k in {3, 5}, pad k // 2, output_padding 1,
    input channels in whole staging chunks, cout % 32 == 0 and a matrix-core filter copy."""
    chunk = mfma_chunk(dtype)
    return (isinstance(filt, ConvFilter) and k in (3, 5) and stride == 2 and pad == k // 2 and out_pad == 1
            and c1 % chunk == 0 and c2 % chunk == 0 and cout % 32 == 0 and filt.for_dtype(dtype)[1] is not None)


def _tconv2x_args(x, x2, filt, k, out_ts, block_ts, out, addend, reservoir):
    n, c1, h, w = x.shape
    c2 = 0 if x2 is None else x2.shape[1]
    if x2 is not None and (x2.shape[0] != n or x2.shape[2:] != x.shape[2:] or x2.dtype != x.dtype):
        raise ValueError("x2 %s incompatible with x %s" % (tuple(x2.shape), tuple(x.shape)))
    # fp32 deltas in the three-term bf16 form where the setting asks for it and the channel counts are whole chunks of 64
    # (the same conditions under which ConvFilter.for_dtype hands out the three-term copy: else the fp32 copy and code)
    x3 = (x.dtype == torch.float32 and isinstance(filt, ConvFilter) and f32_matmul == "bf16x3"
          and c1 % 64 == 0 and c2 % 64 == 0 and filt.shape[3] % 32 == 0
          and filt.plain.is_cuda and filt.plain.shape[0] % 16 == 0)
    if x3:
        plain, mc = filt.for_dtype(torch.float32, x3=True)
        mc_ptr, code = mc.data_ptr(), _lib.DTYPE_F32_BF16X3
    else:
        plain, mc_ptr = _filter_args(filt, k, x.dtype)
        code = delta_dtype(x)
    cin_total, cout = plain.shape[0], plain.shape[3]
    if mc_ptr is None:
        raise ValueError("tconv2x needs a ConvFilter with a matrix-core copy")
    if tuple(out.shape) != (n, cout, 2 * h, 2 * w) or (out_ts.n, out_ts.h, out_ts.w) != (n, 2 * h, 2 * w) \
            or (block_ts.n, block_ts.h, block_ts.w) != (n, h, w):
        raise ValueError("output %s / tile sets do not match twice the input %s" % (tuple(out.shape), tuple(x.shape)))
    for name, t in (("addend", addend), ("reservoir", reservoir)):
        if t is not None and t.shape != out.shape:
            raise ValueError("%s shape %s != output %s" % (name, tuple(t.shape), tuple(out.shape)))
    return n, c1, c2, h, w, plain, mc_ptr, cin_total, cout, code


def tconv2x_masked(x, xmask, x2, x2mask, filt, k, out_ts: TileMask, block_ts: TileMask, out_delta, reservoir=None,
                   act=_lib.ACT_NONE, slope=0.0, addend=None, workspace=None):
    """Stride-2 transposed conv (k in {3, 5}, pad k // 2, output twice the input) of x ++ x2 on the matrix
    cores.  out_ts: MIE_FOOT_TCONV tile set of the output; block_ts: tile set of the 16x16 output blocks at
    input resolution (build_mask_tiles(out_ts, None, ..., FOOT_CONV, 2, 2, 0, block_ts)).
    workspace: as in conv_masked (None: the device's shared one when the plane is small, False: none)."""
    n, c1, c2, h, w, plain, mc_ptr, cin_total, cout, code = _tconv2x_args(x, x2, filt, k, out_ts, block_ts, out_delta,
                                                                    addend, reservoir)
    dt = x.dtype
    _ready(out_ts)
    _ready(block_ts)
    if workspace is None:
        workspace = split_workspace(x.device) if (split_enabled and block_ts.capacity * (cout // 32) <= 128) else False
    ws_ptr, ws_bytes = (None, 0) if workspace is False else (workspace.data_ptr(), workspace.numel() * 4)
    check(lib().mie_tconv2x_masked(
        nhwc_ptr(x, "x", dtype=dt), pix_ptr(xmask, n, h, w, "xmask"), c1, nhwc_ptr(x2, "x2", dtype=dt),
        pix_ptr(x2mask, n, h, w, "x2mask"), c2, h, w, plain.data_ptr(), mc_ptr, cin_total, k, cout, out_ts.ref,
        block_ts.ref, nhwc_ptr(out_delta, "out_delta", dtype=dt), nhwc_ptr(addend, "addend", cout, dtype=dt),
        nhwc_ptr(reservoir, "reservoir"), act, float(slope), code, ws_ptr, ws_bytes, _stream(x)))
    return out_delta


def tconv2x_refresh(x, x2, filt, bias, k, out_ts: TileMask, block_ts: TileMask, out_dense, reservoir=None,
                    act=_lib.ACT_NONE, slope=0.0, addend=None):
    """Dense twin of tconv2x_masked (both tile sets all active): bias, activation and reservoir fill fused."""
    n, c1, c2, h, w, plain, mc_ptr, cin_total, cout, code = _tconv2x_args(x, x2, filt, k, out_ts, block_ts, out_dense,
                                                                    addend, reservoir)
    dt = x.dtype
    if bias is not None and (bias.numel() != cout or bias.dtype != torch.float32 or not bias.is_contiguous()):
        raise ValueError("bias must be contiguous fp32 of %d elements" % cout)
    _ready(out_ts)
    _ready(block_ts)
    check(lib().mie_tconv2x_refresh(
        nhwc_ptr(x, "x", dtype=dt), c1, nhwc_ptr(x2, "x2", dtype=dt), c2, h, w, plain.data_ptr(), mc_ptr, cin_total, k,
        cout, None if bias is None else bias.data_ptr(), out_ts.ref, block_ts.ref,
        nhwc_ptr(out_dense, "out_dense", dtype=dt), nhwc_ptr(addend, "addend", cout, dtype=dt),
        nhwc_ptr(reservoir, "reservoir"), act, float(slope), code, _stream(x)))
    return out_dense


def _same_shape(name, t, ref):
    if t.shape != ref.shape:
        raise ValueError("%s shape %s != %s" % (name, tuple(t.shape), tuple(ref.shape)))


def act_incr(kind, slope, in_delta, reservoir, out_delta, ts: TileMask, out_pixmask=None,
             keep_reservoir=False):
    n, c, h, w = in_delta.shape
    _same_shape("reservoir", reservoir, in_delta)
    _same_shape("out_delta", out_delta, in_delta)
    if (ts.n, ts.h, ts.w) != (n, h, w):
        raise ValueError("tile set %s does not match delta %s" % ((ts.n, ts.h, ts.w), (n, h, w)))
    _ready(ts)
    dt = in_delta.dtype
    check(lib().mie_act_incr(kind, float(slope), nhwc_ptr(in_delta, "in_delta", dtype=dt),
                             nhwc_ptr(reservoir, "reservoir"), nhwc_ptr(out_delta, "out_delta", dtype=dt), c,
                             ts.ref, pix_ptr(out_pixmask, n, h, w, "out_pixmask"),
                             _lib.FLAG_KEEP_RESERVOIR if keep_reservoir else 0, delta_dtype(in_delta),
                             _stream(in_delta)))
    _mark_pix(out_pixmask, from_values=True)
    return out_delta


def kfence_incr(in_delta, carry, k, out_delta, ts: TileMask, out_pixmask=None):
    """k: positive float, or a 1-element fp32 device tensor read by the kernel."""
    n, c, h, w = in_delta.shape
    _same_shape("carry", carry, in_delta)
    _same_shape("out_delta", out_delta, in_delta)
    if (ts.n, ts.h, ts.w) != (n, h, w):
        raise ValueError("tile set %s does not match delta %s" % ((ts.n, ts.h, ts.w), (n, h, w)))
    if isinstance(k, torch.Tensor):
        if k.numel() != 1 or k.dtype != torch.float32:
            raise ValueError("k must be a float or a 1-element fp32 tensor")
        _require_gpu(k, "k")
        k_dev, k_host = k.data_ptr(), 0.0
    else:
        k_dev, k_host = None, float(k)
    _ready(ts)
    dt = in_delta.dtype
    check(lib().mie_kfence_incr(nhwc_ptr(in_delta, "in_delta", dtype=dt), nhwc_ptr(carry, "carry"), k_dev, k_host,
                                nhwc_ptr(out_delta, "out_delta", dtype=dt), c, ts.ref,
                                pix_ptr(out_pixmask, n, h, w, "out_pixmask"), delta_dtype(in_delta),
                                _stream(in_delta)))
    _mark_pix(out_pixmask, from_values=True)
    return out_delta


def mul_incr(d1, m1, r1, d2, m2, r2, out_delta, ts: TileMask, keep_reservoir=False):
    n, c, h, w = d1.shape
    for name, t in (("r1", r1), ("d2", d2), ("r2", r2), ("out_delta", out_delta)):
        _same_shape(name, t, d1)
    _ready(ts)
    dt = d1.dtype
    check(lib().mie_mul_incr(nhwc_ptr(d1, "d1", dtype=dt), pix_ptr(m1, n, h, w, "m1"), nhwc_ptr(r1, "r1"),
                             nhwc_ptr(d2, "d2", dtype=dt), pix_ptr(m2, n, h, w, "m2"), nhwc_ptr(r2, "r2"),
                             nhwc_ptr(out_delta, "out_delta", dtype=dt), c, ts.ref,
                             _lib.FLAG_KEEP_RESERVOIR if keep_reservoir else 0, delta_dtype(d1), _stream(d1)))
    return out_delta


def add_incr(a, ma, b, mb, out_delta, ts: TileMask):
    n, c, h, w = a.shape
    _same_shape("b", b, a)
    _same_shape("out_delta", out_delta, a)
    _ready(ts)
    dt = a.dtype
    check(lib().mie_add_incr(nhwc_ptr(a, "a", dtype=dt), pix_ptr(ma, n, h, w, "ma"), nhwc_ptr(b, "b", dtype=dt),
                             pix_ptr(mb, n, h, w, "mb"), nhwc_ptr(out_delta, "out_delta", dtype=dt), c,
                             ts.ref, delta_dtype(a), _stream(a)))
    return out_delta


def maxpool_incr(in_delta, in_mask, reservoir, k, stride, pad, out_ts: TileMask, out_delta):
    """out_delta = maxpool(reservoir + in_delta) - maxpool(reservoir); the reservoir is only read."""
    n, c, h, w = in_delta.shape
    _same_shape("reservoir", reservoir, in_delta)
    dt = in_delta.dtype
    _ready(out_ts)
    check(lib().mie_maxpool_incr(nhwc_ptr(in_delta, "in_delta", dtype=dt), pix_ptr(in_mask, n, h, w, "in_mask"),
                                 nhwc_ptr(reservoir, "reservoir"), h, w, c, k, stride, pad, out_ts.ref,
                                 nhwc_ptr(out_delta, "out_delta", c, dtype=dt), delta_dtype(in_delta),
                                 _stream(in_delta)))
    return out_delta


def accumulate(in_delta, reservoir, ts: TileMask):
    """reservoir += in_delta at the active pixels of ts."""
    n, c, h, w = in_delta.shape
    _same_shape("reservoir", reservoir, in_delta)
    _ready(ts)
    check(lib().mie_accumulate(nhwc_ptr(in_delta, "in_delta", dtype=in_delta.dtype), nhwc_ptr(reservoir, "reservoir"),
                               c, ts.ref, delta_dtype(in_delta), _stream(in_delta)))
    return reservoir


def scale_incr(in_delta, scale, out_delta, ts: TileMask):
    """out = in * scale[c] over the active tiles of ts (eval-mode batch norm on a delta); in place allowed."""
    n, c, h, w = in_delta.shape
    _same_shape("out_delta", out_delta, in_delta)
    if scale.dtype != torch.float32 or scale.numel() != c or not scale.is_contiguous():
        raise ValueError("scale must be contiguous fp32 [%d]" % c)
    _require_gpu(scale, "scale")
    _ready(ts)
    dt = in_delta.dtype
    check(lib().mie_scale_incr(nhwc_ptr(in_delta, "in_delta", dtype=dt), scale.data_ptr(),
                               nhwc_ptr(out_delta, "out_delta", c, dtype=dt), c, ts.ref, delta_dtype(in_delta),
                               _stream(in_delta)))
    return out_delta


def avgpool_incr(in_delta, in_mask, out_delta):
    """Adaptive average pooling of a delta to the spatial size of out_delta; masked pixels are not read."""
    n, c, h, w = in_delta.shape
    if out_delta.shape[:2] != in_delta.shape[:2] or out_delta.dtype != in_delta.dtype:
        raise ValueError("out_delta %s does not match the input %s" % (tuple(out_delta.shape), tuple(in_delta.shape)))
    ho, wo = out_delta.shape[2:]
    dt = in_delta.dtype
    check(lib().mie_avgpool_incr(nhwc_ptr(in_delta, "in_delta", dtype=dt), pix_ptr(in_mask, n, h, w, "in_mask"),
                                 n, h, w, c, ho, wo, nhwc_ptr(out_delta, "out_delta", c, dtype=dt),
                                 delta_dtype(in_delta), _stream(in_delta)))
    return out_delta


def linear_incr(in_delta, weight_t, out_delta):
    """out[n, o] = sum_i in[n, i] * W[o, i] with weight_t = W.t().contiguous() (fp32 [f_in, f_out])."""
    if in_delta.dim() != 2 or not in_delta.is_contiguous() or out_delta.dim() != 2 or not out_delta.is_contiguous():
        raise ValueError("linear_incr takes contiguous 2-D deltas")
    _require_gpu(in_delta, "in_delta"), _require_gpu(weight_t, "weight_t"), _require_gpu(out_delta, "out_delta")
    n, f_in = in_delta.shape
    if weight_t.dtype != torch.float32 or not weight_t.is_contiguous() or weight_t.shape[0] != f_in:
        raise ValueError("weight_t must be contiguous fp32 [%d, f_out], got %s" % (f_in, tuple(weight_t.shape)))
    f_out = weight_t.shape[1]
    if tuple(out_delta.shape) != (n, f_out) or out_delta.dtype != in_delta.dtype:
        raise ValueError("out_delta must be %s of %s" % ((n, f_out), in_delta.dtype))
    check(lib().mie_linear_incr(in_delta.data_ptr(), n, f_in, weight_t.data_ptr(), f_out, out_delta.data_ptr(),
                                delta_dtype(in_delta), _stream(in_delta)))
    return out_delta


def upsample2x_incr(a, ma, b, mb, out_ts: TileMask, out_delta):
    n, c, h, w = a.shape
    if b is not None:
        _same_shape("b", b, a)
    if tuple(out_delta.shape) != (n, c, 2 * h, 2 * w):
        raise ValueError("out_delta shape %s, expected %s" % (tuple(out_delta.shape), (n, c, 2 * h, 2 * w)))
    _ready(out_ts)
    dt = a.dtype
    check(lib().mie_upsample2x_incr(nhwc_ptr(a, "a", dtype=dt), pix_ptr(ma, n, h, w, "ma"),
                                    nhwc_ptr(b, "b", dtype=dt), pix_ptr(mb, n, h, w, "mb"), h, w, c,
                                    out_ts.ref, nhwc_ptr(out_delta, "out_delta", dtype=dt), delta_dtype(a),
                                    _stream(a)))
    return out_delta


def upsample2x_pair_incr(a0, m0, ts0: TileMask, out0, a1, m1, ts1: TileMask, out1):
    """Two up-samplings of the same geometry in one launch (own input, mask, tile set and output each)."""
    n, c, h, w = a0.shape
    _same_shape("a1", a1, a0)
    for name, o in (("out0", out0), ("out1", out1)):
        if tuple(o.shape) != (n, c, 2 * h, 2 * w):
            raise ValueError("%s shape %s, expected %s" % (name, tuple(o.shape), (n, c, 2 * h, 2 * w)))
    _ready(ts0)
    _ready(ts1)
    dt = a0.dtype
    if a1.dtype != dt:
        raise ValueError("the two inputs differ in dtype")
    check(lib().mie_upsample2x_pair_incr(
        nhwc_ptr(a0, "a0", dtype=dt), pix_ptr(m0, n, h, w, "m0"), ts0.ref, nhwc_ptr(out0, "out0", dtype=dt),
        nhwc_ptr(a1, "a1", dtype=dt), pix_ptr(m1, n, h, w, "m1"), ts1.ref, nhwc_ptr(out1, "out1", dtype=dt),
        h, w, c, delta_dtype(a0), _stream(a0)))
    return out0, out1


def convlstm_gates_incr(gates_delta, gates_res, cprev_delta, cprev_mask, cprev_res, cell_res,
                        h_delta, c_delta, ts: TileMask):
    n, c4, h, w = gates_delta.shape
    hid = c4 // 4
    if c4 != 4 * hid:
        raise ValueError("gates tensor needs 4*hid channels, got %d" % c4)
    _same_shape("gates_res", gates_res, gates_delta)
    for name, t in (("cprev_res", cprev_res), ("cell_res", cell_res), ("h_delta", h_delta),
                    ("c_delta", c_delta)):
        if tuple(t.shape) != (n, hid, h, w):
            raise ValueError("%s shape %s, expected %s" % (name, tuple(t.shape), (n, hid, h, w)))
    _ready(ts)
    dt = gates_delta.dtype
    check(lib().mie_convlstm_gates_incr(
        nhwc_ptr(gates_delta, "gates_delta", dtype=dt), nhwc_ptr(gates_res, "gates_res"),
        nhwc_ptr(cprev_delta, "cprev_delta", dtype=dt), pix_ptr(cprev_mask, n, h, w, "cprev_mask"),
        nhwc_ptr(cprev_res, "cprev_res"), nhwc_ptr(cell_res, "cell_res"),
        nhwc_ptr(h_delta, "h_delta", dtype=dt), nhwc_ptr(c_delta, "c_delta", dtype=dt), hid, ts.ref,
        delta_dtype(gates_delta), _stream(gates_delta)))
    return h_delta, c_delta


def convgru_gates_incr(gates_delta, update_res, cand_res, h_delta, ts: TileMask):
    """ConvGRU gate math on the stacked [update | candidate] conv delta; reservoirs updated in place."""
    n, c2, h, w = gates_delta.shape
    hid = c2 // 2
    if c2 != 2 * hid:
        raise ValueError("gates tensor needs 2*hid channels, got %d" % c2)
    for name, t in (("update_res", update_res), ("cand_res", cand_res), ("h_delta", h_delta)):
        if tuple(t.shape) != (n, hid, h, w):
            raise ValueError("%s shape %s, expected %s" % (name, tuple(t.shape), (n, hid, h, w)))
    _ready(ts)
    dt = gates_delta.dtype
    check(lib().mie_convgru_gates_incr(nhwc_ptr(gates_delta, "gates_delta", dtype=dt), nhwc_ptr(update_res, "update_res"),
                                       nhwc_ptr(cand_res, "cand_res"), nhwc_ptr(h_delta, "h_delta", dtype=dt), hid,
                                       ts.ref, delta_dtype(gates_delta), _stream(gates_delta)))
    return h_delta


def convlstm_gates_refresh(gates_res, interleaved: bool, prev_c, cprev_res, cell_res, h_out, c_out):
    """Dense ConvLSTM state from the gate pre-activations of a refresh; fills the cell reservoirs."""
    n, hid, h, w = h_out.shape
    dt = h_out.dtype
    if tuple(gates_res.shape) != (n, 4 * hid, h, w):
        raise ValueError("gates_res shape %s, expected %s" % (tuple(gates_res.shape), (n, 4 * hid, h, w)))
    for name, t in (("cprev_res", cprev_res), ("cell_res", cell_res)):
        _same_shape(name, t, h_out)
    check(lib().mie_convlstm_gates_refresh(
        nhwc_ptr(gates_res, "gates_res"), 1 if interleaved else 0, nhwc_ptr(prev_c, "prev_c", hid, dtype=dt),
        nhwc_ptr(cprev_res, "cprev_res"), nhwc_ptr(cell_res, "cell_res"), nhwc_ptr(h_out, "h_out", dtype=dt),
        nhwc_ptr(c_out, "c_out", hid, dtype=dt), n, h, w, hid, delta_dtype(h_out), _stream(h_out)))
    return h_out, c_out


def convgru_gates_refresh(update, cand, prev_state, diff_res, update_res, new_state):
    """Dense ConvGRU state from the activated gates of a refresh; fills the product's cached operands."""
    n, hid, h, w = new_state.shape
    dt = new_state.dtype
    check(lib().mie_convgru_gates_refresh(
        nhwc_ptr(update, "update", hid, dtype=dt), nhwc_ptr(cand, "cand", hid, dtype=dt),
        nhwc_ptr(prev_state, "prev_state", hid, dtype=dt), nhwc_ptr(diff_res, "diff_res", hid),
        nhwc_ptr(update_res, "update_res", hid), nhwc_ptr(new_state, "new_state", dtype=dt), n, h, w, hid,
        delta_dtype(new_state), _stream(new_state)))
    return new_state


def mul_dense(a, b, out):
    """out = a * b, dense tensors of one shape, layout (NHWC) and type."""
    dt = out.dtype
    if a.shape != out.shape or b.shape != out.shape:
        raise ValueError("shapes differ: %s %s %s" % (tuple(a.shape), tuple(b.shape), tuple(out.shape)))
    check(lib().mie_mul_dense(nhwc_ptr(a, "a", dtype=dt), nhwc_ptr(b, "b", dtype=dt), nhwc_ptr(out, "out", dtype=dt),
                              out.numel(), delta_dtype(out), _stream(out)))
    return out


def gate_interleave_index(hid: int, device=None) -> torch.Tensor:
    """Column order of the fused gates conv: entry c' (= 4*hc + g) holds the column g*hid + hc of the
    [in | remember | out | cell] x hid order (gate g of hidden channel hc)."""
    cp = torch.arange(4 * hid, device=device)
    return (cp % 4) * hid + cp // 4


def conv_gates_incr(x, xmask, x2, x2mask, filt: ConvFilter, out_ts: TileMask, gates_res, cprev_delta, cprev_mask,
                    cprev_res, cell_res, h_delta, c_delta, workspace=None):
    """3x3 gates conv of a ConvLSTM with the gate chain as its epilogue; `filt` and `gates_res` are in the
    gate-interleaved column order (gate_interleave_index).  workspace: as in conv_masked."""
    n, c1, h, w = x.shape
    c2 = 0 if x2 is None else x2.shape[1]
    dt = x.dtype
    plain, mc_ptr, code = _filter_args(filt, 3, dt, (1, c1, c2, filt.shape[3]), with_code=True)
    cin_total, cout = plain.shape[0], plain.shape[3]
    hid = cout // 4
    if tuple(gates_res.shape) != (n, cout, h, w):
        raise ValueError("gates_res shape %s, expected %s" % (tuple(gates_res.shape), (n, cout, h, w)))
    for name, t in (("cprev_res", cprev_res), ("cell_res", cell_res), ("h_delta", h_delta), ("c_delta", c_delta)):
        if tuple(t.shape) != (n, hid, h, w):
            raise ValueError("%s shape %s, expected %s" % (name, tuple(t.shape), (n, hid, h, w)))
    _ready(out_ts)
    ws_ptr, ws_bytes = _workspace_args(workspace, mc_ptr is not None and out_ts.capacity * (cout // 32) <= 128, x.device)
    check(lib().mie_conv_gates_masked_ws(
        nhwc_ptr(x, "x", dtype=dt), pix_ptr(xmask, n, h, w, "xmask"), c1,
        nhwc_ptr(x2, "x2", dtype=dt), pix_ptr(x2mask, n, h, w, "x2mask"), c2, h, w,
        plain.data_ptr(), mc_ptr, cin_total, hid, out_ts.ref, nhwc_ptr(gates_res, "gates_res"),
        nhwc_ptr(cprev_delta, "cprev_delta", dtype=dt), pix_ptr(cprev_mask, n, h, w, "cprev_mask"),
        nhwc_ptr(cprev_res, "cprev_res"), nhwc_ptr(cell_res, "cell_res"),
        nhwc_ptr(h_delta, "h_delta", dtype=dt), nhwc_ptr(c_delta, "c_delta", dtype=dt), code, ws_ptr, ws_bytes,
        _stream(x)))
    return h_delta, c_delta


def mfma_chunk(dtype) -> int:
    """Input channels per staging chunk of the 3x3 / 5x5 stride-1 matrix-core kernels."""
    return 32 if dtype == torch.float32 else 64


def conv_out_size(h, w, k, stride, pad) -> Tuple[int, int]:
    """Output size formula of the reference wrapper (ext/pointops/pointops_functional.py:25-26)."""
    return (h + 2 * pad - k) // stride + 1, (w + 2 * pad - k) // stride + 1
