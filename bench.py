#!/usr/bin/env python3
"""Benchmark of the masked incremental inference path on one MI355X.

Headline workload (the configuration the metric is quoted on): E2Depth-incr,
random-init weights, one event stream of 5x264x352 voxel grids, one dense
refresh, then incremental steps with 5 % of the pixels carrying a delta
(Poisson(2) event counts x random polarity x 0.1 per bin, smooth blob masks).
A "step" is one incremental frame through the whole network; the deltas are
resident in HBM before the timed region starts and the step is replayed from
a HIP graph.  `--steps` steps are timed between two device synchronisations,
`--repeats` times over; `ms_per_step` is the median of those repeats.

Prints ONE compact JSON line on stdout (kept under 6000 characters: asserted by
tests/test_bench_line.py): frames/s (`value`), ms/frame, the roofline of the
dominant kernel launch (the masked conv layer that takes the most time, timed
with HIP events on the stream it runs on), the CPU baseline (the torch-CPU
oracle of the reference path on the host cores), a check of the first steps
against that oracle, and a {time, roofline fraction} summary of everything
else that is measured: the same network run densely through the same kernels
(all tiles active), 1 % and 20 % density, the dense refresh, the other
benchmark configurations (single masked conv, activation chain, EVFlowNet-incr
with both decoder kinds, batched bf16 E2Depth-incr) and the lossy frontier
(delta quantiser / threshold masks: speed against error).  The full tables
(per-launch table, every configuration with its repeats, every lossy point) go
to `--detail-file` (default gpurun_out/bench_detail.json) and to stderr.
"""
import argparse
import json
import os
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_FP32_MFMA_TFLOPS = 157.3
PEAK_BF16_MFMA_TFLOPS = 2500.0
PEAK_HBM_GBS = 8000.0


def log(msg):
    print("[bench] " + msg, file=sys.stderr, flush=True)


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--repeats", type=int, default=10, help="timed repeats of the --steps loop (median reported)")
    ap.add_argument("--density", type=float, default=0.05)
    ap.add_argument("--height", type=int, default=264)
    ap.add_argument("--width", type=int, default=352)
    ap.add_argument("--batch", type=int, default=1, help="independent event streams per step (8 with 480x640: the batched configuration)")
    ap.add_argument("--cpu-steps", type=int, default=400, help="incremental steps of the CPU baseline (0 = skip)")
    ap.add_argument("--no-graph", action="store_true", help="launch kernels eagerly instead of replaying a HIP graph")
    ap.add_argument("--plan-ahead", choices=["host", "streams", "fork", "off"], default="host",
                    help="plan the next step's tile sets beside this step's kernels: 'host' = planning and compute halves "
                         "as two graphs on two streams, the host keeps their order (it launches a half after the event it "
                         "depends on has fired); 'streams' = the same with the order kept by event waits on the GPU; "
                         "'fork' = one graph per step with the plan forked inside it; 'off' = every step plans its own "
                         "tile sets first")
    ap.add_argument("--copy-input", action="store_true",
                    help="one captured graph and a device-to-device copy of the next delta into its input buffer before every "
                         "replay (default: one graph per resident input, no copy)")
    ap.add_argument("--no-dense", action="store_true", help="skip the all-tiles-active comparator")
    ap.add_argument("--layer-iters", type=int, default=20, help="timed launches per layer for the roofline table")
    ap.add_argument("--no-plan-first", dest="plan_first", action="store_false",
                    help="enqueue each mask build right before its consumer instead of all builds of a step first")
    ap.add_argument("--upconv-all", action="store_true",
                    help="take the one-kernel up-sampling conv for every decoder layer, whatever its size (for measurements)")
    ap.add_argument("--sync-masks", action="store_true", help="build tile sets on the compute stream (no planning stream)")
    ap.add_argument("--in-threshold", type=float, default=None,
                    help="run the network with a threshold mask in front of every conv (a lossy variant: pixels whose delta stays "
                         "within the threshold are dropped for the step); value-dependent masks are built inline, so "
                         "--sync-masks --no-plan-first --plan-ahead off are implied and the oracle check is skipped")
    ap.add_argument("--net", choices=["e2depth", "evflownet"], default="e2depth",
                    help="e2depth: the headline network (5 bins); evflownet: EVFlowNet-incr, 4 bins, moving-edge deltas "
                         "(use --height 256 --width 256)")
    ap.add_argument("--decoder", choices=["upsample", "transposed"], default="upsample",
                    help="decoder kind of --net evflownet")
    ap.add_argument("--dtype", choices=["f32", "bf16"], default="f32",
                    help="element type of deltas and weights (reservoirs and accumulation stay fp32)")
    ap.add_argument("--no-sweep", dest="sweep", action="store_false", help="skip the 1 %% / 20 %% density runs")
    ap.add_argument("--no-configs", dest="configs", action="store_false",
                    help="skip the other benchmark configurations (single conv, activation chain, EVFlowNet-incr, batched bf16)")
    ap.add_argument("--no-lossy", dest="lossy", action="store_false", help="skip the lossy frontier")
    ap.add_argument("--no-refresh", dest="refresh", action="store_false", help="skip the dense-refresh timing")
    ap.add_argument("--f32-matmul", choices=["bf16x3", "native"], default=None,
                    help="how the matrix-core kernels multiply fp32 deltas (default: the library setting, bf16x3 = "
                         "three bf16 terms per value on the bf16 instruction, fp32 accuracy)")
    ap.add_argument("--no-native", dest="native", action="store_false",
                    help="skip the comparison run with the fp32 matrix-core instruction")
    ap.add_argument("--detail-file", default=os.path.join(ROOT, "gpurun_out", "bench_detail.json"),
                    help="where the full tables go (per-launch table, configurations, lossy frontier); stdout carries "
                         "one compact JSON line")
    return ap.parse_args()


class LayerProbe:
    """Times every conv / point-wise entry point of one eager step with HIP events recorded
    on the stream the kernels are launched on, and derives algorithmic bytes / flops from the
    tile-set statistics of that step."""

    def __init__(self, ops, torch, es=4):
        self.ops, self.torch = ops, torch
        self.es = es            # bytes per delta / weight element (reservoirs are always 4)
        self.records = []
        self._orig = {}

    def _wrap(self, name, describe):
        orig = getattr(self.ops, name)
        self._orig[name] = orig
        torch = self.torch

        def wrapped(*a, **kw):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            r = orig(*a, **kw)
            e1.record()
            self.records.append([name, describe(*a, **kw), e0, e1, (orig, a, kw)])
            return r
        setattr(self.ops, name, wrapped)

    def __enter__(self):
        def conv_desc(x, xmask, x2, x2mask, filt, k, stride, pad, out_ts, out_delta, reservoir=None, *a, **kw):
            n, c1, h, w = x.shape
            c2 = 0 if x2 is None else x2.shape[1]
            return dict(kind="conv", k=k, s=stride, cin=c1 + c2, cout=filt.shape[3], h=h, w=w, n=n,
                        xmask=xmask, x2mask=x2mask, ts=out_ts, fused=reservoir is not None)

        def pw_desc(kind, nin, nres):
            def d(*a, **kw):
                ts = [t for t in a if hasattr(t, "pixmask") and hasattr(t, "tiles")][-1]
                t0 = [t for t in a if hasattr(t, "shape") and len(getattr(t, "shape", ())) == 4][0]
                return dict(kind=kind, c=t0.shape[1], ts=ts, nin=nin, nres=nres)
            return d
        def conv_gates_desc(x, xmask, x2, x2mask, filt, out_ts, *a, **kw):
            n, c1, h, w = x.shape
            c2 = 0 if x2 is None else x2.shape[1]
            return dict(kind="conv", k=3, s=1, cin=c1 + c2, cout=filt.shape[3], h=h, w=w, n=n,
                        xmask=xmask, x2mask=x2mask, ts=out_ts, fused=True, gates=True)

        def upconv_desc(a_, amask, b_, bmask, filt, k, pad, out_ts, out_delta, reservoir=None, *a, **kw):
            n, c, h, w = a_.shape
            return dict(kind="conv", k=k, s=1, cin=c, cout=filt.shape[3], h=h, w=w, n=n, xmask=amask,
                        x2mask=bmask, ts=out_ts, fused=reservoir is not None, up=True, two=b_ is not None)

        def upconv_pred_desc(a_, amask, b_, bmask, filt, out_ts, reservoir, act, slope, skip, skip_mask, *a, **kw):
            n, c, h, w = a_.shape
            return dict(kind="conv", k=5, s=1, cin=c, cout=filt.shape[3], h=h, w=w, n=n, xmask=amask, x2mask=bmask,
                        ts=out_ts, fused=True, up=True, two=b_ is not None, pred=True, skip_mask=skip_mask)

        def tconv2x_desc(x, xmask, x2, x2mask, filt, k, out_ts, block_ts, out_delta, reservoir=None, *a, **kw):
            n, c1, h, w = x.shape
            c2 = 0 if x2 is None else x2.shape[1]
            return dict(kind="conv", k=k, s=2, cin=c1 + c2, cout=filt.shape[3], h=h, w=w, n=n, xmask=xmask,
                        x2mask=x2mask, ts=out_ts, fused=reservoir is not None, tconv=True)

        def tconv_desc(x, xmask, filt, k, stride, pad, out_ts, out_delta, reservoir=None, *a, **kw):
            n, c1, h, w = x.shape
            return dict(kind="conv", k=k, s=stride, cin=c1, cout=filt.shape[3], h=h, w=w, n=n, xmask=xmask,
                        x2mask=None, ts=out_ts, fused=reservoir is not None, tconv=True)

        self._wrap("conv_masked", conv_desc)
        self._wrap("tconv2x_masked", tconv2x_desc)
        self._wrap("tconv_masked", tconv_desc)
        self._wrap("upconv_masked", upconv_desc)
        self._wrap("upconv_pred_masked", upconv_pred_desc)
        self._wrap("conv_gates_incr", conv_gates_desc)
        self._wrap("act_incr", pw_desc("act", 1, 1))
        self._wrap("add_incr", pw_desc("add", 2, 0))
        self._wrap("mul_incr", pw_desc("mul", 2, 2))
        self._wrap("upsample2x_incr", pw_desc("up2x", 2, 0))
        self._wrap("convlstm_gates_incr", pw_desc("gates", 4, 6))
        self._wrap("build_mask_tiles", lambda *a, **kw: dict(kind="tiles", ts=a[-1]))
        self._wrap("mask_from_delta", lambda d, t, o: dict(kind="mask", c=d.shape[1], npix=d.shape[0] * d.shape[2] * d.shape[3]))
        return self

    def __exit__(self, *exc):
        for name, orig in self._orig.items():
            setattr(self.ops, name, orig)

    def table(self):
        """One row per launch: ms, algorithmic bytes and flops (counted once per step)."""
        self.torch.cuda.synchronize()
        rows = []
        for name, d, e0, e1, call in self.records:
            ms = e0.elapsed_time(e1)
            row = dict(op=name, ms=ms, call=call)
            if d["kind"] == "conv":
                ts = d["ts"]
                P = d["n"] * d["h"] * d["w"]
                a_in = P if d["xmask"] is None else int(self._pix(d["xmask"]).sum().item())
                if d.get("up") and d["two"]:
                    # up2x(a + b) formed on the fly: both half-resolution inputs are read once, nothing in between
                    a_in += P if d["x2mask"] is None else int(self._pix(d["x2mask"]).sum().item())
                    P *= 2
                a_out = int(ts.pixmask.sum().item())
                cin, cout, k = d["cin"], d["cout"], d["k"]
                es = self.es
                byts = P + a_in * cin * es + cin * cout * k * k * es + ts.capacity * 4
                if d.get("gates"):
                    # gate reservoirs read + written, cell reservoir read + written, previous cell read,
                    # hidden and cell deltas written; the 4*hid-channel gate delta never reaches memory
                    hid = cout // 4
                    byts += a_out * (2 * cout * 4 + 2 * hid * 4 + hid * 4 + 2 * hid * es)
                elif d.get("pred"):
                    # fused tail: the layer's reservoir read + written, its delta never stored; the second delta of the
                    # prediction conv read where its mask is set; prediction reservoir read + written, prediction delta
                    a_skip = a_out if d["skip_mask"] is None else int(self._pix(d["skip_mask"]).sum().item())
                    byts += 2 * a_out * cout * 4 + a_skip * cout * es + a_out * (8 + es)
                else:
                    byts += a_out * cout * es
                    if d["fused"]:
                        byts += 2 * a_out * cout * 4
                flops = 2 * a_out * cin * cout * k * k + (4 * a_out * cout if d.get("pred") else 0)
                if d.get("tconv"):
                    # stride-s transposed conv: an output pixel meets (k/s)^2 taps on average
                    flops = 2 * a_out * cin * cout * k * k // (d["s"] * d["s"])
                row.update(shape="%s%dx%d s%d %d->%d%s @%dx%d" % ("up2x+" if d.get("up") else ("tconv " if d.get("tconv") else ""),
                                                                   k, k, d["s"], cin, cout,
                                                                   "+lstm" if d.get("gates") else ("+pred" if d.get("pred") else ""),
                                                                   ts.h, ts.w),
                           active_tiles=int(ts.counts[0].item()), tiles=ts.capacity, a_out=a_out,
                           bytes=byts, flops=flops)
            elif d["kind"] in ("act", "add", "mul", "up2x", "gates"):
                ts = d["ts"]
                a = int(ts.pixmask.sum().item())
                c = d["c"]
                if d["kind"] == "gates":
                    hid = c // 4
                    byts = a * (4 * hid * self.es + 2 * 4 * hid * 4 + 2 * hid * 4 + hid * 4 + 2 * hid * self.es)
                elif d["kind"] == "up2x":
                    # the two inputs live at a quarter of the output pixels: counted once each
                    byts = a * c * self.es * (1 + d["nin"] / 4.0)
                else:
                    byts = a * c * (self.es * (d["nin"] + 1) + 8 * d["nres"])
                byts += ts.n * ts.h * ts.w
                row.update(shape="%s C=%d @%dx%d" % (d["kind"], c, ts.h, ts.w), a_out=a, bytes=byts, flops=0,
                           active_tiles=int(ts.counts[0].item()), tiles=ts.capacity)
            elif d["kind"] == "tiles":
                ts = d["ts"]
                row.update(shape="tiles @%dx%d" % (ts.h, ts.w), bytes=2 * ts.n * ts.h * ts.w + ts.capacity * 8, flops=0)
            else:
                row.update(shape="mask C=%d" % d["c"], bytes=d["npix"] * (d["c"] * self.es + 1), flops=0)
            rows.append(row)
        return rows

    @staticmethod
    def _pix(m):
        return m.pixmask if hasattr(m, "pixmask") else m




class Workload:
    """One network configuration: net, frame size, batch, element type, delta generator."""

    def __init__(self, net="e2depth", h=264, w=352, batch=1, density=0.05, dtype="f32", decoder="upsample"):
        self.net, self.h, self.w, self.batch, self.density, self.dtype, self.decoder = net, h, w, batch, density, dtype, decoder

    def name(self):
        return "EVFlowNet-incr" if self.net == "evflownet" else "E2Depth-incr"

    def bins(self):
        return 4 if self.net == "evflownet" else 5


class NetBench:
    """A network instance factory + resident inputs + the timing loops for one Workload."""

    def __init__(self, torch, ops, wl, args, n_inputs=16):
        from maskedincrementeval_amd.synthetic import MovingEdges, event_voxel_delta
        self.torch, self.ops, self.wl, self.args = torch, ops, wl, args
        self.dev = torch.device("cuda:0")
        self.dt = torch.bfloat16 if wl.dtype == "bf16" else torch.float32
        self.es = 2 if wl.dtype == "bf16" else 4
        self.peak_mfma = PEAK_BF16_MFMA_TFLOPS if wl.dtype == "bf16" else PEAK_FP32_MFMA_TFLOPS
        self.n_inputs = n_inputs
        nb, bins, h, w = wl.batch, wl.bins(), wl.h, wl.w
        if wl.net == "evflownet":
            from maskedincrementeval_amd.evflownet_incr import MultiResUNetRecurrentIncr
            self.make_net = lambda **kw: MultiResUNetRecurrentIncr(num_bins=4, decoder=wl.decoder, **kw)
            self.run_net = lambda m, x: m([x, None])
            self.run_pipe = lambda m, x, nxt, par: m.forward_pipelined([x, None], [nxt, None], par)
            self.run_planned = lambda m, x, par: m.forward_planned([x, None], par)
            self.run_plan = lambda m, x, par: m.plan_ahead([x, None], par)
            self.out_of = lambda r: r[-1][0]                      # the finest flow scale
            self.refresh_net = lambda m, x: m.forward_refresh_reservoirs(x)
            self.refresh_out = lambda r: r[-1]
        else:
            from maskedincrementeval_amd.e2depth_incr import E2VIDRecurrentIncr
            self.make_net = E2VIDRecurrentIncr
            self.run_net = lambda m, x: m([x, None], None)
            self.run_pipe = lambda m, x, nxt, par: m.forward_pipelined([x, None], [nxt, None], par)
            self.run_planned = lambda m, x, par: m.forward_planned([x, None], par)
            self.run_plan = lambda m, x, par: m.plan_ahead([x, None], par)
            self.out_of = lambda r: r[0][0]
            self.refresh_net = lambda m, x: m.forward_refresh_reservoirs(x, None)
            self.refresh_out = lambda r: r[0]
        self.x0 = torch.randn(nb, bins, h, w, generator=torch.Generator().manual_seed(2)) * 0.5
        self.static_in = self.cl(torch.zeros(nb, bins, h, w))
        self.set_density(wl.density)

    def cl(self, t):
        return t.to(self.dev).to(self.dt).contiguous(memory_format=self.torch.channels_last)

    def set_density(self, p):
        """(Re)generate the resident input deltas at pixel density p (moving edges: p is nominal)."""
        from maskedincrementeval_amd.synthetic import MovingEdges, event_voxel_delta
        torch, wl = self.torch, self.wl
        if wl.net == "evflownet":
            gens = [MovingEdges(wl.h, wl.w, seed=53 + b) for b in range(wl.batch)]
            self.deltas_cpu = [torch.cat([g.step()[0] for g in gens], 0) for _ in range(self.n_inputs)]
        else:
            self.deltas_cpu = [event_voxel_delta(wl.batch, wl.bins(), wl.h, wl.w, p, seed=3000 + i)[0]
                               for i in range(self.n_inputs)]
        self.deltas = [self.cl(d) for d in self.deltas_cpu]
        self.measured_density = float(sum((d != 0).any(1).float().mean().item() for d in self.deltas_cpu) / self.n_inputs)

    def new_model(self, seed=1, **kw):
        from maskedincrementeval_amd.synthetic import seed_module_
        thr = getattr(self.args, "in_threshold", None)
        if thr is not None:
            kw.pop("async_masks", None), kw.pop("plan_first", None)
        m = seed_module_(self.make_net(**kw), seed=seed).to(self.dev).eval()
        if thr is not None:
            from maskedincrementeval_amd.mask_incr_modules import set_input_threshold
            set_input_threshold(m, thr)
        return m

    def step_eager(self, m, i):
        self.static_in.copy_(self.deltas[i % self.n_inputs])
        return self.run_net(m, self.static_in)

    def plan_ahead_mode(self):
        a = self.args
        return None if (a.plan_ahead == "off" or a.copy_input or getattr(a, "in_threshold", None) is not None) else a.plan_ahead

    def timed_run(self, m, tag, steps=None, repeats=None, check_against=None, graph=None, plan_ahead="default"):
        """Refresh, warm up, capture one step per resident input in a HIP graph, then time `steps` steps `repeats`
        times.  The inputs are taken cyclically by one running step counter.  plan_ahead "fork": the graph of
        input i holds step i and, forked beside it, the plan of input i + 1's tile sets (forward_pipelined);
        "streams" / "host": the two halves are graphs of their own, replayed on two streams (forward_planned /
        plan_ahead, ops.LookaheadStepper), ordered by event waits on the GPU / by the host; None: every step plans
        its own tile sets first (forward).
        Returns (median seconds per step, list of the repeats' ms/step, output-check dict)."""
        torch, args = self.torch, self.args
        steps = args.steps if steps is None else steps
        repeats = args.repeats if repeats is None else repeats
        use_graph = (not args.no_graph) if graph is None else graph
        pipe = self.plan_ahead_mode() if plan_ahead == "default" else plan_ahead
        n_in = self.n_inputs
        assert n_in % 2 == 0
        history, check = [], {}
        k = 0                                                # running step counter: input k % n_in
        stepper = None
        if pipe in ("streams", "host"):     # the two halves on two streams: orderings as GPU-side waits / kept by the host
            stepper = self.ops.LookaheadStepper(self.dev, host_ordered=(pipe == "host"))
            pipe = "streams"

        def two_streams(i, compute, plan):
            return stepper.step(i, lambda: compute(i), lambda: plan((i + 1) % n_in))

        def eager(kk):
            i = kk % n_in
            if pipe == "fork":
                return self.run_pipe(m, self.deltas[i], self.deltas[(i + 1) % n_in], i % 2)
            if pipe == "streams":
                return two_streams(i, lambda j: self.run_planned(m, self.deltas[j], j % 2),
                                   lambda j: self.run_plan(m, self.deltas[j], j % 2))
            self.static_in.copy_(self.deltas[i])
            return self.run_net(m, self.static_in)

        def capture(fn):
            g = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g):
                r = fn()
            return g, r
        with torch.no_grad():
            self.refresh_net(m, self.cl(self.x0))
            warm = -(-max(args.warmup, 3) // n_in) * n_in    # whole cycles; also allocates every persistent buffer
            for _ in range(warm):
                eager(k)
                history.append(k % n_in)
                k += 1
            torch.cuda.synchronize()
            replay = graph_outs = None
            if use_graph:
                # One captured graph per resident input: a step then reads its delta where it lies, as it would from the
                # buffer an event front end writes, and no copy into a fixed input buffer is timed (--copy-input: one
                # graph, input copied in front of every replay).
                side = torch.cuda.Stream()
                side.wait_stream(torch.cuda.current_stream())
                with torch.cuda.stream(side):
                    for _ in range(n_in):
                        eager(k)
                        history.append(k % n_in)
                        k += 1
                torch.cuda.current_stream().wait_stream(side)
                torch.cuda.synchronize()
                graphs, graph_outs = [], []
                if pipe == "streams":
                    plans = [None] * n_in
                    for i in range(n_in):                   # in the order of the steps: the networks check it
                        g, r = capture(lambda: self.run_planned(m, self.deltas[i], i % 2))
                        graphs.append(g)
                        graph_outs.append(self.out_of(r))
                        j = (i + 1) % n_in
                        plans[j], _ = capture(lambda: self.run_plan(m, self.deltas[j], j % 2))
                    replay = lambda kk: two_streams(kk % n_in, lambda i: graphs[i].replay(), lambda j: plans[j].replay())
                elif pipe == "fork":
                    for i in range(n_in):
                        g, r = capture(lambda: self.run_pipe(m, self.deltas[i], self.deltas[(i + 1) % n_in], i % 2))
                        graphs.append(g)
                        graph_outs.append(self.out_of(r))
                    replay = lambda kk: graphs[kk % n_in].replay()
                elif args.copy_input:
                    g, r = capture(lambda: self.run_net(m, self.static_in))
                    graphs.append(g)
                    graph_outs.append(self.out_of(r))

                    def replay(kk):
                        self.static_in.copy_(self.deltas[kk % n_in])
                        graphs[0].replay()
                else:
                    for i in range(n_in):
                        g, r = capture(lambda: self.run_net(m, self.deltas[i]))
                        graphs.append(g)
                        graph_outs.append(self.out_of(r))
                    replay = lambda kk: graphs[kk % n_in].replay()
                for _ in range(n_in):
                    replay(k)
                    history.append(k % n_in)
                    k += 1
            step = replay if replay is not None else eager
            per_repeat, enqueue = [], []
            for _ in range(repeats):
                torch.cuda.synchronize()
                t0 = time.perf_counter()
                for _ in range(steps):
                    step(k)
                    k += 1
                t_host = time.perf_counter()
                torch.cuda.synchronize()
                per_repeat.append((time.perf_counter() - t0) / steps)
                enqueue.append((t_host - t0) / steps)
                history.extend((k - steps + j) % n_in for j in range(steps))
            if check_against is not None:
                # The timed configuration (graph replay, planning ahead) against the plain one: a second
                # instance of the network with eager launches and inline mask planning takes the same
                # steps; the next frames of the two must then agree (same kernels over the same tiles).
                ref = check_against()
                self.refresh_net(ref, self.cl(self.x0))
                for i in history:
                    self.run_net(ref, self.deltas[i])
                worst = 0.0
                for _ in range(4):
                    want = self.out_of(self.run_net(ref, self.deltas[k % n_in]))
                    got = step(k)
                    got = graph_outs[k % len(graph_outs)] if replay is not None else self.out_of(got)
                    k += 1
                    worst = max(worst, (got.float() - want.float()).abs().max().item())
                torch.cuda.synchronize()
                check.update(max_abs_diff=worst, frames=4, steps_before=len(history),
                             against="same network, eager launches, inline mask planning")
                log("%s: max |difference| to the eager inline-planning network over 4 frames after %d steps: %.3e"
                    % (tag, len(history), worst))
                if not worst <= 1e-3:
                    raise SystemExit("bench: the timed configuration does not reproduce the plain one (%.3e)" % worst)
        sec = statistics.median(per_repeat)
        log("%s: %.3f ms/step median of %d x %d steps (min %.3f, max %.3f; %s; the host has enqueued a step after %.3f ms)"
            % (tag, 1e3 * sec, repeats, steps, 1e3 * min(per_repeat), 1e3 * max(per_repeat),
               "eager" if replay is None else "HIP graph", 1e3 * statistics.median(enqueue)))
        check["host_enqueue_ms_per_step"] = round(1e3 * statistics.median(enqueue), 4)
        return sec, [round(1e3 * t, 4) for t in per_repeat], check

    def layer_table(self, model, iters):
        """Per-launch table of one step: eager launches with HIP events, mean of `iters` steps."""
        torch, ops = self.torch, self.ops
        with torch.no_grad():
            plan_first, model.plan_first = model.plan_first, False   # one walk per step: every wrapper call timed once
            self.refresh_net(model, self.cl(self.x0))
            self.step_eager(model, 0)
            agg = None
            for it in range(iters):
                with LayerProbe(ops, torch, self.es) as probe:
                    self.step_eager(model, 1 + it)
                rows = probe.table()
                if agg is None:
                    agg = rows
                    for r in agg:
                        r["ms_sum"], r["bytes_sum"], r["flops_sum"] = 0.0, 0, 0
                for r, q in zip(agg, rows):
                    r["ms_sum"] += q["ms"]
                    r["bytes_sum"] += q["bytes"]
                    r["flops_sum"] += q["flops"]
            model.plan_first = plan_first
        layers = []
        for r in agg:
            ms = r["ms_sum"] / iters
            byts, fl = r["bytes_sum"] / iters, r["flops_sum"] / iters
            layers.append(dict(op=r["op"], shape=r["shape"], us=round(1e3 * ms, 2),
                               gbs=round(byts / (ms * 1e-3) / 1e9, 1) if ms > 0 else None,
                               tflops=round(fl / (ms * 1e-3) / 1e12, 2) if ms > 0 else None,
                               bytes=int(byts), flops=int(fl), active_tiles=r.get("active_tiles"), tiles=r.get("tiles")))
        return layers, agg

    def dominant_roofline(self, layers, agg, reps=50):
        """Roofline of the conv launch that takes the most time, re-timed on its own: the same call (same
        tile set, same buffers) launched `reps` times on the launch stream, each launch between two HIP events
        of its own; `us` is the mean of the pairs less what an empty pair reads."""
        torch = self.torch
        convs = [l for l in layers if l["op"] in ("conv_masked", "conv_gates_incr", "upconv_masked", "upconv_pred_masked", "tconv2x_masked")]
        dom = max(convs, key=lambda l: l["us"])
        orig, cargs, ckw = agg[layers.index(dom)]["call"]
        with torch.no_grad():
            for _ in range(5):
                orig(*cargs, **ckw)
            evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(reps)]
            ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            ev0.record()
            for ea, eb in evs:
                ea.record()
                orig(*cargs, **ckw)
                eb.record()
            ev1.record()
            # what an event pair reads with nothing between its two records
            empty = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(reps)]
            for ea, eb in empty:
                ea.record()
                eb.record()
            torch.cuda.synchronize()
        self.event_pair_us = round(1e3 * sum(ea.elapsed_time(eb) for ea, eb in empty) / reps, 2)
        pair_us = 1e3 * sum(ea.elapsed_time(eb) for ea, eb in evs) / reps
        self.dominant_back_to_back_us = round(1e3 * ev0.elapsed_time(ev1) / reps, 2)
        # The figure the roofline uses: what the event pair around a launch reads, less what an empty pair reads (the
        # cost of the two records themselves) -- it agrees with the kernel's average duration in a rocprofv3 kernel
        # trace of the step.  Beside it: `reps` launches of the call captured in one HIP graph and replayed between two
        # events; identical launches back to back find the filter and their operands in cache and run a few per cent
        # faster than the launch does inside a step.
        dom_us = pair_us - self.event_pair_us
        with torch.no_grad():
            graph_us = event_time(torch, lambda: orig(*cargs, **ckw), warm=2, reps=reps)
        dom = dict(dom, us=round(dom_us, 2), gbs=round(dom["bytes"] / dom_us / 1e3, 1),
                   tflops=round(dom["flops"] / dom_us / 1e6, 2))
        mfma_bound = dom["flops"] / max(dom["bytes"], 1) > self.peak_mfma * 1e12 / (PEAK_HBM_GBS * 1e9)
        x3 = self.wl.dtype == "f32" and self._takes_x3(dom)
        if mfma_bound and x3:
            # fp32 deltas multiplied as three bf16 terms: six bf16 matrix-core products per algorithmic multiply, so
            # the bound is the bf16 peak over six; the fraction of the fp32 instruction's peak is given beside it
            peak = round(PEAK_BF16_MFMA_TFLOPS / 6.0, 1)
            roofline = dict(bound="mfma", achieved=dom["tflops"], peak=peak, unit="TFLOP/s",
                            frac=round(dom["tflops"] / peak, 4), traffic=None,
                            peak_basis="bf16 matrix-core peak %.0f TFLOP/s / 6 term products per fp32 multiply" % PEAK_BF16_MFMA_TFLOPS,
                            executed_bf16_tflops=round(6 * dom["tflops"], 1),
                            frac_of_fp32_mfma_peak=round(dom["tflops"] / PEAK_FP32_MFMA_TFLOPS, 4))
        elif mfma_bound:
            roofline = dict(bound="mfma", achieved=dom["tflops"], peak=self.peak_mfma, unit="TFLOP/s",
                            frac=round(dom["tflops"] / self.peak_mfma, 4), traffic=None)
        else:
            roofline = dict(bound="hbm", achieved=dom["gbs"], peak=PEAK_HBM_GBS, unit="GB/s",
                            frac=round(dom["gbs"] / PEAK_HBM_GBS, 4), traffic=None)
        roofline.update(kernel="mie_%s %s" % (dom["op"].replace("_incr", "").replace("conv_gates", "conv_gates_masked"),
                                              dom["shape"]), us=dom["us"],
                        algorithmic_bytes=dom["bytes"], algorithmic_flops=dom["flops"],
                        us_event_pair=round(pair_us, 2), us_graph_of_identical_launches=round(graph_us, 2),
                        us_back_to_back=self.dominant_back_to_back_us,
                        us_empty_event_pair=self.event_pair_us)
        # HBM bytes per launch of that kernel from the committed rocprofv3 --pmc summary, if it covers this
        # shape (FETCH_SIZE + WRITE_SIZE, scaled by the copy-kernel calibration)
        try:
            with open(os.path.join(ROOT, "profiles", "pmc_traffic.json")) as f:
                roofline["traffic"] = json.load(f).get(dom["shape"] + (" bf16x3" if x3 else ""), {}).get("hbm_bytes_per_launch")
        except OSError:
            pass
        return roofline

    def _takes_x3(self, layer):
        """Whether the launch of a per-launch table row ran in the three-term bf16 form (its shape string is
        "KxK sS CIN->COUT..." with the input channels of the first operand)."""
        import re
        m = re.search(r"(\d)x\d s(\d) (\d+)->(\d+)", layer["shape"])
        if m is None:
            return False
        k, s_, cin, cout = (int(g) for g in m.groups())
        return self.ops.f32x3_takes(k, s_, cin, 0, cout)

    def refresh_timing(self, model, reps=30):
        """The dense refresh (every 20-100 frames in the reference's drivers): eager and replayed from a graph."""
        torch = self.torch
        x = self.cl(self.x0)
        with torch.no_grad():
            for _ in range(3):
                self.refresh_net(model, x)
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(reps):
                self.refresh_net(model, x)
            torch.cuda.synchronize()
            eager = (time.perf_counter() - t0) / reps
            side = torch.cuda.Stream()
            side.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(side):
                self.refresh_net(model, x)
            torch.cuda.current_stream().wait_stream(side)
            torch.cuda.synchronize()
            g = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g):
                self.refresh_net(model, x)
            for _ in range(3):
                g.replay()
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(reps):
                g.replay()
            torch.cuda.synchronize()
            graph = (time.perf_counter() - t0) / reps
        log("dense refresh: %.3f ms eager, %.3f ms from a HIP graph" % (1e3 * eager, 1e3 * graph))
        return dict(ms_eager=round(1e3 * eager, 4), ms_graph=round(1e3 * graph, 4))


def event_time(torch, fn, warm=5, reps=50, replays=7):
    """Microseconds of fn(): `reps` calls captured in one HIP graph (launches of 5-15 us are otherwise bound by
    the host's call rate, not by the GPU), the graph replayed `replays` times between HIP events on the launch
    stream; the median replay divided by `reps`."""
    for _ in range(warm):
        fn()
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        fn()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        for _ in range(reps):
            fn()
    g.replay()
    torch.cuda.synchronize()
    times = []
    for _ in range(replays):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        g.replay()
        e1.record()
        torch.cuda.synchronize()
        times.append(1e3 * e0.elapsed_time(e1) / reps)
    return float(statistics.median(times))


def config1_single_conv(torch, ops, _lib):
    """Configuration 1: one masked incremental conv3x3 32 -> 32 on 1x32x264x352 fp32 at 5 % pixel density,
    plain delta output (no fused epilogue): the launch alone, deltas resident."""
    from maskedincrementeval_amd.masked_types import TileMask
    from maskedincrementeval_amd.synthetic import gaussian_delta, he_normal_conv_weight
    dev = torch.device("cuda:0")
    n, c, h, w = 1, 32, 264, 352
    d, m = gaussian_delta(n, c, h, w, 0.05, 0.1, seed=1000)
    x = ops.as_nhwc(d.to(dev).contiguous(memory_format=torch.channels_last))
    mask = m.to(dev)
    filt = ops.ConvFilter(he_normal_conv_weight(c, c, 3, 0).permute(1, 2, 3, 0).contiguous().to(dev))
    ts = TileMask(n, h, w, dev)
    ops.build_mask_tiles(mask, None, n, h, w, _lib.FOOT_CONV, 3, 1, 1, ts)
    out = ops.new_nhwc(n, c, h, w, dev)
    res = ops.new_nhwc(n, c, h, w, dev)
    rows = {}
    for name, r, act in (("delta_only", None, _lib.ACT_NONE), ("fused_reservoir_relu", res, _lib.ACT_RELU)):
        us = event_time(torch, lambda: ops.conv_masked(x, mask, None, None, filt, 3, 1, 1, ts, out, r, act, 0.0))
        a_in, a_out = int(mask.sum().item()), int(ts.pixmask.sum().item())
        byts = n * h * w + a_in * c * 4 + a_out * c * 4 + c * c * 9 * 4 + ts.capacity * 4 + (2 * a_out * c * 4 if r is not None else 0)
        flops = 2 * a_out * c * c * 9
        rows[name] = dict(us=round(us, 2), algorithmic_bytes=byts, algorithmic_flops=flops,
                          gbs=round(byts / us / 1e3, 1), hbm_frac=round(byts / us / 1e3 / PEAK_HBM_GBS, 4),
                          tflops=round(flops / us / 1e6, 2), active_pixels_in=a_in, active_pixels_out=a_out,
                          active_tiles=int(ts.counts[0].item()), tiles=ts.capacity)
    us_build = event_time(torch, lambda: ops.build_mask_tiles(mask, None, n, h, w, _lib.FOOT_CONV, 3, 1, 1, ts))
    rows["build_mask_tiles_us"] = round(us_build, 2)
    rows["dense_bytes"], rows["dense_flops"] = 2 * n * c * h * w * 4, 2 * n * h * w * c * c * 9
    log("config 1 (conv3x3 32->32 @264x352, 5 %%): %.1f us, %.2f MB algorithmic = %.0f GB/s; with reservoir + ReLU %.1f us"
        % (rows["delta_only"]["us"], rows["delta_only"]["algorithmic_bytes"] / 1e6, rows["delta_only"]["gbs"],
           rows["fused_reservoir_relu"]["us"]))
    return rows


def config2_activation_chain(torch, ops, _lib):
    """Configuration 2: masked conv3x3 64 -> 64, incremental LeakyReLU(0.01), incremental ReLU on 1x64x132x176 fp32
    at 1 / 5 / 20 %, a fresh mask every step: microseconds per step of the chain (mask build + conv with the
    LeakyReLU increment fused + ReLU increment with its refined mask), eager launches between two HIP events."""
    from maskedincrementeval_amd import mask_incr_modules as mm
    from maskedincrementeval_amd.synthetic import gaussian_delta, seed_module_
    dev = torch.device("cuda:0")
    n, c, h, w = 1, 64, 132, 176
    conv = seed_module_(mm.nnConvIncr(c, c, 3, 1, 1), seed=2).to(dev).eval()
    leaky = mm.nnReservedActivation(mm.leaky_relu_op(0.01), refine_mask=False)
    relu = mm.nnReluIncr()
    x0 = torch.randn(n, c, h, w, generator=torch.Generator().manual_seed(20))
    cl = lambda t: ops.as_nhwc(t.to(dev).contiguous(memory_format=torch.channels_last))
    out = {}
    with torch.no_grad():
        relu.forward_refresh_reservoirs(conv.forward_refresh_fused(cl(x0), leaky))
        for p in (0.01, 0.05, 0.20):
            ins = [gaussian_delta(n, c, h, w, p, 0.2, seed=2000 + i) for i in range(8)]
            ins = [(cl(d), m.to(dev)) for d, m in ins]
            state = {"i": 0}

            def step():
                d, m = ins[state["i"] % 8]
                state["i"] += 1
                return relu(conv.forward_fused([d, m], leaky))
            us = event_time(torch, step, warm=8, reps=48)
            a = sum(int(m.sum().item()) for _, m in ins) / 8.0
            # algorithmic bytes of the chain: conv (mask, active delta in, delta out, reservoir r+w, filter, tile list)
            # + ReLU increment (delta in, reservoir r+w, delta out, mask)
            ts = conv._tile_set("out_act", n, h, w, dev)
            a_out = int(ts.pixmask.sum().item())
            byts = (n * h * w + a * c * 4 + a_out * c * 12 + c * c * 9 * 4 + ts.capacity * 4) + (a_out * c * 16 + n * h * w)
            out["%.2f" % p] = dict(us_per_step=round(us, 2), algorithmic_bytes=int(byts), gbs=round(byts / us / 1e3, 1),
                                   hbm_frac=round(byts / us / 1e3 / PEAK_HBM_GBS, 4))
            log("config 2 (conv3x3 64->64 + LeakyReLU + ReLU @132x176, %.0f %%): %.1f us/step, %.0f GB/s algorithmic"
                % (100 * p, us, byts / us / 1e3))
    return out


def side_config(torch, ops, args, wl, densities, steps, repeats, layer_iters=3, n_inputs=8, dense=True):
    """ms/step, dominant-kernel roofline and the dense comparator of another network configuration."""
    nb = NetBench(torch, ops, wl, args, n_inputs=n_inputs)
    model = nb.new_model(async_masks=not args.sync_masks, plan_first=args.plan_first)
    rows = {}
    for p in densities:
        if abs(p - wl.density) > 1e-12:
            nb.set_density(p)
            wl.density = p
        tag = "%s %dx%dx%d %s%s @%.0f%%" % (wl.name(), wl.batch, wl.h, wl.w, wl.dtype,
                                          " " + wl.decoder if wl.net == "evflownet" else "", 100 * p)
        sec, reps_ms, _ = nb.timed_run(model, tag, steps=steps, repeats=repeats)
        layers, agg = nb.layer_table(model, layer_iters)
        roof = nb.dominant_roofline(layers, agg, reps=20)
        rows["%.2f" % p] = dict(ms_per_step=round(1e3 * sec, 4), frames_per_s=round(wl.batch / sec, 1),
                                repeats_ms=reps_ms, measured_pixel_density=round(nb.measured_density, 4),
                                algorithmic_gflop_per_step=round(sum(l["flops"] for l in layers) / 1e9, 2),
                                algorithmic_mb_per_step=round(sum(l["bytes"] for l in layers) / 1e6, 1),
                                hbm_frac_whole_step=round(sum(l["bytes"] for l in layers) / sec / 1e9 / PEAK_HBM_GBS, 4),
                                dominant=roof)
    res = dict(workload="%s %dx%dx%dx%d %s%s" % (wl.name(), wl.batch, wl.bins(), wl.h, wl.w, wl.dtype,
                                                 ", %s decoders, moving-edge deltas" % wl.decoder if wl.net == "evflownet" else ""),
               densities=rows)
    if dense:
        dm = nb.new_model(derive_input_mask=False, async_masks=not args.sync_masks, plan_first=args.plan_first)
        dsec, _, _ = nb.timed_run(dm, "  dense (all tiles active, same kernels)", steps=steps, repeats=max(3, repeats // 2))
        res["dense_same_kernels_ms"] = round(1e3 * dsec, 4)
        del dm
    del model, nb
    torch.cuda.empty_cache()
    return res


def main():
    args = parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures ONE GPU (independent event streams shard one per GPU with "
              "no communication); --gpus %d is not run." % args.gpus, file=sys.stderr)
        sys.exit(2)
    import torch
    from maskedincrementeval_amd import _lib, ops

    _lib.lib()   # fail loudly if the HIP library is missing
    if args.upconv_all:
        ops.upconv_max_tiles = ops.upconv_max_chunks = 1 << 30
    if args.f32_matmul is not None:
        ops.f32_matmul = args.f32_matmul
    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        sys.exit(2)
    wl = Workload(args.net, args.height, args.width, args.batch, args.density, args.dtype, args.decoder)
    nb = NetBench(torch, ops, wl, args)
    H, W, dens, NB, BINS, NET_NAME = wl.h, wl.w, wl.density, wl.batch, wl.bins(), wl.name()

    model = nb.new_model(async_masks=not args.sync_masks, plan_first=args.plan_first)
    sec_per_step, repeats_ms, output_check = nb.timed_run(model, "incremental %.0f%%" % (100 * dens),
                                                          check_against=lambda: nb.new_model())

    # ---- per-layer roofline table -------------------------------------------------------------------
    layers, agg = nb.layer_table(model, args.layer_iters)
    roofline = nb.dominant_roofline(layers, agg)
    tot_us = sum(l["us"] for l in layers)
    tot_bytes = sum(l["bytes"] for l in layers)
    tot_flops = sum(l["flops"] for l in layers)
    log("per-launch table (eager, HIP events, mean of %d steps):" % args.layer_iters)
    for l in layers:
        log("  %-22s %-34s %9.2f us %8s GB/s %7s TFLOP/s  tiles %s/%s" % (
            l["op"], l["shape"], l["us"], l["gbs"], l["tflops"], l["active_tiles"], l["tiles"]))
    log("  sum of the eager launches (event pairs, one-set mask builds included) %.1f us; algorithmic %.1f MB, %.2f GFLOP per frame" % (tot_us, tot_bytes / 1e6, tot_flops / 1e9))

    # ---- the same network with the fp32 matrix-core instruction (v_mfma_f32_32x32x2_f32) ------------------
    native = None
    if args.native and args.dtype == "f32" and ops.f32_matmul == "bf16x3":
        ops.f32_matmul = "native"
        try:
            nat_model = nb.new_model(async_masks=not args.sync_masks, plan_first=args.plan_first)
            nat_sec, _, _ = nb.timed_run(nat_model, "incremental, fp32 matrix-core instruction", repeats=max(3, args.repeats // 2))
            del nat_model
        finally:
            ops.f32_matmul = "bf16x3"
        native = dict(ms_per_step=round(1e3 * nat_sec, 4), frames_per_s=round(NB / nat_sec, 1))

    # ---- dense comparator: same kernels, every tile active ---------------------------------------
    dense_sec = None
    if not args.no_dense:
        dense_model = nb.new_model(derive_input_mask=False, async_masks=not args.sync_masks, plan_first=args.plan_first)
        dense_sec, _, _ = nb.timed_run(dense_model, "dense (all tiles active, same kernels)", repeats=max(3, args.repeats // 2))
        del dense_model

    # ---- other densities (same network, same kernels) ------------------------------------------------
    sweep = None
    if args.sweep and wl.net == "e2depth":
        sweep = {"%.2f" % dens: dict(ms_per_step=round(1e3 * sec_per_step, 4), frames_per_s=round(NB / sec_per_step, 1))}
        for p in (0.01, 0.20):
            if abs(p - dens) < 1e-9:
                continue
            nb.set_density(p)
            t, _, _ = nb.timed_run(model, "incremental %.0f%%" % (100 * p), repeats=max(3, args.repeats // 2))
            sweep["%.2f" % p] = dict(ms_per_step=round(1e3 * t, 4), frames_per_s=round(NB / t, 1))
        nb.set_density(dens)

    # ---- dense refresh ---------------------------------------------------------------------------------
    refresh = nb.refresh_timing(model) if args.refresh else None

    # ---- lossy frontier --------------------------------------------------------------------------------
    lossy = None
    if args.lossy and wl.net == "e2depth":
        from maskedincrementeval_amd.lossy import lossy_frontier
        lossy = lossy_frontier(nb, model, log)

    # ---- the other benchmark configurations ---------------------------------------------------------
    configs = None
    if args.configs:
        configs = {}
        configs["c1_single_conv3x3_32to32_264x352_d05"] = config1_single_conv(torch, ops, _lib)
        configs["c2_conv_leakyrelu_relu_64ch_132x176"] = config2_activation_chain(torch, ops, _lib)
        short = dict(steps=min(args.steps, 50), repeats=max(3, args.repeats // 2))
        for dec in ("transposed", "upsample"):
            configs["c4_evflownet_incr_256x256_%s" % dec] = side_config(
                torch, ops, args, Workload("evflownet", 256, 256, 1, 0.03, "f32", dec), [0.03], **short)
        configs["c5_e2depth_incr_bf16_8x480x640"] = side_config(
            torch, ops, args, Workload("e2depth", 480, 640, 8, 0.01, "bf16"), [0.01, 0.20], n_inputs=4,
            steps=min(args.steps, 20), repeats=max(3, args.repeats // 2))

    # ---- CPU baseline: the oracle (torch-CPU restatement of the reference path) -----------------
    cpu = oracle_check = None
    if args.cpu_steps > 0 and args.in_threshold is None:       # the oracle restates the exact network
        torch.set_num_threads(min(os.cpu_count() or 1, 16))
        if args.net == "evflownet":
            from oracle.evflownet_oracle import EVFlowNetOracle
            oracle = EVFlowNetOracle(model.state_dict(), decoder=wl.decoder)
        else:
            from oracle.e2depth_oracle import E2DepthOracle
            oracle = E2DepthOracle(model.state_dict())
        with torch.no_grad():
            # The oracle as the checker: a fresh instance of the timed network (same weights) takes the dense refresh
            # and the first incremental steps of the CPU run, and every output must match the oracle's.
            n_chk = 3
            chk = nb.new_model(async_masks=not args.sync_masks, plan_first=args.plan_first)
            if args.dtype == "f32":
                rtol, atol_of = 1e-4, lambda ref: 1e-5
            else:
                rtol, atol_of = 2e-2, lambda ref: 3 * 2.0 ** -8 * max(float(ref.abs().max()), 1e-3)
            worst = 0.0

            def compare(got, ref, what):
                nonlocal worst
                got = got.float().cpu()
                err = (got - ref).abs().max().item()
                worst = max(worst, err)
                if not torch.allclose(got, ref, rtol=rtol, atol=atol_of(ref)):
                    raise SystemExit("bench: %s differs from the CPU oracle (max |difference| %.3e)" % (what, err))

            ref0 = oracle.refresh(nb.x0)
            got0 = nb.refresh_out(nb.refresh_net(chk, nb.cl(nb.x0)))
            if args.net == "evflownet":
                ref0 = ref0[-1]
            compare(got0, ref0, "the dense refresh")
            for i in range(n_chk):
                ref = oracle.incr(nb.deltas_cpu[i % nb.n_inputs])
                if args.net == "evflownet":
                    ref = ref[-1]
                compare(nb.out_of(nb.step_eager(chk, i)), ref, "incremental step %d" % i)
            oracle_check = dict(max_abs_diff=worst, steps=n_chk, rtol=rtol, atol=atol_of(ref),
                                against="CPU oracle, same weights and inputs: dense refresh + %d incremental steps" % n_chk)
            log("oracle check: refresh + %d steps, max |difference| %.3e" % (n_chk, worst))
            del chk
            t0 = time.perf_counter()
            for i in range(args.cpu_steps):
                oracle.incr(nb.deltas_cpu[(n_chk + i) % nb.n_inputs])
            cdt = (time.perf_counter() - t0) / args.cpu_steps
        cpu = dict(value=round(NB / cdt, 3), unit="frames/s", cores=torch.get_num_threads(), kind="port",
                   ms_per_step=round(1e3 * cdt, 2),
                   sample="%d incremental steps of the same %s %dx%d workload (dense F.conv2d on the "
                          "delta, as the reference executes it), torch-CPU fp32" % (args.cpu_steps, NET_NAME, H, W))
        log("cpu baseline: %.1f ms/frame on %d threads" % (1e3 * cdt, cpu["cores"]))

    x3 = args.dtype == "f32" and ops.f32_matmul == "bf16x3"
    # one basis for every matrix-core fraction of the line: the peak of the instruction that runs (for fp32 deltas
    # in the three-term form the bf16 peak over the six term products of a multiply)
    mfma_peak = PEAK_BF16_MFMA_TFLOPS / 6.0 if x3 else nb.peak_mfma
    detail = {
        "metric": "incremental frames/s + HBM GB/s, %s %dx%d @%g%% delta density" % (NET_NAME, H, W, 100 * dens),
        "value": round(NB / sec_per_step, 2),
        "unit": "frames/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(1e3 * sec_per_step, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": args.dtype,
        "data": "synthetic",
        "config": {"workload": "%s recurrent UNet, random init, %dx%dx%dx%d event voxel deltas, %.0f%% "
                               "active pixels, 1 dense refresh then incremental steps" % (NET_NAME, NB, BINS, H, W, 100 * dens),
                   "density": dens, "height": H, "width": W, "batch": NB, "graph": not args.no_graph, "input": "copied per step" if args.copy_input else "read in place",
                   "timing": "median of %d repeats of %d steps" % (args.repeats, args.steps),
                   "f32_matmul": ops.f32_matmul if args.dtype == "f32" else None,
                   "arithmetic": ARITHMETIC["bf16" if args.dtype == "bf16" else ops.f32_matmul],
                   "mask_planning": {"streams": "one step ahead: plan and compute halves are graphs of their own on two streams, events between the replays",
                                     "host": "one step ahead: plan and compute halves are graphs of their own on two streams, the host keeps their order (it waits for the plan's event before it launches the step, for the step before last before it launches the plan)",
                                     "fork": "one step ahead: the next step's plan forked inside this step's graph",
                                     None: ("inline" if (args.sync_masks or args.in_threshold is not None) else
                                            ("second stream, builds first" if args.plan_first else "second stream"))
                                     }[nb.plan_ahead_mode()],
                   **({"in_threshold": args.in_threshold} if args.in_threshold is not None else {})},
        "roofline": roofline,
        "cpu_baseline": cpu,
        "repeats_ms_per_step": repeats_ms,
        "whole_frame": {"algorithmic_mb": round(tot_bytes / 1e6, 2), "algorithmic_gflop": round(tot_flops / 1e9, 3),
                        "hbm_gbs": round(tot_bytes / sec_per_step / 1e9, 1),
                        "hbm_frac": round(tot_bytes / sec_per_step / 1e9 / PEAK_HBM_GBS, 5),
                        "mfma_tflops": round(tot_flops / sec_per_step / 1e12, 2),
                        "mfma_frac": round(tot_flops / sec_per_step / 1e12 / mfma_peak, 4),
                        "mfma_peak_tflops": round(mfma_peak, 1),
                        "sum_eager_launch_us": round(tot_us, 1),     # per-launch table: eager, one-set mask builds, an event pair per call
                        },
        "f32_native_mfma": native,
        "dense_same_kernels_ms": None if dense_sec is None else round(1e3 * dense_sec, 4),
        "speedup_vs_dense": None if dense_sec is None else round(dense_sec / sec_per_step, 3),
        "density_sweep": sweep,
        "refresh": refresh,
        "lossy_frontier": lossy,
        "configs": configs,
        "output_check": output_check,
        "oracle_check": oracle_check,
        "layers": layers,
    }
    # The bulky tables go to a side file and to stderr; stdout carries one compact line.
    try:
        os.makedirs(os.path.dirname(os.path.abspath(args.detail_file)), exist_ok=True)
        with open(args.detail_file, "w") as f:
            json.dump(detail, f, indent=1)
        log("full tables written to %s" % args.detail_file)
    except OSError as e:
        log("could not write %s: %s" % (args.detail_file, e))
        args.detail_file = None
    print(compact_line(detail, args.detail_file))


ARITHMETIC = {
    "bf16x3": "fp32 deltas, reservoirs, accumulators; matrix-core products as three bf16 terms per value "
              "(six term products per multiply, fp32-class error: tests/test_gpu_f32x3.py)",
    "native": "fp32 deltas, reservoirs, accumulators and matrix-core instruction",
    "bf16": "bf16 deltas and weights, fp32 reservoirs and accumulators",
}
LINE_LIMIT = 6000        # characters of the stdout line (the driver keeps the tail of stdout only)


def _pick(d, keys):
    return None if d is None else {k: d[k] for k in keys if k in d}


def compact_line(detail, detail_file=None):
    """The one JSON line of stdout: the contract keys, `roofline`, `cpu_baseline` and a summary of everything else
    (one {ms_per_step | us, frac, bound, kernel} entry per configuration and density).  The per-launch table, the
    lossy frontier, per-repeat lists and the full `configs` block stay in `detail` (side file, stderr)."""
    line = {k: detail[k] for k in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step",
                                   "higher_is_better", "scaling", "vs_baseline", "dtype", "data")}
    line["config"] = detail["config"]
    roof = detail["roofline"]
    line["roofline"] = _pick(roof, ("bound", "achieved", "peak", "unit", "frac", "traffic", "kernel", "us", "peak_basis",
                                    "frac_of_fp32_mfma_peak", "algorithmic_bytes", "algorithmic_flops"))
    line["cpu_baseline"] = detail["cpu_baseline"]
    line["whole_frame"] = detail.get("whole_frame")
    nat = detail.get("f32_native_mfma")
    line["f32_native_mfma_ms"] = None if nat is None else nat["ms_per_step"]
    line["dense_same_kernels_ms"] = detail.get("dense_same_kernels_ms")
    line["speedup_vs_dense"] = detail.get("speedup_vs_dense")
    sweep = detail.get("density_sweep")
    line["density_sweep_ms"] = None if sweep is None else {p: r["ms_per_step"] for p, r in sweep.items()}
    ref = detail.get("refresh")
    line["refresh_ms"] = None if ref is None else ref["ms_graph"]
    lossy = detail.get("lossy_frontier")
    if lossy is not None:
        best = max((r for r in lossy["points"] if r["method"] != "exact"), key=lambda r: r["speedup"], default=None)
        line["lossy"] = dict(exact_ms=lossy["exact_inline_ms_per_step"], captured=lossy.get("captured"),
                             reaches_5x=bool(lossy["reaches_5x"]),
                             fastest=_pick(best, ("method", "param", "ms_per_step", "speedup", "max_abs_deviation")),
                             threshold_0p01=_pick(next((r for r in lossy["points"] if r["method"] == "threshold"
                                                        and r["param"] == 1e-2), None),
                                                  ("ms_per_step", "speedup", "max_abs_deviation")))
    cfgs = detail.get("configs")
    if cfgs is not None:
        out = {}
        for name, c in cfgs.items():
            if "densities" in c:                      # a network configuration
                for p, r in c["densities"].items():
                    d = r["dominant"]
                    out["%s@%s" % (name, p)] = dict(ms_per_step=r["ms_per_step"], frac=d["frac"], bound=d["bound"],
                                                    kernel=d["kernel"], us=d["us"])
                out[name + "@dense"] = c.get("dense_same_kernels_ms")
            elif "delta_only" in c:                   # the single conv
                for form in ("delta_only", "fused_reservoir_relu"):
                    out["%s/%s" % (name, form)] = dict(us=c[form]["us"], frac=c[form]["hbm_frac"], bound="hbm",
                                                       kernel="mie_conv_masked 3x3 s1 32->32 @264x352")
            else:                                      # the activation chain, one entry per density
                for p, r in c.items():
                    if isinstance(r, dict):
                        out["%s@%s" % (name, p)] = dict(us=r["us_per_step"], frac=r["hbm_frac"], bound="hbm",
                                                        kernel="conv3x3 64->64 + LeakyReLU + ReLU increments")
        out["note"] = "c1/c2: us per call from a replayed HIP graph of 48-50 identical calls (kernel time, not host call rate)"
        line["configs"] = out
    line["output_check"] = _pick(detail.get("output_check"), ("max_abs_diff", "frames", "against"))
    line["oracle_check"] = detail.get("oracle_check")
    line["detail_file"] = detail_file
    text = json.dumps(line)
    if len(text) > LINE_LIMIT:
        # never let the line outgrow what the driver keeps: drop the optional parts, largest first
        for key in ("configs", "lossy", "whole_frame", "density_sweep_ms", "output_check"):
            line[key] = None
            text = json.dumps(line)
            if len(text) <= LINE_LIMIT:
                break
    return text


if __name__ == "__main__":
    main()
