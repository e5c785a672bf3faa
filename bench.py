#!/usr/bin/env python3
"""Benchmark of the masked incremental inference path on one MI355X.

Workload (the configuration the headline metric is quoted on): E2Depth-incr,
random-init weights, one event stream of 5x264x352 voxel grids, one dense
refresh, then incremental steps with 5 % of the pixels carrying a delta
(Poisson(2) event counts x random polarity x 0.1 per bin, smooth blob masks).
A "step" is one incremental frame through the whole network; the deltas are
resident in HBM before the timed region starts and the step is replayed from
a HIP graph.

Prints ONE JSON line: frames/s (`value`), ms/frame, the roofline of the
dominant kernel launch (the masked conv layer that takes the most time,
timed with HIP events on the stream it runs on), a per-layer table, the same
network run densely through the same kernels (all tiles active), and the CPU
baseline (the torch-CPU oracle of the reference path on the host cores).
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_FP32_MFMA_TFLOPS = 157.3
PEAK_BF16_MFMA_TFLOPS = 2500.0
PEAK_HBM_GBS = 8000.0


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--density", type=float, default=0.05)
    ap.add_argument("--height", type=int, default=264)
    ap.add_argument("--width", type=int, default=352)
    ap.add_argument("--batch", type=int, default=1, help="independent event streams per step (8 with 480x640: the batched configuration)")
    ap.add_argument("--cpu-steps", type=int, default=400, help="incremental steps of the CPU baseline (0 = skip)")
    ap.add_argument("--no-graph", action="store_true", help="launch kernels eagerly instead of replaying a HIP graph")
    ap.add_argument("--no-dense", action="store_true", help="skip the all-tiles-active comparator")
    ap.add_argument("--layer-iters", type=int, default=20, help="timed launches per layer for the roofline table")
    ap.add_argument("--no-plan-first", dest="plan_first", action="store_false",
                    help="enqueue each mask build right before its consumer instead of all builds of a step first")
    ap.add_argument("--upconv-all", action="store_true",
                    help="take the one-kernel up-sampling conv for every decoder layer, whatever its size (for measurements)")
    ap.add_argument("--sync-masks", action="store_true", help="build tile sets on the compute stream (no planning stream)")
    ap.add_argument("--net", choices=["e2depth", "evflownet"], default="e2depth",
                    help="e2depth: the headline network (5 bins); evflownet: EVFlowNet-incr, 4 bins, up-sampling decoders "
                         "(the reference's optical-flow configuration: use --height 256 --width 256 --density 0.03)")
    ap.add_argument("--dtype", choices=["f32", "bf16"], default="f32",
                    help="element type of deltas and weights (reservoirs and accumulation stay fp32)")
    ap.add_argument("--kfence-tp", type=float, default=0.0,
                    help="also time the net with every conv's delta quantiser on (k = tp*||x||); reported under \"kfenced\"")
    ap.add_argument("--sweep", action="store_true", help="also time 1 %% and 20 %% density (reported under \"density_sweep\")")
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

        self._wrap("conv_masked", conv_desc)
        self._wrap("upconv_masked", upconv_desc)
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
                else:
                    byts += a_out * cout * es
                    if d["fused"]:
                        byts += 2 * a_out * cout * 4
                row.update(shape="%s%dx%d s%d %d->%d%s @%dx%d" % ("up2x+" if d.get("up") else "", k, k, d["s"], cin, cout,
                                                                   "+lstm" if d.get("gates") else "", ts.h, ts.w),
                           active_tiles=int(ts.counts[0].item()), tiles=ts.capacity, a_out=a_out,
                           bytes=byts, flops=2 * a_out * cin * cout * k * k)
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


def main():
    args = parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures ONE GPU (independent event streams shard one per GPU with "
              "no communication); --gpus %d is not run." % args.gpus, file=sys.stderr)
        sys.exit(2)
    import torch
    from maskedincrementeval_amd import _lib, ops
    from maskedincrementeval_amd.e2depth_incr import E2VIDRecurrentIncr
    from maskedincrementeval_amd.synthetic import event_voxel_delta, seed_module_

    _lib.lib()   # fail loudly if the HIP library is missing
    if args.upconv_all:
        ops.upconv_max_tiles = ops.upconv_max_chunks = 1 << 30
    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        sys.exit(2)
    dev = torch.device("cuda:0")
    H, W, dens, NB = args.height, args.width, args.density, args.batch
    dt = torch.bfloat16 if args.dtype == "bf16" else torch.float32
    es = 2 if args.dtype == "bf16" else 4          # bytes per delta / weight element
    peak_mfma = PEAK_BF16_MFMA_TFLOPS if args.dtype == "bf16" else PEAK_FP32_MFMA_TFLOPS
    cl = lambda t: t.to(dev).to(dt).contiguous(memory_format=torch.channels_last)

    # the two networks differ in their call conventions only: adapters
    if args.net == "evflownet":
        from maskedincrementeval_amd.evflownet_incr import MultiResUNetRecurrentIncr
        BINS, NET_NAME = 4, "EVFlowNet-incr"
        make_net = lambda **kw: MultiResUNetRecurrentIncr(num_bins=4, **kw)
        run_net = lambda m, x: m([x, None])
        out_of = lambda r: r[-1][0]                      # the finest flow scale
        refresh_net = lambda m, x: m.forward_refresh_reservoirs(x)
        refresh_out = lambda r: r[-1]
    else:
        BINS, NET_NAME = 5, "E2Depth-incr"
        make_net = E2VIDRecurrentIncr
        run_net = lambda m, x: m([x, None], None)
        out_of = lambda r: r[0][0]
        refresh_net = lambda m, x: m.forward_refresh_reservoirs(x, None)
        refresh_out = lambda r: r[0]

    model = seed_module_(make_net(async_masks=not args.sync_masks, plan_first=args.plan_first), seed=1).to(dev).eval()
    x0 = torch.randn(NB, BINS, H, W, generator=torch.Generator().manual_seed(2)) * 0.5
    n_inputs = 16
    deltas_cpu = [event_voxel_delta(NB, BINS, H, W, dens, seed=3000 + i)[0] for i in range(n_inputs)]
    deltas = [cl(d) for d in deltas_cpu]
    static_in = cl(torch.zeros(NB, BINS, H, W))

    def step_eager(m, i):
        static_in.copy_(deltas[i % n_inputs])
        return run_net(m, static_in)

    output_check = {}

    def timed_run(m, tag, check_against=None):
        history = []                                       # input index of every step the model takes
        with torch.no_grad():
            refresh_net(m, cl(x0))
            for i in range(max(args.warmup, 3)):           # also allocates every persistent buffer
                step_eager(m, i)
                history.append(i)
            torch.cuda.synchronize()
            graph = None
            if not args.no_graph:
                side = torch.cuda.Stream()
                side.wait_stream(torch.cuda.current_stream())
                with torch.cuda.stream(side):
                    step_eager(m, 0)
                history.append(0)
                torch.cuda.current_stream().wait_stream(side)
                torch.cuda.synchronize()
                graph = torch.cuda.CUDAGraph()
                with torch.cuda.graph(graph):
                    graph_out = out_of(run_net(m, static_in))
                for i in range(3):
                    static_in.copy_(deltas[i % n_inputs])
                    graph.replay()
                    history.append(i)
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for i in range(args.steps):
                if graph is not None:
                    static_in.copy_(deltas[i % n_inputs])
                    graph.replay()
                else:
                    step_eager(m, i)
            torch.cuda.synchronize()
            dt = time.perf_counter() - t0
            history.extend(range(args.steps))
            if check_against is not None:
                # The timed configuration (graph replay, planning stream) against the plain one: a second
                # instance of the network with eager launches and inline mask planning takes the same
                # steps; the next frames of the two must then agree (same kernels over the same tiles).
                ref = check_against()
                refresh_net(ref, cl(x0))
                for i in history:
                    run_net(ref, deltas[i % n_inputs])
                worst = 0.0
                for i in range(4):
                    want = out_of(run_net(ref, deltas[i % n_inputs]))
                    if graph is not None:
                        static_in.copy_(deltas[i % n_inputs])
                        graph.replay()
                        got = graph_out
                    else:
                        got = out_of(step_eager(m, i))
                    worst = max(worst, (got.float() - want.float()).abs().max().item())
                torch.cuda.synchronize()
                output_check.update(max_abs_diff=worst, frames=4, steps_before=len(history),
                                    against="same network, eager launches, inline mask planning")
                print("[bench] %s: max |difference| to the eager inline-planning network over 4 frames after %d steps: %.3e"
                      % (tag, len(history), worst), file=sys.stderr, flush=True)
                if not worst <= 1e-3:
                    raise SystemExit("bench: the timed configuration does not reproduce the plain one (%.3e)" % worst)
        print("[bench] %s: %.3f ms/frame over %d steps (%s)" % (tag, 1e3 * dt / args.steps, args.steps,
              "eager" if graph is None else "HIP graph"), file=sys.stderr, flush=True)
        return dt / args.steps

    sec_per_step = timed_run(model, "incremental %.0f%%" % (100 * dens),
                             check_against=lambda: seed_module_(make_net(), seed=1).to(dev).eval())

    # ---- per-layer roofline table: eager launches with HIP events, several repeats ------------
    with torch.no_grad():
        model.plan_first = False          # one walk per step: the probe times every wrapper call once
        refresh_net(model, cl(x0))
        step_eager(model, 0)
        agg = None
        for it in range(args.layer_iters):
            with LayerProbe(ops, torch, es) as probe:
                step_eager(model, 1 + it)
            rows = probe.table()
            if agg is None:
                agg = rows
                for r in agg:
                    r["ms_sum"] = 0.0
                    r["bytes_sum"] = 0
                    r["flops_sum"] = 0
            for r, q in zip(agg, rows):
                r["ms_sum"] += q["ms"]
                r["bytes_sum"] += q["bytes"]
                r["flops_sum"] += q["flops"]
    layers = []
    for r in agg:
        ms = r["ms_sum"] / args.layer_iters
        byts, fl = r["bytes_sum"] / args.layer_iters, r["flops_sum"] / args.layer_iters
        layers.append(dict(op=r["op"], shape=r["shape"], us=round(1e3 * ms, 2),
                           gbs=round(byts / (ms * 1e-3) / 1e9, 1) if ms > 0 else None,
                           tflops=round(fl / (ms * 1e-3) / 1e12, 2) if ms > 0 else None,
                           bytes=int(byts), flops=int(fl), active_tiles=r.get("active_tiles"), tiles=r.get("tiles")))
    convs = [l for l in layers if l["op"] in ("conv_masked", "conv_gates_incr", "upconv_masked")]
    dom = max(convs, key=lambda l: l["us"])
    # Re-time the dominant launch on its own: the same call (same tile set, same buffers)
    # replayed back to back between two HIP events on the launch stream.
    orig, cargs, ckw = agg[layers.index(dom)]["call"]
    reps = 50
    with torch.no_grad():
        for _ in range(5):
            orig(*cargs, **ckw)
        ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        ev0.record()
        for _ in range(reps):
            orig(*cargs, **ckw)
        ev1.record()
        torch.cuda.synchronize()
    dom_us = 1e3 * ev0.elapsed_time(ev1) / reps
    dom = dict(dom, us=round(dom_us, 2), gbs=round(dom["bytes"] / dom_us / 1e3, 1),
               tflops=round(dom["flops"] / dom_us / 1e6, 2))
    mfma_bound = dom["flops"] / max(dom["bytes"], 1) > peak_mfma * 1e12 / (PEAK_HBM_GBS * 1e9)
    if mfma_bound:
        roofline = dict(bound="mfma", achieved=dom["tflops"], peak=peak_mfma, unit="TFLOP/s",
                        frac=round(dom["tflops"] / peak_mfma, 4), traffic=None)
    else:
        roofline = dict(bound="hbm", achieved=dom["gbs"], peak=PEAK_HBM_GBS, unit="GB/s",
                        frac=round(dom["gbs"] / PEAK_HBM_GBS, 4), traffic=None)
    roofline.update(kernel="mie_conv_masked %s" % dom["shape"], us=dom["us"],
                    algorithmic_bytes=dom["bytes"], algorithmic_flops=dom["flops"])
    # HBM bytes per launch of that kernel from the committed rocprofv3 --pmc summary, if it
    # covers this shape (FETCH_SIZE + WRITE_SIZE, scaled by the copy-kernel calibration)
    try:
        with open(os.path.join(ROOT, "profiles", "pmc_traffic.json")) as f:
            roofline["traffic"] = json.load(f).get(dom["shape"], {}).get("hbm_bytes_per_launch")
    except OSError:
        pass
    tot_us = sum(l["us"] for l in layers)
    tot_bytes = sum(l["bytes"] for l in layers)
    tot_flops = sum(l["flops"] for l in layers)
    print("[bench] per-launch table (eager, HIP events, mean of %d steps):" % args.layer_iters, file=sys.stderr)
    for l in layers:
        print("[bench]   %-22s %-34s %9.2f us %8s GB/s %7s TFLOP/s  tiles %s/%s" % (
            l["op"], l["shape"], l["us"], l["gbs"], l["tflops"], l["active_tiles"], l["tiles"]), file=sys.stderr)
    print("[bench]   sum of kernels %.1f us; algorithmic %.1f MB, %.2f GFLOP per frame" %
          (tot_us, tot_bytes / 1e6, tot_flops / 1e9), file=sys.stderr, flush=True)

    # ---- dense comparator: same kernels, every tile active ---------------------------------------
    model.plan_first = args.plan_first
    dense_sec = None
    if not args.no_dense:
        dense_model = seed_module_(make_net(derive_input_mask=False, async_masks=not args.sync_masks,
                                            plan_first=args.plan_first), seed=1).to(dev).eval()
        dense_sec = timed_run(dense_model, "dense (all tiles active, same kernels)")
        del dense_model

    # ---- lossy variant: delta quantiser in front of every conv ------------------------------------
    kfenced = None
    if args.kfence_tp > 0:
        from maskedincrementeval_amd.mask_incr_modules import set_kfence
        kf_model = seed_module_(make_net(async_masks=not args.sync_masks), seed=1).to(dev).eval()
        set_kfence(kf_model, args.kfence_tp)
        t = timed_run(kf_model, "quantised deltas (tp = %g)" % args.kfence_tp)
        # deviation of the accumulated prediction from the exact incremental net, same inputs
        with torch.no_grad():
            acc = []
            for m in (model, kf_model):
                pred = refresh_out(refresh_net(m, cl(x0))).clone()
                for i in range(n_inputs):
                    pred += out_of(step_eager(m, i))
                acc.append(pred)
            torch.cuda.synchronize()
            dev_abs = (acc[0] - acc[1]).abs().max().item()
        kfenced = dict(tp=args.kfence_tp, ms_per_step=round(1e3 * t, 4), frames_per_s=round(1 / t, 1),
                       max_abs_deviation_after_16_steps=dev_abs)
        print("[bench] quantised deltas: max |deviation| of the prediction after %d steps = %.3e" %
              (n_inputs, dev_abs), file=sys.stderr, flush=True)
        del kf_model

    # ---- other densities (same network, same kernels) ------------------------------------------------
    sweep = None
    if args.sweep:
        sweep = {"%.2f" % dens: dict(ms_per_step=round(1e3 * sec_per_step, 4), frames_per_s=round(1 / sec_per_step, 1))}
        keep = list(deltas)
        for p in (0.01, 0.20):
            if abs(p - dens) < 1e-9:
                continue
            deltas[:] = [cl(event_voxel_delta(NB, 5, H, W, p, seed=3000 + i)[0]) for i in range(n_inputs)]
            t = timed_run(model, "incremental %.0f%%" % (100 * p))
            sweep["%.2f" % p] = dict(ms_per_step=round(1e3 * t, 4), frames_per_s=round(1 / t, 1))
        deltas[:] = keep

    # ---- CPU baseline: the oracle (torch-CPU restatement of the reference path) -----------------
    cpu = None
    if args.cpu_steps > 0:
        torch.set_num_threads(min(os.cpu_count() or 1, 16))
        if args.net == "evflownet":
            from oracle.evflownet_oracle import EVFlowNetOracle
            oracle = EVFlowNetOracle(model.state_dict(), decoder="upsample")
        else:
            from oracle.e2depth_oracle import E2DepthOracle
            oracle = E2DepthOracle(model.state_dict())
        with torch.no_grad():
            oracle.refresh(x0)
            oracle.incr(deltas_cpu[0])
            t0 = time.perf_counter()
            for i in range(args.cpu_steps):
                oracle.incr(deltas_cpu[(1 + i) % n_inputs])
            cdt = (time.perf_counter() - t0) / args.cpu_steps
        cpu = dict(value=round(NB / cdt, 3), unit="frames/s", cores=torch.get_num_threads(), kind="port",
                   ms_per_step=round(1e3 * cdt, 2),
                   sample="%d incremental steps of the same %s %dx%d workload (dense F.conv2d on the "
                          "delta, as the reference executes it), torch-CPU fp32" % (args.cpu_steps, NET_NAME, H, W))
        print("[bench] cpu baseline: %.1f ms/frame on %d threads" % (1e3 * cdt, cpu["cores"]), file=sys.stderr, flush=True)

    result = {
        # the headline metric's name; `value` is its frames/s part, the HBM GB/s part is in
        # "hbm_gbs_whole_frame" and per launch in "layers"
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
                   "density": dens, "height": H, "width": W, "batch": NB, "graph": not args.no_graph,
                   "mask_planning": "inline" if args.sync_masks else ("second stream, builds first" if args.plan_first else "second stream")},
        "roofline": roofline,
        "cpu_baseline": cpu,
        "hbm_gbs_whole_frame": round(tot_bytes / sec_per_step / 1e9, 1),
        "hbm_frac_whole_frame": round(tot_bytes / sec_per_step / 1e9 / PEAK_HBM_GBS, 5),
        "algorithmic_mb_per_frame": round(tot_bytes / 1e6, 2),
        "algorithmic_gflop_per_frame": round(tot_flops / 1e9, 3),
        "sum_kernel_us": round(tot_us, 1),
        "dense_same_kernels_ms": None if dense_sec is None else round(1e3 * dense_sec, 4),
        "speedup_vs_dense": None if dense_sec is None else round(dense_sec / sec_per_step, 3),
        "density_sweep": sweep,
        "kfenced": kfenced,
        "output_check": output_check,
        "layers": layers,
    }
    print(json.dumps(result))


if __name__ == "__main__":
    main()
