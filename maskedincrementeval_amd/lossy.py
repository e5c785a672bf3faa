"""The lossy frontier of the incremental path: how much faster a frame gets when small deltas are
suppressed, and what that costs in accuracy.

With exact masks the deltas of a 5 %-dense input densify with depth (a 5x5 head, three stride-2 stages
and the 3x3 ConvLSTM convs dilate every blob), so most of the network runs on every tile.  The reference
holds two ways to win sparsity back, both lossy:

* the delta quantiser `KFencedMaskModule` (incr_modules/mask_incr_modules.py:21-47): multiples of k pass,
  the remainder is carried to later steps, so the error per element stays below k / 2;
* a threshold mask, maxpool(abs(x)) >= thr (incr_modules/utils.py:22-25, utils/str_sparse_utils.py:10-11):
  pixels whose delta is small in every channel are dropped for good.

`lossy_frontier` switches one of them on in front of every conv, sweeps its parameter, and reports per
point: ms/frame (HIP graph, masks planned inline because they depend on values), the fraction of active
tiles per conv stage, and the deviation of the accumulated prediction after 50 steps from the exact
network on the same inputs.
"""
import statistics
import time

import torch

from . import _lib
from .mask_incr_modules import nnConvIncr, set_input_threshold, set_kfence


def conv_tile_fractions(model):
    """[(module name, active tiles, tiles)] of the output tile set every incremental conv built last."""
    rows = []
    for name, m in model.named_modules():
        if not isinstance(m, nnConvIncr):
            continue
        sets = [b for key, b in m._ib().items() if key[0] == "t"]
        if not sets:
            continue
        ts = max(sets, key=lambda t: t.capacity)      # its own output set (helper sets are never larger)
        best = max(int(t.counts[_lib.CNT_ACTIVE].item()) / t.capacity for t in sets if t.capacity == ts.capacity)
        rows.append((name, round(best, 4), ts.capacity))
    return rows


def lossy_frontier(nb, exact_model, log, steps=50, time_steps=50, repeats=5):
    """nb: bench.NetBench of the E2Depth-incr workload; exact_model: its loss-free network.  Returns a dict
    with one row per (method, parameter): ms_per_step, speedup over the exact incremental net,
    mean fraction of active tiles, per-stage fractions, max / mean |deviation| of the accumulated
    prediction after `steps` steps."""
    points = [("kfence_rms", tp) for tp in (0.02, 0.05, 0.1, 0.2, 0.5)] + \
             [("kfence_l2", 1e-4)] + \
             [("threshold", thr) for thr in (1e-4, 1e-3, 1e-2, 3e-2, 1e-1)]
    n_in = nb.n_inputs

    def accumulate(m):
        with torch.no_grad():
            pred = nb.refresh_out(nb.refresh_net(m, nb.cl(nb.x0))).float().clone()
            for i in range(steps):
                pred += nb.out_of(nb.step_eager(m, i)).float()
        torch.cuda.synchronize()
        return pred

    def timed(m):
        """ms/step from HIP graphs of one step with inline mask planning, one graph per resident input (a step
        reads its delta where it lies, as the exact network's timed steps do)."""
        with torch.no_grad():
            nb.refresh_net(m, nb.cl(nb.x0))
            for i in range(5):
                nb.step_eager(m, i)
            torch.cuda.synchronize()
            side = torch.cuda.Stream()
            side.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(side):
                nb.run_net(m, nb.deltas[0])
            torch.cuda.current_stream().wait_stream(side)
            torch.cuda.synchronize()
            graphs = []
            for i in range(n_in):
                g = torch.cuda.CUDAGraph()
                with torch.cuda.graph(g):
                    nb.run_net(m, nb.deltas[i])
                graphs.append(g)
            for i in range(n_in):
                graphs[i].replay()
            per = []
            for _ in range(repeats):
                torch.cuda.synchronize()
                t0 = time.perf_counter()
                for i in range(time_steps):
                    graphs[i % n_in].replay()
                torch.cuda.synchronize()
                per.append((time.perf_counter() - t0) / time_steps)
        return statistics.median(per)

    exact = accumulate(exact_model)
    base = nb.new_model()                                # exact masks, inline planning: the time to beat
    t_exact = timed(base)
    frac_exact = conv_tile_fractions(base)
    mean_exact = sum(f for _, f, _ in frac_exact) / len(frac_exact)
    rows = [dict(method="exact", param=None, ms_per_step=round(1e3 * t_exact, 4), speedup=1.0,
                 mean_active_tile_fraction=round(mean_exact, 4), max_abs_deviation=0.0, mean_abs_deviation=0.0,
                 stages={n_: f for n_, f, _ in frac_exact})]
    del base
    for method, param in points:
        m = nb.new_model()
        if method == "threshold":
            set_input_threshold(m, param)
        else:
            set_kfence(m, param, norm="rms" if method == "kfence_rms" else "l2")
        acc = accumulate(m)
        dev = (acc - exact).abs()
        t = timed(m)
        fr = conv_tile_fractions(m)
        mean_fr = sum(f for _, f, _ in fr) / len(fr)
        rows.append(dict(method=method, param=param, ms_per_step=round(1e3 * t, 4), speedup=round(t_exact / t, 3),
                         mean_active_tile_fraction=round(mean_fr, 4),
                         max_abs_deviation=round(dev.max().item(), 6), mean_abs_deviation=round(dev.mean().item(), 6),
                         stages={n_: f for n_, f, _ in fr}))
        log("lossy %-10s %-7g: %.3f ms/frame (x%.2f), active tiles %.0f %%, |deviation| after %d steps max %.2e mean %.2e"
            % (method, param, 1e3 * t, t_exact / t, 100 * mean_fr, steps, dev.max().item(), dev.mean().item()))
        del m
    torch.cuda.empty_cache()
    best = [r for r in rows if r["speedup"] >= 5.0]
    return dict(steps=steps, exact_inline_ms_per_step=round(1e3 * t_exact, 4), captured=True,
                note="prediction is a sigmoid output in (0, 1); deviation is of refresh + sum of %d increments "
                     "against the exact incremental network on the same inputs" % steps,
                reaches_5x=[dict(method=r["method"], param=r["param"], max_abs_deviation=r["max_abs_deviation"])
                            for r in best],
                points=rows)
