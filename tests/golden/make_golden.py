"""Writes tests/golden/vectors.npz: small seeded input / expected-output vectors for the hot path.

The reference holds no golden vectors of its own (its tests assert identities, tests/test_pointops.py,
tests/test_network.py) and its Python cannot be imported here, so these vectors come from this
repository's CPU oracle (oracle/), which tests/test_oracle_pinning.py pins against closed forms,
brute force and torch library routines.  They freeze that pinned behaviour: a later change of the
oracle or of a kernel that moves a result shows up against data, not only against the oracle of
the day.  Run from the repository root:  python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

from maskedincrementeval_amd.synthetic import (blob_mask, gaussian_delta, he_normal_conv_weight,  # noqa: E402
                                               random_events)
from oracle import events_oracle as eo  # noqa: E402
from oracle import incr_oracle as io  # noqa: E402
from oracle import mask_oracle as mo  # noqa: E402


def main():
    torch.manual_seed(0)
    out = {}
    # 1. masks: footprints, ordered tile lists, stale lists over two steps
    m0 = np.stack([blob_mask(37, 53, 0.06, seed=11 + b) for b in range(2)])
    m1 = np.stack([blob_mask(37, 53, 0.04, seed=21 + b) for b in range(2)])
    out["mask_in0"], out["mask_in1"] = m0, m1
    for k, s, p in ((3, 1, 1), (5, 2, 2)):
        f0, f1 = mo.footprint_conv(m0, k, s, p), mo.footprint_conv(m1, k, s, p)
        t0, t1 = mo.tile_list(f0), mo.tile_list(f1)
        tag = "k%ds%d" % (k, s)
        out["foot0_" + tag], out["foot1_" + tag] = f0, f1
        out["tiles0_" + tag], out["tiles1_" + tag] = t0, t1
        out["stale1_" + tag] = mo.stale_list(t0, t1)
    out["foot_up2x"] = mo.footprint_up2x(m0)
    # 2. conv3x3 -> LeakyReLU(0.01) -> ReLU chain, three steps (the activation-chain configuration in small)
    n, c, h, w = 1, 8, 16, 24
    wt = he_normal_conv_weight(8, c, 3, seed=3)
    r_leaky = torch.randn(n, 8, h, w, generator=torch.Generator().manual_seed(4))
    r_relu = io.leaky_relu(r_leaky).clone()
    out["chain_w"], out["chain_r0"] = wt.numpy(), r_leaky.numpy()
    res1, res2 = io.Reserve(r_leaky.clone()), io.Reserve(r_relu.clone())
    for step in range(3):
        d, m = gaussian_delta(n, c, h, w, 0.08, 0.2, seed=50 + step)
        y = io.conv_incr(d, wt, 1, 1)
        y = io.act_incr(io.leaky_relu, res1, y)
        y = io.act_incr(torch.relu, res2, y)
        out["chain_d%d" % step], out["chain_m%d" % step] = d.numpy(), m.numpy()
        out["chain_out%d" % step] = y.numpy()
    out["chain_res_leaky"], out["chain_res_relu"] = res1.reservoir.numpy(), res2.reservoir.numpy()
    # 3. fused ConvLSTM gate chain, two steps
    hid, cin = 8, 8
    gw = he_normal_conv_weight(4 * hid, cin + hid, 3, seed=6)
    gb = torch.randn(4 * hid, generator=torch.Generator().manual_seed(7)) * 0.1
    x0 = torch.randn(1, cin, 12, 16, generator=torch.Generator().manual_seed(8))
    cell = io.ConvLSTMOracle(gw, gb, hid)
    h0, c0 = cell.refresh(x0, None)
    out["lstm_w"], out["lstm_b"], out["lstm_x0"] = gw.numpy(), gb.numpy(), x0.numpy()
    out["lstm_h0"], out["lstm_c0"] = h0.numpy(), c0.numpy()
    for step in range(2):
        d, m = gaussian_delta(1, cin, 12, 16, 0.1, 0.3, seed=60 + step)
        dh, dc = cell.incr(d)
        out["lstm_d%d" % step], out["lstm_m%d" % step] = d.numpy(), m.numpy()
        out["lstm_dh%d" % step], out["lstm_dc%d" % step] = dh.numpy(), dc.numpy()
    # 4. delta quantiser, three steps
    carry = io.Reserve(torch.zeros(1, 4, 16, 16))
    for step in range(3):
        d, m = gaussian_delta(1, 4, 16, 16, 0.2, 0.1, seed=70 + step)
        f = io.kfenced(carry, torch.tensor(0.125), d)
        out["kf_d%d" % step], out["kf_m%d" % step], out["kf_f%d" % step] = d.numpy(), m.numpy(), f.numpy()
    out["kf_carry"] = carry.reservoir.numpy()
    # 5. event front end: frame and window delta with reflection padding
    ev = random_events(1500, 30, 20, 0.0, 0.08, seed=5, density=0.3)
    out["ev"] = ev
    out["ev_frame"], out["ev_frame_mask"] = eo.frame(ev, "voxelgrid", 5, 20, 30, 0.05, 0.01, pad=(3, 3, 2, 2))
    out["ev_delta"], out["ev_delta_mask"] = eo.frame_delta(ev, "voxelgrid", 5, 20, 30, 0.05, 0.01, 0.012,
                                                           pad=(3, 3, 2, 2))
    ev_pm = ev.copy()
    ev_pm[:, 3] = np.where(ev_pm[:, 3] == 0, -1.0, ev_pm[:, 3])      # the histogram counts p == -1 / +1
    hist, hmask = eo.frame(ev_pm, "histogram", 5, 20, 30, 0.05, 0.01)
    out["ev_hist"], out["ev_hist_mask"] = hist, hmask
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "vectors.npz")
    np.savez_compressed(path, **{k: np.ascontiguousarray(v) for k, v in out.items()})
    print("wrote %s (%d arrays, %.1f KB)" % (path, len(out), os.path.getsize(path) / 1024))


if __name__ == "__main__":
    main()
