"""Single-kernel micro-benchmark: one masked conv layer (or a plain device copy) launched
repeatedly, timed with HIP events on the launch stream.

    python -m maskedincrementeval_amd.kernel_bench --cin 256 --cout 128 --k 5 --h 66 --w 88
    python -m maskedincrementeval_amd.kernel_bench --copy-mb 256

Meant to be run under `rocprofv3 --kernel-trace --stats` or `rocprofv3 --pmc ...`: the process
launches little else than the kernel of interest.  `--copy-mb` runs a device-to-device copy of
known size, the reference point for scaling FETCH_SIZE / WRITE_SIZE counter readings.
Prints one JSON line.
"""
import argparse
import json

import torch

from . import _lib, ops
from .masked_types import TileMask
from .synthetic import blob_mask, he_normal_conv_weight


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--cin", type=int, default=256)
    ap.add_argument("--cout", type=int, default=128)
    ap.add_argument("--k", type=int, default=5)
    ap.add_argument("--stride", type=int, default=1)
    ap.add_argument("--h", type=int, default=66)
    ap.add_argument("--w", type=int, default=88)
    ap.add_argument("--n", type=int, default=1)
    ap.add_argument("--density", type=float, default=1.0, help="fraction of active input pixels (1 = dense)")
    ap.add_argument("--fused-act", type=int, default=1, help="1: reservoir + ReLU epilogue, 0: plain delta")
    ap.add_argument("--path", choices=["auto", "valu", "mfma"], default="auto")
    ap.add_argument("--dtype", choices=["f32", "bf16"], default="f32", help="element type of the deltas and of the matrix-core filter copy")
    ap.add_argument("--iters", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--copy-mb", type=int, default=0, help="run a plain copy of this many MiB instead")
    ap.add_argument("--op", choices=["conv", "act", "mul", "add", "up2x", "gates", "mask"], default="conv",
                    help="conv (default), or one of the bandwidth-bound incremental ops on an n x cin x h x w delta: "
                         "act = reservoir + ReLU increment, mul = product-rule multiply, add = skip sum, "
                         "up2x = bilinear x2 of a sum of two deltas (h, w = output size), gates = ConvLSTM gate chain "
                         "(cin = hidden channels), mask = the tile-mask build of a k x k conv (footprint pass + ordered "
                         "tile compaction) over an n x h x w pixel mask")
    ap.add_argument("--up2x", action="store_true",
                    help="the conv reads up2x(a + b) of two deltas at half of --h/--w (mie_upconv_masked; 5x5 stride 1)")
    args = ap.parse_args()
    _lib.lib()
    dev = torch.device("cuda:0")
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)

    if args.copy_mb > 0:
        nbytes = args.copy_mb << 20
        src = torch.empty(nbytes // 4, dtype=torch.float32, device=dev).normal_()
        dst = torch.empty_like(src)
        for _ in range(args.warmup):
            dst.copy_(src)
        torch.cuda.synchronize()
        e0.record()
        for _ in range(args.iters):
            dst.copy_(src)
        e1.record()
        torch.cuda.synchronize()
        us = 1e3 * e0.elapsed_time(e1) / args.iters
        print(json.dumps(dict(kernel="copy", bytes_read=nbytes, bytes_written=nbytes, us=round(us, 2),
                              gbs=round(2 * nbytes / us / 1e3, 1), iters=args.iters)))
        return

    n, cin, cout, k, s, h, w = args.n, args.cin, args.cout, args.k, args.stride, args.h, args.w
    p = k // 2
    if args.op == "mask":
        return mask_build(args, dev, e0, e1)
    if args.op != "conv":
        return pointwise(args, dev, e0, e1)
    if args.up2x:
        return up2x_conv(args, dev, e0, e1)
    ho, wo = ops.conv_out_size(h, w, k, s, p)
    g = torch.Generator().manual_seed(0)
    x = torch.randn((n, cin, h, w), generator=g)
    if args.density < 1.0:
        m = torch.stack([torch.from_numpy(blob_mask(h, w, args.density, seed=b)) for b in range(n)]).view(n, 1, h, w)
        x = x * m.float()
        mask = m.to(dev)
    else:
        mask = None
    dt = torch.bfloat16 if args.dtype == "bf16" else torch.float32
    es = 2 if args.dtype == "bf16" else 4
    x = ops.as_nhwc(x.to(dev).to(dt).contiguous(memory_format=torch.channels_last))
    filt = ops.ConvFilter(he_normal_conv_weight(cout, cin, k, 0).permute(1, 2, 3, 0).contiguous().to(dev))
    ts = TileMask(n, ho, wo, dev)
    ops.build_mask_tiles(mask, None, n, h, w, _lib.FOOT_CONV, k, s, p, ts)
    out = ops.new_nhwc(n, cout, ho, wo, dev, dt)
    res = ops.new_nhwc(n, cout, ho, wo, dev) if args.fused_act else None
    act = _lib.ACT_RELU if args.fused_act else _lib.ACT_NONE
    path = dict(auto=_lib.PATH_AUTO, valu=_lib.PATH_VALU, mfma=_lib.PATH_MFMA)[args.path]

    def launch():
        ops.conv_masked(x, mask, None, None, filt, k, s, p, ts, out, res, act, 0.0, path)

    for _ in range(args.warmup):
        launch()
    torch.cuda.synchronize()
    e0.record()
    for _ in range(args.iters):
        launch()
    e1.record()
    torch.cuda.synchronize()
    us = 1e3 * e0.elapsed_time(e1) / args.iters
    a_in = n * h * w if mask is None else int(mask.sum().item())
    a_out = int(ts.pixmask.sum().item())
    tiles = int(ts.counts[0].item())
    flops = 2 * a_out * cin * cout * k * k
    # algorithmic bytes: mask, active delta, emitted delta, reservoir read+write, filter, tile list
    byts = n * h * w + a_in * cin * es + a_out * cout * es + cin * cout * k * k * es + ts.capacity * 4
    if args.fused_act:
        byts += 2 * a_out * cout * 4
    print(json.dumps(dict(kernel="mie_conv_masked", shape="%dx%d s%d %d->%d @%dx%d n=%d" % (k, k, s, cin, cout, ho, wo, n),
                          dtype=args.dtype, density=args.density, active_tiles=tiles, tiles=ts.capacity, us=round(us, 2),
                          algorithmic_flops=flops, algorithmic_bytes=byts,
                          tile_flops=2 * tiles * 64 * cin * cout * k * k,
                          tflops=round(flops / us / 1e6, 2), gbs=round(byts / us / 1e3, 1), iters=args.iters)))


def mask_build(args, dev, e0, e1):
    """The tile-mask build in front of a k x k conv: dilated pixel mask + tile flags (k_mask_footprint), then the
    ascending active / stale tile lists (k_compact_tiles).  Algorithmic bytes: input and output pixel masks, one
    flag word per tile read and written, the tile list."""
    n, k, s, h, w = args.n, args.k, args.stride, args.h, args.w
    p = k // 2
    ho, wo = ops.conv_out_size(h, w, k, s, p)
    m = torch.stack([torch.from_numpy(blob_mask(h, w, args.density, seed=b)) for b in range(n)]).view(n, 1, h, w)
    mask = m.to(torch.uint8).to(dev)
    ts = TileMask(n, ho, wo, dev)
    launch = lambda: ops.build_mask_tiles(mask, None, n, h, w, _lib.FOOT_CONV, k, s, p, ts)
    for _ in range(args.warmup):
        launch()
    torch.cuda.synchronize()
    e0.record()
    for _ in range(args.iters):
        launch()
    e1.record()
    torch.cuda.synchronize()
    us = 1e3 * e0.elapsed_time(e1) / args.iters
    tiles = int(ts.counts[0].item())
    byts = n * h * w + n * ho * wo + ts.capacity * 8 + tiles * 4
    print(json.dumps(dict(kernel="mie_build_mask_tiles", shape="%dx%d s%d @%dx%d n=%d" % (k, k, s, h, w, n),
                          density=args.density, active_tiles=tiles, tiles=ts.capacity, us=round(us, 2),
                          algorithmic_bytes=byts, gbs=round(byts / us / 1e3, 1), iters=args.iters)))


def up2x_conv(args, dev, e0, e1):
    """mie_upconv_masked at output size --h x --w: two dense half-resolution inputs, reservoir + ReLU epilogue."""
    n, cin, cout, k, h, w = args.n, args.cin, args.cout, args.k, args.h, args.w
    hl, wl = h // 2, w // 2
    dt = torch.bfloat16 if args.dtype == "bf16" else torch.float32
    es = 2 if args.dtype == "bf16" else 4
    g = torch.Generator().manual_seed(0)
    a, b = (ops.as_nhwc(torch.randn((n, cin, hl, wl), generator=g).to(dev).to(dt)
                        .contiguous(memory_format=torch.channels_last)) for _ in range(2))
    filt = ops.ConvFilter(he_normal_conv_weight(cout, cin, k, 0).permute(1, 2, 3, 0).contiguous().to(dev))
    ts_up, ts = TileMask(n, 2 * hl, 2 * wl, dev), TileMask(n, 2 * hl, 2 * wl, dev)
    ops.build_mask_tiles(None, None, n, hl, wl, _lib.FOOT_UP2X, 0, 0, 0, ts_up)
    ops.build_mask_tiles(ts_up, None, n, 2 * hl, 2 * wl, _lib.FOOT_CONV, k, 1, k // 2, ts)
    out = ops.new_nhwc(n, cout, 2 * hl, 2 * wl, dev, dt)
    res = ops.new_nhwc(n, cout, 2 * hl, 2 * wl, dev)

    def launch():
        ops.upconv_masked(a, None, b, None, filt, k, k // 2, ts, out, res, _lib.ACT_RELU)

    for _ in range(args.warmup):
        launch()
    torch.cuda.synchronize()
    e0.record()
    for _ in range(args.iters):
        launch()
    e1.record()
    torch.cuda.synchronize()
    us = 1e3 * e0.elapsed_time(e1) / args.iters
    a_out = int(ts.pixmask.sum().item())
    flops = 2 * a_out * cin * cout * k * k
    # algorithmic bytes: both half-resolution inputs once, emitted delta, reservoir read + write, filter, tile list
    byts = 2 * n * hl * wl * (1 + cin * es) + a_out * cout * (es + 8) + cin * cout * k * k * es + ts.capacity * 4
    print(json.dumps(dict(kernel="mie_upconv_masked", shape="up2x+%dx%d s1 %d->%d @%dx%d n=%d" % (k, k, cin, cout, 2 * hl, 2 * wl, n),
                          dtype=args.dtype, active_tiles=int(ts.counts[0].item()), tiles=ts.capacity, us=round(us, 2),
                          algorithmic_flops=flops, algorithmic_bytes=byts, tflops=round(flops / us / 1e6, 2),
                          gbs=round(byts / us / 1e3, 1), iters=args.iters)))


def pointwise(args, dev, e0, e1):
    """One bandwidth-bound incremental op.  Algorithmic bytes: every delta, mask byte and reservoir the op must
    touch on the active pixels, once (A = active pixels, s = element size of the deltas, reservoirs fp32)."""
    n, c, h, w = args.n, args.cin, args.h, args.w
    dt = torch.bfloat16 if args.dtype == "bf16" else torch.float32
    es = 2 if args.dtype == "bf16" else 4
    g = torch.Generator().manual_seed(0)
    hi, wi = (h // 2, w // 2) if args.op == "up2x" else (h, w)

    def delta(ch, seed):
        t = torch.randn((n, ch, hi, wi), generator=g)
        if args.density < 1.0:
            m = torch.stack([torch.from_numpy(blob_mask(hi, wi, args.density, seed=seed + b)) for b in range(n)])
            m = m.view(n, 1, hi, wi)
            t = t * m.float()
            mk = m.to(torch.uint8).to(dev)
        else:
            mk = None
        return ops.as_nhwc(t.to(dev).to(dt).contiguous(memory_format=torch.channels_last)), mk

    res = lambda ch: ops.as_nhwc(torch.randn((n, ch, h, w), generator=g).to(dev).contiguous(memory_format=torch.channels_last))
    ts = TileMask(n, h, w, dev)
    if args.op == "act":
        d, m = delta(c, 0)
        r, out = res(c), ops.new_nhwc(n, c, h, w, dev, dt)
        ops.build_mask_tiles(m, None, n, h, w, _lib.FOOT_CONV, 1, 1, 0, ts)
        launch = lambda: ops.act_incr(_lib.ACT_RELU, 0.0, d, r, out, ts)
        per_px = c * (es + 8 + es) + 1                     # delta in, reservoir read + write, delta out, mask byte
    elif args.op == "mul":
        d1, m1 = delta(c, 0)
        d2, m2 = delta(c, 100)
        r1, r2, out = res(c), res(c), ops.new_nhwc(n, c, h, w, dev, dt)
        ops.build_mask_tiles(m1, m2, n, h, w, _lib.FOOT_CONV, 1, 1, 0, ts)
        launch = lambda: ops.mul_incr(d1, m1, r1, d2, m2, r2, out, ts)
        per_px = c * (2 * es + 16 + es) + 2                # two deltas, two reservoirs read + write, delta out
    elif args.op == "add":
        a, ma = delta(c, 0)
        b, mb = delta(c, 100)
        out = ops.new_nhwc(n, c, h, w, dev, dt)
        ops.build_mask_tiles(ma, mb, n, h, w, _lib.FOOT_CONV, 1, 1, 0, ts)
        launch = lambda: ops.add_incr(a, ma, b, mb, out, ts)
        per_px = c * 3 * es + 2
    elif args.op == "up2x":
        a, ma = delta(c, 0)
        b, mb = delta(c, 100)
        out = ops.new_nhwc(n, c, h, w, dev, dt)
        ops.build_mask_tiles(ma, mb, n, hi, wi, _lib.FOOT_UP2X, 0, 0, 0, ts)
        launch = lambda: ops.upsample2x_incr(a, ma, b, mb, ts, out)
        per_px = c * es + (2 * c * es + 2) / 4.0           # delta out; both inputs at a quarter of the pixels
    else:
        gd, m = delta(4 * c, 0)
        gr, cpr, cr = res(4 * c), res(c), res(c)
        hd, cd = ops.new_nhwc(n, c, h, w, dev, dt), ops.new_nhwc(n, c, h, w, dev, dt)
        ops.build_mask_tiles(m, None, n, h, w, _lib.FOOT_CONV, 1, 1, 0, ts)
        launch = lambda: ops.convlstm_gates_incr(gd, gr, None, None, cpr, cr, hd, cd, ts)
        # gate deltas, gate reservoirs read + write, cell reservoir read + write, cached previous cell, two deltas out
        per_px = c * (4 * es + 32 + 8 + 4 + 2 * es) + 1
    for _ in range(args.warmup):
        launch()
    torch.cuda.synchronize()
    e0.record()
    for _ in range(args.iters):
        launch()
    e1.record()
    torch.cuda.synchronize()
    us = 1e3 * e0.elapsed_time(e1) / args.iters
    active = int(ts.pixmask.sum().item())
    byts = int(active * per_px) + ts.capacity * 4
    print(json.dumps(dict(kernel="mie_%s_incr" % {"gates": "convlstm_gates", "up2x": "upsample2x"}.get(args.op, args.op),
                          shape="%dx%dx%dx%d" % (n, c, h, w), dtype=args.dtype, density=args.density,
                          active_pixels=active, active_tiles=int(ts.counts[0].item()), tiles=ts.capacity,
                          us=round(us, 2), algorithmic_bytes=byts, gbs=round(byts / us / 1e3, 1),
                          hbm_frac=round(byts / us / 1e3 / 8000.0, 3), iters=args.iters)))


if __name__ == "__main__":
    main()
