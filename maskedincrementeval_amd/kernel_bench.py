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


if __name__ == "__main__":
    main()
