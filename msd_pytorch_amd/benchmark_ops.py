"""Per-operator timing on gfx950, priced against the HBM roofline.

Takes the place of the reference's CUDA block-size tuner
(benchmarks/benchmark_block_sizes.py): the launch shapes are fixed inside the
library for gfx950, so what is swept here is the problem (rank, image size,
input channels, dilation) and what is reported is each operator's time, its
algorithmic bytes per second and the fraction of the 8 TB/s HBM peak.

    python -m msd_pytorch_amd.benchmark_ops --ndim 2 --size 1024 --channels 1 10 50 100
    python -m msd_pytorch_amd.benchmark_ops --ndim 3 --size 128 --channels 1 10 25 50 --csv out.csv
"""
import argparse
import csv
import sys

import torch

from . import msd_custom_convolutions as cc

HBM_PEAK = 8.0e12


def time_op(fn, iters, warmup=2):
    """Mean seconds per call, HIP events on the current stream."""
    for _ in range(warmup):
        fn()
    start = torch.cuda.Event(enable_timing=True)
    stop = torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(iters):
        fn()
    stop.record()
    stop.synchronize()
    return start.elapsed_time(stop) * 1e-3 / iters


def bench_case(ndim, size, batch, c_in, width, dilation, iters, ops=("forward", "backward_x", "backward_kb")):
    spatial = (size,) * ndim if isinstance(size, int) else tuple(size)
    dev = "cuda"
    torch.manual_seed(0)
    stack = torch.randn(batch, c_in + width, *spatial, device=dev)
    grads = torch.randn(batch, c_in + width, *spatial, device=dev)
    k = torch.randn(width, c_in, *([3] * ndim), device=dev) * (1.0 / (c_in * 3 ** ndim)) ** 0.5
    bias = torch.zeros(width, device=dev)
    gk = torch.zeros_like(k)
    gb = torch.zeros_like(bias)
    x, y = stack[:, :c_in], stack[:, c_in:]
    gx, gy = grads[:, :c_in], grads[:, c_in:]
    n = batch
    for s in spatial:
        n *= s
    wbytes = width * c_in * 3 ** ndim * 4
    table = {
        "forward": (lambda: cc.conv_relu_forward(x, k, bias, y, dilation), (c_in + width) * n * 4 + wbytes),
        "backward_x": (lambda: cc.conv_relu_backward_x(y, gy, k, gx, dilation),
                       (2 * c_in + 2 * width) * n * 4 + wbytes),
        "backward_kb": (lambda: cc.conv_relu_backward_kb(y, gy, x, gk, gb, dilation),
                        (c_in + 2 * width) * n * 4 + wbytes),
        # the three plain backward operators in one call (what the dense block runs per layer)
        "backward_xkb": (lambda: cc.conv_backward_xkb(gy, x, k, gx, gk, gb, dilation),
                         (3 * c_in + 2 * width) * n * 4 + 2 * wbytes),
    }
    cc.conv_relu_forward(x, k, bias, y, dilation)
    rows = []
    for name in ops:
        fn, nbytes = table[name]
        t = time_op(fn, iters)
        rows.append({"op": name, "ndim": ndim, "spatial": "x".join(map(str, spatial)), "batch": batch,
                     "c_in": c_in, "width": width, "dilation": dilation, "us": t * 1e6,
                     "GBps": nbytes / t / 1e9, "frac_hbm": nbytes / t / HBM_PEAK,
                     "Mvoxel_per_s": n / t / 1e6})
    return rows


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--ndim", type=int, default=2, choices=(2, 3))
    ap.add_argument("--size", type=int, nargs="+", default=[1024])
    ap.add_argument("--batch", type=int, default=1)
    ap.add_argument("--channels", type=int, nargs="+", default=[1, 10, 50, 100])
    ap.add_argument("--width", type=int, default=1)
    ap.add_argument("--dilations", type=int, nargs="+", default=[1, 10])
    ap.add_argument("--iters", type=int, default=10)
    ap.add_argument("--ops", nargs="+", default=["forward", "backward_x", "backward_kb"])
    ap.add_argument("--generic", action="store_true", help="force the shape-generic kernels")
    ap.add_argument("--tune", nargs="*", default=[], metavar="KEY=VALUE",
                    help="launch-shape overrides passed to msd_set_tuning, e.g. bwdx.vec3d=2")
    ap.add_argument("--csv", default=None)
    args = ap.parse_args(argv)

    from . import _native
    lib = _native.load()
    lib.msd_set_kernel_path(1 if args.generic else 0)
    for item in args.tune:
        key, value = item.split("=")
        if lib.msd_set_tuning(key.encode(), int(value)) != 0:
            sys.exit(_native.last_error())
    size = args.size[0] if len(args.size) == 1 else tuple(args.size)
    rows = []
    print(f"{'op':12s} {'spatial':>14s} {'C':>4s} {'d':>3s} {'us':>10s} {'GB/s':>9s} {'%HBM':>6s} {'Mvox/s':>9s}")
    for c in args.channels:
        for d in args.dilations:
            for r in bench_case(args.ndim, size, args.batch, c, args.width, d, args.iters, args.ops):
                rows.append(r)
                print(f"{r['op']:12s} {r['spatial']:>14s} {r['c_in']:4d} {r['dilation']:3d} {r['us']:10.1f} "
                      f"{r['GBps']:9.1f} {100 * r['frac_hbm']:6.1f} {r['Mvoxel_per_s']:9.1f}", flush=True)
    if args.csv:
        with open(args.csv, "w", newline="") as f:
            w = csv.DictWriter(f, fieldnames=list(rows[0].keys()))
            w.writeheader()
            w.writerows(rows)
    return 0


if __name__ == "__main__":
    sys.exit(main())
