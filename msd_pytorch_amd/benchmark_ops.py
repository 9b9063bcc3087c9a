"""Per-operator timing and launch-shape sweep on gfx950, priced against the HBM roofline.

Takes the place of the reference's CUDA block-size tuner
(benchmarks/benchmark_block_sizes.py: every power-of-two thread block per operator, a
slope-of-time estimate with a confidence interval, CSV) and of its timeit helper
(msd_pytorch/bench.py).  Here the launch shapes are chosen inside the library for gfx950;
what can be varied from outside is the library's own set of launch-shape parameters
(msd_set_tuning: voxels per lane, rows per forward tile, channel groups per workgroup, tile
shape and numbering, workgroups per launch, ...).

Two modes:

  table (default)  each operator's time, algorithmic GB/s and fraction of the 8 TB/s HBM peak
                   over a grid of problems (rank, image size, input channels, dilation):
      python -m msd_pytorch_amd.benchmark_ops --ndim 2 --size 1024 --channels 1 10 50 100
      python -m msd_pytorch_amd.benchmark_ops --ndim 3 --size 128 --channels 1 10 25 50 --csv out.csv

  --sweep          for every problem and operator, every combination of the launch-shape
                   parameters that operator reads, timed against the library's default; prints
                   the best setting beside the default and writes every measurement to the CSV:
      python -m msd_pytorch_amd.benchmark_ops --sweep --ndim 3 --size 128 --channels 16 48 \\
             --dilations 1 5 10 --ops forward backward_xkb --csv sweep.csv

Times are the slope of a least-squares line through the wall time of 1, 2, 4 and 8
back-to-back calls (each run synchronised at both ends, repeated `--trials` times), which
removes the fixed cost of a launch and of the synchronisation from the estimate, with the
90 % confidence interval of the slope (Moreno & Fischmeister 2017, the method the reference's
tuner uses).
"""
import argparse
import csv
import itertools
import math
import sys
import time

HBM_PEAK = 8.0e12

# Launch-shape parameters each operator reads, with the values worth trying (the first value
# listed is not special: the library's default is measured separately, with every parameter
# unset).  {r} is the rank, 2 or 3.
SWEEP_GRID = {
    "forward": {
        2: {"fwd.vec2d": (1, 2, 4), "fwd.rows2d": (2, 3, 4, 5, 6), "fwd.split": (1, 2, 4)},
        3: {"fwd.vec3d": (1, 2, 4), "fwd.lattice3d": (24, 33, 44), "fwd.split": (1, 2, 4), "fwd.class3d": (0, 1)},
    },
    "backward_x": {
        2: {"bwdx.vec2d": (1, 2, 4), "bwdx.unroll2d": (2, 4), "bwdx.min_blocks": (256, 1024, 4096)},
        3: {"bwdx.vec3d": (1, 2, 4), "bwdx.unroll3d": (2, 4), "bwdx.min_blocks": (256, 1024, 4096)},
    },
    "backward_kb": {
        2: {"bwdk.vec2d": (1, 2, 4), "bwdk.rows": (0, 1), "bwdk.blocks": (256, 512, 1024)},
        3: {"bwdk.fused3d": (0, 1), "bwdk.vec3d": (1, 2), "bwdk.rows": (0, 1), "bwdk.blocks": (256, 512, 1024)},
    },
    "backward_xkb": {
        2: {"bwdk.vec2d": (1, 2, 4), "bwdk.blocks": (256, 512, 768, 1024), "bwdk.interleave": (0, 1)},
        3: {"bwdk.vec3d": (1, 2), "bwdk.blocks": (256, 512, 768, 1024), "bwdk.interleave": (0, 1)},
    },
}
ORDER_KNOB = {"xcd_remap": (0, 1)}      # workgroup order by XCD: read by every operator (--with-order)

CSV_FIELDS = ["op", "ndim", "spatial", "batch", "c_in", "width", "dilation", "setting", "us", "us_ci_low",
              "us_ci_high", "GBps", "frac_hbm", "Mvoxel_per_s"]


def enumerate_settings(op, ndim, with_order=False, limit=None):
    """All combinations of the launch-shape parameters of `op` at rank `ndim`, as dicts;
    the empty dict (library defaults) comes first."""
    grid = dict(SWEEP_GRID[op][ndim])
    if with_order:
        grid.update(ORDER_KNOB)
    keys = list(grid)
    out = [{}]
    for values in itertools.product(*(grid[k] for k in keys)):
        out.append(dict(zip(keys, values)))
        if limit is not None and len(out) > limit:
            break
    return out


def setting_name(setting):
    return ";".join(f"{k}={v}" for k, v in setting.items()) or "default"


def _t_quantile_95(dof):
    """95th percentile of Student's t with `dof` degrees of freedom."""
    try:
        from scipy import stats
        return float(stats.t.ppf(0.95, dof))
    except ImportError:        # Cornish-Fisher expansion around the normal quantile
        z = 1.6448536269514722
        return z + (z ** 3 + z) / (4 * dof) + (5 * z ** 5 + 16 * z ** 3 + 3 * z) / (96 * dof ** 2)


def fit_slope(counts, seconds):
    """Least-squares slope of seconds over counts and its 90 % confidence interval."""
    n = len(counts)
    mx = sum(counts) / n
    my = sum(seconds) / n
    sxx = sum((c - mx) ** 2 for c in counts)
    slope = sum((c - mx) * (s - my) for c, s in zip(counts, seconds)) / sxx
    intercept = my - slope * mx
    if n <= 2:
        return slope, (slope, slope)
    sse = sum((s - (intercept + slope * c)) ** 2 for c, s in zip(counts, seconds))
    half = _t_quantile_95(n - 2) * math.sqrt(sse / (n - 2) / sxx)
    return slope, (slope - half, slope + half)


def slope_time(run, counts=(1, 2, 4, 8), trials=3, clock=time.perf_counter):
    """Seconds per call of `run(n)` (which makes n calls and waits for them): slope of the wall
    time over n, after a warm-up of max(counts) calls."""
    run(max(counts))
    xs, ys = [], []
    for _ in range(trials):
        for n in counts:
            t0 = clock()
            run(n)
            ys.append(clock() - t0)
            xs.append(n)
    return fit_slope(xs, ys)


def algorithmic_bytes(op, ndim, n, c_in, width):
    wbytes = width * c_in * 3 ** ndim * 4
    return {"forward": (c_in + width) * n * 4 + wbytes,
            "backward_x": (2 * c_in + 2 * width) * n * 4 + wbytes,
            "backward_kb": (c_in + 2 * width) * n * 4 + wbytes,
            "backward_xkb": (3 * c_in + 2 * width) * n * 4 + 2 * wbytes}[op]


class Problem:
    """One layer's tensors on the GPU and a callable per operator."""

    def __init__(self, ndim, size, batch, c_in, width, dilation):
        import torch
        from . import msd_custom_convolutions as cc
        self.ndim, self.batch, self.c_in, self.width, self.dilation = ndim, batch, c_in, width, dilation
        self.spatial = (size,) * ndim if isinstance(size, int) else tuple(size)
        torch.manual_seed(0)
        dev = "cuda"
        stack = torch.randn(batch, c_in + width, *self.spatial, device=dev)
        grads = torch.randn(batch, c_in + width, *self.spatial, device=dev)
        k = torch.randn(width, c_in, *([3] * ndim), device=dev) * (1.0 / (c_in * 3 ** ndim)) ** 0.5
        bias = torch.zeros(width, device=dev)
        gk, gb = torch.zeros_like(k), torch.zeros_like(bias)
        x, y = stack[:, :c_in], stack[:, c_in:]
        gx, gy = grads[:, :c_in], grads[:, c_in:]
        d = dilation
        self.nvox = batch * math.prod(self.spatial)
        self.calls = {
            "forward": lambda: cc.conv_relu_forward(x, k, bias, y, d),
            "backward_x": lambda: cc.conv_relu_backward_x(y, gy, k, gx, d),
            "backward_kb": lambda: cc.conv_relu_backward_kb(y, gy, x, gk, gb, d),
            # the three plain backward operators in one call (what the dense block runs per layer)
            "backward_xkb": lambda: cc.conv_backward_xkb(gy, x, k, gx, gk, gb, d),
        }
        self._sync = torch.cuda.synchronize
        self._keep = (stack, grads, k, bias, gk, gb)
        self.calls["forward"]()

    def measure(self, op, trials):
        call, sync = self.calls[op], self._sync

        def run(n):
            sync()
            for _ in range(n):
                call()
            sync()
        return slope_time(run, trials=trials)

    def row(self, op, setting, seconds, ci):
        nbytes = algorithmic_bytes(op, self.ndim, self.nvox, self.c_in, self.width)
        return {"op": op, "ndim": self.ndim, "spatial": "x".join(map(str, self.spatial)), "batch": self.batch,
                "c_in": self.c_in, "width": self.width, "dilation": self.dilation, "setting": setting_name(setting),
                "us": seconds * 1e6, "us_ci_low": ci[0] * 1e6, "us_ci_high": ci[1] * 1e6,
                "GBps": nbytes / seconds / 1e9, "frac_hbm": nbytes / seconds / HBM_PEAK,
                "Mvoxel_per_s": self.nvox / seconds / 1e6}


class applied:
    """msd_set_tuning for the duration of a with-block."""

    def __init__(self, lib, setting):
        self.lib, self.setting = lib, setting

    def __enter__(self):
        for key, value in self.setting.items():
            if self.lib.msd_set_tuning(key.encode(), int(value)) != 0:
                raise ValueError(self.lib.msd_last_error().decode())

    def __exit__(self, *exc):
        for key in self.setting:
            self.lib.msd_set_tuning(key.encode(), -1)
        return False


def sweep_cell(problem, op, settings, trials, lib, measure=None):
    """Rows for one (problem, operator): one per setting, the library default first.
    `measure(problem, op, trials)` may be replaced (the tests do)."""
    measure = measure or (lambda p, o, t: p.measure(o, t))
    rows = []
    for setting in settings:
        with applied(lib, setting):
            seconds, ci = measure(problem, op, trials)
        rows.append(problem.row(op, setting, seconds, ci))
    return rows


def best_of(rows):
    """(default row, best row): the best is the fastest whose confidence interval lies below the
    default's, else the default itself: a difference inside the noise is no recommendation."""
    default = rows[0]
    best = min(rows, key=lambda r: r["us"])
    if best is not default and best["us_ci_high"] >= default["us_ci_low"]:
        best = default
    return default, best


def write_csv(path, rows):
    with open(path, "w", newline="") as f:
        w = csv.DictWriter(f, fieldnames=CSV_FIELDS)
        w.writeheader()
        w.writerows(rows)


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--ndim", type=int, default=2, choices=(2, 3))
    ap.add_argument("--size", type=int, nargs="+", default=[1024])
    ap.add_argument("--batch", type=int, default=1)
    ap.add_argument("--channels", type=int, nargs="+", default=[1, 10, 50, 100])
    ap.add_argument("--width", type=int, default=1)
    ap.add_argument("--dilations", type=int, nargs="+", default=[1, 10])
    ap.add_argument("--trials", type=int, default=3, help="repetitions of the 1, 2, 4, 8-call series")
    ap.add_argument("--ops", nargs="+", default=["forward", "backward_x", "backward_kb"],
                    choices=sorted(SWEEP_GRID))
    ap.add_argument("--generic", action="store_true", help="force the shape-generic kernels")
    ap.add_argument("--tune", nargs="*", default=[], metavar="KEY=VALUE",
                    help="launch-shape overrides passed to msd_set_tuning, e.g. bwdx.vec3d=2")
    ap.add_argument("--sweep", action="store_true", help="time every launch-shape setting of each operator")
    ap.add_argument("--with-order", action="store_true", help="--sweep: also vary the workgroup order (xcd_remap)")
    ap.add_argument("--limit", type=int, default=None, help="--sweep: at most this many settings per operator")
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
    if not args.sweep:
        print(f"{'op':12s} {'spatial':>14s} {'C':>4s} {'d':>3s} {'us':>10s} {'GB/s':>9s} {'%HBM':>6s} {'Mvox/s':>9s}")
    for c in args.channels:
        for d in args.dilations:
            problem = Problem(args.ndim, size, args.batch, c, args.width, d)
            for op in args.ops:
                if not args.sweep:
                    seconds, ci = problem.measure(op, args.trials)
                    r = problem.row(op, {}, seconds, ci)
                    rows.append(r)
                    print(f"{r['op']:12s} {r['spatial']:>14s} {r['c_in']:4d} {r['dilation']:3d} {r['us']:10.1f} "
                          f"{r['GBps']:9.1f} {100 * r['frac_hbm']:6.1f} {r['Mvoxel_per_s']:9.1f}", flush=True)
                    continue
                cell = sweep_cell(problem, op, enumerate_settings(op, args.ndim, args.with_order, args.limit),
                                  args.trials, lib)
                rows.extend(cell)
                default, best = best_of(cell)
                print(f"{op:12s} {default['spatial']:>12s} C={c:<4d} d={d:<3d} default {default['us']:8.1f} us "
                      f"({100 * default['frac_hbm']:4.1f} % HBM)   best {best['us']:8.1f} us  {best['setting']}"
                      f"   [{len(cell)} settings]", flush=True)
            del problem
    if args.csv:
        write_csv(args.csv, rows)
    return 0


if __name__ == "__main__":
    sys.exit(main())
