#!/usr/bin/env python3
"""Headline benchmark: MSD train step (forward + backward) on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload C|D|A|B|E1|E2]

Prints ONE JSON line.  `value` is megavoxels per second of one training step
(batch * voxels / step time) of the workload, inputs resident in HBM.  The
`roofline` object prices the kernel class that takes the most time against the
HBM peak using its ALGORITHMIC bytes (every input channel read once per layer,
the gradient stack read and written once per layer), timed with HIP events on
the launch stream in an instrumented repeat of the same K steps.  The
`cpu_baseline` object times the CPU oracle (a C/OpenMP port of the reference
kernels) on a bounded sample of the same network.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
# fp32 peak of MI355X (matrix cores, or packed vector instructions); plain (non-packed) vector
# fp32, which the build rules leave to the forward kernel's multiply-adds, peaks at half of it
FP32_PEAK_TFLOPS = 157.3
PIPE = {"forward": "fp32 VALU, non-packed (78.6 TFLOP/s of the 157.3 peak)",
        "backward_x": "fp32 VALU, non-packed (78.6 TFLOP/s of the 157.3 peak)",
        "backward_kb": "fp32 MFMA 16x16x4",
        "backward_xkb": "fp32 MFMA 16x16x4 (weight gradient) + fp32 VALU (input gradient), half of the flops each"}

# kernel families (as named in the profile summaries) whose HBM traffic belongs to a class
FAMILIES = {"forward": ("fwd_lattice",), "backward_xkb": ("bwd_rows_fused", "bwd_one_channel", "reduce_columns"),
            "backward_kb": ("bwdk_rows", "bwdk_mfma"), "backward_x": ("relu_mask", "bwdx_rows", "bwdx_one_channel")}
# families that are the second pass of an operator call, not a call of their own
SECOND_PASS = ("reduce_columns",)


def profiled_traffic(name, split3d=False):
    """HBM-side bytes per pass of the network for each kernel class, read from the committed
    rocprofv3 summary of this workload (profiles/bench_workload_<name>_*.txt, block "HBM-side
    bytes per pass": FETCH_SIZE + WRITE_SIZE per dispatch, scaled by what the same counters
    read for a 1 GiB device copy).  Counters cannot be read from inside this script.  The
    summary also holds how many dispatches of each family one pass of the network made when
    the counters were taken (block "dispatches per pass"); a class whose main kernels are
    launched another number of times now (the kernels or the grouping of layers changed since)
    gets no figure.  Returns ({class: (bytes, dispatches of its main kernels or None)}, file
    name) or ({}, None) when no summary is there."""
    import glob
    import re
    files = sorted(glob.glob(os.path.join(ROOT, "profiles", f"bench_workload_{name}_*_kernels.txt")))
    if not files:
        return {}, None
    per_family, dispatches, block = {}, {}, None
    with open(files[0]) as fh:
        for line in fh:
            if line.startswith("# HBM-side bytes per pass"):
                block = "bytes"
                continue
            if line.startswith("# dispatches per pass"):
                block = "dispatches"
                continue
            m = re.match(r"#\s+(\S+)\s+([0-9.]+) GB", line) if block == "bytes" else None
            n = re.match(r"#\s+(\S+)\s+([0-9]+)\s*$", line) if block == "dispatches" else None
            if m:
                per_family[m.group(1)] = float(m.group(2)) * 1e9
            elif n:
                dispatches[n.group(1)] = int(n.group(2))
            else:
                block = None
    out = {}
    families = dict(FAMILIES)
    if split3d:
        # the weight gradients of two layers per pass are instances of the fused kernel's family
        families["backward_kb"] = ("bwd_rows_fused", "reduce_columns", "bwdk_rows", "bwdk_mfma")
        families["backward_xkb"] = ()
    for cls, fams in families.items():
        found = [per_family[f] for f in fams if f in per_family]
        if found:
            main = [dispatches[f] for f in fams if f in dispatches and f not in SECOND_PASS]
            out[cls] = (sum(found), sum(main) if main else None)
    return out, os.path.relpath(files[0], ROOT)


WORKLOADS = {
    # name: (kind, ndim, c_in, c_out/labels, depth, width, batch, spatial, adam)
    "A": ("regression", 2, 1, 1, 10, 1, 1, (256, 256), False),
    "B": ("regression", 2, 1, 1, 100, 1, 4, (512, 512), True),
    "C": ("segmentation", 2, 1, 4, 100, 1, 1, (1024, 1024), False),
    "D": ("regression", 3, 1, 1, 50, 1, 1, (128, 128, 128), False),
    "E1": ("regression", 2, 2, 2, 200, 2, 1, (2048, 2048), False),
    "E2": ("regression", 3, 1, 1, 30, 1, 1, (256, 256, 256), False),
}
DESCRIPTION = {
    "A": "MSDRegressionModel 2D depth 10 width 1, 1x1x256x256, MSE, fwd+bwd",
    "B": "MSDRegressionModel 2D depth 100 width 1, 4x1x512x512, MSE, fwd+bwd+Adam",
    "C": "MSDSegmentationModel 2D depth 100 width 1 (4 labels), 1x1x1024x1024, NLL, fwd+bwd",
    "D": "MSDRegressionModel 3D depth 50 width 1, 1x1x128x128x128, MSE, fwd+bwd",
    "E1": "MSDRegressionModel 2D depth 200 width 2, 1x2x2048x2048, MSE, fwd+bwd (13.5 GB of stacks)",
    "E2": "MSDRegressionModel 3D depth 30 width 1, 1x1x256x256x256, MSE, fwd+bwd",
}


def make_data(name, torch):
    kind, ndim, c_in, c_out, depth, width, batch, spatial, adam = WORKLOADS[name]
    torch.manual_seed(0)
    if kind == "segmentation":
        # piecewise-constant blobs (32x32 random labels, nearest-upsampled) + noise
        grid = torch.randint(0, c_out, (batch, 1, 32, 32))
        labels = torch.nn.functional.interpolate(grid.float(), size=spatial, mode="nearest").long()
        x = labels.float() / (c_out - 1) + 0.05 * torch.randn(batch, 1, *spatial)
        return x, labels
    x = torch.rand(batch, c_in, *spatial)
    if name == "B":
        blur = torch.tensor([[1., 2., 1.], [2., 4., 2.], [1., 2., 1.]]).view(1, 1, 3, 3) / 16
        return x, torch.nn.functional.conv2d(x, blur, padding=1)
    return x, x + 0.1 * torch.randn_like(x)


def make_model(name, torch):
    from msd_pytorch_amd import MSDRegressionModel, MSDSegmentationModel
    kind, ndim, c_in, c_out, depth, width, batch, spatial, adam = WORKLOADS[name]
    torch.manual_seed(0)
    if kind == "segmentation":
        model = MSDSegmentationModel(c_in, c_out, depth, width, ndim=ndim)
    else:
        model = MSDRegressionModel(c_in, c_out, depth, width, ndim=ndim)
    # the final layer starts at zero, which makes every hidden gradient zero
    # on the first step; give it small random weights so the backward pass
    # carries real data
    model.msd.final_layer.linear.weight.data.normal_(0, 0.01)
    return model


def algorithmic_work(name, fused, paired=False, triple_from=32, kpairs=False, chainpairs=False):
    """Per-step algorithmic bytes and flops of each kernel class, fp32, per layer with C input
    and w output channels over N voxels and K = 9 or 27 taps:
    bytes: forward (C + w) N 4, backward_x (2C + 2w) N 4, backward_k+bias (C + 2w) N 4, the fused
    backward_x + backward_k+bias pass (3C + 2w) N 4, each plus the w*C*K weights; the
    separate ReLU-mask pass of the top layer 3 w N 4 (counted with backward_x);
    flops: 2 C w K N for each of forward, backward_x and backward_k (the fused pass does two).
    `fused` says which way the library ran the layers above the first (it reports a
    non-zero call count for the fused class); layer 0 needs no input gradient.
    `paired`: the library runs the layers of a 2D block of width 1 in groups of n = 3 (where the
    group's layers share at least `triple_from` channels; None: never) or 2 layers, from the top,
    while the group's lowest layer is above layer 0: the top j layers of the group over the
    single channel that the layer below them wrote, (3 + 2j) N 4 bytes, for j = 1 .. n - 1, and
    one pass over the c channels below all n layers with the layers as its n output channels,
    (3c + 2n) N 4 bytes: what that algorithm has to move, a half to a third of the per-layer
    figure.  The per-layer figure is returned as well, under "backward_xkb_per_layer".
    `kpairs`: the library runs a 3D block of width 1 as a chain of backward_x launches with the
    weight and bias gradients of two layers per pass over x beside it (layers depth-1 and depth-2,
    ... down to 1 and 0; an odd lowest layer alone): a pair reads the C input channels of its
    upper layer once and two output gradients, (C + 4) N 4 bytes.
    `chainpairs`: that chain takes the same pairs: the upper layer over the one channel the lower
    layer wrote, 4 N 4 bytes (the channel's gradient read and written, its activation, the upper
    output gradient), then one read-modify-write pass over the C - 1 channels below with both
    layers' shares, (2 (C - 1) + 2) N 4 bytes.
    Returns (bytes per class, flops per class, voxels per step)."""
    kind, ndim, c_in, c_out, depth, width, batch, spatial, adam = WORKLOADS[name]
    n = batch
    for s in spatial:
        n *= s
    K = 3 ** ndim
    nbytes = {"forward": 0, "backward_x": 3 * width * n * 4, "backward_kb": 0, "backward_xkb": 0,
              "backward_xkb_per_layer": 0}
    flops = {"forward": 0, "backward_x": 0, "backward_kb": 0, "backward_xkb": 0}
    in_pair = set()
    if fused and paired:
        i = depth - 1
        while i - 1 > 0:
            first = c_in + width * i             # channels that layer i reads
            m = 3 if triple_from is not None and i - 2 > 0 and first - 2 >= max(triple_from, 1) else 2
            in_pair.update(range(i - m + 1, i + 1))
            c = first - (m - 1)                  # channels below all layers of the group
            for j in range(1, m):
                nbytes["backward_xkb"] += (3 + 2 * j) * n * 4 + 2 * j * K * 4
            nbytes["backward_xkb"] += (3 * c + 2 * m) * n * 4 + 2 * (m * c * K * 4)
            i -= m
    for i in range(depth):
        C = c_in + width * i
        wts = width * C * K * 4
        op = 2 * C * width * K * n
        nbytes["forward"] += (C + width) * n * 4 + wts
        flops["forward"] += op
        if i > 0 and fused:
            per_layer = (3 * C + 2 * width) * n * 4 + 2 * wts
            nbytes["backward_xkb_per_layer"] += per_layer
            if i not in in_pair:
                nbytes["backward_xkb"] += per_layer
            flops["backward_xkb"] += 2 * op
            continue
        upper, lower = (depth - 1 - i) % 2 == 0 and i > 0, (depth - 1 - i) % 2 == 1
        if chainpairs and (upper or lower):
            if i > 0:                         # (layer 0's pass would only serve a gradient of the block's input)
                nbytes["backward_x"] += 4 * n * 4 + K * 4 if upper else (2 * C + 2) * n * 4 + 2 * wts
                flops["backward_x"] += op if i > 1 else 2 * K * n
        elif i > 0:
            nbytes["backward_x"] += (2 * C + 2 * width) * n * 4 + wts
            flops["backward_x"] += op
        flops["backward_kb"] += op
        if kpairs and (depth - 1 - i) % 2 == 1:
            continue                          # the lower layer of a pair: counted with the upper one
        if kpairs and i > 0:
            nbytes["backward_kb"] += (C + 4 * width) * n * 4 + 2 * wts
        else:
            nbytes["backward_kb"] += (C + 2 * width) * n * 4 + wts
    return nbytes, flops, n


def kernel_times(lib, torch, run_steps):
    """Per-class kernel time of `run_steps()`: the library brackets its operator launches
    with HIP events recorded on the launch stream (msd_profile_enable; inside the block
    loops one pair of events per run of launches of one class) and msd_profile_read sums the
    elapsed times after a synchronise."""
    import ctypes
    lib.msd_profile_enable(1)
    run_steps()
    torch.cuda.synchronize()
    ms = (ctypes.c_double * 4)()
    calls = (ctypes.c_int64 * 4)()
    rc = lib.msd_profile_read(ms, calls)
    lib.msd_profile_enable(0)
    if rc != 0:
        raise RuntimeError(lib.msd_last_error().decode())
    names = ("forward", "backward_x", "backward_kb", "backward_xkb")
    return {n: (ms[i], calls[i]) for i, n in enumerate(names)}


def cpu_baseline(name, budget_s=18.0):
    """Time the CPU oracle's dense-block forward+backward on a bounded sample: the same
    network on the workload's own image when a calibration run prices that within 15 % of
    the edge the time budget allows (or below it), else on a smaller image of that edge.
    Workloads that cost well under the budget (A) are repeated and the best run is quoted."""
    import torch
    import oracle
    kind, ndim, c_in, c_out, depth, width, batch, spatial, adam = WORKLOADS[name]
    host_cpus = os.cpu_count() or 1
    threads = min(host_cpus, int(os.environ.get("OMP_NUM_THREADS", "16")))
    oracle.set_num_threads(threads)
    torch.manual_seed(0)
    dil = [(i % 10) + 1 for i in range(depth)]
    weights = [torch.randn(width, c_in + width * i, *([3] * ndim)) * (2.0 / (3 ** ndim * (c_in + i))) ** 0.5
               for i in range(depth)]
    bias = torch.zeros(depth * width)

    def run(size):
        x = torch.rand(1, c_in, *size)
        g = torch.randn(1, c_in + depth * width, *size)
        t0 = time.perf_counter()
        res = oracle.block_forward(x, dil, bias, weights)
        oracle.block_backward(res, g, dil, bias, weights)
        return time.perf_counter() - t0

    small = (64, 64) if ndim == 2 else (16, 16, 16)
    t_small = run(small)
    # scale the edge so the sample costs about budget_s (cost is linear in voxels)
    scale = (budget_s / max(t_small, 1e-6)) ** (1.0 / ndim)
    own = max(spatial)
    edge = int(max(small[0], min(small[0] * scale, own)))
    if edge >= 0.85 * own:
        edge = own
    size = tuple(spatial) if edge == own else (edge,) * ndim
    nv = 1
    for e in size:
        nv *= e
    t = run(size)
    repeats = 1
    while t * repeats < 1.0 and repeats < 20:        # a sample of milliseconds: best of several
        t = min(t, run(size))
        repeats += 1
    return {"value": round(nv / t / 1e6, 4), "unit": "Mvoxel/s", "cores": threads, "host_cpus": host_cpus,
            "kind": "port", "seconds": round(t, 4),
            "sample": f"C/OpenMP oracle on {threads} threads (the host reports {host_cpus} CPUs), dense block "
                      f"forward+backward, depth {depth} width {width}, 1x{c_in}x{'x'.join(map(str, size))} "
                      f"fp32, {t:.3g} s" + (f" (best of {repeats})" if repeats > 1 else "")
                      + ("" if edge == own else f"; the workload's own edge is {own}")}


def measure(name, args, lib, torch, steps=None, warmup=None, cpu=True):
    """One workload: K timed steps, the per-class kernel times of a repeat of them, the
    roofline of the class that takes the most time, the CPU baseline."""
    import copy
    args = copy.copy(args)
    args.steps = steps or args.steps
    args.warmup = args.warmup if warmup is None else warmup
    kind, ndim, c_in, c_out, depth, width, batch, spatial, adam = WORKLOADS[name]
    model = make_model(name, torch)
    x, target = make_data(name, torch)
    model.set_input(x)          # inputs resident in HBM before the timed region
    model.set_target(target)

    # one batch of MSDModel.train: forward, zero_grad, backward and, where the workload has
    # it, the Adam update, on the batch resident in HBM; like train, the loop does not read
    # the loss back between steps
    def step():
        model.step_async(update=adam)

    eager_step = step
    if args.graph:
        from msd_pytorch_amd import GraphedStep
        if adam:
            model.optimizer = torch.optim.Adam(model.msd.parameters(), capturable=True)
        step = GraphedStep(model, update=adam)    # the per-kernel timing below runs the eager step

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    ms_per_step = elapsed / args.steps * 1e3
    loss = float(model.get_loss())          # of the last timed step: the steps computed something

    _, _, nvox = algorithmic_work(name, False)
    result = {
        "value": round(nvox / (ms_per_step * 1e-3) / 1e6, 3),
        "unit": "Mvoxel/s",
        "ms_per_step": round(ms_per_step, 4),
        "steps": args.steps, "warmup": args.warmup,
        "loss": loss,
        "config": {"workload": f"{name}: {DESCRIPTION[name]}", "depth": depth, "width": width,
                   "batch": batch, "spatial": list(spatial), "hip_graph": bool(args.graph)},
    }

    if not args.no_kernel_timing:
        totals = kernel_times(lib, torch, lambda: [eager_step() for _ in range(args.steps)])
        # 2D blocks of width 1 run their layers two or three at a time in the backward pass
        # (block.pair; block.triple: from how many shared channels three, 0 never, 32 by default)
        tuned = dict(kv.replace(" ", "").split("=") for kv in args.tune)
        paired = ndim == 2 and width == 1 and tuned.get("block.pair") != "0" and tuned.get("block.fuse") != "0"
        triple = int(tuned.get("block.triple", -1))
        triple_from = None if triple == 0 else (32 if triple < 0 else triple)
        # 3D blocks of width 1 may run as a chain of backward_x launches with the weight gradients
        # two layers per pass on a second stream (block.split3d); the instrumented repeat runs both
        # on one stream, so the classes' times add up to more than the step's backward pass
        split3d = ndim == 3 and width == 1 and totals["backward_xkb"][1] == 0 and \
            0 < totals["backward_kb"][1] // args.steps < depth
        bytes_per_step, flops_per_step, _ = algorithmic_work(name, totals["backward_xkb"][1] > 0, paired, triple_from,
                                                             kpairs=split3d,
                                                             chainpairs=split3d and tuned.get("block.chainpair") != "0")
        kernels = {}
        for cls, (ms, launches) in totals.items():
            if launches == 0:
                continue
            per_step_s = ms / args.steps * 1e-3
            gbs = bytes_per_step[cls] / per_step_s / 1e9
            tfl = flops_per_step[cls] / per_step_s / 1e12
            kernels[cls] = {"ms_per_step": round(per_step_s * 1e3, 4), "calls_per_step": launches // args.steps,
                            "avg_call_us": round(ms / launches * 1e3, 2),
                            "algorithmic_GB_per_step": round(bytes_per_step[cls] / 1e9, 3),
                            "GBps": round(gbs, 1), "frac_hbm": round(gbs / HBM_PEAK_GBS, 4),
                            "algorithmic_GFLOP_per_step": round(flops_per_step[cls] / 1e9, 2),
                            "TFLOPs": round(tfl, 2), "frac_fp32": round(tfl / FP32_PEAK_TFLOPS, 4),
                            "Mvoxel_per_s": round(nvox / per_step_s / 1e6, 2)}
            if cls == "backward_xkb" and paired:
                # the same time priced with the bytes of one fused pass per layer, for comparison
                per_layer = bytes_per_step["backward_xkb_per_layer"]
                kernels[cls]["layers_in_groups"] = True
                kernels[cls]["per_layer_GB_per_step"] = round(per_layer / 1e9, 3)
                kernels[cls]["per_layer_GBps"] = round(per_layer / per_step_s / 1e9, 1)
        dominant = max(kernels, key=lambda c: kernels[c]["ms_per_step"])
        dom = kernels[dominant]
        # the committed counter figures describe the library's default launch shapes
        traffic, source = ({}, None) if args.tune else profiled_traffic(name, split3d)
        if split3d:
            result["config"]["backward"] = ("chain of backward_x launches (two layers per pass); weight gradients two "
                                            "layers per pass on a second stream (kernel classes timed on one stream)")
        per_launch, profiled_calls = traffic.get(dominant, (None, None))
        stale = per_launch is not None and profiled_calls is not None and profiled_calls != dom["calls_per_step"]
        if stale:
            per_launch = None
        by_flops = dom["frac_fp32"] > dom["frac_hbm"]
        roof = {"bound": "mfma" if by_flops else "hbm", "kernel": dominant,
                "achieved": dom["TFLOPs"] if by_flops else dom["GBps"],
                "peak": FP32_PEAK_TFLOPS if by_flops else HBM_PEAK_GBS,
                "unit": "TFLOP/s" if by_flops else "GB/s",
                "frac": dom["frac_fp32"] if by_flops else dom["frac_hbm"],
                # HBM-side bytes per launch (fetch + write counters of the committed rocprofv3
                # summary), to be compared with the algorithmic bytes per launch
                "traffic": round(per_launch / dom["calls_per_step"]) if per_launch else None,
                "traffic_source": source if per_launch else None,
                **({"traffic_note": f"{source} was taken with {profiled_calls} launches of this class per step, "
                                    f"this run makes {dom['calls_per_step']}: counters not comparable"} if stale else {}),
                "algorithmic_bytes_per_launch": round(bytes_per_step[dominant] / dom["calls_per_step"]),
                "algorithmic_flops_per_launch": round(flops_per_step[dominant] / dom["calls_per_step"]),
                "avg_launch_us": dom["avg_call_us"],
                "hbm": {"achieved_GBps": dom["GBps"], "peak_GBps": HBM_PEAK_GBS, "frac": dom["frac_hbm"]},
                "fp32": {"achieved_TFLOPs": dom["TFLOPs"], "peak_TFLOPs": FP32_PEAK_TFLOPS, "frac": dom["frac_fp32"],
                         "pipe": PIPE[dominant]},
                "timed": "HIP events on the launch stream around the library's operator launches "
                         "(msd_profile_enable; one pair per run of launches of one class), in a repeat of "
                         "the K timed steps"}
        result["roofline"] = roof
        result["kernels"] = kernels
        result["hot_path_ms_per_step"] = round(sum(k["ms_per_step"] for k in kernels.values()), 4)

    if cpu and not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(name)
    del model
    torch.cuda.empty_cache()
    return result


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--workload", default=None, choices=sorted(WORKLOADS),
                    help="one workload only (default: the 2D headline C, then the 3D headline D as 'headline_3d')")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-kernel-timing", action="store_true")
    ap.add_argument("--tune", action="append", default=[], metavar="KEY=VALUE",
                    help="launch-shape knob passed to msd_set_tuning (repeatable)")
    ap.add_argument("--graph", action="store_true",
                    help="replay the step from a HIP graph (GraphedStep): for workloads bound by launch overhead")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="run one 1 GiB device copy first (reference dispatch for scaling rocprof byte counters)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on ONE GPU; --gpus must be 1 (no multi-GPU path exists)")

    import torch
    from msd_pytorch_amd import _native
    lib = _native.load()
    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible")

    for kv in args.tune:
        key, _, val = kv.partition("=")
        if lib.msd_set_tuning(key.encode(), int(val)) != 0:
            sys.exit("bench.py: " + lib.msd_last_error().decode())

    if args.calibrate_copy:
        src = torch.empty(1 << 28, dtype=torch.float32, device="cuda").normal_()
        dst = torch.empty_like(src)
        dst.copy_(src)          # reads 1 GiB, writes 1 GiB
        torch.cuda.synchronize()
        del src, dst

    first = measure(args.workload or "C", args, lib, torch)
    result = {
        "metric": "MSD train-step Mvoxel/s",
        "value": first.pop("value"),
        "unit": first.pop("unit"),
        "n_gpus": 1, "steps": first.pop("steps"), "warmup": first.pop("warmup"),
        "ms_per_step": first.pop("ms_per_step"),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
    }
    result.update(first)
    if args.workload is None:
        # the metric is quoted on two configurations: the 3D one rides in the same line
        result["headline_3d"] = measure("D", args, lib, torch)
        # the other configurations, each for a few steps: throughput, loss, and every kernel
        # class against the HBM roofline (A is launch-bound and cache-resident: its fractions
        # say so, they are not a bandwidth claim)
        others = {}
        for name in ("A", "B", "E1", "E2"):
            # (A's step is a fraction of a millisecond of launches: more of them for a steady figure)
            few = (50, 10) if name == "A" else (min(args.steps, 5), min(args.warmup, 2))
            r = measure(name, args, lib, torch, steps=few[0], warmup=few[1], cpu=False)
            r["frac_hbm"] = {cls: k["frac_hbm"] for cls, k in r.get("kernels", {}).items()}
            others[name] = r
        result["workloads"] = others
        if not args.no_cpu_baseline:
            # the first configuration as the baseline file words it: the whole step on the CPU
            result["cpu_baseline_A"] = cpu_baseline("A")
    print(json.dumps(result))


if __name__ == "__main__":
    main()
