"""Train, save, reload and apply a mixed-scale dense network on images from disk.

The workflow of the reference's examples/getting_started.py with this package:
ImageDataset -> DataLoader -> MSDRegressionModel / MSDSegmentationModel ->
set_normalization -> train / validate -> save -> load -> predict.  Without
``--train-input`` / ``--train-target`` a small synthetic data set (noisy discs,
TIFF files) is written to a temporary directory first, so the script runs as it
is on a machine with one GPU:

    python -m msd_pytorch_amd.examples.getting_started --task segmentation --epochs 3
    python -m msd_pytorch_amd.examples.getting_started --task regression \\
        --train-input "~/data/train/noisy/*.tiff" --train-target "~/data/train/clean/*.tiff"
"""
import argparse
import sys
import tempfile
from pathlib import Path

import numpy as np
import torch
from torch.utils.data import DataLoader

import msd_pytorch as mp
from msd_pytorch.image_dataset import write_tiff


def write_synthetic_set(folder, count, size, num_labels, seed):
    """``count`` images of random discs: label maps in ``label/``, the label value plus
    noise in ``noisy/``.  Returns the two glob patterns."""
    rng = np.random.default_rng(seed)
    folder = Path(folder)
    (folder / "noisy").mkdir(parents=True, exist_ok=True)
    (folder / "label").mkdir(parents=True, exist_ok=True)
    yy, xx = np.mgrid[:size, :size]
    for i in range(count):
        label = np.zeros((size, size), dtype=np.uint8)
        for _ in range(6):
            cy, cx, r = rng.integers(0, size), rng.integers(0, size), rng.integers(size // 10, size // 4)
            label[(yy - cy) ** 2 + (xx - cx) ** 2 < r * r] = rng.integers(1, num_labels)
        noisy = label.astype(np.float32) + rng.normal(0, 0.5, label.shape).astype(np.float32)
        write_tiff(folder / "noisy" / f"img_{i}.tiff", noisy)
        write_tiff(folder / "label" / f"img_{i}.tiff", label)
    return str(folder / "noisy" / "*.tiff"), str(folder / "label" / "*.tiff")


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--task", choices=("regression", "segmentation"), default="segmentation")
    ap.add_argument("--train-input", default=None, help="glob pattern of the training inputs")
    ap.add_argument("--train-target", default=None, help="glob pattern of the training targets")
    ap.add_argument("--val-input", default=None)
    ap.add_argument("--val-target", default=None)
    ap.add_argument("--labels", type=int, nargs="+", default=[0, 1, 2, 3, 4],
                    help="label values of the target images (segmentation)")
    ap.add_argument("--depth", type=int, default=30)
    ap.add_argument("--width", type=int, default=1)
    ap.add_argument("--dilations", type=int, nargs="+", default=list(range(1, 11)))
    ap.add_argument("--loss", choices=("L1", "L2"), default="L2")
    ap.add_argument("--epochs", type=int, default=10)
    ap.add_argument("--batch-size", type=int, default=3)
    ap.add_argument("--synthetic-size", type=int, default=128)
    ap.add_argument("--synthetic-count", type=int, default=9)
    ap.add_argument("--out", default=None, help="folder for the checkpoint and the predictions")
    args = ap.parse_args(argv)

    if not torch.cuda.is_available():
        sys.exit("getting_started needs a GPU: the convolutions of this package run on the device only")
    scratch = None
    if args.train_input is None or args.train_target is None:
        scratch = tempfile.TemporaryDirectory(prefix="msd_getting_started_")
        args.train_input, args.train_target = write_synthetic_set(
            Path(scratch.name) / "train", args.synthetic_count, args.synthetic_size, len(args.labels), seed=0)
        args.val_input, args.val_target = write_synthetic_set(
            Path(scratch.name) / "val", 3, args.synthetic_size, len(args.labels), seed=1)
        print(f"synthetic data written to {scratch.name}")
    out = Path(args.out) if args.out else Path(scratch.name if scratch else ".")
    out.mkdir(parents=True, exist_ok=True)

    segmentation = args.task == "segmentation"
    labels = args.labels if segmentation else None

    def loader(inputs, targets, shuffle):
        ds = mp.ImageDataset(inputs, targets, labels=labels)
        return ds, DataLoader(ds, args.batch_size, shuffle=shuffle)

    train_ds, train_dl = loader(args.train_input, args.train_target, True)
    val_dl = loader(args.val_input, args.val_target, False)[1] if args.val_input else None
    c_in = train_ds[0][0].shape[0]

    def new_model():
        if segmentation:
            return mp.MSDSegmentationModel(c_in, train_ds.num_labels, args.depth, args.width,
                                           dilations=args.dilations)
        c_out = train_ds[0][1].shape[0]
        return mp.MSDRegressionModel(c_in, c_out, args.depth, args.width, dilations=args.dilations,
                                     loss=args.loss)

    model = new_model()
    model.set_normalization(train_dl)
    checkpoint = out / "msd_network.torch"
    best = float("inf")
    history = []
    for epoch in range(args.epochs):
        model.train(train_dl, 1)
        train_error = model.validate(train_dl)
        val_error = model.validate(val_dl) if val_dl is not None else train_error
        history.append((train_error, val_error))
        print(f"{epoch:05} training error {train_error:0.6f} validation error {val_error:0.6f}", flush=True)
        if val_error < best:
            best = val_error
            model.save(checkpoint, epoch)

    # a fresh model, restored from disk, applied to the validation (or training) inputs
    model = new_model()
    epoch = model.load(checkpoint)
    print(f"restored epoch {epoch} from {checkpoint}")
    apply_glob = args.val_input or args.train_input
    ds = mp.ImageDataset(apply_glob, apply_glob)
    saved = 0
    with torch.no_grad():
        for i, (inp, _) in enumerate(DataLoader(ds, args.batch_size, shuffle=False)):
            output = model.net(inp.cuda())
            prediction = output.argmax(1).to(torch.uint8) if segmentation else output[:, 0]
            for b, image in enumerate(prediction.cpu().numpy()):
                write_tiff(out / f"output_{i * args.batch_size + b:05d}.tif", image)
                saved += 1
    print(f"{saved} predictions written to {out}")
    result = {"history": history, "best": best, "epoch": epoch, "predictions": saved, "out": str(out)}
    if scratch is not None and args.out is None:
        scratch.cleanup()
    return result


if __name__ == "__main__":
    main()
