"""Known-answer fixtures (tests/golden/*.npz, written by tests/golden/make_golden.py
from the fp64 oracle) and one case worked by hand."""
import glob
import os

import numpy as np
import pytest
import torch

import oracle

GOLDEN = sorted(glob.glob(os.path.join(os.path.dirname(__file__), "golden", "*.npz")))


def load(path, dtype, device="cpu"):
    z = np.load(path)   # plain arrays only; allow_pickle stays False
    t = {name: torch.from_numpy(z[name]).to(dtype).to(device) for name in ("x", "k", "bias", "gy", "y", "gx", "gk", "gb")}
    t["d"] = int(z["dilation"])
    return t


def run(ops, t):
    y = torch.empty_like(t["y"])
    gx, gk, gb = torch.zeros_like(t["gx"]), torch.zeros_like(t["gk"]), torch.zeros_like(t["gb"])
    ops.conv_relu_forward(t["x"], t["k"], t["bias"], y, t["d"])
    # gradients are taken at the fixture's own output so that the ReLU mask is the same
    ops.conv_relu_backward_x(t["y"], t["gy"], t["k"], gx, t["d"])
    ops.conv_relu_backward_k(t["y"], t["gy"], t["x"], gk, t["d"])
    ops.conv_relu_backward_bias(t["y"], t["gy"], gb)
    return y, gx, gk, gb


def close(a, b, tol):
    a, b = a.double().cpu(), b.double().cpu()
    return (a - b).abs().max().item() <= tol * max(b.abs().max().item(), 1e-30)


def test_fixtures_exist():
    assert len(GOLDEN) >= 5


def test_hand_worked_strip():
    # 1x5 strip, dilation 1, all-ones 3x3 kernel: the three kernel rows all fold onto
    # the single image row, so out[w] = 3 * (x[fold(w-1)] + x[w] + x[fold(w+1)])
    x = torch.tensor([1., 2., 3., 4., 5.]).view(1, 1, 1, 5)
    y = torch.empty_like(x)
    oracle.conv_relu_forward(x, torch.ones(1, 1, 3, 3), torch.zeros(1), y, 1)
    assert y.flatten().tolist() == [12., 18., 27., 36., 42.]


@pytest.mark.parametrize("path", GOLDEN, ids=[os.path.basename(p)[:-4] for p in GOLDEN])
def test_oracle_f32_matches_fixture(path):
    t = load(path, torch.float32)
    y, gx, gk, gb = run(oracle, t)
    assert close(y, t["y"], 1e-5) and close(gx, t["gx"], 1e-4)
    assert close(gk, t["gk"], 1e-4) and close(gb, t["gb"], 1e-4)


@pytest.mark.parametrize("path", GOLDEN, ids=[os.path.basename(p)[:-4] for p in GOLDEN])
def test_oracle_f64_reproduces_fixture(path):
    t = load(path, torch.float64)
    y, gx, gk, gb = run(oracle, t)
    for got, want in ((y, t["y"]), (gx, t["gx"]), (gk, t["gk"]), (gb, t["gb"])):
        assert close(got, want, 1e-13)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype,tol_f,tol_g", [(torch.float32, 1e-5, 1e-4), (torch.float64, 1e-12, 1e-12)])
@pytest.mark.parametrize("path", GOLDEN, ids=[os.path.basename(p)[:-4] for p in GOLDEN])
def test_hip_matches_fixture(path, dtype, tol_f, tol_g):
    from msd_pytorch_amd import msd_custom_convolutions as cc
    t = load(path, dtype, device="cuda")
    y, gx, gk, gb = run(cc, t)
    torch.cuda.synchronize()
    assert close(y, t["y"], tol_f) and close(gx, t["gx"], tol_g)
    assert close(gk, t["gk"], tol_g) and close(gb, t["gb"], tol_g)
