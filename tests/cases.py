"""Problem shapes shared by the oracle and the GPU parity tests."""
import torch

SHAPES_2D = [
    # (B, C_in, C_out, spatial, dilation)
    (1, 1, 1, (1, 5), 1),      # strip: height == dilation (reference tests/test_msd_block.py:11)
    (2, 3, 5, (3, 6), 1),      # size = 2d+1
    (2, 3, 5, (7, 14), 3),     # size = 2d+1 for d = 3
    (1, 2, 2, (3, 3), 3),      # size == d in both axes: every tap folds
    (1, 4, 1, (10, 13), 10),   # size == d in one axis
    (2, 3, 2, (13, 21), 3),    # gradcheck shape of reference tests/test_conv2d.py:488-515
    (1, 5, 3, (29, 58), 10),
]
SHAPES_3D = [
    (1, 1, 1, (1, 1, 5), 1),
    (2, 3, 2, (3, 6, 9), 1),
    (1, 2, 2, (2, 2, 2), 2),   # size == d on every axis
    (1, 3, 2, (5, 7, 11), 2),
    (2, 2, 3, (7, 14, 21), 3),
    (1, 2, 1, (11, 13, 7), 3),  # gradcheck shape of reference tests/test_conv3d.py:376-405
]
ALL_SHAPES = SHAPES_2D + SHAPES_3D

# larger, fp32 only: shapes that reach the specialised kernels (contiguous rows,
# one or two output channels, rows longer than a wavefront, ragged tails)
SHAPES_FAST = [
    (1, 1, 1, (64, 64), 1),
    (1, 7, 1, (70, 133), 3),
    (2, 5, 1, (37, 256), 10),
    (1, 12, 2, (129, 200), 4),
    (1, 33, 1, (96, 260), 7),
    (4, 3, 1, (64, 128), 2),
    (1, 3, 1, (16, 32, 64), 1),
    (1, 6, 1, (20, 21, 70), 3),
    (2, 4, 2, (12, 33, 65), 2),
    (1, 9, 1, (32, 32, 128), 10),
    (1, 3, 1, (3, 5, 600), 2),       # 3D rows longer than the forward kernel's 512 lanes: 4 voxels per lane
    (1, 2, 1, (2, 4, 601), 1),       # the same, odd: shape-generic forward
    (1, 2, 2, (3, 2100), 3),         # 2D, long ragged rows, two output channels
    (1, 5, 3, (40, 132), 2),         # three output channels: the specialised kernels in groups of 2 + 1
    (2, 4, 5, (9, 12, 68), 3),       # 3D, five output channels: 2 + 2 + 1
    (1, 3, 4, (6, 1022), 4),         # four output channels, rows of 2 voxels per lane
]


def make_problem(shape, dtype, device="cpu", seed=0):
    """Input and output as channel slices of one stack, as the dense block
    passes them: batch stride = (C_in + C_out) * plane."""
    B, C, Wd, size, d = shape
    gen = torch.Generator().manual_seed(seed)
    ndim = len(size)
    stack = torch.randn(B, C + Wd, *size, dtype=dtype, generator=gen)
    gstack = torch.randn(B, C + Wd, *size, dtype=dtype, generator=gen)
    k = torch.randn(Wd, C, *([3] * ndim), dtype=dtype, generator=gen) / (3.0 ** ndim * C) ** 0.5
    bias = torch.randn(Wd, dtype=dtype, generator=gen) * 0.1
    stack, gstack, k, bias = (t.to(device) for t in (stack, gstack, k, bias))
    return dict(stack=stack, gstack=gstack, x=stack[:, :C], y=stack[:, C:], gx=gstack[:, :C], gy=gstack[:, C:],
                k=k, bias=bias, d=d, C=C, Wd=Wd)


def problem_on(problem, device):
    """The same problem (same values) on another device, with the same aliasing of the
    channel slices."""
    C = problem["C"]
    stack, gstack = problem["stack"].to(device), problem["gstack"].to(device)
    return dict(stack=stack, gstack=gstack, x=stack[:, :C], y=stack[:, C:], gx=gstack[:, :C], gy=gstack[:, C:],
                k=problem["k"].to(device), bias=problem["bias"].to(device), d=problem["d"], C=C, Wd=problem["Wd"])


def rel_err(got, want):
    """max |got - want| / max |want|: the parity measure of every tolerance in these tests."""
    got, want = got.detach().double().cpu(), want.detach().double().cpu()
    scale = max(want.abs().max().item(), 1e-30)
    return (got - want).abs().max().item() / scale
