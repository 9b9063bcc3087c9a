"""Seeded random problems against the CPU oracle: operators and whole blocks at shapes nobody
picked by hand (ragged rows, row lengths around the kernels' limits, dilations up to the
smallest extent, one or two output channels, batches, channel counts around the blocks of
16).  Tolerances: forward rel. 1e-5, gradients rel. 1e-4 (fp32)."""
import random

import pytest
import torch

import oracle
from cases import rel_err
from parity import check_operator_problem

pytestmark = pytest.mark.gpu


def _random_shape(rng, ndim):
    # row lengths: multiples of 4 (specialised kernels) and others (shape-generic kernels)
    w = rng.choice([rng.randrange(32, 300), 4 * rng.randrange(16, 140), 64, 128, 256, 260, 512, 1024, 1028])
    if ndim == 2:
        size = (rng.randrange(1, 48), w)
    else:
        w = min(w, rng.choice([260, 260, 600]))
        size = (rng.randrange(1, 12), rng.randrange(1, 14), w)
    d = rng.randrange(1, min(min(size), 10) + 1)
    c_in = rng.choice([1, 2, 3, 7, 15, 16, 17, 31, 32, 33, 40])
    if ndim == 3:
        c_in = min(c_in, 33)
    width = rng.choice([1, 1, 1, 2])
    batch = rng.choice([1, 1, 2, 3])
    return (batch, c_in, width, size, d)


def _cases(seed, n):
    rng = random.Random(seed)
    return [_random_shape(rng, rng.choice([2, 2, 3])) for _ in range(n)]


def _wide_cases(seed, n):
    # 2D rows longer than one workgroup covers: whole segments of 256 * V voxels (V = 4, 2 or,
    # with two output channels, 2) and others; dilations on both sides of the halo's limit of 128
    rng = random.Random(seed)
    out = []
    for _ in range(n):
        w = rng.choice([1536, 2048, 2048, 2560, 3072, 4096, 2052])
        h = rng.randrange(1, 160)
        d = rng.choice([rng.randrange(1, min(h, 12) + 1), rng.randrange(1, h + 1)])
        out.append((rng.choice([1, 2]), rng.choice([1, 3, 17]), rng.choice([1, 2]), (h, w), d))
    return out


def _extreme_cases(seed, n):
    # the corners: rows of 1 to 8192 voxels (beyond every kernel's row limit), flat images,
    # channel counts around the chunks of 128, dilations up to the smallest extent and around
    # the halo limit, layers of up to five output channels, batches of five
    rng = random.Random(seed)
    out = []
    for _ in range(n):
        ndim = rng.choice([2, 2, 3])
        if ndim == 2:
            w = rng.choice([1, 2, 3, 5, 31, 33, 63, 65, 255, 257, 1023, 1025, 4096, 4100, 5000, 8192,
                            rng.randrange(1, 6000)])
            h = rng.choice([1, 2, 3, rng.randrange(1, 40), rng.randrange(100, 300)])
            if w * h > 600000:
                h = max(1, 600000 // w)
            size = (h, w)
        else:
            w = rng.choice([1, 2, 31, 33, 65, 255, 257, 511, 513, 520, 1024, 1030, 2048, rng.randrange(1, 1200)])
            a, b = rng.choice([1, 2, 3, rng.randrange(1, 30)]), rng.choice([1, 2, 5, rng.randrange(1, 30)])
            while w * a * b > 400000 and (a > 1 or b > 1):
                a, b = max(1, a // 2), max(1, b // 2)
            size = (a, b, w)
        m = min(size)
        d = max(1, rng.choice([1, m, rng.randrange(1, m + 1), min(m, 127), min(m, 129)]))
        c_in = rng.choice([1, 2, 16, 17, 64, 65, 128, 129, 140])
        if c_in * size[-1] * (size[0] if ndim == 2 else size[0] * size[1]) > 6e6:
            c_in = rng.choice([1, 2, 3])
        out.append((rng.choice([1, 2, 5]), c_in, rng.choice([1, 1, 2, 3, 5]), size, d))
    return out


@pytest.mark.parametrize("shape", _cases(2024, 40) + _wide_cases(77, 10) + _extreme_cases(901, 30), ids=lambda s: "B%d-C%d-w%d-%s-d%d" % (
    s[0], s[1], s[2], "x".join(map(str, s[3])), s[4]))
def test_random_operator_problems(shape):
    from msd_pytorch_amd import msd_custom_convolutions as cc
    check_operator_problem(cc, shape)


def _block_cases(seed, n):
    rng = random.Random(seed)
    out = []
    for _ in range(n):
        ndim = rng.choice([2, 2, 3])
        w = rng.choice([4 * rng.randrange(16, 100), 64, 128, 256, 132, rng.randrange(33, 200)])
        size = (rng.randrange(4, 40), w) if ndim == 2 else (rng.randrange(3, 9), rng.randrange(3, 10), min(w, 132))
        depth = rng.choice([1, 2, 5, 9, 17, 20])
        width = rng.choice([1, 1, 2])
        dil = [rng.randrange(1, min(min(size), 10) + 1) for _ in range(depth)]
        out.append((ndim, size, rng.choice([1, 2, 3]), width, depth, rng.choice([1, 2]), dil))
    return out


@pytest.mark.parametrize("case", _block_cases(77, 16), ids=lambda c: "%dd-%s-c%d-w%d-depth%d-B%d" % (
    c[0], "x".join(map(str, c[1])), c[2], c[3], c[4], c[5]))
def test_random_blocks(case):
    from msd_pytorch_amd.msd_block import msd_block
    ndim, size, c_in, width, depth, batch, dil = case
    gen = torch.Generator().manual_seed(5)
    x = torch.randn(batch, c_in, *size, generator=gen)
    ws = [torch.randn(width, c_in + width * i, *([3] * ndim), generator=gen) *
          (2.0 / (3 ** ndim * (c_in + width * i))) ** 0.5 for i in range(depth)]
    bias = torch.randn(depth * width, generator=gen) * 0.1
    g = torch.randn(batch, c_in + depth * width, *size, generator=gen)
    want = oracle.block_forward(x.double(), dil, bias.double(), [w.double() for w in ws])
    xd = x.cuda().requires_grad_(True)
    bd = bias.cuda().requires_grad_(True)
    wd = [w.cuda().requires_grad_(True) for w in ws]
    got = msd_block(xd, dil, bd, *wd)
    got.backward(g.cuda())
    torch.cuda.synchronize()
    assert rel_err(got, want) <= 1e-5
    # The backward oracle takes its ReLU masks from the stack the GPU computed: an activation
    # within rounding of zero may have the other sign in double precision, and one flipped
    # mask in an upper layer changes every gradient below it by far more than the tolerance.
    want_gx, want_gb, want_gw = oracle.block_backward(got.detach().double().cpu(), g.double(), dil, bias.double(),
                                                      [w.double() for w in ws])
    assert rel_err(xd.grad, want_gx) <= 1e-4
    assert rel_err(bd.grad, want_gb) <= 1e-4
    assert max(rel_err(a.grad, b) for a, b in zip(wd, want_gw)) <= 1e-4
