"""The symmetric ("reflection") index map of the GPU kernels, bit for bit.

reflect(i, n) of the reference (kernel_utils.cuh:30-38) decides which input voxel each of
the 9 (27) taps of an output voxel reads.  With the input holding its own linear voxel index
(integers below 2^24, exact in fp32), a kernel that is 1 at one tap and 0 elsewhere, zero bias
and no ReLU, the forward output IS the index that tap read: it must EQUAL the indices
gathered with the oracle's reflect(), for every tap, every extent n <= 64 with every
dilation 1 <= d <= n, and the extents of the benchmark configurations with d = 1..10, on both
kernel families (specialised and shape-generic).

The backward-input operators are the adjoint of that gather (the reference expresses it with
tap-swap tables, conv2d_backward_x.cu:153-185, conv3d_backward_x.cu:167-216): with integer
output gradients and small integer weights every sum is exact, so the result must EQUAL the
scatter-add of the output gradient along the same index vectors."""
import functools

import pytest
import torch

import oracle

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def cc():
    from msd_pytorch_amd import msd_custom_convolutions
    return msd_custom_convolutions


@pytest.fixture(scope="module")
def lib():
    from msd_pytorch_amd import _native
    lib = _native.load()
    yield lib
    lib.msd_set_kernel_path(0)


@functools.lru_cache(maxsize=None)
def _axis(n, d):
    """(3, n) int64: the input coordinate that tap 0, 1, 2 of output coordinate i reads."""
    return torch.tensor([[oracle.reflect(i + (t - 1) * d, n) for i in range(n)] for t in range(3)])


def _tap_indices(size, d, taps):
    """For each tap (p, q[, r]) in `taps`, the linear index of the voxel it reads: (T, *size) int64."""
    ndim = len(size)
    axes = [_axis(n, d).cuda() for n in size]
    strides = [1] * ndim
    for a in range(ndim - 2, -1, -1):
        strides[a] = strides[a + 1] * size[a + 1]
    out = []
    for tap in taps:
        lin = torch.zeros(size, dtype=torch.int64, device="cuda")
        for a in range(ndim):
            shape = [1] * ndim
            shape[a] = size[a]
            lin = lin + (axes[a][tap[a]] * strides[a]).view(shape)
        out.append(lin)
    return torch.stack(out)


def _all_taps(ndim):
    if ndim == 2:
        return [(q, r) for q in range(3) for r in range(3)]
    return [(p, q, r) for p in range(3) for q in range(3) for r in range(3)]


def _forward_reads(cc, size, d, dtype, relu=False, group=27):
    """Runs one launch per tap with a one-hot kernel and compares the output with the expected
    index, `group` taps per comparison.  Returns the number of mismatching voxels."""
    ndim = len(size)
    taps = _all_taps(ndim)
    nvox = 1
    for n in size:
        nvox *= n
    assert nvox <= 1 << 24
    x = torch.arange(nvox, dtype=dtype, device="cuda").view(1, 1, *size)
    zero = torch.zeros(1, dtype=dtype, device="cuda")
    bad = 0
    fwd = cc.conv_relu_forward if relu else cc.conv_forward
    for g0 in range(0, len(taps), group):
        chunk = taps[g0:g0 + group]
        y = torch.full((1, len(chunk), *size), -1.0, dtype=dtype, device="cuda")
        for j, tap in enumerate(chunk):
            k = torch.zeros(1, 1, *([3] * ndim), dtype=dtype, device="cuda")
            k[(0, 0) + tap] = 1.0
            fwd(x, k, zero, y[:, j:j + 1], d)
        want = _tap_indices(size, d, chunk).to(dtype)
        bad += int((y[0] != want).sum())
    return bad


def _sweep(n_max):
    return [(n, d) for n in range(1, n_max + 1) for d in range(1, n + 1)]


@pytest.mark.parametrize("path", [0, 1], ids=["specialised", "generic"])
def test_forward_reads_the_reflected_voxel_2d_all_extents(cc, lib, path):
    lib.msd_set_kernel_path(path)
    try:
        for n, d in _sweep(64):
            # square images (the fold along x and y at once; rows of 32 voxels and more take the
            # specialised kernels) and short images with long rows (the fold along y in the
            # specialised kernels for every n)
            for size in ((n, n), (n, 128)) if path == 0 else ((n, n),):
                assert _forward_reads(cc, size, d, torch.float32) == 0, (size, d)
    finally:
        lib.msd_set_kernel_path(0)


@pytest.mark.parametrize("path", [0, 1], ids=["specialised", "generic"])
def test_forward_reads_the_reflected_voxel_3d_all_extents(cc, lib, path):
    lib.msd_set_kernel_path(path)
    try:
        for n, d in _sweep(64):
            for size in ((n, n, n), (n, n, 64)) if path == 0 else ((n, n, n),):
                assert _forward_reads(cc, size, d, torch.float32) == 0, (size, d)
    finally:
        lib.msd_set_kernel_path(0)


def test_forward_reads_the_reflected_voxel_f64(cc):
    for n, d in _sweep(24):
        assert _forward_reads(cc, (n, n), d, torch.float64) == 0, (n, d)
        assert _forward_reads(cc, (n, n, n), d, torch.float64) == 0, (n, d)


CONFIG_SIZES = [(256, 256), (512, 512), (1024, 1024), (2048, 2048), (128, 128, 128)]


@pytest.mark.parametrize("size", CONFIG_SIZES, ids=lambda s: "x".join(map(str, s)))
@pytest.mark.parametrize("path", [0, 1], ids=["specialised", "generic"])
def test_forward_reads_the_reflected_voxel_at_the_benchmark_extents(cc, lib, size, path):
    lib.msd_set_kernel_path(path)
    try:
        for d in range(1, 11):
            assert _forward_reads(cc, size, d, torch.float32, relu=(d % 2 == 0), group=9) == 0, d
    finally:
        lib.msd_set_kernel_path(0)


def test_forward_reads_the_reflected_voxel_256_cubed(cc):
    # 2^24 voxels: the largest volume whose indices are exact in fp32; three taps at a time
    for d in (1, 10):
        assert _forward_reads(cc, (256, 256, 256), d, torch.float32, group=3) == 0, d


# ---- the adjoint: backward_x and the one-pass backward_xkb

def _adjoint_expected(size, d, weights, gy):
    """sum over taps t of weights[t] * scatter-add of gy along the index tap t reads, in int64."""
    ndim = len(size)
    taps = _all_taps(ndim)
    nvox = gy.numel()
    want = torch.zeros(nvox, dtype=torch.int64, device="cuda")
    src = gy.view(-1).to(torch.int64)
    for g0 in range(0, len(taps), 9):
        chunk = taps[g0:g0 + 9]
        idx = _tap_indices(size, d, chunk)
        for j, tap in enumerate(chunk):
            w = int(weights[tap])
            if w:
                want.index_add_(0, idx[j].view(-1), src * w)
    return want.view(size)


def _adjoint_mismatches(cc, size, d, dtype, one_hot=None, fused=False):
    ndim = len(size)
    nvox = 1
    for n in size:
        nvox *= n
    gen = torch.Generator(device="cuda").manual_seed(nvox * 31 + d)
    gy = torch.randint(-500, 501, (1, 1, *size), generator=gen, device="cuda").to(dtype)
    weights = torch.zeros([3] * ndim, dtype=torch.int64)
    if one_hot is None:
        weights = torch.arange(1, 3 ** ndim + 1).view([3] * ndim)      # a distinct weight per tap
    else:
        weights[one_hot] = 1
    k = weights.to(dtype).view(1, 1, *([3] * ndim)).cuda()
    prefill = torch.randint(-100, 101, (1, 1, *size), generator=gen, device="cuda").to(dtype)   # accumulate semantics
    gx = prefill.clone()
    if fused:
        x = torch.randint(-3, 4, (1, 1, *size), generator=gen, device="cuda").to(dtype)
        gk = torch.zeros_like(k)
        cc.conv_backward_xkb(gy, x, k, gx, gk, None, d)
    else:
        cc.conv_backward_x(gy, k, gx, d)
    want = _adjoint_expected(size, d, weights, gy[0, 0]) + prefill[0, 0].to(torch.int64)
    return int((gx[0, 0].to(torch.int64) != want).sum())


@pytest.mark.parametrize("path", [0, 1], ids=["specialised", "generic"])
@pytest.mark.parametrize("fused", [False, True], ids=["backward_x", "backward_xkb"])
def test_backward_is_the_exact_adjoint_all_extents(cc, lib, path, fused):
    lib.msd_set_kernel_path(path)
    try:
        for n, d in _sweep(64):
            sizes = [(n, n), (n, n, n)]
            if path == 0:
                sizes += [(n, 256), (n, n, 128)]         # rows the specialised kernels take, for every n
            for size in sizes:
                assert _adjoint_mismatches(cc, size, d, torch.float32, fused=fused) == 0, (size, d)
    finally:
        lib.msd_set_kernel_path(0)


def test_backward_is_the_exact_adjoint_per_tap_and_f64(cc):
    for n, d in _sweep(9):
        for size in ((n, n), (n, 128), (n, n, n), (n, n, 128)):
            for tap in _all_taps(len(size)):
                assert _adjoint_mismatches(cc, size, d, torch.float32, one_hot=tap) == 0, (size, d, tap)
            assert _adjoint_mismatches(cc, size, d, torch.float64) == 0, (size, d)


@pytest.mark.parametrize("size", CONFIG_SIZES, ids=lambda s: "x".join(map(str, s)))
@pytest.mark.parametrize("path", [0, 1], ids=["specialised", "generic"])
def test_backward_is_the_exact_adjoint_at_the_benchmark_extents(cc, lib, size, path):
    lib.msd_set_kernel_path(path)
    try:
        for d in range(1, 11):
            assert _adjoint_mismatches(cc, size, d, torch.float32) == 0, d
            assert _adjoint_mismatches(cc, size, d, torch.float32, fused=True) == 0, d
        for tap in _all_taps(len(size)):
            assert _adjoint_mismatches(cc, size, 7, torch.float32, one_hot=tap, fused=True) == 0, tap
    finally:
        lib.msd_set_kernel_path(0)
