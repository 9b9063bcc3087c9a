"""Parity of the HIP operators (called through the C ABI of libmsd_hip.so via
msd_pytorch_amd.msd_custom_convolutions) with the CPU oracle on identical
seeded inputs.

Tolerances (max |diff| / max |ref|): fp32 forward 1e-5, fp32 gradients 1e-4
(their summation order differs from the oracle's), fp64 1e-11."""
import pytest
import torch

import oracle
from cases import ALL_SHAPES, SHAPES_FAST, make_problem, rel_err

pytestmark = pytest.mark.gpu

TOL_FWD = {torch.float32: 1e-5, torch.float64: 1e-11}
TOL_GRAD = {torch.float32: 1e-4, torch.float64: 1e-11}


@pytest.fixture(scope="module")
def cc():
    from msd_pytorch_amd import msd_custom_convolutions
    return msd_custom_convolutions


def run_all(ops, p, relu):
    """forward, backward_x (accumulating into noise), backward_k, backward_bias."""
    gk = torch.zeros_like(p["k"])
    gb = torch.zeros_like(p["bias"])
    if relu:
        ops.conv_relu_forward(p["x"], p["k"], p["bias"], p["y"], p["d"])
        ops.conv_relu_backward_x(p["y"], p["gy"], p["k"], p["gx"], p["d"])
        ops.conv_relu_backward_k(p["y"], p["gy"], p["x"], gk, p["d"])
        ops.conv_relu_backward_bias(p["y"], p["gy"], gb)
    else:
        ops.conv_forward(p["x"], p["k"], p["bias"], p["y"], p["d"])
        ops.conv_backward_x(p["gy"], p["k"], p["gx"], p["d"])
        ops.conv_backward_k(p["gy"], p["x"], gk, p["d"])
        ops.conv_backward_bias(p["gy"], gb)
    return gk, gb


def check_case(cc, shape, dtype, relu):
    ref = make_problem(shape, dtype)
    dev = make_problem(shape, dtype, device="cuda")
    want_gk, want_gb = run_all(oracle, ref, relu)
    got_gk, got_gb = run_all(cc, dev, relu)
    torch.cuda.synchronize()
    # the whole stack: the input channels must be untouched, the output channels match
    assert rel_err(dev["stack"], ref["stack"]) <= TOL_FWD[dtype], "forward"
    assert torch.equal(dev["x"].cpu(), ref["x"]), "forward wrote outside its output channels"
    assert rel_err(dev["gstack"], ref["gstack"]) <= TOL_GRAD[dtype], "backward_x"
    assert torch.equal(dev["gy"].cpu(), ref["gy"]), "backward_x wrote outside grad_input"
    assert rel_err(got_gk, want_gk) <= TOL_GRAD[dtype], "backward_k"
    assert rel_err(got_gb, want_gb) <= TOL_GRAD[dtype], "backward_bias"


@pytest.mark.parametrize("relu", [1, 0])
@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
@pytest.mark.parametrize("shape", ALL_SHAPES)
def test_small_shapes(cc, shape, dtype, relu):
    check_case(cc, shape, dtype, relu)


@pytest.mark.parametrize("relu", [1, 0])
@pytest.mark.parametrize("shape", SHAPES_FAST)
def test_larger_shapes_f32(cc, shape, relu):
    check_case(cc, shape, torch.float32, relu)


@pytest.mark.parametrize("shape", [SHAPES_FAST[1], SHAPES_FAST[7]])
def test_larger_shapes_f64(cc, shape):
    check_case(cc, shape, torch.float64, 1)


def test_fused_weight_and_bias_gradient(cc):
    for shape in (SHAPES_FAST[3], SHAPES_FAST[8]):
        p = make_problem(shape, torch.float32, device="cuda")
        cc.conv_relu_forward(p["x"], p["k"], p["bias"], p["y"], p["d"])
        gk0, gb0 = torch.zeros_like(p["k"]), torch.zeros_like(p["bias"])
        cc.conv_relu_backward_k(p["y"], p["gy"], p["x"], gk0, p["d"])
        cc.conv_relu_backward_bias(p["y"], p["gy"], gb0)
        gk1, gb1 = torch.full_like(p["k"], 2.0), torch.full_like(p["bias"], -1.0)   # accumulate semantics
        cc.conv_relu_backward_kb(p["y"], p["gy"], p["x"], gk1, gb1, p["d"])
        assert rel_err(gk1 - 2.0, gk0) <= 1e-5
        assert rel_err(gb1 + 1.0, gb0) <= 1e-5


def test_weight_gradient_is_deterministic(cc):
    p = make_problem(SHAPES_FAST[4], torch.float32, device="cuda")
    cc.conv_relu_forward(p["x"], p["k"], p["bias"], p["y"], p["d"])
    runs = []
    for _ in range(3):
        gk, gb = torch.zeros_like(p["k"]), torch.zeros_like(p["bias"])
        cc.conv_relu_backward_kb(p["y"], p["gy"], p["x"], gk, gb, p["d"])
        runs.append((gk.clone(), gb.clone()))
    for gk, gb in runs[1:]:
        assert torch.equal(gk, runs[0][0]) and torch.equal(gb, runs[0][1])


def test_output_is_written_in_place_and_constant_input(cc):
    # ones (*) ones = 9 * C everywhere, borders included (reference tests/test_conv2d.py:47-72)
    for size, taps in (((20, 33), 9), ((6, 9, 70), 27)):
        x = torch.ones(1, 3, *size, device="cuda")
        k = torch.ones(2, 3, *([3] * len(size)), device="cuda")
        y = torch.empty(1, 2, *size, device="cuda")
        ptr = y.data_ptr()
        for d in (1, 2, 5):
            cc.conv_relu_forward(x, k, torch.zeros(2, device="cuda"), y, d)
            assert y.data_ptr() == ptr
            assert torch.equal(y, torch.full_like(y, 3.0 * taps))


def test_dilation_error(cc):
    # reference tests/test_conv2d.py:76-90: 2x2 image, d = 1, 2 fine, d = 3 raises
    x = torch.zeros(1, 1, 2, 2, device="cuda")
    k = torch.zeros(1, 1, 3, 3, device="cuda")
    b = torch.zeros(1, device="cuda")
    y = torch.zeros(1, 1, 2, 2, device="cuda")
    cc.conv_forward(x, k, b, y, 1)
    cc.conv_forward(x, k, b, y, 2)
    with pytest.raises(RuntimeError):
        cc.conv_forward(x, k, b, y, 3)
    with pytest.raises(RuntimeError):
        cc.conv_relu_forward(x, k, b, y, 0)
    torch.cuda.synchronize()


def test_dtype_and_device_errors(cc):
    # reference tests/test_conv2d.py:93-106
    x = torch.zeros(1, 1, 5, 5, device="cuda")
    k = torch.zeros(1, 1, 3, 3, device="cuda")
    b = torch.zeros(1, device="cuda")
    y = torch.zeros(1, 1, 5, 5, device="cuda")
    with pytest.raises(RuntimeError):
        cc.conv_forward(x.double(), k, b, y, 1)
    with pytest.raises(RuntimeError):
        cc.conv_forward(x.cpu(), k, b, y, 1)
    with pytest.raises(RuntimeError):
        cc.conv_relu_forward(x, torch.zeros(1, 1, 3, 6, device="cuda")[..., ::2], b, y, 1)   # non-contiguous kernel
    with pytest.raises(RuntimeError):
        cc.conv_relu_forward(x, torch.zeros(1, 2, 3, 3, device="cuda"), b, y, 1)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
@pytest.mark.parametrize("shape", [ALL_SHAPES[5], ALL_SHAPES[10], SHAPES_FAST[3], SHAPES_FAST[8]])
def test_mask_once_then_plain_operators(cc, shape, dtype):
    # masking the gradient in place and calling the plain operators (what the dense
    # block does) equals the three conv_relu_backward_* operators
    p = make_problem(shape, dtype, device="cuda")
    cc.conv_relu_forward(p["x"], p["k"], p["bias"], p["y"], p["d"])
    gx0 = p["gx"].clone()
    gk0, gb0 = torch.zeros_like(p["k"]), torch.zeros_like(p["bias"])
    cc.conv_relu_backward_x(p["y"], p["gy"], p["k"], gx0, p["d"])
    cc.conv_relu_backward_kb(p["y"], p["gy"], p["x"], gk0, gb0, p["d"])

    gy = p["gy"].clone()
    cc.relu_mask_gradient(p["y"], gy)
    assert torch.equal(gy, p["gy"] * (p["y"] > 0))
    gx1 = p["gx"].clone()
    gk1, gb1 = torch.zeros_like(p["k"]), torch.zeros_like(p["bias"])
    cc.conv_backward_x(gy, p["k"], gx1, p["d"])
    cc.conv_backward_kb(gy, p["x"], gk1, gb1, p["d"])
    tol = 1e-5 if dtype == torch.float32 else 1e-12
    assert rel_err(gx1, gx0) <= tol and rel_err(gk1, gk0) <= tol and rel_err(gb1, gb0) <= tol


# shapes the one-pass kernel behind conv_backward_xkb takes (one output channel, rows of whole
# 4-voxel groups, at least one wavefront per row), beside the SHAPES_FAST ones that qualify
SHAPES_XKB = [
    (1, 17, 1, (5, 256), 2),          # 4 voxels per lane, 4 rows per workgroup, 2 channel blocks
    (2, 3, 1, (9, 1024), 9),          # one row per workgroup, dilation == height
    (1, 40, 1, (6, 7, 128), 3),       # 3D, 3 channel blocks
    (1, 2, 1, (4, 5, 68), 4),         # 3D, ragged row
    (2, 5, 2, (7, 128), 2),           # two output channels: 2 voxels per lane, 2 rows per workgroup
    (1, 35, 2, (12, 512), 5),         # two output channels, 3 channel blocks, one row per workgroup
    (1, 16, 2, (9, 68), 3),           # two output channels, one voxel per lane, exactly one channel block
    # rows longer than one workgroup covers: cut into segments with a halo of `dilation` values
    (1, 3, 1, (5, 2048), 1),          # 2 segments of 1024
    (2, 18, 1, (7, 2048), 5),         # 2 channel blocks, folds in y
    (1, 4, 1, (130, 1536), 128),      # 3 segments of 512, the largest dilation the halo takes
    (1, 2, 1, (140, 2048), 129),      # dilation past that: the separate kernels
    (1, 5, 2, (8, 1024), 7),          # two output channels: four voxels per lane, one tile per row
    (1, 3, 2, (4, 2048), 3),          # two output channels: 2 segments of 1024
    # rows that are not whole groups of four voxels (unaligned rows of the input stack)
    (1, 3, 1, (6, 750), 2),           # 2 voxels per lane, a short second segment
    (2, 18, 1, (5, 1001), 3),         # odd: one voxel per lane, 4 segments
    (1, 3, 1, (8, 1025), 5),          # the last segment holds one voxel: its mirrored taps come from the halo
    (1, 5, 2, (7, 1022), 4),          # two output channels
    (1, 4, 1, (9, 250), 3),           # whole rows per team, the last group of four is half empty
    (1, 7, 1, (5, 6, 130), 2),        # 3D
    (1, 3, 1, (4, 5, 127), 1),        # 3D, odd
    (1, 3, 1, (4, 5, 512), 3),        # 3D rows of 512 voxels: two voxels per lane
    (2, 18, 1, (3, 4, 300), 2),       # 3D, two voxels per lane, lanes past the row's end, folds in z and y
]


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
@pytest.mark.parametrize("shape", SHAPES_XKB + [ALL_SHAPES[5], ALL_SHAPES[9], SHAPES_FAST[0], SHAPES_FAST[3],
                                                SHAPES_FAST[5], SHAPES_FAST[6], SHAPES_FAST[9]])
def test_backward_xkb_equals_the_three_operators(cc, shape, dtype):
    # one call (one pass over the channels where the fused kernel applies; fp64, two output
    # channels in 3D and odd row lengths take the separate kernels) against the oracle's
    # conv_backward_x, conv_backward_k and conv_backward_bias, all accumulating
    ref = make_problem(shape, dtype, seed=5)
    dev = make_problem(shape, dtype, device="cuda", seed=5)
    want_gk, want_gb = torch.ones_like(ref["k"]), torch.full_like(ref["bias"], 2.0)
    oracle.conv_backward_x(ref["gy"], ref["k"], ref["gx"], ref["d"])
    oracle.conv_backward_k(ref["gy"], ref["x"], want_gk, ref["d"])
    oracle.conv_backward_bias(ref["gy"], want_gb)
    got_gk, got_gb = torch.ones_like(dev["k"]), torch.full_like(dev["bias"], 2.0)
    cc.conv_backward_xkb(dev["gy"], dev["x"], dev["k"], dev["gx"], got_gk, got_gb, dev["d"])
    torch.cuda.synchronize()
    assert rel_err(dev["gstack"], ref["gstack"]) <= TOL_GRAD[dtype], "grad_input"
    assert torch.equal(dev["gy"].cpu(), ref["gy"]), "wrote outside grad_input"
    assert rel_err(got_gk, want_gk) <= TOL_GRAD[dtype], "grad_kernel"
    assert rel_err(got_gb, want_gb) <= TOL_GRAD[dtype], "grad_bias"


def test_backward_xkb_without_bias_and_errors(cc):
    p = make_problem(SHAPES_FAST[0], torch.float32, device="cuda")
    gk = torch.zeros_like(p["k"])
    gk2 = torch.zeros_like(p["k"])
    gx2 = p["gx"].clone()
    cc.conv_backward_xkb(p["gy"], p["x"], p["k"], p["gx"], gk, None, p["d"])
    cc.conv_backward_x(p["gy"], p["k"], gx2, p["d"])
    cc.conv_backward_k(p["gy"], p["x"], gk2, p["d"])
    assert rel_err(p["gx"], gx2) <= 1e-5 and rel_err(gk, gk2) <= 1e-5
    with pytest.raises(RuntimeError):
        cc.conv_backward_xkb(p["gy"], p["x"], p["k"], p["gx"], gk, None, 65)      # dilation > size
    with pytest.raises(RuntimeError):
        cc.conv_backward_xkb(p["gy"].cpu(), p["x"], p["k"], p["gx"], gk, None, 1)  # CPU tensor


# The reference's own value tests (tests/test_conv2d.py:126-186, tests/test_conv3d.py:323-374):
# away from the borders symmetric padding plays no part, so the centre of the output must
# agree with torch's zero-padded dilated convolution.  Their parameter grid, in double; torch's
# convolution runs on the CPU (an independent implementation, no GPU library involved).
REFERENCE_VALUE_GRID = [(2, 3, 5, d, size) for d in (1, 3, 10) for size in (2 * d + 1, 29, 50)]


@pytest.mark.parametrize("ndim", [2, 3])
@pytest.mark.parametrize("B,c_in,c_out,d,size", REFERENCE_VALUE_GRID)
def test_centre_agrees_with_torch_convolution(ndim, B, c_in, c_out, d, size):
    import torch.nn.functional as F
    from msd_pytorch_amd.conv2d import conv2d_forward
    from msd_pytorch_amd.conv3d import conv3d_relu
    shape = (size, 2 * size) if ndim == 2 else (size, 2 * size, 3 * size)
    gen = torch.Generator().manual_seed(d * 100 + size)
    x = torch.randn(B, c_in, *shape, dtype=torch.double, generator=gen)
    k = torch.randn(c_out, c_in, *([3] * ndim), dtype=torch.double, generator=gen)
    bias = torch.randn(c_out, dtype=torch.double, generator=gen)
    y = torch.zeros(B, c_out, *shape, dtype=torch.double, device="cuda")
    if ndim == 2:
        conv2d_forward(x.cuda(), k.cuda(), bias.cuda(), y, d)
        want = F.conv2d(x, k, bias, padding=d, dilation=d)
    else:
        conv3d_relu(x.cuda(), k.cuda(), bias.cuda(), y, 1, d)
        want = F.relu(F.conv3d(x, k, bias, padding=d, dilation=d))
    assert want.shape == y.shape
    centre = (slice(None), slice(None)) + (slice(d, -d),) * ndim
    assert torch.allclose(y.cpu()[centre], want[centre], rtol=1e-10, atol=1e-10)


@pytest.mark.parametrize("ndim,size", [(2, 128), (3, 44)])
@pytest.mark.parametrize("c_out", [1, 2])
@pytest.mark.parametrize("d", [1, 4, 10])
def test_centre_agrees_with_torch_convolution_f32_specialised(ndim, size, c_out, d):
    # the same check at shapes the specialised fp32 kernels take (rows of 256 / 132 voxels,
    # one or two output channels); tolerance: forward, relative 1e-5
    import torch.nn.functional as F
    shape = (size, 2 * size) if ndim == 2 else (size, size + 3, 3 * size)
    gen = torch.Generator().manual_seed(d)
    x = torch.randn(2, 7, *shape, generator=gen)
    k = torch.randn(c_out, 7, *([3] * ndim), generator=gen) * 0.2
    bias = torch.randn(c_out, generator=gen)
    y = torch.zeros(2, c_out, *shape, device="cuda")
    from msd_pytorch_amd import msd_custom_convolutions as native
    native.conv_relu_forward(x.cuda(), k.cuda(), bias.cuda(), y, d)
    conv = F.conv2d if ndim == 2 else F.conv3d
    want = F.relu(conv(x.double(), k.double(), bias.double(), padding=d, dilation=d))
    centre = (slice(None), slice(None)) + (slice(d, -d),) * ndim
    assert rel_err(y.cpu()[centre], want[centre]) <= 1e-5
