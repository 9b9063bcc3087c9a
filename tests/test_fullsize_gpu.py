"""Properties that do not need the oracle, checked at the image sizes of the
workloads (1024 x 1024 and 128^3; 4 x 512^2, 2048^2 with two output channels and
256^3 for the last one): adjoint identities, constants, linearity, and agreement
of the specialised kernels with the shape-generic ones."""
import pytest
import torch

from cases import rel_err

pytestmark = pytest.mark.gpu

SIZES = [((1024, 1024), 6), ((128, 128, 128), 5)]


@pytest.fixture(scope="module")
def cc():
    from msd_pytorch_amd import msd_custom_convolutions
    return msd_custom_convolutions


def dot(a, b):
    return (a.double() * b.double()).sum().item()


@pytest.mark.parametrize("size,C", SIZES)
@pytest.mark.parametrize("d", [1, 7, 10])
def test_adjoint_identities(cc, size, C, d):
    # <A f, g> == <f, A^T g> and <A_x k, g> == <k, A_x^T g>  (reference tests/test_conv2d.py:218-311)
    torch.manual_seed(d)
    nd = len(size)
    f = torch.randn(1, C, *size, device="cuda")
    g = torch.randn(1, 1, *size, device="cuda")
    k = torch.randn(1, C, *([3] * nd), device="cuda")
    zero = torch.zeros(1, device="cuda")
    Af = torch.empty_like(g)
    cc.conv_forward(f, k, zero, Af, d)
    ATg = torch.zeros_like(f)
    cc.conv_backward_x(g, k, ATg, d)
    lhs, rhs = dot(Af, g), dot(f, ATg)
    assert abs(lhs - rhs) <= 1e-4 * max(abs(lhs), abs(rhs), (Af.double().norm() * g.double().norm()).item() * 1e-2)
    gk = torch.zeros_like(k)
    cc.conv_backward_k(g, f, gk, d)
    rhs2 = dot(k, gk)
    assert abs(lhs - rhs2) <= 1e-4 * max(abs(lhs), abs(rhs2), (Af.double().norm() * g.double().norm()).item() * 1e-2)


@pytest.mark.parametrize("size,C", SIZES)
def test_constants_and_linearity(cc, size, C):
    nd = len(size)
    taps = 3 ** nd
    x = torch.ones(1, C, *size, device="cuda")
    k = torch.ones(1, C, *([3] * nd), device="cuda")
    y = torch.empty(1, 1, *size, device="cuda")
    for d in (1, 10):
        cc.conv_relu_forward(x, k, torch.zeros(1, device="cuda"), y, d)
        assert torch.equal(y, torch.full_like(y, float(C * taps)))
    torch.manual_seed(0)
    a, b = torch.randn_like(x), torch.randn_like(x)
    k = torch.randn_like(k)
    zero = torch.zeros(1, device="cuda")
    ya, yb, yab = torch.empty_like(y), torch.empty_like(y), torch.empty_like(y)
    cc.conv_forward(a, k, zero, ya, 3)
    cc.conv_forward(b, k, zero, yb, 3)
    cc.conv_forward(2 * a - b, k, zero, yab, 3)
    assert rel_err(yab, 2 * ya - yb) <= 1e-5


@pytest.mark.parametrize("size,C", SIZES)
@pytest.mark.parametrize("d", [1, 10])
def test_specialised_kernels_agree_with_generic_ones(cc, size, C, d):
    from msd_pytorch_amd import _native
    lib = _native.load()
    torch.manual_seed(1)
    nd = len(size)
    stack = torch.randn(1, C + 1, *size, device="cuda")
    grads = torch.randn(1, C + 1, *size, device="cuda")
    k = torch.randn(1, C, *([3] * nd), device="cuda") * 0.2
    bias = torch.randn(1, device="cuda") * 0.1
    results = []
    try:
        for path in (1, 0):
            lib.msd_set_kernel_path(path)
            s, g = stack.clone(), grads.clone()
            gk, gb = torch.zeros_like(k), torch.zeros_like(bias)
            cc.conv_relu_forward(s[:, :C], k, bias, s[:, C:], d)
            cc.conv_relu_backward_x(s[:, C:], g[:, C:], k, g[:, :C], d)
            cc.conv_relu_backward_kb(s[:, C:], g[:, C:], s[:, :C], gk, gb, d)
            results.append((s, g, gk, gb))
    finally:
        lib.msd_set_kernel_path(0)
    (s0, g0, gk0, gb0), (s1, g1, gk1, gb1) = results
    assert rel_err(s1, s0) <= 1e-5
    assert rel_err(g1, g0) <= 1e-4
    assert rel_err(gk1, gk0) <= 1e-4
    assert rel_err(gb1, gb0) <= 1e-4


# the image sizes of the other workloads: 4 x 512^2 (batch), 2048^2 with two output
# channels per layer, 256^3
OTHER_SIZES = [(4, (512, 512), 6, 1), (1, (2048, 2048), 4, 2), (1, (256, 256, 256), 3, 1), (2, (512, 512), 18, 2)]


@pytest.mark.parametrize("batch,size,C,width", OTHER_SIZES)
@pytest.mark.parametrize("d", [2, 9])
def test_other_workload_sizes_specialised_against_generic(cc, batch, size, C, width, d):
    _compare_kernel_families(cc, batch, size, C, width, d)


# stacks of more than 2^30 values (4 GiB): the one-pass backward kernel then addresses the input
# channels block by block; 2048-wide rows are also cut into segments
BIG_STACKS = [(1, (2048, 2048), 258, 2, 7), (1, (128, 128, 128), 520, 1, 3)]


@pytest.mark.parametrize("batch,size,C,width,d", BIG_STACKS)
def test_big_stacks_specialised_against_generic(cc, batch, size, C, width, d):
    _compare_kernel_families(cc, batch, size, C, width, d)


def _compare_kernel_families(cc, batch, size, C, width, d):
    # every operator, and the three plain backward operators as one call, on both kernel families
    from msd_pytorch_amd import _native
    lib = _native.load()
    torch.manual_seed(2)
    nd = len(size)
    stack = torch.randn(batch, C + width, *size, device="cuda")
    grads = torch.randn(batch, C + width, *size, device="cuda")
    k = torch.randn(width, C, *([3] * nd), device="cuda") * 0.2
    bias = torch.randn(width, device="cuda") * 0.1
    results = []
    try:
        for path in (1, 0):
            lib.msd_set_kernel_path(path)
            s, g, g2 = stack.clone(), grads.clone(), grads.clone()
            gk, gb = torch.zeros_like(k), torch.zeros_like(bias)
            gk2, gb2 = torch.zeros_like(k), torch.zeros_like(bias)
            cc.conv_relu_forward(s[:, :C], k, bias, s[:, C:], d)
            # both families mask with the activations of the first forward pass: one that is
            # within rounding of zero may come out with the other sign from the other kernel
            m = results[0][0] if results else s
            cc.conv_relu_backward_x(m[:, C:], g[:, C:], k, g[:, :C], d)
            cc.conv_relu_backward_kb(m[:, C:], g[:, C:], m[:, :C], gk, gb, d)
            cc.conv_backward_xkb(g2[:, C:], s[:, :C], k, g2[:, :C], gk2, gb2, d)
            results.append((s, g, gk, gb, g2, gk2, gb2))
    finally:
        lib.msd_set_kernel_path(0)
    generic, fast = results
    for name, a, b, tol in zip(("forward", "backward_x", "backward_k", "backward_bias", "xkb grad_input",
                                "xkb grad_kernel", "xkb grad_bias"), fast, generic,
                               (1e-5, 1e-4, 1e-4, 1e-4, 1e-4, 1e-4, 1e-4)):
        assert rel_err(a, b) <= tol, name
