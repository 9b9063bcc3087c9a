"""Pins the CPU oracle (oracle/) against things that share no code with it:
numpy's symmetric padding, stock torch convolutions and autograd, closed forms
and adjoint identities.  The reference's own tests hold no stored vectors; the
checks below are the ones they make (tests/test_conv2d.py, tests/test_conv3d.py,
tests/test_msd_block.py of the reference), done element-wise."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

import oracle
from composite import conv_sym, dense_block, symmetric_index

torch.manual_seed(0)

SHAPES_2D = [
    # (B, C_in, C_out, (H, W), dilation)
    (1, 1, 1, (1, 5), 1),      # strip: height == dilation (reference tests/test_msd_block.py:11)
    (2, 3, 5, (3, 6), 1),      # size = 2d+1
    (2, 3, 5, (7, 14), 3),     # size = 2d+1 for d = 3
    (1, 2, 2, (3, 3), 3),      # size == d in both axes: every tap folds
    (1, 4, 1, (10, 13), 10),   # size == d in one axis
    (2, 3, 2, (13, 21), 3),    # the gradcheck shape of reference tests/test_conv2d.py:488-515
    (1, 5, 3, (29, 58), 10),
]
SHAPES_3D = [
    (1, 1, 1, (1, 1, 5), 1),
    (2, 3, 2, (3, 6, 9), 1),
    (1, 2, 2, (2, 2, 2), 2),   # size == d on every axis
    (1, 3, 2, (5, 7, 11), 2),
    (2, 2, 3, (7, 14, 21), 3),
    (1, 2, 1, (11, 13, 7), 3),  # the gradcheck shape of reference tests/test_conv3d.py:376-405
]
ALL_SHAPES = SHAPES_2D + SHAPES_3D


def make(B, C, Wd, size, dtype, strided=True):
    """Input/output as channel slices of one stack (batch stride = C_total * plane)."""
    ndim = len(size)
    stack = torch.randn(B, C + Wd, *size, dtype=dtype)
    x = stack[:, :C] if strided else stack[:, :C].contiguous()
    y = stack[:, C:]
    k = torch.randn(Wd, C, *([3] * ndim), dtype=dtype)
    bias = torch.randn(Wd, dtype=dtype)
    return x, k, bias, y


# ---------------------------------------------------------------- index map

def test_reflect_equals_numpy_symmetric():
    for n in range(1, 41):
        for d in range(1, n + 1):
            want = np.pad(np.arange(n), d, mode="symmetric")
            got = [oracle.reflect(i, n) for i in range(-d, n + d)]
            assert got == want.tolist(), (n, d)


def test_reflect_brute_force_table():
    # unfold the axis by mirroring about the half-sample edges, no closed form
    for n in range(1, 13):
        tile = list(range(n)) + list(range(n - 1, -1, -1))  # period 2n
        for i in range(-n, 2 * n):
            assert oracle.reflect(i, n) == tile[i % (2 * n)], (i, n)


def test_reflect_differs_from_torch_reflect():
    # torch's "reflect" does not repeat the edge sample: -1 -> 1, here -1 -> 0
    assert oracle.reflect(-1, 5) == 0
    assert oracle.reflect(5, 5) == 4


# ---------------------------------------------------------------- forward

@pytest.mark.parametrize("shape", ALL_SHAPES)
@pytest.mark.parametrize("relu", [0, 1])
def test_forward_vs_composite_f64(shape, relu):
    B, C, Wd, size, d = shape
    x, k, bias, y = make(B, C, Wd, size, torch.float64)
    op = oracle.conv_relu_forward if relu else oracle.conv_forward
    op(x, k, bias, y, d)
    want = conv_sym(x, k, bias, d, relu=bool(relu))
    assert torch.allclose(y, want, rtol=1e-12, atol=1e-12)


@pytest.mark.parametrize("shape", ALL_SHAPES)
def test_forward_vs_composite_f32(shape):
    B, C, Wd, size, d = shape
    x, k, bias, y = make(B, C, Wd, size, torch.float32)
    oracle.conv_relu_forward(x, k, bias, y, d)
    want = conv_sym(x.double(), k.double(), bias.double(), d).float()
    assert (y - want).abs().max() <= 1e-5 * max(1.0, want.abs().max().item())


@pytest.mark.parametrize("ndim", [2, 3])
def test_forward_constant_input(ndim):
    # symmetric padding keeps constants: ones (*) ones = taps * C everywhere,
    # borders included (cf. reference tests/test_conv2d.py:47-72)
    size = (6, 9) if ndim == 2 else (4, 6, 5)
    C = 3
    x = torch.ones(1, C, *size)
    k = torch.ones(2, C, *([3] * ndim))
    bias = torch.zeros(2)
    y = torch.empty(1, 2, *size)
    for d in (1, 2, 4):
        oracle.conv_relu_forward(x, k, bias, y, d)
        assert torch.equal(y, torch.full_like(y, C * 3 ** ndim))


def test_forward_zero_weights_gives_clamped_bias():
    x = torch.randn(2, 3, 8, 9)
    k = torch.zeros(2, 3, 3, 3)
    bias = torch.tensor([0.75, -0.5])
    y = torch.empty(2, 2, 8, 9)
    oracle.conv_relu_forward(x, k, bias, y, 2)
    assert torch.equal(y[:, 0], torch.full_like(y[:, 0], 0.75))
    assert torch.equal(y[:, 1], torch.zeros_like(y[:, 1]))


@pytest.mark.parametrize("d", [1, 3, 10])
@pytest.mark.parametrize("ndim", [2, 3])
def test_forward_interior_vs_stock_dilated_conv(d, ndim):
    # the reference's own check (tests/test_conv2d.py:154-185, tests/test_conv3d.py:336-373):
    # away from the border, the op is torch's zero-padded dilated convolution
    s = 2 * d + 3
    size = (s, 2 * s) if ndim == 2 else (s, s + 1, s + 2)
    x = torch.randn(2, 3, *size, dtype=torch.float64)
    k = torch.randn(5, 3, *([3] * ndim), dtype=torch.float64)
    bias = torch.randn(5, dtype=torch.float64)
    y = torch.empty(2, 5, *size, dtype=torch.float64)
    oracle.conv_forward(x, k, bias, y, d)
    conv = F.conv2d if ndim == 2 else F.conv3d
    want = conv(x, k, bias, dilation=d, padding=d)
    inner = (slice(None), slice(None)) + (slice(d, -d),) * ndim
    assert torch.allclose(y[inner], want[inner], rtol=1e-12, atol=1e-12)


# ---------------------------------------------------------------- gradients

def autograd_reference(x, k, bias, d, relu, gy):
    x = x.detach().clone().requires_grad_(True)
    k = k.detach().clone().requires_grad_(True)
    bias = bias.detach().clone().requires_grad_(True)
    y = conv_sym(x, k, bias, d, relu=relu)
    y.backward(gy)
    return y.detach(), x.grad, k.grad, bias.grad


@pytest.mark.parametrize("shape", ALL_SHAPES)
@pytest.mark.parametrize("relu", [0, 1])
def test_gradients_vs_autograd_f64(shape, relu):
    B, C, Wd, size, d = shape
    x, k, bias, y = make(B, C, Wd, size, torch.float64)
    gstack = torch.randn(B, C + Wd, *size, dtype=torch.float64)
    gy = gstack[:, C:]
    want_y, want_gx, want_gk, want_gb = autograd_reference(x, k, bias, d, bool(relu), gy)
    if relu:
        oracle.conv_relu_forward(x, k, bias, y, d)
    else:
        oracle.conv_forward(x, k, bias, y, d)
    assert torch.allclose(y, want_y, rtol=1e-12, atol=1e-12)

    # backward_x accumulates: prefill with noise and compare the difference
    gx = gstack[:, :C]
    before = gx.clone()
    gk = torch.zeros_like(k)
    gb = torch.zeros_like(bias)
    if relu:
        oracle.conv_relu_backward_x(y, gy, k, gx, d)
        oracle.conv_relu_backward_k(y, gy, x, gk, d)
        oracle.conv_relu_backward_bias(y, gy, gb)
    else:
        oracle.conv_backward_x(gy, k, gx, d)
        oracle.conv_backward_k(gy, x, gk, d)
        oracle.conv_backward_bias(gy, gb)
    assert torch.allclose(gx - before, want_gx, rtol=1e-10, atol=1e-10)
    assert torch.allclose(gk, want_gk, rtol=1e-10, atol=1e-10)
    assert torch.allclose(gb, want_gb, rtol=1e-10, atol=1e-10)


def test_weight_and_bias_gradients_accumulate():
    x, k, bias, y = make(2, 3, 2, (6, 7), torch.float64)
    gy = torch.randn_like(y)
    oracle.conv_relu_forward(x, k, bias, y, 2)
    gk0, gb0 = torch.zeros_like(k), torch.zeros_like(bias)
    oracle.conv_relu_backward_k(y, gy, x, gk0, 2)
    oracle.conv_relu_backward_bias(y, gy, gb0)
    gk1, gb1 = torch.full_like(k, 3.0), torch.full_like(bias, -2.0)
    oracle.conv_relu_backward_k(y, gy, x, gk1, 2)
    oracle.conv_relu_backward_bias(y, gy, gb1)
    assert torch.allclose(gk1 - 3.0, gk0)
    assert torch.allclose(gb1 + 2.0, gb0)


@pytest.mark.parametrize("ndim,size,d", [(2, (7, 13), 3), (3, (11, 7, 9), 3), (2, (3, 4), 3)])
def test_adjoint_identity_in_x(ndim, size, d):
    # <A f, g> == <f, A^T g>  (reference tests/test_conv2d.py:218-262, tests/test_conv3d.py:109-154)
    for _ in range(5):
        f = torch.randn(2, 5, *size, dtype=torch.float64)
        g = torch.randn(2, 3, *size, dtype=torch.float64)
        k = torch.randn(3, 5, *([3] * ndim), dtype=torch.float64)
        Af = torch.empty_like(g)
        oracle.conv_forward(f, k, torch.zeros(3, dtype=torch.float64), Af, d)
        ATg = torch.zeros_like(f)
        oracle.conv_backward_x(g, k, ATg, d)
        assert torch.allclose((Af * g).sum(), (f * ATg).sum(), rtol=1e-10)


@pytest.mark.parametrize("ndim,size,d", [(2, (25, 31), 10), (3, (9, 11, 7), 4)])
def test_adjoint_identity_in_k(ndim, size, d):
    # <A_x k, g> == <k, A_x^T g>  (reference tests/test_conv2d.py:265-311, tests/test_conv3d.py:159-207)
    x = torch.randn(2, 4, *size, dtype=torch.float64)
    g = torch.randn(2, 3, *size, dtype=torch.float64)
    k = torch.randn(3, 4, *([3] * ndim), dtype=torch.float64)
    Ak = torch.empty_like(g)
    oracle.conv_forward(x, k, torch.zeros(3, dtype=torch.float64), Ak, d)
    gk = torch.zeros_like(k)
    oracle.conv_backward_k(g, x, gk, d)
    assert torch.allclose((Ak * g).sum(), (k * gk).sum(), rtol=1e-10)


def test_backward_x_dense_jacobian_tiny():
    # brute force: column j of the Jacobian is A applied to the j-th unit image
    H, W, d = 4, 5, 2
    k = torch.randn(1, 1, 3, 3, dtype=torch.float64)
    zero = torch.zeros(1, dtype=torch.float64)
    J = torch.empty(H * W, H * W, dtype=torch.float64)
    for j in range(H * W):
        e = torch.zeros(H * W, dtype=torch.float64)
        e[j] = 1
        out = torch.empty(1, 1, H, W, dtype=torch.float64)
        oracle.conv_forward(e.view(1, 1, H, W), k, zero, out, d)
        J[:, j] = out.flatten()
    g = torch.randn(1, 1, H, W, dtype=torch.float64)
    gx = torch.zeros(1, 1, H, W, dtype=torch.float64)
    oracle.conv_backward_x(g, k, gx, d)
    assert torch.allclose(gx.flatten(), J.t() @ g.flatten(), rtol=1e-12, atol=1e-12)


def test_bias_gradient_is_masked_sum():
    # reference tests/test_conv2d.py:314-330
    y = torch.randn(3, 4, 9, 8, dtype=torch.float64)
    gy = torch.randn_like(y)
    gb = torch.zeros(4, dtype=torch.float64)
    oracle.conv_relu_backward_bias(y, gy, gb)
    assert torch.allclose(gb, (gy * (y > 0)).sum((0, 2, 3)))
    gb.zero_()
    oracle.conv_backward_bias(gy, gb)
    assert torch.allclose(gb, gy.sum((0, 2, 3)))


# ---------------------------------------------------------------- dense block

@pytest.mark.parametrize("ndim,size", [(2, (13, 21)), (3, (5, 7, 11)), (2, (1, 5))])
@pytest.mark.parametrize("width", [1, 2])
def test_block_vs_dense_composite(ndim, size, width):
    c_in = 3
    dil = [1, 2, 3] if min(size) >= 3 else [1, 1, 1]
    weights = [torch.randn(width, c_in + width * i, *([3] * ndim), dtype=torch.float64) * 0.3
               for i in range(len(dil))]
    bias = torch.randn(width * len(dil), dtype=torch.float64) * 0.1
    x = torch.randn(2, c_in, *size, dtype=torch.float64)

    xr = x.clone().requires_grad_(True)
    wr = [w.clone().requires_grad_(True) for w in weights]
    br = bias.clone().requires_grad_(True)
    want = dense_block(xr, dil, br, wr)
    g = torch.randn_like(want)
    want.backward(g)

    result = oracle.block_forward(x, dil, bias, weights)
    assert torch.allclose(result, want.detach(), rtol=1e-12, atol=1e-12)
    gx, gb, gws = oracle.block_backward(result, g, dil, bias, weights)
    assert torch.allclose(gx, xr.grad, rtol=1e-10, atol=1e-10)
    assert torch.allclose(gb, br.grad, rtol=1e-10, atol=1e-10)
    for a, b in zip(gws, wr):
        assert torch.allclose(a, b.grad, rtol=1e-10, atol=1e-10)
