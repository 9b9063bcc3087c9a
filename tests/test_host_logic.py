"""Host-side logic without a GPU.  The operator module's functions are replaced
by the CPU oracle (test infrastructure) so that the dense-block loop, the module
and the argument checks can be exercised on CPU tensors; the shipped package has
no such path."""
import math

import pytest
import torch

import oracle
from composite import dense_block

import msd_pytorch_amd
from msd_pytorch_amd import msd_custom_convolutions as cc
from msd_pytorch_amd.conv2d import conv2d_relu
from msd_pytorch_amd.conv3d import conv3d_relu
from msd_pytorch_amd.msd_block import MSDBlock, MSDBlock2d, MSDBlock3d, msd_block
from msd_pytorch_amd.msd_model import _moments, scaling_module
from msd_pytorch_amd.msd_module import MSDFinalLayer, MSDModule, init_convolution_weights, units_in_front

OPS = ["conv_forward", "conv_backward_x", "conv_backward_k", "conv_backward_bias", "conv_relu_forward",
       "conv_relu_backward_x", "conv_relu_backward_k", "conv_relu_backward_bias"]


@pytest.fixture
def oracle_ops(monkeypatch):
    for name in OPS:
        monkeypatch.setattr(cc, name, getattr(oracle, name))

    def kb(output, grad_output, input, grad_kernel, grad_bias, dilation, block_size=None):
        oracle.conv_relu_backward_k(output, grad_output, input, grad_kernel, dilation)
        if grad_bias is not None:
            oracle.conv_relu_backward_bias(output, grad_output, grad_bias)
    monkeypatch.setattr(cc, "conv_relu_backward_kb", kb)

    def plain_kb(grad_output, input, grad_kernel, grad_bias, dilation, block_size=None):
        oracle.conv_backward_k(grad_output, input, grad_kernel, dilation)
        if grad_bias is not None:
            oracle.conv_backward_bias(grad_output, grad_bias)
    monkeypatch.setattr(cc, "conv_backward_kb", plain_kb)

    def block_forward(stack, c_in, dilations, bias, weights):
        first, b0 = c_in, 0
        for w, d in zip(weights, dilations):
            n = w.shape[0]
            oracle.conv_relu_forward(stack[:, :first], w, bias[b0:b0 + n], stack[:, first:first + n], d)
            first, b0 = first + n, b0 + n
    monkeypatch.setattr(cc, "block_forward", block_forward)

    def block_backward(stack, grads, c_in, dilations, weights, grad_weights, grad_bias, need_input_grad):
        last = stack.shape[1]
        b1 = last - c_in
        for idx in reversed(range(len(weights))):
            n = weights[idx].shape[0]
            first, b0 = last - n, b1 - n
            out_i, gout_i = stack[:, first:last], grads[:, first:last]
            if idx > 0 or need_input_grad:
                oracle.conv_relu_backward_x(out_i, gout_i, weights[idx], grads[:, :first], dilations[idx])
            if grad_weights[idx] is not None:
                oracle.conv_relu_backward_k(out_i, gout_i, stack[:, :first], grad_weights[idx], dilations[idx])
            if grad_bias is not None:
                oracle.conv_relu_backward_bias(out_i, gout_i, grad_bias[b0:b1])
            last, b1 = first, b0
    monkeypatch.setattr(cc, "block_backward", block_backward)

    def mask(output, grad_output):
        grad_output.mul_((output > 0).to(grad_output.dtype))
    monkeypatch.setattr(cc, "relu_mask_gradient", mask)


def test_top_level_alias_of_the_native_module():
    import msd_custom_convolutions   # the name the reference's Python layers import (conv2d.py:5)
    assert msd_custom_convolutions is cc
    for name in OPS:
        assert callable(getattr(msd_custom_convolutions, name))


# ------------------------------------------------------------ argument checks

def test_cpu_tensors_are_rejected_like_the_reference():
    x = torch.zeros(1, 1, 5, 5)
    with pytest.raises(RuntimeError, match="GPU"):
        cc.conv_relu_forward(x, torch.zeros(1, 1, 3, 3), torch.zeros(1), x.clone(), 1)
    with pytest.raises(RuntimeError, match="GPU"):
        cc.conv_relu_backward_kb(x, x, x, torch.zeros(1, 1, 3, 3), torch.zeros(1), 1)


def test_dilation_accepts_any_integer_type():
    # the reference's pybind11 int caster takes numpy and torch integer scalars
    # (MSDModule(dilations=np.arange(1, 11)) works upstream); bool and float are refused
    import numpy as np
    img = torch.zeros(1, 1, 8, 8)
    for d in (3, np.int64(3), np.int32(3), torch.tensor(3), np.arange(1, 11)[2]):
        got = cc._check_dilation("f", img, d)
        assert got == 3 and type(got) is int
    for bad in (True, 2.0, np.float32(2), "2", None):
        with pytest.raises(TypeError):
            cc._check_dilation("f", img, bad)


def test_check_helpers_raise_runtime_error():
    with pytest.raises(RuntimeError, match="Dilation must be 1 or greater"):
        cc._check_dilation("f", torch.zeros(1, 1, 4, 4), 0)
    with pytest.raises(RuntimeError, match="Dilation cannot be greater"):
        cc._check_dilation("f", torch.zeros(1, 1, 2, 2), 3)
    cc._check_dilation("f", torch.zeros(1, 1, 2, 2), 2)
    with pytest.raises(RuntimeError, match="3x3"):
        cc._check_kernel("f", torch.zeros(1, 1, 3, 5))
    with pytest.raises(RuntimeError, match="4 or 5 dimensional"):
        cc._check_kernel("f", torch.zeros(1, 3, 3))
    with pytest.raises(RuntimeError, match="contiguous"):
        cc._check_kernel("f", torch.zeros(2, 2, 3, 6)[..., ::2])
    with pytest.raises(RuntimeError, match="same type"):
        cc._check_same_type("f", [("a", torch.zeros(1)), ("b", torch.zeros(1, dtype=torch.float64))])
    with pytest.raises(RuntimeError, match="float32 and float64"):
        cc._check_same_type("f", [("a", torch.zeros(1, dtype=torch.float16))])
    with pytest.raises(RuntimeError, match="batch"):
        cc._check_in_out_shape("f", torch.zeros(1, 1, 4, 4), torch.zeros(2, 1, 4, 4))
    with pytest.raises(RuntimeError, match="shape"):
        cc._check_in_out_shape("f", torch.zeros(1, 1, 4, 4), torch.zeros(1, 1, 4, 5))


# ------------------------------------------------------------ dense block

@pytest.mark.parametrize("ndim,size", [(2, (13, 21)), (3, (5, 7, 11)), (2, (1, 5))])
@pytest.mark.parametrize("width", [1, 2])
def test_block_function_vs_dense_composite(oracle_ops, ndim, size, width):
    c_in = 3
    dil = [1, 2, 3] if min(size) >= 3 else [1, 1, 1]
    torch.manual_seed(1)
    ws = [(torch.randn(width, c_in + width * i, *([3] * ndim), dtype=torch.float64) * 0.3).requires_grad_(True)
          for i in range(len(dil))]
    bias = (torch.randn(width * len(dil), dtype=torch.float64) * 0.1).requires_grad_(True)
    x = torch.randn(2, c_in, *size, dtype=torch.float64, requires_grad=True)
    g = torch.randn(2, c_in + width * len(dil), *size, dtype=torch.float64)

    got = msd_block(x, dil, bias, *ws)
    got.backward(g)
    grads = [t.grad.clone() for t in (x, bias, *ws)]
    for t in (x, bias, *ws):
        t.grad = None
    want = dense_block(x, dil, bias, ws)
    want.backward(g)
    assert torch.allclose(got, want, rtol=1e-12, atol=1e-12)
    for a, t in zip(grads, (x, bias, *ws)):
        assert torch.allclose(a, t.grad, rtol=1e-10, atol=1e-10)


def test_block_skips_gradients_that_are_not_needed(oracle_ops):
    x = torch.randn(1, 2, 6, 7, dtype=torch.float64)              # no grad wanted for the input
    w0 = torch.randn(1, 2, 3, 3, dtype=torch.float64, requires_grad=True)
    w1 = torch.randn(1, 3, 3, 3, dtype=torch.float64)             # frozen layer
    bias = torch.zeros(2, dtype=torch.float64, requires_grad=True)
    out = msd_block(x, [1, 2], bias, w0, w1)
    out.sum().backward()
    assert w0.grad is not None and bias.grad is not None and w1.grad is None


def test_block_argument_errors(oracle_ops):
    x = torch.zeros(1, 1, 4, 4)
    w = torch.zeros(1, 1, 3, 3)
    with pytest.raises(AssertionError):
        msd_block(x, [1, 1], torch.zeros(2), w)             # depth mismatch
    with pytest.raises(AssertionError):
        msd_block(x, [1], torch.zeros(3), w)                # bias length
    with pytest.raises(ValueError):
        msd_block(torch.zeros(1, 1, 4), [1], torch.zeros(1), w)


def test_block_parameters_and_init():
    torch.manual_seed(0)
    blk = MSDBlock(2, [1, 2, 4], width=3, ndim=3)
    names = dict(blk.named_parameters())
    assert sorted(names) == ["bias", "weight0", "weight1", "weight2"]
    assert names["bias"].shape == (9,)
    assert [tuple(names[f"weight{i}"].shape) for i in range(3)] == [(3, 2, 3, 3, 3), (3, 5, 3, 3, 3), (3, 8, 3, 3, 3)]
    assert isinstance(MSDBlock2d(1, [1]), MSDBlock) and isinstance(MSDBlock3d(1, [1]), MSDBlock)
    with pytest.raises(ValueError):
        MSDBlock(1, [1], ndim=4)
    # same RNG draws, in the same order, as msd_block.py:183-191: kaiming_uniform(a=sqrt(5)) then the bias
    torch.manual_seed(0)
    ref_w = [torch.nn.init.kaiming_uniform_(torch.empty_like(names[f"weight{i}"]), a=math.sqrt(5)) for i in range(3)]
    bound = 1 / math.sqrt(2 * 27)
    ref_b = torch.nn.init.uniform_(torch.empty(9), -bound, bound)
    for i in range(3):
        assert torch.equal(names[f"weight{i}"].data, ref_w[i])
    assert torch.equal(names["bias"].data, ref_b)


# ------------------------------------------------------------ module

def test_units_in_front_and_init_std():
    assert units_in_front(3, 2, 0) == 3 and units_in_front(3, 2, 5) == 13
    torch.manual_seed(0)
    w = torch.empty(4, 50, 3, 3)
    init_convolution_weights(w, c_in=1, c_out=2, width=1, depth=100)
    want = math.sqrt(2 / (9 * (1 + 99) + 2))     # msd_module.py:54-57
    assert abs(w.std().item() - want) < 0.05 * want


def test_module_structure_and_zero_output(oracle_ops):
    with pytest.raises(ValueError):
        MSDModule(1, 1, 0, 1)
    with pytest.raises(ValueError):
        MSDModule(1, 1, 1, 0)
    net = MSDModule(2, 3, depth=5, width=2, dilations=[1, 2, 3]).double()
    assert net.dilations == [1, 2, 3, 1, 2]
    keys = set(net.state_dict())
    assert {"msd_block.bias", "msd_block.weight0", "msd_block.weight4", "final_layer.linear.weight",
            "final_layer.linear.bias"} <= keys
    assert net.final_layer.linear.weight.shape == (3, 2 + 2 * 5, 1)
    # the final layer starts at zero, so an untrained network outputs exactly zero (tests/test_msd_module.py:11-16)
    out = net(torch.randn(2, 2, 9, 8, dtype=torch.float64))
    assert out.shape == (2, 3, 9, 8) and torch.equal(out, torch.zeros_like(out))


def test_module_gradcheck(oracle_ops):
    # tests/test_msd_module.py:19-41 of the reference, on a smaller image
    torch.manual_seed(0)
    net = MSDModule(2, 2, depth=4, width=2, dilations=[1, 2, 3]).double()
    net.final_layer.linear.weight.data.normal_()
    x = torch.randn(1, 2, 7, 6, dtype=torch.float64, requires_grad=True)
    assert torch.autograd.gradcheck(net, (x,), eps=1e-6, atol=1e-5, raise_exception=True)


@pytest.mark.parametrize("ndim", [2, 3])
def test_final_layer_is_a_1x1_convolution(ndim):
    # tests/test_msd_module.py:44-84
    torch.manual_seed(0)
    size = (5, 6) if ndim == 2 else (3, 4, 5)
    fl = MSDFinalLayer(4, 3)
    fl.linear.weight.data.normal_()
    fl.linear.bias.data.normal_()
    conv = torch.nn.Conv2d(4, 3, 1) if ndim == 2 else torch.nn.Conv3d(4, 3, 1)
    conv.weight.data = fl.linear.weight.data.view_as(conv.weight)
    conv.bias.data = fl.linear.bias.data
    x = torch.randn(2, 4, *size)
    assert torch.allclose(fl(x), conv(x), atol=1e-6)


def test_single_layer_functions_return_the_output_buffer(oracle_ops):
    for fn, size in ((conv2d_relu, (6, 7)), (conv3d_relu, (4, 5, 6))):
        nd = len(size)
        x = torch.randn(1, 2, *size, dtype=torch.float64, requires_grad=True)
        w = torch.randn(3, 2, *([3] * nd), dtype=torch.float64, requires_grad=True)
        b = torch.randn(3, dtype=torch.float64, requires_grad=True)
        out = torch.empty(1, 3, *size, dtype=torch.float64)
        y = fn(x, w, b, out, 1, 2)
        assert y.data_ptr() == out.data_ptr()
        assert torch.autograd.gradcheck(lambda x_, w_, b_: fn(x_, w_, b_, torch.empty_like(out), 1, 2), (x, w, b),
                                        eps=1e-6, atol=1e-5)


# ------------------------------------------------------------ model helpers

def test_scaling_module_is_frozen_identity():
    sm = scaling_module(3)
    x = torch.randn(2, 3, 4, 5)
    assert torch.allclose(sm(x), x)
    assert not any(p.requires_grad for p in sm.parameters())
    assert isinstance(scaling_module(2, conv3d=True), torch.nn.Conv3d)


def test_moments():
    torch.manual_seed(0)
    pairs = [(torch.randn(4, 1, 8, 8) * 3 + 2, torch.randn(4, 2, 8, 8) * 0.5 - 1) for _ in range(5)]
    mean_in, std_in, mean_out, std_out = _moments(iter(pairs))     # a one-shot iterable is enough
    allx, ally = torch.cat([p[0] for p in pairs]), torch.cat([p[1] for p in pairs])
    assert abs(mean_in - allx.mean().item()) < 1e-5
    assert abs(std_in - allx.std(unbiased=False).item()) < 1e-4
    assert abs(mean_out - ally.mean().item()) < 1e-5
    assert abs(std_out - ally.std(unbiased=False).item()) < 1e-4
    with pytest.raises(ValueError):
        _moments([])


def test_match_module_prefix():
    from collections import OrderedDict
    from msd_pytorch_amd.msd_model import match_module_prefix
    plain = OrderedDict([("0.weight", 1), ("1.msd_block.weight0", 2), ("1.final_layer.linear.bias", 3)])
    wrapped = OrderedDict(("module." + k, v) for k, v in plain.items())
    assert match_module_prefix(plain, plain.keys()) is plain
    assert match_module_prefix(wrapped, wrapped.keys()) is wrapped
    stripped = match_module_prefix(wrapped, plain.keys())
    assert list(stripped.items()) == list(plain.items()) and isinstance(stripped, OrderedDict)
    assert list(match_module_prefix(plain, wrapped.keys()).items()) == list(wrapped.items())
    # a dictionary where only some keys carry the prefix is left alone (load_state_dict reports it)
    mixed = OrderedDict([("module.a", 1), ("b", 2)])
    assert match_module_prefix(mixed, plain.keys()) is mixed


def test_package_exports():
    for name in ("MSDRegressionModel", "MSDSegmentationModel", "MSDModule", "MSDBlock2d", "MSDBlock3d",
                 "ImageDataset", "ImageStack", "InputError"):
        assert hasattr(msd_pytorch_amd, name)
