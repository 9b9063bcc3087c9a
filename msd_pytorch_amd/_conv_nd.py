"""Single-layer autograd wrappers shared by conv2d.py and conv3d.py.

The reference spells these out twice (conv2d.py:40-145, conv3d.py:40-149); the
behaviour is the same in both ranks, so it is written once here:

* ``forward(ctx, input, weight, bias, output, stride, dilation)`` writes into
  the caller's ``output`` tensor and returns that same tensor; ``stride`` is a
  dummy kept for signature compatibility (conv2d.py:42);
* ``backward`` makes ``grad_output`` contiguous, allocates zeroed gradient
  buffers and lets the three backward operators accumulate into them
  (conv2d.py:100-123).
"""
import torch
from torch.autograd import Function
from torch.nn import Parameter

from . import msd_custom_convolutions as cc


def make_function(relu, name):
    if relu:
        class _Fn(Function):
            @staticmethod
            def forward(ctx, input, weight, bias, output, stride, dilation):
                ctx.dilation = dilation
                cc.conv_relu_forward(input, weight, bias, output.data, dilation)
                ctx.save_for_backward(input, output, weight, bias)
                return output

            @staticmethod
            def backward(ctx, grad_output):
                input, output, weight, bias = ctx.saved_tensors
                grad_output = grad_output.contiguous()
                grad_input = torch.zeros_like(input)
                cc.conv_relu_backward_x(output, grad_output, weight, grad_input, ctx.dilation)
                grad_weight = torch.zeros_like(weight)
                grad_bias = torch.zeros_like(bias)
                cc.conv_relu_backward_kb(output, grad_output, input, grad_weight, grad_bias, ctx.dilation)
                return grad_input, grad_weight, grad_bias, None, None, None, None
    else:
        class _Fn(Function):
            @staticmethod
            def forward(ctx, input, weight, bias, output, stride, dilation):
                ctx.dilation = dilation
                ctx.save_for_backward(input, weight, bias)
                cc.conv_forward(input, weight, bias, output.data, dilation)
                return output

            @staticmethod
            def backward(ctx, grad_output):
                input, weight, bias = ctx.saved_tensors
                grad_output = grad_output.contiguous()
                grad_input = torch.zeros_like(input)
                cc.conv_backward_x(grad_output, weight, grad_input, ctx.dilation)
                grad_weight = torch.zeros_like(weight)
                cc.conv_backward_k(grad_output, input, grad_weight, ctx.dilation)
                grad_bias = torch.zeros_like(bias)
                cc.conv_backward_bias(grad_output, grad_bias)
                return grad_input, grad_weight, grad_bias, None, None, None, None

    _Fn.__name__ = _Fn.__qualname__ = name
    return _Fn


def make_module(apply, ndim, name):
    class _Module(torch.nn.Module):
        """Layer with its own (uninitialised) weight and bias that writes into the
        caller-supplied ``output`` buffer (conv2d.py:73-89, conv3d.py:77-93)."""

        def __init__(self, output, in_channels, out_channels, kernel_size=3, dilation=1):
            super().__init__()
            device = output.device
            self.weight = Parameter(torch.empty(out_channels, in_channels, *([kernel_size] * ndim), device=device))
            self.bias = Parameter(torch.empty(out_channels, device=device))
            self.output = output
            self.dilation = dilation
            self.stride = 1

        def forward(self, input):
            assert self.output.is_cuda
            return apply(input, self.weight, self.bias, self.output, self.stride, self.dilation)

    _Module.__name__ = _Module.__qualname__ = name
    return _Module


def make_ops(defaults):
    """The eight per-rank operator wrappers.

    ``defaults`` maps an operator name to the default of its ``block_size``
    keyword (the reference's tuned CUDA block shapes, conv2d.py:8-37 and
    conv3d.py:8-37); the value is accepted and ignored by the native library.
    """
    def forward(input, weight, bias, output, dilation, block_size=defaults["forward"]):
        cc.conv_forward(input, weight, bias, output, dilation, block_size=tuple(block_size))

    def backward_x(grad_output, weight, grad_input, dilation, block_size=defaults["backward_x"]):
        cc.conv_backward_x(grad_output, weight, grad_input, dilation, block_size=tuple(block_size))

    def backward_k(grad_output, input, grad_weight, dilation, block_size=defaults["backward_k"]):
        cc.conv_backward_k(grad_output, input, grad_weight, dilation, block_size=tuple(block_size))

    def backward_bias(grad_output, grad_bias, block_size=defaults["backward_bias"]):
        cc.conv_backward_bias(grad_output, grad_bias, block_size=tuple(block_size))

    def relu_forward(input, weight, bias, output, dilation, block_size=defaults["relu_forward"]):
        cc.conv_relu_forward(input, weight, bias, output, dilation, block_size=tuple(block_size))

    def relu_backward_x(output, grad_output, weight, grad_input, dilation,
                        block_size=defaults["relu_backward_x"]):
        cc.conv_relu_backward_x(output, grad_output, weight, grad_input, dilation, block_size=tuple(block_size))

    def relu_backward_k(output, grad_output, input, grad_weight, dilation,
                        block_size=defaults["relu_backward_k"]):
        cc.conv_relu_backward_k(output, grad_output, input, grad_weight, dilation, block_size=tuple(block_size))

    def relu_backward_bias(output, grad_output, grad_bias, block_size=defaults["relu_backward_bias"]):
        cc.conv_relu_backward_bias(output, grad_output, grad_bias, block_size=tuple(block_size))

    def relu_backward_kb(output, grad_output, input, grad_weight, grad_bias, dilation, block_size=None):
        cc.conv_relu_backward_kb(output, grad_output, input, grad_weight, grad_bias, dilation)

    return {f.__name__: f for f in (forward, backward_x, backward_k, backward_bias, relu_forward,
                                    relu_backward_x, relu_backward_k, relu_backward_bias, relu_backward_kb)}
