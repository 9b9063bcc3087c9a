"""Mixed-scale dense block: ``depth`` dilated conv+ReLU layers that all write
into ONE growing channel stack; layer ``i`` reads every channel in front of it.

API of the reference's msd_block.py: ``MSDBlockFunction(input, dilations, bias,
*weights)`` (:8-134), ``msd_block``, ``MSDBlock``/``MSDBlock2d``/``MSDBlock3d``
with parameters ``weight{i}`` of shape ``(width, c_in + width*i, 3, 3[, 3])``
and one flat ``bias`` of ``depth * width`` (:140-249), so checkpoints are
interchangeable.
"""
import math

import torch

from . import msd_custom_convolutions as cc


def block_stack_forward(input, dilations, bias, weights):
    """The channel stack of the dense block: the input followed by every layer's output
    (argument checks and layer loop of msd_block.py:8-58)."""
    if len(dilations) != len(weights):
        raise AssertionError("number of weights does not match depth")
    if input.dim() not in (4, 5):
        raise ValueError("Input to MSDBlock must be 2D or 3D")
    widths = [w.shape[0] for w in weights]
    if len(bias) != sum(widths):
        raise AssertionError("number of biases does not match number of output channels from weights")
    c_in = input.shape[1]
    stack = input.new_empty(input.shape[0], c_in + sum(widths), *input.shape[2:])
    stack[:, :c_in] = input
    # the layer loop of msd_block.py:40-58 runs inside the native library
    cc.block_forward(stack, c_in, list(dilations), bias, list(weights))
    return stack


def block_stack_backward(stack, grads, dilations, bias, weights, need_input, need_bias, need_weights):
    """The reverse layer loop of msd_block.py:89-130 on ``grads``, the gradient of the
    whole stack, which must be private to the caller: it is overwritten.  Returns
    (grad_input, grad_bias, grad_weights).

    Per layer the native library masks the layer's slice of ``grads`` once in place (the
    slice is not read again afterwards) and then applies the plain backward operators;
    the reference masks on the fly in each of conv_relu_backward_x / _k / _bias."""
    grad_bias = torch.zeros_like(bias) if need_bias else None
    grad_weights = [None] * len(weights)
    # one zero-filled buffer for all weight gradients (one fill instead of one per layer)
    wanted = [w for w, need in zip(weights, need_weights) if need]
    flat = stack.new_zeros(sum(w.numel() for w in wanted))
    offset = 0
    for idx, weight in enumerate(weights):
        if need_weights[idx]:
            grad_weights[idx] = flat[offset:offset + weight.numel()].view_as(weight)
            offset += weight.numel()
    c_in = weights[0].shape[1]
    cc.block_backward(stack, grads, c_in, list(dilations), list(weights), grad_weights,
                      grad_bias if need_bias else None, bool(need_input))
    return (grads[:, :c_in] if need_input else None), grad_bias, grad_weights


class MSDBlockFunction(torch.autograd.Function):
    @staticmethod
    def forward(ctx, input, dilations, bias, *weights):
        stack = block_stack_forward(input, dilations, bias, weights)
        ctx.dilations = tuple(dilations)
        ctx.save_for_backward(bias, stack, *weights)
        return stack

    @staticmethod
    def backward(ctx, grad_output):
        bias, stack, *weights = ctx.saved_tensors
        if grad_output.dim() != stack.dim():
            raise AssertionError("Mismatched tensor dimensions.")
        need_input, _, need_bias, *need_weights = ctx.needs_input_grad
        # Working copy of the incoming gradient (autograd may hand the same tensor to
        # others): layer idx adds its input gradient to channels [0, first), which later
        # iterations consume.
        grads = grad_output.clone()
        grad_input, grad_bias, grad_weights = block_stack_backward(
            stack, grads, ctx.dilations, bias, weights, need_input, need_bias, need_weights)
        return (grad_input, None, grad_bias, *grad_weights)


msd_block = MSDBlockFunction.apply


class MSDBlock(torch.nn.Module):
    def __init__(self, in_channels, dilations, width=1, ndim=2):
        """Mixed-scale dense block.

        in_channels : number of input channels
        dilations   : one dilation per layer (its length is the depth)
        width       : output channels per layer
        ndim        : 2 or 3

        The output has ``in_channels + len(dilations) * width`` channels: the
        input followed by every layer's output.
        """
        super().__init__()
        if ndim not in (2, 3):
            raise ValueError("ndim must be 2 or 3")
        self.kernel_size = (3,) * ndim
        self.width = width
        self.dilations = dilations

        depth = len(dilations)
        self.bias = torch.nn.Parameter(torch.empty(depth * width))
        self.weights = []
        for i in range(depth):
            weight = torch.nn.Parameter(torch.empty(width, in_channels + width * i, *self.kernel_size))
            self.register_parameter(f"weight{i}", weight)
            self.weights.append(weight)
        self.reset_parameters()

    def reset_parameters(self):
        # same draws, in the same order, as msd_block.py:183-191
        for weight in self.weights:
            torch.nn.init.kaiming_uniform_(weight, a=math.sqrt(5))
        fan_in, _ = torch.nn.init._calculate_fan_in_and_fan_out(self.weights[0])
        bound = 1 / math.sqrt(fan_in)
        torch.nn.init.uniform_(self.bias, -bound, bound)

    def forward(self, input):
        # Look the weights up by attribute on every call: after a device move,
        # a DataParallel replication or torch.nn.utils.prune the list made in
        # __init__ may hold stale tensors (msd_block.py:193-209).
        weights = (getattr(self, f"weight{i}") for i in range(len(self.weights)))
        return msd_block(input, self.dilations, self.bias, *weights)


class MSDBlock2d(MSDBlock):
    def __init__(self, in_channels, dilations, width=1):
        super().__init__(in_channels, dilations, width=width, ndim=2)


class MSDBlock3d(MSDBlock):
    def __init__(self, in_channels, dilations, width=1):
        super().__init__(in_channels, dilations, width=width, ndim=3)
