"""MSD network module: dense block + final 1x1 layer (reference msd_module.py)."""
from math import sqrt

import torch

from . import msd_custom_convolutions as cc
from .msd_block import MSDBlock, block_stack_backward, block_stack_forward


def units_in_front(c_in, width, layer_depth):
    """Number of channels that hidden layer ``layer_depth`` (zero-based) reads:
    the network inputs plus the outputs of every earlier layer."""
    return c_in + width * layer_depth


def init_convolution_weights(conv_weight, c_in, c_out, width, depth):
    """Normal(0, sqrt(2 / n)) initialisation of Pelt & Sethian (PNAS 115(2), 2018),
    with n = taps * (c_in + width * (depth - 1)) + c_out, as msd_module.py:27-57."""
    taps = 1
    for s in conv_weight.shape[2:]:
        taps *= s
    n = taps * (c_in + width * (depth - 1)) + c_out
    conv_weight.normal_(0, sqrt(2 / n))


class MSDFinalFunction(torch.autograd.Function):
    """out = bias + weight . stack over the channel axis, one native pass over the
    stack forward and one backward (which produces the gradient of the whole stack)."""

    @staticmethod
    def forward(ctx, input, weight, bias):
        # the input is only needed for the weight and bias gradients: a frozen layer (the
        # models' scaling layers) does not keep the activation alive
        ctx.save_for_backward(input if any(ctx.needs_input_grad[1:]) else None, weight)
        ctx.input_shape = input.shape
        output = torch.empty(input.shape[0], weight.shape[0], *input.shape[2:], dtype=input.dtype,
                             device=input.device)
        cc.final_forward(input, weight, bias, output)
        return output

    @staticmethod
    def backward(ctx, grad_output):
        input, weight = ctx.saved_tensors
        if not cc.final_layer_supported(grad_output):
            grad_output = grad_output.contiguous()
        grad_input = torch.empty(ctx.input_shape, dtype=weight.dtype, device=weight.device) \
            if ctx.needs_input_grad[0] else None
        grad_weight = torch.empty_like(weight) if ctx.needs_input_grad[1] else None
        grad_bias = torch.empty(weight.shape[0], dtype=weight.dtype, device=weight.device) \
            if ctx.needs_input_grad[2] else None
        cc.final_backward(input, grad_output, weight, grad_input, grad_weight, grad_bias)
        return grad_input, grad_weight, grad_bias


class MSDNetFunction(torch.autograd.Function):
    """Dense block and final layer as ONE autograd node:
    ``(input, dilations, bias, final_weight, final_bias, *weights) -> output``.

    Same values as ``MSDFinalFunction(MSDBlockFunction(...))``.  The channel stack stays
    inside the node, so in backward the final layer writes the gradient of the whole stack
    straight into a fresh buffer that the block's reverse loop then owns: the stack-sized
    copy that MSDBlockFunction.backward has to take of its incoming gradient
    (msd_block.py:82-83) is not needed."""

    @staticmethod
    def forward(ctx, input, dilations, bias, final_weight, final_bias, *weights):
        stack = block_stack_forward(input, dilations, bias, weights)
        output = torch.empty(input.shape[0], final_weight.shape[0], *input.shape[2:], dtype=input.dtype,
                             device=input.device)
        cc.final_forward(stack, final_weight, final_bias, output)
        ctx.dilations = tuple(dilations)
        ctx.save_for_backward(bias, stack, final_weight, *weights)
        return output

    @staticmethod
    def backward(ctx, grad_output):
        bias, stack, final_weight, *weights = ctx.saved_tensors
        need_input, _, need_bias, need_fw, need_fb, *need_weights = ctx.needs_input_grad
        if not cc.final_layer_supported(grad_output):
            grad_output = grad_output.contiguous()
        block_needed = need_input or need_bias or any(need_weights)
        grads = torch.empty_like(stack) if block_needed else None
        grad_fw = torch.empty_like(final_weight) if need_fw else None
        grad_fb = torch.empty(final_weight.shape[0], dtype=final_weight.dtype, device=final_weight.device) \
            if need_fb else None
        cc.final_backward(stack, grad_output, final_weight, grads, grad_fw, grad_fb)
        grad_input, grad_bias, grad_weights = (None, None, [None] * len(weights))
        if block_needed:
            grad_input, grad_bias, grad_weights = block_stack_backward(
                stack, grads, ctx.dilations, bias, weights, need_input, need_bias, need_weights)
        return (grad_input, None, grad_bias, grad_fw, grad_fb, *grad_weights)


class MSDNetLossFunction(torch.autograd.Function):
    """Dense block, final layer, an optional frozen 1x1 output scaling and the loss as ONE
    autograd node:
    ``(input, dilations, bias, final_weight, final_bias, scale_weight, scale_bias, target, kind,
    *weights) -> (loss, output)``.

    ``kind`` is "mse", "l1" (output = scale(final(stack)), loss against ``target``) or "nll"
    (output = log_softmax(final(stack)), int64 labels).  The pass that computes the final layer
    also computes the loss, its gradient with respect to the layer's output and the layer's own
    parameter gradients, so the backward pass starts from a tensor of c_out channels and never
    reads the stack for the final layer again.  ``output`` is returned for the caller's use and
    is NOT differentiable (a loss of the caller's own built on it gets no gradient: run the
    modules one by one for that, ``MSDModel.fuse_loss = False``); the scaling layer's parameters
    get no gradient (they are frozen in
    the models, msd_model.py:8-45)."""

    @staticmethod
    def forward(ctx, input, dilations, bias, final_weight, final_bias, scale_weight, scale_bias, target, kind,
                *weights):
        stack = block_stack_forward(input, dilations, bias, weights)
        c_out = final_weight.shape[0]
        fw = final_weight.view(c_out, -1)
        if scale_weight is not None:
            sw = scale_weight.view(c_out, c_out)
            w_eff = (sw @ fw).contiguous()
            b_eff = sw @ final_bias + scale_bias
        else:
            sw, w_eff, b_eff = None, fw.contiguous(), final_bias
        need_fw, need_fb = ctx.needs_input_grad[3], ctx.needs_input_grad[4]
        g_w = torch.empty_like(w_eff) if need_fw or need_fb else None
        g_b = torch.empty_like(b_eff) if need_fw or need_fb else None
        output, loss, grad_out = cc.final_forward_loss(stack, w_eff, b_eff, kind, target, g_w, g_b)
        ctx.dilations = tuple(dilations)
        ctx.save_for_backward(bias, stack, w_eff, grad_out, g_w, g_b, sw, *weights)
        ctx.final_shape = final_weight.shape
        ctx.mark_non_differentiable(output)
        return loss, output

    @staticmethod
    def backward(ctx, grad_loss, _grad_output):
        bias, stack, w_eff, grad_out, g_w, g_b, sw, *weights = ctx.saved_tensors
        need_input, _, need_bias, need_fw, need_fb, *rest = ctx.needs_input_grad
        need_weights = rest[4:]
        grad_fw = grad_fb = None
        if need_fw or need_fb:
            # chain through the frozen scaling layer: W_eff = S W, b_eff = S b + t
            gw, gb = (sw.t() @ g_w, sw.t() @ g_b) if sw is not None else (g_w, g_b)
            grad_fw = (gw * grad_loss).view(ctx.final_shape) if need_fw else None
            grad_fb = gb * grad_loss if need_fb else None
        grad_input, grad_bias, grad_weights = (None, None, [None] * len(weights))
        if need_input or need_bias or any(need_weights):
            grads = torch.empty_like(stack)
            cc.final_backward(None, grad_out * grad_loss, w_eff, grads, None, None)
            grad_input, grad_bias, grad_weights = block_stack_backward(
                stack, grads, ctx.dilations, bias, weights, need_input, need_bias, need_weights)
        return (grad_input, None, grad_bias, grad_fw, grad_fb, None, None, None, None, *grad_weights)


class MSDFinalLayer(torch.nn.Module):
    """1x1 convolution over the whole channel stack, zero-initialised.

    The parameters live in ``linear = Conv1d(c_in, c_out, 1)``, which keeps the
    state-dict keys of msd_module.py:60-88.  On the GPU the layer runs as one native
    pass over the stack; elsewhere (CPU tensors, other dtypes) torch's Conv1d on the
    (B, C, voxels) view computes it."""

    def __init__(self, c_in, c_out):
        super().__init__()
        self.c_in = c_in
        self.c_out = c_out
        self.linear = torch.nn.Conv1d(c_in, c_out, 1)
        self.reset_parameters()

    def forward(self, input):
        if cc.final_layer_supported(input) and input.dtype == self.linear.weight.dtype:
            return MSDFinalFunction.apply(input, self.linear.weight, self.linear.bias)
        b, c, *size = input.shape
        flat = input.view(b, c, -1)
        return self.linear(flat).view(b, self.c_out, *size)

    def reset_parameters(self):
        self.linear.weight.data.zero_()
        self.linear.bias.data.zero_()


class MSDModule(torch.nn.Module):
    def __init__(self, c_in, c_out, depth, width, dilations=[1, 2, 3, 4, 5, 6, 7, 8, 9, 10], ndim=2):
        """Mixed-scale dense network.

        c_in, c_out : input / output channels
        depth       : number of hidden layers
        width       : channels per hidden layer
        dilations   : list of dilations, repeated cyclically over the layers
                      (default 1..10; [1, 2, 4, 8] is a common alternative)
        ndim        : 2 or 3
        """
        super().__init__()
        if depth < 1:
            raise ValueError(f"Depth must be at least 1. Got: {depth}.")
        if width < 1:
            raise ValueError(f"Width must be at least 1. Got: {width}.")
        self.c_in = c_in
        self.c_out = c_out
        self.depth = depth
        self.width = width
        self.dilations = [dilations[i % len(dilations)] for i in range(depth)]

        self.msd_block = MSDBlock(c_in, self.dilations, width, ndim=ndim)
        self.final_layer = MSDFinalLayer(c_in=c_in + width * depth, c_out=c_out)
        self.reset_parameters()

    def reset_parameters(self):
        for w in self.msd_block.weights:
            init_convolution_weights(w.data, self.c_in, self.c_out, self.width, self.depth)
        self.msd_block.bias.data.zero_()
        self.final_layer.reset_parameters()

    def _hooked(self):
        """True when a hook sits on the block, the final layer or its Conv1d: hooks see
        the modules' own calls, so the modules are then called one by one."""
        for m in (self.msd_block, self.final_layer, self.final_layer.linear):
            if m._forward_hooks or m._forward_pre_hooks or m._backward_hooks or m._backward_pre_hooks:
                return True
        return False

    def forward(self, input):
        linear = self.final_layer.linear
        if cc.final_layer_supported(input) and input.dim() in (4, 5) and input.dtype == linear.weight.dtype \
                and linear.bias is not None and not self._hooked():
            # block + final layer as one autograd node (no copy of the stack's gradient)
            block = self.msd_block
            weights = (getattr(block, f"weight{i}") for i in range(len(block.weights)))
            return MSDNetFunction.apply(input, block.dilations, block.bias, linear.weight, linear.bias, *weights)
        return self.final_layer(self.msd_block(input))

    def forward_loss(self, input, target, kind, scale=None):
        """(loss, output) of the network followed by an optional frozen 1x1 ``scale`` layer and
        the loss ``kind`` ("mse", "l1", "nll"), as one autograd node (MSDNetLossFunction), or
        None where that node does not apply (the caller then runs the modules one by one):
        CPU tensors, more than 8 output channels, hooks on the sub-modules, a scaling layer
        that is being trained."""
        linear = self.final_layer.linear
        if not (cc.final_layer_supported(input) and input.dim() in (4, 5) and input.dtype == linear.weight.dtype
                and linear.bias is not None and not self._hooked() and self.c_out <= 8
                and target.device == input.device):
            return None
        sw = sb = None
        if scale is not None:
            if scale.weight.requires_grad or scale.bias is None or scale.bias.requires_grad \
                    or scale.weight.dtype != input.dtype or scale._forward_hooks or scale._forward_pre_hooks:
                return None
            sw, sb = scale.weight, scale.bias
        if kind == "nll":
            if target.dtype != torch.int64 or tuple(target.shape) != (input.shape[0], *input.shape[2:]):
                return None
            target = target.contiguous()
        else:
            if target.dtype != input.dtype or tuple(target.shape) != (input.shape[0], self.c_out, *input.shape[2:]) \
                    or not cc.final_layer_supported(target):
                return None
        block = self.msd_block
        weights = (getattr(block, f"weight{i}") for i in range(len(block.weights)))
        return MSDNetLossFunction.apply(input, block.dilations, block.bias, linear.weight, linear.bias, sw, sb,
                                        target, kind, *weights)
