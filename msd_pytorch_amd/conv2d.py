"""2D dilated 3x3 convolution: operator wrappers and single-layer autograd
Functions/Modules under the names of the reference's conv2d.py (:8-145)."""
from ._conv_nd import make_function, make_module, make_ops

_BLOCK = (0, 16, 16)     # the reference's default for every 2D operator; ignored here
_ops = make_ops({name: _BLOCK for name in (
    "forward", "backward_x", "backward_k", "backward_bias",
    "relu_forward", "relu_backward_x", "relu_backward_k", "relu_backward_bias")})

conv2d_forward = _ops["forward"]
conv2d_backward_x = _ops["backward_x"]
conv2d_backward_k = _ops["backward_k"]
conv2d_backward_bias = _ops["backward_bias"]
conv2d_relu_forward = _ops["relu_forward"]
conv2d_relu_backward_x = _ops["relu_backward_x"]
conv2d_relu_backward_k = _ops["relu_backward_k"]
conv2d_relu_backward_bias = _ops["relu_backward_bias"]
conv2d_relu_backward_kb = _ops["relu_backward_kb"]   # weights + bias in one pass; not in the reference

Conv2dFunction = make_function(False, "Conv2dFunction")
Conv2dReluFunction = make_function(True, "Conv2dReluFunction")
conv2d = Conv2dFunction.apply
conv2d_relu = Conv2dReluFunction.apply
Conv2dModule = make_module(conv2d, 2, "Conv2dModule")
Conv2dReluModule = make_module(conv2d_relu, 2, "Conv2dReluModule")
