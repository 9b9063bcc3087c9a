"""3D dilated 3x3x3 convolution: operator wrappers and single-layer autograd
Functions/Modules under the names of the reference's conv3d.py (:8-149)."""
from ._conv_nd import make_function, make_module, make_ops

# the reference's tuned CUDA block shapes (z, y, x), conv3d.py:8-37; ignored here
_ops = make_ops({
    "forward": (8, 8, 8), "backward_x": (4, 4, 4), "backward_k": (8, 8, 8), "backward_bias": (8, 8, 8),
    "relu_forward": (2, 2, 32), "relu_backward_x": (2, 4, 16), "relu_backward_k": (2, 8, 16),
    "relu_backward_bias": (8, 8, 8)})

conv3d_forward = _ops["forward"]
conv3d_backward_x = _ops["backward_x"]
conv3d_backward_k = _ops["backward_k"]
conv3d_backward_bias = _ops["backward_bias"]
conv3d_relu_forward = _ops["relu_forward"]
conv3d_relu_backward_x = _ops["relu_backward_x"]
conv3d_relu_backward_k = _ops["relu_backward_k"]
conv3d_relu_backward_bias = _ops["relu_backward_bias"]
conv3d_relu_backward_kb = _ops["relu_backward_kb"]   # weights + bias in one pass; not in the reference

Conv3DFunction = make_function(False, "Conv3DFunction")
Conv3DReluFunction = make_function(True, "Conv3DReluFunction")
conv3d = Conv3DFunction.apply
conv3d_relu = Conv3DReluFunction.apply
Conv3DModule = make_module(conv3d, 3, "Conv3DModule")
Conv3DReluModule = make_module(conv3d_relu, 3, "Conv3DReluModule")
