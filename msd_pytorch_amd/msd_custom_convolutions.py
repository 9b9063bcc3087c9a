"""The eight operators of the reference's native module, on MI355X.

Drop-in for the pybind11 module ``msd_custom_convolutions`` of the reference
(msd_custom_convolutions.cpp:343-369): same function names, same positional
arguments, same in-place semantics, ``RuntimeError`` on every invalid call.
The tensors' device pointers, sizes and strides are handed to the C ABI of
``libmsd_hip.so`` on torch's current stream; no tensor is copied or retained.

``block_size`` is accepted for compatibility and ignored: the launch shapes are
chosen by the library for gfx950.
"""
import ctypes
import operator

import torch

from . import _native

_DTYPES = {torch.float32: _native.MSD_F32, torch.float64: _native.MSD_F64}


def _fail(fn, msg):
    raise RuntimeError(f"{fn}: {msg}")


def _check_same_gpu(fn, named):
    """torch::checkAllSameGPU (msd_custom_convolutions.cpp:98)."""
    first = named[0][1]
    for name, t in named:
        if not isinstance(t, torch.Tensor):
            raise TypeError(f"{fn}: argument '{name}' must be a torch.Tensor")
        if not t.is_cuda:
            _fail(fn, f"Expected tensor for argument '{name}' to be on a GPU, but it is on {t.device}")
        if t.device != first.device:
            _fail(fn, f"Expected all tensors on the same GPU, but '{name}' is on {t.device} "
                      f"and '{named[0][0]}' is on {first.device}")


def _check_same_type(fn, named):
    """torch::checkAllSameType (msd_custom_convolutions.cpp:99)."""
    first = named[0][1]
    for name, t in named:
        if t.dtype != first.dtype:
            _fail(fn, f"Expected '{name}' to have the same type as '{named[0][0]}' "
                      f"({first.dtype}), but it has {t.dtype}")
    if first.dtype not in _DTYPES:
        _fail(fn, f"only float32 and float64 are supported, got {first.dtype}")


def _check_in_out_shape(fn, a, b):
    """checkInOutShape (msd_custom_convolutions.cpp:68-83)."""
    if a.dim() != b.dim():
        _fail(fn, f"tensors must have the same number of dimensions, got {a.dim()} and {b.dim()}")
    if a.dim() not in (4, 5):
        _fail(fn, f"expected a 4- or 5-dimensional tensor, got {a.dim()} dimensions")
    if a.shape[0] != b.shape[0]:
        _fail(fn, "Input batch dimension does not match output batch dimension. ")
    if tuple(a.shape[2:]) != tuple(b.shape[2:]):
        _fail(fn, "Input shape does not match output shape. ")


def _check_kernel(fn, kernel):
    """checkKernel3x3 + checkContiguous (msd_custom_convolutions.cpp:25-37,100)."""
    if kernel.dim() not in (4, 5):
        _fail(fn, "Expected 4 or 5 dimensional kernel.")
    if any(s != 3 for s in kernel.shape[2:]):
        _fail(fn, "Kernel shape must be 3x3" if kernel.dim() == 4 else "Kernel shape must be 3x3x3")
    if not kernel.is_contiguous():
        _fail(fn, "Expected kernel to be contiguous")


def _check_dim(fn, name, t, dim):
    if t.dim() != dim:
        _fail(fn, f"Expected {dim}-dimensional tensor for '{name}', but got {t.dim()} dimensions")


def _check_dilation(fn, t, dilation):
    """checkDilation (msd_custom_convolutions.cpp:39-52).  Returns the dilation as a Python
    int: like the reference's pybind11 int caster, any integer type is accepted (numpy and
    torch integer scalars), bool and float are not."""
    if isinstance(dilation, (bool, float)):
        raise TypeError(f"{fn}: dilation must be an int")
    try:
        dilation = operator.index(dilation)
    except TypeError:
        raise TypeError(f"{fn}: dilation must be an int") from None
    if dilation <= 0:
        _fail(fn, "Dilation must be 1 or greater")
    if any(dilation > s for s in t.shape[2:]):
        _fail(fn, "Dilation cannot be greater than size of image. ")
    return dilation


def _check_block_size(fn, block_size):
    if block_size is None:
        return
    if len(tuple(block_size)) != 3:
        raise TypeError(f"{fn}: block_size must be a tuple of three ints (z, y, x)")


def _head(data, c_in, c_out, dilation):
    """dtype, ndim, batch, c_in, c_out, spatial, dilation."""
    return (_DTYPES[data.dtype], data.dim() - 2, data.shape[0], c_in, c_out,
            _native.i64_array(tuple(data.shape[2:])), dilation)


def _view(t):
    return ctypes.c_void_p(t.data_ptr()), _native.i64_array(t.stride())


def _stream(t):
    return ctypes.c_void_p(torch.cuda.current_stream(t.device).cuda_stream)


def _workspace(data, c_in, c_out):
    lib = _native.load()
    need = lib.msd_workspace_bytes(_DTYPES[data.dtype], data.dim() - 2, data.shape[0], c_in, c_out,
                                   _native.i64_array(tuple(data.shape[2:])))
    if need < 0:
        _fail("workspace", _native.last_error())
    ws = torch.empty(max(int(need), 8), dtype=torch.uint8, device=data.device)
    return ws, ctypes.c_void_p(ws.data_ptr()), int(need)


def _call(fn_name, device, *args):
    lib = _native.load()
    with torch.cuda.device(device):
        rc = getattr(lib, fn_name)(*args)
    if rc != _native.MSD_OK:
        raise RuntimeError(_native.last_error())


def _forward(fn, native, input, kernel, bias, output, dilation, block_size):
    _check_same_gpu(fn, [("input", input), ("kernel", kernel), ("bias", bias), ("output", output)])
    _check_same_type(fn, [("input", input), ("kernel", kernel), ("bias", bias), ("output", output)])
    _check_kernel(fn, kernel)
    _check_in_out_shape(fn, input, output)
    for name, t in (("input", input), ("kernel", kernel), ("output", output)):
        _check_dim(fn, name, t, kernel.dim())
    _check_dim(fn, "bias", bias, 1)
    if kernel.shape[1] != input.shape[1]:
        _fail(fn, "Kernel shape does not match input channels. ")
    if kernel.shape[0] != output.shape[1]:
        _fail(fn, "Kernel shape does not match output channels. ")
    if bias.shape[0] != output.shape[1]:
        _fail(fn, "Bias shape does not match output channels. ")
    dilation = _check_dilation(fn, input, dilation)
    _check_block_size(fn, block_size)
    bias = bias.contiguous()
    _call(native, input.device, *_head(input, input.shape[1], output.shape[1], dilation), *_view(input),
          ctypes.c_void_p(kernel.data_ptr()), ctypes.c_void_p(bias.data_ptr()), *_view(output), _stream(input))


def conv_forward(input, kernel, bias, output, dilation, block_size=None):
    """output = bias + conv(input) (msd_custom_convolutions.cpp:85-117)."""
    _forward("conv_forward", "msd_conv_forward", input, kernel, bias, output, dilation, block_size)


def conv_relu_forward(input, kernel, bias, output, dilation, block_size=None):
    """output = max(0, bias + conv(input)) (msd_custom_convolutions.cpp:213-245)."""
    _forward("conv_relu_forward", "msd_conv_relu_forward", input, kernel, bias, output, dilation, block_size)


def _backward_x(fn, native, output, grad_output, kernel, grad_input, dilation, block_size):
    relu = output is not None
    named = [("grad_input", grad_input), ("kernel", kernel)]
    if relu:
        named.append(("output", output))
    named.append(("grad_output", grad_output))
    _check_same_gpu(fn, named)
    _check_same_type(fn, named)
    _check_kernel(fn, kernel)
    _check_in_out_shape(fn, grad_input, grad_output)
    if relu:
        _check_in_out_shape(fn, grad_input, output)
    for name, t in named:
        _check_dim(fn, name, t, kernel.dim())
    if kernel.shape[1] != grad_input.shape[1]:
        _fail(fn, "Kernel shape does not match input channels. ")
    if kernel.shape[0] != grad_output.shape[1] or (relu and kernel.shape[0] != output.shape[1]):
        _fail(fn, "Kernel shape does not match output channels. ")
    dilation = _check_dilation(fn, grad_input, dilation)
    _check_block_size(fn, block_size)
    head = _head(grad_input, grad_input.shape[1], grad_output.shape[1], dilation)
    views = (*_view(output),) if relu else ()
    _call(native, grad_input.device, *head, *views, *_view(grad_output), ctypes.c_void_p(kernel.data_ptr()),
          *_view(grad_input), _stream(grad_input))


def conv_backward_x(grad_output, kernel, grad_input, dilation, block_size=None):
    """grad_input += conv^T(grad_output) (msd_custom_convolutions.cpp:119-148)."""
    _backward_x("conv_backward_x", "msd_conv_backward_x", None, grad_output, kernel, grad_input, dilation,
                block_size)


def conv_relu_backward_x(output, grad_output, kernel, grad_input, dilation, block_size=None):
    """grad_input += conv^T(grad_output * [output > 0]) (msd_custom_convolutions.cpp:247-281)."""
    _backward_x("conv_relu_backward_x", "msd_conv_relu_backward_x", output, grad_output, kernel, grad_input,
                dilation, block_size)


def _backward_k(fn, native, output, grad_output, input, grad_kernel, grad_bias, dilation, block_size):
    relu = output is not None
    named = [("input", input), ("grad_kernel", grad_kernel)]
    if relu:
        named.append(("output", output))
    named.append(("grad_output", grad_output))
    if grad_bias is not None:
        named.append(("grad_bias", grad_bias))
    _check_same_gpu(fn, named)
    _check_same_type(fn, named)
    _check_kernel(fn, grad_kernel)
    _check_in_out_shape(fn, input, grad_output)
    if relu:
        _check_in_out_shape(fn, input, output)
    for name, t in named:
        if name != "grad_bias":
            _check_dim(fn, name, t, grad_kernel.dim())
    if grad_kernel.shape[1] != input.shape[1]:
        _fail(fn, "Kernel shape does not match input channels. ")
    if grad_kernel.shape[0] != grad_output.shape[1] or (relu and grad_kernel.shape[0] != output.shape[1]):
        _fail(fn, "Kernel shape does not match output channels. ")
    if grad_bias is not None:
        _check_dim(fn, "grad_bias", grad_bias, 1)
        if grad_bias.shape[0] != grad_output.shape[1]:
            _fail(fn, "Bias shape does not match output channels. ")
        if not grad_bias.is_contiguous():
            _fail(fn, "Expected grad_bias to be contiguous")
    dilation = _check_dilation(fn, input, dilation)
    _check_block_size(fn, block_size)
    c_in, c_out = input.shape[1], grad_output.shape[1]
    head = _head(input, c_in, c_out, dilation)
    views = (*_view(output),) if relu else ()
    grads = (ctypes.c_void_p(grad_kernel.data_ptr()),)
    if native in ("msd_conv_relu_backward_kb", "msd_conv_backward_kb", "msd_conv_relu_backward_kb_static"):
        grads += (ctypes.c_void_p(grad_bias.data_ptr() if grad_bias is not None else 0),)
    if native == "msd_conv_relu_backward_kb_static":
        # the library's own scratch buffer: nothing is allocated for this call
        _call(native, input.device, *head, *views, *_view(grad_output), *_view(input), *grads, _stream(input))
        return
    ws, ws_ptr, ws_bytes = _workspace(input, c_in, c_out)
    _call(native, input.device, *head, *views, *_view(grad_output), *_view(input), *grads, ws_ptr, ws_bytes,
          _stream(input))


def conv_backward_k(grad_output, input, grad_kernel, dilation, block_size=None):
    """grad_kernel += d/dkernel (msd_custom_convolutions.cpp:150-178)."""
    _backward_k("conv_backward_k", "msd_conv_backward_k", None, grad_output, input, grad_kernel, None, dilation,
                block_size)


def conv_relu_backward_k(output, grad_output, input, grad_kernel, dilation, block_size=None):
    """grad_kernel += d/dkernel with the ReLU mask (msd_custom_convolutions.cpp:283-316)."""
    _backward_k("conv_relu_backward_k", "msd_conv_relu_backward_k", output, grad_output, input, grad_kernel, None,
                dilation, block_size)


def conv_relu_backward_kb(output, grad_output, input, grad_kernel, grad_bias, dilation, block_size=None):
    """conv_relu_backward_k and conv_relu_backward_bias in one pass (the pair of
    calls msd_block.py:113-126 makes per layer).  Not part of the reference's module."""
    _backward_k("conv_relu_backward_kb", "msd_conv_relu_backward_kb", output, grad_output, input, grad_kernel,
                grad_bias, dilation, block_size)


def conv_relu_backward_kb_static(output, grad_output, input, grad_kernel, grad_bias, dilation, block_size=None):
    """conv_relu_backward_kb for callers that cannot allocate device memory (HIP graph
    capture, serving loops): the partial sums go through a 32 MiB buffer inside the library
    instead of a workspace tensor.  Raises RuntimeError for problems that need more; calls
    that overlap on one GPU race.  Not part of the reference's module."""
    _backward_k("conv_relu_backward_kb_static", "msd_conv_relu_backward_kb_static", output, grad_output, input,
                grad_kernel, grad_bias, dilation, block_size)


def conv_backward_kb(grad_output, input, grad_kernel, grad_bias, dilation, block_size=None):
    """conv_backward_k and conv_backward_bias in one pass.  Not part of the reference's module."""
    _backward_k("conv_backward_kb", "msd_conv_backward_kb", None, grad_output, input, grad_kernel, grad_bias,
                dilation, block_size)


def conv_backward_xkb(grad_output, input, kernel, grad_input, grad_kernel, grad_bias, dilation, block_size=None):
    """conv_backward_x, conv_backward_k and conv_backward_bias of one layer in one call
    (one pass over the input channels where the fused kernel applies): grad_input,
    grad_kernel and grad_bias (or None) are accumulated into.  Not part of the reference's
    module."""
    fn = "conv_backward_xkb"
    named = [("grad_output", grad_output), ("input", input), ("kernel", kernel), ("grad_input", grad_input),
             ("grad_kernel", grad_kernel)] + ([("grad_bias", grad_bias)] if grad_bias is not None else [])
    _check_same_gpu(fn, named)
    _check_same_type(fn, named)
    _check_kernel(fn, kernel)
    _check_kernel(fn, grad_kernel)
    if tuple(kernel.shape) != tuple(grad_kernel.shape):
        _fail(fn, "Expected grad_kernel to be shaped like kernel")
    _check_in_out_shape(fn, input, grad_output)
    if tuple(grad_input.shape) != tuple(input.shape):
        _fail(fn, "Input shape does not match output shape. ")
    for name, t in named[:5]:
        _check_dim(fn, name, t, kernel.dim())
    if kernel.shape[1] != input.shape[1]:
        _fail(fn, "Kernel shape does not match input channels. ")
    if kernel.shape[0] != grad_output.shape[1]:
        _fail(fn, "Kernel shape does not match output channels. ")
    if grad_bias is not None and (grad_bias.dim() != 1 or grad_bias.shape[0] != grad_output.shape[1]
                                  or not grad_bias.is_contiguous()):
        _fail(fn, "Bias shape does not match output channels. ")
    dilation = _check_dilation(fn, input, dilation)
    _check_block_size(fn, block_size)
    c_in, c_out = input.shape[1], grad_output.shape[1]
    ws, ws_ptr, ws_bytes = _workspace(input, c_in, c_out)
    _call("msd_conv_backward_xkb", input.device, *_head(input, c_in, c_out, dilation), *_view(grad_output),
          *_view(input), ctypes.c_void_p(kernel.data_ptr()), *_view(grad_input),
          ctypes.c_void_p(grad_kernel.data_ptr()),
          ctypes.c_void_p(grad_bias.data_ptr() if grad_bias is not None else 0), ws_ptr, ws_bytes, _stream(input))


def relu_mask_gradient(output, grad_output):
    """grad_output *= (output > 0), in place: the mask the three conv_relu_backward_*
    operators of a layer apply on the fly, applied once (for callers that own
    grad_output, like the dense block's private gradient stack).  Not part of the
    reference's module."""
    fn = "relu_mask_gradient"
    _check_same_gpu(fn, [("output", output), ("grad_output", grad_output)])
    _check_same_type(fn, [("output", output), ("grad_output", grad_output)])
    if tuple(output.shape) != tuple(grad_output.shape) or output.dim() not in (4, 5):
        _fail(fn, "output and grad_output must be 4- or 5-dimensional tensors of the same shape")
    _call("msd_relu_mask_gradient", output.device, _DTYPES[output.dtype], output.dim() - 2, output.shape[0],
          output.shape[1], _native.i64_array(tuple(output.shape[2:])), *_view(output), *_view(grad_output),
          _stream(output))


def _backward_bias(fn, native, output, grad_output, grad_bias, block_size):
    relu = output is not None
    named = [("grad_bias", grad_bias)]
    if relu:
        named.append(("output", output))
    named.append(("grad_output", grad_output))
    _check_same_gpu(fn, named)
    _check_same_type(fn, named)
    if relu:
        _check_in_out_shape(fn, output, grad_output)
    elif grad_output.dim() not in (4, 5):
        _fail(fn, f"expected a 4- or 5-dimensional tensor, got {grad_output.dim()} dimensions")
    _check_dim(fn, "grad_bias", grad_bias, 1)
    if grad_bias.shape[0] != grad_output.shape[1]:
        _fail(fn, "Bias shape does not match output channels. ")
    if not grad_bias.is_contiguous():
        _fail(fn, "Expected grad_bias to be contiguous")
    _check_block_size(fn, block_size)
    c_out = grad_output.shape[1]
    ws, ws_ptr, ws_bytes = _workspace(grad_output, 0, c_out)
    head = (_DTYPES[grad_output.dtype], grad_output.dim() - 2, grad_output.shape[0], c_out,
            _native.i64_array(tuple(grad_output.shape[2:])))
    views = (*_view(output),) if relu else ()
    _call(native, grad_output.device, *head, *views, *_view(grad_output), ctypes.c_void_p(grad_bias.data_ptr()),
          ws_ptr, ws_bytes, _stream(grad_output))


def conv_backward_bias(grad_output, grad_bias, block_size=None):
    """grad_bias += grad_output summed over batch and voxels (msd_custom_convolutions.cpp:180-211)."""
    _backward_bias("conv_backward_bias", "msd_conv_backward_bias", None, grad_output, grad_bias, block_size)


def conv_relu_backward_bias(output, grad_output, grad_bias, block_size=None):
    """grad_bias += grad_output summed where output > 0 (msd_custom_convolutions.cpp:318-338)."""
    _backward_bias("conv_relu_backward_bias", "msd_conv_relu_backward_bias", output, grad_output, grad_bias,
                   block_size)


# ---------------------------------------------------------------------------
# Dense block as one native call per direction (not part of the reference's
# module: there the loops of msd_block.py:40-58 and :89-130 run in Python).
# ---------------------------------------------------------------------------

def _check_block(fn, stack, c_in, dilations, bias, weights):
    named = [("stack", stack), ("bias", bias)] + [(f"weight{i}", w) for i, w in enumerate(weights)]
    _check_same_gpu(fn, named)
    _check_same_type(fn, named)
    if stack.dim() not in (4, 5):
        _fail(fn, f"expected a 4- or 5-dimensional stack, got {stack.dim()} dimensions")
    if len(dilations) != len(weights):
        _fail(fn, "number of weights does not match depth")
    channels = c_in
    checked = []
    for i, (w, d) in enumerate(zip(weights, dilations)):
        _check_kernel(fn, w)
        _check_dim(fn, f"weight{i}", w, stack.dim())
        if w.shape[1] != channels:
            _fail(fn, "Kernel shape does not match input channels. ")
        checked.append(_check_dilation(fn, stack, d))
        channels += w.shape[0]
    if channels != stack.shape[1]:
        _fail(fn, "Kernel shape does not match output channels. ")
    _check_dim(fn, "bias", bias, 1)
    if bias.shape[0] != channels - c_in:
        _fail(fn, "Bias shape does not match output channels. ")
    return checked


def _block_head(stack, c_in, dilations, weights):
    widths = _native.i64_array([w.shape[0] for w in weights])
    return (_DTYPES[stack.dtype], stack.dim() - 2, stack.shape[0], c_in, len(weights), widths,
            _native.i64_array(tuple(stack.shape[2:])), _native.i64_array(list(dilations)))


def _ptr_array(tensors):
    return (ctypes.c_void_p * len(tensors))(*[t.data_ptr() if t is not None else None for t in tensors])


def block_forward(stack, c_in, dilations, bias, weights):
    """Fill channels [c_in, end) of ``stack`` layer by layer; channels [0, c_in)
    hold the block's input.  Layer i: conv_relu_forward(stack[:, :C_i], weights[i],
    bias slice, stack[:, C_i:C_i + width_i], dilations[i])."""
    fn = "block_forward"
    dilations = _check_block(fn, stack, c_in, dilations, bias, weights)
    bias = bias.contiguous()
    _call("msd_block_forward", stack.device, *_block_head(stack, c_in, dilations, weights), *_view(stack),
          _ptr_array(weights), ctypes.c_void_p(bias.data_ptr()), _stream(stack))


def block_backward(stack, grads, c_in, dilations, weights, grad_weights, grad_bias, need_input_grad):
    """Backward of the whole block.  ``grads`` holds dL/dstack and is overwritten
    (it is the caller's private working copy); afterwards grads[:, :c_in] is
    dL/dinput.  ``grad_weights[i]`` (zero-filled, or None to skip) and ``grad_bias``
    (zero-filled, or None) are accumulated into."""
    fn = "block_backward"
    dilations = _check_block(fn, stack, c_in, dilations,
                             torch.empty(stack.shape[1] - c_in, dtype=stack.dtype, device=stack.device)
                             if grad_bias is None else grad_bias, weights)
    named = [("stack", stack), ("grads", grads)] + [(f"grad_weight{i}", g) for i, g in enumerate(grad_weights)
                                                    if g is not None]
    _check_same_gpu(fn, named)
    _check_same_type(fn, named)
    if tuple(grads.shape) != tuple(stack.shape):
        _fail(fn, "Input shape does not match output shape. ")
    for g, w in zip(grad_weights, weights):
        if g is not None and (tuple(g.shape) != tuple(w.shape) or not g.is_contiguous()):
            _fail(fn, "grad_weights must be contiguous and shaped like the weights")
    if grad_bias is not None and not grad_bias.is_contiguous():
        _fail(fn, "Expected grad_bias to be contiguous")
    head = _block_head(stack, c_in, dilations, weights)
    lib = _native.load()
    need = lib.msd_block_workspace_bytes(head[0], head[1], head[2], c_in, head[4], head[5], head[6])
    if need < 0:
        _fail(fn, "invalid block geometry")
    ws = torch.empty(max(int(need), 8), dtype=torch.uint8, device=stack.device)
    _call("msd_block_backward", stack.device, *head, *_view(stack), *_view(grads), _ptr_array(weights),
          _ptr_array(grad_weights), ctypes.c_void_p(grad_bias.data_ptr() if grad_bias is not None else 0),
          1 if need_input_grad else 0, ctypes.c_void_p(ws.data_ptr()), int(need), _stream(stack))


# ---------------------------------------------------------------------------
# Final 1x1 layer over the channel stack (msd_module.py:60-88 of the reference,
# which leaves it to torch's Conv1d).
# ---------------------------------------------------------------------------

def final_layer_supported(input):
    """True when the native final layer can take ``input`` (B, C, *spatial) as it
    is: on the GPU, float32/float64, every channel plane contiguous."""
    if not input.is_cuda or input.dtype not in _DTYPES or input.dim() < 3:
        return False
    plane = input[0, 0]
    return plane.is_contiguous() and input.numel() > 0


def _flat_strides(t):
    """(voxels per channel, batch stride, channel stride) of (B, C, *spatial)."""
    nvox = 1
    for s in t.shape[2:]:
        nvox *= s
    return nvox, t.stride(0), t.stride(1)


def final_forward(input, weight, bias, output):
    """output[b, o] = bias[o] + sum_c weight[o, c] * input[b, c]; weight is
    (c_out, c_in) or Conv1d's (c_out, c_in, 1)."""
    fn = "final_forward"
    named = [("input", input), ("weight", weight), ("output", output)] + ([("bias", bias)] if bias is not None else [])
    _check_same_gpu(fn, named)
    _check_same_type(fn, named)
    c_out, c_in = weight.shape[0], weight.shape[1]
    if weight.numel() != c_out * c_in or not weight.is_contiguous():
        _fail(fn, "Expected weight to be contiguous and shaped (c_out, c_in[, 1])")
    if input.shape[1] != c_in or output.shape[1] != c_out or tuple(input.shape[2:]) != tuple(output.shape[2:]) \
            or input.shape[0] != output.shape[0]:
        _fail(fn, "Input shape does not match output shape. ")
    if not (final_layer_supported(input) and final_layer_supported(output)):
        _fail(fn, "Expected channel planes to be contiguous")
    nvox, isb, isc = _flat_strides(input)
    _, osb, osc = _flat_strides(output)
    _call("msd_final_forward", input.device, _DTYPES[input.dtype], input.shape[0], c_in, c_out, nvox,
          ctypes.c_void_p(input.data_ptr()), isb, isc, ctypes.c_void_p(weight.data_ptr()),
          ctypes.c_void_p(bias.data_ptr() if bias is not None else 0), ctypes.c_void_p(output.data_ptr()), osb, osc,
          _stream(input))


def final_backward(input, grad_output, weight, grad_input, grad_weight, grad_bias):
    """Gradients of final_forward; grad_input (or None), grad_weight (or None) and
    grad_bias (or None) are OVERWRITTEN.  ``input`` may be None when neither grad_weight nor
    grad_bias is wanted (a frozen layer): grad_input does not depend on it."""
    fn = "final_backward"
    if input is None and (grad_weight is not None or grad_bias is not None or grad_input is None):
        _fail(fn, "input may only be omitted when grad_input is the only gradient wanted")
    shaped = input if input is not None else grad_input
    named = [("grad_output", grad_output), ("weight", weight)]
    named += [(n, t) for n, t in (("input", input), ("grad_input", grad_input), ("grad_weight", grad_weight),
                                  ("grad_bias", grad_bias)) if t is not None]
    _check_same_gpu(fn, named)
    _check_same_type(fn, named)
    c_out, c_in = weight.shape[0], weight.shape[1]
    if weight.numel() != c_out * c_in or not weight.is_contiguous():
        _fail(fn, "Expected weight to be contiguous and shaped (c_out, c_in[, 1])")
    if grad_weight is not None and (grad_weight.numel() != c_out * c_in or not grad_weight.is_contiguous()):
        _fail(fn, "Expected grad_weight to be contiguous and shaped like weight")
    if grad_bias is not None and (grad_bias.numel() != c_out or not grad_bias.is_contiguous()):
        _fail(fn, "Expected grad_bias to be contiguous with c_out elements")
    if shaped.shape[1] != c_in or grad_output.shape[1] != c_out or shaped.shape[0] != grad_output.shape[0] \
            or tuple(shaped.shape[2:]) != tuple(grad_output.shape[2:]):
        _fail(fn, "Input shape does not match output shape. ")
    if grad_input is not None and tuple(grad_input.shape) != tuple(shaped.shape):
        _fail(fn, "Input shape does not match output shape. ")
    for t in (input, grad_output, grad_input):
        if t is not None and not final_layer_supported(t):
            _fail(fn, "Expected channel planes to be contiguous")
    nvox, isb, isc = _flat_strides(shaped)
    _, gsb, gsc = _flat_strides(grad_output)
    xsb, xsc = (grad_input.stride(0), grad_input.stride(1)) if grad_input is not None else (0, 0)
    need, ws = 0, None
    if grad_weight is not None or grad_bias is not None:
        # partial sums of the weight and bias gradients (fixed-order reduction)
        need = _native.load().msd_final_workspace_bytes(_DTYPES[shaped.dtype], shaped.shape[0], c_in, c_out, nvox)
        if need < 0:
            _fail(fn, _native.last_error())
        ws = torch.empty(max(int(need), 8), dtype=torch.uint8, device=shaped.device)

    def ptr(t):
        return ctypes.c_void_p(t.data_ptr() if t is not None else 0)

    input = shaped      # only its geometry is used when the caller passed None
    _call("msd_final_backward", input.device, _DTYPES[input.dtype], input.shape[0], c_in, c_out, nvox, ptr(input), isb,
          isc, ptr(grad_output), gsb, gsc, ptr(weight), ptr(grad_input), xsb, xsc, ptr(grad_weight), ptr(grad_bias),
          ptr(ws), int(need), _stream(input))


LOSS_KINDS = {"mse": _native.LOSS_MSE, "l1": _native.LOSS_L1, "nll": _native.LOSS_NLL}


def final_forward_loss(input, weight, bias, kind, target, grad_weight=None, grad_bias=None):
    """Final layer, loss and the loss's gradient in one pass over ``input`` (B, C, *spatial):
    ``kind`` "mse" / "l1" (target shaped like the output) or "nll" (log-softmax over the output
    channels, int64 labels (B, *spatial)); 'mean' reduction; at most 8 output channels.
    Returns (output, loss, grad_output) with grad_output = d loss / d (bias + weight . input);
    ``grad_weight`` / ``grad_bias`` (or None) are overwritten with the layer's parameter
    gradients."""
    fn = "final_forward_loss"
    if kind not in LOSS_KINDS:
        raise ValueError(f"{fn}: kind must be one of {sorted(LOSS_KINDS)}")
    named = [("input", input), ("weight", weight), ("target", target)]
    named += [(n, t) for n, t in (("bias", bias), ("grad_weight", grad_weight), ("grad_bias", grad_bias))
              if t is not None]
    _check_same_gpu(fn, named)
    _check_same_type(fn, [(n, t) for n, t in named if n != "target" or kind != "nll"])
    c_out, c_in = weight.shape[0], weight.shape[1]
    if weight.numel() != c_out * c_in or not weight.is_contiguous():
        _fail(fn, "Expected weight to be contiguous and shaped (c_out, c_in[, 1])")
    if c_out > 8:
        _fail(fn, "at most 8 output channels")
    if input.shape[1] != c_in:
        _fail(fn, "Kernel shape does not match input channels. ")
    if not final_layer_supported(input):
        _fail(fn, "Expected channel planes to be contiguous")
    for name, t, n in (("bias", bias, c_out), ("grad_bias", grad_bias, c_out), ("grad_weight", grad_weight, c_out * c_in)):
        if t is not None and (t.numel() != n or not t.is_contiguous()):
            _fail(fn, f"Expected {name} to be contiguous with {n} elements")
    out_shape = (input.shape[0], c_out, *input.shape[2:])
    nvox, isb, isc = _flat_strides(input)
    if kind == "nll":
        if target.dtype != torch.int64 or tuple(target.shape) != (input.shape[0], *input.shape[2:]) \
                or not target.is_contiguous():
            _fail(fn, "Expected contiguous int64 labels shaped (B, *spatial)")
        tsb, tsc = nvox, 0
    else:
        if tuple(target.shape) != out_shape or not final_layer_supported(target):
            _fail(fn, "Expected a target shaped like the output with contiguous channel planes")
        _, tsb, tsc = _flat_strides(target)
    output = torch.empty(out_shape, dtype=input.dtype, device=input.device)
    grad_output = torch.empty_like(output)
    loss = torch.empty((), dtype=input.dtype, device=input.device)
    _, osb, osc = _flat_strides(output)
    lib = _native.load()
    need = lib.msd_final_workspace_bytes(_DTYPES[input.dtype], input.shape[0], c_in, c_out, nvox)
    if need < 0:
        _fail(fn, _native.last_error())
    ws = torch.empty(max(int(need), 8), dtype=torch.uint8, device=input.device)

    def ptr(t):
        return ctypes.c_void_p(t.data_ptr() if t is not None else 0)

    _call("msd_final_forward_loss", input.device, _DTYPES[input.dtype], LOSS_KINDS[kind], input.shape[0], c_in, c_out,
          nvox, ptr(input), isb, isc, ptr(weight), ptr(bias), ptr(target), tsb, tsc, ptr(output), osb, osc,
          ptr(grad_output), osb, osc, ptr(grad_weight), ptr(grad_bias), ptr(loss), ptr(ws), int(need), _stream(input))
    return output, loss, grad_output
