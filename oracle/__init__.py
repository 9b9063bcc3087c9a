"""TEST INFRASTRUCTURE ONLY: CPU oracle for the dilated conv (+ReLU) path.

Loads ``libmsd_oracle.so`` (plain C, built by ``oracle/Makefile``) and exposes
the eight reference operators (msd_custom_convolutions.cpp:343-369) on CPU
torch tensors, plus the dense-block host loop of msd_block.py:8-134 on top of
them.  Only the tests, the smoke check and the benchmark's CPU-baseline leg may
import this package; the shipped package never does.
"""
import ctypes
import os
import subprocess

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libmsd_oracle.so")
_lib = None

_i64p = ctypes.POINTER(ctypes.c_int64)


def build(force=False):
    """Compile the C oracle in place (gcc only)."""
    if force:
        subprocess.run(["make", "-C", _HERE, "-B"], check=True, capture_output=True)
    else:
        subprocess.run(["make", "-C", _HERE], check=True, capture_output=True)


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = ctypes.CDLL(_LIB_PATH)
        _lib.msd_oracle_reflect.restype = ctypes.c_int
        _lib.msd_oracle_reflect.argtypes = [ctypes.c_int, ctypes.c_int]
    return _lib


def reflect(i, n):
    """Symmetric index fold of kernel_utils.cuh:30-38."""
    return lib().msd_oracle_reflect(int(i), int(n))


def _sfx(t):
    if t.dtype == torch.float32:
        return "f32"
    if t.dtype == torch.float64:
        return "f64"
    raise TypeError(f"oracle supports float32/float64, got {t.dtype}")


def _arr(vals):
    return (ctypes.c_int64 * len(vals))(*[int(v) for v in vals])


def _view(t):
    """(pointer, five element strides {b, c, z, y, x}) of a 4-D or 5-D CPU tensor."""
    assert t.device.type == "cpu"
    s = list(t.stride())
    if t.dim() == 4:
        s = [s[0], s[1], 0, s[2], s[3]]
    return ctypes.c_void_p(t.data_ptr()), _arr(s)


def _size(t):
    sp = list(t.shape[2:])
    if len(sp) == 2:
        sp = [1] + sp
    return _arr(sp)


def _same_dtype(*ts):
    d = ts[0].dtype
    for t in ts:
        if t.dtype != d:
            raise RuntimeError("oracle: tensors must share one dtype")


def _forward(relu, input, kernel, bias, output, dilation):
    _same_dtype(input, kernel, bias, output)
    ndim = kernel.dim() - 2
    kernel = kernel.contiguous()
    bias = bias.contiguous()
    xp, xs = _view(input)
    yp, ys = _view(output)
    fn = getattr(lib(), "msd_oracle_conv_forward_" + _sfx(input))
    fn(ctypes.c_int(ndim), ctypes.c_int(relu), ctypes.c_int64(input.shape[0]),
       ctypes.c_int64(input.shape[1]), ctypes.c_int64(output.shape[1]), _size(input),
       ctypes.c_int(dilation), xp, xs, ctypes.c_void_p(kernel.data_ptr()),
       ctypes.c_void_p(bias.data_ptr()), yp, ys)


def _backward_x(relu, output, grad_output, kernel, grad_input, dilation):
    _same_dtype(grad_output, kernel, grad_input)
    ndim = kernel.dim() - 2
    kernel = kernel.contiguous()
    op, os_ = _view(output) if relu else (ctypes.c_void_p(0), _arr([0] * 5))
    gp, gs = _view(grad_output)
    xp, xs = _view(grad_input)
    fn = getattr(lib(), "msd_oracle_conv_backward_x_" + _sfx(grad_input))
    fn(ctypes.c_int(ndim), ctypes.c_int(relu), ctypes.c_int64(grad_input.shape[0]),
       ctypes.c_int64(grad_input.shape[1]), ctypes.c_int64(grad_output.shape[1]),
       _size(grad_input), ctypes.c_int(dilation), op, os_, gp, gs,
       ctypes.c_void_p(kernel.data_ptr()), xp, xs)


def _backward_k(relu, output, grad_output, input, grad_kernel, dilation):
    _same_dtype(grad_output, input, grad_kernel)
    assert grad_kernel.is_contiguous()
    ndim = grad_kernel.dim() - 2
    op, os_ = _view(output) if relu else (ctypes.c_void_p(0), _arr([0] * 5))
    gp, gs = _view(grad_output)
    xp, xs = _view(input)
    fn = getattr(lib(), "msd_oracle_conv_backward_k_" + _sfx(input))
    fn(ctypes.c_int(ndim), ctypes.c_int(relu), ctypes.c_int64(input.shape[0]),
       ctypes.c_int64(input.shape[1]), ctypes.c_int64(grad_output.shape[1]), _size(input),
       ctypes.c_int(dilation), op, os_, gp, gs, xp, xs,
       ctypes.c_void_p(grad_kernel.data_ptr()))


def _backward_bias(relu, output, grad_output, grad_bias):
    _same_dtype(grad_output, grad_bias)
    assert grad_bias.is_contiguous()
    ndim = grad_output.dim() - 2
    op, os_ = _view(output) if relu else (ctypes.c_void_p(0), _arr([0] * 5))
    gp, gs = _view(grad_output)
    fn = getattr(lib(), "msd_oracle_conv_backward_bias_" + _sfx(grad_output))
    fn(ctypes.c_int(ndim), ctypes.c_int(relu), ctypes.c_int64(grad_output.shape[0]),
       ctypes.c_int64(grad_output.shape[1]), _size(grad_output), op, os_, gp, gs,
       ctypes.c_void_p(grad_bias.data_ptr()))


# The eight operators, argument order as in msd_custom_convolutions.cpp:343-369.
# block_size is accepted and ignored.

def conv_forward(input, kernel, bias, output, dilation, block_size=None):
    _forward(0, input, kernel, bias, output, dilation)


def conv_backward_x(grad_output, kernel, grad_input, dilation, block_size=None):
    _backward_x(0, None, grad_output, kernel, grad_input, dilation)


def conv_backward_k(grad_output, input, grad_kernel, dilation, block_size=None):
    _backward_k(0, None, grad_output, input, grad_kernel, dilation)


def conv_backward_bias(grad_output, grad_bias, block_size=None):
    _backward_bias(0, None, grad_output, grad_bias)


def conv_relu_forward(input, kernel, bias, output, dilation, block_size=None):
    _forward(1, input, kernel, bias, output, dilation)


def conv_relu_backward_x(output, grad_output, kernel, grad_input, dilation, block_size=None):
    _backward_x(1, output, grad_output, kernel, grad_input, dilation)


def conv_relu_backward_k(output, grad_output, input, grad_kernel, dilation, block_size=None):
    _backward_k(1, output, grad_output, input, grad_kernel, dilation)


def conv_relu_backward_bias(output, grad_output, grad_bias, block_size=None):
    _backward_bias(1, output, grad_output, grad_bias)


def set_num_threads(n):
    """Thread count of the OpenMP loops in the C oracle."""
    omp = ctypes.CDLL("libgomp.so.1")
    omp.omp_set_num_threads(int(n))


def block_forward(input, dilations, bias, weights):
    """Dense-block forward of msd_block.py:8-62: one growing channel stack,
    layer i reads channels [0, start) and writes [start, start + width)."""
    c_in = input.shape[1]
    total = c_in + sum(w.shape[0] for w in weights)
    result = input.new_empty(input.shape[0], total, *input.shape[2:])
    result[:, :c_in] = input
    start, b0 = c_in, 0
    for w, d in zip(weights, dilations):
        n = w.shape[0]
        conv_relu_forward(result[:, :start], w, bias[b0:b0 + n], result[:, start:start + n], d)
        start += n
        b0 += n
    return result


def block_backward(result, grad_output, dilations, bias, weights):
    """Dense-block backward of msd_block.py:64-134: walk the layers in reverse
    on a clone of the incoming gradient; backward_x accumulates into the
    channels in front of the layer.  Returns (grad_input, grad_bias, grad_weights)."""
    gradients = grad_output.clone()
    grad_bias = torch.zeros_like(bias)
    grad_weights = [None] * len(weights)
    end, b1 = result.shape[1], bias.shape[0]
    for idx in reversed(range(len(weights))):
        w = weights[idx]
        n = w.shape[0]
        start, b0 = end - n, b1 - n
        out_i, gout_i = result[:, start:end], gradients[:, start:end]
        conv_relu_backward_x(out_i, gout_i, w, gradients[:, :start], dilations[idx])
        gw = torch.zeros_like(w)
        conv_relu_backward_k(out_i, gout_i, result[:, :start], gw, dilations[idx])
        grad_weights[idx] = gw
        conv_relu_backward_bias(out_i, gout_i, grad_bias[b0:b1])
        end, b1 = start, b0
    return gradients[:, :weights[0].shape[1]], grad_bias, grad_weights
