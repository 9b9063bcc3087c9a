"""Stock-torch statement of the operator, independent of the C oracle and of
the HIP kernels: gather with the symmetric index map, then a stock dilated
convolution without padding, then the clamp.  Autograd through it gives
gradients that share no code with either implementation under test."""
import numpy as np
import torch
import torch.nn.functional as F


def symmetric_index(n, d):
    """Source index for each position of an axis of length n padded by d on
    both sides, numpy 'symmetric' convention (edge sample repeated)."""
    return torch.from_numpy(np.pad(np.arange(n), d, mode="symmetric").astype(np.int64))


def pad_symmetric(x, d):
    for axis in range(2, x.dim()):
        x = x.index_select(axis, symmetric_index(x.shape[axis], d))
    return x


def conv_sym(x, k, bias, d, relu=True):
    conv = F.conv2d if k.dim() == 4 else F.conv3d
    y = conv(pad_symmetric(x, d), k, bias, dilation=d)
    return y.clamp_min(0) if relu else y


def dense_block(x, dilations, bias, weights, relu=True):
    """cat([x, relu(conv_sym(x))]) loop: the mixed-scale dense block."""
    b0 = 0
    for w, d in zip(weights, dilations):
        n = w.shape[0]
        x = torch.cat([x, conv_sym(x, w, bias[b0:b0 + n], d, relu)], dim=1)
        b0 += n
    return x
