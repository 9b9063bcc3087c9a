"""Parity checks shared by the GPU test files: one operator problem, or one dense block,
run through the HIP library (C ABI) and through the CPU oracle on the same seeded data.

Tolerances (max |diff| / max |ref|, fp32): forward 1e-5, gradients 1e-4."""
import torch

import oracle
from cases import make_problem, problem_on, rel_err


def bias_close(got, want, terms, tol=1e-4):
    """A bias gradient is one long sum per channel, which may cancel to almost nothing, so the
    error cannot be measured against the sum itself alone.  The floor is a thousandth of the
    sum of the magnitudes: with tol = 1e-4 that allows 1e-7 * sum|terms|, about two units of
    fp32 round-off on the magnitudes.  The kernels add a few terms per lane in sequence and
    then go up a tree of about 17 levels (lanes, waves, workgroups, the column reduction), so
    their worst case is (terms per lane + 17) * 6e-8 * sum|terms| and their typical error, for
    terms of mixed sign, several orders below that."""
    floor = 1e-3 * terms.abs().double().sum(dim=[0] + list(range(2, terms.dim()))).max().item()
    diff = (got.double().cpu() - want.double()).abs().max().item()
    return diff <= tol * max(want.abs().max().item(), floor)


def check_operator_problem(cc, shape, seed=7, plain=True):
    """conv_relu_forward and the three conv_relu_backward_* operators (accumulating), the plain
    operators (conv_forward, conv_backward_x, conv_backward_kb) and the three plain backward
    operators as one call (conv_backward_xkb), against the oracle.  ``plain=False`` leaves the
    one-by-one plain operators out (problems of several GB, where each oracle call takes
    seconds): the kernels are the same template with the mask compiled out."""
    ref = make_problem(shape, torch.float32, seed=seed)
    dev = problem_on(ref, "cuda")
    d = ref["d"]
    oracle.conv_relu_forward(ref["x"], ref["k"], ref["bias"], ref["y"], d)
    cc.conv_relu_forward(dev["x"], dev["k"], dev["bias"], dev["y"], d)
    assert rel_err(dev["stack"], ref["stack"]) <= 1e-5, "conv_relu_forward"
    assert torch.equal(dev["x"].cpu(), ref["x"]), "conv_relu_forward wrote outside its output channels"
    dev["y"].copy_(ref["y"])                    # same mask on both sides
    want_gk, want_gb = torch.ones_like(ref["k"]), torch.full_like(ref["bias"], -1.0)
    oracle.conv_relu_backward_x(ref["y"], ref["gy"], ref["k"], ref["gx"], d)
    oracle.conv_relu_backward_k(ref["y"], ref["gy"], ref["x"], want_gk, d)
    oracle.conv_relu_backward_bias(ref["y"], ref["gy"], want_gb)
    got_gk, got_gb = torch.ones_like(dev["k"]), torch.full_like(dev["bias"], -1.0)
    cc.conv_relu_backward_x(dev["y"], dev["gy"], dev["k"], dev["gx"], d)
    cc.conv_relu_backward_k(dev["y"], dev["gy"], dev["x"], got_gk, d)
    cc.conv_relu_backward_bias(dev["y"], dev["gy"], got_gb)
    torch.cuda.synchronize()
    assert rel_err(dev["gstack"], ref["gstack"]) <= 1e-4, "conv_relu_backward_x"
    assert torch.equal(dev["gy"].cpu(), ref["gy"]), "conv_relu_backward_x wrote outside grad_input"
    assert rel_err(got_gk, want_gk) <= 1e-4, "conv_relu_backward_k"
    assert bias_close(got_gb, want_gb, ref["gy"] * (ref["y"] > 0)), "conv_relu_backward_bias"
    if not plain:
        # the fused pass on the same data: grad_input accumulates once more, no mask
        want_gk, want_gb = torch.zeros_like(ref["k"]), torch.zeros_like(ref["bias"])
        oracle.conv_backward_x(ref["gy"], ref["k"], ref["gx"], d)
        oracle.conv_backward_k(ref["gy"], ref["x"], want_gk, d)
        oracle.conv_backward_bias(ref["gy"], want_gb)
        got_gk, got_gb = torch.zeros_like(dev["k"]), torch.zeros_like(dev["bias"])
        cc.conv_backward_xkb(dev["gy"], dev["x"], dev["k"], dev["gx"], got_gk, got_gb, d)
        torch.cuda.synchronize()
        assert rel_err(dev["gstack"], ref["gstack"]) <= 1e-4, "conv_backward_xkb grad_input"
        assert rel_err(got_gk, want_gk) <= 1e-4, "conv_backward_xkb grad_kernel"
        assert bias_close(got_gb, want_gb, ref["gy"]), "conv_backward_xkb grad_bias"
        return
    del ref, dev
    # the plain (no-ReLU) operators one by one
    ref3 = make_problem(shape, torch.float32, seed=seed + 2)
    dev3 = problem_on(ref3, "cuda")
    want_gk, want_gb = torch.zeros_like(ref3["k"]), torch.zeros_like(ref3["bias"])
    oracle.conv_forward(ref3["x"], ref3["k"], ref3["bias"], ref3["y"], d)
    oracle.conv_backward_x(ref3["gy"], ref3["k"], ref3["gx"], d)
    oracle.conv_backward_k(ref3["gy"], ref3["x"], want_gk, d)
    oracle.conv_backward_bias(ref3["gy"], want_gb)
    got_gk, got_gb = torch.zeros_like(dev3["k"]), torch.zeros_like(dev3["bias"])
    cc.conv_forward(dev3["x"], dev3["k"], dev3["bias"], dev3["y"], d)
    cc.conv_backward_x(dev3["gy"], dev3["k"], dev3["gx"], d)
    cc.conv_backward_kb(dev3["gy"], dev3["x"], got_gk, got_gb, d)
    torch.cuda.synchronize()
    assert rel_err(dev3["stack"], ref3["stack"]) <= 1e-5, "conv_forward"
    assert rel_err(dev3["gstack"], ref3["gstack"]) <= 1e-4, "conv_backward_x"
    assert rel_err(got_gk, want_gk) <= 1e-4, "conv_backward_kb grad_kernel"
    assert bias_close(got_gb, want_gb, ref3["gy"]), "conv_backward_kb grad_bias"
    # the three plain operators in one call
    del ref3, dev3
    ref2 = make_problem(shape, torch.float32, seed=seed + 1)
    dev2 = problem_on(ref2, "cuda")
    want_gk, want_gb = torch.zeros_like(ref2["k"]), torch.zeros_like(ref2["bias"])
    oracle.conv_backward_x(ref2["gy"], ref2["k"], ref2["gx"], d)
    oracle.conv_backward_k(ref2["gy"], ref2["x"], want_gk, d)
    oracle.conv_backward_bias(ref2["gy"], want_gb)
    got_gk, got_gb = torch.zeros_like(dev2["k"]), torch.zeros_like(dev2["bias"])
    cc.conv_backward_xkb(dev2["gy"], dev2["x"], dev2["k"], dev2["gx"], got_gk, got_gb, d)
    torch.cuda.synchronize()
    assert rel_err(dev2["gstack"], ref2["gstack"]) <= 1e-4, "conv_backward_xkb grad_input"
    assert rel_err(got_gk, want_gk) <= 1e-4, "conv_backward_xkb grad_kernel"
    assert bias_close(got_gb, want_gb, ref2["gy"]), "conv_backward_xkb grad_bias"


def block_problem(ndim, size, c_in, width, depth, batch, dilations=None, seed=0):
    """Input, dilations (1..10 in turn unless given), bias, weights and the gradient of the
    whole stack, fp32 on the CPU."""
    gen = torch.Generator().manual_seed(seed)
    dil = list(dilations) if dilations is not None else [min((i % 10) + 1, min(size)) for i in range(depth)]
    taps = 3 ** ndim
    ws = [torch.randn(width, c_in + width * i, *([3] * ndim), generator=gen)
          * (2.0 / (taps * (c_in + width * max(depth - 1, 1)) + 1)) ** 0.5 for i in range(depth)]
    bias = torch.randn(width * depth, generator=gen) * 0.05
    x = torch.rand(batch, c_in, *size, generator=gen)
    g = torch.randn(batch, c_in + width * depth, *size, generator=gen)
    return x, dil, bias, ws, g


def check_block(ndim, size, c_in, width, depth, batch, dilations=None, seed=0, input_grad=True):
    """msd_block forward + backward (native layer loops) against the fp64 oracle: the whole
    stack, grad_input (unless the input takes no gradient), every weight gradient and the bias
    gradient."""
    from msd_pytorch_amd.msd_block import msd_block
    x, dil, bias, ws, g = block_problem(ndim, size, c_in, width, depth, batch, dilations, seed)
    xd = x.cuda().requires_grad_(input_grad)
    bd = bias.cuda().requires_grad_(True)
    wd = [w.cuda().requires_grad_(True) for w in ws]
    got = msd_block(xd, dil, bd, *wd)
    got.backward(g.cuda())
    torch.cuda.synchronize()
    ws64 = [w.double() for w in ws]
    want = oracle.block_forward(x.double(), dil, bias.double(), ws64)
    assert rel_err(got, want) <= 1e-5, "stack"
    del want
    # The backward oracle takes its ReLU masks from the stack the GPU computed: an activation
    # within rounding of zero may have the other sign in double precision, and one flipped
    # mask in an upper layer changes every gradient below it by far more than the tolerance.
    want_gx, want_gb, want_gw = oracle.block_backward(got.detach().double().cpu(), g.double(), dil, bias.double(),
                                                      ws64)
    if input_grad:
        assert rel_err(xd.grad, want_gx) <= 1e-4, "grad_input"
    else:
        assert xd.grad is None
    assert rel_err(bd.grad, want_gb) <= 1e-4, "grad_bias"
    worst = max((rel_err(a.grad, b), i) for i, (a, b) in enumerate(zip(wd, want_gw)))
    assert worst[0] <= 1e-4, "grad_weight of layer %d" % worst[1]
