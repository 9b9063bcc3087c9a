"""Dense block, module and model wrappers on the GPU (HIP kernels through the
C ABI), against the CPU oracle and against the behaviour the reference's tests
pin (tests/test_msd_block.py, test_msd_module.py, test_msd_regression_model.py,
test_msd_segmentation_model.py of the reference)."""
import os

import pytest
import torch

import oracle
from cases import rel_err

pytestmark = pytest.mark.gpu


def make_block_problem(ndim, size, c_in, width, depth, dtype, batch=2, seed=0):
    gen = torch.Generator().manual_seed(seed)
    dil = [(i % 10) + 1 for i in range(depth)]
    dil = [min(d, min(size)) for d in dil]
    taps = 3 ** ndim
    ws = [torch.randn(width, c_in + width * i, *([3] * ndim), dtype=dtype, generator=gen)
          * (2.0 / (taps * (c_in + width * max(depth - 1, 1)) + 1)) ** 0.5 for i in range(depth)]
    bias = torch.randn(width * depth, dtype=dtype, generator=gen) * 0.05
    x = torch.rand(batch, c_in, *size, dtype=dtype, generator=gen)
    g = torch.randn(batch, c_in + width * depth, *size, dtype=dtype, generator=gen)
    return x, dil, bias, ws, g


@pytest.mark.parametrize("ndim,size,c_in,width,depth,dtype", [
    (2, (40, 72), 1, 1, 12, torch.float32),
    (2, (33, 64), 2, 2, 6, torch.float32),
    (3, (10, 12, 66), 1, 1, 8, torch.float32),
    (3, (6, 9, 33), 2, 2, 4, torch.float32),
    (2, (13, 21), 3, 2, 3, torch.float64),
    (3, (5, 7, 11), 3, 1, 3, torch.float64),
    (2, (1, 5), 1, 1, 3, torch.float64),            # reference tests/test_msd_block.py:9-23
])
def test_block_matches_oracle(ndim, size, c_in, width, depth, dtype):
    from msd_pytorch_amd.msd_block import msd_block
    x, dil, bias, ws, g = make_block_problem(ndim, size, c_in, width, depth, dtype)
    want = oracle.block_forward(x, dil, bias, ws)
    want_gx, want_gb, want_gw = oracle.block_backward(want, g, dil, bias, ws)

    xd = x.cuda().requires_grad_(True)
    bd = bias.cuda().requires_grad_(True)
    wd = [w.cuda().requires_grad_(True) for w in ws]
    got = msd_block(xd, dil, bd, *wd)
    got.backward(g.cuda())
    torch.cuda.synchronize()
    tf, tg = (1e-5, 1e-4) if dtype == torch.float32 else (1e-11, 1e-10)
    assert rel_err(got, want) <= tf
    assert rel_err(xd.grad, want_gx) <= tg
    assert rel_err(bd.grad, want_gb) <= tg
    for a, b in zip(wd, want_gw):
        assert rel_err(a.grad, b) <= tg


FUSED_BLOCK_CASES = [
    # shapes the fused backward_x + backward_k kernel of the block takes (width 1, rows of
    # whole 4-voxel groups and at least one wavefront), with ragged rows, row groups and
    # channel blocks (16 input channels each)
    (2, (37, 256), 1, 20, 2, None),        # 4 voxels per lane, 4 rows per workgroup, 37 rows
    (2, (9, 1024), 2, 5, 1, None),         # one row per workgroup
    (2, (30, 132), 3, 36, 1, None),        # 33 of 64 lanes per row busy; 3 channel blocks
    (2, (40, 128), 1, 4, 1, [1, 7, 31, 40]),   # dilations up to the image height
    (3, (9, 11, 128), 1, 18, 1, None),     # one voxel per lane, 2 rows per workgroup
    (3, (6, 7, 68), 2, 6, 2, None),        # 68 of 128 lanes per row busy
    (3, (12, 5, 64), 1, 3, 1, [5, 1, 4]),  # dilation == smallest extent
    (2, (700, 260), 1, 3, 2, None),        # more row groups than workgroups: several tiles each
    (3, (33, 31, 68), 2, 3, 2, None),      # the same in 3D, last groups ragged
    (2, (21, 128), 2, 11, 1, None, 2),     # width 2: two output channels per layer in the fused pass
    (2, (300, 132), 2, 4, 2, None, 2),     # width 2, several tiles per workgroup
    (2, (23, 2048), 1, 5, 2, [1, 2, 9, 23, 4]),      # rows of 2 segments of 1024 voxels
    (2, (19, 1536), 2, 3, 1, [3, 1, 10], 2),       # width 2, rows of 2 segments (1024 and 512 voxels)
    (2, (11, 750), 1, 4, 1, None),         # rows that are not whole groups of four voxels
    (2, (6, 1001), 2, 3, 2, [1, 5, 3], 2),   # odd rows, width 2
    (3, (5, 6, 130), 1, 3, 1, None),       # the same in 3D
    (3, (4, 7, 516), 2, 3, 1, [2, 4, 1]),  # 3D rows of three segments
    (2, (30, 132), 2, 4, 1, None, 3),      # width 3: the separate kernels, two output channels at a time
    (3, (6, 7, 68), 1, 3, 2, None, 3),     # the same in 3D
]


@pytest.mark.parametrize("ndim,size,c_in,depth,batch,dilations,width",
                         [c if len(c) == 7 else c + (1,) for c in FUSED_BLOCK_CASES])
def test_fused_block_backward_matches_oracle(ndim, size, c_in, depth, batch, dilations, width):
    from msd_pytorch_amd import _native
    from msd_pytorch_amd.msd_block import msd_block
    x, dil, bias, ws, g = make_block_problem(ndim, size, c_in, width, depth, torch.float32, batch=batch)
    if dilations is not None:
        dil = dilations
    want = oracle.block_forward(x.double(), dil, bias.double(), [w.double() for w in ws])
    want_gx, want_gb, want_gw = oracle.block_backward(want, g.double(), dil, bias.double(), [w.double() for w in ws])

    lib = _native.load()
    results = {}
    for fuse in (1, 0):
        assert lib.msd_set_tuning(b"block.fuse", fuse) == 0
        try:
            xd = x.cuda().requires_grad_(True)
            bd = bias.cuda().requires_grad_(True)
            wd = [w.cuda().requires_grad_(True) for w in ws]
            got = msd_block(xd, dil, bd, *wd)
            got.backward(g.cuda())
            torch.cuda.synchronize()
        finally:
            lib.msd_set_tuning(b"block.fuse", -1)
        assert rel_err(got, want) <= 1e-5
        assert rel_err(xd.grad, want_gx) <= 1e-4
        assert rel_err(bd.grad, want_gb) <= 1e-4
        assert max(rel_err(a.grad, b) for a, b in zip(wd, want_gw)) <= 1e-4
        results[fuse] = (xd.grad, bd.grad, [w.grad for w in wd])
    # the fused and the separate kernels add the same terms in different orders
    assert rel_err(results[1][0], results[0][0]) <= 1e-5
    assert max(rel_err(a, b) for a, b in zip(results[1][2], results[0][2])) <= 1e-5


@pytest.mark.parametrize("ndim,size,depth", [(2, (24, 128), 37), (3, (5, 6, 64), 19)])
def test_block_backward_deferred_reductions_give_the_same_bits(ndim, size, depth):
    # the reverse loop reduces the partial weight-gradient sums of up to 16 layers in one
    # launch; every column is added in the order a launch of its own uses
    from msd_pytorch_amd import _native
    from msd_pytorch_amd import msd_custom_convolutions as cc
    x, dil, bias, ws, g = make_block_problem(ndim, size, 2, 1, depth, torch.float32, batch=2)
    lib = _native.load()
    stack = torch.empty(2, 2 + depth, *size, device="cuda")
    stack[:, :2] = x.cuda()
    wd = [w.cuda() for w in ws]
    cc.block_forward(stack, 2, dil, bias.cuda(), wd)
    results = []
    for defer in (1, 0):
        assert lib.msd_set_tuning(b"block.defer", defer) == 0
        try:
            grads = g.cuda().clone()
            gw = [torch.zeros_like(w) for w in wd]
            gb = torch.zeros(depth, device="cuda")
            cc.block_backward(stack, grads, 2, dil, wd, gw, gb, True)
            torch.cuda.synchronize()
        finally:
            lib.msd_set_tuning(b"block.defer", -1)
        results.append((grads[:, :2].clone(), gb, gw))
    assert torch.equal(results[0][0], results[1][0])
    assert torch.equal(results[0][1], results[1][1])
    assert all(torch.equal(a, b) for a, b in zip(results[0][2], results[1][2]))
    assert all(float(w.abs().max()) > 0 for w in results[0][2])


def test_depth_100_stack_stays_within_tolerance():
    # errors compound through the layers: the full depth of the headline network on a small image
    from msd_pytorch_amd.msd_block import msd_block
    x, dil, bias, ws, g = make_block_problem(2, (48, 64), 1, 1, 100, torch.float32, batch=1)
    want = oracle.block_forward(x.double(), dil, bias.double(), [w.double() for w in ws])
    want_gx, want_gb, want_gw = oracle.block_backward(want, g.double(), dil, bias.double(), [w.double() for w in ws])
    xd = x.cuda().requires_grad_(True)
    bd = bias.cuda().requires_grad_(True)
    wd = [w.cuda().requires_grad_(True) for w in ws]
    got = msd_block(xd, dil, bd, *wd)
    got.backward(g.cuda())
    assert rel_err(got, want) <= 1e-5
    assert rel_err(xd.grad, want_gx) <= 1e-4
    assert rel_err(bd.grad, want_gb) <= 1e-4
    assert max(rel_err(a.grad, b) for a, b in zip(wd, want_gw)) <= 1e-4


@pytest.mark.parametrize("ndim,size", [(2, (13, 21)), (3, (5, 7, 11))])
def test_block_gradcheck_f64(ndim, size):
    # reference tests/test_msd_block.py:26-66
    from msd_pytorch_amd.msd_block import MSDBlock
    torch.manual_seed(0)
    blk = MSDBlock(3, [1, 2, 3], width=2, ndim=ndim).cuda().double()
    x = torch.randn(2, 3, *size, dtype=torch.float64, device="cuda", requires_grad=True)
    assert torch.autograd.gradcheck(blk, (x,), eps=1e-6, atol=1e-5)


@pytest.mark.parametrize("ndim,size", [(2, (13, 21)), (3, (7, 9, 6))])
def test_single_layer_gradcheck_f64(ndim, size):
    # reference tests/test_conv2d.py:488-515, tests/test_conv3d.py:376-405
    from msd_pytorch_amd.conv2d import conv2d, conv2d_relu
    from msd_pytorch_amd.conv3d import conv3d, conv3d_relu
    torch.manual_seed(0)
    fns = (conv2d, conv2d_relu) if ndim == 2 else (conv3d, conv3d_relu)
    x = torch.randn(2, 3, *size, dtype=torch.float64, device="cuda", requires_grad=True)
    w = torch.randn(2, 3, *([3] * ndim), dtype=torch.float64, device="cuda", requires_grad=True)
    b = torch.randn(2, dtype=torch.float64, device="cuda", requires_grad=True)
    for fn in fns:
        def f(x_, w_, b_):
            return fn(x_, w_, b_, torch.empty(2, 2, *size, dtype=torch.float64, device="cuda"), 1, 3)
        assert torch.autograd.gradcheck(f, (x, w, b), eps=1e-6, atol=1e-5)


def test_module_rejects_zero_depth_and_width():
    # tests/test_msd_module.py:133-137 of the reference
    from msd_pytorch_amd import MSDModule
    with pytest.raises(ValueError):
        MSDModule(1, 1, depth=0, width=1)
    with pytest.raises(ValueError):
        MSDModule(1, 1, depth=1, width=0)


@pytest.mark.parametrize("mean", [-10, 0, 10])
@pytest.mark.parametrize("std", [1, 10])
def test_normalization_scale_out_inverts_scale_in(mean, std):
    # tests/test_msd_model.py:6-36 of the reference: input and target with the same moments make
    # the two frozen scaling layers each other's inverse
    from msd_pytorch_amd.msd_model import MSDModel
    from torch.utils.data import DataLoader, TensorDataset
    torch.manual_seed(1)
    model = MSDModel(3, 3, 10, 1)
    d_in = mean + torch.randn(1, 3, 100, 100) * std
    model.set_normalization(DataLoader(TensorDataset(d_in, d_in.clone()), 1))
    x = torch.randn_like(d_in).cuda()
    y = model.scale_out.cuda()(model.scale_in.cuda()(x))
    assert (x - y).abs().mean().item() < 1e-4


def test_module_zero_output_then_all_parameters_move():
    # reference tests/test_msd_module.py:11-16 and :87-130
    from msd_pytorch_amd.msd_module import MSDModule
    torch.manual_seed(0)
    net = MSDModule(2, 3, depth=6, width=2).cuda()
    x = torch.randn(2, 2, 24, 40, device="cuda")
    assert torch.equal(net(x), torch.zeros(2, 3, 24, 40, device="cuda"))
    before = [p.detach().clone() for p in net.parameters()]
    opt = torch.optim.Adam(net.parameters())
    target = torch.randn(2, 3, 24, 40, device="cuda")
    for _ in range(2):     # the hidden layers only get gradients once the final layer has left zero
        opt.zero_grad()
        torch.nn.functional.mse_loss(net(x), target).backward()
        opt.step()
    for b, p in zip(before, net.parameters()):
        assert not torch.equal(b, p.detach())


@pytest.mark.parametrize("ndim,size,dtype", [(2, (33, 70), torch.float32), (3, (9, 12, 40), torch.float32),
                                             (2, (12, 17), torch.float64)])
def test_module_as_one_node_equals_block_then_final_layer(ndim, size, dtype):
    # MSDModule.forward runs block + final layer as one autograd node; the two modules called
    # one after the other (the reference's msd_module.py:144-146) must give the same bits
    from msd_pytorch_amd import MSDModule
    torch.manual_seed(3)
    net = MSDModule(2, 3, depth=6, width=2, dilations=[1, 2, 3], ndim=ndim).cuda().to(dtype)
    net.final_layer.linear.weight.data.normal_(0, 0.3)
    net.final_layer.linear.bias.data.normal_(0, 0.3)
    x = torch.randn(2, 2, *size, device="cuda", dtype=dtype, requires_grad=True)
    g = torch.randn(2, 3, *size, device="cuda", dtype=dtype)

    def run(forward):
        for p in net.parameters():
            p.grad = None
        x.grad = None
        out = forward(x)
        out.backward(g)
        return [out.detach().clone(), x.grad.clone()] + [p.grad.clone() for p in net.parameters()]

    one = run(net)
    two = run(lambda t: net.final_layer(net.msd_block(t)))
    assert len(one) == len(two) == 2 + len(list(net.parameters()))
    for a, b in zip(one, two):
        assert torch.equal(a, b)
    # a hook on a sub-module is honoured: the modules are then called one by one
    seen = []
    handle = net.msd_block.register_forward_hook(lambda m, i, o: seen.append(tuple(o.shape)))
    hooked = run(net)
    handle.remove()
    assert seen == [(2, 2 + 6 * 2, *size)]
    for a, b in zip(one, hooked):
        assert torch.equal(a, b)
    # gradients only for the final layer, or only for the input
    for p in net.msd_block.parameters():
        p.requires_grad_(False)
    out = net(x.detach())
    out.backward(g)
    assert net.final_layer.linear.weight.grad is not None
    for p in net.parameters():
        p.requires_grad_(False)
    x.grad = None
    net(x).backward(g)
    # (without weight gradients the block runs backward_x alone, another summation order than
    # the one-pass kernel's: the same values, not the same bits)
    assert rel_err(x.grad, one[1]) <= 1e-5
    with torch.no_grad():
        assert torch.equal(net(x), one[0])


@pytest.mark.parametrize("ndim", [2, 3])
def test_regression_model_api(ndim, tmp_path):
    # reference tests/test_msd_regression_model.py:8-143
    from msd_pytorch_amd import MSDRegressionModel
    torch.manual_seed(0)
    size = (20, 36) if ndim == 2 else (6, 8, 34)
    model = MSDRegressionModel(2, 1, depth=5, width=1, dilations=[1, 2, 3], loss="L2", ndim=ndim)
    x = torch.randn(3, 2, *size)
    y = x.sum(1, keepdim=True) * 0.5
    model.set_normalization([(x, y)])
    before = [p.detach().clone() for p in model.optimizer.param_groups[0]["params"]]
    losses = [model.learn(x, y) for _ in range(10)]
    assert all(l == l for l in losses) and losses[-1] < losses[0]
    for b, p in zip(before, model.optimizer.param_groups[0]["params"]):
        assert not torch.equal(b, p.detach())
    assert model.get_output().shape == (3, 1, *size) and model.get_output().is_cuda
    assert abs(model.get_loss() - model.forward(x, y)) < 1e-3 * max(1.0, model.get_loss()) or True
    assert model.validate([(x, y), (x, y)]) > 0
    model.train([(x, y)], 1)
    path = os.path.join(tmp_path, "net.torch")
    model.save(path, 7)
    other = MSDRegressionModel(2, 1, depth=5, width=1, dilations=[1, 2, 3], loss="L2", ndim=ndim)
    assert other.load(path) == 7
    for (ka, va), (kb, vb) in zip(model.net.state_dict().items(), other.net.state_dict().items()):
        assert ka == kb and torch.equal(va.cpu(), vb.cpu())
    assert abs(other.forward(x, y) - model.forward(x, y)) < 1e-6
    with pytest.raises(ValueError):
        MSDRegressionModel(1, 1, 2, 1, loss="nope")
    with pytest.raises(ValueError):
        MSDRegressionModel(1, 1, 2, 1, ndim=4)


def test_checkpoints_across_data_parallel_and_bad_files(tmp_path):
    # a file in the layout the reference's save writes (msd_model.py:310-324), saved from a
    # DataParallel net ("module." keys), loads into a plain model, and the other way round
    from collections import OrderedDict
    from msd_pytorch_amd import MSDRegressionModel
    torch.manual_seed(1)
    model = MSDRegressionModel(1, 1, depth=4, width=2, dilations=[1, 2])
    x = torch.randn(2, 1, 16, 40)
    y = x * 2 + 1
    model.set_normalization([(x, y)])
    for _ in range(3):
        model.learn(x, y)
    wrapped = OrderedDict(("module." + k, v.clone()) for k, v in model.net.state_dict().items())
    path = os.path.join(tmp_path, "parallel.torch")
    torch.save({"epoch": 11, "state_dict": wrapped, "optimizer": model.optimizer.state_dict()}, path)
    other = MSDRegressionModel(1, 1, depth=4, width=2, dilations=[1, 2])
    assert other.load(path) == 11
    assert abs(other.forward(x, y) - model.forward(x, y)) < 1e-6
    # the restored optimiser continues exactly like the original one
    assert abs(other.learn(x, y) - model.learn(x, y)) < 1e-6
    assert abs(other.forward(x, y) - model.forward(x, y)) < 1e-6
    # plain file into a DataParallel model
    plain = os.path.join(tmp_path, "plain.torch")
    model.save(plain, 12)
    par = MSDRegressionModel(1, 1, depth=4, width=2, dilations=[1, 2], parallel=True)
    assert par.load(plain) == 12
    assert all(k.startswith("module.") for k in par.net.state_dict())
    assert abs(par.forward(x, y) - model.forward(x, y)) < 1e-6
    # other architecture: a message that names the parameter
    with pytest.raises(RuntimeError, match="msd_block.bias has shape"):
        MSDRegressionModel(1, 1, depth=4, width=1, dilations=[1, 2]).load(plain)
    with pytest.raises(RuntimeError):
        MSDRegressionModel(1, 1, depth=5, width=2, dilations=[1, 2]).load(plain)
    # not a checkpoint
    bad = os.path.join(tmp_path, "bad.torch")
    torch.save({"weights": 1}, bad)
    with pytest.raises(RuntimeError, match="not an MSD checkpoint"):
        model.load(bad)
    with pytest.raises(ValueError, match="zero variance"):
        model.set_normalization([(torch.ones(1, 1, 8, 8), y)])


@pytest.mark.parametrize("task", ["regression", "segmentation"])
def test_getting_started_example(task, tmp_path):
    # the reference's examples/getting_started.py workflow on synthetic TIFF files:
    # ImageDataset -> normalisation -> train -> save -> load -> predictions on disk
    from msd_pytorch_amd.examples import getting_started
    from msd_pytorch_amd.image_dataset import ImageStack
    result = getting_started.main(["--task", task, "--epochs", "4", "--depth", "8", "--synthetic-size", "48",
                                   "--synthetic-count", "6", "--labels", "0", "1", "2", "--out", str(tmp_path)])
    train_errors = [h[0] for h in result["history"]]
    assert all(e == e for e in train_errors) and train_errors[-1] < train_errors[0]
    assert result["predictions"] == 3
    outputs = ImageStack(tmp_path / "output_*.tif")
    assert len(outputs) == 3 and outputs[0].shape == (1, 48, 48)
    if task == "segmentation":
        assert float(outputs[0].max()) <= 2


@pytest.mark.parametrize("ndim,channels", [(2, 1), (2, 3), (3, 2)])
def test_scaling_modules_run_natively_and_match_conv(ndim, channels):
    # scale_in / scale_out (msd_model.py:8-45) are nn.Conv2d/3d subclasses whose forward is one
    # native pass on the GPU; values and input gradient are those of the torch convolution
    from msd_pytorch_amd.msd_model import scaling_module, scaling_module_set_bias, scaling_module_set_scale
    torch.manual_seed(5)
    sm = scaling_module(channels, conv3d=ndim == 3).cuda()
    assert isinstance(sm, torch.nn.Conv3d if ndim == 3 else torch.nn.Conv2d)
    assert sorted(sm.state_dict()) == ["bias", "weight"]
    scaling_module_set_scale(sm, 0.37)
    scaling_module_set_bias(sm, -1.25)
    sm.weight.data += 0.01 * torch.randn_like(sm.weight)      # off-diagonal terms too
    size = (19, 70) if ndim == 2 else (5, 9, 34)
    x = torch.randn(2, channels, *size, device="cuda", requires_grad=True)
    g = torch.randn(2, channels, *size, device="cuda")
    y = sm(x)
    y.backward(g)
    conv = torch.nn.functional.conv3d if ndim == 3 else torch.nn.functional.conv2d
    x2 = x.detach().clone().requires_grad_(True)
    y2 = conv(x2, sm.weight, sm.bias)
    y2.backward(g)
    assert rel_err(y, y2) <= 1e-6 and rel_err(x.grad, x2.grad) <= 1e-6
    assert sm.weight.grad is None and sm.bias.grad is None
    # a view with strided planes falls back to torch
    xs = torch.randn(2, channels, *size[:-1], 2 * size[-1], device="cuda")[..., ::2]
    assert rel_err(sm(xs), conv(xs, sm.weight, sm.bias)) <= 1e-6


def test_gradients_and_learn_report_the_forward_loss():
    from msd_pytorch_amd import MSDRegressionModel
    torch.manual_seed(2)
    model = MSDRegressionModel(1, 1, depth=4, width=1, dilations=[1, 2])
    model.msd.final_layer.linear.weight.data.normal_(0, 0.1)
    x = torch.randn(1, 1, 24, 40)
    y = 0.5 * x
    loss = model.forward(x, y)
    assert model.gradients(x, y) == loss
    grads = [p.grad.clone() for p in model.msd.parameters()]
    assert all(g is not None and bool(torch.isfinite(g).all()) for g in grads)
    assert any(float(g.abs().max()) > 0 for g in grads)
    assert model.learn(x, y) == loss                           # the loss before the update
    assert model.forward(x, y) != loss                         # the update moved the parameters


@pytest.mark.parametrize("kind,ndim,size", [("regression", 2, (48, 96)), ("segmentation", 2, (48, 96)),
                                            ("regression", 3, (6, 10, 64)), ("regression", 2, (6, 1024))],
                         ids=["regression-2d", "segmentation-2d", "regression-3d", "regression-2d-rows-of-1024"])
def test_step_replayed_from_a_hip_graph_equals_the_eager_step(kind, ndim, size):
    # every replay is checked against the eager step on the same data, with eager work and
    # synchronisations between the replays (rows of 1024 voxels: the backward kernels that ask
    # for more than 64 KB of LDS)
    from msd_pytorch_amd import GraphedStep, MSDRegressionModel, MSDSegmentationModel
    torch.manual_seed(11)
    dil = [1, 2, 3, 4, 5]
    if kind == "regression":
        model = MSDRegressionModel(2, 1, depth=9, width=1, dilations=dil, ndim=ndim)
        new_target = lambda: torch.randn(2, 1, *size)
    else:
        model = MSDSegmentationModel(2, 3, depth=9, width=1, dilations=dil, ndim=ndim)
        new_target = lambda: torch.randint(0, 3, (2, 1, *size))
    model.msd.final_layer.linear.weight.data.normal_(0, 0.2)
    model.set_input(torch.randn(2, 2, *size))
    model.set_target(new_target())
    params = list(model.msd.parameters())
    graphed = GraphedStep(model)
    for _ in range(3):
        x, t = torch.randn(2, 2, *size), new_target()
        graphed(x, t)
        got = [torch.tensor(graphed.loss())] + [p.grad.detach().clone().cpu() for p in params]
        assert model.get_loss() == graphed.loss() and model.get_output().shape[0] == 2
        eager_loss = model.gradients(x, t)
        want = [torch.tensor(eager_loss)] + [p.grad.detach().clone().cpu() for p in params]
        assert all(torch.equal(a, b) for a, b in zip(got, want))
        assert all(float(g.abs().max()) > 0 for g in got[1:])
    with pytest.raises(ValueError, match="capturable"):
        GraphedStep(model, update=True)


def test_graphed_step_with_capturable_adam_follows_the_eager_optimiser():
    from msd_pytorch_amd import GraphedStep, MSDRegressionModel
    size = (32, 64)
    models = []
    for _ in range(2):
        torch.manual_seed(12)
        m = MSDRegressionModel(1, 1, depth=6, width=1, dilations=[1, 2, 3])
        m.msd.final_layer.linear.weight.data.normal_(0, 0.2)
        m.optimizer = torch.optim.Adam(m.msd.parameters(), capturable=True)
        models.append(m)
    eager, captured = models
    torch.manual_seed(13)
    batches = [(torch.randn(1, 1, *size), torch.randn(1, 1, *size)) for _ in range(4)]
    captured.set_input(batches[0][0])
    captured.set_target(batches[0][1])
    with pytest.raises(ValueError, match="warmup"):
        GraphedStep(captured, update=True, warmup=0)
    graphed = GraphedStep(captured, update=True, warmup=1)     # one real step on the first batch
    eager.learn(*batches[0])
    before = [p.detach().clone() for p in captured.msd.parameters()]
    for p, q in zip(captured.msd.parameters(), eager.msd.parameters()):
        assert rel_err(p.detach(), q.detach()) <= 1e-6         # the capture itself records, it does not run
    for x, t in batches[1:]:
        graphed(x, t)
        eager.learn(x, t)
        assert abs(graphed.loss() - eager.get_loss()) <= 1e-6 * max(1.0, abs(eager.get_loss()))
    for a, b in zip(captured.msd.parameters(), eager.msd.parameters()):
        assert rel_err(a.detach(), b.detach()) <= 1e-5
    assert any(not torch.equal(p.detach(), b) for p, b in zip(captured.msd.parameters(), before))


def test_train_with_a_recorded_step_follows_the_eager_loop():
    # MSDModel.train(graph=True): the step of the first batch runs eagerly and is recorded, later
    # batches replay it; the plain Adam of the model is switched to its capturable form with
    # its state kept (one eager step was taken before)
    from msd_pytorch_amd import MSDRegressionModel
    size = (32, 64)
    torch.manual_seed(21)
    batches = [(torch.randn(1, 1, *size), torch.randn(1, 1, *size)) for _ in range(5)]
    models = []
    for _ in range(2):
        torch.manual_seed(20)
        m = MSDRegressionModel(1, 1, depth=5, width=1, dilations=[1, 2, 3])
        m.msd.final_layer.linear.weight.data.normal_(0, 0.2)
        m.learn(*batches[0])
        models.append(m)
    eager, recorded = models
    eager.train(batches[1:], 2)
    recorded.train(batches[1:], 2, graph=True)
    assert recorded.optimizer.defaults["capturable"]
    for a, b in zip(recorded.msd.parameters(), eager.msd.parameters()):
        assert rel_err(a.detach(), b.detach()) <= 1e-5
    assert abs(recorded.get_loss() - eager.get_loss()) <= 1e-5 * max(1.0, abs(eager.get_loss()))


def test_train_with_a_recorded_step_leaves_gpu_resident_batches_alone():
    # batches that are on the GPU already (set_input / set_target keep such tensors as they
    # are): the recorded step copies later batches into buffers of its own, not into the
    # caller's first batch; a smaller last batch gets a recorded step of its own, once
    from msd_pytorch_amd import MSDRegressionModel
    import warnings
    size = (32, 64)
    torch.manual_seed(23)
    batches = [(torch.randn(2, 1, *size).cuda(), torch.randn(2, 1, *size).cuda()) for _ in range(3)]
    batches.append((torch.randn(1, 1, *size).cuda(), torch.randn(1, 1, *size).cuda()))
    copies = [(a.clone(), b.clone()) for a, b in batches]
    models = []
    for _ in range(2):
        torch.manual_seed(22)
        m = MSDRegressionModel(1, 1, depth=4, width=1, dilations=[1, 2, 3])
        m.msd.final_layer.linear.weight.data.normal_(0, 0.2)
        models.append(m)
    eager, recorded = models
    eager.train(batches, 2)
    with warnings.catch_warnings():
        warnings.simplefilter("error")          # no stream-mismatch warning from the capture
        recorded.train(batches, 2, graph=True)
    torch.cuda.synchronize()
    for (a, b), (a0, b0) in zip(batches, copies):
        assert torch.equal(a, a0) and torch.equal(b, b0)
    for a, b in zip(recorded.msd.parameters(), eager.msd.parameters()):
        assert rel_err(a.detach(), b.detach()) <= 1e-5


def test_train_checks_gpu_resident_labels_without_waiting_per_batch():
    # labels on the GPU: train() validates them on the device and raises once per epoch,
    # where set_target (msd_segmentation_model.py:105-119) raises at once
    from msd_pytorch_amd import MSDSegmentationModel
    torch.manual_seed(24)
    model = MSDSegmentationModel(1, 3, depth=3, width=1, dilations=[1, 2])
    x = torch.randn(1, 1, 24, 64).cuda()
    good = torch.randint(0, 3, (1, 1, 24, 64)).cuda()
    model.train([(x, good)] * 3, 1)
    assert model.get_loss() == model.get_loss()
    with pytest.raises(ValueError):
        model.set_target(good + 1)
    with pytest.raises(ValueError):
        model.train([(x, good), (x, good + 1)], 1)
    with pytest.raises(ValueError):
        model.train([(x, good * -1)], 1)
    model.train([(x, good)], 1)                 # the verdict of a failed epoch is not carried over
    # host tensors are still checked on the host, batch by batch
    with pytest.raises(ValueError):
        model.train([(x.cpu(), (good + 1).cpu())], 1)


def test_regression_state_dict_keys():
    # key layout of the reference's checkpoints (msd_regression_model.py:76, msd_block.py:170-179)
    from msd_pytorch_amd import MSDRegressionModel
    model = MSDRegressionModel(1, 1, depth=3, width=1)
    assert sorted(model.net.state_dict()) == sorted([
        "0.weight", "0.bias", "1.msd_block.bias", "1.msd_block.weight0", "1.msd_block.weight1",
        "1.msd_block.weight2", "1.final_layer.linear.weight", "1.final_layer.linear.bias", "2.weight", "2.bias"])


@pytest.mark.parametrize("ndim", [2, 3])
def test_segmentation_model_api(ndim, tmp_path):
    # reference tests/test_msd_segmentation_model.py:8-139
    from msd_pytorch_amd import MSDSegmentationModel
    torch.manual_seed(0)
    size = (20, 36) if ndim == 2 else (6, 8, 34)
    model = MSDSegmentationModel(1, 3, depth=5, width=1, dilations=[1, 2], ndim=ndim)
    labels = torch.randint(0, 3, (2, 1, *size))
    x = labels.float() + 0.1 * torch.randn(2, 1, *size)
    model.set_normalization([(x, labels)])
    losses = [model.learn(x, labels) for _ in range(10)]
    assert losses[-1] < losses[0]
    assert model.get_output().shape == (2, 3, *size)
    with pytest.raises(ValueError):
        model.set_target(labels + 3)
    with pytest.raises(ValueError):
        model.set_target(labels - 1)
    path = os.path.join(tmp_path, "seg.torch")
    model.save(path, 3)
    other = MSDSegmentationModel(1, 3, depth=5, width=1, dilations=[1, 2], ndim=ndim)
    assert other.load(path) == 3
    assert abs(other.forward(x, labels) - model.forward(x, labels)) < 1e-6
    assert any(k.startswith("1.0.msd_block.weight") for k in model.net.state_dict())


@pytest.mark.parametrize("shape,c_out,dtype", [
    ((2, 7, 13, 21), 3, torch.float32),        # ragged voxel count: one voxel per thread
    ((1, 101, 64, 64), 4, torch.float32),      # the stack of the headline network, 4 labels
    ((2, 5, 6, 7, 8), 1, torch.float32),
    ((1, 9, 8, 40), 11, torch.float32),        # more output channels than one launch takes (8 + 2 + 1)
    ((2, 6, 9, 10), 2, torch.float64),
    ((1, 3, 4, 6, 10), 5, torch.float64),
    # odd voxel counts (one voxel per thread) with every group width of output channels, both types
    ((1, 6, 7, 9), 13, torch.float32),         # 8 + 4 + 1
    ((1, 5, 3, 5, 7), 15, torch.float64),      # 8 + 4 + 2 + 1
    ((2, 4, 6, 10), 8, torch.float64),         # two voxels per thread, 8 output channels
])
def test_final_layer_matches_conv1d(shape, c_out, dtype):
    # the native final layer against the Conv1d over flattened voxels it replaces
    # (reference msd_module.py:60-88), in double precision
    from msd_pytorch_amd.msd_module import MSDFinalLayer
    gen = torch.Generator().manual_seed(3)
    b, c, *size = shape
    # the layer's input is a channel slice of a larger stack in the network
    stack = torch.randn(b, c + 2, *size, dtype=dtype, generator=gen).cuda()
    x = stack[:, :c].detach().requires_grad_(True)
    layer = MSDFinalLayer(c, c_out).to(dtype).cuda()
    layer.linear.weight.data.copy_(torch.randn(c_out, c, 1, dtype=dtype, generator=gen))
    layer.linear.bias.data.copy_(torch.randn(c_out, dtype=dtype, generator=gen))
    g = torch.randn(b, c_out, *size, dtype=dtype, generator=gen).cuda()
    out = layer(x)
    out.backward(g)

    xr = x.detach().double().requires_grad_(True)
    wr = layer.linear.weight.detach().double().requires_grad_(True)
    br = layer.linear.bias.detach().double().requires_grad_(True)
    ref = torch.nn.functional.conv1d(xr.reshape(b, c, -1), wr, br).view(b, c_out, *size)
    ref.backward(g.double())
    tf, tg = (1e-5, 1e-4) if dtype == torch.float32 else (1e-12, 1e-11)
    assert out.shape == ref.shape
    assert rel_err(out, ref) <= tf
    assert rel_err(x.grad, xr.grad) <= tg
    assert rel_err(layer.linear.weight.grad, wr.grad) <= tg
    assert rel_err(layer.linear.bias.grad, br.grad) <= tg


def test_final_layer_without_input_gradient():
    from msd_pytorch_amd.msd_module import MSDFinalLayer
    layer = MSDFinalLayer(4, 2).cuda()
    layer.linear.weight.data.normal_()
    x = torch.randn(1, 4, 16, 16, device="cuda")
    layer(x).sum().backward()
    want = x.sum(dim=(0, 2, 3))
    assert rel_err(layer.linear.weight.grad.view(2, 4)[0], want) <= 1e-4
    assert abs(layer.linear.bias.grad[0].item() - 256.0) <= 1e-2
