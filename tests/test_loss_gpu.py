"""The final layer fused with the loss (msd_final_forward_loss) against torch in double
precision: output, loss value, the gradient handed to the backward pass and the layer's
parameter gradients, for the three losses of the reference's models (MSELoss and L1Loss of
msd_regression_model.py:5, LogSoftmax + NLLLoss of msd_segmentation_model.py:61-68), and the
models with and without the fused node.

Tolerances: fp32 values 1e-5 and gradients 1e-4 relative to the largest reference magnitude;
fp64 1e-11."""
import pytest
import torch
import torch.nn.functional as F

from cases import rel_err

pytestmark = pytest.mark.gpu


def reference(kind, x, w, b, target):
    """torch, double precision: (output, loss, d loss / d pre-activation, grad_w, grad_b)."""
    x, w, b = x.double(), w.double().requires_grad_(True), b.double().requires_grad_(True)
    pre = torch.einsum("oc,bc...->bo...", w, x) + b.view(1, -1, *([1] * (x.dim() - 2)))
    pre.retain_grad()
    if kind == "nll":
        out = F.log_softmax(pre, dim=1)
        loss = F.nll_loss(out, target)
    else:
        out = pre
        loss = F.mse_loss(out, target.double()) if kind == "mse" else F.l1_loss(out, target.double())
    loss.backward()
    return out.detach(), loss.detach(), pre.grad, w.grad, b.grad


CASES = [
    # (batch, c_in, c_out, spatial)
    (1, 7, 1, (33, 64)),
    (3, 12, 2, (17, 31)),          # odd plane size: one voxel per thread
    (2, 5, 4, (6, 10, 12)),
    (1, 21, 5, (40, 44)),
    (2, 3, 8, (5, 6, 8)),
    # odd plane sizes with 1, 4 and 8 output channels; an even one with 2
    (1, 4, 1, (7, 9)),
    (2, 6, 4, (3, 5, 7)),
    (1, 5, 8, (9, 11)),
    (1, 9, 2, (8, 12)),
    # more than 64 and more than 128 input channels (sixteen channels per wave; the walk-twice kernel),
    # several tiles per workgroup and a ragged last tile
    (1, 70, 4, (24, 50)),
    (2, 101, 4, (130, 258)),
    (1, 51, 1, (12, 40, 64)),
    (1, 130, 2, (16, 20)),
    (1, 33, 3, (700, 1030)),
]


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
@pytest.mark.parametrize("kind", ["mse", "l1", "nll"])
@pytest.mark.parametrize("batch,c_in,c_out,spatial", CASES)
def test_fused_loss_matches_torch(batch, c_in, c_out, spatial, kind, dtype):
    if dtype == torch.float64 and batch * c_in * spatial[0] * spatial[1] > 1 << 20:
        pytest.skip("the large cases are there for the fp32 kernels")
    check_fused_loss(batch, c_in, c_out, spatial, kind, dtype)


# One small case per compiled form of the single-read kernel: voxels per lane (4: plane size a
# multiple of four and at most 64 channels; 2: even planes otherwise; 1: odd planes) x channels
# per wave and pass (8 up to 64 channels, 16 above) x output channels (1, 2, 3 or 4) x loss.
SINGLE_READ_FORMS = [
    # (c_in, spatial)
    (20, (8, 16)),      # 4 voxels, 8 channels
    (20, (6, 7)),       # 2 voxels, 8 channels
    (20, (5, 7)),       # 1 voxel,  8 channels
    (70, (6, 8)),       # 2 voxels, 16 channels
    (70, (5, 7)),       # 1 voxel,  16 channels
]


@pytest.mark.parametrize("kind", ["mse", "l1", "nll"])
@pytest.mark.parametrize("c_out", [1, 2, 3])
@pytest.mark.parametrize("c_in,spatial", SINGLE_READ_FORMS)
def test_fused_loss_every_form_of_the_single_read_kernel(c_in, spatial, c_out, kind):
    check_fused_loss(2, c_in, c_out, spatial, kind, torch.float32)


@pytest.mark.parametrize("kind", ["mse", "l1", "nll"])
@pytest.mark.parametrize("batch,c_in,c_out,spatial", CASES)
def test_fused_loss_walking_the_stack_twice_matches_torch(batch, c_in, c_out, spatial, kind):
    # the kernel that reads the stack twice (what fp64, wide stacks and more than four output
    # channels take), forced for the shapes the single-read kernel would take
    from msd_pytorch_amd import _native
    lib = _native.load()
    assert lib.msd_set_tuning(b"final.tiled", 0) == 0
    try:
        check_fused_loss(batch, c_in, c_out, spatial, kind, torch.float32)
    finally:
        lib.msd_set_tuning(b"final.tiled", -1)


def test_fused_loss_is_reproducible():
    from msd_pytorch_amd import msd_custom_convolutions as cc
    gen = torch.Generator().manual_seed(9)
    x = torch.randn(2, 90, 64, 130, generator=gen).cuda()
    w, b = (torch.randn(4, 90, generator=gen) * 0.2).cuda(), torch.randn(4, generator=gen).cuda()
    t = torch.randint(0, 4, (2, 64, 130), generator=gen).cuda()
    runs = []
    for _ in range(3):
        gw, gb = torch.empty(4, 90, device="cuda"), torch.empty(4, device="cuda")
        out, loss, g = cc.final_forward_loss(x, w, b, "nll", t, gw, gb)
        runs.append((out.clone(), loss.clone(), g.clone(), gw, gb))
    for r in runs[1:]:
        assert all(torch.equal(a, b) for a, b in zip(r, runs[0]))


def check_fused_loss(batch, c_in, c_out, spatial, kind, dtype):
    from msd_pytorch_amd import msd_custom_convolutions as cc
    gen = torch.Generator().manual_seed(c_in * 100 + c_out)
    # the input is a channel slice of a larger stack, as the dense block hands it over
    stack = torch.randn(batch, c_in + 2, *spatial, generator=gen, dtype=dtype)
    x = stack[:, :c_in]
    w = torch.randn(c_out, c_in, generator=gen, dtype=dtype) * 0.3
    b = torch.randn(c_out, generator=gen, dtype=dtype)
    if kind == "nll":
        target = torch.randint(0, c_out, (batch, *spatial), generator=gen)
    else:
        target = torch.randn(batch, c_out, *spatial, generator=gen, dtype=dtype)
    want_out, want_loss, want_g, want_gw, want_gb = reference(kind, x, w, b, target)

    xd = stack.cuda()[:, :c_in]
    gw = torch.full((c_out, c_in), 7.0, dtype=dtype, device="cuda")      # overwritten, not accumulated into
    gb = torch.full((c_out,), 7.0, dtype=dtype, device="cuda")
    out, loss, g = cc.final_forward_loss(xd, w.cuda(), b.cuda(), kind, target.cuda(), gw, gb)
    tv, tg = (1e-5, 1e-4) if dtype == torch.float32 else (1e-11, 1e-11)
    assert rel_err(out, want_out) <= tv
    assert abs(loss.item() - want_loss.item()) <= tv * max(abs(want_loss.item()), 1e-30)
    assert rel_err(g, want_g) <= tg
    assert rel_err(gw, want_gw) <= tg and rel_err(gb, want_gb) <= tg
    # without parameter gradients: same values, and the stack gradient from g alone
    out2, loss2, g2 = cc.final_forward_loss(xd, w.cuda(), b.cuda(), kind, target.cuda())
    assert torch.equal(out2, out) and torch.equal(g2, g) and loss2.item() == loss.item()
    gx = torch.empty(batch, c_in, *spatial, dtype=dtype, device="cuda")
    cc.final_backward(None, g, w.cuda(), gx, None, None)
    want_gx = torch.einsum("oc,bo...->bc...", w.double(), want_g)
    assert rel_err(gx, want_gx) <= tg


def test_fused_loss_rejects_what_it_does_not_take():
    from msd_pytorch_amd import msd_custom_convolutions as cc
    x = torch.zeros(1, 3, 8, 8, device="cuda")
    with pytest.raises(RuntimeError, match="8 output channels"):
        cc.final_forward_loss(x, torch.zeros(9, 3, device="cuda"), None, "mse", torch.zeros(1, 9, 8, 8, device="cuda"))
    with pytest.raises(RuntimeError, match="int64 labels"):
        cc.final_forward_loss(x, torch.zeros(2, 3, device="cuda"), None, "nll", torch.zeros(1, 8, 8, device="cuda"))
    with pytest.raises(ValueError):
        cc.final_forward_loss(x, torch.zeros(2, 3, device="cuda"), None, "huber", torch.zeros(1, 2, 8, 8, device="cuda"))


def _grads(model):
    return {n: p.grad.clone() for n, p in model.net.named_parameters() if p.grad is not None}


@pytest.mark.parametrize("ndim,size", [(2, (40, 64)), (3, (8, 10, 32))])
@pytest.mark.parametrize("loss", ["L2", "L1"])
def test_regression_model_with_and_without_the_fused_loss(ndim, size, loss):
    from msd_pytorch_amd import MSDRegressionModel
    torch.manual_seed(3)
    model = MSDRegressionModel(2, 3, 7, 1, loss=loss, ndim=ndim)
    model.msd.final_layer.linear.weight.data.normal_(0, 0.1)
    model.msd.final_layer.linear.bias.data.normal_(0, 0.1)
    x = torch.rand(2, 2, *size)
    t = torch.randn(2, 3, *size)
    model.set_normalization([(x, t)])                      # non-trivial scaling layers
    results = []
    for fused in (True, False):
        model.fuse_loss = fused
        value = model.gradients(x, t)
        results.append((value, model.output.clone(), _grads(model)))
    (l1, o1, g1), (l0, o0, g0) = results
    assert type(model.loss.grad_fn).__name__ != "MSDNetLossFunctionBackward"      # the last run was unfused
    assert abs(l1 - l0) <= 1e-5 * abs(l0)
    assert rel_err(o1, o0) <= 1e-5
    assert set(g1) == set(g0) and len(g1) >= 9
    for name in g0:
        assert rel_err(g1[name], g0[name]) <= 1e-4, name
    model.fuse_loss = True
    model.forward(x, t)
    assert type(model.loss.grad_fn).__name__ == "MSDNetLossFunctionBackward"


@pytest.mark.parametrize("ndim,size", [(2, (40, 64)), (3, (8, 10, 32))])
def test_segmentation_model_with_and_without_the_fused_loss(ndim, size):
    from msd_pytorch_amd import MSDSegmentationModel
    torch.manual_seed(4)
    model = MSDSegmentationModel(1, 4, 6, 1, ndim=ndim)
    model.msd.final_layer.linear.weight.data.normal_(0, 0.2)
    x = torch.rand(2, 1, *size)
    t = torch.randint(0, 4, (2, 1, *size))
    results = []
    for fused in (True, False):
        model.fuse_loss = fused
        value = model.gradients(x, t)
        results.append((value, model.output.clone(), _grads(model)))
    (l1, o1, g1), (l0, o0, g0) = results
    assert abs(l1 - l0) <= 1e-5 * abs(l0)
    assert rel_err(o1, o0) <= 1e-5
    for name in g0:
        assert rel_err(g1[name], g0[name]) <= 1e-4, name
    # learning works through the fused node
    model.fuse_loss = True
    before = [p.detach().clone() for p in model.msd.parameters()]
    first = model.learn(x, t)
    for _ in range(5):
        last = model.learn(x, t)
    assert last < first
    assert all(not torch.equal(a, b) for a, b in zip(before, model.msd.parameters()))


def test_loss_gradient_scales_with_the_incoming_gradient():
    # (3 * loss).backward() must give three times the gradients
    from msd_pytorch_amd import MSDRegressionModel
    torch.manual_seed(5)
    model = MSDRegressionModel(1, 1, 4, 1)
    model.msd.final_layer.linear.weight.data.normal_(0, 0.1)
    x, t = torch.rand(1, 1, 32, 64), torch.rand(1, 1, 32, 64)
    model._launch_forward(x, t)
    model.optimizer.zero_grad()
    model.loss.backward(retain_graph=True)
    once = _grads(model)
    model.optimizer.zero_grad()
    (3 * model.loss).backward()
    for name, g in _grads(model).items():
        assert rel_err(g, 3 * once[name]) <= 1e-6, name


def test_a_hook_anywhere_in_the_net_switches_the_fused_loss_off():
    # forward hooks see a module's own call: with one on any module of `net` (here the outer
    # Sequential and the LogSoftmax, which the fused node never calls) the modules run one by one
    from msd_pytorch_amd import MSDSegmentationModel
    torch.manual_seed(6)
    model = MSDSegmentationModel(1, 3, 4, 1)
    model.msd.final_layer.linear.weight.data.normal_(0, 0.2)
    x, t = torch.rand(1, 1, 24, 64), torch.randint(0, 3, (1, 1, 24, 64))
    plain = model.forward(x, t)
    assert type(model.loss.grad_fn).__name__ == "MSDNetLossFunctionBackward"
    for module in (model.net, model.net[1][1], model.scale_in):
        seen = []
        handle = module.register_forward_hook(lambda m, i, o: seen.append(tuple(o.shape)))
        hooked = model.forward(x, t)
        handle.remove()
        assert seen == [(1, 1 if module is model.scale_in else 3, 24, 64)]
        assert type(model.loss.grad_fn).__name__ != "MSDNetLossFunctionBackward"
        assert abs(hooked - plain) <= 1e-5 * abs(plain)
    model.forward(x, t)
    assert type(model.loss.grad_fn).__name__ == "MSDNetLossFunctionBackward"
