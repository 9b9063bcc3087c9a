"""msd_conv_relu_backward_kb_static: the weight + bias gradient through the library's own
scratch buffer, for callers that cannot allocate device memory.  It runs the same kernels as
msd_conv_relu_backward_kb, so the results must be the same bits; the buffer keeps the last
call's contents, so a smaller problem is run right after a larger one."""
import ctypes

import pytest
import torch

from cases import make_problem

pytestmark = pytest.mark.gpu


def _i64(values):
    from msd_pytorch_amd import _native
    return _native.i64_array(tuple(values))


def _ptr(t):
    return ctypes.c_void_p(t.data_ptr() if t is not None else 0)


def _both(lib, p, with_bias=True):
    """grad_kernel and grad_bias from the entry point with a workspace and from the one
    without, both called through the C ABI, both accumulating into the same start values."""
    from msd_pytorch_amd import _native
    x, y, gy = p["x"], p["y"], p["gy"]
    dtype = _native.MSD_F32 if x.dtype == torch.float32 else _native.MSD_F64
    ndim = x.dim() - 2
    head = (dtype, ndim, x.shape[0], x.shape[1], y.shape[1], _i64(x.shape[2:]), p["d"])
    views = (_ptr(y), _i64(y.stride()), _ptr(gy), _i64(gy.stride()), _ptr(x), _i64(x.stride()))
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    need = lib.msd_workspace_bytes(dtype, ndim, x.shape[0], x.shape[1], y.shape[1], _i64(x.shape[2:]))
    assert 0 < need <= _native.STATIC_SCRATCH_BYTES
    ws = torch.empty(need, dtype=torch.uint8, device="cuda")
    out = []
    for static in (False, True):
        gk = torch.full_like(p["k"], 0.5)
        gb = torch.full_like(p["bias"], -2.0) if with_bias else None
        if static:
            rc = lib.msd_conv_relu_backward_kb_static(*head, *views, _ptr(gk), _ptr(gb), stream)
        else:
            rc = lib.msd_conv_relu_backward_kb(*head, *views, _ptr(gk), _ptr(gb), _ptr(ws), need, stream)
        assert rc == 0, lib.msd_last_error().decode()
        torch.cuda.synchronize()
        out.append((gk, gb))
    return out


# a larger problem first, then smaller ones: matrix-core row kernel (2D, 3D), the variant
# with a plane-sized masked gradient in the scratch (rows that are not whole groups of four
# voxels fall to it or to the shape-generic kernel), fp64 on the shape-generic kernel
SEQUENCE = [
    ((2, 40, 2, (96, 512), 3), torch.float32),
    ((1, 7, 1, (33, 128), 2), torch.float32),
    ((1, 19, 1, (12, 20, 128), 2), torch.float32),
    ((1, 3, 1, (5, 6, 64), 1), torch.float32),
    ((1, 5, 1, (40, 2052), 4), torch.float32),
    ((2, 3, 2, (9, 77), 5), torch.float32),
    ((1, 6, 2, (20, 50), 3), torch.float64),
    ((1, 2, 1, (4, 5, 6), 2), torch.float64),
]


def test_static_scratch_gives_the_same_bits_call_after_call():
    from msd_pytorch_amd import _native
    from msd_pytorch_amd import msd_custom_convolutions as cc
    lib = _native.load()
    for i, (shape, dtype) in enumerate(SEQUENCE):
        p = make_problem(shape, dtype, device="cuda", seed=20 + i)
        cc.conv_relu_forward(p["x"], p["k"], p["bias"], p["y"], p["d"])
        (gk0, gb0), (gk1, gb1) = _both(lib, p)
        assert torch.equal(gk0, gk1), (shape, "grad_kernel")
        assert torch.equal(gb0, gb1), (shape, "grad_bias")
        assert float((gk1 - 0.5).abs().max()) > 0
        (gk0, _), (gk1, _) = _both(lib, p, with_bias=False)
        assert torch.equal(gk0, gk1), (shape, "grad_kernel without bias")


def test_static_scratch_matches_the_oracle_and_the_python_wrapper():
    import oracle
    from cases import rel_err
    from msd_pytorch_amd import msd_custom_convolutions as cc
    for shape in ((1, 21, 1, (64, 256), 5), (1, 4, 1, (9, 10, 68), 3)):
        ref = make_problem(shape, torch.float32, seed=3)
        dev = make_problem(shape, torch.float32, device="cuda", seed=3)
        oracle.conv_relu_forward(ref["x"], ref["k"], ref["bias"], ref["y"], ref["d"])
        dev["y"].copy_(ref["y"])
        want_gk, want_gb = torch.zeros_like(ref["k"]), torch.zeros_like(ref["bias"])
        oracle.conv_relu_backward_k(ref["y"], ref["gy"], ref["x"], want_gk, ref["d"])
        oracle.conv_relu_backward_bias(ref["y"], ref["gy"], want_gb)
        gk, gb = torch.zeros_like(dev["k"]), torch.zeros_like(dev["bias"])
        cc.conv_relu_backward_kb_static(dev["y"], dev["gy"], dev["x"], gk, gb, dev["d"])
        assert rel_err(gk, want_gk) <= 1e-4 and rel_err(gb, want_gb) <= 1e-4


def _static_call(lib, p, gk, gb):
    from msd_pytorch_amd import _native
    x, y, gy = p["x"], p["y"], p["gy"]
    ndim = x.dim() - 2
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    rc = lib.msd_conv_relu_backward_kb_static(
        _native.MSD_F32, ndim, x.shape[0], x.shape[1], y.shape[1], _i64(x.shape[2:]), p["d"], _ptr(y), _i64(y.stride()),
        _ptr(gy), _i64(gy.stride()), _ptr(x), _i64(x.stride()), _ptr(gk), _ptr(gb), stream)
    assert rc == 0, lib.msd_last_error().decode()


@pytest.mark.parametrize("shape", [(1, 19, 1, (48, 512), 3), (1, 9, 1, (10, 12, 128), 2)])
def test_static_scratch_allocates_nothing_and_can_be_captured(shape):
    # what the entry point is for: no device memory is taken by a call (free bytes of the
    # device unchanged across raw C-ABI calls), and once the first call on the device has
    # looked the buffer's address up, a call can be recorded into a HIP graph; every replay
    # (with eager work between the replays) gives the bits of the eager call
    from msd_pytorch_amd import _native
    from msd_pytorch_amd import msd_custom_convolutions as cc
    lib = _native.load()
    p = make_problem(shape, torch.float32, device="cuda", seed=41)
    cc.conv_relu_forward(p["x"], p["k"], p["bias"], p["y"], p["d"])
    gk, gb = torch.zeros_like(p["k"]), torch.zeros_like(p["bias"])
    _static_call(lib, p, gk, gb)                       # first call: looks the address up
    torch.cuda.synchronize()
    want_gk, want_gb = gk.clone(), gb.clone()
    free_before = torch.cuda.mem_get_info()[0]
    for _ in range(3):
        gk.zero_(), gb.zero_()
        _static_call(lib, p, gk, gb)
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free_before
    assert torch.equal(gk, want_gk) and torch.equal(gb, want_gb)

    graph = torch.cuda.CUDAGraph()
    gk.zero_(), gb.zero_()
    torch.cuda.synchronize()
    with torch.cuda.graph(graph):
        _static_call(lib, p, gk, gb)                   # accumulates into gk, gb
    for replay in range(3):
        gk.zero_(), gb.zero_()
        other = make_problem((1, 3, 1, (20, 64), 1), torch.float32, device="cuda", seed=50 + replay)
        cc.conv_relu_forward(other["x"], other["k"], other["bias"], other["y"], other["d"])
        ogk, ogb = torch.zeros_like(other["k"]), torch.zeros_like(other["bias"])
        _static_call(lib, other, ogk, ogb)             # eager work through the same buffer in between
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(gk, want_gk) and torch.equal(gb, want_gb), replay


def test_static_scratch_rejects_what_does_not_fit():
    from msd_pytorch_amd import _native
    from msd_pytorch_amd import msd_custom_convolutions as cc
    lib = _native.load()
    # 256^3: the masked-gradient plane alone is 64 MiB
    spatial = (256, 256, 256)
    assert lib.msd_workspace_bytes(0, 3, 1, 2, 1, _i64(spatial)) > _native.STATIC_SCRATCH_BYTES
    x = torch.zeros(1, 2, *spatial, device="cuda")
    y = torch.zeros(1, 1, *spatial, device="cuda")
    gk = torch.zeros(1, 2, 3, 3, 3, device="cuda")
    with pytest.raises(RuntimeError, match="static buffer"):
        cc.conv_relu_backward_kb_static(y, y, x, gk, None, 1)
    assert float(gk.abs().max()) == 0
