"""Every launch-shape setting of msd_set_tuning against the CPU oracle.

The library picks voxels per lane, rows per forward tile, channel groups, tile numbering and
workgroup order by image size; each choice is a different template instance or code path, and
some are reached by default only at particular sizes.  Here every setting is forced in turn on
problems small enough for the oracle, so that each instance meets the oracle at least once
whatever the defaults are.  Results may only differ in floating-point summation order:
tolerances forward 1e-5, gradients 1e-4 (fp32)."""
import itertools

import pytest
import torch

from cases import rel_err
from parity import check_block, check_operator_problem

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def cc():
    from msd_pytorch_amd import msd_custom_convolutions
    return msd_custom_convolutions


class tuning:
    """Sets the given knobs for the duration of a with-block, then restores the defaults."""

    def __init__(self, settings):
        from msd_pytorch_amd import _native
        self.lib = _native.load()
        self.settings = settings

    def __enter__(self):
        for key, value in self.settings.items():
            assert self.lib.msd_set_tuning(key.encode(), value) == 0, key
        return self

    def __exit__(self, *exc):
        for key in self.settings:
            self.lib.msd_set_tuning(key.encode(), -1)
        return False


# (B, C_in, C_out, spatial, dilation)
IMG_A = (1, 5, 1, (23, 256), 3)          # rows of 256: 64 lanes at 4 voxels per lane
IMG_B = (2, 18, 1, (9, 1024), 7)         # one row per workgroup, two blocks of 16 channels, folds in y
IMG_C = (1, 35, 2, (12, 512), 5)         # two output channels, three channel blocks
IMG_D = (1, 3, 1, (70, 128), 1)          # dilation 1, many row groups
VOL_A = (1, 6, 1, (7, 9, 128), 2)
VOL_B = (1, 19, 1, (5, 6, 256), 3)       # rows of 256: up to 4 voxels per lane in the forward pass
VOL_C = (2, 4, 2, (6, 7, 128), 1)        # two output channels
VOL_D = (1, 3, 1, (40, 40, 64), 1)       # more than 128 lattices per residue class: tiles in 4 x 4 blocks
VOL_E = (1, 17, 1, (24, 20, 64), 3)      # lattices of 3 x 3 rows

FORWARD_2D = [({"fwd.rows2d": r, "fwd.vec2d": v}, s)
              for r, v in itertools.product((2, 3, 4, 5, 6), (1, 2, 4)) for s in (IMG_A, IMG_B)]
FORWARD_2D += [({"fwd.vec2d": v}, IMG_C) for v in (1, 2, 4)]
FORWARD_3D = [({"fwd.vec3d": v}, s) for v in (1, 2, 4) for s in (VOL_A, VOL_B, VOL_C)]
FORWARD_3D += [({"fwd.class3d": c}, s) for c in (0, 1) for s in (VOL_A, VOL_D, VOL_E)]
FORWARD_3D += [({"fwd.lattice3d": m}, s) for m in (24, 33, 44) for s in (VOL_A, VOL_D, VOL_E)]
FORWARD_3D += [({"fwd.lattice3d": 44, "fwd.split": k}, VOL_E) for k in (1, 4)]
SPLIT = [({"fwd.split": k}, s) for k in (1, 2, 4) for s in (IMG_A, IMG_C, VOL_A, VOL_C)]
ORDER = [({"xcd_remap": r}, s) for r in (0, 1) for s in (IMG_B, IMG_D, VOL_A, VOL_D)]
BACKWARD_K = [({"bwdk.vec2d": v}, s) for v in (1, 2, 4) for s in (IMG_A, IMG_B, IMG_C)]
# ("bwdk.fused3d": 0 keeps a 3D layer of one or two output channels on the kernels that these
# parameters shape; by default it goes through the weight-gradient-only form of the fused kernel)
BACKWARD_K += [({"bwdk.vec3d": v, "bwdk.fused3d": 0}, s) for v in (1, 2) for s in (VOL_A, VOL_B)]
BACKWARD_K += [({"bwdk.fused3d": f}, s) for f in (0, 1) for s in (VOL_A, VOL_B, VOL_C, VOL_D, VOL_E)]
BACKWARD_K += [({"bwdk.rows": r, "bwdk.fused3d": 0}, s) for r in (0, 1) for s in (IMG_A, IMG_B, VOL_A)]
BACKWARD_K += [({"bwdk.rows": 0, "bwdk.vec2d": v}, IMG_B) for v in (2, 4)]
BACKWARD_K += [({"bwdk.interleave": i, "bwdk.fused3d": f}, s) for i in (0, 1) for f in (0, 1) for s in (IMG_D, VOL_D)]
BACKWARD_K += [({"bwdk.blocks": n, "bwdk.fused3d": f}, s) for n in (8, 40) for f in (0, 1) for s in (IMG_D, VOL_A)]
BACKWARD_X = [({"bwdx.vec2d": v, "bwdx.unroll2d": u}, s) for v in (1, 2, 4) for u in (2, 4) for s in (IMG_A, IMG_C)]
BACKWARD_X += [({"bwdx.vec3d": v, "bwdx.unroll3d": u}, s) for v in (1, 2, 4) for u in (2, 4) for s in (VOL_B, VOL_C)]
BACKWARD_X += [({"bwdx.min_blocks": n}, s) for n in (1, 4096) for s in (IMG_B, VOL_B)]


# Template instances of the one-pass backward kernel that neither the cases above nor the
# other test files reach: (voxels per lane, blocks of 16 channels per launch, output channels,
# variant for unaligned or long rows) chosen by row length, channel count and width.
INSTANCES = [
    ({}, (1, 40, 1, (6, 1001), 3)),                  # odd rows: one voxel per lane, 33-64 channels
    ({"bwdk.vec2d": 1}, (1, 70, 2, (8, 128), 2)),    # one voxel per lane, two output channels, > 64 channels
    ({}, (1, 9, 2, (9, 256), 2)),                    # two voxels per lane, two output channels, one block
    ({}, (1, 20, 1, (6, 750), 2)),                   # rows of whole pairs only: two voxels per lane, two blocks
    ({}, (1, 20, 2, (9, 256), 3)),
    ({"bwdk.vec2d": 2}, (1, 40, 1, (9, 256), 2)),
    ({}, (1, 40, 1, (6, 750), 2)),
    ({}, (1, 40, 2, (5, 1022), 4)),
    ({"bwdk.vec2d": 2}, (1, 70, 1, (9, 256), 2)),
    ({}, (1, 70, 2, (9, 256), 3)),
    ({}, (1, 70, 2, (5, 1022), 4)),
    ({}, (1, 40, 1, (5, 2048), 3)),                  # rows of two segments, 33-64 channels
    ({}, (1, 70, 1, (5, 6, 64), 2)),                 # 3D, more than 64 channels
    ({"bwdk.rows": 0, "bwdk.vec2d": 2}, (1, 40, 1, (9, 256), 2)),
    ({"bwdk.rows": 0, "bwdk.vec2d": 2}, (1, 70, 1, (9, 256), 2)),
    ({"bwdk.rows": 0, "bwdk.vec2d": 2}, (1, 3, 1, (9, 256), 2)),
    ({"bwdk.rows": 0, "bwdk.vec2d": 4}, (1, 40, 1, (9, 256), 2)),
    ({"bwdk.rows": 0, "bwdk.vec3d": 2, "bwdk.fused3d": 0}, (1, 40, 1, (5, 6, 128), 2)),
    ({"bwdk.rows": 0, "bwdk.vec3d": 4, "bwdk.fused3d": 0}, (1, 3, 1, (5, 6, 128), 2)),
    ({"bwdk.rows": 0, "bwdk.vec3d": 4, "bwdk.fused3d": 0}, (1, 20, 1, (5, 6, 128), 2)),
    ({"bwdk.rows": 0, "bwdk.vec3d": 4, "bwdk.fused3d": 0}, (1, 40, 1, (5, 6, 128), 2)),
    ({"bwdk.rows": 0, "bwdk.vec3d": 4, "bwdk.fused3d": 0}, (1, 70, 1, (5, 6, 128), 2)),
    ({"bwdk.vec2d": 1}, (1, 40, 1, (9, 128), 2)),
    ({"bwdk.vec2d": 1}, (1, 70, 1, (9, 128), 2)),   # one voxel per lane, one output channel, > 64 channels
    ({"bwdk.vec2d": 2}, (1, 70, 1, (9, 128), 2)),
    ({"bwdk.vec2d": 4}, (1, 70, 1, (9, 256), 2)),
    ({"bwdk.vec3d": 1, "bwdk.fused3d": 0}, (1, 20, 1, (5, 6, 64), 2)),
    ({"bwdk.vec3d": 1, "bwdk.fused3d": 0}, (1, 40, 1, (5, 6, 64), 2)),
    ({"bwdk.vec3d": 2, "bwdk.fused3d": 0}, (1, 40, 1, (5, 6, 128), 2)),
    ({"bwdk.vec3d": 2, "bwdk.fused3d": 0}, (1, 70, 1, (5, 6, 128), 2)),
    ({"bwdx.vec2d": 4, "bwdx.unroll2d": 4}, (1, 5, 1, (4, 2048), 3)),     # rows of 512 lanes
    ({"bwdx.vec2d": 4, "bwdx.unroll2d": 4}, (1, 5, 2, (4, 2048), 3)),
    ({"bwdx.vec3d": 4, "bwdx.unroll3d": 2}, (1, 5, 1, (3, 4, 2048), 3)),
    ({"bwdx.vec3d": 4, "bwdx.unroll3d": 4}, (1, 5, 2, (3, 4, 2048), 3)),
    ({"bwdx.vec3d": 2, "bwdx.unroll3d": 2}, (1, 5, 1, (5, 6, 128), 2)),
    ({"bwdx.vec3d": 1, "bwdx.unroll3d": 4}, (1, 5, 1, (5, 6, 128), 2)),
    ({"fwd.vec3d": 2}, (1, 6, 1, (5, 6, 256), 2)),
    ({"fwd.vec3d": 4}, (1, 6, 2, (5, 6, 256), 2)),
    ({"fwd.vec3d": 2}, (1, 6, 2, (5, 6, 256), 2)),
    ({"fwd.vec2d": 1}, (1, 6, 2, (9, 128), 2)),
    ({"bwdk.vec2d": 2}, (1, 9, 2, (9, 256), 2)),
    ({"bwdk.vec2d": 2}, (1, 70, 2, (9, 256), 3)),
    ({"bwdk.vec2d": 2}, (1, 20, 2, (9, 256), 3)),
    ({"bwdk.vec2d": 1}, (1, 20, 1, (9, 128), 2)),
    ({"bwdx.vec2d": 1, "bwdx.unroll2d": 4}, (1, 6, 2, (9, 128), 2)),
    ({"bwdx.vec3d": 4, "bwdx.unroll3d": 2}, (1, 5, 1, (3, 4, 1536), 3)),   # 3D rows of 384 lanes
    ({"bwdx.vec3d": 4, "bwdx.unroll3d": 4}, (1, 5, 1, (3, 4, 1536), 3)),
    ({"bwdx.vec3d": 4, "bwdx.unroll3d": 4}, (1, 5, 2, (3, 4, 768), 3)),
    # two output channels, rows cut into segments but otherwise like the plain kernel's (whole
    # groups of four voxels, aligned): the segment-only instances, by channel blocks and voxels per lane
    ({}, (1, 9, 2, (5, 1280), 3)),
    ({}, (1, 20, 2, (8, 1280), 7)),
    ({}, (1, 40, 2, (4, 1280), 2)),
    ({}, (1, 70, 2, (6, 1280), 5)),
    ({}, (2, 20, 2, (10, 4096), 9)),
    ({"bwdk.vec2d": 2}, (1, 9, 2, (5, 1280), 3)),
    ({"bwdk.vec2d": 2}, (1, 20, 2, (8, 1280), 7)),
    ({"bwdk.vec2d": 2}, (1, 40, 2, (4, 1280), 2)),
    ({"bwdk.vec2d": 2}, (1, 70, 2, (6, 1280), 5)),
    ({"bwdk.vec2d": 1}, (1, 9, 2, (5, 1280), 3)),
    ({"bwdk.vec2d": 1}, (1, 20, 2, (8, 1280), 7)),
    ({"bwdk.vec2d": 1}, (1, 40, 2, (4, 1280), 2)),
    ({"bwdk.vec2d": 1}, (1, 70, 2, (6, 1280), 5)),
    ({}, (1, 20, 2, (5, 1026), 3)),                  # long rows of whole pairs only: the full LONG instance, two blocks
    # two output channels at four voxels per lane (the waves' tiles lie over the staged rows in
    # LDS): rows of one to four waves, one to four rows per workgroup, by channel blocks
    ({}, (1, 9, 2, (5, 1024), 3)),
    ({}, (2, 20, 2, (7, 1024), 6)),
    ({}, (1, 40, 2, (4, 768), 2)),
    ({}, (1, 70, 2, (6, 1024), 5)),
    ({"bwdk.vec2d": 4}, (1, 20, 2, (9, 512), 8)),
    ({"bwdk.vec2d": 4}, (2, 40, 2, (10, 256), 1)),
    ({"bwdk.vec2d": 4}, (1, 100, 2, (13, 256), 12)),
    # three output channels in one fused pass (rows of whole groups of four voxels): rows that
    # one workgroup covers (one to four rows each, lanes past the row's end) and rows in
    # segments; one, two and four channel blocks per chunk, more than one chunk
    ({}, (1, 9, 3, (7, 512), 3)),
    ({}, (2, 20, 3, (9, 256), 8)),
    ({}, (1, 40, 3, (5, 384), 2)),
    ({}, (1, 100, 3, (6, 512), 5)),
    ({}, (1, 9, 3, (7, 192), 3)),
    ({}, (2, 40, 3, (5, 64), 2)),
    ({}, (1, 70, 3, (6, 100), 5)),
    ({}, (1, 9, 3, (7, 1024), 3)),
    ({}, (2, 20, 3, (9, 1280), 8)),
    ({}, (1, 40, 3, (5, 2048), 2)),
    ({}, (1, 130, 3, (6, 1024), 5)),
    ({}, (1, 20, 3, (7, 1026), 3)),                  # not covered by the fused kernel: two passes
    # 3D rows of 257 to 512 voxels: the fused backward at two voxels per lane (tiles over the
    # staged rows), by channel blocks
    ({}, (1, 9, 1, (3, 4, 512), 3)),
    ({}, (2, 20, 1, (4, 3, 384), 2)),
    ({}, (1, 40, 1, (3, 5, 512), 1)),
    ({}, (1, 70, 1, (2, 4, 512), 2)),
    ({"bwdk.vec3d": 2, "bwdk.fused3d": 0}, (1, 20, 1, (5, 6, 128), 2)),
    ({}, (1, 40, 1, (4, 5, 130), 2)),                # 3D rows that are not whole groups of four voxels, 33-64 channels
]


def _id(case):
    settings, s = case
    knobs = ",".join("%s=%d" % kv for kv in settings.items())
    return "%s-B%d-C%d-w%d-%s-d%d" % (knobs, s[0], s[1], s[2], "x".join(map(str, s[3])), s[4])


# 3D, one input and one output channel: the lean backward_x kernel at four, two and one voxel
# per lane, and the general kernel on the same shapes
INSTANCES += [(settings, shape) for settings in ({}, {"bwdx.lean1": 0})
              for shape in ((2, 1, 1, (5, 6, 128), 2), (1, 1, 1, (4, 5, 66), 3), (1, 1, 1, (3, 5, 33), 1),
                            (1, 1, 1, (6, 7, 256), 6))]
# the 3D entries without a setting of their own once more on the separate weight-gradient kernels
INSTANCES += [({"bwdk.fused3d": 0}, shape) for settings, shape in INSTANCES if not settings and len(shape[3]) == 3]


@pytest.mark.parametrize("case", FORWARD_2D + FORWARD_3D + SPLIT + ORDER + BACKWARD_K + BACKWARD_X + INSTANCES,
                         ids=_id)
def test_operators_under_a_forced_setting(cc, case):
    settings, shape = case
    with tuning(settings):
        check_operator_problem(cc, shape, seed=3)


BLOCK_SETTINGS = [{"block.snake": 0}, {"block.snake": 1}, {"block.fuse": 0}, {"block.defer": 0},
                  {"xcd_remap": 0}, {"bwdk.interleave": 0}, {"fwd.class3d": 0}, {"fwd.lattice3d": 44},
                  {"block.pair": 0}, {"block.pair": 1}, {"block.pair": 1, "block.defer": 0},
                  {"block.pair": 1, "block.snake": 0}, {"block.triple": 1}, {"block.triple": 0},
                  {"block.triple": 1, "block.defer": 0}, {"block.triple": 1, "block.snake": 0}]


@pytest.mark.parametrize("settings", BLOCK_SETTINGS, ids=lambda s: ",".join("%s=%d" % kv for kv in s.items()))
@pytest.mark.parametrize("ndim,size", [(2, (21, 256)), (3, (6, 9, 128))])
def test_block_under_a_forced_setting(ndim, size, settings):
    with tuning(settings):
        check_block(ndim, size, 2, 1, 19, 2)


# The backward pass of a 2D block of one-channel layers takes the layers two at a time (the
# pair's second launch gathers two output gradients with two dilations in one pass over the
# channels both layers read).  Cases: equal and very different dilations in a pair, dilations
# that fold on both sides of a small image, odd and even depths (a layer left over at the
# bottom), more than one input channel, rows that one workgroup covers (256, 512 voxels), rows
# cut into segments (1280, 2050: not a multiple of four), rows of 768 and 1024 voxels (four per
# lane) and short odd rows.
PAIR_BLOCKS = [
    # (size, c_in, depth, batch, dilations)
    ((21, 256), 1, 6, 2, [1, 10, 2, 9, 3, 8]),
    ((21, 256), 3, 7, 1, [5, 5, 5, 1, 1, 7, 2]),
    ((12, 512), 2, 5, 1, [12, 1, 11, 2, 6]),
    ((9, 1280), 1, 6, 1, [1, 4, 9, 2, 3, 7]),
    ((7, 2050), 1, 4, 1, [3, 1, 6, 2]),
    ((11, 1024), 1, 7, 1, [1, 10, 2, 9, 3, 8, 4]),  # four voxels per lane in the pair's pass
    ((6, 768), 2, 4, 2, [5, 1, 2, 5]),
    ((33, 70), 2, 9, 2, [1, 2, 3, 4, 5, 6, 7, 8, 9]),
    ((20, 255), 1, 5, 1, [2, 7, 1, 4, 3]),          # odd rows: one voxel per lane in the one-channel step
    ((40, 64), 1, 20, 1, None),
    ((10, 384), 1, 7, 1, [3, 1, 4, 1, 5, 9, 2]),    # two voxels per lane in the one-channel steps
    ((9, 192), 2, 6, 1, [1, 3, 2, 4, 1, 2]),        # one voxel per lane in the one-channel steps
    ((8, 1280), 40, 6, 1, [2, 7, 1, 8, 2, 8]),      # three layers over more than 32 channels (the default's threshold)
    ((6, 512), 70, 3, 2, [6, 1, 3]),                # three layers, channels in two chunks of the grid
]

# "triples": three layers at a time wherever the kernels cover it (by default only where the
# layers share at least 32 channels), two or one where they do not or where fewer are left
GROUPINGS = {"triples": {"block.triple": 1}, "pairs": {"block.triple": 0}, "default": {}, "single": {"block.pair": 0}}


@pytest.mark.parametrize("grouping", list(GROUPINGS))
@pytest.mark.parametrize("case", PAIR_BLOCKS, ids=lambda c: "x".join(map(str, c[0])) + "-d%d" % c[2])
def test_block_backward_two_or_three_layers_at_a_time(case, grouping):
    size, c_in, depth, batch, dilations = case
    with tuning(GROUPINGS[grouping]):
        check_block(2, size, c_in, 1, depth, batch, dilations=dilations, seed=11)


def _random_one_channel_blocks(n):
    from test_random_shapes_gpu import _block_cases
    return [c for c in _block_cases(4242, 80) if c[0] == 2 and c[3] == 1 and c[4] >= 5][:n]


@pytest.mark.parametrize("case", _random_one_channel_blocks(12), ids=lambda c: "%s-c%d-depth%d-B%d" % (
    "x".join(map(str, c[1])), c[2], c[4], c[5]))
def test_random_blocks_three_layers_at_a_time(case):
    # seeded random 2D blocks of one-channel layers (ragged and odd rows among them: where the
    # three-layer kernels do not apply the walk falls back to two layers or one)
    import test_random_shapes_gpu
    with tuning({"block.triple": 1}):
        test_random_shapes_gpu.test_random_blocks(case)


def test_paired_and_single_backward_agree_when_the_input_needs_no_gradient():
    # the model path: the block's input is data, so the lowest layer takes the weight-gradient
    # kernel alone and the pairs start one layer higher
    from msd_pytorch_amd.msd_block import msd_block
    from parity import block_problem
    from cases import rel_err
    x, dil, bias, ws, g = block_problem(2, (19, 384), 1, 1, 8, 2, seed=5)
    grads = {}
    for pair in (0, 1, 3):
        with tuning({"block.pair": 0} if pair == 0 else {"block.triple": int(pair == 3)}):
            bd = bias.cuda().requires_grad_(True)
            wd = [w.cuda().requires_grad_(True) for w in ws]
            out = msd_block(x.cuda(), dil, bd, *wd)
            out.backward(g.cuda())
            torch.cuda.synchronize()
            grads[pair] = [bd.grad.clone()] + [w.grad.clone() for w in wd]
    for a, b, c in zip(grads[0], grads[1], grads[3]):
        assert rel_err(a, b) <= 1e-5 and rel_err(a, c) <= 1e-5


# 3D blocks of one-channel layers: the reverse loop as a chain of backward_x launches with the
# weight gradients two layers per pass beside it ("block.split3d": on a second stream, on the
# caller's stream, or off = one fused launch per layer).  (size, c_in, depth, batch, dilations)
SPLIT_BLOCKS_3D = [
    ((6, 7, 64), 1, 6, 1, [1, 2, 3]),            # even depth: pairs down to layers (1, 0)
    ((5, 9, 128), 2, 7, 2, [3, 1, 2, 5]),        # odd depth: the lowest layer on its own; batch of 2
    ((12, 10, 128), 1, 9, 1, [10, 1, 7, 2]),     # dilations up to the extents: every row folds
    ((4, 6, 256), 3, 4, 1, [2, 1]),              # rows of 256 voxels: one row per workgroup
    ((9, 8, 64), 15, 5, 1, [1, 4, 2]),           # 16 to 20 channels: two blocks of 16 in the upper pairs
    ((6, 6, 64), 62, 5, 1, [2, 3]),              # 63 to 67 channels: two chunks of the grid
    ((7, 5, 96), 1, 5, 1, [1, 2]),               # rows the row kernels take with half-empty waves
    ((24, 128, 128), 42, 6, 1, [1, 10, 3, 7, 5, 2]),   # the headline volume's rows, 43 to 47 channels
]
SPLIT_MODES = {"two-streams": {"block.split3d": 1}, "one-stream": {"block.split3d": 2}, "fused": {"block.split3d": 0},
               "default": {}, "chain-of-single-layers": {"block.split3d": 1, "block.chainpair": 0}}


@pytest.mark.parametrize("mode", list(SPLIT_MODES))
@pytest.mark.parametrize("case", SPLIT_BLOCKS_3D, ids=lambda c: "x".join(map(str, c[0])) + "-c%d-d%d" % (c[1], c[2]))
def test_block_backward_3d_chain_and_paired_weight_gradients(case, mode):
    size, c_in, depth, batch, dilations = case
    dilations = [dilations[i % len(dilations)] for i in range(depth)]
    with tuning(SPLIT_MODES[mode]):
        check_block(3, size, c_in, 1, depth, batch, dilations=dilations, seed=17)


# The chain's two-layer pass by voxels per lane and channels in flight (rows of 128 voxels take
# any of the three widths).
@pytest.mark.parametrize("unroll", [2, 4])
@pytest.mark.parametrize("vec", [1, 2, 4])
def test_block_backward_3d_paired_chain_by_vector_width(vec, unroll):
    with tuning({"block.split3d": 1, "bwdx.vec3d": vec, "bwdx.unroll3d": unroll}):
        check_block(3, (6, 5, 128), 2, 1, 7, 1, dilations=[2, 1, 3, 1, 5, 2, 4], seed=29)
        check_block(3, (4, 9, 128), 1, 1, 4, 2, dilations=[1, 3, 2, 4], seed=31)


def test_block_backward_3d_without_input_gradient():
    # the lowest pair then skips its pass over the block's input channels
    for depth in (4, 5):
        with tuning({"block.split3d": 1}):
            check_block(3, (5, 6, 64), 2, 1, depth, 1, dilations=[1, 2, 3, 1, 2][:depth], seed=37, input_grad=False)


def test_block_backward_3d_modes_give_the_same_bits_run_after_run():
    # the second stream changes when things run, not what is added in which order: run after run
    # the bits are the same.  On one stream the weight-gradient passes use more workgroups (more
    # partial sums per column): the same sums in another grouping.
    from msd_pytorch_amd.msd_block import msd_block
    from parity import block_problem
    x, dil, bias, ws, g = block_problem(3, (10, 12, 128), 1, 1, 8, 1, seed=23)
    runs = []
    for mode in ("two-streams", "two-streams", "one-stream", "one-stream"):
        with tuning(SPLIT_MODES[mode]):
            xd = x.cuda().requires_grad_(True)
            bd = bias.cuda().requires_grad_(True)
            wd = [w.cuda().requires_grad_(True) for w in ws]
            msd_block(xd, dil, bd, *wd).backward(g.cuda())
            torch.cuda.synchronize()
            runs.append([xd.grad.clone(), bd.grad.clone()] + [w.grad.clone() for w in wd])
    assert all(torch.equal(a, b) for a, b in zip(runs[0], runs[1]))
    assert all(torch.equal(a, b) for a, b in zip(runs[2], runs[3]))
    assert torch.equal(runs[0][0], runs[2][0])              # grad_input: the same launches
    assert all(rel_err(a, b) <= 1e-5 for a, b in zip(runs[0], runs[2]))
