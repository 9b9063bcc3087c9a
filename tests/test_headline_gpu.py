"""The benchmark workloads at their real sizes against the CPU oracle: the dense blocks of
the two headline configurations (2D depth 100 at 1024 x 1024, 3D depth 50 at 128^3) and of
the batch configuration (2D depth 100, 4 x 512 x 512) and the small one (depth 10, 256 x 256),
forward and backward, and single layers at those image sizes with the channel counts the deep
layers have; of the two stress configurations (2D width 2 at 2048 x 2048, 3D at 256^3) single
layers at their own image sizes with the channel counts of their deep ends.  These are the
kernel instances that carry the benchmark: rows of 1024 (512, 128) voxels with more than 32
input channels select other template instances than small test images do.

Tolerances (max |diff| / max |ref|, fp32): forward 1e-5, gradients 1e-4."""
import pytest
import torch

from parity import check_block, check_operator_problem

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def cc():
    from msd_pytorch_amd import msd_custom_convolutions
    return msd_custom_convolutions


# (ndim, size, c_in, width, depth, batch)
HEADLINE_BLOCKS = {
    "C-2d-d100-1024x1024": (2, (1024, 1024), 1, 1, 100, 1),
    "D-3d-d50-128x128x128": (3, (128, 128, 128), 1, 1, 50, 1),
    "B-2d-d100-4x512x512": (2, (512, 512), 1, 1, 100, 4),
    "A-2d-d10-256x256": (2, (256, 256), 1, 1, 10, 1),
}


@pytest.mark.parametrize("name", list(HEADLINE_BLOCKS))
def test_headline_block_matches_oracle(name):
    # dilations 1..10 in turn, as in the benchmark (msd_module.py:122 of the reference)
    check_block(*HEADLINE_BLOCKS[name])


# Layers of the deep end of those blocks: channel counts on both sides of the blocks of 16
# input channels the weight gradient is computed in and of the chunks of 64 and 128 channels
# a launch takes; the smallest, a middle and the largest dilation of the workloads.
LAYERS_2D = [(batch, c, 1, size, d)
             for batch, size in ((1, (1024, 1024)), (4, (512, 512)))
             for c in (33, 64, 65, 100)
             for d in (1, 5, 10)]
LAYERS_3D = [(1, c, 1, (128, 128, 128), d) for c in (16, 17, 33, 50) for d in (1, 5, 10)]


def _id(s):
    return "B%d-C%d-%s-d%d" % (s[0], s[1], "x".join(map(str, s[3])), s[4])


@pytest.mark.parametrize("shape", LAYERS_2D + LAYERS_3D, ids=_id)
def test_headline_layer_matches_oracle(cc, shape):
    check_operator_problem(cc, shape, seed=11)


# The stress configurations at their own image sizes: one layer of the width-2 network at
# 2048 x 2048 with 130 input channels (rows of two segments, more than 128 channels) and one of
# the 3D network at 256^3 with 30, at the smallest and the largest dilation.  A problem is
# 2 x 2.2 GB on either side and an oracle call takes seconds, so the plain operators are run
# through the fused call only.
LAYERS_STRESS = [(1, 130, 2, (2048, 2048), 1), (1, 130, 2, (2048, 2048), 10),
                 (1, 30, 1, (256, 256, 256), 1), (1, 30, 1, (256, 256, 256), 10)]


@pytest.mark.parametrize("shape", LAYERS_STRESS, ids=_id)
def test_stress_layer_matches_oracle(cc, shape):
    import os
    need = 6 * (shape[1] + shape[2]) * 4
    for s in shape[3]:
        need *= s
    have = os.sysconf("SC_PAGE_SIZE") * os.sysconf("SC_PHYS_PAGES")
    if have < 2 * need:
        pytest.skip(f"host memory: {have >> 30} GiB, this problem wants {2 * need >> 30} GiB to be safe")
    check_operator_problem(cc, shape, seed=13, plain=False)
