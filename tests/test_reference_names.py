"""The reference's import names resolve to this implementation (msd_pytorch/__init__.py:21-25,
examples/getting_started.py:4, the import lines of msd_pytorch/tests/*.py)."""
import importlib

import pytest

SUBMODULES = ["conv2d", "conv3d", "msd_block", "msd_module", "msd_model", "msd_regression_model",
              "msd_segmentation_model", "image_dataset", "errors", "bench"]


def test_package_name_of_the_reference_imports():
    import msd_pytorch as mp
    import msd_pytorch_amd
    assert mp.MSDRegressionModel is msd_pytorch_amd.MSDRegressionModel
    assert mp.MSDSegmentationModel is msd_pytorch_amd.MSDSegmentationModel
    assert mp.ImageDataset is msd_pytorch_amd.ImageDataset
    assert mp.__version__ == msd_pytorch_amd.__version__


@pytest.mark.parametrize("name", SUBMODULES)
def test_submodule_names_of_the_reference_import(name):
    module = importlib.import_module(f"msd_pytorch.{name}")
    assert module is importlib.import_module(f"msd_pytorch_amd.{name}")
    import msd_pytorch
    assert getattr(msd_pytorch, name) is module


def test_names_the_reference_tests_import():
    # the import lines of the reference's own tests, verbatim
    from msd_pytorch.conv2d import (Conv2dModule, conv2d, conv2d_forward, conv2d_backward_x,  # noqa: F401
                                    conv2d_backward_k, conv2d_backward_bias, Conv2dReluModule, conv2d_relu,
                                    conv2d_relu_forward, conv2d_relu_backward_x, conv2d_relu_backward_k,
                                    conv2d_relu_backward_bias)
    from msd_pytorch.conv3d import (Conv3DReluModule, conv3d_relu, Conv3DModule, conv3d,  # noqa: F401
                                    conv3d_forward, conv3d_backward_x, conv3d_backward_k, conv3d_backward_bias,
                                    conv3d_relu_forward)
    from msd_pytorch.errors import InputError  # noqa: F401
    from msd_pytorch.msd_model import MSDModel  # noqa: F401
    from msd_pytorch.msd_module import MSDModule, MSDFinalLayer  # noqa: F401
    from msd_pytorch.msd_regression_model import MSDRegressionModel  # noqa: F401
    from msd_pytorch.msd_segmentation_model import MSDSegmentationModel  # noqa: F401
    import msd_pytorch.image_dataset as img_ds
    import msd_pytorch.msd_block as msd_block
    import msd_pytorch.msd_module as msd_module
    import msd_custom_convolutions as cc
    assert hasattr(img_ds, "ImageDataset") and hasattr(msd_block, "MSDBlock2d") and hasattr(msd_module, "MSDModule")
    for op in ("conv_forward", "conv_backward_x", "conv_backward_k", "conv_backward_bias", "conv_relu_forward",
               "conv_relu_backward_x", "conv_relu_backward_k", "conv_relu_backward_bias"):
        assert callable(getattr(cc, op))
