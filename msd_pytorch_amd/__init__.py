"""MI355X-native implementation of the msd_pytorch hot path (dilated conv+ReLU
dense blocks) behind the reference's Python API."""
import sys as _sys

__version__ = "0.1.0"

from . import msd_custom_convolutions  # noqa: E402
from . import conv2d, conv3d  # noqa: E402,F401
from .msd_block import MSDBlock, MSDBlock2d, MSDBlock3d, MSDBlockFunction, msd_block  # noqa: E402,F401
from .msd_module import MSDFinalLayer, MSDModule  # noqa: E402,F401
from .errors import Error, InputError  # noqa: E402,F401
from .image_dataset import ImageDataset, ImageStack  # noqa: E402,F401
from .msd_model import GraphedStep  # noqa: E402,F401
from .msd_regression_model import MSDRegressionModel  # noqa: E402,F401
from .msd_segmentation_model import MSDSegmentationModel  # noqa: E402,F401

# The reference's Python layers import the native operators as a top-level
# module (conv2d.py:5); make that name resolve to this implementation.
_sys.modules.setdefault("msd_custom_convolutions", msd_custom_convolutions)
