"""The reference's package name (``import msd_pytorch as mp``,
examples/getting_started.py:4; msd_pytorch/__init__.py:21-25) bound to the MI355X
implementation: every public name and every sub-module of ``msd_pytorch_amd`` is
reachable here under the name the reference gives it, so user code and tests written
against the reference import unchanged.  Nothing is defined here; the objects are the
same objects (``msd_pytorch.MSDRegressionModel is msd_pytorch_amd.MSDRegressionModel``)."""
import importlib as _importlib
import sys as _sys

import msd_pytorch_amd as _impl

__version__ = _impl.__version__

# sub-modules the reference has (msd_pytorch/*.py) and their counterparts here
_SUBMODULES = ("conv2d", "conv3d", "msd_block", "msd_module", "msd_model", "msd_regression_model",
               "msd_segmentation_model", "image_dataset", "errors", "bench", "msd_custom_convolutions",
               "benchmark_ops")
for _name in _SUBMODULES:
    _module = _importlib.import_module(f"msd_pytorch_amd.{_name}")
    _sys.modules[f"{__name__}.{_name}"] = _module
    globals()[_name] = _module

for _name in dir(_impl):
    if not _name.startswith("_") and _name not in globals():
        globals()[_name] = getattr(_impl, _name)

del _name, _module
