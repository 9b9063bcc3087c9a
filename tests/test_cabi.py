"""The C ABI of libmsd_hip.so without a GPU: the library loads, exports every
function include/msd_hip.h declares, and rejects invalid arguments before
touching the device (no kernel is launched by anything in this file)."""
import ctypes
import os
import re

import pytest

from msd_pytorch_amd import _native

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "msd_hip.h")


def declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(msd_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_the_eight_reference_operators():
    names = declared_functions()
    for op in ("conv_forward", "conv_backward_x", "conv_backward_k", "conv_backward_bias", "conv_relu_forward",
               "conv_relu_backward_x", "conv_relu_backward_k", "conv_relu_backward_bias"):
        assert "msd_" + op in names


def test_library_exports_every_declared_symbol():
    lib = ctypes.CDLL(_native.LIB_PATH)
    for name in declared_functions():
        assert hasattr(lib, name), f"{name} is declared in msd_hip.h but not exported"


def test_binding_table_matches_header():
    assert sorted(_native.PROTOTYPES) == declared_functions()


def test_abi_version():
    assert _native.load().msd_abi_version() == _native.ABI_VERSION


def i64(*v):
    return _native.i64_array(v)


FAKE = ctypes.c_void_p(0x1000)   # never dereferenced: every call below fails validation first


def forward_args(dtype=0, ndim=2, batch=1, c_in=1, c_out=1, spatial=(4, 4), dilation=1, inp=FAKE, strides=None):
    strides = strides or i64(*([1] * (ndim + 2)))
    return (dtype, ndim, batch, c_in, c_out, i64(*spatial), dilation, inp, strides, FAKE, FAKE, FAKE, strides,
            ctypes.c_void_p(0))


@pytest.mark.parametrize("kwargs,needle", [
    (dict(dilation=0), "Dilation must be 1 or greater"),
    (dict(dilation=5), "Dilation cannot be greater than size of image"),
    (dict(spatial=(2, 2), dilation=3), "Dilation cannot be greater than size of image"),   # reference tests/test_conv2d.py:76-90
    (dict(ndim=4, spatial=(4, 4, 4, 4)), "2 or 3 spatial dimensions"),
    (dict(dtype=7), "dtype"),
    (dict(batch=0), "positive"),
    (dict(c_in=0), "positive"),
    (dict(spatial=(0, 4)), "positive"),
    (dict(inp=ctypes.c_void_p(0)), "input is NULL"),
    (dict(strides=_native.i64_array((1, 1, -1, 1))), "negative stride"),
])
def test_forward_rejects_invalid_arguments(kwargs, needle):
    lib = _native.load()
    for fn in (lib.msd_conv_forward, lib.msd_conv_relu_forward):
        rc = fn(*forward_args(**kwargs))
        assert rc == _native.MSD_ERR_INVALID
        assert needle in _native.last_error()


def test_backward_k_rejects_missing_workspace():
    lib = _native.load()
    s = i64(1, 1, 1, 1)
    rc = lib.msd_conv_relu_backward_k(0, 2, 1, 1, 1, i64(4, 4), 1, FAKE, s, FAKE, s, FAKE, s, FAKE,
                                      ctypes.c_void_p(0), 0, ctypes.c_void_p(0))
    assert rc == _native.MSD_ERR_WORKSPACE
    assert "workspace" in _native.last_error()


def test_static_scratch_entry_point_rejects_before_touching_the_device():
    # msd_conv_relu_backward_kb_static: geometry errors and problems larger than the
    # library's scratch buffer are refused before any HIP call
    lib = _native.load()
    s2, s3 = i64(1, 1, 1, 1), i64(1, 1, 1, 1, 1)
    null = ctypes.c_void_p(0)
    rc = lib.msd_conv_relu_backward_kb_static(0, 2, 1, 1, 1, i64(4, 4), 5, FAKE, s2, FAKE, s2, FAKE, s2, FAKE, null, null)
    assert rc == _native.MSD_ERR_INVALID and "Dilation cannot be greater" in _native.last_error()
    big = i64(256, 256, 256)
    assert lib.msd_workspace_bytes(0, 3, 1, 2, 1, big) > _native.STATIC_SCRATCH_BYTES
    rc = lib.msd_conv_relu_backward_kb_static(0, 3, 1, 2, 1, big, 1, FAKE, s3, FAKE, s3, FAKE, s3, FAKE, null, null)
    assert rc == _native.MSD_ERR_WORKSPACE and "static buffer" in _native.last_error()
    header = open(HEADER).read()
    assert "#define MSD_STATIC_SCRATCH_BYTES (32 * 1024 * 1024)" in header
    assert _native.STATIC_SCRATCH_BYTES == 32 * 1024 * 1024


def test_workspace_query():
    lib = _native.load()
    n32 = lib.msd_workspace_bytes(0, 2, 1, 10, 1, i64(64, 64))
    n64 = lib.msd_workspace_bytes(1, 2, 1, 10, 1, i64(64, 64))
    assert n32 > 0 and n64 == 2 * n32
    assert lib.msd_workspace_bytes(0, 5, 1, 10, 1, i64(64, 64)) < 0


def test_tuning_hook_rejects_unknown_key():
    lib = _native.load()
    assert lib.msd_set_tuning(b"no.such.knob", 1) == _native.MSD_ERR_INVALID
    assert lib.msd_set_tuning(b"xcd_remap", -1) == _native.MSD_OK
    # every key the header documents is known to the library
    import re
    header = open(os.path.join(ROOT, "include", "msd_hip.h")).read()
    doc = header[header.index("Keys:"):header.index("Unknown keys")]
    keys = re.findall(r'"([a-z0-9_.]+)"', doc)
    assert len(keys) == len(set(keys)) >= 18
    for key in keys:
        assert lib.msd_set_tuning(key.encode(), -1) == _native.MSD_OK, key
    assert lib.msd_set_kernel_path(2) == _native.MSD_ERR_INVALID
    assert lib.msd_set_kernel_path(0) == _native.MSD_OK
