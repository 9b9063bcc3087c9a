"""ctypes binding of libmsd_hip.so (the C ABI declared in include/msd_hip.h).

The library is the only implementation of the operators: there is no CPU or
pure-torch fallback, and a missing library is an ImportError."""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
# MSD_HIP_LIBRARY names another build of the library (same C ABI), e.g. one compiled with
# different tuning constants, for side-by-side measurements
LIB_PATH = os.environ.get("MSD_HIP_LIBRARY") or os.path.join(_HERE, "libmsd_hip.so")
ABI_VERSION = 1

MSD_F32, MSD_F64 = 0, 1
MSD_OK, MSD_ERR_INVALID, MSD_ERR_HIP, MSD_ERR_WORKSPACE = 0, 1, 2, 3
LOSS_MSE, LOSS_L1, LOSS_NLL = 0, 1, 2
STATIC_SCRATCH_BYTES = 32 * 1024 * 1024   # MSD_STATIC_SCRATCH_BYTES of the header

_c_int = ctypes.c_int
_c_i64 = ctypes.c_int64
_i64p = ctypes.POINTER(ctypes.c_int64)
_ptr = ctypes.c_void_p

_HEAD = [_c_int, _c_int, _c_i64, _c_i64, _c_i64, _i64p, _c_int]   # dtype ndim batch c_in c_out spatial dilation
_VIEW = [_ptr, _i64p]
_WS = [_ptr, _c_i64]

# name -> argument types; every symbol that include/msd_hip.h declares
PROTOTYPES = {
    "msd_last_error": (ctypes.c_char_p, []),
    "msd_abi_version": (_c_int, []),
    "msd_set_kernel_path": (_c_int, [_c_int]),
    "msd_set_tuning": (_c_int, [ctypes.c_char_p, _c_int]),
    "msd_workspace_bytes": (_c_i64, [_c_int, _c_int, _c_i64, _c_i64, _c_i64, _i64p]),
    "msd_conv_forward": (_c_int, _HEAD + _VIEW + [_ptr, _ptr] + _VIEW + [_ptr]),
    "msd_conv_relu_forward": (_c_int, _HEAD + _VIEW + [_ptr, _ptr] + _VIEW + [_ptr]),
    "msd_conv_backward_x": (_c_int, _HEAD + _VIEW + [_ptr] + _VIEW + [_ptr]),
    "msd_conv_relu_backward_x": (_c_int, _HEAD + _VIEW + _VIEW + [_ptr] + _VIEW + [_ptr]),
    "msd_conv_backward_k": (_c_int, _HEAD + _VIEW + _VIEW + [_ptr] + _WS + [_ptr]),
    "msd_conv_relu_backward_k": (_c_int, _HEAD + _VIEW + _VIEW + _VIEW + [_ptr] + _WS + [_ptr]),
    "msd_conv_backward_bias": (_c_int, [_c_int, _c_int, _c_i64, _c_i64, _i64p] + _VIEW + [_ptr] + _WS + [_ptr]),
    "msd_conv_relu_backward_bias": (_c_int, [_c_int, _c_int, _c_i64, _c_i64, _i64p] + _VIEW + _VIEW + [_ptr]
                                    + _WS + [_ptr]),
    "msd_conv_relu_backward_kb": (_c_int, _HEAD + _VIEW + _VIEW + _VIEW + [_ptr, _ptr] + _WS + [_ptr]),
    "msd_conv_relu_backward_kb_static": (_c_int, _HEAD + _VIEW + _VIEW + _VIEW + [_ptr, _ptr, _ptr]),
    "msd_conv_backward_kb": (_c_int, _HEAD + _VIEW + _VIEW + [_ptr, _ptr] + _WS + [_ptr]),
    "msd_conv_backward_xkb": (_c_int, _HEAD + _VIEW + _VIEW + [_ptr] + _VIEW + [_ptr, _ptr] + _WS + [_ptr]),
    "msd_relu_mask_gradient": (_c_int, [_c_int, _c_int, _c_i64, _c_i64, _i64p] + _VIEW + _VIEW + [_ptr]),
    "msd_block_workspace_bytes": (_c_i64, [_c_int, _c_int, _c_i64, _c_i64, _c_int, _i64p, _i64p]),
    "msd_block_forward": (_c_int, [_c_int, _c_int, _c_i64, _c_i64, _c_int, _i64p, _i64p, _i64p] + _VIEW
                          + [ctypes.POINTER(ctypes.c_void_p), _ptr, _ptr]),
    "msd_block_backward": (_c_int, [_c_int, _c_int, _c_i64, _c_i64, _c_int, _i64p, _i64p, _i64p] + _VIEW + _VIEW
                           + [ctypes.POINTER(ctypes.c_void_p), ctypes.POINTER(ctypes.c_void_p), _ptr, _c_int]
                           + _WS + [_ptr]),
    "msd_final_workspace_bytes": (_c_i64, [_c_int, _c_i64, _c_i64, _c_i64, _c_i64]),
    "msd_final_forward": (_c_int, [_c_int, _c_i64, _c_i64, _c_i64, _c_i64, _ptr, _c_i64, _c_i64, _ptr, _ptr,
                                   _ptr, _c_i64, _c_i64, _ptr]),
    "msd_final_backward": (_c_int, [_c_int, _c_i64, _c_i64, _c_i64, _c_i64, _ptr, _c_i64, _c_i64, _ptr, _c_i64, _c_i64,
                                    _ptr, _ptr, _c_i64, _c_i64, _ptr, _ptr] + _WS + [_ptr]),
    "msd_final_forward_loss": (_c_int, [_c_int, _c_int, _c_i64, _c_i64, _c_i64, _c_i64, _ptr, _c_i64, _c_i64, _ptr, _ptr,
                                        _ptr, _c_i64, _c_i64, _ptr, _c_i64, _c_i64, _ptr, _c_i64, _c_i64, _ptr, _ptr,
                                        _ptr] + _WS + [_ptr]),
    "msd_profile_enable": (_c_int, [_c_int]),
    "msd_profile_read": (_c_int, [ctypes.POINTER(ctypes.c_double), _i64p]),
}

_lib = None


def load():
    """Load the library once; raise ImportError if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            f"{LIB_PATH} is missing: build it with `make -C {os.path.join(_HERE, 'csrc')}` "
            "(needs hipcc; there is no fallback implementation)")
    lib = ctypes.CDLL(LIB_PATH)
    for name, (restype, argtypes) in PROTOTYPES.items():
        fn = getattr(lib, name)          # AttributeError if a declared symbol is not exported
        fn.restype = restype
        fn.argtypes = argtypes
    if lib.msd_abi_version() != ABI_VERSION:
        raise ImportError(f"{LIB_PATH}: ABI version {lib.msd_abi_version()}, expected {ABI_VERSION}")
    _lib = lib
    return lib


def last_error():
    return load().msd_last_error().decode()


def i64_array(values):
    return (ctypes.c_int64 * len(values))(*values)
