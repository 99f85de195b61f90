"""ctypes binding of libmonet_hip.so (the C ABI declared in include/monet_hip.h).

The library is the only compute path: if it is missing or a call fails the
caller gets an exception, never a fallback.
"""
import ctypes
import os
from ctypes import (POINTER, Structure, c_char_p, c_double, c_float, c_int, c_int32, c_int64,
                    c_size_t, c_uint32, c_void_p)
from pathlib import Path

import torch

# MONET_HIP_LIBRARY overrides the in-tree build (e.g. to load an instrumented build).
LIB_PATH = Path(os.environ.get("MONET_HIP_LIBRARY",
                               Path(__file__).resolve().parent / "libmonet_hip.so"))
ABI_VERSION = 1

MN_OK, MN_EINVAL, MN_EUNSUPPORTED, MN_ELAUNCH, MN_ELIMIT = 0, 1, 2, 3, 4


class MonetHipError(RuntimeError):
    """A libmonet_hip entry point returned a non-zero status."""

    def __init__(self, fn, status, text):
        super().__init__(f"{fn} failed: status {status} ({text})")
        self.status = status


class Conv2d(Structure):
    """Mirror of `struct mn_conv2d`."""
    _fields_ = [(k, c_int32) for k in
                ("N", "C", "H", "W", "K", "R", "S", "sH", "sW", "pH", "pW", "dH", "dW", "P", "Q",
                 "groups")]


CONV_FWD, CONV_BWD_DATA, CONV_BWD_WEIGHT = 0, 1, 2
F32 = 0
BF16 = 1   # bf16 tensors in channels-last order (see include/monet_hip.h)


class Pool2d(Structure):
    """Mirror of `struct mn_pool2d`."""
    _fields_ = [(k, c_int32) for k in
                ("N", "C", "H", "W", "kH", "kW", "sH", "sW", "pH", "pW", "dH", "dW", "PH", "PW")]


_P = c_void_p
_SIGNATURES = {
    # name: (restype, argtypes); restype c_int means "status code, checked"
    "mn_abi_version": (c_int, []),
    "mn_status_string": (c_char_p, [c_int]),
    "mn_init": (c_int, []),
    "mn_pack_bits": (c_int, [_P, _P, c_size_t, _P]),
    "mn_unpack_bits": (c_int, [_P, _P, c_size_t, _P]),
    "mn_unpack_bits_mul_f32": (c_int, [_P, _P, _P, c_size_t, _P]),
    "mn_pack_nibbles": (c_int, [_P, _P, c_size_t, _P]),
    "mn_unpack_nibbles": (c_int, [_P, _P, c_size_t, _P]),
    "mn_relu_fwd_mask_f32": (c_int, [_P, _P, _P, c_size_t, _P]),
    "mn_add_relu_fwd_f32": (c_int, [_P, _P, c_float, _P, _P, c_size_t, _P]),
    "mn_relu_bwd_mask_f32": (c_int, [_P, _P, _P, c_size_t, _P]),
    "mn_relu_bwd_ref_f32": (c_int, [_P, _P, c_float, _P, c_size_t, _P]),
    "mn_pool_out_size": (c_int64, [c_int64, c_int64, c_int64, c_int64, c_int64, c_int]),
    "mn_maxpool_fwd_idx_f32": (c_int, [POINTER(Pool2d), _P, _P, _P, _P]),
    "mn_maxpool_bwd_idx_f32": (c_int, [POINTER(Pool2d), _P, _P, _P, _P]),
    "mn_bn_ws_bytes": (c_size_t, [c_int64, c_int64, c_int64]),
    "mn_bn_fwd_train_f32": (c_int, [_P, _P, _P, _P, _P, _P, _P, _P, c_int64, c_int64, c_int64,
                                    c_double, c_double, _P, c_size_t, _P]),
    "mn_bn_fwd_apply_f32": (c_int, [_P, _P, _P, _P, _P, _P, c_int64, c_int64, c_int64, _P]),
    "mn_bn_bwd_from_x_f32": (c_int, [_P, _P, _P, _P, _P, _P, _P, _P, c_int64, c_int64, c_int64,
                                     _P, c_size_t, _P]),
    "mn_bn_bwd_from_y_f32": (c_int, [_P, _P, _P, _P, _P, _P, _P, _P, c_int64, c_int64, c_int64,
                                     _P, c_size_t, _P]),
    "mn_bn_bwd_from_y_f32_limits": (c_int, [_P, _P, _P, _P, _P, _P, _P, _P, c_int64, c_int64,
                                            c_int64, _P, c_size_t, c_uint32, c_uint32, c_uint32, c_uint32,
                                            _P]),
    "mn_bn_ws_status": (c_int, [_P, c_size_t, c_int64, c_int64, c_int64, _P]),
    "mn_bn_wait_status": (c_int, [_P, _P]),
    "mn_bn_bwd_from_y_static_f32": (c_int, [_P, _P, _P, _P, _P, _P, _P, _P, c_int64, c_int64,
                                            c_int64, _P]),
    "mn_bn_relu_fwd_train_f32": (c_int, [_P, _P, _P, _P, _P, _P, _P, _P, c_int64, c_int64, c_int64,
                                         c_double, c_double, _P, c_size_t, _P]),
    "mn_bn_relu_fwd_apply_f32": (c_int, [_P, _P, _P, _P, _P, _P, c_int64, c_int64, c_int64, _P]),
    "mn_bn_relu_bwd_from_x_f32": (c_int, [_P, _P, _P, _P, _P, _P, _P, _P, _P, c_int64, c_int64,
                                          c_int64, _P, c_size_t, _P]),
    "mn_bn_add_relu_fwd_train_f32": (c_int, [_P, _P, _P, _P, _P, _P, c_double, _P, _P, _P, c_int64,
                                             c_int64, c_int64, c_double, c_double, _P, c_size_t, _P]),
    "mn_bn_add_relu_fwd_apply_f32": (c_int, [_P, _P, _P, _P, _P, _P, c_double, _P, c_int64, c_int64,
                                             c_int64, _P]),
    "mn_bn_add_relu_bwd_f32": (c_int, [_P, _P, _P, _P, _P, _P, c_double, _P, _P, _P, _P, c_int64,
                                       c_int64, c_int64, _P, c_size_t, _P]),
    "mn_bn_add_relu_mask_fwd_train_f32": (c_int, [_P, _P, _P, _P, _P, _P, c_double, _P, _P, _P, _P,
                                                  c_int64, c_int64, c_int64, c_double, c_double, _P,
                                                  c_size_t, _P]),
    "mn_bn_add_relu_mask_fwd_apply_f32": (c_int, [_P, _P, _P, _P, _P, _P, c_double, _P, _P, c_int64,
                                                  c_int64, c_int64, _P]),
    "mn_bn_add_relu_mask_bwd_f32": (c_int, [_P, _P, _P, _P, _P, _P, c_double, _P, _P, _P, _P, c_int64,
                                            c_int64, c_int64, _P, c_size_t, _P]),
    "mn_softmax_fwd_f32": (c_int, [_P, _P, c_int64, c_int64, c_int64, _P]),
    "mn_softmax_bwd_f32": (c_int, [_P, _P, _P, c_int64, c_int64, c_int64, _P]),
    "mn_xent_bwd_f32": (c_int, [_P, _P, _P, c_int64, c_int64, c_int64, c_float, _P]),
    "mn_conv_n_variants": (c_int, [c_int]),
    "mn_conv_n_variants_for": (c_int, [c_int, c_int]),
    "mn_conv_ws_bytes": (c_int, [POINTER(Conv2d), c_int, c_int, c_int, POINTER(c_size_t)]),
    "mn_conv_fwd": (c_int, [POINTER(Conv2d), _P, _P, _P, _P, _P, c_size_t, c_int, c_int, _P]),
    "mn_conv_bwd_data": (c_int, [POINTER(Conv2d), _P, _P, _P, _P, c_size_t, c_int, c_int, _P]),
    "mn_conv_bwd_data_accumulate": (c_int, [POINTER(Conv2d), _P, _P, _P, _P, c_size_t, c_int, c_int,
                                            _P]),
    "mn_conv_bwd_weight": (c_int, [POINTER(Conv2d), _P, _P, _P, _P, c_size_t, c_int, c_int, _P]),
    "mn_conv_bwd_weight_bias": (c_int, [POINTER(Conv2d), _P, _P, _P, _P, _P, c_size_t, c_int, c_int,
                                        _P]),
}
# entry points whose int return value is NOT a status code
_UNCHECKED = {"mn_abi_version", "mn_conv_n_variants", "mn_conv_n_variants_for"}

_lib = None


def load():
    """Load the shared library once; raise if it is absent or of another ABI."""
    global _lib
    if _lib is not None:
        return _lib
    if not LIB_PATH.exists():
        raise ImportError(
            f"{LIB_PATH} is not built. Run `python -m monet_amd.build` (needs hipcc); "
            "there is no fallback implementation.")
    lib = ctypes.CDLL(str(LIB_PATH))
    for name, (res, args) in _SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError if the symbol is missing
        fn.restype = res
        fn.argtypes = args
    if lib.mn_abi_version() != ABI_VERSION:
        raise ImportError(f"{LIB_PATH} has ABI {lib.mn_abi_version()}, expected {ABI_VERSION}")
    _lib = lib
    return lib


def exported_names():
    return list(_SIGNATURES)


def call(name, *args):
    """Call a status-returning entry point; raise MonetHipError on failure."""
    lib = load()
    st = getattr(lib, name)(*args)
    if name not in _UNCHECKED and _SIGNATURES[name][0] is c_int and st != MN_OK:
        raise MonetHipError(name, st, lib.mn_status_string(st).decode())
    return st


def ptr(t):
    """Device pointer of a tensor (None -> NULL)."""
    return None if t is None else t.data_ptr()


_initialised = set()


def stream_ptr(device=None):
    """hipStream_t of torch's current stream on `device`.  The first call for a device also
    runs the library's per-device set-up (mn_init), so that no entry point has to do it on
    its first call, which may be under stream capture."""
    index = torch.cuda.current_device() if device is None else torch.device(device).index
    if index is None:
        index = torch.cuda.current_device()
    if index not in _initialised:
        with torch.cuda.device(index):
            call("mn_init")
        _initialised.add(index)
    return torch.cuda.current_stream(device).cuda_stream


def require_gpu_tensor(t, name, dtype=None):
    if not isinstance(t, torch.Tensor) or not t.is_cuda:
        raise RuntimeError(f"{name} must be a GPU tensor: these operators have no CPU implementation")
    if dtype is not None and t.dtype != dtype:
        raise RuntimeError(f"{name} must have dtype {dtype}, got {t.dtype}")
    return t
