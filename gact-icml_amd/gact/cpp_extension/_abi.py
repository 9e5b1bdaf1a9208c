"""ctypes binding of libgact_hip.so.

The library is loaded once, on first use.  A missing library is an error, never a fallback: the HIP
kernels are the only implementation of the device path.
"""
import ctypes
import os

import torch  # imported first so that the library binds to the HIP runtime torch already loaded

_LIB = None
LIB_PATH = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "lib", "libgact_hip.so")

F32, F16, BF16 = 0, 1, 2
NOISE_CONST, NOISE_INJECT, NOISE_REF, NOISE_FAST = 0, 1, 2, 3
NOISE_MODES = {"deterministic": NOISE_CONST, "inject": NOISE_INJECT, "reference": NOISE_REF, "fast": NOISE_FAST}
GROUP = 256
ABI_VERSION = 7


class BatchEntry(ctypes.Structure):
    """Mirror of gact_batch_entry in include/gact_hip.h."""

    _fields_ = [
        ("x", ctypes.c_void_p),
        ("numel", ctypes.c_int64),
        ("dtype", ctypes.c_int32),
        ("reserved", ctypes.c_int32),
        ("seed", ctypes.c_uint64),
        ("first_block", ctypes.c_int64),
        ("packed_offset", ctypes.c_int64),
        ("stats_offset", ctypes.c_int64),
    ]


_vp, _i32, _i64, _u64, _f64 = ctypes.c_void_p, ctypes.c_int, ctypes.c_int64, ctypes.c_uint64, ctypes.c_double

# name -> (restype, argtypes); exactly the entry points include/gact_hip.h declares
SIGNATURES = {
    "gact_strerror": (ctypes.c_char_p, [_i32]),
    "gact_abi_version": (_i32, []),
    "gact_packed_bytes": (_i64, [_i32, _i64, _i64, _i64]),
    "gact_minimax": (_i32, [_vp, _i32, _i64, _i64, _vp, _vp, _vp]),
    "gact_pack": (_i32, [_vp, _vp, _vp, _i32, _i32, _i64, _i64, _i64, _i32, _u64, _vp, _vp, _vp, _vp]),
    "gact_unpack": (_i32, [_vp, _i32, _vp, _vp, _i32, _i64, _i64, _i64, _vp, _vp]),
    "gact_quantize": (_i32, [_vp, _i32, _i64, _i32, _i32, _u64, _vp, _vp, _vp, _vp, _vp, _vp]),
    "gact_quantize_seeded": (_i32, [_vp, _i32, _i64, _i32, _i32, _u64, _vp, _vp, _vp, _vp, _vp, _vp, _vp]),
    "gact_dequantize": (_i32, [_vp, _i32, _vp, _vp, _i32, _i64, _vp, _vp]),
    "gact_launch_geometry": (_i32, [_i32, _i32, _i32, _i64, _vp, _vp, _vp]),
    "gact_mask_pack": (_i32, [_vp, _i64, _vp, _vp]),
    "gact_mask_unpack": (_i32, [_vp, _i64, _vp, _vp]),
    "gact_calc_precision": (_i32, [_vp, _vp, _vp, _i64, _f64]),
    "gact_calc_precision_device": (_i32, [_vp, _vp, _vp, _i64, _f64, _vp, _vp]),
    "gact_batch_workspace_bytes": (_i64, [_i64, _i64]),
    "gact_batch_plan": (_i32, [_vp, _vp, _i64, _i64, _i64, _vp, _vp]),
    "gact_quantize_batched": (_i32, [_vp, _vp, _i64, _i64, _i32, _i32, _vp, _vp, _vp, _vp, _vp]),
    "gact_dequantize_batched": (_i32, [_vp, _vp, _i64, _i64, _vp, _vp, _vp, _vp, _vp]),
    "gact_quantize_batched_static": (_i32, [_vp, _vp, _i64, _i64, _i64, _i32, _i32, _vp, _vp, _vp, _vp, _vp]),
}


def lib():
    global _LIB
    if _LIB is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                "libgact_hip.so is not built (%s): run `python gact-icml_amd/build.py`; "
                "there is no fallback implementation" % LIB_PATH)
        L = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(L, name)
            fn.restype = res
            fn.argtypes = args
        if L.gact_abi_version() != ABI_VERSION:
            raise RuntimeError("libgact_hip.so has ABI version %d, expected %d" % (L.gact_abi_version(), ABI_VERSION))
        _LIB = L
    return _LIB


def check(code):
    """Turn a status code into the RuntimeError the reference's TORCH_CHECK would have raised."""
    if code != 0:
        raise RuntimeError("gact: " + lib().gact_strerror(code).decode())


def dtype_code(dtype):
    if dtype == torch.float32:
        return F32
    if dtype == torch.float16:
        return F16
    if dtype == torch.bfloat16:     # the fused and the batched entry points only
        return BF16
    raise RuntimeError("gact: only float32, float16 and bfloat16 are supported, got %s" % dtype)


def stream_of(t):
    """Raw HIP stream torch currently launches on for t's device."""
    return torch._C._cuda_getCurrentRawStream(t.device.index)


_ONE_GPU = None


def call_on(device, fn, *args):
    """Call a library entry point with `device` current (the kernels launch on the current HIP device) and
    turn its status into RuntimeError.  With a single visible GPU there is nothing to switch."""
    global _ONE_GPU
    if _ONE_GPU is None:
        _ONE_GPU = torch.cuda.device_count() == 1
    if _ONE_GPU:
        code = fn(*args)
    else:
        with torch.cuda.device(device):
            code = fn(*args)
    if code != 0:
        check(code)


def ptr(t):
    return t.data_ptr() if t is not None else None


def aligned(t):
    """The kernels use 16-byte loads; fresh torch allocations always qualify, offset views may not."""
    return t.data_ptr() % 16 == 0
