"""ctypes binding of libmpsa.so (the C ABI declared in include/mpsa.h).

PyTorch is used for device memory and streams only: tensors are handed over as raw device
pointers, sizes and element strides, and kernels are enqueued on torch's current stream.
"""

import ctypes
import os

import torch

BF16, F16, F32, F8E5M2 = 0, 1, 2, 3
FMT_E4M3, FMT_E5M2, FMT_E2M1 = 0, 1, 4
MODE_MXFP4, MODE_MXFP8, MODE_DIAG, MODE_ROUTED, MODE_MIXED = 0, 1, 2, 3, 4

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.environ.get("MPSA_LIB_PATH") or os.path.join(os.path.dirname(_HERE), "lib", "libmpsa.so")

_i64, _int, _vp, _f32 = ctypes.c_int64, ctypes.c_int, ctypes.c_void_p, ctypes.c_float
_p64 = ctypes.POINTER(ctypes.c_int64)

# name -> (restype, argtypes); must list every symbol include/mpsa.h declares
SIGNATURES = {
    "mpsa_version": (_int, []),
    "mpsa_last_error": (ctypes.c_char_p, []),
    "mpsa_init": (_int, []),
    "mpsa_e2m1_encode": (_int, [_vp, _i64, _vp, _vp]),
    "mpsa_e2m1_decode": (_int, [_vp, _i64, _vp, _vp]),
    "mpsa_e8m0_encode": (_int, [_vp, _i64, _vp, _vp]),
    "mpsa_e8m0_decode": (_int, [_vp, _i64, _vp, _vp]),
    "mpsa_fp8_encode": (_int, [_vp, _i64, _int, _vp, _vp]),
    "mpsa_e2m1_pack": (_int, [_vp, _i64, _i64, _i64, _vp, _vp]),
    "mpsa_e2m1_unpack": (_int, [_vp, _i64, _i64, _i64, _vp, _vp]),
    "mpsa_scales_to_5d": (_int, [_vp, _i64, _i64, _i64, _vp, _vp]),
    "mpsa_scales_from_5d": (_int, [_vp, _i64, _i64, _i64, _vp, _vp]),
    "mpsa_quantize_mx": (_int, [_vp, _int, _i64, _i64, _i64, _i64, _p64, _vp, _f32, _int, _int, _vp, _vp, _i64, _vp]),
    "mpsa_seq_mean_workspace": (_i64, [_i64, _i64, _i64, _i64]),
    "mpsa_seq_mean": (_int, [_vp, _int, _i64, _i64, _i64, _i64, _p64, _vp, _vp, _vp]),
    "mpsa_seq_mean_static": (_int, [_vp, _int, _i64, _i64, _i64, _i64, _p64, _vp, _vp]),
    "mpsa_quantize_mx_dual": (_int, [_vp, _int, _i64, _i64, _i64, _i64, _p64, _vp, _f32, _int, _int, _int,
                                     _vp, _vp, _vp, _vp, _i64, _vp]),
    "mpsa_gemm_mx": (_int, [_vp, _vp, _int, _vp, _vp, _int, _i64, _i64, _i64, _vp, _int, _i64, _vp]),
    "mpsa_gemm_mx_batched": (_int, [_vp, _vp, _int, _vp, _vp, _int, _i64, _i64, _i64, _i64, _i64, _i64, _vp, _int, _i64, _vp]),
    "mpsa_gemm_mx_packed": (_int, [_vp, _vp, _int, _vp, _vp, _int, _i64, _i64, _i64, _vp, _int, _i64, _vp]),
    "mpsa_gemm_mx_batched_packed": (_int, [_vp, _vp, _int, _vp, _vp, _int, _i64, _i64, _i64, _i64, _i64, _i64, _vp, _int, _i64, _vp]),
    "mpsa_v_tiles": (_int, [_vp, _int, _i64, _i64, _i64, _i64, _p64, _int, _vp, _vp]),
    "mpsa_attn_prepare": (_int, [_vp, _p64, _vp, _p64, _vp, _p64, _int, _i64, _i64, _i64, _i64, _i64, _i64, _int, _int, _int,
                                 _f32, _vp] + [_vp] * 9 + [_vp]),
    "mpsa_attn_fwd": (_int, [_vp] * 8 + [_int, _vp, _int, _vp, _int, _p64,
                             _i64, _i64, _i64, _i64, _i64, _i64, _int, _int, _int, _vp]),
    "mpsa_attn_fwd_q16": (_int, [_vp, _p64, _int, _f32] + [_vp] * 4 + [_int, _vp, _int, _vp, _int, _p64,
                                 _i64, _i64, _i64, _i64, _i64, _int, _int, _int, _vp]),
    "mpsa_attn_fwd_q16_supported": (_int, [_i64, _i64, _i64, _i64, _i64, _int, _int, _int]),
    "mpsa_attn_fwd_skip": (_int, [_vp] * 8 + [_int, _vp, _int, _vp, _int, _p64,
                                  _i64, _i64, _i64, _i64, _i64, _i64, _int, _int, _int, _f32, _vp, _vp]),
    "mpsa_route_workspace": (_i64, [_i64, _i64, _i64, _i64, _i64, _i64, _int]),
    "mpsa_route_tiles": (_int, [_vp, _vp, _i64, _i64, _i64, _i64, _i64, _i64, _int, _int, _f32, _f32, _vp, _vp, _vp, _vp, _vp]),
    "mpsa_skip_route_supported": (_int, [_i64, _i64, _i64, _int, _int, _int]),
    "mpsa_skip_route_workspace": (_i64, [_i64, _i64, _i64, _i64, _int]),
    "mpsa_skip_route": (_int, [_vp] * 8 + [_int, _i64, _i64, _i64, _i64, _i64, _i64, _int, _int, _int, _f32, _vp, _vp, _vp, _vp, _vp, _vp]),
    "mpsa_attn_fwd_routed": (_int, [_vp] * 8 + [_int, _vp, _int, _vp, _int, _p64,
                                    _i64, _i64, _i64, _i64, _i64, _i64, _int, _int, _vp, _vp, _vp]),
}

_lib = None


class MpsaError(RuntimeError):
    """A libmpsa entry point returned a negative status."""

    def __init__(self, code, message):
        super().__init__(f"libmpsa error {code}: {message}")
        self.code = code


def lib():
    """Load libmpsa.so once.  Raises if it has not been built -- there is no fallback."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing: build it with `python mp-sparse-attn_amd/build.py` "
                "(hipcc, gfx950). The MXFP path has no CPU or eager fallback.")
        handle = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(handle, name)
            fn.restype = res
            fn.argtypes = args
        _lib = handle
        # set-up of the current device up front, so that even a caller's first launch there can be captured into a HIP
        # graph.  Other devices are set up by the entry points on their first use (mpsa_ensure_init); a caller that wants
        # to capture a first call on another device calls mpsa_init() with that device current.  (No device here means no
        # set-up: the entry points report their own errors.)
        if torch.cuda.is_available():
            status = handle.mpsa_init()
            if status != 0:
                raise MpsaError(status, handle.mpsa_last_error().decode("utf-8", "replace"))
    return _lib


def check(status):
    if status != 0:
        raise MpsaError(status, lib().mpsa_last_error().decode("utf-8", "replace"))


def dtype_id(dtype):
    if dtype == torch.bfloat16:
        return BF16
    if dtype == torch.float16:
        return F16
    if dtype == torch.float32:
        return F32
    if dtype == torch.float8_e5m2:
        return F8E5M2
    raise ValueError(f"unsupported dtype {dtype}")


def require_device(*tensors):
    for t in tensors:
        if not isinstance(t, torch.Tensor) or not t.is_cuda:
            raise RuntimeError("the MXFP path runs on HIP device tensors only (got a %s tensor); "
                               "there is no CPU fallback" % (t.device if isinstance(t, torch.Tensor) else type(t)))


def stream_ptr(device=None):
    return ctypes.c_void_p(torch.cuda.current_stream(device).cuda_stream)


def ptr(t):
    return ctypes.c_void_p(t.data_ptr()) if t is not None else ctypes.c_void_p(0)


def strides4(t):
    assert t.dim() == 4
    return (ctypes.c_int64 * 4)(*t.stride())
