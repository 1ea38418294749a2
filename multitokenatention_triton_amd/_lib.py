"""ctypes binding of libmta_hip.so (the C ABI declared in include/mta_hip.h).

The library is built in-tree by ``build.py`` (``make -C csrc``) and must exist: there
is no CPU or eager fallback.  Loading it does not need a GPU; calling a compute entry
point does.
"""
from __future__ import annotations

import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libmta_hip.so")

# dtype codes of include/mta_hip.h
MTA_F32, MTA_BF16, MTA_F16 = 0, 1, 2
MTA_CAUSAL_LOWER_ONLY = 2  # `causal` of the conv / head-mixing entry points: nothing written above the diagonal

_c = ctypes
_vp, _i64, _int, _f32 = _c.c_void_p, _c.c_int64, _c.c_int, _c.c_float

# name -> (restype, argtypes); one entry per declaration in include/mta_hip.h
SIGNATURES = {
    "mta_abi_version": (_int, []),
    "mta_strerror": (_c.c_char_p, [_int]),
    "mta_conv2d_fwd": (_int, [_vp, _vp, _vp, _i64, _i64, _i64, _i64, _int, _int, _int, _int, _int, _vp]),
    "mta_conv2d_scaled_fwd": (_int, [_vp, _vp, _vp, _i64, _i64, _i64, _i64, _int, _int, _int, _f32, _int, _int, _vp]),
    "mta_headmix_fwd": (_int, [_vp, _vp, _vp, _i64, _i64, _i64, _i64, _int, _int, _f32, _int, _int, _vp]),
    "mta_headmix_softmax_fwd": (_int, [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _int, _int, _int, _int, _int, _vp]),
    "mta_headmix_softmax_bias_fwd": (_int, [_vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _int, _int, _int, _int, _int, _vp]),
    "mta_conv2d_headmix_fwd": (_int, [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _int, _int, _int, _int, _int, _int, _int, _int, _vp]),
    "mta_qk_conv_fwd": (_int, [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _int, _int, _int, _f32, _int, _int, _int, _vp]),
    "mta_qk_conv_supported": (_int, [_i64, _i64, _int, _int, _int, _int]),
    "mta_causal_pv_band_fwd": (_int, [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _int, _int, _vp]),
    "mta_band_zero_fwd": (_int, [_vp, _vp, _i64, _i64, _i64, _int, _vp]),
    "mta_mask_fill_fwd": (_int, [_vp, _vp, _vp, _i64, _i64, _i64, _i64, _int, _int, _int, _int, _int, _vp]),
    "mta_mask_add_fwd": (_int, [_vp, _vp, _vp, _i64, _i64, _i64, _i64, _int, _int, _int, _int, _vp]),
    "mta_qk_conv_tri_fwd": (_int, [_vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _int, _int, _f32, _int, _int, _int, _vp]),
    "mta_headmix_softmax_tri_fwd": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _int, _int, _int, _int, _vp]),
    "mta_causal_pv_tri_fwd": (_int, [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _int, _int, _vp]),
    "mta_headmix_softmax_tri_supported": (_int, [_i64, _i64, _int, _int, _int, _int, _int, _int, _int, _int]),
    "mta_qk_conv_band_fwd": (_int, [_vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _int, _int, _f32, _int, _int, _int, _vp]),
    "mta_headmix_softmax_band_fwd": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _int, _int, _int, _int, _int, _vp]),
    "mta_conv2d_tril_fwd": (_int, [_vp, _vp, _vp, _i64, _i64, _i64, _i64, _int, _int, _int, _int, _vp]),
    "mta_headmix_tril_fwd": (_int, [_vp, _vp, _vp, _i64, _i64, _i64, _i64, _int, _int, _int, _vp]),
    "mta_softmax_bwd": (_int, [_vp, _vp, _vp, _i64, _i64, _i64, _i64, _int, _int, _int, _vp]),
    "mta_causal_pv_fwd": (_int, [_vp, _vp, _vp, _i64, _i64, _i64, _i64, _int, _int, _vp]),
    "mta_causal_ptx_fwd": (_int, [_vp, _vp, _vp, _i64, _i64, _i64, _i64, _int, _int, _vp]),
    "mta_conv_attn_fwd_lse": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _int, _int, _int, _f32, _int, _int, _vp]),
    "mta_conv2d_bwd_input": (_int, [_vp, _vp, _vp, _i64, _i64, _i64, _i64, _int, _int, _int, _int, _int, _vp]),
    "mta_conv2d_bwd_weight_workspace": (_i64, [_i64, _i64, _i64, _i64, _int, _int]),
    "mta_conv2d_bwd_weight": (_int, [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _int, _int, _int, _int, _vp]),
    "mta_conv2d_bwd_weight_noalloc": (_int, [_vp, _vp, _vp, _i64, _i64, _i64, _i64, _int, _int, _int, _int, _vp]),
    "mta_headmix_bwd_input": (_int, [_vp, _vp, _vp, _i64, _i64, _i64, _i64, _int, _int, _int, _int, _vp]),
    "mta_headmix_bwd_weight_workspace": (_i64, [_i64, _i64, _i64, _i64]),
    "mta_headmix_bwd_weight": (_int, [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _int, _int, _vp]),
    "mta_probe_head_weight": (_int, [_vp, _i64, _int, _vp, _vp]),
    "mta_probe_conv_kernel": (_int, [_vp, _i64, _int, _int, _int, _vp, _vp]),
    "mta_conv_attn_fwd": (_int, [_vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _int, _int, _int, _f32, _int, _int, _vp]),
}

_lib = None


class MTALibraryError(RuntimeError):
    pass


def load() -> ctypes.CDLL:
    """Load libmta_hip.so once; raise loudly when it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise MTALibraryError(
            f"{LIB_PATH} is missing: build it with `python -m multitokenatention_triton_amd.build` "
            "(hipcc --offload-arch=gfx950). There is no fallback path.")
    lib = ctypes.CDLL(LIB_PATH)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError = header/library mismatch
        fn.restype, fn.argtypes = res, args
    _lib = lib
    return lib


def strerror(code: int) -> str:
    return load().mta_strerror(int(code)).decode()


MTA_ERR_UNSUPPORTED = -9


def check(code: int, what: str) -> None:
    """0 -> ok; negative -> ValueError (argument rejected); positive -> RuntimeError (HIP)."""
    if code == 0:
        return
    msg = f"{what}: {strerror(code)} (code {code})"
    if code < 0:
        raise ValueError(msg)
    raise RuntimeError(msg)
