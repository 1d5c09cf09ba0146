"""ctypes binding of libmercury_hip.so (the C ABI declared in include/mercury_hip.h).

The library is the only implementation: there is no CPU or eager-PyTorch fallback, and a
missing library is an error, not a reason to take another path.
"""
from __future__ import annotations

import ctypes
import os
from ctypes import c_float, c_int, c_int64, c_void_p
from typing import Optional

import torch

# MERCURY_HIP_LIB is a deployment option: the path of the built library when it is not kept next to the package.
LIB_PATH = os.environ.get("MERCURY_HIP_LIB") or os.path.join(
    os.path.dirname(os.path.abspath(__file__)), "csrc", "libmercury_hip.so")
ABI_VERSION = 3      # MHIP_ABI_VERSION of include/mercury_hip.h the signatures below were written against

MHIP_BF16, MHIP_E4M3, MHIP_F32 = 0, 1, 2
MASK_NONE, MASK_CAUSAL = 0, 1

_lib = None

_I, _L, _F, _P = c_int, c_int64, c_float, c_void_p
_SIGNATURES = {
    "mhip_version": (c_int, []),
    "mhip_abi_version": (c_int, []),
    "mhip_init": (c_int, []),
    "mhip_error_string": (ctypes.c_char_p, [_I]),
    "mhip_attn_fwd_block": (c_int, [_P] * 5 + [_I] * 6 + [_L] * 12 + [_F, _I, _I, _P, _P, _P, _P]),
    "mhip_attn_bwd_workspace_bytes": (c_int64, [_I] * 6),
    "mhip_attn_bwd_block": (c_int, [_P] * 10 + [_I] * 6 + [_L] * 15 + [_F, _I, _I, _P, _P]),
    "mhip_attn_bwd_block_noalloc": (c_int, [_P] * 10 + [_I] * 6 + [_L] * 15 + [_F, _I, _I, _P]),
    "mhip_lse_merge": (c_int, [_P] * 8 + [_I] * 4 + [_L] * 17 + [_P]),
    "mhip_lse_merge_many": (c_int, [_P, _P, _P, _P, _I, _P, _P] + [_I] * 4 + [_L] * 2 + [_P]),
    "mhip_flash_reduce": (c_int, [_P] * 3 + [_L, _I, _P]),
    "mhip_tree_merge": (c_int, [_P] * 3 + [_L, _I, _I, _P]),
    "mhip_pack_reduce": (c_int, [_P] * 4 + [_I] * 4 + [_P]),
    "mhip_unpack": (c_int, [_P] * 3 + [_I] * 4 + [_P]),
    "mhip_grad_accumulate": (c_int, [_P] * 3 + [_L, _P]),
    "mhip_quantize_e4m3": (c_int, [_P, _I, _L, _P, _P, _P, _P]),
}
EXPORTED_SYMBOLS = tuple(_SIGNATURES)


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing: build it with `python -m mercury_artifact_amd.csrc.build` "
                "(hipcc, gfx950). There is no fallback implementation.")
        handle = ctypes.CDLL(LIB_PATH)
        try:
            handle.mhip_abi_version.restype = c_int
            built = handle.mhip_abi_version()
        except AttributeError:
            built = None
        if built != ABI_VERSION:
            raise RuntimeError(f"{LIB_PATH} was built with ABI version {built}, this package calls version "
                               f"{ABI_VERSION}: rebuild it with `python -m mercury_artifact_amd.csrc.build`")
        for name, (res, args) in _SIGNATURES.items():
            fn = getattr(handle, name)
            fn.restype = res
            fn.argtypes = args
        _lib = handle
    return _lib


def check(code: int, what: str) -> None:
    if code != 0:
        msg = lib().mhip_error_string(code).decode()
        raise RuntimeError(f"{what}: {msg} (code {code})")


def ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()


def stream_of(t: torch.Tensor) -> int:
    return torch.cuda.current_stream(t.device).cuda_stream


def require_cuda(*tensors: Optional[torch.Tensor]) -> None:
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise RuntimeError("mercury_artifact_amd operators run on the GPU only; got a "
                               f"{t.device} tensor (there is no CPU fallback)")
