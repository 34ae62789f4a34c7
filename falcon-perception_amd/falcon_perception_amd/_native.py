"""ctypes binding of libfp_paged_kv.so (declared in include/fp_paged_kv.h).

The library is the only compute path of this package: there is no eager or CPU
fallback.  If it is missing, `lib()` raises and so does every operator.
"""

from __future__ import annotations

import ctypes
import os
from ctypes import c_char_p, c_float, c_int, c_int32, c_int64, c_void_p

import torch

_LIB_DIR = os.path.join(os.path.dirname(os.path.abspath(__file__)), "_lib")
LIB_PATH = os.path.join(_LIB_DIR, "libfp_paged_kv.so")

FP_ABI_VERSION = 7
NOALLOC_SCRATCH_BYTES = 64 << 20  # FP_NOALLOC_SCRATCH_BYTES
FP_DTYPE = {torch.float32: 0, torch.bfloat16: 1, torch.float16: 2}
FP_INDEX = {torch.int32: 0, torch.int64: 1}

# name -> (restype, argtypes); mirrors include/fp_paged_kv.h one to one
SIGNATURES = {
    "fp_abi_version": (c_int, []),
    "fp_last_error": (c_char_p, []),
    "fp_kv_append": (c_int, [
        c_void_p, c_void_p, c_void_p, c_void_p,
        c_int64, c_int64, c_int64, c_int64, c_int64, c_int64,
        c_void_p, c_int64, c_void_p, c_void_p, c_int,
        c_int32, c_int32, c_int32, c_int32, c_int32, c_int32, c_int32,
        c_int64, c_int, c_int, c_void_p]),
    "fp_kv_gather": (c_int, [
        c_void_p, c_void_p, c_int64, c_int64, c_int64,
        c_void_p, c_int64, c_void_p, c_void_p, c_int,
        c_int32, c_int32, c_int32, c_int32, c_int32, c_int32, c_int32,
        c_int64, c_int, c_void_p]),
    "fp_convert_block_ids": (c_int, [
        c_void_p, c_void_p, c_void_p, c_int64, c_void_p,
        c_int32, c_int32, c_int32, c_int32, c_int32, c_void_p]),
    "fp_paged_decode_default_split": (c_int32, [c_int32, c_int32, c_int32, c_int32]),
    "fp_paged_decode_workspace_bytes": (c_int64, [c_int32, c_int32, c_int32, c_int32, c_int32]),
    "fp_paged_decode": (c_int, [
        c_void_p, c_int64, c_int64, c_void_p, c_void_p,
        c_void_p, c_int64, c_void_p, c_void_p, c_int,
        c_void_p, c_int64, c_int64, c_void_p, c_void_p,
        c_void_p, c_int64,
        c_int32, c_int32, c_int32, c_int32, c_int32, c_int32, c_int32, c_int32,
        c_int64, c_int32, c_int32, c_float, c_int, c_void_p, c_int64, c_void_p]),
    "fp_paged_decode_plan_bytes": (c_int64, []),
    "fp_paged_decode_plan": None,  # same signature as fp_paged_decode, filled in below
    "fp_paged_decode_partial": None,
    "fp_paged_decode_merge": None,
    "fp_paged_decode_append": None,  # two row pointers and four strides in front of the same list
    "fp_paged_decode_noalloc": None,  # the same list without the workspace pair
    "fp_qkv_norm_rope_append": (c_int, [
        c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int64, c_int64, c_int64,
        c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_void_p, c_void_p,
        c_void_p, c_int64, c_void_p, c_void_p, c_int,
        c_int32, c_int32, c_int32, c_int32, c_int32, c_int32, c_int32, c_int32,
        c_int64, c_float, c_int, c_int, c_void_p]),
    "fp_hybrid_row_limits": (c_int, [c_void_p, c_void_p, c_void_p, c_int32, c_int32, c_int64, c_int64,
                                     c_void_p, c_void_p, c_void_p]),
    "fp_paged_prefill": (c_int, [
        c_void_p, c_int64, c_int64, c_void_p, c_void_p,
        c_void_p, c_int64, c_void_p, c_void_p,
        c_void_p, c_int64, c_int64, c_void_p, c_void_p,
        c_int32, c_int32, c_int32, c_int32, c_int32, c_int32, c_int32,
        c_int64, c_float, c_float, c_int, c_void_p, c_int64, c_void_p, c_int32, c_void_p]),
    "fp_paged_prefill_tile_rows": (c_int32, [c_int32, c_int32, c_int32, c_int32, c_int, c_int64]),
    "fp_paged_prefill_tile_order": (c_int, [c_void_p, c_void_p, c_int32, c_int32, c_void_p, c_void_p]),
    "fp_paged_prefill_workspace_bytes": (c_int64, [c_int32, c_int32, c_int32, c_int32, c_int]),
}

SIGNATURES["fp_probe_mfma_softmax"] = (c_int, [c_int, c_int, c_int, c_int, c_void_p, c_int64, c_void_p])
SIGNATURES["fp_paged_decode_plan"] = SIGNATURES["fp_paged_decode"]
SIGNATURES["fp_paged_decode_partial"] = SIGNATURES["fp_paged_decode"]
SIGNATURES["fp_paged_decode_merge"] = SIGNATURES["fp_paged_decode"]
_d = SIGNATURES["fp_paged_decode"][1]
SIGNATURES["fp_paged_decode_noalloc"] = (c_int, _d[:15] + _d[17:-3] + _d[-1:])  # no workspace and no plan (pointer, size)
SIGNATURES["fp_paged_decode_append"] = (c_int, [c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int64]
                                        + SIGNATURES["fp_paged_decode"][1])

_lib = None


def lib() -> ctypes.CDLL:
    """The loaded library; raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing: build it with `python falcon-perception_amd/build_native.py` "
                "(hipcc, gfx950). This package has no other compute path."
            )
        handle = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(handle, name)  # AttributeError names a missing export
            fn.restype = res
            fn.argtypes = args
        got = handle.fp_abi_version()
        if got != FP_ABI_VERSION:
            raise RuntimeError(f"libfp_paged_kv.so has ABI {got}, this package expects {FP_ABI_VERSION}")
        _lib = handle
    return _lib


def check(rc: int, what: str) -> None:
    if rc < 0:
        msg = lib().fp_last_error().decode("utf-8", "replace")
        raise RuntimeError(f"{what} failed ({rc}): {msg}")


def stream_ptr(device) -> int:
    return torch.cuda.current_stream(device).cuda_stream


def require_cuda(*tensors) -> None:
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise RuntimeError(
                "falcon_perception_amd operators run on the GPU only (got a tensor on "
                f"{t.device}); there is no CPU path."
            )


def dtype_code(dtype: torch.dtype) -> int:
    try:
        return FP_DTYPE[dtype]
    except KeyError:
        raise RuntimeError(f"unsupported KV dtype {dtype}; supported: float32, bfloat16, float16") from None


def index_code(t: torch.Tensor) -> int:
    try:
        return FP_INDEX[t.dtype]
    except KeyError:
        raise RuntimeError(f"index tensor must be int32 or int64, got {t.dtype}") from None
