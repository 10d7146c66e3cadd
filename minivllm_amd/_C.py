"""ctypes binding of libminivllm_amd.so (the C ABI in include/minivllm_amd.h).

There is no CPU or PyTorch fallback: if the library is missing or a call
fails, the operators raise.
"""
from __future__ import annotations

import ctypes
import os

import torch

_LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "libminivllm_amd.so")
_lib = None

DTYPE_CODES = {torch.float32: 0, torch.bfloat16: 1, torch.float16: 2}

c_void_p, c_int, c_int64, c_size_t, c_float = (ctypes.c_void_p, ctypes.c_int, ctypes.c_int64,
                                                ctypes.c_size_t, ctypes.c_float)
c_uint64 = ctypes.c_uint64

# name -> (restype, argtypes); mirrors include/minivllm_amd.h one to one
SIGNATURES = {
    "mvllm_version": (c_int, []),
    "mvllm_status_string": (ctypes.c_char_p, [c_int]),
    "mvllm_store_kvcache": (c_int, [c_void_p] * 5 + [c_int64, c_int64, c_int, c_int, c_int, c_void_p]),
    "mvllm_store_kvcache_int8": (c_int, [c_void_p] * 7 + [c_int64, c_int64, c_int, c_int, c_int, c_void_p]),
    "mvllm_paged_decode_workspace_bytes": (c_size_t, [c_int] * 5),
    "mvllm_paged_decode_plan": (c_int, [c_int] * 8 + [ctypes.POINTER(c_int)] * 3),
    "mvllm_paged_decode": (c_int, [c_void_p] * 5 + [c_int, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int,
                                                     c_int64, c_float, c_int, c_void_p, c_size_t, c_void_p]),
    "mvllm_paged_decode_noalloc": (c_int, [c_void_p] * 5 + [c_int, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int,
                                                             c_int64, c_float, c_int, c_void_p]),
    "mvllm_paged_decode_int8": (c_int, [c_void_p] * 7 + [c_int, c_void_p, c_int, c_int, c_int, c_int, c_int,
                                                          c_int, c_int64, c_float, c_int, c_void_p, c_size_t,
                                                          c_void_p]),
    "mvllm_prefill_plan": (c_int, [c_int] * 6 + [ctypes.POINTER(c_int)]),
    "mvllm_prefill_varlen": (c_int, [c_void_p] * 5 + [c_int, c_int64, c_int, c_int, c_int, c_float, c_int,
                                                       c_void_p]),
    "mvllm_prefill_paged": (c_int, [c_void_p] * 5 + [c_int, c_void_p, c_void_p, c_int, c_int64, c_int, c_int, c_int,
                                                      c_int, c_int64, c_float, c_int, c_void_p]),
    "mvllm_prefill_paged_int8": (c_int, [c_void_p] * 7 + [c_int, c_void_p, c_void_p, c_int, c_int64, c_int, c_int, c_int,
                                           c_int, c_int64, c_float, c_int, c_void_p]),
    "mvllm_prefill_paged_staged_workspace_bytes": (c_size_t, [c_int] * 7),
    "mvllm_prefill_paged_staged": (c_int, [c_void_p] * 5 + [c_int, c_void_p, c_void_p, c_int, c_int64, c_int, c_int, c_int, c_int,
                                             c_int, c_int64, c_float, c_int, c_void_p, c_size_t, c_void_p]),
    "mvllm_prefill_paged_int8_staged": (c_int, [c_void_p] * 7 + [c_int, c_void_p, c_void_p, c_int, c_int64, c_int, c_int, c_int, c_int,
                                                  c_int, c_int64, c_float, c_int, c_void_p, c_size_t, c_void_p]),
    "mvllm_prefill_paged_split_plan": (c_int, [c_int, c_int64] + [c_int] * 7),
    "mvllm_prefill_paged_split_workspace_bytes": (c_size_t, [c_int, c_int64] + [c_int] * 7),
    "mvllm_prefill_paged_split": (c_int, [c_void_p] * 5 + [c_int, c_void_p, c_void_p, c_int, c_int64, c_int, c_int, c_int, c_int,
                                            c_int, c_int64, c_float, c_int, c_int, c_void_p, c_size_t, c_void_p]),
    "mvllm_prefill_paged_int8_split": (c_int, [c_void_p] * 7 + [c_int, c_void_p, c_void_p, c_int, c_int64, c_int, c_int, c_int, c_int,
                                                 c_int, c_int64, c_float, c_int, c_int, c_void_p, c_size_t, c_void_p]),
    "mvllm_sample_tokens_workspace_bytes": (c_size_t, [c_int, c_int]),
    "mvllm_sample_tokens": (c_int, [c_void_p, c_void_p, c_int64, c_void_p, c_void_p, c_uint64, c_uint64, c_int, c_int,
                                    c_int, c_void_p, c_size_t, c_void_p]),
    "mvllm_sample_tokens_dev_offset": (c_int, [c_void_p, c_void_p, c_int64, c_void_p, c_uint64, c_void_p, c_int, c_int,
                                               c_int, c_void_p, c_size_t, c_void_p]),
    "mvllm_decode_advance": (c_int, [c_void_p] * 7 + [c_int64, c_int, c_void_p]),
    "mvllm_add_rms_norm": (c_int, [c_void_p] * 5 + [c_float, c_int64, c_int, c_int64, c_int64, c_int, c_void_p]),
    "mvllm_silu_and_mul": (c_int, [c_void_p, c_void_p, c_int64, c_int, c_int64, c_int, c_void_p]),
    "mvllm_lm_head_sample_workspace_bytes": (c_size_t, [c_int, c_int]),
    "mvllm_lm_head_sample": (c_int, [c_void_p, c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_uint64,
                                     c_uint64, c_void_p, c_int, c_int, c_int, c_int, c_void_p, c_size_t,
                                     c_void_p]),
    "mvllm_linear_small_m": (c_int, [c_void_p] * 4 + [c_int64, c_int, c_int, c_int, c_int, c_void_p]),
    "mvllm_norm_linear_small_m": (c_int, [c_void_p] * 5 + [c_float, c_void_p, c_void_p, c_int64, c_int, c_int, c_int,
                                                            c_int, c_int, c_void_p]),
    "mvllm_linear_small_m_plan": (c_int, [c_int] * 6 + [ctypes.POINTER(c_int)]),
    "mvllm_qk_norm_rope_store": (c_int, [c_void_p] * 6 + [c_int64] * 3 + [c_void_p, c_float, c_void_p, c_int64,
                                                           c_void_p, c_void_p] + [c_void_p] * 4 +
                                 [c_int, c_int64, c_int64, c_int, c_int, c_int, c_int, c_void_p]),
}


class MinivllmAmdError(RuntimeError):
    pass


def lib_path() -> str:
    return _LIB_PATH


def load():
    """Load the shared library once; raise if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(_LIB_PATH):
        raise MinivllmAmdError(
            f"{_LIB_PATH} not found: build it with `python -m minivllm_amd._build` "
            "(there is no fallback path)")
    lib = ctypes.CDLL(_LIB_PATH)
    for name, (restype, argtypes) in SIGNATURES.items():
        fn = getattr(lib, name)      # AttributeError if the symbol is missing
        fn.restype = restype
        fn.argtypes = argtypes
    _lib = lib
    return lib


def check(status: int, what: str) -> None:
    """0 -> ok; <0 -> ValueError with the library's text; >0 -> RuntimeError (hipError_t)."""
    if status == 0:
        return
    if status < 0:
        text = load().mvllm_status_string(status).decode()
        raise ValueError(f"{what}: {text} (status {status})")
    raise MinivllmAmdError(f"{what}: HIP error {status}")


def dtype_code(dtype: torch.dtype) -> int:
    try:
        return DTYPE_CODES[dtype]
    except KeyError:
        raise ValueError(f"unsupported dtype {dtype}; expected float32, bfloat16 or float16") from None


def current_stream_ptr(device) -> int:
    return torch.cuda.current_stream(device).cuda_stream


def require_cuda(*tensors) -> None:
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise MinivllmAmdError("minivllm_amd operators need tensors on a GPU device; "
                                   "there is no CPU path")
