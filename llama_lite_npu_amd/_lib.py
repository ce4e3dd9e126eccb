"""ctypes binding of liblitekv.so (the C ABI declared in include/litekv.h).

The library is the only implementation of the path: if it has not been built
(``python -m llama_lite_npu_amd.build``) loading raises, there is no CPU or
PyTorch fallback behind these functions.
"""

from __future__ import annotations

import ctypes
from ctypes import c_char_p, c_float, c_int32, c_int64, c_size_t, c_void_p
from pathlib import Path

# PyTorch-ROCm ships its own HIP runtime under the soname the library links
# against; importing torch first makes both share one runtime (and one set of
# streams and allocations).
import torch  # noqa: F401

LIB_PATH = Path(__file__).resolve().parent / "csrc" / "liblitekv.so"

ABI_VERSION = 3

# name -> (restype, argtypes); mirrors include/litekv.h declaration by declaration.
SIGNATURES = {
    "litekv_abi_version": (c_int32, []),
    "litekv_last_error": (c_char_p, []),
    "litekv_kv_append": (
        c_int32,
        [c_void_p, c_void_p, c_int64, c_int64, c_void_p, c_void_p, c_int32, c_int32, c_int32,
         c_int64, c_void_p],
    ),
    "litekv_qk_norm_rope_append": (
        c_int32,
        [c_void_p, c_int64, c_void_p, c_int64, c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_void_p,
         c_int64, c_void_p, c_void_p, c_int32, c_int32, c_int32, c_int32, c_int64, c_float, c_void_p],
    ),
    "litekv_page_gather": (
        c_int32,
        [c_void_p, c_void_p, c_void_p, c_void_p, c_int32, c_int64, c_int64, c_int64, c_void_p],
    ),
    "litekv_page_copy": (
        c_int32,
        [c_void_p, c_void_p, c_void_p, c_int32, c_int64, c_int64, c_void_p],
    ),
    "litekv_paged_decode_workspace_bytes": (c_size_t, [c_int32, c_int32, c_int32, c_int32]),
    "litekv_paged_decode": (
        c_int32,
        [c_void_p, c_int64, c_void_p, c_void_p, c_int32, c_void_p, c_void_p, c_void_p, c_size_t,
         c_int32, c_int32, c_int32, c_int32, c_int32, c_int64, c_int32, c_int32, c_float,
         c_void_p],
    ),
    "litekv_paged_decode_static": (
        c_int32,
        [c_void_p, c_int64, c_void_p, c_void_p, c_int32, c_void_p, c_void_p,
         c_int32, c_int32, c_int32, c_int32, c_int32, c_int64, c_int32, c_int32, c_float,
         c_void_p],
    ),
    "litekv_paged_decode_fp8": (
        c_int32,
        [c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_int32, c_void_p, c_void_p, c_void_p, c_size_t,
         c_int32, c_int32, c_int32, c_int32, c_int32, c_int64, c_int32, c_int32, c_float,
         c_void_p],
    ),
    "litekv_paged_decode_int8": (
        c_int32,
        [c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_int32, c_void_p, c_void_p, c_void_p, c_size_t,
         c_int32, c_int32, c_int32, c_int32, c_int32, c_int64, c_int32, c_int32, c_float,
         c_void_p],
    ),
    "litekv_paged_decode_append": (
        c_int32,
        [c_void_p, c_int64, c_void_p, c_void_p, c_int32, c_void_p, c_void_p, c_void_p, c_int64, c_int64,
         c_void_p, c_void_p, c_size_t, c_int32, c_int32, c_int32, c_int32, c_int32, c_int64, c_int32,
         c_int32, c_float, c_void_p],
    ),
    "litekv_paged_decode_append_fp8": (
        c_int32,
        [c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_int32, c_void_p, c_void_p, c_void_p, c_int64,
         c_int64, c_void_p, c_void_p, c_size_t, c_int32, c_int32, c_int32, c_int32, c_int32, c_int64,
         c_int32, c_int32, c_float, c_void_p],
    ),
    "litekv_paged_decode_append_int8": (
        c_int32,
        [c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_int32, c_void_p, c_void_p, c_void_p, c_int64,
         c_int64, c_void_p, c_void_p, c_size_t, c_int32, c_int32, c_int32, c_int32, c_int32, c_int64,
         c_int32, c_int32, c_float, c_void_p],
    ),
    "litekv_paged_decode_split": (
        c_int32,
        [c_void_p, c_int64, c_void_p, c_void_p, c_int32, c_void_p, c_void_p, c_void_p, c_size_t,
         c_int32, c_int32, c_int32, c_int32, c_int32, c_int64, c_int32, c_int32, c_float,
         c_void_p],
    ),
    "litekv_paged_decode_merge": (
        c_int32,
        [c_void_p, c_void_p, c_void_p, c_size_t, c_int32, c_int32, c_int32, c_int32, c_int32,
         c_int32, c_void_p],
    ),
    "litekv_paged_decode_balanced_chunks": (c_int32, [c_int32]),
    "litekv_paged_decode_prefix_chunks": (c_int32, [c_int32, c_int32, c_int32, c_int32, c_int32, c_int32, c_int32]),
    "litekv_paged_decode_balanced_workspace_bytes": (c_size_t, [c_int32, c_int32, c_int32, c_int32]),
    "litekv_decode_plan_bytes": (c_size_t, [c_int32, c_int32, c_int32, c_int32]),
    "litekv_decode_plan_bytes_paged": (c_size_t, [c_int32, c_int32, c_int32, c_int32, c_int32]),
    "litekv_decode_plan": (
        c_int32,
        [c_void_p, c_int32, c_void_p, c_int32, c_int32, c_int32, c_int64, c_int32, c_void_p, c_size_t,
         c_void_p],
    ),
    "litekv_paged_decode_balanced": (
        c_int32,
        [c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_size_t, c_void_p, c_void_p, c_int64,
         c_int64, c_void_p, c_void_p, c_size_t, c_int32, c_int32, c_int32, c_int32, c_int32,
         c_int64, c_int32, c_int32, c_float, c_void_p],
    ),
    "litekv_paged_decode_prefix_workspace_bytes": (c_size_t, [c_int32, c_int32, c_int32, c_int32]),
    "litekv_decode_plan_prefix": (
        c_int32,
        [c_void_p, c_int32, c_void_p, c_int32, c_int32, c_int32, c_int64, c_int32, c_int32, c_void_p,
         c_size_t, c_void_p],
    ),
    "litekv_paged_decode_prefix": (
        c_int32,
        [c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_void_p, c_size_t, c_void_p, c_void_p,
         c_int64, c_int64, c_void_p, c_void_p, c_size_t, c_int32, c_int32, c_int32, c_int32, c_int32,
         c_int64, c_int32, c_int32, c_int32, c_float, c_void_p],
    ),
    "litekv_paged_decode_prefix_fp8": (
        c_int32,
        [c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_size_t, c_void_p, c_void_p,
         c_int64, c_int64, c_void_p, c_void_p, c_size_t, c_int32, c_int32, c_int32, c_int32, c_int32,
         c_int64, c_int32, c_int32, c_int32, c_float, c_void_p],
    ),
    "litekv_paged_decode_prefix_int8": (
        c_int32,
        [c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_size_t, c_void_p, c_void_p,
         c_int64, c_int64, c_void_p, c_void_p, c_size_t, c_int32, c_int32, c_int32, c_int32, c_int32,
         c_int64, c_int32, c_int32, c_int32, c_float, c_void_p],
    ),
    "litekv_kv_append_fp8": (
        c_int32,
        [c_void_p, c_void_p, c_int64, c_int64, c_void_p, c_void_p, c_void_p, c_int32, c_int32, c_int32,
         c_int64, c_void_p],
    ),
    "litekv_kv_append_int8": (
        c_int32,
        [c_void_p, c_void_p, c_int64, c_int64, c_void_p, c_void_p, c_void_p, c_int32, c_int32, c_int32,
         c_int64, c_void_p],
    ),
    "litekv_qk_norm_rope_append_fp8": (
        c_int32,
        [c_void_p, c_int64, c_void_p, c_int64, c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_void_p,
         c_int64, c_void_p, c_void_p, c_void_p, c_int32, c_int32, c_int32, c_int32, c_int64, c_float, c_void_p],
    ),
    "litekv_qk_norm_rope_append_int8": (
        c_int32,
        [c_void_p, c_int64, c_void_p, c_int64, c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_void_p,
         c_int64, c_void_p, c_void_p, c_void_p, c_int32, c_int32, c_int32, c_int32, c_int64, c_float, c_void_p],
    ),
    "litekv_page_dequant": (
        c_int32,
        [c_void_p, c_void_p, c_void_p, c_void_p, c_int32, c_void_p, c_int32, c_int32, c_int32, c_int64,
         c_int64, c_void_p],
    ),
    "litekv_page_dequant_int8": (
        c_int32,
        [c_void_p, c_void_p, c_void_p, c_void_p, c_int32, c_void_p, c_int32, c_int32, c_int32, c_int64,
         c_int64, c_void_p],
    ),
    "litekv_paged_decode_balanced_fp8": (
        c_int32,
        [c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_void_p, c_size_t, c_void_p, c_void_p, c_int64,
         c_int64, c_void_p, c_void_p, c_size_t, c_int32, c_int32, c_int32, c_int32, c_int32,
         c_int64, c_int32, c_int32, c_float, c_void_p],
    ),
    "litekv_paged_decode_balanced_int8": (
        c_int32,
        [c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_void_p, c_size_t, c_void_p, c_void_p, c_int64,
         c_int64, c_void_p, c_void_p, c_size_t, c_int32, c_int32, c_int32, c_int32, c_int32,
         c_int64, c_int32, c_int32, c_float, c_void_p],
    ),
    "litekv_decode_advance": (
        c_int32,
        [c_void_p, c_int64, c_int32, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
         c_int64, c_int32, c_void_p, c_int32, c_int32, c_int64, c_int32, c_void_p],
    ),
    "litekv_profile_next_decode": (c_int32, [c_void_p, c_void_p]),
    "litekv_paged_prefill": (
        c_int32,
        [c_void_p, c_int64, c_void_p, c_void_p, c_int32, c_void_p, c_void_p, c_void_p, c_int64,
         c_int32, c_int32, c_int32, c_int32, c_int32, c_int64, c_int32, c_float, c_void_p],
    ),
    "litekv_paged_prefill_split_workspace_bytes": (c_size_t, [c_int64, c_int32, c_int32, c_int32]),
    "litekv_paged_prefill_key_slices": (c_int32, [c_int32, c_int32, c_int32, c_int32, c_int32, c_int64]),
    "litekv_paged_prefill_split": (
        c_int32,
        [c_void_p, c_int64, c_void_p, c_void_p, c_int32, c_void_p, c_void_p, c_void_p, c_int64,
         c_int32, c_int32, c_int32, c_int32, c_int32, c_int64, c_int32, c_int64, c_int32, c_void_p, c_size_t,
         c_float, c_void_p],
    ),
    "litekv_paged_prefill_split_q8": (
        c_int32,
        [c_void_p, c_int64, c_void_p, c_void_p, c_int32, c_void_p, c_int32, c_void_p, c_void_p, c_void_p, c_int64,
         c_int32, c_int32, c_int32, c_int32, c_int32, c_int64, c_int32, c_int64, c_int32, c_void_p, c_size_t,
         c_float, c_void_p],
    ),
    "litekv_paged_prefill_fp8": (
        c_int32,
        [c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_int32, c_void_p, c_void_p, c_void_p, c_int64,
         c_int32, c_int32, c_int32, c_int32, c_int32, c_int64, c_int32, c_float, c_void_p],
    ),
    "litekv_paged_prefill_int8": (
        c_int32,
        [c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_int32, c_void_p, c_void_p, c_void_p, c_int64,
         c_int32, c_int32, c_int32, c_int32, c_int32, c_int64, c_int32, c_float, c_void_p],
    ),
    "litekv_varlen_prefill": (
        c_int32,
        [c_void_p, c_int64, c_void_p, c_int64, c_void_p, c_int64, c_void_p, c_void_p, c_void_p,
         c_int64, c_int32, c_int32, c_int32, c_int32, c_int32, c_int64, c_float, c_void_p],
    ),
}

_lib = None


class LiteKVError(RuntimeError):
    """A liblitekv entry point returned a non-zero status."""


def load() -> ctypes.CDLL:
    """Loads liblitekv.so once and declares every prototype."""
    global _lib
    if _lib is not None:
        return _lib
    if not LIB_PATH.exists():
        raise LiteKVError(
            f"{LIB_PATH} is missing: build it with `python -m llama_lite_npu_amd.build` "
            "(there is no fallback implementation)"
        )
    lib = ctypes.CDLL(str(LIB_PATH))
    for name, (restype, argtypes) in SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError names a symbol the library does not export
        fn.restype = restype
        fn.argtypes = argtypes
    got = lib.litekv_abi_version()
    if got != ABI_VERSION:
        raise LiteKVError(f"liblitekv ABI {got} != binding ABI {ABI_VERSION}; rebuild the library")
    _lib = lib
    return lib


def check(status: int) -> None:
    """Raises LiteKVError carrying litekv_last_error() when status != 0."""
    if status != 0:
        msg = load().litekv_last_error()
        raise LiteKVError(f"liblitekv status {status}: {msg.decode() if msg else '?'}")
