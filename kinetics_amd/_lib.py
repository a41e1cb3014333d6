"""ctypes binding of libkinetics_amd.so (the C ABI in include/kinetics_amd.h).

There is no CPU fallback: if the library is missing, loading raises and every
op of this package is unusable.
"""
from __future__ import annotations

import ctypes
from ctypes import c_char_p, c_float, c_int, c_int64, c_size_t, c_void_p
from pathlib import Path

# torch must be imported before the library is opened: both need the HIP runtime
# (libamdhip64.so.7) and the process must end up with exactly one copy of it --
# the one torch already loaded is found by its soname.
import torch  # noqa: F401

LIB_PATH = Path(__file__).resolve().parent / "libkinetics_amd.so"

KIN_OK = 0
KIN_ERR_NULL_POINTER = 1
KIN_ERR_BAD_SHAPE = 2
KIN_ERR_UNSUPPORTED = 3
KIN_ERR_WORKSPACE = 4
KIN_ERR_LAUNCH = 5
KIN_ERR_PAGE_TABLE = 6
KIN_ERR_MISALIGNED = 7

# name -> (restype, argtypes); mirrors include/kinetics_amd.h declaration by declaration.
_P = c_void_p
SIGNATURES = {
    "kin_version": (c_int, []),
    "kin_last_error": (c_char_p, []),
    "kin_status_string": (c_char_p, [c_int]),
    "kin_append_paged_kv": (c_int, [_P, _P, _P, _P, _P, _P, _P, c_int, c_int, c_int, c_int, c_int64, c_int, _P, c_int, _P]),
    "kin_append_paged_kv_ragged": (
        c_int,
        [_P, _P, _P, _P, _P, _P, _P, _P, c_int, c_int64, c_int, c_int, c_int, c_int, c_int64, c_int, _P, c_int, _P],
    ),
    "kin_build_kbar": (c_int, [_P, _P, _P, _P, _P, c_int, c_int, c_int, c_int, c_int64, c_int, _P, c_int, _P]),
    "kin_block_score_topk": (
        c_int,
        [_P, _P, _P, _P, _P, c_int, c_int, c_int, _P, _P, _P, _P, c_int, c_int, c_int, c_int, c_int, c_int, c_int, _P,
         c_size_t, _P, c_int, _P],
    ),
    "kin_sel_list_capacity": (c_int, [c_int, c_int, c_int]),
    "kin_decode_workspace_bytes": (c_size_t, [c_int, c_int, c_int, c_int, c_int, c_int]),
    "kin_decode_auto_splits": (c_int, [c_int, c_int, c_int]),
    "kin_sparse_paged_decode": (
        c_int,
        [_P, _P, _P, _P, _P, _P, _P, _P, c_size_t, c_int, c_int, c_int, c_int, c_int, c_int64, c_int, c_int, c_float,
         c_int, _P],
    ),
    "kin_dense_paged_decode": (
        c_int,
        [_P, _P, _P, _P, _P, _P, _P, _P, c_size_t, c_int, c_int, c_int, c_int, c_int, c_int64, c_int, c_int, c_float,
         c_int, _P],
    ),
    "kin_blocktopk_decode_step": (
        c_int,
        [_P, _P, _P, _P, _P, _P, _P, _P, c_int, c_int, c_int, _P, _P, _P, _P, c_int, c_int, c_int, c_int, c_int, c_int64,
         c_int, c_int, c_int, c_float, _P, c_size_t, _P, c_int, _P, _P],
    ),
    "kin_step_workspace_bytes": (c_size_t, [c_int, c_int, c_int]),
    "kin_static_scratch_bytes": (c_size_t, []),
    "kin_set_team_spin_limit": (c_int, [c_int]),
    "kin_blocktopk_decode_step_static": (
        c_int,
        [_P, _P, _P, _P, _P, _P, _P, _P, c_int, c_int, c_int, _P, _P, _P, _P, c_int, c_int, c_int, c_int, c_int, c_int64,
         c_int, c_int, c_int, c_float, _P, c_int, _P, _P],
    ),
    "kin_token_topk_workspace_bytes": (c_size_t, [c_int, c_int, c_int]),
    "kin_token_topk_decode": (
        c_int,
        [_P, _P, _P, _P, _P, c_int, c_int, c_int, c_int, _P, _P, _P, _P, _P, c_size_t, c_int, c_int, c_int, c_int, c_int,
         c_int64, c_int, c_int, c_float, _P],
    ),
    "kin_strided_topk_workspace_bytes": (c_size_t, [c_int, c_int, c_int]),
    "kin_strided_topk_decode": (
        c_int,
        [_P, _P, _P, _P, _P, c_int, c_int, c_int, c_int, c_int, c_int, _P, _P, _P, _P, _P, c_size_t, c_int, c_int, c_int,
         c_int, c_int, c_int64, c_int, c_int, c_float, _P],
    ),
    "kin_build_slot_page_table": (c_int, [_P, _P, c_int, c_int, c_int, _P, _P, _P, _P]),
    "kin_page_pool_init": (c_int, [_P, _P, _P, c_int, c_int, _P]),
    "kin_page_pool_reserve": (c_int, [_P, _P, c_int, c_int, c_int, _P, _P, _P, _P, c_int, _P]),
    "kin_page_pool_release": (c_int, [_P, c_int, c_int, _P, _P, _P, _P, c_int, c_int, _P]),
    "kin_build_pool_page_table": (c_int, [_P, _P, c_int, c_int, c_int, _P, _P, _P, _P, _P, c_int, _P]),
    "kin_check_page_table": (c_int, [_P, _P, _P, c_int, c_int, c_int64, c_int64, _P, _P]),
    "kin_rms_norm": (c_int, [_P, _P, _P, _P, c_int64, c_int, c_int64, c_int64, c_float, _P]),
    "kin_qkv_norm_split": (c_int, [_P, c_int64, _P, _P, c_float, _P, _P, _P, c_int, c_int, c_int, c_int, _P]),
    "kin_gated_act": (c_int, [_P, _P, _P, c_int64, c_int, c_int64, c_int64, c_int, _P]),
}

# the float16 twins have the signatures of their bfloat16 originals
for _name in ("kin_append_paged_kv", "kin_build_kbar", "kin_append_paged_kv_ragged", "kin_block_score_topk",
              "kin_sparse_paged_decode", "kin_dense_paged_decode", "kin_blocktopk_decode_step", "kin_rms_norm",
              "kin_qkv_norm_split", "kin_gated_act", "kin_token_topk_decode", "kin_strided_topk_decode"):
    SIGNATURES[_name + "_f16"] = SIGNATURES[_name]

_lib = None


class KineticsError(RuntimeError):
    """A non-OK status from the C ABI that is not an argument error."""


def load() -> ctypes.CDLL:
    """Open the library once and bind every declared entry point."""
    global _lib
    if _lib is not None:
        return _lib
    if not LIB_PATH.exists():
        raise ImportError(
            f"{LIB_PATH} is missing: build it with `python -m kinetics_amd.build` "
            "(there is no fallback implementation)"
        )
    lib = ctypes.CDLL(str(LIB_PATH))
    for name, (restype, argtypes) in SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError if the symbol is not exported
        fn.restype = restype
        fn.argtypes = argtypes
    _lib = lib
    return lib


def check(status: int) -> None:
    """Raise the Python exception that corresponds to a C status code:
    argument errors -> ValueError, everything else -> KineticsError."""
    if status == KIN_OK:
        return
    lib = load()
    name = lib.kin_status_string(status).decode()
    msg = lib.kin_last_error().decode()
    text = f"{name}: {msg}"
    if status in (KIN_ERR_NULL_POINTER, KIN_ERR_BAD_SHAPE, KIN_ERR_UNSUPPORTED, KIN_ERR_MISALIGNED):
        raise ValueError(text)
    raise KineticsError(text)
