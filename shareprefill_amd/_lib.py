"""ctypes binding of libshareprefill_hip.so (the C ABI declared in include/shareprefill_hip.h).

There is no fallback: if the library is missing or a symbol is absent, importing the product path
raises.  Build the library with `python -m shareprefill_amd.build`.
"""

from __future__ import annotations

import ctypes as C
import os

# SHAREPREFILL_HIP_LIB overrides the in-tree library path (e.g. to try an experimental build)
LIB_PATH = os.environ.get("SHAREPREFILL_HIP_LIB") or os.path.join(os.path.dirname(os.path.abspath(__file__)), "csrc",
                                                                  "libshareprefill_hip.so")

SP_DEC_VS, SP_DEC_DENSE, SP_DEC_SHARE, SP_DEC_QA = 0, 1, 2, 3
SP_FLAG_LOGITS_BF16 = 1


def SP_FLAG_SCALE_DIM(head_dim: int) -> int:
    """flags bits 8..15: the head_dim the selection's 1/sqrt(head_dim) is formed from when q / k are zero-padded."""
    return (head_dim // 8) << 8


SP_POOL_TAIL_TRUE_LENGTH, SP_POOL_TAIL_RESCALE = 0, 1
SP_POOL_TYPES = {"avg": 0, "max": 1, "min": 2, "maxabs": 3, "sum": 4}  # attn/utils.py:255
SP_ATTN_V_REPACKED = 1
SP_ATTN_PAIR_ROWS = 2
SP_ATTN_HALF_CHANNELS = 4
SP_DECODE_STATIC_SCRATCH_BYTES = 8 << 20


class ClusterStateStruct(C.Structure):
    """struct sp_cluster_state (host struct holding device pointers)."""

    _fields_ = [
        ("n_clusters", C.c_int32), ("nb", C.c_int32), ("nbw", C.c_int32), ("struct_bytes", C.c_int32),
        ("info", C.c_void_p), ("ratio", C.c_void_p), ("vert", C.c_void_p), ("slash", C.c_void_p),
        ("cols", C.c_void_p), ("dists", C.c_void_p), ("pattern", C.c_void_p), ("accum", C.c_void_p),
        ("avg_map", C.c_void_p),
    ]


_P, _I64, _I32, _U32, _F, _D, _SZ = C.c_void_p, C.c_int64, C.c_int32, C.c_uint32, C.c_float, C.c_double, C.c_size_t
_ST = C.POINTER(ClusterStateStruct)

# name -> (restype, argtypes); must list every function the header declares
SIGNATURES = {
    "sp_version": (_I32, []),
    "sp_arch": (C.c_char_p, []),
    "sp_last_error": (C.c_char_p, []),
    "sp_diag_mfma_bf16": (_I32, [_I32, _I32, _P, _P]),
    "sp_diag_mfma_flops": (_D, [_I32]),
    "sp_pool_avg_bf16": (_I32, [_P, _P, _I64, _I32, _I32, _I64, _I64, _I32, _I32, _P, _P]),
    "sp_pool_bf16": (_I32, [_P, _P, _I64, _I32, _I32, _I64, _I64, _I32, _I32, _P]),
    "sp_lastq_scores_workspace_bytes": (_SZ, [_I64, _I32, _I32]),
    "sp_lastq_scores_bf16": (_I32, [_P, _P, _I64, _I32, _I32, _I32, _I64, _I64, _I64, _I64, _I32, _U32, _P, _SZ,
                                    _P, _P, _P, _P, _P]),
    "sp_cover_count": (_I32, [_P, _I32, _I64, _F, _P, _P, _SZ, _P]),
    "sp_cover_budgets": (_I32, [_P, _P, _I32, _I64, _I32, _F, _I32, _I32, _P, _P, _P, _SZ, _P]),
    "sp_queryaware_test_bf16": (_I32, [_P, _P, _P, _I64, _I32, _I32, _I32, _I64, _I64, _I32, _U32, _F, _P, _P, _P,
                                       _P]),
    "sp_share_decide": (_I32, [_ST, _P, _I32, _I32, _P, _P, _P, _P, _P, _I32, _F, _D, _P, _P, _P, _P, _P, _P]),
    "sp_build_mask": (_I32, [_ST, _P, _P, _P, _P, _P, _P, _I32, _I32, _P, _P]),
    "sp_queryaware_select_score": (_F, [_D, _I32]),
    "sp_queryaware_select_bf16": (_I32, [_P, _P, _P, _I32, _I32, _I32, _I32, _U32, _D, _P, _P, _P, _SZ, _P]),
    "sp_cover_select_workspace_bytes": (_SZ, [_I32]),
    "sp_cover_select_global": (_I32, [_P, _P, _I32, _I32, _F, _P, _P, _SZ, _P]),
    "sp_attn_workspace_bytes": (_SZ, [_I64, _I32, _I32, _I32, _I32]),
    "sp_attn_pivot_scratch_bytes": (_SZ, [_I64, _I32]),
    "sp_attn_last_launch_clocks": (_I32, [_P, _I64, _I32, _I32, _I32, _P, _P]),
    "sp_attn_last_launch_pairing": (_I32, [_P, _I64, _I32, _I32, _I32, _I32, _P, _P]),
    "sp_attn_repack_v_bf16": (_I32, [_P, _I64, _I32, _I32, _I64, _I64, _I32, _P, _SZ, _P]),
    "sp_block_sparse_attn_fwd_bf16": (_I32, [_P, _P, _P, _I64, _I32, _I32, _I32, _I64, _I64, _I64, _I64, _I64, _I64,
                                             _I32, _F, _P, _P, _P, _P, _P, _SZ, _U32, _P]),
    "sp_decode_workspace_bytes": (_SZ, [_I64, _I32, _I32]),
    "sp_decode_attn_bf16": (_I32, [_P, _P, _P, _I64, _I32, _I32, _I32, _I64, _I64, _I64, _I64, _I64, _F, _P, _P, _SZ,
                                   _P]),
    "sp_decode_attn_static_bf16": (_I32, [_P, _P, _P, _I64, _I32, _I32, _I32, _I64, _I64, _I64, _I64, _I64, _F, _P, _P]),
    "sp_rope_inplace_bf16": (_I32, [_P, _P, _P, _P, _I64, _I32, _I32, _I32, _I64, _I64, _I64, _I64, _I64, _P]),
    "sp_pivot_update": (_I32, [_ST, _P, _P, _P, _I32, _I32, _F, _P]),
    "sp_cover_select_rows": (_I32, [_P, _I32, _F, _P, _P]),
    "sp_mask_row_pointers": (_I32, [_P, _I32, _I32, _P, _P]),
    "sp_block_idx_to_mask": (_I32, [_P, _I64, _I64, _I32, _I32, _P, _P]),
    "sp_block_idx_row_pointers": (_I32, [_P, _I64, _I64, _I32, _I32, _P, _P]),
}

_lib = None


class SharePrefillLibraryError(RuntimeError):
    pass


def load(path: str = LIB_PATH):
    """Loads the shared library and binds every declared entry point.  Raises if anything is missing."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(path):
        raise SharePrefillLibraryError(
            f"{path} not found: the HIP extension is not built (python -m shareprefill_amd.build). "
            "There is no CPU fallback for the SharePrefill attention path.")
    lib = C.CDLL(path)
    for name, (res, args) in SIGNATURES.items():
        try:
            fn = getattr(lib, name)
        except AttributeError as exc:
            raise SharePrefillLibraryError(f"{path} does not export {name}") from exc
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


def check(status: int, what: str):
    if status != 0:
        msg = load().sp_last_error().decode("utf-8", "replace")
        if status == -2:
            raise NotImplementedError(f"{what}: {msg}")
        if status == -1:
            raise ValueError(f"{what}: {msg}")
        raise RuntimeError(f"{what} failed with status {status}: {msg}")
