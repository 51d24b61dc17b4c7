"""ctypes binding of ``libmoba_hip.so`` (the C ABI declared in include/moba_hip.h).

The library is loaded from the package directory and nowhere else; if it is missing
the operator raises -- there is no fallback path.
"""

from __future__ import annotations

import ctypes
import os
from ctypes import POINTER, c_char_p, c_float, c_int, c_int64, c_size_t, c_void_p

c_strides = POINTER(c_int64)  # {q token, q head, k/v token, k/v head} in elements, or None for packed tensors

_HERE = os.path.dirname(os.path.abspath(__file__))
# MOBA_HIP_LIBRARY overrides the location (e.g. to try a differently built library)
LIB_PATH = os.environ.get("MOBA_HIP_LIBRARY") or os.path.join(_HERE, "libmoba_hip.so")

_lib = None

_SIGNATURES = {
    "moba_version": (c_int, []),
    "moba_strerror": (c_char_p, [c_int]),
    "moba_plan": (c_int, [c_void_p, c_int, c_int, c_int, c_int, c_void_p]),
    "moba_plan_fill": (c_int, [c_void_p, c_int, c_int, c_int, c_int, c_void_p, c_void_p]),
    "moba_plan_sizes": (c_int, [c_void_p, c_int, c_int, c_int, c_void_p]),
    "moba_chunk_mean_workspace_bytes": (c_size_t, [c_int, c_int, c_int, c_int]),
    "moba_chunk_mean": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int, c_int, c_int, c_int, c_strides,
                                c_int, c_void_p, c_int64, c_void_p]),
    "moba_chunk_mean_static_capacity": (c_size_t, []),
    "moba_chunk_mean_static": (c_int, [c_void_p, c_void_p, c_void_p, c_int64, c_int, c_int, c_int, c_int, c_strides,
                                       c_int, c_void_p]),
    "moba_gate_topk": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                               c_int64, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_strides, c_int,
                               c_void_p]),
    "moba_topk_from_scores": (c_int, [c_void_p, c_void_p, c_int64, c_int, c_int, c_int, c_void_p]),
    "moba_build_lists": (c_int, [c_void_p] * 10 + [c_int64] + [c_int] * 7 + [c_int64, c_int, c_int, c_void_p, c_void_p,
                                                                             c_int64, c_int, c_void_p]),
    "moba_tile_tables": (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int64, c_void_p]),
    "moba_fwd_tile_rows": (c_int, []),
    "moba_bwd_tile_rows": (c_int, []),
    "moba_fwd_partials": (c_int, [c_void_p] * 16 + [c_int64, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int64,
                                                   c_int64, c_int, c_strides, c_void_p, c_void_p, c_float, c_int,
                                                   c_int, c_int64, c_void_p]),
    "moba_fwd_merge": (c_int, [c_void_p] * 5 + [c_int64, c_int, c_int, c_int, c_int, c_void_p, c_void_p, c_int, c_int64,
                                               c_int, c_void_p]),
    "moba_fwd_key_split": (c_int, [c_int64, c_int, c_int, c_int, c_int64, c_int64]),
    "moba_fwd_is_queued": (c_int, [c_int64, c_int64, c_int]),
    "moba_fwd": (c_int, [c_void_p] * 17 + [c_int, c_int64, c_void_p, c_void_p,
                                          c_int64, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int64, c_int64,
                                          c_int, c_strides, c_void_p, c_void_p, c_float, c_int, c_void_p]),
    "moba_bwd_dkv_scratch_bytes": (ctypes.c_size_t, [c_int64, c_int, c_int64]),
    "moba_bwd_dq_key_split": (c_int, [c_int64, c_int, c_int, c_int, c_int64, c_int64]),
    "moba_bwd": (c_int, [c_void_p] * 23 + [c_int, c_int64] + [c_void_p] * 5 + [c_int64, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int64, c_int64,
                                          c_int64, c_int, c_strides, c_void_p, c_void_p, c_int64, c_float, c_int, c_void_p]),
    "moba_mfma_probe": (c_int, [c_void_p, c_void_p, c_int, c_int, c_void_p]),
    "moba_decode_splits": (c_int, [c_int, c_int, c_int]),
    "moba_decode": (c_int, [c_void_p] * 6 + [c_int] * 5 + [c_int64] * 4 + [c_float, c_int, c_void_p]),
}
OPTIONAL = set()


class PlanStruct(ctypes.Structure):
    """moba_plan_t of include/moba_hip.h."""
    _fields_ = ([("S", c_int64)] + [(n, ctypes.c_int32) for n in ("nseq", "chunk", "topk", "N", "F", "K", "P", "cmax", "fallback",
                                                               "fwd_tile_rows", "bwd_tile_rows", "dense_local", "NA")]
                + [("pairs_per_head", c_int64), ("fwd_self_tiles", c_int64), ("bwd_self_tiles", c_int64),
                   ("kv_tiles", c_int64), ("merge_tokens", c_int64), ("flops_per_head_per_dim", ctypes.c_double)]
                + [("off_" + n, c_int64) for n in ("cu_seqlens", "chunk_tok", "achunk_tok", "fwd_self_tile_prefix",
                                                   "fwd_self_tile_chunk", "self_tile_prefix", "self_tile_chunk",
                                                   "kv_tile_prefix", "kv_tile_chunk", "chunk_self_end", "achunk_direct",
                                                   "mrg_start", "mrg_prefix", "seq_fbase",
                                                   "fchunk_tok", "chunk_fb", "chunk_local", "pair_off", "chunk_fid")]
                + [("table_ints", c_int64)])


class SizesStruct(ctypes.Structure):
    """moba_sizes_t of include/moba_hip.h."""
    _fields_ = [(n, c_int64) for n in ("kbar_elems", "chunk_mean_workspace_bytes", "sel_ints", "cnt_ints", "seg_off_ints",
                                       "seg_dest_ints", "fwd_hist_bound", "bwd_hist_bound", "part_rows", "redo_ints",
                                       "lse_floats", "delta_floats")]
ABI_VERSION = 115  # MOBA_ABI_VERSION of include/moba_hip.h, the signatures above
DTYPE_BF16, DTYPE_F16 = 0, 1


def load():
    """Return the loaded library, building nothing: a missing library is an error."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            f"{LIB_PATH} is missing: build it with `python -m moba_amd.build` (needs hipcc, gfx950). "
            "moba_amd has no fallback implementation."
        )
    lib = ctypes.CDLL(LIB_PATH)
    for name, (res, args) in _SIGNATURES.items():
        try:
            fn = getattr(lib, name)
        except AttributeError:
            if name in OPTIONAL:
                continue
            raise
        fn.restype = res
        fn.argtypes = args
    if lib.moba_version() != ABI_VERSION:
        raise RuntimeError(f"{LIB_PATH} was built for version {lib.moba_version()} of the C ABI, this binding is for "
                           f"{ABI_VERSION}: rebuild it with `python -m moba_amd.build`")
    _lib = lib
    return lib


def exported_symbols():
    return list(_SIGNATURES)


def check(code: int, what: str):
    if code != 0:
        msg = load().moba_strerror(code).decode()
        raise RuntimeError(f"{what} failed with code {code}: {msg}")
