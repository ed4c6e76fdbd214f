"""ctypes binding of libblockrank_hip.so (the C ABI declared in include/blockrank_hip.h).

There is no fallback: if the library is missing, every entry point raises.  Build it with
``python -m blockrank_amd.build``.
"""
from __future__ import annotations

import ctypes
from ctypes import c_char_p, c_float, c_int, c_int64, c_size_t, c_void_p
from pathlib import Path

LIB_PATH = Path(__file__).resolve().parent / "libblockrank_hip.so"

BR_DTYPE_F32 = 0
BR_DTYPE_BF16 = 1
BR_DTYPE_F16 = 2

BR_ERR_ARG = 1
BR_ERR_SPACE = 2
BR_ERR_HIP = 3
BR_ERR_PLAN = 4

_I64x3 = c_int64 * 3


class BrPrefillOptions(ctypes.Structure):
    """struct BrPrefillOptions of include/blockrank_hip.h (same members, same order)."""
    _fields_ = [("struct_bytes", c_size_t), ("ev_start", c_void_p), ("ev_stop", c_void_p), ("score_part", c_void_p),
                ("score_part_bytes", c_size_t), ("score_rows", ctypes.c_int32), ("rank_R", ctypes.c_int32), ("fp8_tokens", c_int64),
                ("lse", c_void_p), ("lse_strides", c_void_p), ("rope_cos", c_void_p), ("rope_sin", c_void_p),
                ("rope_strides", c_void_p), ("rank_rows", c_void_p), ("rank_scores", c_void_p), ("rank_scale", c_float)]


# name -> (restype, argtypes); the single place that mirrors include/blockrank_hip.h
SIGNATURES = {
    "br_version": (c_int, []),
    "br_last_error": (c_char_p, []),
    "br_tile_tokens": (c_int, [c_int, c_int]),
    "br_plan_ints": (c_size_t, [c_int, c_int, c_int, c_int, c_int]),
    "br_plan_check": (c_int, [c_void_p, c_void_p]),
    "br_plan_rearm": (c_int, [c_void_p, c_void_p]),
    "br_plan_build": (c_int, [c_void_p, c_int, c_int, c_int, c_int, c_int, c_void_p, c_size_t, c_void_p]),
    "br_plan_build_from_lengths": (c_int, [c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_void_p, c_size_t, c_void_p]),
    "br_plan_build_packed": (c_int, [c_void_p, c_int, c_int, c_int, c_int, c_int, c_void_p, c_size_t, c_void_p]),
    "br_prefill_workspace_bytes": (c_size_t, [c_int, c_int, c_int, c_int]),
    "br_prefill_fwd": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int,
                               c_void_p, c_void_p, c_void_p, c_void_p, c_float, c_int, c_void_p, c_size_t, c_void_p]),
    "br_prefill_noalloc_max_workspace_bytes": (c_size_t, []),
    "br_prefill_fwd_noalloc": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int,
                                       c_void_p, c_void_p, c_void_p, c_void_p, c_float, c_int, c_void_p]),
    "br_prefill_fwd_events": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int,
                                      c_void_p, c_void_p, c_void_p, c_void_p, c_float, c_int, c_void_p, c_size_t, c_void_p,
                                      c_void_p, c_void_p]),
    "br_score_partials_bytes": (c_size_t, [c_int, c_int, c_int, c_int, c_int]),
    "br_prefill_fwd_scores": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int,
                                      c_void_p, c_void_p, c_void_p, c_void_p, c_float, c_int, c_void_p, c_size_t,
                                      c_int, c_void_p, c_size_t, c_void_p, c_void_p, c_void_p]),
    "br_prefill_fwd_ex": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int,
                                  c_void_p, c_void_p, c_void_p, c_void_p, c_float, c_int, c_void_p, c_size_t, c_void_p, c_void_p]),
    "br_prefill_fp8qk_workspace_bytes": (c_size_t, [c_int, c_int, c_int, c_int, c_int, c_int64]),
    "br_prefill_fwd_fp8qk": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int,
                                     c_void_p, c_void_p, c_void_p, c_void_p, c_float, c_int64, c_void_p, c_size_t,
                                     c_int, c_void_p, c_size_t, c_void_p, c_void_p, c_void_p]),
    "br_doc_scores_from_partials": (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_float,
                                            c_void_p, c_void_p, c_void_p]),
    "br_doc_scores_workspace_bytes": (c_size_t, [c_int, c_int, c_int, c_int]),
    "br_doc_scores": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_int,
                              c_void_p, c_void_p, c_float, c_float, c_int, c_void_p, c_void_p, c_void_p, c_size_t, c_void_p]),
    "br_last_block_logits": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_int,
                                     c_void_p, c_void_p, c_float, c_float, c_int, c_void_p, c_void_p]),
    "br_last_block_logits_bwd": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_int,
                                         c_void_p, c_void_p, c_float, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p]),
    "br_prefill_fwd_lse": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int,
                                   c_void_p, c_void_p, c_void_p, c_void_p, c_float, c_void_p, c_size_t, c_void_p, c_void_p, c_void_p]),
    "br_prefill_bwd_workspace_bytes": (c_size_t, [c_int, c_int, c_int, c_int, c_int, c_int64]),
    "br_prefill_bwd": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                               c_int, c_int, c_int, c_int, c_int, c_int,
                               c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                               c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                               c_float, c_int64, c_void_p, c_size_t, c_void_p]),
    "br_rmsnorm": (c_int, [c_void_p, c_void_p, c_void_p, c_int64, c_int, c_int64, c_int64, c_float, c_int, c_void_p]),
    "br_silu_mul": (c_int, [c_void_p, c_void_p, c_void_p, c_int64, c_int, c_void_p]),
    "br_rope_qk": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int,
                           c_void_p, c_void_p, c_void_p, c_int, c_void_p]),
}

_lib = None


class BlockRankLibraryError(RuntimeError):
    """libblockrank_hip.so is missing or unusable."""


def load() -> ctypes.CDLL:
    """Load the library (once).  Raises BlockRankLibraryError if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not LIB_PATH.exists():
        raise BlockRankLibraryError(
            f"{LIB_PATH} not found: the HIP kernels are not built (run `python -m blockrank_amd.build`); "
            "blockrank_amd has no CPU or PyTorch fallback")
    try:
        lib = ctypes.CDLL(str(LIB_PATH))
    except OSError as e:  # pragma: no cover - depends on the machine
        raise BlockRankLibraryError(f"cannot load {LIB_PATH}: {e}") from e
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


def last_error() -> str:
    return load().br_last_error().decode("utf-8", "replace")


def check(rc: int) -> None:
    """Turn a non-zero return code into the exception the reference's Python would have raised:
    argument problems are AssertionError (the reference uses bare asserts), the rest RuntimeError."""
    if rc == 0:
        return
    msg = last_error()
    if rc == BR_ERR_ARG:
        raise AssertionError(msg)
    raise RuntimeError(f"libblockrank_hip error {rc}: {msg}")


def strides3(t, packed: bool = False) -> ctypes.Array:
    """Element strides (batch, head, token) of a logical (B, heads, S, D) tensor; a packed layout has
    one token axis for the whole batch, i.e. batch stride 0."""
    s = t.stride()
    return _I64x3(0 if packed else s[0], s[1], s[2])
