"""ctypes binding of ``libacache_hip.so`` (the C ABI declared in include/acache_hip.h).

The library is the only compute path of this package: if it is missing or a
symbol cannot be resolved, importing the ops fails with an explicit error —
there is no CPU or eager-PyTorch fallback.
"""
from __future__ import annotations

import ctypes
import os
from ctypes import c_char_p, c_float, c_int32, c_int64, c_void_p
from pathlib import Path

LIB_PATH = Path(__file__).resolve().parent / "libacache_hip.so"

BF16, F16, F32 = 0, 1, 2

# name -> (restype, argtypes); mirrors include/acache_hip.h one to one
SIGNATURES = {
    "acache_abi_version": (c_int32, []),
    "acache_last_error": (c_char_p, []),
    "acache_relocate_rope_gather": (c_int32, [
        c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
        c_int64, c_int32, c_int32, c_int32, c_int32, c_int64, c_int32, c_int64, c_int64, c_void_p]),
    "acache_materialize_relocated_affix": (c_int32, [
        c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int32,
        c_int32, c_int32, c_int32, c_int32, c_int64, c_int32, c_int64, c_void_p]),
    "acache_kv_scatter": (c_int32, [
        c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
        c_int64, c_int32, c_int32, c_int32, c_int32, c_int64,
        c_int64, c_int64, c_int64, c_int64, c_void_p]),
    "acache_rope_qk_scatter": (c_int32, [
        c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
        c_int32, c_int64, c_int32, c_int32, c_int32, c_int32, c_int64,
        c_int64, c_int64, c_int64, c_void_p]),
    "acache_affix_importance_workspace_bytes": (c_int64, [c_int64, c_int32, c_int32, c_int32, c_int32, c_int32, c_int32]),
    "acache_affix_importance": (c_int32, [
        c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int32, c_float,
        c_int32, c_int64, c_int32, c_int64, c_int64, c_int32, c_int32, c_int32, c_int32, c_int32, c_int64,
        c_int64, c_int64, c_int64, c_int64, c_int64, c_void_p, c_int64, c_void_p]),
    "acache_affix_importance_noalloc_max_bytes": (c_int64, []),
    "acache_affix_importance_noalloc": (c_int32, [
        c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int32, c_float,
        c_int32, c_int64, c_int32, c_int64, c_int64, c_int32, c_int32, c_int32, c_int32, c_int32, c_int64,
        c_int64, c_int64, c_int64, c_int64, c_int64, c_void_p]),
    "acache_topk_anchors": (c_int32, [
        c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int32, c_int32, c_int32, c_void_p]),
    "acache_argmax_confidence": (c_int32, [
        c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int32, c_void_p]),
    "acache_commit_tokens": (c_int32, [
        c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int32, c_int64, c_float, c_void_p]),
    "acache_block_table_slots": (c_int32, [
        c_void_p, c_void_p, c_void_p, c_int32, c_int32, c_int32, c_int64, c_void_p]),
    "acache_build_slot_layout": (c_int32, [
        c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
        c_int32, c_int32, c_int32, c_int32, c_int64, c_void_p]),
    "acache_swiglu": (c_int32, [c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int64, c_int32, c_void_p]),
    "acache_add_rms_norm": (c_int32, [
        c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int64, c_int64, c_int64, c_float,
        c_int32, c_void_p]),
    "acache_varlen_attn": (c_int32, [
        c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
        c_float,
        c_int32, c_void_p, c_void_p, c_void_p, c_void_p, c_int32,
        c_int32, c_int64, c_int64,
        c_int32, c_int32, c_int32, c_int32, c_int64,
        c_int64, c_int64, c_int64, c_int64, c_int64, c_int64,
        c_void_p]),
    "acache_varlen_attn_planned": (c_int32, [
        c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
        c_float,
        c_int32, c_void_p, c_void_p, c_void_p, c_void_p, c_int32,
        c_int32, c_int64, c_int64,
        c_int32, c_int32, c_int32, c_int32, c_int64,
        c_int64, c_int64, c_int64, c_int64, c_int64, c_int64,
        c_void_p, c_int64, c_void_p]),
    "acache_varlen_attn_plan": (c_int64, [c_void_p, c_void_p, c_int32, c_int32, c_int32, c_int32, c_void_p, c_int64]),
}


class AcacheLibraryError(RuntimeError):
    """The HIP library is missing, stale, or returned an error code."""


_lib = None


def load() -> ctypes.CDLL:
    """Load the in-tree library once and bind every declared entry point."""
    global _lib
    if _lib is not None:
        return _lib
    if not LIB_PATH.exists():
        raise AcacheLibraryError(
            f"{LIB_PATH} not found. Build it with `python -m acache_amd.build` "
            "(needs hipcc; no GPU required). There is no fallback path."
        )
    lib = ctypes.CDLL(os.fspath(LIB_PATH))
    for name, (restype, argtypes) in SIGNATURES.items():
        try:
            fn = getattr(lib, name)
        except AttributeError as exc:
            raise AcacheLibraryError(
                f"{LIB_PATH} does not export {name}; rebuild with `python -m acache_amd.build`."
            ) from exc
        fn.restype = restype
        fn.argtypes = argtypes
    _lib = lib
    return lib


def check(code: int, what: str) -> None:
    """Raise for a non-zero return code of a library call."""
    if code == 0:
        return
    msg = load().acache_last_error()
    text = msg.decode("utf-8", "replace") if msg else ""
    if code < 0:
        raise ValueError(f"{what}: {text} (acache error {code})")
    raise AcacheLibraryError(f"{what}: HIP error {code}: {text}")
