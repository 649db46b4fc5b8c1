"""The C-ABI library loads, exports every symbol the header declares, and rejects bad
arguments before touching a device (no compute call is made here)."""
import ctypes
import re
from pathlib import Path

import pytest

from acache_amd import _lib

ROOT = Path(__file__).resolve().parents[1]
HEADER = ROOT / "include" / "acache_hip.h"


def _declared_functions():
    text = re.sub(r"/\*.*?\*/", "", HEADER.read_text(), flags=re.S)
    return sorted(set(re.findall(r"\b(acache_[a-z_0-9]+)\s*\(", text)))


def test_header_and_binding_table_agree():
    assert _declared_functions() == sorted(_lib.SIGNATURES)


def test_library_exports_every_declared_symbol():
    lib = _lib.load()
    for name in _declared_functions():
        assert hasattr(lib, name), name
    assert lib.acache_abi_version() == 4


def test_argument_errors_are_reported_without_a_device():
    lib = _lib.load()
    buf = ctypes.create_string_buffer(64)
    p = ctypes.addressof(buf) & ~15 | 16  # any non-NULL, 16-byte aligned address; never dereferenced
    # unknown dtype
    rc = lib.acache_materialize_relocated_affix(p, p, p, p, 8, 4, 1, 1, 2, 64, 9, 32, 16, 0, None)
    assert rc == -2 and b"dtype" in lib.acache_last_error()
    # destination overlaps the source rows
    rc = lib.acache_materialize_relocated_affix(p, p, p, p, 2, 4, 1, 1, 2, 64, 0, 32, 16, 0, None)
    assert rc == -5 and b"overlap" in lib.acache_last_error()
    # destination outside the cache
    rc = lib.acache_materialize_relocated_affix(p, p, p, p, 30, 4, 1, 1, 2, 64, 0, 32, 16, 0, None)
    assert rc == -4
    # shift beyond the table
    rc = lib.acache_materialize_relocated_affix(p, p, p, p, 8, 4, 16, 1, 2, 64, 0, 32, 16, 0, None)
    assert rc == -4
    # unsupported head_dim: half a bf16 row of 100 elements is not a whole number of 16-byte chunks
    rc = lib.acache_materialize_relocated_affix(p, p, p, p, 8, 4, 1, 1, 2, 100, 0, 32, 16, 0, None)
    assert rc == -3
    # NULL payload
    rc = lib.acache_relocate_rope_gather(None, p, p, p, p, None, None, None, 4, 1, 2, 64, 0, 32, 0, 0, 0, None)
    assert rc == -1
    # delta without tables
    rc = lib.acache_relocate_rope_gather(p, p, p, p, p, p, None, None, 4, 1, 2, 64, 0, 32, 0, 0, 0, None)
    assert rc == -7
    # misaligned pointer
    rc = lib.acache_relocate_rope_gather(p + 2, p, p, p, p, None, None, None, 4, 1, 2, 64, 0, 32, 0, 0, 0, None)
    assert rc == -6
    # scatter: token stride smaller than a row
    rc = lib.acache_kv_scatter(p, p, p, p, p, 4, 1, 2, 64, 0, 32, 64, 128, 0, 0, None)
    assert rc == -3
    # top-k: bad index width
    rc = lib.acache_topk_anchors(p, p, p, p, None, 1, 2, 3, None)
    assert rc == -2
    # empty work is a successful no-op
    assert lib.acache_kv_scatter(None, None, None, None, None, 0, 1, 2, 64, 0, 32, 128, 128, 0, 0, None) == 0
    assert lib.acache_topk_anchors(None, None, None, None, None, 1, 0, 4, None) == 0


def test_check_raises_value_error_for_argument_errors():
    lib = _lib.load()
    rc = lib.acache_topk_anchors(None, None, None, None, None, 1, 2, 3, None)
    with pytest.raises(ValueError, match="idx_bytes"):
        _lib.check(rc, "topk_anchors")


def test_ops_fail_loudly_when_the_library_is_missing(monkeypatch, tmp_path):
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", tmp_path / "libacache_hip.so")
    with pytest.raises(_lib.AcacheLibraryError, match="no fallback"):
        _lib.load()
