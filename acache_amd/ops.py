"""Operator layer of the affix-KV reuse path on MI355X.

Every function here keeps the name, argument order and error behaviour of the
reference callable it replaces and forwards to ``libacache_hip.so`` through the
C ABI (raw device pointers + the current HIP stream).  torch is used only to
allocate outputs and to read pointers, shapes and strides.

Reference callables mirrored (paths relative to the reference tree):
  materialize_relocated_affix   nano-vdllm/model/acache_attention.py:88-128
  acache_attention              nano-vdllm/model/acache_attention.py:643-738
  baseline_ragged_attention     nano-vdllm/model/acache_attention.py:525-582
  baseline_decode_attention     nano-vdllm/model/acache_attention.py:585-640
  store_kvcache                 nano-vdllm/model/attention.py:34-41
  select_anchor_tokens          llada/generate_ACache.py:225-262
Additions with no single reference callable (documented at each function):
  relocate_rope_gather, kv_scatter_layers, topk_anchors, block_table_slots.
"""
from __future__ import annotations

import os

import math
from itertools import accumulate as _accumulate

import torch

from . import _lib

_DTYPE_CODE = {torch.bfloat16: _lib.BF16, torch.float16: _lib.F16, torch.float32: _lib.F32}


def _code(t: torch.Tensor) -> int:
    try:
        return _DTYPE_CODE[t.dtype]
    except KeyError:
        raise ValueError(f"unsupported dtype {t.dtype}; expected bfloat16, float16 or float32") from None


def _stream(t: torch.Tensor) -> int:
    return torch.cuda.current_stream(t.device).cuda_stream


def _ptr(t: torch.Tensor | None) -> int | None:
    if t is None or t.numel() == 0:
        return None
    return t.data_ptr()


def _i32(t: torch.Tensor, name: str) -> torch.Tensor:
    assert t.is_cuda, f"{name} must be a device tensor"
    if t.dtype != torch.int32:
        t = t.to(torch.int32)
    return t if t.is_contiguous() else t.contiguous()


def _rope_f32(t: torch.Tensor) -> torch.Tensor:
    """RoPE tables are consumed as contiguous fp32 ``[rows, D]``.

    The LLaDA engine already keeps them in fp32 (model_runner.py:269-271); the
    Dream engine's bf16 tables (model_runner.py:260-267) are widened, the
    rotation itself is always evaluated in fp32 registers.
    """
    assert t.is_cuda and t.dim() == 2
    if t.dtype != torch.float32:
        t = t.float()
    return t if t.is_contiguous() else t.contiguous()


def _layered_cache_view(cache: torch.Tensor) -> tuple[int, int, int, int, int]:
    """(L, num_slots, H_kv, D, layer_stride) of a ``[L, S, H, D]`` or ``[L, NB, BS, H, D]`` cache."""
    if cache.dim() == 5:
        L, nb, bs, h, d = cache.shape
        assert cache.stride(4) == 1 and cache.stride(3) == d and cache.stride(2) == h * d
        assert cache.stride(1) == bs * h * d, "cache blocks must be contiguous"
        return L, nb * bs, h, d, cache.stride(0)
    assert cache.dim() == 4
    L, s, h, d = cache.shape
    assert cache.stride(3) == 1 and cache.stride(2) == d and cache.stride(1) == h * d
    return L, s, h, d, cache.stride(0)


# ----------------------------------------------------------------------------
# relocation
# ----------------------------------------------------------------------------
def materialize_relocated_affix(
    k_cache: torch.Tensor,
    v_cache: torch.Tensor,
    rope_cos: torch.Tensor,
    rope_sin: torch.Tensor,
    dst_slot: int,
    affix_len: int,
    affix_shift: int,
):
    """Copy affix rows ``[0, affix_len)`` to ``[dst_slot, dst_slot+affix_len)``, keys rotated by ``affix_shift``.

    Same contract as the reference wrapper; all layers go in ONE launch instead
    of the reference's per-layer loop (acache_attention.py:103).
    """
    assert k_cache.dim() == 4 and v_cache.shape == k_cache.shape
    assert k_cache.is_cuda and v_cache.is_cuda
    assert rope_cos.is_cuda and rope_sin.is_cuda
    assert v_cache.stride() == k_cache.stride() and v_cache.dtype == k_cache.dtype
    L, S, H, D, layer_stride = _layered_cache_view(k_cache)
    cos, sin = _rope_f32(rope_cos), _rope_f32(rope_sin)
    assert cos.shape == sin.shape and cos.shape[1] == D
    lib = _lib.load()
    with torch.cuda.device(k_cache.device):
        rc = lib.acache_materialize_relocated_affix(
            _ptr(k_cache), _ptr(v_cache), _ptr(cos), _ptr(sin),
            int(dst_slot), int(affix_len), int(affix_shift),
            L, H, D, _code(k_cache), S, cos.shape[0], layer_stride, _stream(k_cache))
    _lib.check(rc, "materialize_relocated_affix")


def relocate_rope_gather(
    k_cache: torch.Tensor,
    v_cache: torch.Tensor,
    slot_mapping: torch.Tensor,
    deltas: torch.Tensor | None = None,
    rope_cos: torch.Tensor | None = None,
    rope_sin: torch.Tensor | None = None,
    out_k: torch.Tensor | None = None,
    out_v: torch.Tensor | None = None,
):
    """Gather cached K/V rows into the packed varlen layout, re-rotating relocated keys.

    ``k_cache``/``v_cache``: ``[L, S, H_kv, D]`` or ``[L, NB, BS, H_kv, D]``.
    ``slot_mapping`` int32 ``[T]`` is the concatenation of every request's read
    slot map (``cu_seqlens`` offsets are the caller's); ``deltas`` int32 ``[T]``
    holds the position shift of each row (0 = bit copy).  Returns
    ``(out_k, out_v)`` of shape ``[L, T, H_kv, D]``.

    This is the stand-alone form of what the reference does inside its attention
    kernel for every query tile (acache_attention.py:475-497): done once here,
    the packed buffers can feed any varlen attention.
    """
    assert k_cache.is_cuda and v_cache.is_cuda and slot_mapping.is_cuda
    assert v_cache.shape == k_cache.shape and v_cache.stride() == k_cache.stride()
    assert v_cache.dtype == k_cache.dtype
    L, S, H, D, layer_stride = _layered_cache_view(k_cache)
    slots = _i32(slot_mapping, "slot_mapping")
    T = slots.numel()
    cos = sin = None
    rope_rows = 0
    if deltas is not None:
        if rope_cos is None or rope_sin is None:
            raise ValueError("Post-RoPE affix relocation requires shifts and RoPE tables.")
        deltas = _i32(deltas, "deltas")
        assert deltas.numel() == T
        cos, sin = _rope_f32(rope_cos), _rope_f32(rope_sin)
        assert cos.shape == sin.shape and cos.shape[1] == D
        rope_rows = cos.shape[0]
    if out_k is None:
        out_k = torch.empty(L, T, H, D, dtype=k_cache.dtype, device=k_cache.device)
    if out_v is None:
        out_v = torch.empty(L, T, H, D, dtype=k_cache.dtype, device=k_cache.device)
    assert out_k.shape == (L, T, H, D) and out_v.shape == (L, T, H, D)
    assert out_k.dtype == k_cache.dtype and out_v.dtype == k_cache.dtype
    assert out_k[0].is_contiguous() and out_v[0].is_contiguous()
    assert out_k.stride(0) == out_v.stride(0)
    lib = _lib.load()
    with torch.cuda.device(k_cache.device):
        rc = lib.acache_relocate_rope_gather(
            _ptr(out_k), _ptr(out_v), _ptr(k_cache), _ptr(v_cache),
            _ptr(slots), _ptr(deltas), _ptr(cos), _ptr(sin),
            T, L, H, D, _code(k_cache), S, rope_rows, layer_stride, out_k.stride(0),
            _stream(k_cache))
    _lib.check(rc, "relocate_rope_gather")
    return out_k, out_v


# ----------------------------------------------------------------------------
# scatter
# ----------------------------------------------------------------------------
def store_kvcache(
    key: torch.Tensor,
    value: torch.Tensor,
    k_cache: torch.Tensor,
    v_cache: torch.Tensor,
    slot_mapping: torch.Tensor,
):
    """Write ``key[i]``/``value[i]`` to cache slot ``slot_mapping[i]`` (``-1`` = skip)."""
    N, num_heads, head_dim = key.shape
    D = num_heads * head_dim
    assert key.stride(-1) == 1 and value.stride(-1) == 1
    assert key.stride(1) == head_dim and value.stride(1) == head_dim
    assert k_cache.stride(1) == D and v_cache.stride(1) == D
    assert slot_mapping.numel() == N
    assert key.is_cuda and k_cache.is_cuda and key.dtype == k_cache.dtype == value.dtype == v_cache.dtype
    slots = _i32(slot_mapping, "slot_mapping")
    num_slots = k_cache.numel() // D
    assert k_cache.is_contiguous() and v_cache.is_contiguous()
    lib = _lib.load()
    with torch.cuda.device(key.device):
        rc = lib.acache_kv_scatter(
            _ptr(k_cache), _ptr(v_cache), _ptr(key), _ptr(value), _ptr(slots),
            N, 1, num_heads, head_dim, _code(key), num_slots,
            key.stride(0), value.stride(0), 0, 0, _stream(key))
    _lib.check(rc, "store_kvcache")


def rope_qk_scatter(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor | None,
    positions: torch.Tensor,
    rope_cos: torch.Tensor,
    rope_sin: torch.Tensor,
    k_cache: torch.Tensor | None = None,
    v_cache: torch.Tensor | None = None,
    slot_mapping: torch.Tensor | None = None,
):
    """Rotate ``q`` and ``k`` in place to their positions and write ``k`` / ``v`` to their cache slots, one launch.

    ``q``: ``[N, H, D]``, ``k`` / ``v``: ``[N, H_kv, D]`` (token stride free, heads contiguous: views of a fused
    projection are fine); ``positions``: int64 ``[N]``; tables fp32 ``[rows, D]``.  Without ``slot_mapping`` only
    the rotation is done.  Rotary application of nano-vdllm/model/modeling_llada.py:412-453 followed by
    ``store_kvcache`` (nano-vdllm/model/attention.py:34-41).
    """
    N, H, D = q.shape
    H_kv = k.shape[1]
    assert k.shape == (N, H_kv, D) and q.is_cuda and q.dtype == k.dtype
    assert q.stride(-1) == 1 and k.stride(-1) == 1 and q.stride(1) == D and k.stride(1) == D
    assert positions.dtype == torch.int64 and positions.numel() == N and positions.is_contiguous()
    assert rope_cos.dtype == torch.float32 and rope_cos.is_contiguous() and rope_cos.shape[1] == D
    assert rope_sin.dtype == torch.float32 and rope_sin.is_contiguous() and rope_sin.shape == rope_cos.shape
    slots = None
    num_slots = 0
    if slot_mapping is not None:
        assert v is not None and k_cache is not None and v_cache is not None
        assert v.shape == k.shape and v.stride(-1) == 1 and v.stride(1) == D and v.dtype == q.dtype
        assert k_cache.is_contiguous() and v_cache.is_contiguous() and k_cache.dtype == q.dtype == v_cache.dtype
        assert slot_mapping.numel() == N
        slots = _i32(slot_mapping, "slot_mapping")
        num_slots = k_cache.numel() // (H_kv * D)
    lib = _lib.load()
    with torch.cuda.device(q.device):
        rc = lib.acache_rope_qk_scatter(
            _ptr(q), _ptr(k), _ptr(v) if slots is not None else None,
            _ptr(k_cache) if slots is not None else None, _ptr(v_cache) if slots is not None else None,
            _ptr(positions), _ptr(slots) if slots is not None else None, _ptr(rope_cos), _ptr(rope_sin),
            rope_cos.shape[0], N, H, H_kv, D, _code(q), num_slots,
            q.stride(0), k.stride(0), v.stride(0) if slots is not None else 0, _stream(q))
    _lib.check(rc, "rope_qk_scatter")


def argmax_confidence(logits: torch.Tensor, picks: torch.Tensor | None = None):
    """``(token, confidence)`` per row of ``logits`` (``[..., V]``): the arg-max token (or ``picks``) and
    ``exp(logit[token] - logsumexp(row))`` in fp32, one streaming pass per row
    (nano-vdllm/model_runner.py:2279-2296)."""
    V = logits.shape[-1]
    flat = logits.reshape(-1, V)
    assert flat.is_cuda and flat.stride(-1) == 1
    R = flat.shape[0]
    conf = torch.empty(R, dtype=torch.float32, device=logits.device)
    if picks is None:
        token = torch.empty(R, dtype=torch.int64, device=logits.device)
        picks_flat = None
    else:
        picks_flat = picks.reshape(-1).to(torch.int64).contiguous()
        assert picks_flat.numel() == R
        token = picks_flat
    lib = _lib.load()
    with torch.cuda.device(logits.device):
        rc = lib.acache_argmax_confidence(
            _ptr(token) if picks is None else None, _ptr(conf), _ptr(flat), _ptr(picks_flat) if picks is not None else None,
            R, V, flat.stride(0) if R > 1 else max(V, flat.stride(0)), _code(flat), _stream(flat))
    _lib.check(rc, "argmax_confidence")
    return token.view(logits.shape[:-1]), conf.view(logits.shape[:-1])


def commit_tokens(blocks: torch.Tensor, proposal: torch.Tensor, confidence: torch.Tensor,
                  committed_rows: torch.Tensor, mask_id: int, threshold: float) -> None:
    """Write the accepted proposals into ``blocks`` (``[n, L]`` int64, in place): positions that hold ``mask_id``
    and are proposed another token are accepted when their confidence reaches ``threshold``; a row with such
    positions and none accepted takes its most confident one.  ``committed_rows`` (one int32 on the device) grows
    by the number of rows that accepted something.  The rule of ``ModelRunner.get_transfer_index`` plus the write
    of its picks (nano-vdllm/model_runner.py:2297-2314, 2262-2266) in one launch."""
    assert blocks.is_cuda and blocks.dim() == 2 and blocks.dtype == torch.int64 and blocks.is_contiguous()
    assert proposal.shape == blocks.shape and proposal.dtype == torch.int64 and proposal.is_contiguous()
    assert confidence.shape == blocks.shape and confidence.dtype == torch.float32 and confidence.is_contiguous()
    assert committed_rows.is_cuda and committed_rows.dtype == torch.int32 and committed_rows.numel() == 1
    lib = _lib.load()
    with torch.cuda.device(blocks.device):
        rc = lib.acache_commit_tokens(_ptr(blocks), _ptr(proposal), _ptr(confidence), _ptr(committed_rows),
                                      blocks.shape[0], blocks.shape[1], int(mask_id), float(threshold), _stream(blocks))
    _lib.check(rc, "commit_tokens")


def swiglu(gate_up: torch.Tensor, hidden: int) -> torch.Tensor:
    """``silu(gate_up[..., :hidden]) * gate_up[..., hidden:]`` of a merged gate / up projection in one pass (the
    MLP activation of the decoder block: ``act(ff_proj(x)) * up_proj(x)``)."""
    assert gate_up.is_cuda and gate_up.shape[-1] == 2 * hidden and gate_up.stride(-1) == 1
    flat = gate_up.reshape(-1, 2 * hidden)
    out = torch.empty(flat.shape[0], hidden, dtype=gate_up.dtype, device=gate_up.device)
    lib = _lib.load()
    with torch.cuda.device(gate_up.device):
        rc = lib.acache_swiglu(_ptr(out), _ptr(flat), flat.shape[0], hidden,
                               flat.stride(0) if flat.shape[0] > 1 else 2 * hidden, hidden, _code(flat), _stream(flat))
    _lib.check(rc, "swiglu")
    return out.view(*gate_up.shape[:-1], hidden)


def add_rms_norm(x: torch.Tensor, delta: torch.Tensor | None, weight: torch.Tensor, eps: float):
    """Residual add and RMS layer norm in one pass: returns ``(x + delta, norm(x + delta))`` where
    ``norm(s) = s * rsqrt(mean(s^2) + eps) * weight`` (statistics in fp32, one rounding).  With ``delta`` None the
    first element is ``x`` itself.  ``x``: ``[..., d]`` with contiguous rows; nothing is modified in place."""
    d = x.shape[-1]
    assert x.is_cuda and x.stride(-1) == 1 and weight.shape == (d,)
    flat = x.reshape(-1, d)
    M = flat.shape[0]
    y = torch.empty(M, d, dtype=x.dtype, device=x.device)
    w = (weight if weight.dtype == x.dtype else weight.to(x.dtype)).contiguous()
    total = dl = None
    if delta is not None:
        assert delta.shape == x.shape and delta.dtype == x.dtype and delta.stride(-1) == 1
        dl = delta.reshape(-1, d)
        total = torch.empty(M, d, dtype=x.dtype, device=x.device)
    stride = lambda t: t.stride(0) if M > 1 else d
    lib = _lib.load()
    with torch.cuda.device(x.device):
        rc = lib.acache_add_rms_norm(_ptr(total), _ptr(flat), _ptr(dl), _ptr(w), _ptr(y), M, d,
                                     d, stride(flat), stride(dl) if dl is not None else d, d, float(eps),
                                     _code(flat), _stream(flat))
    _lib.check(rc, "add_rms_norm")
    return (total.view(x.shape) if total is not None else x), y.view(x.shape)


def affix_importance(
    importance: torch.Tensor,
    q: torch.Tensor,
    k_cache: torch.Tensor,
    mask_rows: torch.Tensor,
    cu_mask: torch.Tensor,
    affix_len: int,
    max_mask_rows: int,
    softmax_scale: float | None = None,
    affix_shifts: torch.Tensor | None = None,
    rope_cos: torch.Tensor | None = None,
    rope_sin: torch.Tensor | None = None,
    affix_slot0: int = 0,
    workspace: torch.Tensor | None = None,
) -> torch.Tensor:
    """Add one layer's affix importance to ``importance`` (fp32 ``[B, >= affix_len]``).

    For each request the [MASK] queries ``q[mask_rows[cu_mask[b]:cu_mask[b+1]]]`` attend to the cached affix keys
    ``k_cache`` slots ``affix_slot0 .. + affix_len`` (relocated by ``affix_shifts[b]``: the queries are rotated by
    the opposite angle, the keys are read as cached); the softmax runs over the
    affix keys only and its columns are summed over queries and heads (nano-vdllm/model_runner.py:730-773).
    ``workspace``: optional uint8 scratch of ``affix_importance_workspace_bytes`` bytes, allocated here if absent;
    the string ``"builtin"`` selects ``acache_affix_importance_noalloc``, which keeps its scratch in a fixed device
    array inside the library (allocates nothing; rejects calls that need more than that array holds; calls on
    one GPU must not overlap).
    """
    Tq, H, D = q.shape
    H_kv = k_cache.shape[-2]
    kc = k_cache.view(-1, H_kv, D)
    assert importance.dtype == torch.float32 and importance.dim() == 2 and importance.stride(1) == 1
    assert q.is_cuda and q.dtype == kc.dtype and q.stride(-1) == 1 and kc.is_contiguous()
    B = cu_mask.numel() - 1
    assert importance.shape[0] >= B and importance.shape[1] >= affix_len
    rows = _i32(mask_rows, "mask_rows")
    cu = _i32(cu_mask, "cu_mask")
    total = rows.numel()
    relocate = affix_shifts is not None
    if relocate and (rope_cos is None or rope_sin is None):
        raise ValueError("Post-RoPE affix relocation requires shifts and RoPE tables.")
    shifts = _i32(affix_shifts, "affix_shifts") if relocate else None
    scale = softmax_scale if softmax_scale is not None else D ** -0.5
    lib = _lib.load()
    common = (
        _ptr(importance), _ptr(q), _ptr(kc), _ptr(rows), _ptr(cu), _ptr(shifts),
        _ptr(rope_cos) if relocate else None, _ptr(rope_sin) if relocate else None,
        rope_cos.shape[0] if relocate else 0, float(scale),
        affix_len, affix_slot0, B, Tq, total, max_mask_rows, H, H_kv, D, _code(q), kc.shape[0],
        importance.stride(0), q.stride(0), q.stride(1), kc.stride(0), kc.stride(1))
    if isinstance(workspace, str):
        if workspace != "builtin":
            raise ValueError("workspace: a uint8 tensor, None or 'builtin'")
        with torch.cuda.device(q.device):
            rc = lib.acache_affix_importance_noalloc(*common, _stream(q))
        _lib.check(rc, "affix_importance_noalloc")
        return importance
    need = lib.acache_affix_importance_workspace_bytes(total, B, H, H_kv, D, affix_len, int(relocate))
    if workspace is None:
        workspace = torch.empty(max(need, 16), dtype=torch.uint8, device=q.device)
    assert workspace.is_cuda and workspace.numel() * workspace.element_size() >= need
    with torch.cuda.device(q.device):
        rc = lib.acache_affix_importance(*common, _ptr(workspace), workspace.numel() * workspace.element_size(),
                                         _stream(q))
    _lib.check(rc, "affix_importance")
    return importance


def affix_importance_workspace_bytes(total_mask_rows: int, batch: int, num_heads: int, num_kv_heads: int,
                                     head_dim: int, affix_len: int, relocated: bool) -> int:
    """Bytes of scratch ``affix_importance`` needs: row statistics, per-head partial sums and the packed copy of
    the [MASK] queries (counter-rotated when ``affix_shifts`` are given; made either way, so ``relocated`` does
    not change the size)."""
    return int(_lib.load().acache_affix_importance_workspace_bytes(
        total_mask_rows, batch, num_heads, num_kv_heads, head_dim, affix_len, int(relocated)))


def build_slot_layout(lengths, affix_spans, anchors, block_tables: torch.Tensor, block_size: int,
                      shared_slot_offset: int = 0, anchor_counts=None):
    """Read slot maps and recompute lists of a batch in one launch (``Sequence.finalize_slot_mapping``,
    nano-vdllm/sequence.py:169-202, for every request at once).

    ``lengths``: tokens per request; ``affix_spans``: ``(start, end)`` per request; ``anchors``: ascending anchor
    positions per request as lists, or — with ``anchor_counts`` giving the number per request — one int32 device
    tensor holding them back to back (the output of ``topk_anchors``, which then never visits the host);
    ``block_tables``: int32 ``[B, max_blocks]`` on the device (-1 padded).
    Returns ``(read_slots, recompute_pos, recompute_slots, cu_len, cu_rec)``, the first three int32 device tensors.
    """
    device = block_tables.device
    B = len(lengths)
    assert block_tables.is_cuda and block_tables.dtype == torch.int32 and block_tables.is_contiguous()
    on_device = anchor_counts is not None
    counts = [int(c) for c in anchor_counts] if on_device else [len(a) for a in anchors]
    assert block_tables.shape[0] == B == len(affix_spans) == len(counts)
    rec = [k + n - (e - s) for n, (s, e), k in zip(lengths, affix_spans, counts)]
    cu_len = [0] + list(_accumulate(lengths))
    cu_rec = [0] + list(_accumulate(rec))
    cu_anc = [0] + list(_accumulate(counts))
    flat_anchors = [] if on_device else [p for a in anchors for p in a]
    meta = torch.tensor(cu_len + cu_rec + cu_anc + [s for s, _ in affix_spans] + [e for _, e in affix_spans]
                        + (flat_anchors or [0]), dtype=torch.int32).to(device, non_blocking=True)
    o = 0
    parts = []
    for n in (B + 1, B + 1, B + 1, B, B, max(len(flat_anchors), 1)):
        parts.append(meta[o:o + n])
        o += n
    d_len, d_rec, d_anc, d_start, d_end, d_anchors = parts
    if on_device and cu_anc[-1] > 0:
        d_anchors = _i32(anchors, "anchors")
        assert d_anchors.is_cuda and d_anchors.numel() == cu_anc[-1]
    read = torch.empty(cu_len[-1], dtype=torch.int32, device=device)
    rpos = torch.empty(cu_rec[-1], dtype=torch.int32, device=device)
    rslot = torch.empty(cu_rec[-1], dtype=torch.int32, device=device)
    lib = _lib.load()
    with torch.cuda.device(device):
        rc = lib.acache_build_slot_layout(
            _ptr(read), _ptr(rpos) or read.data_ptr(), _ptr(rslot) or read.data_ptr(), _ptr(d_len), _ptr(d_rec),
            _ptr(d_start), _ptr(d_end), _ptr(d_anc), _ptr(d_anchors), _ptr(block_tables), B, block_tables.shape[1],
            block_size, shared_slot_offset, cu_len[-1], _stream(block_tables))
    _lib.check(rc, "build_slot_layout")
    return read, rpos, rslot, cu_len, cu_rec


def kv_scatter_layers(
    key: torch.Tensor,
    value: torch.Tensor,
    k_cache: torch.Tensor,
    v_cache: torch.Tensor,
    slot_mapping: torch.Tensor,
):
    """``store_kvcache`` for all layers in one launch.

    ``key``/``value``: ``[L, N, H_kv, D]``; caches ``[L, S, H_kv, D]`` or
    ``[L, NB, BS, H_kv, D]``.  The reference issues one ``store_kvcache`` launch
    per layer from ``Attention.forward`` (attention.py:72); when the recomputed
    anchor rows of all layers are available together this form moves them in a
    single grid.
    """
    assert key.dim() == 4 and value.shape == key.shape
    L, N, H, D = key.shape
    Lc, S, Hc, Dc, cache_layer_stride = _layered_cache_view(k_cache)
    assert (Lc, Hc, Dc) == (L, H, D) and v_cache.shape == k_cache.shape
    assert v_cache.stride() == k_cache.stride()
    assert key.stride(3) == 1 and key.stride(2) == D and value.stride() == key.stride()
    assert key.dtype == k_cache.dtype == value.dtype == v_cache.dtype
    slots = _i32(slot_mapping, "slot_mapping")
    assert slots.numel() == N
    lib = _lib.load()
    with torch.cuda.device(key.device):
        rc = lib.acache_kv_scatter(
            _ptr(k_cache), _ptr(v_cache), _ptr(key), _ptr(value), _ptr(slots),
            N, L, H, D, _code(key), S,
            key.stride(1), value.stride(1), key.stride(0), cache_layer_stride, _stream(key))
    _lib.check(rc, "kv_scatter_layers")


# ----------------------------------------------------------------------------
# anchor selection
# ----------------------------------------------------------------------------
def topk_anchors(
    scores: torch.Tensor,
    cu_affix: torch.Tensor,
    cu_k: torch.Tensor,
    total_k: int,
    offsets: torch.Tensor | None = None,
    largest: bool = True,
    out_dtype: torch.dtype = torch.int64,
) -> torch.Tensor:
    """Ragged per-request top-k; returns the selected indices ascending per request.

    Request ``b`` owns ``scores[cu_affix[b]:cu_affix[b+1]]`` and receives
    ``cu_k[b+1]-cu_k[b]`` indices (plus ``offsets[b]``) at ``out[cu_k[b]:cu_k[b+1]]``.
    Equal scores are resolved towards the lower index.  ``total_k`` is
    ``cu_k[-1]`` known on the host, so no device synchronisation is needed.
    Replaces ``torch.topk(...).indices.sort()`` (model_runner.py:833-843).
    """
    assert scores.is_cuda and scores.dtype == torch.float32 and scores.is_contiguous()
    assert out_dtype in (torch.int32, torch.int64)
    cu_affix = _i32(cu_affix, "cu_affix")
    cu_k = _i32(cu_k, "cu_k")
    B = cu_affix.numel() - 1
    assert cu_k.numel() == B + 1
    out = torch.empty(int(total_k), dtype=out_dtype, device=scores.device)
    if B <= 0 or total_k == 0:
        return out
    if offsets is not None:
        offsets = _i32(offsets, "offsets")
        assert offsets.numel() == B
    lib = _lib.load()
    with torch.cuda.device(scores.device):
        rc = lib.acache_topk_anchors(
            _ptr(out), scores.data_ptr(), _ptr(cu_affix), _ptr(cu_k), _ptr(offsets),
            1 if largest else 0, B, out.element_size(), _stream(scores))
    _lib.check(rc, "topk_anchors")
    return out


def select_anchor_tokens(
    importance_scores: torch.Tensor,
    k: int,
    selection_mode: str = "top",
) -> torch.Tensor:
    """``(B, A)`` scores -> ``(B, K)`` int64 anchor indices, ascending per row.

    Mirror of the HF-path selector (llada/generate_ACache.py:225-262): modes
    ``top``, ``bottom`` and ``random``; ``ValueError`` for a negative ``k`` or an
    unknown mode.  ``top``/``bottom`` run the HIP radix select; ``random`` draws
    ``torch.randperm`` per row exactly as the reference does.
    """
    B, affix_length = importance_scores.shape
    if k < 0:
        raise ValueError(f"k must be non-negative, got {k}")
    k = min(k, affix_length)
    if selection_mode == "random":
        picks = torch.stack([
            torch.randperm(affix_length, device=importance_scores.device)[:k] for _ in range(B)
        ])
        return picks.sort(dim=-1).values
    if selection_mode not in ("top", "bottom"):
        raise ValueError(f"Unknown selection_mode={selection_mode!r}")
    scores = importance_scores.float().contiguous()
    dev = scores.device
    cu_affix = torch.arange(0, (B + 1) * affix_length, max(affix_length, 1), dtype=torch.int32, device=dev)[: B + 1]
    if affix_length == 0:
        cu_affix = torch.zeros(B + 1, dtype=torch.int32, device=dev)
    cu_k = torch.arange(0, (B + 1) * k, max(k, 1), dtype=torch.int32, device=dev)[: B + 1]
    if k == 0:
        cu_k = torch.zeros(B + 1, dtype=torch.int32, device=dev)
    out = topk_anchors(scores.view(-1), cu_affix, cu_k, B * k, largest=(selection_mode == "top"))
    return out.view(B, k)


# ----------------------------------------------------------------------------
# attention
# ----------------------------------------------------------------------------
def block_table_slots(
    block_tables: torch.Tensor, cu_seqlens_k: torch.Tensor, block_size: int, total_k: int
) -> torch.Tensor:
    """Flat slot map ``bt[b, n // BS] * BS + n % BS`` for every request position."""
    block_tables = _i32(block_tables, "block_tables")
    cu_seqlens_k = _i32(cu_seqlens_k, "cu_seqlens_k")
    B, max_blocks = block_tables.shape
    out = torch.empty(int(total_k), dtype=torch.int32, device=block_tables.device)
    lib = _lib.load()
    with torch.cuda.device(block_tables.device):
        rc = lib.acache_block_table_slots(
            _ptr(out), _ptr(block_tables), _ptr(cu_seqlens_k), B, max_blocks, int(block_size),
            int(total_k), _stream(block_tables))
    _lib.check(rc, "block_table_slots")
    return out


def attention_plan(cu_seqlens_q, cu_seqlens_k, num_heads: int, num_kv_heads: int, device,
                   slots_per_xcd: int | None = None) -> torch.Tensor:
    """Dispatch plan for :func:`acache_attention` calls over these lengths: ``[blocks, 2]`` int32 on ``device``.

    The prefix sums are read on the host (lists or CPU tensors cost nothing; device tensors are copied back,
    which synchronises).  The plan depends only on the lengths and head counts, so one plan serves every layer
    of a forward pass.  It orders the (request, query tile, head) units so that the hardware's in-order hand-out
    of workgroups packs each XCD's slots tightly; results are bit-identical with and without it.  No counterpart
    in the reference, whose Triton grid is (query block, head, request) in launch order (acache_attention.py:721).
    """
    cq = torch.as_tensor(cu_seqlens_q, dtype=torch.int32, device="cpu").contiguous()
    ck = torch.as_tensor(cu_seqlens_k, dtype=torch.int32, device="cpu").contiguous()
    assert cq.numel() == ck.numel() and cq.numel() >= 1
    B = cq.numel() - 1
    device = torch.device(device)
    if slots_per_xcd is None:
        slots_per_xcd = max(1, torch.cuda.get_device_properties(device).multi_processor_count // 8) * 2
    lib = _lib.load()
    args = (cq.data_ptr(), ck.data_ptr(), B, int(num_heads), int(num_kv_heads), int(slots_per_xcd))
    blocks = lib.acache_varlen_attn_plan(*args, None, 0)
    if blocks < 0:
        _lib.check(int(blocks), "attention_plan")
    plan = torch.empty(max(int(blocks), 0), 2, dtype=torch.int32, pin_memory=device.type == "cuda")
    if blocks > 0:
        rc = lib.acache_varlen_attn_plan(*args, plan.data_ptr(), int(blocks))
        if rc < 0:
            _lib.check(int(rc), "attention_plan")
    return plan.to(device, non_blocking=True)


def _varlen_attn(q, k_cache, v_cache, cu_q, cu_k, slots, scale, shared_prefix_len,
                 shared_kv_lens, affix_shifts, cos, sin, plan=None):
    total_q, H, D = q.shape
    Hkv = k_cache.shape[-2]
    assert k_cache.shape[-1] == D and v_cache.shape == k_cache.shape
    assert v_cache.stride() == k_cache.stride() and v_cache.dtype == k_cache.dtype == q.dtype
    num_slots = k_cache.numel() // (Hkv * D) if k_cache.is_contiguous() else None
    if k_cache.dim() == 4:
        assert k_cache.stride(0) == k_cache.shape[1] * k_cache.stride(1), "cache blocks must be contiguous"
        slot_stride, head_stride = k_cache.stride(1), k_cache.stride(2)
        num_slots = k_cache.shape[0] * k_cache.shape[1]
    else:
        assert k_cache.dim() == 3
        slot_stride, head_stride = k_cache.stride(0), k_cache.stride(1)
        num_slots = k_cache.shape[0]
    out = torch.empty_like(q)
    B = cu_q.numel() - 1
    rope_rows = 0 if cos is None else cos.shape[0]
    lib = _lib.load()
    plan_blocks = 0
    if plan is not None:
        assert plan.is_cuda and plan.dtype == torch.int32 and plan.dim() == 2 and plan.shape[1] == 2
        assert plan.is_contiguous()
        plan_blocks = plan.shape[0]
        if plan_blocks == 0:
            plan = None
    with torch.cuda.device(q.device):
        rc = lib.acache_varlen_attn_planned(
            _ptr(out), _ptr(q), _ptr(k_cache), _ptr(v_cache), _ptr(cu_q), _ptr(cu_k), _ptr(slots),
            float(scale), int(shared_prefix_len), _ptr(shared_kv_lens), _ptr(affix_shifts),
            _ptr(cos), _ptr(sin), rope_rows,
            B, total_q, slots.numel(), H, Hkv, D, _code(q), num_slots,
            q.stride(0), q.stride(1), out.stride(0), out.stride(1), slot_stride, head_stride,
            _ptr(plan), plan_blocks, _stream(q))
    _lib.check(rc, "acache_attention")
    return out


def acache_attention(
    q: torch.Tensor,
    k_cache: torch.Tensor,
    v_cache: torch.Tensor,
    cu_seqlens_q: torch.Tensor,
    cu_seqlens_k: torch.Tensor,
    read_slot_mapping: torch.Tensor,
    softmax_scale: float | None = None,
    shared_prefix_len: int = 0,
    shared_kv_lens: torch.Tensor | None = None,
    affix_shifts: torch.Tensor | None = None,
    rope_cos: torch.Tensor | None = None,
    rope_sin: torch.Tensor | None = None,
    plan: torch.Tensor | None = None,
):
    """Bidirectional varlen attention over K/V read through ``read_slot_mapping``.

    Argument order, mode selection and ``ValueError`` conditions follow the
    reference wrapper (acache_attention.py:643-738); ``plan`` (from :func:`attention_plan`
    for the same lengths) is an addition that only changes the order the units run in.
    Differences: no host
    synchronisation (the reference reads ``max_q`` and the table-size check back
    with ``.item()``, lines 667 and 685); a key whose shift exceeds the table is
    left unrotated instead of reading out of bounds; rows of requests without
    keys are zeros.
    """
    assert q.dim() == 3
    assert q.is_cuda and k_cache.is_cuda and v_cache.is_cuda
    assert cu_seqlens_q.is_cuda and cu_seqlens_k.is_cuda and read_slot_mapping.is_cuda
    assert q.stride(-1) == 1
    assert k_cache.stride(-1) == 1 and v_cache.stride(-1) == 1
    head_dim = q.shape[-1]
    batch = cu_seqlens_q.numel() - 1
    if softmax_scale is None:
        softmax_scale = head_dim ** -0.5
    apply_relocation = shared_prefix_len > 0 and affix_shifts is not None
    query_side_relocation = apply_relocation and shared_kv_lens is not None
    if apply_relocation and (rope_cos is None or rope_sin is None or affix_shifts is None):
        raise ValueError("Post-RoPE affix relocation requires shifts and RoPE tables.")
    if (rope_cos is None) != (rope_sin is None):
        raise ValueError("rope_cos and rope_sin must be provided together.")
    cos = sin = shifts = shared = None
    if apply_relocation:
        assert affix_shifts.is_cuda and affix_shifts.numel() == batch
        assert rope_cos.dim() == 2 and rope_sin.shape == rope_cos.shape
        assert rope_cos.shape[1] == head_dim
        cos, sin = _rope_f32(rope_cos), _rope_f32(rope_sin)
        shifts = _i32(affix_shifts, "affix_shifts")
        if query_side_relocation:
            assert shared_kv_lens.is_cuda and shared_kv_lens.numel() == batch
            shared = _i32(shared_kv_lens, "shared_kv_lens")
    return _varlen_attn(
        q, k_cache, v_cache, _i32(cu_seqlens_q, "cu_seqlens_q"), _i32(cu_seqlens_k, "cu_seqlens_k"),
        _i32(read_slot_mapping, "read_slot_mapping"), softmax_scale,
        shared_prefix_len if apply_relocation else 0, shared, shifts, cos, sin, plan)


def baseline_ragged_attention(
    q: torch.Tensor,
    k_cache: torch.Tensor,
    v_cache: torch.Tensor,
    cu_seqlens_q: torch.Tensor,
    cu_seqlens_k: torch.Tensor,
    block_tables: torch.Tensor,
    softmax_scale: float | None = None,
    total_k: int | None = None,
    plan: torch.Tensor | None = None,
):
    """Varlen attention over block-table paged K/V (full-recompute baseline).

    ``total_k`` (= ``cu_seqlens_k[-1]``) may be passed by callers that know it on
    the host; otherwise it is read back from the device once.
    """
    assert q.dim() == 3
    assert block_tables is not None
    assert q.is_cuda and k_cache.is_cuda and v_cache.is_cuda and block_tables.is_cuda
    if softmax_scale is None:
        softmax_scale = q.shape[-1] ** -0.5
    if total_k is None:
        total_k = int(cu_seqlens_k[-1].item())
    cu_k = _i32(cu_seqlens_k, "cu_seqlens_k")
    slots = block_table_slots(block_tables, cu_k, k_cache.shape[1], total_k)
    return _varlen_attn(q, k_cache, v_cache, _i32(cu_seqlens_q, "cu_seqlens_q"), cu_k, slots,
                        softmax_scale, 0, None, None, None, None, plan)


def baseline_decode_attention(
    q: torch.Tensor,
    k_cache: torch.Tensor,
    v_cache: torch.Tensor,
    seqlens: torch.Tensor,
    block_tables: torch.Tensor,
    softmax_scale: float | None = None,
    total_k: int | None = None,
):
    """Batched ``[B, Tq, H, D]`` queries against block-table paged K/V of ``seqlens[b]`` keys."""
    assert q.dim() == 4
    assert block_tables is not None
    assert q.is_cuda and k_cache.is_cuda and v_cache.is_cuda and block_tables.is_cuda
    batch, query_len, num_heads, head_dim = q.shape
    if softmax_scale is None:
        softmax_scale = head_dim ** -0.5
    seqlens = _i32(seqlens, "seqlens")
    cu_k = torch.zeros(batch + 1, dtype=torch.int32, device=q.device)
    cu_k[1:] = torch.cumsum(seqlens, 0)
    if total_k is None:
        total_k = int(cu_k[-1].item())
    cu_q = torch.arange(0, (batch + 1) * query_len, query_len, dtype=torch.int32, device=q.device)
    slots = block_table_slots(block_tables, cu_k, k_cache.shape[1], total_k)
    q3 = q.reshape(batch * query_len, num_heads, head_dim)
    out = _varlen_attn(q3, k_cache, v_cache, cu_q, cu_k, slots, softmax_scale, 0, None, None, None, None)
    return out.view(batch, query_len, num_heads, head_dim)


def anchor_budget(anchor_ratio: float, affix_len: int) -> int:
    """``K = min(ceil(ratio * A), A)`` on the Python double product (sequence.py:147)."""
    return min(math.ceil(anchor_ratio * affix_len), affix_len)
