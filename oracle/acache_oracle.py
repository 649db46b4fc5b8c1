"""CPU oracle for the affix-KV reuse path.  TEST INFRASTRUCTURE ONLY.

This module restates, on the CPU, the arithmetic of the reference's hot path so
that the HIP kernels can be checked against it.  It is imported only by
``tests/``, by ``__graft_entry__.smoke()`` and by the ``cpu_baseline`` leg of
``bench.py``; the product package ``acache_amd`` never imports it and has no CPU
fallback.

Every function cites the reference lines it follows (paths relative to the
reference tree).  The formulations are the ones the reference's own tests use as
ground truth (``nano-vdllm/tests/test_attention_kernels.py``): torch CPU tensor
expressions for the floating-point parts, plain Python/numpy for index work.

How each function is pinned (see tests/test_oracle.py):
  rope_table / apply_rope / rotate   closed forms R(0)=I, R(a)R(b)=R(a+b),
                                     R(-d)R(d)=I, pair-norm invariance, an
                                     independent float64 evaluation, and the C
                                     restatement in oracle/acache_oracle.c
  relocate_rope_gather / materialize geometry of the reference's bit-exact test
                                     (test_attention_kernels.py:127-165),
                                     gather∘scatter = identity
  store_kvcache                      brute force per element, -1 skip
  topk_anchors                       torch.topk value multiset; brute-force
                                     enumeration on tiny inputs; tie order is
                                     NOT defined by the reference (torch.topk):
                                     "parity unpinned" at ties, the rule here is
                                     the contract "lower index wins"
  dense_attention / acache_attention torch.nn.functional.scaled_dot_product_attention,
                                     uniform-V and permutation invariants, mode
                                     equivalences key-side == materialised ==
                                     query-side
  finalize_slot_mapping /
  attention_read_layout              golden vectors held by the reference's tests
                                     (test_model_runner_acache.py:26-47,
                                     test_sequence_spans.py:11-45)
"""
from __future__ import annotations

import math

import numpy as np
import torch


# --------------------------------------------------------------------------- RoPE
def rope_table(length: int, head_dim: int, theta: float = 10000.0, dtype=torch.float32):
    """``cos, sin`` of shape ``[length, head_dim]`` with the ``cat(freqs, freqs)`` layout.

    nano-vdllm/model/modeling_llada.py:392-398 (production, theta from config) and
    nano-vdllm/tests/test_attention_kernels.py:118-124 (test helper, theta 1e4):
    ``inv_freq = 1/theta**(arange(0,D,2)/D)`` in fp32, ``freqs = outer(pos, inv_freq)``
    in fp32, then cos/sin of the concatenation.
    """
    inv_freq = 1.0 / (theta ** (torch.arange(0, head_dim, 2, dtype=torch.float32) / head_dim))
    freqs = torch.outer(torch.arange(length, dtype=torch.float32), inv_freq)
    emb = torch.cat((freqs, freqs), dim=-1)
    return emb.cos().to(dtype), emb.sin().to(dtype)


def rot_half(x: torch.Tensor) -> torch.Tensor:
    """``cat(-x[..., D/2:], x[..., :D/2])`` (acache_attention.py:45,55; modeling_llada.py:404-410)."""
    half = x.shape[-1] // 2
    return torch.cat((-x[..., half:], x[..., :half]), dim=-1)


def apply_rope(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor) -> torch.Tensor:
    """``(x*cos + rot_half(x)*sin).to(x.dtype)`` with per-token rows broadcast over heads.

    nano-vdllm/tests/test_attention_kernels.py:112-115.  ``x``: ``[T, H, D]``;
    ``cos``/``sin``: ``[T, D]``.  With fp32 tables a bf16 ``x`` is promoted to
    fp32, both products and the sum are rounded separately, and the result is
    rounded once to ``x.dtype``.
    """
    return (x * cos[:, None, :] + rot_half(x) * sin[:, None, :]).to(x.dtype)


def rope_qk_scatter(q, k, v, positions, cos, sin, k_cache=None, v_cache=None, slot_mapping=None):
    """RoPE at ``positions`` on q and k, then scatter of the rotated k and of v (fused step in front of attention).

    Composition of ``apply_rope`` (rotary application of nano-vdllm/model/modeling_llada.py:412-453: fp32
    ``x*cos + rot_half(x)*sin`` with the table rows of the position ids, cast back) and ``store_kvcache``
    (nano-vdllm/model/attention.py:22-41).  Returns the rotated ``(q, k)``; the caches are updated in place.
    """
    idx = positions.long()
    q_rot = apply_rope(q, cos[idx], sin[idx])
    k_rot = apply_rope(k, cos[idx], sin[idx])
    if slot_mapping is not None:
        store_kvcache(k_rot, v, k_cache, v_cache, slot_mapping)
    return q_rot, k_rot


def argmax_confidence(logits, picks=None):
    """Token and confidence of the transfer rule, nano-vdllm/model_runner.py:2279-2296: ``x0 = argmax`` (or the
    given picks) and ``exp(logit[x0] - logsumexp(row))`` on the fp32 up-cast."""
    rows = logits.reshape(-1, logits.shape[-1]).float()
    x0 = rows.argmax(dim=-1) if picks is None else picks.reshape(-1).long()
    chosen = rows.gather(-1, x0[:, None]).squeeze(-1)
    conf = torch.exp(chosen - torch.logsumexp(rows, dim=-1))
    return x0.view(logits.shape[:-1]), conf.view(logits.shape[:-1])


def affix_importance(q, k_cache, mask_rows, cu_mask, affix_len, scale=None, affix_shifts=None, cos=None, sin=None,
                     affix_slot0=0):
    """One layer's affix importance ``[B, affix_len]`` fp32 (nano-vdllm/model_runner.py:730-773).

    Per request: the cached affix keys (slots ``affix_slot0 ..``, cached at positions ``0 .. A-1``) are re-rotated
    to start at ``affix_shifts[b]`` (rounded to the cache dtype, like ``block.rotary_emb`` there), the [MASK]
    queries are scored against them, the softmax runs over the affix keys only, and the weights are summed over
    queries and heads.  The reference evaluates ``matmul`` / ``softmax`` in the model dtype; this restatement uses
    fp32 for both, which is what the bound "within tolerance" is stated against.
    """
    H, D = q.shape[1], q.shape[2]
    flat = _flat(k_cache)
    H_kv = flat.shape[1]
    scale = D ** -0.5 if scale is None else scale
    B = len(cu_mask) - 1
    out = torch.zeros(B, affix_len, dtype=torch.float32)
    keys = flat[affix_slot0:affix_slot0 + affix_len]
    for b in range(B):
        rows = mask_rows[int(cu_mask[b]):int(cu_mask[b + 1])].long()
        if rows.numel() == 0 or affix_len == 0:
            continue
        k = keys
        shift = int(affix_shifts[b]) if affix_shifts is not None else 0
        if shift:
            k = rotate(keys, torch.full((affix_len,), shift, dtype=torch.int32), cos, sin)
        kh = k.float().permute(1, 0, 2).repeat_interleave(H // H_kv, dim=0)          # [H, A, D]
        qh = q[rows].float().permute(1, 0, 2)                                           # [H, M, D]
        w = torch.softmax(torch.matmul(qh, kh.transpose(-2, -1)) * scale, dim=-1)       # [H, M, A]
        out[b] = w.sum(dim=(0, 1))
    return out


def rotate(x: torch.Tensor, delta: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor) -> torch.Tensor:
    """Rotate rows ``x[t]`` (``[T, H, D]``) by signed per-row position shifts ``delta[t]``.

    Key-side relocation rule of acache_attention.py:481-497: table row ``|delta|``,
    ``sin`` negated where ``delta < 0``.  Rows with ``delta == 0`` are returned
    unchanged (bit copies).
    """
    delta = delta.to(torch.long)
    c = cos[delta.abs()]
    s = sin[delta.abs()]
    s = torch.where((delta < 0)[:, None], -s, s)
    y = apply_rope(x, c.float(), s.float())
    return torch.where((delta == 0)[:, None, None], x, y)


def rotate_query_inverse(q: torch.Tensor, shift: int, cos: torch.Tensor, sin: torch.Tensor) -> torch.Tensor:
    """``q' = (q*cos[s] - rot_half(q)*sin[s]).to(q.dtype)`` (acache_attention.py:399-419)."""
    c = cos[shift].float()
    s = sin[shift].float()
    return (q * c - rot_half(q) * s).to(q.dtype)


# ------------------------------------------------------------------ slots / layout
def anchor_budget(anchor_ratio: float, affix_len: int) -> int:
    """``min(ceil(ratio*A), A)`` on the Python double product (nano-vdllm/sequence.py:147)."""
    return min(math.ceil(anchor_ratio * affix_len), affix_len)


def ceil_to_int(value: float) -> int:
    """HF-path spelling of the same ceiling (llada/generate_ACache.py:37-41)."""
    integer = int(value)
    return integer if value == integer else integer + 1


def slots_from_block_table(block_table, length: int, block_size: int) -> list[int]:
    """``bt[p // BS] * BS + p % BS`` for ``p < length`` (acache_attention.py:194-196; model_runner.py:1100-1110)."""
    return [int(block_table[p // block_size]) * block_size + p % block_size for p in range(length)]


def private_slots(block_table, num_private_slots: int, block_size: int) -> list[int]:
    """Slots of a request's own blocks, block by block (nano-vdllm/sequence.py:171-179)."""
    out: list[int] = []
    nblocks = -(-num_private_slots // block_size)
    for i in range(nblocks):
        start = int(block_table[i]) * block_size
        n = block_size if i != nblocks - 1 else num_private_slots - (nblocks - 1) * block_size
        out.extend(range(start, start + n))
    return out


def finalize_slot_mapping(
    num_tokens: int,
    affix_start: int,
    affix_end: int,
    anchor_positions: list[int],
    block_table,
    block_size: int,
    shared_slot_offset: int = 0,
):
    """Pure-Python restatement of ``Sequence.finalize_slot_mapping`` (nano-vdllm/sequence.py:169-202).

    Returns ``(read_slot_map, recompute_positions, recompute_slot_mapping)``.
    """
    affix_len = affix_end - affix_start
    k = len(anchor_positions)
    priv = private_slots(block_table, k + num_tokens - affix_len, block_size)
    anchor_slots, dynamic_slots = priv[:k], priv[k:]
    non_affix = list(range(affix_start)) + list(range(affix_end, num_tokens))
    assert len(dynamic_slots) == len(non_affix)
    slot_of = {}
    for pos, slot in zip(sorted(anchor_positions), anchor_slots):
        slot_of[pos] = slot
    read = [-1] * num_tokens
    for local, pos in enumerate(range(affix_start, affix_end)):
        read[pos] = slot_of.get(pos, shared_slot_offset + local)
    for pos, slot in zip(non_affix, dynamic_slots):
        read[pos] = slot
        slot_of[pos] = slot
    recompute_positions = sorted(slot_of)
    return read, recompute_positions, [slot_of[p] for p in recompute_positions]


def attention_read_layout(read_slot_map, shared_slot_offset, shared_prefix_len, affix_start, use_query_relocation):
    """Shared slots packed first for query-side relocation (nano-vdllm/model_runner.py:275-282)."""
    if not use_query_relocation or affix_start == 0:
        return list(read_slot_map), 0
    lo, hi = shared_slot_offset, shared_slot_offset + shared_prefix_len
    shared = [s for s in read_slot_map if lo <= s < hi]
    rest = [s for s in read_slot_map if not (lo <= s < hi)]
    return shared + rest, len(shared)


def key_side_deltas(read_slot_map, shared_prefix_len: int) -> list[int]:
    """``delta[n] = n - slot`` for rows with ``slot < shared_prefix_len``, else 0 (acache_attention.py:481-482)."""
    return [n - s if s < shared_prefix_len else 0 for n, s in enumerate(read_slot_map)]


# ------------------------------------------------------------- gather / scatter
def _flat(cache: torch.Tensor) -> torch.Tensor:
    """View a ``[..., H, D]`` cache layer as ``[num_slots, H, D]``."""
    return cache.reshape(-1, cache.shape[-2], cache.shape[-1])


def relocate_rope_gather(k_cache, v_cache, slot_map, delta, cos, sin):
    """Un-fused relocate + re-rotate + gather over all layers.

    ``k_cache``/``v_cache``: ``[L, S, H, D]`` (or ``[L, NB, BS, H, D]``);
    ``K_out[l, t] = rotate(K[l, slot[t]], delta[t])``, ``V_out[l, t] = V[l, slot[t]]``.
    The gather is ``flat_cache[slots.long()]`` exactly as the reference's tests
    build ``eff_k`` (test_attention_kernels.py:524-531); the rotation is the
    key-side rule (acache_attention.py:480-497).
    """
    L = k_cache.shape[0]
    idx = torch.as_tensor(slot_map, dtype=torch.long)
    ks, vs = [], []
    for l in range(L):
        k = _flat(k_cache[l]).index_select(0, idx)
        v = _flat(v_cache[l]).index_select(0, idx)
        if delta is not None:
            k = rotate(k, torch.as_tensor(delta), cos, sin)
        ks.append(k)
        vs.append(v)
    return torch.stack(ks), torch.stack(vs)


def materialize_relocated_affix(k_cache, v_cache, cos, sin, dst_slot: int, affix_len: int, affix_shift: int):
    """In-place copy of affix rows with rotated keys (acache_attention.py:29-85, 88-128).

    ``k_cache``/``v_cache``: ``[L, S, H, D]``.  ``K[l, dst+t] = rotate(K[l, t], shift)``,
    ``V[l, dst+t] = V[l, t]``; expected value as in test_attention_kernels.py:158-165.
    """
    L = k_cache.shape[0]
    for l in range(L):
        src_k = k_cache[l, :affix_len].clone()
        c = cos[affix_shift].float().expand(affix_len, -1)
        s = sin[affix_shift].float().expand(affix_len, -1)
        k_cache[l, dst_slot:dst_slot + affix_len] = apply_rope(src_k, c, s)
        v_cache[l, dst_slot:dst_slot + affix_len] = v_cache[l, :affix_len].clone()


def store_kvcache(key, value, k_cache, v_cache, slot_mapping):
    """``cache.flat[slot] = row`` for ``slot != -1`` (nano-vdllm/model/attention.py:22-31)."""
    fk, fv = _flat(k_cache), _flat(v_cache)
    for i, slot in enumerate(torch.as_tensor(slot_mapping).tolist()):
        if slot == -1:
            continue
        fk[slot] = key[i]
        fv[slot] = value[i]


# ------------------------------------------------------------------------ top-k
def topk_anchors(scores, k: int, largest: bool = True, offset: int = 0) -> list[int]:
    """Indices of the ``k`` best scores, ascending, ties to the lower index.

    nano-vdllm/model_runner.py:833-843 (``torch.topk`` then ``.sort()`` then
    ``+ affix_start``).  torch does not define which of several equal scores is
    returned; the contract here is the stable order
    ``sorted(range(A), key=(-score, index))[:k]``.
    """
    s = np.asarray(torch.as_tensor(scores, dtype=torch.float32).numpy(), dtype=np.float32)
    s = np.where(s == 0, np.float32(0), s)  # -0.0 == +0.0
    a = s.shape[0]
    k = min(int(k), a)
    key = -s if largest else s
    # NaN ranks as the largest value (torch.topk convention)
    key = np.where(np.isnan(s), -np.inf if largest else np.inf, key)
    order = np.lexsort((np.arange(a), key))  # primary: key ascending; secondary: index
    return sorted(int(i) + offset for i in order[:k])


# -------------------------------------------------------------------- attention
def dense_attention_reference(q, k, v, num_heads: int, num_kv_heads: int, scale: float | None = None):
    """fp32 ``softmax(Q K^T * scale) V`` per head with ``kv_head = h // group``.

    nano-vdllm/tests/test_attention_kernels.py:88-109.  ``q``: ``[Tq, H, D]``;
    ``k``/``v``: ``[Tk, H_kv, D]``; result in ``q.dtype``.
    """
    dtype = q.dtype
    group = num_heads // num_kv_heads
    qf, kf, vf = q.float(), k.float(), v.float()
    out = torch.empty_like(qf)
    if scale is None:
        scale = q.shape[-1] ** -0.5
    for h in range(num_heads):
        g = h // group
        scores = torch.matmul(qf[:, h], kf[:, g].transpose(0, 1)) * scale
        out[:, h] = torch.matmul(torch.softmax(scores, dim=-1), vf[:, g])
    return out.to(dtype)


def acache_attention(
    q, k_cache, v_cache, cu_seqlens_q, cu_seqlens_k, read_slot_mapping,
    softmax_scale=None, shared_prefix_len=0, shared_kv_lens=None, affix_shifts=None,
    rope_cos=None, rope_sin=None,
):
    """Varlen bidirectional attention through a slot map, three relocation modes.

    Semantics of nano-vdllm/model/acache_attention.py:337-514 / 643-738, evaluated
    per request with fp32 dense attention:
      plain       K_b[n] = K[slot[n]]
      key side    rows with slot < shared_prefix_len rotated by n - slot, rounded
                  to the cache dtype (line 497)
      query side  first shared_kv_lens[b] keys scored against
                  q' = round(q*cos[s] - rot_half(q)*sin[s]) (line 419)
    Requests without keys produce zeros (the reference leaves them uninitialised).
    """
    num_heads, head_dim = q.shape[1], q.shape[2]
    num_kv_heads = k_cache.shape[-2]
    group = num_heads // num_kv_heads
    scale = head_dim ** -0.5 if softmax_scale is None else softmax_scale
    fk, fv = _flat(k_cache), _flat(v_cache)
    cu_q = torch.as_tensor(cu_seqlens_q).tolist()
    cu_k = torch.as_tensor(cu_seqlens_k).tolist()
    slots_all = torch.as_tensor(read_slot_mapping, dtype=torch.long)
    apply_reloc = shared_prefix_len > 0 and affix_shifts is not None
    query_side = apply_reloc and shared_kv_lens is not None
    out = torch.zeros_like(q)
    for b in range(len(cu_q) - 1):
        q_b = q[cu_q[b]:cu_q[b + 1]]
        slots = slots_all[cu_k[b]:cu_k[b + 1]]
        if q_b.shape[0] == 0 or slots.numel() == 0:
            continue
        k_b, v_b = fk[slots], fv[slots]
        if apply_reloc and not query_side:
            n = torch.arange(slots.numel())
            delta = torch.where(slots < shared_prefix_len, n - slots, torch.zeros_like(n))
            k_b = rotate(k_b, delta, rope_cos, rope_sin)
        qf, kf, vf = q_b.float(), k_b.float(), v_b.float()
        if query_side:
            shared_len = int(torch.as_tensor(shared_kv_lens)[b])
            shift = int(torch.as_tensor(affix_shifts)[b])
            q_shared = rotate_query_inverse(q_b, shift, rope_cos, rope_sin).float()
        for h in range(num_heads):
            g = h // group
            scores = torch.matmul(qf[:, h], kf[:, g].T)
            if query_side and shared_len > 0:
                scores[:, :shared_len] = torch.matmul(q_shared[:, h], kf[:shared_len, g].T)
            probs = torch.softmax(scores * scale, dim=-1)
            out[cu_q[b]:cu_q[b + 1], h] = torch.matmul(probs, vf[:, g]).to(q.dtype)
    return out


# --------------------------------------------------------------- token transfer
def get_transfer_index(logits, mask_index, x, threshold: float = 0.9):
    """Greedy (temperature 0) confidence-threshold token transfer.

    nano-vdllm/model_runner.py:2279-2314 with ``remasking='low_confidence'``:
    ``x0 = argmax``, ``p = exp(logit[x0] - logsumexp)``, transfer where
    ``p >= threshold`` among masked positions, and force the most confident
    masked position of a row that would otherwise transfer nothing.
    """
    lf = logits.float()
    x0 = lf.argmax(dim=-1)
    p = torch.exp(torch.gather(lf, -1, x0.unsqueeze(-1)).squeeze(-1) - torch.logsumexp(lf, dim=-1))
    x0 = torch.where(mask_index, x0, x)
    conf = torch.where(mask_index, p, torch.full_like(p, -float("inf")))
    transfer = (conf >= threshold) & mask_index
    needs = mask_index.any(dim=1) & ~transfer.any(dim=1)
    rows = torch.where(needs)[0]
    transfer[rows, conf.argmax(dim=1)[rows]] = True
    return x0, transfer
