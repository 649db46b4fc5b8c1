"""``Attention`` module: scatter fresh K/V into the paged cache, then attend through it.

Mirror of nano-vdllm/model/attention.py:44-123: same constructor, the same
externally-set attributes (``k_cache``, ``v_cache``, ``use_reference_attention``,
``shared_prefix_len``, ``relocation_rope_cos``, ``relocation_rope_sin``) and the same
dispatch on the global ``Context``.  Every branch runs the HIP kernels of this
package; the reference's two flash-attn branches map onto them as well
(``flash_attn_varlen_func`` on fresh q/k/v is varlen attention with an identity
slot map over ``k``/``v`` themselves, ``flash_attn_with_kvcache`` is the block-table
decode form), so no external attention library is needed.
"""
from __future__ import annotations

import torch
from torch import nn

from . import ops
from .utils import get_context


class Attention(nn.Module):
    def __init__(self, num_heads, head_dim, num_kv_heads, scale=None):
        super().__init__()
        self.num_heads = num_heads
        self.head_dim = head_dim
        self.num_kv_heads = num_kv_heads
        self.scale = scale
        self.use_reference_attention = False
        self.shared_prefix_len = 0
        self.relocation_rope_cos = self.relocation_rope_sin = torch.tensor([])
        self.k_cache = self.v_cache = torch.tensor([])
        # optional observer called as probe(self, q) before attention; used by the
        # anchor-selection pass to accumulate affix importance (model_runner.py:730-773
        # patches forward for the same purpose)
        self.probe = None

    def forward(self, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, kv_stored: bool = False):
        """``kv_stored``: the caller has already written ``k`` / ``v`` to ``context.slot_mapping`` (the fused
        rotary + scatter launch); everything else is the reference's ``forward(q, k, v)``."""
        context = get_context()
        k_cache, v_cache = self.k_cache, self.v_cache
        assert k_cache.numel() and v_cache.numel()
        batched = k.dim() == 4  # [B, L, H, D] block refinement input
        if batched:
            bs, seqlen = k.shape[:2]
            k = k.reshape(bs * seqlen, self.num_kv_heads, self.head_dim)
            v = v.reshape(bs * seqlen, self.num_kv_heads, self.head_dim)
        if not kv_stored:
            ops.store_kvcache(k, v, k_cache, v_cache, context.slot_mapping)
        if self.probe is not None:
            self.probe(self, q)
        scale = self.scale if self.scale is not None else self.head_dim ** -0.5
        if context.use_acache:
            q3 = q.reshape(-1, self.num_heads, self.head_dim) if q.dim() == 4 else q
            if (self.shared_prefix_len > 0 and context.affix_shifts is not None and context.max_seqlen_k
                    and self.relocation_rope_cos.shape[0] < context.max_seqlen_k):
                # a shift is a position inside its request, so the longest request bounds every shift; the kernels
                # only clamp out-of-table rows for memory safety and would return unrotated keys (the reference
                # asserts the same bound after a device read-back, acache_attention.py:685)
                raise ValueError(f"relocation RoPE table has {self.relocation_rope_cos.shape[0]} rows, "
                                 f"the longest request needs {context.max_seqlen_k}")
            o = ops.acache_attention(
                q3, k_cache, v_cache, context.cu_seqlens_q, context.cu_seqlens_k,
                context.read_slot_mapping, scale, self.shared_prefix_len,
                context.shared_kv_lens, context.affix_shifts,
                self.relocation_rope_cos if self.relocation_rope_cos.numel() else None,
                self.relocation_rope_sin if self.relocation_rope_sin.numel() else None,
                plan=context.attention_plan,
            )
            return o.view(bs, seqlen, self.num_heads, self.head_dim) if q.dim() == 4 else o
        if context.is_caching:
            if self.use_reference_attention:
                # fresh (unpaged) q, k, v: identity slot map over the rows just computed
                total = k.shape[0]
                slots = torch.arange(total, dtype=torch.int32, device=k.device)
                return ops.acache_attention(q, k, v, context.cu_seqlens_q, context.cu_seqlens_k, slots, scale,
                                            plan=context.attention_plan)
            total_k = getattr(context, "total_k", None)
            return ops.baseline_ragged_attention(
                q, k_cache, v_cache, context.cu_seqlens_q, context.cu_seqlens_k, context.block_tables,
                scale, total_k=total_k if total_k is not None else int(context.cu_seqlens_k[-1].item()),
                plan=context.attention_plan)
        q4 = q if q.dim() == 4 else q.view(-1, 1, self.num_heads, self.head_dim)
        total_k = getattr(context, "total_k", None)
        return ops.baseline_decode_attention(q4, k_cache, v_cache, context.seqlens, context.block_tables, scale,
                                             total_k=total_k)
