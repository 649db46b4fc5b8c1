"""Batch-1 ACache generation for Dream-shaped models, with the signatures of ``dream/generate_ACache.py``.

Same engine path as ``acache_amd.generate_acache`` (paged cache, HIP kernels); what differs is the decoding
rule of Dream (dream/generate_ACache.py:425-737):

* logits are aligned one position to the left (line 47-49): token ``i`` is read from the hidden state of the
  previous recomputed position, inside a refinement step from the previous position of the block;
* a block refresh commits only the block's first token (lines 686-690); the remaining
  ``steps_per_block - 1`` steps share the transfer quota (lines 692-696);
* with ``anchor_ratio`` reaching the whole affix, every affix token is an anchor and no importance pass is
  run (lines 556-562).

``precomputed_affix_cache`` may use Dream's HF layout: per layer ``(k, v)`` of shape ``[1, A, H_kv * D]`` with
keys before RoPE.
"""
from __future__ import annotations

from typing import Optional, Tuple

import torch

from .generate_acache import (  # noqa: F401  (same public names as the reference module)
    _coerce_bool, _generate, ceil_to_int, compute_attention_importance_cross_affix, gather_tokens_for_recompute,
    get_num_transfer_tokens, get_transfer_index, get_transfer_index_dynamic, sample_tokens, select_anchor_tokens)


def _align_logits_for_dream(logits: torch.Tensor) -> torch.Tensor:
    """Row ``i`` takes the logits of row ``i - 1``; row 0 keeps its own."""
    return torch.cat([logits[:, :1], logits[:, :-1]], dim=1)


def generate_with_anchor_attention(
    model,
    prompt: torch.Tensor,
    steps: int = 128,
    gen_length: int = 128,
    block_length: int = 128,
    temperature: float = 0.0,
    remasking: str = "low_confidence",
    mask_id: int = 126336,
    threshold: Optional[float] = None,
    factor: Optional[float] = None,
    affix_start: int = 0,
    affix_end: Optional[int] = None,
    generation_start: Optional[int] = None,
    anchor_ratio: float = 0.1,
    selection_mode: str = "top",
    drop_non_anchor: bool = False,
    precomputed_affix_cache: Optional[Tuple[Tuple[torch.Tensor, torch.Tensor], ...]] = None,
) -> Tuple[torch.Tensor, int]:
    """Dream decoding with affix-KV reuse; returns ``(x, nfe)`` like the reference."""
    return _generate(model, prompt, steps, gen_length, block_length, temperature, remasking, mask_id, threshold, factor,
                     affix_start, affix_end, generation_start, anchor_ratio, selection_mode, drop_non_anchor,
                     precomputed_affix_cache, dream=True)
