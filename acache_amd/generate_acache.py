"""Batch-1 ACache generation entry points with the signatures of the reference's HF path.

Reference: ``llada/generate_ACache.py`` (``ceil_to_int`` 37-41,
``compute_attention_importance_cross_affix`` 44-222, ``select_anchor_tokens`` 225-262,
``gather_tokens_for_recompute`` 265-308, ``generate_with_anchor_attention`` 311-629) and the
transfer helpers of ``llada/generate.py`` (61-83, 298-376).

The reference runs this path on dense ``[B, H, L, D]`` caches of an HF-style model.  Here the same
algorithm — affix K/V computed once, K anchors chosen by cross-affix importance, anchors and
non-affix tokens recomputed at every block boundary, block-only refinement in between — runs on
the paged engine of this package (``ModelRunner`` + HIP kernels).  Consequences for callers:

* ``model`` is the checkpoint model object the reference's caller passes (llada/eval_ACache.py:100-107, 189):
  the engine model is built around its parameter tensors on first use (the q/k/v and gate/up projections become
  merged copies, everything else is shared: ``llada.adopt_state``; settings the engine's decoder stack does not
  implement raise ``TypeError``).  An engine model
  (``acache_amd.llada.LLaDAModelLM``) or a ready ``ModelRunner`` is taken as it is;
* ``precomputed_affix_cache`` is optional.  ``None``: the affix is encoded once into the shared
  slots.  A per-layer tuple of ``(k, v)`` with the HF layout ``[1, H_kv, A, D]`` and PRE-RoPE keys
  (llada/generate_ACache.py:153) is rotated to positions ``0..A-1`` and scattered into the shared
  slots instead of being recomputed (the Dream layout ``[1, A, H_kv * D]`` is accepted too);
* ``drop_non_anchor`` is served by leaving the frozen affix rows out of the request's read slot map:
  anchors and non-affix tokens keep their position ids and never see the dropped tokens
  (the reference's compact kept-position sequence, llada/generate_ACache.py:478-491).
"""
from __future__ import annotations

from typing import Optional, Tuple

import torch
import torch.nn.functional as F

from .checkpoint import engine_model_for

from . import ops
from .config import Config
from .model_runner import ModelRunner
from .ops import select_anchor_tokens  # noqa: F401  (re-exported: same name as the reference)
from .sequence import Sequence
from .utils import add_gumbel_noise, reset_context


def _coerce_bool(value, default: bool, arg_name: str) -> bool:
    """``None`` -> default; bools and numbers by truth value; otherwise the usual string spellings
    (llada/generate_ACache.py:21-35: the evaluation CLI hands strings through)."""
    if value is None:
        return default
    if isinstance(value, (bool, int, float)):
        return bool(value)
    text = str(value).strip().lower()
    if text in ("1", "true", "yes", "y", "on"):
        return True
    if text in ("0", "false", "no", "n", "off"):
        return False
    raise ValueError(f"{arg_name} must be a boolean-like value, got {value!r}.")


def ceil_to_int(value: float) -> int:
    integer = int(value)
    return integer if value == integer else integer + 1


def gather_tokens_for_recompute(x, anchor_global_indices, block_start: int, block_end: int):
    """Tokens at the anchor positions followed by the block tokens, and the mask of replaced positions."""
    B, L = x.shape
    replace_position = torch.zeros(B, L, dtype=torch.bool, device=x.device)
    replace_position.scatter_(1, anchor_global_indices, True)
    replace_position[:, block_start:block_end] = True
    gathered = torch.cat([x.gather(1, anchor_global_indices), x[:, block_start:block_end]], dim=1)
    return gathered, replace_position


def get_num_transfer_tokens(block_mask_index: torch.Tensor, steps: int) -> torch.Tensor:
    """``(B, steps)`` tokens to commit per step: masked count split evenly, remainder to the first steps."""
    total = block_mask_index.sum(dim=1)
    base = torch.div(total, steps, rounding_mode="floor")
    rem = total - base * steps
    cols = torch.arange(steps, device=block_mask_index.device).unsqueeze(0)
    return (base.unsqueeze(1) + (cols < rem.unsqueeze(1))).to(torch.long)


def get_transfer_index(logits, temperature, remasking, mask_index, x, num_transfer_tokens, threshold=None):
    """HF-path token transfer (llada/generate.py:298-376): threshold mode or per-row quota mode."""
    x0 = torch.argmax(add_gumbel_noise(logits, temperature=temperature), dim=-1)
    if remasking == "low_confidence":
        p = F.softmax(logits.to(torch.float64), dim=-1)
        x0_p = torch.gather(p, dim=-1, index=x0.unsqueeze(-1)).squeeze(-1)
    elif remasking == "random":
        x0_p = torch.rand(x0.shape, device=x0.device, dtype=torch.float64)
    else:
        raise NotImplementedError(remasking)
    x0 = torch.where(mask_index, x0, x)
    confidence = torch.where(mask_index, x0_p, torch.full_like(x0_p, torch.finfo(x0_p.dtype).min))
    if threshold is not None:
        transfer = mask_index & (confidence >= threshold)
        force = torch.zeros_like(transfer).scatter_(1, confidence.argmax(dim=1, keepdim=True), True)
        return x0, (transfer | force) & mask_index
    if num_transfer_tokens is None:
        raise ValueError("num_transfer_tokens must be a tensor when threshold is None.")
    k = num_transfer_tokens.reshape(-1).to(torch.long).clamp(min=0)
    _, idx = torch.sort(confidence, dim=1, descending=True)
    cols = torch.arange(confidence.shape[1], device=confidence.device).unsqueeze(0)
    picked = torch.zeros_like(confidence, dtype=torch.int8).scatter(1, idx, (cols < k.unsqueeze(1)).to(torch.int8))
    return x0, picked.bool() & mask_index


def get_transfer_index_dynamic(logits, temperature, remasking, mask_index, x, num_transfer_tokens, factor=1):
    """Dynamic-threshold transfer (llada/generate.py:379-420).

    Per row, with n masked tokens and their confidences sorted descending c_1 >= ... >= c_n: commit the
    leading tokens while c_i >= 1 - factor / (i + 1) (the first always passes), stopping at the first
    failure.  The reference's loop leaves ``top_i`` at the failing index, or at n - 1 when nothing fails, and
    then adds one when ``top_i`` is 0 or n - 1; both quirks are kept: a row whose only failure is its last
    token commits all n.  ``num_transfer_tokens`` is ignored, as in the reference.
    """
    x0 = torch.argmax(add_gumbel_noise(logits, temperature=temperature), dim=-1)
    if remasking == "low_confidence":
        p = F.softmax(logits.to(torch.float64), dim=-1)
        x0_p = torch.gather(p, dim=-1, index=x0.unsqueeze(-1)).squeeze(-1)
    elif remasking == "random":
        x0_p = torch.rand(x0.shape, device=x0.device, dtype=torch.float64)
    else:
        raise NotImplementedError(remasking)
    x0 = torch.where(mask_index, x0, x)
    confidence = torch.where(mask_index, x0_p, torch.full_like(x0_p, float("-inf")))
    transfer = torch.zeros_like(x0, dtype=torch.bool)
    counts = mask_index.sum(dim=1).tolist()
    ordered, order = torch.sort(confidence, dim=1, descending=True, stable=True)
    ordered = ordered.tolist()
    for j, n in enumerate(counts):
        if n == 0:
            continue
        top_i = 0
        for top_i in range(n):
            thresh = -1.0 if top_i == 0 else 1.0 - factor / (top_i + 2)
            if ordered[j][top_i] < thresh:
                break
        if top_i == 0 or top_i == n - 1:
            top_i += 1
        transfer[j, order[j, :top_i]] = True
    return x0, transfer


# ------------------------------------------------------------------------------------------ engine glue
def _as_runner(model, *, mask_id, block_length, gen_length, anchor_ratio, selection_mode, threshold,
               temperature, remasking, total_len, affix_len) -> ModelRunner:
    if isinstance(model, ModelRunner):
        runner = model
        runner.config.anchor_ratio = anchor_ratio
        runner.config.selection_mode = selection_mode
        runner.config.block_length = block_length
        runner.config.gen_length = gen_length
        return runner
    model = engine_model_for(model)
    bs = 256
    blocks = 2 * (-(-affix_len // bs)) + -(-(total_len + affix_len) // bs) + 2
    cfg = Config(hf_config=model.config, mask_id=mask_id, recompute_batch_size=1, max_num_seqs=1,
                 gen_length=gen_length, block_length=block_length, remasking=remasking,
                 threshold=threshold if threshold is not None else 0.9, cache_block_size=bs,
                 num_kvcache_blocks=blocks, temperature=temperature, enable_acache=True,
                 anchor_ratio=anchor_ratio, selection_mode=selection_mode)
    return ModelRunner(model, cfg)


def _ingest_affix_cache(runner: ModelRunner, affix_tokens, affix_cache):
    """Place an HF-layout affix cache (pre-RoPE keys, ``[1, H_kv, A, D]`` per layer) into the shared slots."""
    n = len(affix_tokens)
    bs = runner.config.cache_block_size
    shared_blocks = -(-n // bs)
    runner.block_manager.reserve_prefix(shared_blocks)
    blocks = runner._llada_blocks()
    assert len(affix_cache) == len(blocks), "precomputed_affix_cache must have one (key, value) pair per layer"
    positions = torch.arange(n, device=runner.device)
    slots = torch.arange(n, dtype=torch.int32, device=runner.device)
    hkv, hd = runner.kv_cache.shape[-2], runner.kv_cache.shape[-1]
    for (k, v), block in zip(affix_cache, blocks):
        if k.dim() == 4:   # LLaDA HF layout [1, H_kv, A, D]
            k = k[0].permute(1, 0, 2)
            v = v[0].permute(1, 0, 2)
        else:              # Dream HF layout [1, A, H_kv * D] (dream/generate_ACache.py:198)
            k = k[0].view(n, hkv, hd)
            v = v[0].view(n, hkv, hd)
        k = k.contiguous().to(runner.kv_cache.dtype)
        v = v.contiguous().to(runner.kv_cache.dtype)
        if getattr(runner.config.hf_config, "rope", True):
            _, k = block.rotary_emb(k, k, positions, max(n, runner.config.hf_config.max_sequence_length))
        ops.store_kvcache(k.contiguous(), v, block.attn.k_cache, block.attn.v_cache, slots)
    runner.shared_prefix_len = n
    runner.shared_prefix_blocks = shared_blocks
    runner.shared_prefix_token_ids = tuple(affix_tokens)
    runner.acache_ready = True


@torch.no_grad()
def compute_attention_importance_cross_affix(model, full_input_ids, affix_cache=None, mask_id=126336,
                                             affix_start=0, affix_len=None):
    """``(1, A)`` fp32 importance of every affix token for the [MASK] queries of ``full_input_ids``.

    Same quantity as llada/generate_ACache.py:44-222 (softmax over the affix keys only, summed over
    layers, heads and mask queries), computed by the engine's probe forward.
    """
    assert full_input_ids.shape[0] == 1
    tokens = full_input_ids[0].tolist()
    if affix_len is None:
        assert affix_cache is not None, "affix_len or affix_cache is required"
        sample_k = affix_cache[0][0]
        affix_len = sample_k.shape[2] if sample_k.dim() == 4 else sample_k.shape[1]
    runner = _as_runner(model, mask_id=mask_id, block_length=1, gen_length=0, anchor_ratio=1.0,
                        selection_mode="top", threshold=None, temperature=0.0, remasking="low_confidence",
                        total_len=len(tokens), affix_len=affix_len)
    affix_end = affix_start + affix_len
    if affix_len == 0 or affix_len >= len(tokens):  # nothing to score, or no query outside the affix
        return torch.zeros(1, affix_len, dtype=torch.float32, device=runner.device)
    # zero-length generation window anchored on a non-affix position (the probe only needs the queries)
    anchor_pos = 0 if affix_start > 0 else affix_end
    seq = Sequence(tokens, gen_length=0, block_length=1, cache_block_size=runner.config.cache_block_size,
                   mask_id=mask_id, prompt_affix_start=affix_start, prompt_affix_end=affix_end,
                   generation_start=anchor_pos)
    _ensure_affix(runner, seq, affix_cache)
    seq.enable_acache(affix_len, 1.0, affix_start=affix_start, affix_end=affix_end)
    return runner._compute_affix_importance([seq])


def _ensure_affix(runner, seq, affix_cache):
    affix_tokens = seq.prompt_affix_token_ids
    if runner.acache_ready and runner.shared_prefix_token_ids == tuple(affix_tokens):
        return
    if runner.acache_ready:  # a different affix: start from a clean cache layout
        runner.allocate_kv_cache(runner.config.num_kvcache_blocks)
    if affix_cache is None:
        runner._precompute_shared_prefix(list(affix_tokens))
    else:
        _ingest_affix_cache(runner, affix_tokens, affix_cache)


@torch.no_grad()
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
    """Generate with affix-KV reuse: recompute anchors + non-affix tokens per block, keep the rest frozen.

    Returns ``(x, nfe)`` with ``x`` of shape ``(1, prompt_len [+ gen_length])`` like the reference.
    """
    return _generate(model, prompt, steps, gen_length, block_length, temperature, remasking, mask_id, threshold, factor,
                     affix_start, affix_end, generation_start, anchor_ratio, selection_mode, drop_non_anchor,
                     precomputed_affix_cache, dream=False)


def sample_tokens(logits, temperature=0.0):
    """``(confidence, token)`` per row: arg-max of the softmax at temperature 0, a categorical draw from
    ``softmax(logits / temperature)`` otherwise (dream/model/generation_utils_block.py:80-112 without top-p/top-k)."""
    if temperature > 0:
        logits = logits / temperature
    probs = torch.softmax(logits, dim=-1)
    if temperature > 0:
        x0 = torch.distributions.Categorical(probs=probs).sample()
        return torch.gather(probs, -1, x0.unsqueeze(-1)).squeeze(-1), x0
    return probs.max(dim=-1)


def _shift_right(logits):
    """Dream alignment (dream/generate_ACache.py:47-49): row i takes the logits of row i - 1, row 0 keeps its own."""
    return torch.cat([logits[:, :1], logits[:, :-1]], dim=1)


@torch.no_grad()
def _generate(model, prompt, steps, gen_length, block_length, temperature, remasking, mask_id, threshold, factor,
              affix_start, affix_end, generation_start, anchor_ratio, selection_mode, drop_non_anchor,
              precomputed_affix_cache, dream: bool):
    """Shared body of the LLaDA (llada/generate_ACache.py:311-629) and Dream (dream/generate_ACache.py:425-737)
    entry points.  Dream differs in four places: all-anchor selection skips the importance pass, logits are taken
    one compact position to the left, a block refresh commits only the block's first token, and the remaining
    ``steps_per_block - 1`` steps share the quota."""
    B = prompt.shape[0]
    assert B == 1, "generate_with_anchor_attention currently supports batch_size=1."
    drop_non_anchor = _coerce_bool(drop_non_anchor, default=False, arg_name="drop_non_anchor")
    Lp = int(prompt.shape[1])
    assert gen_length % block_length == 0
    num_blocks = gen_length // block_length
    assert steps % num_blocks == 0
    steps_per_block = steps // num_blocks

    tokens = prompt[0].tolist()
    if generation_start is None:
        gen_start, total_len = Lp, Lp + gen_length
    else:
        gen_start = int(generation_start)
        if gen_start < 0:
            raise ValueError("generation_start must be non-negative.")
        if gen_start + gen_length > Lp:
            raise ValueError("generation_start + gen_length must be <= prompt length for infill mode.")
        total_len = Lp
    if affix_end is None:
        affix_end = Lp
    if affix_end > total_len:
        raise ValueError("affix_end must be <= sequence length.")
    if not affix_start <= affix_end:
        raise ValueError("affix_start must be <= affix_end.")
    if gen_start < affix_end and gen_start + gen_length > affix_start:
        raise ValueError(
            "Generation span must not overlap affix span. "
            f"Got generation=[{gen_start}, {gen_start + gen_length}), affix=[{affix_start}, {affix_end}).")
    affix_len = affix_end - affix_start
    if precomputed_affix_cache is not None:
        sample_k = precomputed_affix_cache[0][0]
        cached_len = sample_k.shape[2] if sample_k.dim() == 4 else sample_k.shape[1]
        if cached_len != affix_len:
            raise ValueError(
                f"precomputed_affix_cache length {cached_len} does not match expected affix length {affix_len}.")

    runner = _as_runner(model, mask_id=mask_id, block_length=block_length, gen_length=gen_length,
                        anchor_ratio=anchor_ratio, selection_mode=selection_mode, threshold=threshold,
                        temperature=temperature, remasking=remasking, total_len=total_len, affix_len=affix_len)
    device = runner.device
    seq = Sequence(tokens, block_length=block_length, gen_length=gen_length,
                   cache_block_size=runner.config.cache_block_size, mask_id=mask_id,
                   prompt_affix_start=affix_start, prompt_affix_end=affix_end, generation_start=generation_start)
    nfe = 0
    if affix_len > 0:
        _ensure_affix(runner, seq, precomputed_affix_cache)
    k = min(ceil_to_int(anchor_ratio * affix_len), affix_len)
    seq.enable_acache(affix_len, anchor_ratio, affix_start=affix_start, affix_end=affix_end)
    assert seq.num_anchor_tokens == k
    if dream and k >= affix_len and affix_len > 0:
        anchors = list(range(affix_start, affix_end))   # every affix token is an anchor: nothing to rank
    elif k > 0:
        if selection_mode == "random":
            anchors = (torch.randperm(affix_len, device=device)[:k].sort().values + affix_start).tolist()
        else:
            anchors = runner._compute_anchor_positions(seq)
        nfe += 1
    else:
        anchors = []
    seq.set_anchor_positions(anchors)
    seq.drop_non_anchor = drop_non_anchor
    if not drop_non_anchor:  # nothing of the frozen affix is read in the strict ablation: no relocated copy needed
        runner._reserve_single_sequence_relocation_workspace(seq)
    runner.block_manager.allocate(seq)
    runner._finalize_sequence_layout(seq)

    offsets = torch.arange(block_length, device=device)
    try:
        for nb in range(num_blocks):
            seq.current_block_idx = nb
            s = gen_start + nb * block_length
            block = torch.tensor(seq.token_ids[s:s + block_length], dtype=torch.long, device=device).unsqueeze(0)
            quotas = get_num_transfer_tokens(block == mask_id, steps_per_block)
            # block boundary: recompute anchors + every non-affix token against the frozen affix
            input_ids, positions, block_starts = runner.prepare_caching_acache([seq])
            keep = (block_starts.unsqueeze(1) + offsets).flatten().long()
            if dream:  # logits of the compact position to the left (the first compact row keeps its own)
                keep = (keep - 1).clamp_(min=0)
            logits = runner.model(input_ids, position_ids=positions, logits_keep_indices=keep).logits.unsqueeze(0)
            nfe += 1
            decoding_positions = None
            if dream:
                # commit only the block's first token, then share the quota over the remaining steps
                _, seed = sample_tokens(logits, temperature=temperature)
                block[:, 0] = seed[:, 0]
                quotas = (get_num_transfer_tokens(block == mask_id, steps_per_block - 1)
                          if factor is None and threshold is None and steps_per_block > 1 else None)
            for i in range(1 if dream else 0, steps_per_block):
                if i > 0:
                    if (block == mask_id).sum() == 0:
                        break
                    if decoding_positions is None:
                        decoding_positions = runner.prepare_decoding_acache([seq])
                    logits = runner.model(block, position_ids=decoding_positions).logits
                    if dream:
                        logits = _shift_right(logits)
                    nfe += 1
                if factor is None:
                    quota = None if threshold is not None else quotas[:, i - 1 if dream else i]
                    x0, transfer = get_transfer_index(logits, temperature, remasking, block == mask_id, block, quota,
                                                      threshold)
                else:
                    x0, transfer = get_transfer_index_dynamic(logits, temperature, remasking, block == mask_id, block,
                                                              None, factor)
                block = torch.where(transfer, x0, block)
            seq.token_ids[s:s + block_length] = block[0].tolist()
    finally:
        reset_context()
        runner.block_manager.deallocate(seq)
        if runner._relocated_affix_slot_offset is not None:
            runner.block_manager.release_prefix_tail(runner.shared_prefix_blocks)
            runner._relocated_affix_slot_offset = None
    return torch.tensor([seq.token_ids], dtype=torch.long, device=device), nfe
