"""Engine flags.  Field names and defaults follow nano-vdllm/config.py:5-29.

``hf_config`` is any object exposing the model shape (``n_heads`` /
``num_attention_heads``, ``n_kv_heads`` / ``num_key_value_heads``, ``d_model`` /
``hidden_size``, ``n_layers`` / ``num_hidden_layers``, ``vocab_size``,
``rope_theta``); no transformers dependency is needed.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any


@dataclass
class Config:
    hf_config: Any = None
    mask_id: int = 126336
    recompute_batch_size: int = 4
    max_num_seqs: int = 0
    gen_length: int = 1024
    block_length: int = 1024
    remasking: str = "low_confidence"  # 'low_confidence', 'random', 'none'
    threshold: float = 0.9
    cache_block_size: int = 256
    max_num_batched_tokens: int = 16384
    gpu_memory_utilization: float = 0.9
    num_kvcache_blocks: int = -1
    temperature: float = 0.0
    enable_acache: bool = False
    enable_dkv_cache: bool = False
    dkv_steps: int = 0
    dkv_cache_interval: int = 8
    anchor_ratio: float = 0.05
    selection_mode: str = "top"
    use_reference_attention: bool = False
    acache_memory_reserve_gb: float = 4.0
    profile_timing: bool = False
    model_type: str = "llada"
    # not in the reference: replay the block-refinement forward from a captured HIP graph (same kernels, same
    # results, no per-launch host cost); re-captured whenever the attention metadata of the step changes
    decode_hip_graph: bool = False
    # not in the reference (which probes one request per forward, model_runner.py:873): requests per
    # anchor-selection probe forward; 0 = all newly admitted requests at once.  Selection is the same either way
    # (the importance kernels are deterministic and requests do not interact).
    anchor_selection_batch_size: int = 1
