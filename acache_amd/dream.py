"""Dream-shaped engine model: the same decoder stack as ``acache_amd.llada`` with grouped-query attention and
biased q/k/v projections (Dream-v0-Instruct-7B is a Qwen2.5-7B-shaped masked-diffusion model:
28 query heads, 4 KV heads, head_dim 128, rope theta 1e6; nano-vdllm/model/modeling_dream.py:157-199 for the
rotary tables and the attention layout).  Token ``i`` is predicted from the hidden state of position ``i - 1``;
that shift is applied by the generation loop (``acache_amd.generate_acache_dream``), not by the model.
"""
from __future__ import annotations

from dataclasses import dataclass

from .llada import LLaDAConfig, LLaDAModelLM


@dataclass
class DreamConfig(LLaDAConfig):
    vocab_size: int = 152064
    d_model: int = 3584
    n_heads: int = 28
    n_kv_heads: int | None = 4
    n_layers: int = 28
    mlp_hidden_size: int = 18944
    rope_theta: float = 1000000.0
    max_sequence_length: int = 4096
    rms_norm_eps: float = 1e-6
    mask_token_id: int = 151666
    qkv_bias: bool = True


class DreamModelLM(LLaDAModelLM):
    """Random-init Dream-shaped model with the call contract the runner expects."""

    def __init__(self, config: DreamConfig, init_std: float = 0.02):
        super().__init__(config, init_std=init_std)
