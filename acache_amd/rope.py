"""RoPE tables in the layout the relocation kernels consume.

``cos, sin`` are fp32 ``[length, head_dim]`` with the ``cat(freqs, freqs)``
layout, built exactly as the reference model builds them
(nano-vdllm/model/modeling_llada.py:392-398; Dream: modeling_dream.py:164-170):
``inv_freq = 1 / theta**(arange(0, D, 2)/D)`` and the outer product with the
positions are evaluated in fp32 before cos/sin.
"""
from __future__ import annotations

import torch


def rope_table(length: int, head_dim: int, theta: float, device=None):
    exponents = torch.arange(0, head_dim, 2, dtype=torch.float32, device=device) / head_dim
    inv_freq = 1.0 / (theta ** exponents)
    positions = torch.arange(length, dtype=torch.float32, device=device)
    freqs = torch.outer(positions, inv_freq)
    emb = torch.cat((freqs, freqs), dim=-1)
    return emb.cos(), emb.sin()
