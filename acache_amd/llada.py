"""LLaDA-shaped masked-diffusion transformer for the engine path (torch-ROCm GEMMs + HIP attention).

The reference's nano-vdllm model (nano-vdllm/model/modeling_llada.py) cannot be
imported without flash-attn and is outside the hot path; the engine only needs a
model with the same call contract:

    model(input_ids, position_ids=..., logits_keep_indices=None).logits
    model.model.forward(input_ids=..., position_ids=..., compute_logits=False)
    model.device

and the same layer shape as LLaDA-8B: pre-norm blocks with RMSNorm, separate
bias-free q/k/v projections, rotate-half RoPE applied in fp32 at the given
logical positions (modeling_llada.py:412-453), the paged ``Attention`` module, and
a SwiGLU MLP; untied output head.  Inputs are ragged ``[T]`` (cache refresh) or
batched ``[B, L]`` (block refinement), exactly as the runner passes them.
"""
from __future__ import annotations

from dataclasses import dataclass
from types import SimpleNamespace

import torch
from torch import nn
import torch.nn.functional as F

from . import ops
from .attention import Attention
from .utils import get_context
from .rope import rope_table


@dataclass
class LLaDAConfig:
    vocab_size: int = 126464
    d_model: int = 4096
    n_heads: int = 32
    n_kv_heads: int | None = None
    n_layers: int = 32
    mlp_hidden_size: int = 12288
    rope: bool = True
    rope_theta: float = 500000.0
    max_sequence_length: int = 4096
    rms_norm_eps: float = 1e-5
    mask_token_id: int = 126336
    weight_tying: bool = False
    qkv_bias: bool = False  # Dream / Qwen2-style attention projections carry a bias

    @property
    def effective_n_kv_heads(self) -> int:
        return self.n_heads if self.n_kv_heads is None else self.n_kv_heads


class RMSNorm(nn.Module):
    def __init__(self, dim: int, eps: float):
        super().__init__()
        self.weight = nn.Parameter(torch.ones(dim))
        self.eps = eps

    def forward(self, x):
        # statistics in fp32; the normalised value is rounded to the activation type before the weight multiplies
        # it, as in the reference (llada/model/modeling_llada.py:338-350) and in ops.add_rms_norm
        xf = x.float()
        y = (xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + self.eps)).to(x.dtype)
        return self.weight.to(x.dtype) * y


class RotaryEmbedding(nn.Module):
    """fp32 tables ``[max_pos, D]``; ``get_rotary_embedding`` returns ``(sin, cos)`` like the reference (line 372)."""

    def __init__(self, config: LLaDAConfig):
        super().__init__()
        self.config = config
        self.head_dim = config.d_model // config.n_heads
        self._cos = self._sin = None

    def get_rotary_embedding(self, seq_len: int, device):
        if self._cos is None or self._cos.shape[0] < seq_len or self._cos.device != torch.device(device):
            n = max(seq_len, self.config.max_sequence_length)
            self._cos, self._sin = rope_table(n, self.head_dim, self.config.rope_theta, device=device)
        return self._sin[:seq_len], self._cos[:seq_len]

    def forward(self, q, k, position_ids, max_pos=None):
        max_pos = max_pos or self.config.max_sequence_length
        sin, cos = self.get_rotary_embedding(max_pos, q.device)
        s = sin[position_ids].unsqueeze(-2)
        c = cos[position_ids].unsqueeze(-2)

        def rot(x):
            xf = x.float()
            h = xf.shape[-1] // 2
            return (xf * c + torch.cat((-xf[..., h:], xf[..., :h]), -1) * s).type_as(x)

        return rot(q), rot(k)


class LLaDABlock(nn.Module):
    def __init__(self, config: LLaDAConfig):
        super().__init__()
        self.config = config
        d, h, hkv = config.d_model, config.n_heads, config.effective_n_kv_heads
        self.head_dim = d // h
        self.attn_norm = RMSNorm(d, config.rms_norm_eps)
        self.ff_norm = RMSNorm(d, config.rms_norm_eps)
        self.q_proj = nn.Linear(d, h * self.head_dim, bias=config.qkv_bias)
        self.k_proj = nn.Linear(d, hkv * self.head_dim, bias=config.qkv_bias)
        self.v_proj = nn.Linear(d, hkv * self.head_dim, bias=config.qkv_bias)
        self.attn_out = nn.Linear(h * self.head_dim, d, bias=False)
        self.ff_proj = nn.Linear(d, config.mlp_hidden_size, bias=False)
        self.up_proj = nn.Linear(d, config.mlp_hidden_size, bias=False)
        self.ff_out = nn.Linear(config.mlp_hidden_size, d, bias=False)
        self.rotary_emb = RotaryEmbedding(config)
        self.attn = Attention(h, self.head_dim, hkv)
        self._fused = {}

    def _fuse(self, name, linears):
        """One weight (and bias) for several projections of the same input: the parameters of ``linears`` become
        views of one concatenated tensor, so the state dict keeps the reference's names and shapes while the
        forward runs a single, wider GEMM.  Rebuilt when the parameters have been moved or replaced."""
        first = linears[0].weight
        cached = self._fused.get(name)
        if cached is None or cached[0].data_ptr() != first.data_ptr() or cached[0].dtype != first.dtype:
            with torch.no_grad():
                w = torch.cat([lin.weight for lin in linears]).contiguous()
                b = torch.cat([lin.bias for lin in linears]).contiguous() if linears[0].bias is not None else None
                row = 0
                for lin in linears:
                    n = lin.weight.shape[0]
                    lin.weight.data = w[row:row + n]
                    if b is not None:
                        lin.bias.data = b[row:row + n]
                    row += n
            cached = self._fused[name] = (w, b)
        return cached

    def fuse_projections(self):
        """Build the merged q/k/v and gate/up weights now rather than on the first forward, so that whoever sizes
        the KV cache from free device memory afterwards already sees them."""
        self._fuse("qkv", (self.q_proj, self.k_proj, self.v_proj))
        self._fuse("gate_up", (self.ff_proj, self.up_proj))

    @staticmethod
    def _hooked(*linears):
        # a projection somebody observes (forward hooks) keeps its own forward call
        return any(lin._forward_hooks or lin._forward_pre_hooks for lin in linears)

    def fusable(self, x) -> bool:
        """The merged-launch form of the block applies: GPU inference with nobody observing the sub-modules."""
        return (x.is_cuda and not torch.is_grad_enabled() and self.config.rope and not self._forward_hooks
                and not self._forward_pre_hooks
                and not self._hooked(self.attn_norm, self.ff_norm, self.q_proj, self.k_proj, self.v_proj,
                                     self.attn_out, self.ff_proj, self.up_proj, self.ff_out))

    def forward(self, x, position_ids, max_pos, pending=None, defer_residual=False):
        """``pending``: a residual term the previous block left un-added; it is folded into this block's first
        layer norm.  ``defer_residual``: return ``(x, mlp_out)`` instead of their sum, for the next block (or the
        final norm) to fold in the same way.  Both only with ``fusable(x)``; the plain call is the reference's."""
        h, hkv, hd = self.config.n_heads, self.config.effective_n_kv_heads, self.head_dim
        if pending is not None or defer_residual:
            x, y = ops.add_rms_norm(x, pending, self.attn_norm.weight, self.attn_norm.eps)
        else:
            y = self.attn_norm(x)
        lead = y.shape[:-1]
        if y.is_cuda and not torch.is_grad_enabled() and not self._hooked(self.q_proj, self.k_proj, self.v_proj):
            # q, k and v are column views of one projection (the kernels take token strides)
            qkv = F.linear(y, *self._fuse("qkv", (self.q_proj, self.k_proj, self.v_proj)))
            q = qkv[..., :h * hd].view(*lead, h, hd)
            k = qkv[..., h * hd:(h + hkv) * hd].view(*lead, hkv, hd)
            v = qkv[..., (h + hkv) * hd:].view(*lead, hkv, hd)
        else:
            q = self.q_proj(y).view(*lead, h, hd)
            k = self.k_proj(y).view(*lead, hkv, hd)
            v = self.v_proj(y).view(*lead, hkv, hd)
        if self.config.rope and q.is_cuda:
            # rotary application and the K/V cache write in one launch (q and k are rotated in place)
            sin, cos = self.rotary_emb.get_rotary_embedding(max_pos or self.config.max_sequence_length, q.device)
            ops.rope_qk_scatter(q.view(-1, h, hd), k.view(-1, hkv, hd), v.view(-1, hkv, hd),
                                position_ids.reshape(-1).contiguous(), cos, sin,
                                self.attn.k_cache, self.attn.v_cache, get_context().slot_mapping)
            o = self.attn(q, k, v, kv_stored=True)
        else:
            if self.config.rope:
                q, k = self.rotary_emb(q, k, position_ids, max_pos)
            o = self.attn(q, k, v)
        attn = self.attn_out(o.reshape(*lead, h * hd))
        fused = x.is_cuda and not torch.is_grad_enabled() and not self._hooked(self.ff_norm, self.ff_proj, self.up_proj)
        if fused:
            # residual add and layer norm in one pass over the row, then gate and up as one GEMM and SwiGLU in
            # one pass
            x, y = ops.add_rms_norm(x, attn, self.ff_norm.weight, self.ff_norm.eps)
            gu = F.linear(y, *self._fuse("gate_up", (self.ff_proj, self.up_proj)))
            mlp = self.ff_out(ops.swiglu(gu, self.config.mlp_hidden_size))
            return (x, mlp) if defer_residual else x + mlp
        x = x + attn
        y = self.ff_norm(x)
        return x + self.ff_out(F.silu(self.ff_proj(y)) * self.up_proj(y))


class LLaDAModel(nn.Module):
    def __init__(self, config: LLaDAConfig):
        super().__init__()
        self.config = config
        self.transformer = nn.ModuleDict(dict(
            wte=nn.Embedding(config.vocab_size, config.d_model),
            blocks=nn.ModuleList([LLaDABlock(config) for _ in range(config.n_layers)]),
            ln_f=RMSNorm(config.d_model, config.rms_norm_eps),
            ff_out=nn.Linear(config.d_model, config.vocab_size, bias=False),
        ))

    def forward(self, input_ids, position_ids=None, compute_logits=True, logits_keep_indices=None):
        if position_ids is None:
            position_ids = torch.arange(input_ids.shape[-1], device=input_ids.device).expand_as(input_ids)
        # rows of the rotary table: the configured length, or more when the runner serves a longer request
        max_pos = max(self.config.max_sequence_length, int(getattr(self, "rope_positions", 0)))
        x = self.transformer["wte"](input_ids)
        blocks = self.transformer["blocks"]
        ln_f = self.transformer["ln_f"]
        if len(blocks) and all(block.fusable(x) for block in blocks) and not ln_f._forward_hooks:
            # every residual add rides along with the layer norm that follows it
            pending = None
            for block in blocks:
                x, pending = block(x, position_ids, max_pos, pending=pending, defer_residual=True)
            if not compute_logits:
                return SimpleNamespace(logits=None, hidden_states=x + pending)
            _, x = ops.add_rms_norm(x, pending, ln_f.weight, ln_f.eps)
        else:
            for block in blocks:
                x = block(x, position_ids, max_pos)
            if not compute_logits:
                return SimpleNamespace(logits=None, hidden_states=x)
            x = ln_f(x)
        if logits_keep_indices is not None:  # logits of the listed ragged rows only
            x = x.reshape(-1, x.shape[-1]).index_select(0, logits_keep_indices)
        return SimpleNamespace(logits=self.transformer["ff_out"](x))


class LLaDAModelLM(nn.Module):
    """Outer wrapper with the attribute layout the runner walks (``.model.transformer.blocks``)."""

    def __init__(self, config: LLaDAConfig, init_std: float = 0.02):
        super().__init__()
        self.config = config
        self.model = LLaDAModel(config)
        for name, p in self.named_parameters():
            if p.dim() > 1 or name.endswith("_proj.bias"):  # norm weights stay at one
                nn.init.normal_(p, mean=0.0, std=init_std)

    @property
    def device(self):
        return next(self.parameters()).device

    def forward(self, input_ids, position_ids=None, logits_keep_indices=None, compute_logits=True):
        return self.model(input_ids, position_ids=position_ids, compute_logits=compute_logits,
                          logits_keep_indices=logits_keep_indices)


# ---------------------------------------------------------------------------------------------------
# Taking over a checkpoint model object
#
# The HF path of the reference hands its entry points the checkpoint's own model class
# (llada/eval_ACache.py:100-107 loads llada/model/modeling_llada.py:LLaDAModelLM in bf16 and passes it to
# generate_with_anchor_attention, :189).  That class attends over dense [B, H, L, D] caches inside its own
# forward and cannot run on the paged engine, but its parameters can: this module's blocks use the same
# parameter names, so the engine model is built around the checkpoint's tensors (adopt_state says which of them
# end up copied).

def _plain(value):
    """Configuration enums of the checkpoint (StrEnum members) and plain strings compare alike."""
    value = getattr(value, "value", value)
    return value.lower() if isinstance(value, str) else value


def config_from_checkpoint(cfg) -> LLaDAConfig:
    """The engine's configuration for a checkpoint configuration (llada/model/configuration_llada.py:154-381).
    Raises ``TypeError`` naming every setting this decoder stack does not implement."""
    needed = ("d_model", "n_heads", "n_layers", "vocab_size")
    if any(not hasattr(cfg, name) for name in needed):
        raise TypeError(f"not a LLaDA checkpoint configuration: {type(cfg).__name__} lacks one of {needed}")
    get = lambda name, default=None: getattr(cfg, name, default)
    wanted = {
        "rope": True, "alibi": False, "block_type": "llama", "layer_norm_type": "rms", "activation_type": "silu",
        "include_bias": False, "attention_layer_norm": False, "input_emb_norm": False, "scale_logits": False,
        "layer_norm_with_affine": True,
    }
    problems = [f"{name}={_plain(get(name))!r} (supported: {value!r})" for name, value in wanted.items()
                if hasattr(cfg, name) and _plain(get(name)) != value]
    if get("block_group_size", 1) not in (None, 1):
        problems.append(f"block_group_size={get('block_group_size')} (supported: 1)")
    if problems:
        raise TypeError("this engine's LLaDA decoder stack does not implement: " + ", ".join(problems))
    n_heads = int(cfg.n_heads)
    if get("n_kv_heads") is not None:
        n_kv = int(cfg.n_kv_heads)
    else:
        n_kv = 1 if get("multi_query_attention") is True else n_heads
    hidden = get("mlp_hidden_size")
    if hidden is None:
        hidden = int(get("mlp_ratio", 4)) * int(cfg.d_model)
    mask_id = get("mask_token_id")
    return LLaDAConfig(
        vocab_size=int(get("embedding_size") or cfg.vocab_size), d_model=int(cfg.d_model), n_heads=n_heads,
        n_kv_heads=n_kv, n_layers=int(cfg.n_layers), mlp_hidden_size=int(hidden), rope=True,
        rope_theta=float(get("rope_theta", 10000.0)), max_sequence_length=int(get("max_sequence_length", 1024)),
        rms_norm_eps=float(get("rms_norm_eps", 1e-5)),
        mask_token_id=int(mask_id) if mask_id is not None else LLaDAConfig.mask_token_id,
        weight_tying=bool(get("weight_tying", False)), qkv_bias=bool(get("include_qkv_bias", False)))


def _engine_dtype(state):
    """Parameters as the engine takes them: its paged cache is bf16 (as the reference's, model_runner.py:206-208), so
    bf16 tensors are used as they are (no copy) and any other floating type is converted to bf16."""
    return {name: t if t.dtype == torch.bfloat16 or not t.is_floating_point() else t.to(torch.bfloat16)
            for name, t in state.items()}


def adopt_state(engine_cls, config: LLaDAConfig, state: dict):
    """An ``engine_cls`` model built around the tensors of ``state``.  Embedding, norms, output projections, the
    MLP down projection and the head ARE those tensors.  The q/k/v and gate/up projections are merged into one
    weight each (built here, on a GPU, so that a KV cache sized afterwards accounts for them): new tensors of the
    same total size, so while the caller keeps the checkpoint object these projections (about three quarters of
    a decoder block, 9.6 GB of LLaDA-8B's 16 GB in bf16) are resident twice.  Floating-point parameters that are
    not bf16 are converted, which copies them as well."""
    with torch.device("meta"):
        engine = engine_cls(config)
    state = _engine_dtype(state)
    tied = config.weight_tying and "model.transformer.ff_out.weight" not in state
    if tied:  # the checkpoint scores against the embedding matrix (modeling_llada.py: F.linear(x, wte.weight))
        state = dict(state)
        state["model.transformer.ff_out.weight"] = state["model.transformer.wte.weight"]
    engine.load_state_dict(state, strict=True, assign=True)
    for p in engine.parameters():
        p.requires_grad_(False)
    if next(engine.parameters()).is_cuda:
        with torch.no_grad():
            for block in engine.model.transformer["blocks"]:
                block.fuse_projections()
    return engine.eval()


def engine_model_from_checkpoint(model) -> "LLaDAModelLM":
    """The engine model for a checkpoint-style LLaDA model object: same configuration, the same parameter tensors.
    ``model`` needs ``.config`` and ``.state_dict()`` with the checkpoint's names (``model.transformer.blocks.N.*``)."""
    config = config_from_checkpoint(model.config)
    state = model.state_dict()
    if not any(name.startswith("model.transformer.blocks.") for name in state):
        raise TypeError(f"{type(model).__name__}: no 'model.transformer.blocks.*' parameters in its state dict")
    try:
        return adopt_state(LLaDAModelLM, config, state)
    except RuntimeError as e:  # load_state_dict lists missing / unexpected / mis-shaped entries
        raise TypeError(f"{type(model).__name__}: its parameters do not fit the engine's LLaDA model: {e}") from e
