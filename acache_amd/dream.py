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


# ---------------------------------------------------------------------------------------------------
# Taking over a checkpoint model object (dream/eval_ACache.py hands dream/model/modeling_dream.py:DreamModel to
# dream/generate_ACache.py).  The checkpoint's decoder layers are Qwen2-shaped; their parameters map one to one
# onto this package's block:
#   model.embed_tokens -> wte            model.layers.N.input_layernorm          -> blocks.N.attn_norm
#   model.norm         -> ln_f           model.layers.N.post_attention_layernorm -> blocks.N.ff_norm
#   lm_head            -> ff_out         model.layers.N.self_attn.{q,k,v}_proj   -> blocks.N.{q,k,v}_proj
#   model.layers.N.self_attn.o_proj -> blocks.N.attn_out
#   model.layers.N.mlp.{gate,up,down}_proj -> blocks.N.{ff_proj,up_proj,ff_out}   (modeling_dream.py:286-343, 624-629, 793-799, 945)
_LAYER_NAMES = {
    "input_layernorm": "attn_norm", "post_attention_layernorm": "ff_norm",
    "self_attn.q_proj": "q_proj", "self_attn.k_proj": "k_proj", "self_attn.v_proj": "v_proj",
    "self_attn.o_proj": "attn_out", "mlp.gate_proj": "ff_proj", "mlp.up_proj": "up_proj", "mlp.down_proj": "ff_out",
}
_TOP_NAMES = {"model.embed_tokens": "wte", "model.norm": "ln_f", "lm_head": "ff_out"}


def config_from_checkpoint(cfg) -> DreamConfig:
    """The engine's configuration for a checkpoint configuration (dream/model/configuration_dream.py:31-97)."""
    needed = ("hidden_size", "num_attention_heads", "num_hidden_layers", "intermediate_size", "vocab_size")
    if any(not hasattr(cfg, name) for name in needed):
        raise TypeError(f"not a Dream checkpoint configuration: {type(cfg).__name__} lacks one of {needed}")
    get = lambda name, default=None: getattr(cfg, name, default)
    problems = []
    scaling = get("rope_scaling")
    if scaling and (scaling.get("rope_type", scaling.get("type", "default")) != "default"):
        problems.append(f"rope_scaling={scaling!r} (supported: none)")
    if get("use_sliding_window", False):
        problems.append("use_sliding_window=True (supported: False)")
    if str(get("hidden_act", "silu")).lower() != "silu":
        problems.append(f"hidden_act={get('hidden_act')!r} (supported: 'silu')")
    if problems:
        raise TypeError("this engine's Dream decoder stack does not implement: " + ", ".join(problems))
    mask_id = get("mask_token_id")
    return DreamConfig(
        vocab_size=int(cfg.vocab_size), d_model=int(cfg.hidden_size), n_heads=int(cfg.num_attention_heads),
        n_kv_heads=int(get("num_key_value_heads") or cfg.num_attention_heads), n_layers=int(cfg.num_hidden_layers),
        mlp_hidden_size=int(cfg.intermediate_size), rope_theta=float(get("rope_theta", 10000.0)),
        max_sequence_length=int(get("max_position_embeddings", 4096)), rms_norm_eps=float(get("rms_norm_eps", 1e-6)),
        mask_token_id=int(mask_id) if mask_id is not None else DreamConfig.mask_token_id,
        weight_tying=bool(get("tie_word_embeddings", False)), qkv_bias=True)


def _engine_name(name: str):
    """Checkpoint parameter name -> this package's name; ``None`` for entries the engine has no use for."""
    for top, ours in _TOP_NAMES.items():
        if name.startswith(top + "."):
            return f"model.transformer.{ours}.{name[len(top) + 1:]}"
    if name.startswith("model.layers."):
        index, _, rest = name[len("model.layers."):].partition(".")
        module, _, leaf = rest.rpartition(".")
        if module in _LAYER_NAMES:
            return f"model.transformer.blocks.{index}.{_LAYER_NAMES[module]}.{leaf}"
    return None


def engine_model_from_checkpoint(model) -> "DreamModelLM":
    """The engine model for a checkpoint-style Dream model object: same configuration, the same parameter tensors
    under this package's names.  Buffers of the checkpoint's rotary modules (``inv_freq``) are not parameters and
    are dropped; the engine builds its tables from ``rope_theta``."""
    from .llada import adopt_state

    config = config_from_checkpoint(model.config)
    state = {}
    for name, tensor in model.state_dict().items():
        ours = _engine_name(name)
        if ours is not None:
            state[ours] = tensor
        elif not name.endswith("inv_freq"):
            raise TypeError(f"{type(model).__name__}: parameter {name!r} has no place in the engine's Dream model")
    if not any(name.startswith("model.transformer.blocks.") for name in state):
        raise TypeError(f"{type(model).__name__}: no 'model.layers.*' parameters in its state dict")
    try:
        return adopt_state(DreamModelLM, config, state)
    except RuntimeError as e:
        raise TypeError(f"{type(model).__name__}: its parameters do not fit the engine's Dream model: {e}") from e
