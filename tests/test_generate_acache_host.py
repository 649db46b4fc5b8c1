"""Host-side rules of the HF-signature entry points (no GPU): token transfer and argument handling.

Expected values are worked out by hand from the rule in llada/generate.py:379-420 (dynamic threshold)
and llada/generate.py:298-376 (threshold / quota), not by re-running the formula.
"""
import math

import pytest
import torch

from acache_amd.generate_acache import (_coerce_bool, ceil_to_int, get_num_transfer_tokens, get_transfer_index,
                                        get_transfer_index_dynamic)

V = 16
MASK = 99


def _logits(confidences, winners):
    """Rows whose softmax puts `confidence` on `winner` and spreads the rest evenly (so argmax = winner)."""
    rows = []
    for c, w in zip(confidences, winners):
        p = torch.full((V,), (1.0 - c) / (V - 1), dtype=torch.float64)
        p[w] = c
        rows.append(p.log())
    return torch.stack(rows).unsqueeze(0).float()


def _run_dynamic(confidences, masked, factor=1.0):
    n = len(confidences)
    winners = [(3 * i + 1) % V for i in range(n)]
    x = torch.tensor([[MASK if m else 7 for m in masked]])
    mask_index = x == MASK
    x0, transfer = get_transfer_index_dynamic(_logits(confidences, winners), 0.0, "low_confidence", mask_index, x, None, factor)
    for i in range(n):  # argmax where masked, the old token elsewhere
        assert x0[0, i].item() == (winners[i] if masked[i] else 7)
    return transfer[0].tolist()


def test_dynamic_threshold_stops_at_first_failure():
    # thresholds for factor 1: -, 2/3, 3/4, 4/5 ; sorted confidences .99 .9 .5 .4 -> third fails -> 2 tokens
    assert _run_dynamic([0.5, 0.99, 0.4, 0.9], [True] * 4) == [False, True, False, True]


def test_dynamic_threshold_failure_at_last_position_commits_everything():
    # sorted .99 .9 .8 .1: only the last fails; the reference's index bump then commits all four
    assert _run_dynamic([0.1, 0.99, 0.8, 0.9], [True] * 4) == [True] * 4
    # n = 2: sorted .9 .1, the second fails at the last index -> both
    assert _run_dynamic([0.9, 0.1], [True, True]) == [True, True]


def test_dynamic_threshold_all_pass_and_single_and_none():
    assert _run_dynamic([0.85, 0.99, 0.8, 0.9], [True] * 4) == [True] * 4      # .8 >= 4/5 exactly passes
    assert _run_dynamic([0.3, 0.5, 0.4, 0.2], [True] * 4) == [False, True, False, False]  # second (.4 < 2/3) fails
    assert _run_dynamic([0.3], [True]) == [True]                                  # one masked token always goes
    assert _run_dynamic([0.9, 0.9], [False, False]) == [False, False]              # nothing masked
    # unmasked positions never transfer and do not count towards n
    assert _run_dynamic([0.99, 0.5, 0.95, 0.4], [False, True, True, True]) == [False, False, True, False]


def test_dynamic_threshold_factor_scales_thresholds():
    # factor 0.5: thresholds -, 1-.5/3=.833, 1-.5/4=.875 ; sorted .99 .85 .5 -> second passes, third fails at last -> all
    assert _run_dynamic([0.99, 0.85, 0.5], [True] * 3, factor=0.5) == [True, True, True]
    # sorted .99 .8 .5 .4 with factor .5: second (.8 < .833) fails -> 1 token
    assert _run_dynamic([0.99, 0.8, 0.5, 0.4], [True] * 4, factor=0.5) == [True, False, False, False]


def test_threshold_mode_forces_best_token():
    x = torch.tensor([[MASK, MASK, 5]])
    logits = _logits([0.6, 0.7, 0.99], [1, 2, 3])
    x0, transfer = get_transfer_index(logits, 0.0, "low_confidence", x == MASK, x, None, threshold=0.9)
    assert transfer[0].tolist() == [False, True, False]      # nothing reaches 0.9: the most confident masked token goes
    assert x0[0].tolist() == [1, 2, 5]
    x0, transfer = get_transfer_index(logits, 0.0, "low_confidence", x == MASK, x, None, threshold=0.65)
    assert transfer[0].tolist() == [False, True, False]
    x0, transfer = get_transfer_index(logits, 0.0, "low_confidence", x == MASK, x, None, threshold=0.5)
    assert transfer[0].tolist() == [True, True, False]


def test_quota_mode_and_transfer_schedule():
    x = torch.tensor([[MASK, MASK, MASK, 5]])
    logits = _logits([0.6, 0.8, 0.7, 0.99], [1, 2, 3, 4])
    _, transfer = get_transfer_index(logits, 0.0, "low_confidence", x == MASK, x, torch.tensor([2]), None)
    assert transfer[0].tolist() == [False, True, True, False]
    with pytest.raises(ValueError):
        get_transfer_index(logits, 0.0, "low_confidence", x == MASK, x, None, None)
    # 7 masked tokens over 3 steps: 3, 2, 2
    sched = get_num_transfer_tokens(torch.tensor([[True] * 7 + [False]]), 3)
    assert sched.tolist() == [[3, 2, 2]]


def test_coerce_bool_and_ceil():
    assert _coerce_bool(None, True, "x") is True and _coerce_bool(None, False, "x") is False
    assert _coerce_bool("Yes", False, "x") is True and _coerce_bool(" off ", True, "x") is False
    assert _coerce_bool(0, True, "x") is False and _coerce_bool(2.5, False, "x") is True
    with pytest.raises(ValueError):
        _coerce_bool("maybe", False, "x")
    assert ceil_to_int(3.0) == 3 and ceil_to_int(3.0000001) == 4 and ceil_to_int(0.07 * 100) == math.ceil(0.07 * 100) == 8


def _llada_checkpoint_config(**changes):
    """The fields of llada/model/configuration_llada.py the fixture's model was built with
    (tests/golden/make_hf_path_vectors.py), as a plain namespace."""
    from types import SimpleNamespace

    fields = dict(d_model=256, n_heads=2, n_layers=2, mlp_hidden_size=128, vocab_size=64, embedding_size=64,
                  mask_token_id=63, eos_token_id=0, pad_token_id=0, rope=True, rope_theta=10000.0, alibi=False,
                  block_type="llama", activation_type="silu", layer_norm_type="rms", rms_norm_eps=1e-5,
                  include_bias=False, include_qkv_bias=False, weight_tying=False, input_emb_norm=False,
                  flash_attention=False, max_sequence_length=256, scale_logits=False, n_kv_heads=None,
                  multi_query_attention=None, mlp_ratio=4)
    fields.update(changes)
    return SimpleNamespace(**fields)


class CheckpointModelDouble:
    """Stands where the checkpoint's model object stands in the reference's call (llada/eval_ACache.py:189): a
    class of another package with ``.config`` and ``.state_dict()`` under the checkpoint's parameter names."""

    def __init__(self, config, state):
        self.config, self._state = config, state

    def state_dict(self):
        return self._state


def _fixture_weights():
    from pathlib import Path

    return torch.load(Path(__file__).resolve().parent / "golden" / "hf_path_vectors.pt", weights_only=True)["weights"]


def test_objects_that_are_no_checkpoint_model_are_rejected_with_a_type_error():
    from acache_amd.generate_acache import generate_with_anchor_attention

    class Foreign(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.model = torch.nn.Linear(4, 4)
            self.config = object()

    prompt = torch.arange(2, 10).unsqueeze(0)
    args = dict(steps=4, gen_length=4, block_length=4, mask_id=MASK, affix_start=0, affix_end=4)
    with pytest.raises(TypeError, match="neither a LLaDA nor a Dream configuration"):
        generate_with_anchor_attention(Foreign(), prompt, **args)
    with pytest.raises(TypeError, match="checkpoint model object"):
        generate_with_anchor_attention(object(), prompt, **args)
    # a LLaDA configuration with settings this decoder stack lacks: every one of them is named
    odd = CheckpointModelDouble(_llada_checkpoint_config(alibi=True, block_type="sequential"), _fixture_weights())
    with pytest.raises(TypeError, match=r"alibi=True.*block_type='sequential'"):
        generate_with_anchor_attention(odd, prompt, **args)
    # parameters that do not fit the configuration
    short = CheckpointModelDouble(_llada_checkpoint_config(n_layers=3), _fixture_weights())
    with pytest.raises(TypeError, match="do not fit"):
        generate_with_anchor_attention(short, prompt, **args)


def test_checkpoint_model_is_adopted_without_copying_its_weights():
    """The reference's own parameter names (the fixture holds the state dict of llada/model/modeling_llada.py's
    LLaDAModelLM) load as they are, and the engine model's parameters are those very tensors."""
    from acache_amd.checkpoint import engine_model_for as _engine_model
    from acache_amd.llada import LLaDAModelLM

    weights = _fixture_weights()
    checkpoint_model = CheckpointModelDouble(_llada_checkpoint_config(), weights)
    engine = _engine_model(checkpoint_model)
    assert isinstance(engine, LLaDAModelLM) and not engine.training
    cfg = engine.config
    assert (cfg.d_model, cfg.n_heads, cfg.effective_n_kv_heads, cfg.n_layers, cfg.mlp_hidden_size) == (256, 2, 2, 2, 128)
    assert (cfg.vocab_size, cfg.mask_token_id, cfg.rope_theta, cfg.max_sequence_length) == (64, 63, 10000.0, 256)
    state = engine.state_dict()
    assert set(state) == set(weights)
    assert all(state[name].data_ptr() == weights[name].data_ptr() for name in weights)
    assert not any(p.requires_grad for p in engine.parameters())
    assert _engine_model(checkpoint_model) is engine          # built once per checkpoint object
    assert _engine_model(engine) is engine                    # an engine model passes through
    # fp32 weights are converted for the kernels (bf16), tied embeddings score against the embedding matrix
    tied = {k: v.float() for k, v in weights.items() if k != "model.transformer.ff_out.weight"}
    engine32 = _engine_model(CheckpointModelDouble(_llada_checkpoint_config(weight_tying=True), tied))
    assert all(p.dtype == torch.bfloat16 for p in engine32.parameters())
    head, wte = engine32.model.transformer["ff_out"].weight, engine32.model.transformer["wte"].weight
    assert head.data_ptr() == wte.data_ptr()


def test_dream_checkpoint_names_map_onto_the_engine_model():
    """dream/model/modeling_dream.py's parameter names (read from its module definitions, :286-343, 624-629,
    793-799, 945; that model does not construct in this environment, so no state dict of it is on file)."""
    from types import SimpleNamespace

    from acache_amd import dream

    cfg = dream.DreamConfig(vocab_size=64, d_model=256, n_heads=4, n_kv_heads=2, n_layers=2, mlp_hidden_size=128,
                            max_sequence_length=128, mask_token_id=63)
    ours = dream.DreamModelLM(cfg).to(torch.bfloat16)
    theirs = {}
    for i in range(2):
        b = f"model.transformer.blocks.{i}."
        sd = ours.state_dict()
        for proj in "qkv":
            theirs[f"model.layers.{i}.self_attn.{proj}_proj.weight"] = sd[b + f"{proj}_proj.weight"]
            theirs[f"model.layers.{i}.self_attn.{proj}_proj.bias"] = sd[b + f"{proj}_proj.bias"]
        theirs[f"model.layers.{i}.self_attn.o_proj.weight"] = sd[b + "attn_out.weight"]
        theirs[f"model.layers.{i}.mlp.gate_proj.weight"] = sd[b + "ff_proj.weight"]
        theirs[f"model.layers.{i}.mlp.up_proj.weight"] = sd[b + "up_proj.weight"]
        theirs[f"model.layers.{i}.mlp.down_proj.weight"] = sd[b + "ff_out.weight"]
        theirs[f"model.layers.{i}.input_layernorm.weight"] = sd[b + "attn_norm.weight"]
        theirs[f"model.layers.{i}.post_attention_layernorm.weight"] = sd[b + "ff_norm.weight"]
    theirs["model.embed_tokens.weight"] = sd["model.transformer.wte.weight"]
    theirs["model.norm.weight"] = sd["model.transformer.ln_f.weight"]
    theirs["lm_head.weight"] = sd["model.transformer.ff_out.weight"]
    theirs["model.rotary_emb.inv_freq"] = torch.zeros(64)           # a buffer the engine does not take
    hf_cfg = SimpleNamespace(vocab_size=64, hidden_size=256, intermediate_size=128, num_hidden_layers=2,
                             num_attention_heads=4, num_key_value_heads=2, hidden_act="silu",
                             max_position_embeddings=128, rms_norm_eps=1e-6, rope_theta=1e6, rope_scaling=None,
                             use_sliding_window=False, mask_token_id=63, tie_word_embeddings=False)
    engine = dream.engine_model_from_checkpoint(CheckpointModelDouble(hf_cfg, theirs))
    assert isinstance(engine, dream.DreamModelLM) and engine.config.qkv_bias and engine.config.effective_n_kv_heads == 2
    got = engine.state_dict()
    assert set(got) == set(sd) and all(torch.equal(got[k], sd[k]) for k in sd)
    hf_cfg.rope_scaling = {"rope_type": "yarn", "factor": 4.0}
    with pytest.raises(TypeError, match="rope_scaling"):
        dream.engine_model_from_checkpoint(CheckpointModelDouble(hf_cfg, theirs))
    hf_cfg.rope_scaling = None
    theirs["model.layers.0.self_attn.q_norm.weight"] = torch.zeros(4)
    with pytest.raises(TypeError, match="has no place"):
        dream.engine_model_from_checkpoint(CheckpointModelDouble(hf_cfg, theirs))
