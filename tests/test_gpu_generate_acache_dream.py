"""Dream-shaped batch-1 entry point (dream/generate_ACache.py) on the paged engine: GQA model with biased
q/k/v projections, left-shifted logits, first-token seeding."""
import pytest
import torch

from acache_amd import generate_acache_dream as GD
from acache_amd.dream import DreamConfig, DreamModelLM

pytestmark = pytest.mark.gpu
MASK = 63


def _model(device, seed=0):
    torch.manual_seed(seed)
    cfg = DreamConfig(vocab_size=64, d_model=256, n_heads=4, n_kv_heads=2, n_layers=2, mlp_hidden_size=128,
                      max_sequence_length=128, mask_token_id=MASK, rope_theta=10000.0)
    model = DreamModelLM(cfg, init_std=0.08).to(device=device, dtype=torch.bfloat16).eval()
    with torch.no_grad():
        # these loops run a fixed number of steps (no spin is possible); a 64-token random head that answers [MASK]
        # would only leave a hole in the window, which the fill assertions below would then report as a failure
        model.model.transformer["ff_out"].weight[MASK].zero_()
    assert model.model.transformer["blocks"][0].q_proj.bias is not None
    return cfg, model


def _dense_logits(model, tokens, device):
    """Plain full-sequence forward of the same weights through the engine's attention (no cache reuse)."""
    from acache_amd.config import Config
    from acache_amd.model_runner import ModelRunner
    from acache_amd.sequence import Sequence
    from acache_amd.utils import reset_context
    cfg = Config(hf_config=model.config, mask_id=MASK, max_num_seqs=1, recompute_batch_size=1, gen_length=0,
                 block_length=1, cache_block_size=256, num_kvcache_blocks=4, enable_acache=False)
    runner = ModelRunner(model, cfg)
    seq = Sequence(list(tokens), gen_length=0, block_length=1, cache_block_size=256, mask_id=MASK)
    runner.block_manager.allocate(seq)
    try:
        ids, pos = runner.prepare_caching([seq])[:2]
        return runner.model(ids, position_ids=pos).logits.float()
    finally:
        reset_context()
        runner.block_manager.deallocate(seq)


def test_align_helper():
    x = torch.arange(12.0).view(1, 4, 3)
    y = GD._align_logits_for_dream(x)
    assert y[0, 0].tolist() == x[0, 0].tolist() and y[0, 1:].tolist() == x[0, :-1].tolist()


@pytest.mark.parametrize("placement", ["prefix", "infix", "suffix"])
@pytest.mark.parametrize("mode", ["threshold", "quota", "factor"])
def test_dream_generation_fills_the_window(device, placement, mode):
    cfg, model = _model(device)
    affix = list(range(20, 36))
    if placement == "prefix":
        prompt, kw = affix + [3, 4, 5], dict(affix_start=0, affix_end=16)
    elif placement == "infix":
        prompt, kw = [3, 4] + affix + [5, 6], dict(affix_start=2, affix_end=18)
    else:
        prompt, kw = [3, 4] + [MASK] * 8 + affix, dict(affix_start=10, affix_end=26, generation_start=2)
    extra = dict(threshold=0.9) if mode == "threshold" else dict(factor=1.0) if mode == "factor" else {}
    x, nfe = GD.generate_with_anchor_attention(
        model, torch.tensor([prompt], device=device), steps=8, gen_length=8, block_length=4, mask_id=MASK,
        anchor_ratio=0.25, **extra, **kw)
    gen_start = kw.get("generation_start", len(prompt))
    assert (x[0, gen_start:gen_start + 8] != MASK).all()
    keep = [i for i in range(len(prompt)) if not gen_start <= i < gen_start + 8]
    assert x[0, keep].tolist() == [prompt[i] for i in keep]
    if mode == "quota":
        assert nfe == 1 + 8      # importance pass + one refresh and three refinements per block of four
    else:
        assert 1 + 2 <= nfe <= 1 + 8


def test_first_token_of_a_block_comes_from_the_previous_position(device):
    """Dream reads token i from the hidden state of position i - 1.  With every affix token an anchor the refresh
    is a full recompute, so the first generated token must be the arg-max of the dense forward's logits at the
    position just before the window, and no importance pass is counted."""
    cfg, model = _model(device, seed=7)
    prompt = [3, 4] + list(range(10, 26)) + [5, 6, 7]
    x, nfe = GD.generate_with_anchor_attention(
        model, torch.tensor([prompt], device=device), steps=4, gen_length=4, block_length=4, mask_id=MASK,
        anchor_ratio=1.0, affix_start=2, affix_end=18)
    assert nfe == 4            # no importance pass; one refresh + three quota steps
    dense = _dense_logits(model, prompt + [MASK] * 4, device)
    top2 = dense[len(prompt) - 1].topk(2).values
    if (top2[0] - top2[1]).item() > 0.05:   # skip the comparison only if bf16 noise could flip the arg-max
        assert x[0, len(prompt)].item() == dense[len(prompt) - 1].argmax().item()


def test_dream_hf_layout_affix_cache(device):
    """Per-layer (k, v) in Dream's layout [1, A, H_kv * D], keys before RoPE, gives the same tokens as the engine's
    own affix forward."""
    cfg, model = _model(device, seed=2)
    affix = list(range(10, 40))
    prompt = [3, 4] + affix + [5, 6, 7]
    args = dict(steps=8, gen_length=8, block_length=4, mask_id=MASK, threshold=0.9, anchor_ratio=0.2,
                affix_start=2, affix_end=32)
    captured, hooks = [], []
    for block in model.model.transformer["blocks"]:
        store = {}
        hooks.append(block.k_proj.register_forward_hook(lambda m, i, o, s=store: s.__setitem__("k", o.detach().clone())))
        hooks.append(block.v_proj.register_forward_hook(lambda m, i, o, s=store: s.__setitem__("v", o.detach().clone())))
        captured.append(store)
    _dense_logits(model, affix, device)          # affix alone at positions 0..A-1: its projections before RoPE
    for h in hooks:
        h.remove()
    cache = tuple((s["k"].view(1, len(affix), -1), s["v"].view(1, len(affix), -1)) for s in captured)
    assert cache[0][0].shape == (1, 30, 2 * 64)
    ref, _ = GD.generate_with_anchor_attention(model, torch.tensor([prompt], device=device), **args)
    got, _ = GD.generate_with_anchor_attention(model, torch.tensor([prompt], device=device),
                                               precomputed_affix_cache=cache, **args)
    assert got.tolist() == ref.tolist()
    with pytest.raises(ValueError, match="does not match"):
        GD.generate_with_anchor_attention(model, torch.tensor([prompt], device=device), precomputed_affix_cache=cache,
                                          **{**args, "affix_end": 31})


def test_batched_engine_applies_the_dream_rule(device):
    """ModelRunner with model_type='dream' (model_runner.py:56-78, 1525-1552, 1703): shifted keep indices at a
    refresh, first-token seeding, block-shifted refinement logits.  For a single request it must commit the tokens
    of the HF-signature Dream entry point, with and without affix reuse."""
    from acache_amd.config import Config
    from acache_amd.model_runner import ModelRunner
    from acache_amd.sequence import Sequence
    cfg, model = _model(device, seed=9)
    affix = list(range(10, 26))
    prompt = [3, 4] + affix + [5, 6, 7]
    want, _ = GD.generate_with_anchor_attention(
        model, torch.tensor([prompt], device=device), steps=8, gen_length=8, block_length=4, mask_id=MASK,
        threshold=0.9, anchor_ratio=0.25, affix_start=2, affix_end=18)
    serve = Config(hf_config=cfg, mask_id=MASK, recompute_batch_size=1, max_num_seqs=1, gen_length=8, block_length=4,
                   threshold=0.9, cache_block_size=256, num_kvcache_blocks=8, temperature=0.0, enable_acache=True,
                   anchor_ratio=0.25, model_type="dream")
    runner = ModelRunner(model, serve)
    seq = Sequence(list(prompt), gen_length=8, block_length=4, cache_block_size=256, mask_id=MASK,
                   prompt_affix_start=2, prompt_affix_end=18)
    out, nfe = runner.generate_with_acache([seq])
    assert out[0] == want[0, -8:].tolist()
    # full recompute on the same weights: every position is predicted from its left neighbour too
    base = ModelRunner(model, Config(hf_config=cfg, mask_id=MASK, recompute_batch_size=1, max_num_seqs=1, gen_length=8,
                                     block_length=4, threshold=0.9, cache_block_size=256, num_kvcache_blocks=8,
                                     temperature=0.0, enable_acache=False, model_type="dream"))
    seq_b = Sequence(list(prompt), gen_length=8, block_length=4, cache_block_size=256, mask_id=MASK)
    out_b, _ = base.generate_with_dual_cache([seq_b])
    assert len(out_b[0]) == 8 and MASK not in out_b[0]
    # anchor_ratio 1.0 recomputes the whole affix: ACache must then agree with full recompute (bf16 noise aside)
    full = ModelRunner(model, Config(hf_config=cfg, mask_id=MASK, recompute_batch_size=1, max_num_seqs=1, gen_length=8,
                                     block_length=4, threshold=0.9, cache_block_size=256, num_kvcache_blocks=8,
                                     temperature=0.0, enable_acache=True, anchor_ratio=1.0, model_type="dream"))
    seq_f = Sequence(list(prompt), gen_length=8, block_length=4, cache_block_size=256, mask_id=MASK,
                     prompt_affix_start=2, prompt_affix_end=18)
    out_f, _ = full.generate_with_acache([seq_f])
    assert sum(a == b for a, b in zip(out_f[0], out_b[0])) >= 6


def test_checkpoint_model_object_gives_the_same_tokens(device):
    """The call as dream/eval_ACache.py makes it: ``model`` is the checkpoint's model object (here a stand-in with
    dream/model/modeling_dream.py's configuration fields and parameter names around the same weights).  The engine
    model is built around those tensors and must generate exactly what the engine model itself generates."""
    from types import SimpleNamespace

    from .test_generate_acache_host import CheckpointModelDouble

    cfg, model = _model(device)
    sd = model.state_dict()
    theirs = {"model.embed_tokens.weight": sd["model.transformer.wte.weight"],
              "model.norm.weight": sd["model.transformer.ln_f.weight"],
              "lm_head.weight": sd["model.transformer.ff_out.weight"],
              "model.rotary_emb.inv_freq": torch.zeros(64, device=device)}
    names = {"self_attn.q_proj": "q_proj", "self_attn.k_proj": "k_proj", "self_attn.v_proj": "v_proj",
             "self_attn.o_proj": "attn_out", "mlp.gate_proj": "ff_proj", "mlp.up_proj": "up_proj",
             "mlp.down_proj": "ff_out", "input_layernorm": "attn_norm", "post_attention_layernorm": "ff_norm"}
    for i in range(cfg.n_layers):
        for hf, ours in names.items():
            for leaf in ("weight", "bias"):
                key = f"model.transformer.blocks.{i}.{ours}.{leaf}"
                if key in sd:
                    theirs[f"model.layers.{i}.{hf}.{leaf}"] = sd[key].clone()   # clone: the engine model re-points its own views
    hf_cfg = SimpleNamespace(vocab_size=64, hidden_size=256, intermediate_size=128, num_hidden_layers=2,
                             num_attention_heads=4, num_key_value_heads=2, hidden_act="silu",
                             max_position_embeddings=128, rms_norm_eps=cfg.rms_norm_eps, rope_theta=10000.0,
                             rope_scaling=None, use_sliding_window=False, mask_token_id=MASK, tie_word_embeddings=False)
    checkpoint_model = CheckpointModelDouble(hf_cfg, theirs)
    prompt = torch.tensor([[3, 4] + list(range(20, 36)) + [5, 6]], device=device)
    kw = dict(steps=8, gen_length=8, block_length=4, mask_id=MASK, anchor_ratio=0.25, affix_start=2, affix_end=18,
              threshold=0.9)
    want, nfe_want = GD.generate_with_anchor_attention(model, prompt, **kw)
    got, nfe_got = GD.generate_with_anchor_attention(checkpoint_model, prompt, **kw)
    assert nfe_got == nfe_want and torch.equal(got, want)
