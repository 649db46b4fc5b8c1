"""Batch-1 entry points with the HF path's signatures (llada/generate_ACache.py) on the paged engine."""
from pathlib import Path

import pytest
import torch

from acache_amd import generate_acache as G
from acache_amd.llada import LLaDAConfig, LLaDAModelLM

pytestmark = pytest.mark.gpu
MASK = 63


def _model(device, seed=0):
    torch.manual_seed(seed)
    cfg = LLaDAConfig(vocab_size=64, d_model=256, n_heads=4, n_layers=2, mlp_hidden_size=128,
                      max_sequence_length=128, mask_token_id=MASK, rope_theta=10000.0)
    model = LLaDAModelLM(cfg, init_std=0.08).to(device=device, dtype=torch.bfloat16).eval()
    with torch.no_grad():
        # these loops run a fixed number of steps (no spin is possible); a 64-token random head that answers [MASK]
        # would only leave a hole in the window, which the fill assertions below would then report as a failure
        model.model.transformer["ff_out"].weight[MASK].zero_()
        model.model.transformer["ff_out"].weight[0] += 0.05
    return cfg, model


FIXTURE = Path(__file__).resolve().parent / "golden" / "hf_path_vectors.pt"


def _fixture(device, as_checkpoint_object=False):
    """The reference's own outputs (tests/golden/make_hf_path_vectors.py ran llada/generate_ACache.py on the CPU in
    fp32 over a 2-layer random model with 2 heads of 128) and a model with the same weights: this package's engine
    model, or a stand-in for the checkpoint model object the reference's caller passes (configuration fields and
    state dict of llada/model/modeling_llada.py's class, no forward of its own)."""
    data = torch.load(FIXTURE, weights_only=True)
    if as_checkpoint_object:
        from .test_generate_acache_host import CheckpointModelDouble, _llada_checkpoint_config

        weights = {name: t.to(device) for name, t in data["weights"].items()}
        return data["cases"], CheckpointModelDouble(_llada_checkpoint_config(), weights)
    model = LLaDAModelLM(LLaDAConfig(**data["config"]))
    model.load_state_dict(data["weights"])       # same parameter names as the reference's LLaDAModelLM
    return data["cases"], model.to(device=device, dtype=torch.bfloat16).eval()


@pytest.mark.parametrize("as_checkpoint_object", [False, True])
def test_importance_matches_the_reference_fixture(device, as_checkpoint_object):
    """compute_attention_importance_cross_affix against the values the reference returned for prefix, infix and
    suffix placement.  The reference ran in fp32, the engine in bf16 with the relocation on the query side:
    measured difference 0.044 absolute / 4.6 % relative at most; bound 0.06 / 6 %, and the total weight (mask rows x
    heads x layers, which a per-layer weighting slip would change) within 0.5 %.  The anchors chosen from the two
    importance vectors must be the same tokens."""
    cases, model = _fixture(device, as_checkpoint_object)
    for c in cases:
        kw = c["kwargs"]
        cache = tuple((k.to(device), v.to(device)) for k, v in c["affix_cache"])
        got = G.compute_attention_importance_cross_affix(model, c["masked_input"].to(device), cache, mask_id=MASK,
                                                         affix_start=kw["affix_start"]).cpu()
        want = c["importance"]
        assert got.shape == want.shape
        torch.testing.assert_close(got, want, rtol=6e-2, atol=6e-2, msg=lambda m: f"{c['name']}: {m}")
        assert abs(got.sum().item() - want.sum().item()) <= 5e-3 * want.sum().item(), c["name"]
        k = G.ceil_to_int(kw["anchor_ratio"] * want.shape[1])
        assert (G.select_anchor_tokens(got.to(device), k, "top").tolist()
                == G.select_anchor_tokens(want.to(device), k, "top").tolist()), c["name"]


@pytest.mark.parametrize("as_checkpoint_object", [False, True])
@pytest.mark.parametrize("from_cache", [True, False])
def test_generation_matches_the_reference_fixture(device, from_cache, as_checkpoint_object):
    """generate_with_anchor_attention against the reference's returned sequence and forward count, with the HF-layout
    affix cache the reference was given and with the engine's own affix precompute.  Prompt positions and the
    number of forwards must be equal; of the 8 generated tokens at most one may differ (fp32 there, bf16 here: an
    arg-max near a tie can flip; measured: none differs).  ``as_checkpoint_object``: the call as the reference's
    caller makes it, with the checkpoint's model object in the ``model`` argument."""
    cases, model = _fixture(device, as_checkpoint_object)
    for c in cases:
        kw = dict(c["kwargs"])
        cache = tuple((k.to(device), v.to(device)) for k, v in c["affix_cache"]) if from_cache else None
        x, nfe = G.generate_with_anchor_attention(model, c["prompt"].to(device), precomputed_affix_cache=cache, **kw)
        want = c["x"]
        assert nfe == c["nfe"] and x.shape == want.shape, c["name"]
        start = kw.get("generation_start", c["prompt"].shape[1])
        window = slice(start, start + kw["gen_length"])
        outside = torch.ones(want.shape[1], dtype=torch.bool)
        outside[window] = False
        assert torch.equal(x.cpu()[0, outside], want[0, outside]), c["name"]
        assert int((x.cpu()[0, window] != want[0, window]).sum()) <= 1, (c["name"], x[0, window].tolist(), want[0, window].tolist())
        assert (x[0, window] != MASK).all()


def test_helpers_match_the_reference_definitions(device):
    assert [G.ceil_to_int(v) for v in (0.0, 2.0, 2.1, 7.000000000000001)] == [0, 2, 3, 8]
    x = torch.arange(20, device=device).view(2, 10)
    anchors = torch.tensor([[1, 3], [0, 2]], device=device)
    gathered, replace = G.gather_tokens_for_recompute(x, anchors, 6, 8)
    assert gathered.tolist() == [[1, 3, 6, 7], [10, 12, 16, 17]]
    assert replace[0].nonzero().flatten().tolist() == [1, 3, 6, 7]
    mask = torch.tensor([[True] * 7 + [False]], device=device)
    assert G.get_num_transfer_tokens(mask, 3).tolist() == [[3, 2, 2]]
    logits = torch.zeros(1, 4, 8, device=device)
    logits[0, 0, 5] = 9.0
    logits[0, 2, 1] = 3.0
    m = torch.tensor([[True, True, True, False]], device=device)
    cur = torch.full((1, 4), MASK, device=device)
    x0, t = G.get_transfer_index(logits, 0.0, "low_confidence", m, cur, torch.tensor([2], device=device))
    assert t.tolist() == [[True, False, True, False]] and x0[0, 0] == 5 and x0[0, 3] == MASK
    x0, t = G.get_transfer_index(logits, 0.0, "low_confidence", m, cur, None, threshold=0.99)
    assert t.tolist() == [[True, False, False, False]]


@pytest.mark.parametrize("placement", ["prefix", "infix", "suffix"])
@pytest.mark.parametrize("use_threshold", [True, False])
def test_generate_with_anchor_attention_fills_the_window(device, placement, use_threshold):
    cfg, model = _model(device)
    affix = list(range(20, 36))
    if placement == "prefix":
        prompt, kw = affix + [3, 4, 5], dict(affix_start=0, affix_end=16)
    elif placement == "infix":
        prompt, kw = [3, 4] + affix + [5, 6], dict(affix_start=2, affix_end=18)
    else:  # generation window inside the prompt, affix after it
        prompt, kw = [3, 4] + [MASK] * 8 + affix, dict(affix_start=10, affix_end=26, generation_start=2)
    x, nfe = G.generate_with_anchor_attention(
        model, torch.tensor([prompt], device=device), steps=8, gen_length=8, block_length=4, mask_id=MASK,
        threshold=0.9 if use_threshold else None, anchor_ratio=0.25, **kw)
    total = len(prompt) + (0 if placement == "suffix" else 8)
    assert x.shape == (1, total)
    gen_start = kw.get("generation_start", len(prompt))
    assert (x[0, gen_start:gen_start + 8] != MASK).all()
    keep = [i for i in range(len(prompt)) if not gen_start <= i < gen_start + 8]
    assert x[0, keep].tolist() == [prompt[i] for i in keep]
    if use_threshold:
        assert 1 + 2 <= nfe <= 1 + 8
    else:
        assert nfe == 1 + 8          # importance pass + exactly `steps` forwards in quota mode


def test_precomputed_hf_layout_affix_cache_equals_engine_precompute(device):
    """A per-layer (k, v) cache in the HF layout ([1, H_kv, A, D], keys before RoPE) lands in the same shared
    slots as the engine's own affix forward, and generation from it gives the same tokens."""
    cfg, model = _model(device, seed=2)
    affix = list(range(10, 40))
    prompt = [3, 4] + affix + [5, 6, 7]
    args = dict(steps=8, gen_length=8, block_length=4, mask_id=MASK, threshold=0.9, anchor_ratio=0.2,
                affix_start=2, affix_end=32)
    captured = []
    hooks = []
    for block in model.model.transformer["blocks"]:
        store = {}
        captured.append(store)
        hooks.append(block.k_proj.register_forward_hook(lambda m, i, o, s=store: s.__setitem__("k", o.detach().clone())))
        hooks.append(block.v_proj.register_forward_hook(lambda m, i, o, s=store: s.__setitem__("v", o.detach().clone())))
    runner = G._as_runner(model, mask_id=MASK, block_length=4, gen_length=8, anchor_ratio=0.2, selection_mode="top",
                          threshold=0.9, temperature=0.0, remasking="low_confidence", total_len=len(prompt) + 8,
                          affix_len=30)
    with torch.inference_mode():
        runner._precompute_shared_prefix(affix)
    for h in hooks:
        h.remove()
    H, D = cfg.n_heads, cfg.d_model // cfg.n_heads
    hf_cache = tuple((s["k"].view(30, H, D).permute(1, 0, 2).unsqueeze(0), s["v"].view(30, H, D).permute(1, 0, 2).unsqueeze(0))
                     for s in captured)
    shared_ref = runner.kv_cache[:, :, 0, :30].clone()
    x_ref, nfe_ref = G.generate_with_anchor_attention(runner, torch.tensor([prompt], device=device), **args)

    x_hf, nfe_hf = G.generate_with_anchor_attention(model, torch.tensor([prompt], device=device),
                                                    precomputed_affix_cache=hf_cache, **args)
    assert torch.equal(x_hf, x_ref) and nfe_hf == nfe_ref
    runner2 = G._as_runner(model, mask_id=MASK, block_length=4, gen_length=8, anchor_ratio=0.2, selection_mode="top",
                           threshold=0.9, temperature=0.0, remasking="low_confidence", total_len=len(prompt) + 8,
                           affix_len=30)
    G._ingest_affix_cache(runner2, affix, hf_cache)
    assert torch.equal(runner2.kv_cache[:, :, 0, :30], shared_ref)


def test_importance_entry_point_and_anchor_selection(device):
    cfg, model = _model(device, seed=3)
    affix = list(range(10, 30))
    x = torch.tensor([[3, 4] + affix + [5] + [MASK] * 4], device=device)
    imp = G.compute_attention_importance_cross_affix(model, x, None, mask_id=MASK, affix_start=2, affix_len=20)
    assert imp.shape == (1, 20) and imp.dtype == torch.float32
    # softmax rows sum to 1: total importance = mask queries x heads x layers
    assert abs(imp.sum().item() - 4 * cfg.n_heads * cfg.n_layers) < 0.5
    idx = G.select_anchor_tokens(imp, 5, "top")
    assert idx.shape == (1, 5) and idx[0].tolist() == sorted(torch.topk(imp[0], 5).indices.tolist())


def test_drop_non_anchor_never_sees_the_dropped_affix_tokens(device):
    """Strict ablation (llada/generate_ACache.py:478-491): with the frozen affix rows left out of attention, the
    output may depend on the affix only through the anchors.  Ratio 0 keeps no anchor, so two different affixes of
    the same length must give the same generation; ratio 1 keeps every affix token, so nothing is dropped and the
    result equals the ordinary path."""
    cfg, model = _model(device, seed=4)
    head, tail = [3, 4], [5, 6, 7]
    args = dict(steps=8, gen_length=8, block_length=4, mask_id=MASK, threshold=0.9, affix_start=2, affix_end=22)
    outs = []
    for affix in (list(range(10, 30)), list(range(40, 60))):
        prompt = torch.tensor([head + affix + tail], device=device)
        x, nfe = G.generate_with_anchor_attention(model, prompt, anchor_ratio=0.0, drop_non_anchor=True, **args)
        assert x.shape == (1, prompt.shape[1] + 8) and (x[0, -8:] != MASK).all()
        outs.append(x[0, -8:].tolist())
    assert outs[0] == outs[1]
    prompt = torch.tensor([head + list(range(10, 30)) + tail], device=device)
    full_drop, _ = G.generate_with_anchor_attention(model, prompt, anchor_ratio=1.0, drop_non_anchor="true", **args)
    full_keep, _ = G.generate_with_anchor_attention(model, prompt, anchor_ratio=1.0, drop_non_anchor=False, **args)
    assert full_drop.tolist() == full_keep.tolist()


def test_dynamic_threshold_factor_runs_and_bounds_nfe(device):
    cfg, model = _model(device, seed=5)
    prompt = torch.tensor([[3, 4] + list(range(10, 30)) + [5, 6]], device=device)
    x, nfe = G.generate_with_anchor_attention(model, prompt, steps=8, gen_length=8, block_length=4, mask_id=MASK,
                                              factor=1.0, anchor_ratio=0.25, affix_start=2, affix_end=22)
    assert (x[0, -8:] != MASK).all()
    # every step commits at least one token: at most 4 forwards per block of 4, at least 1; plus the importance pass
    assert 1 + 2 <= nfe <= 1 + 8


def test_argument_errors(device):
    cfg, model = _model(device)
    p = torch.tensor([[3, 4, 5, 6]], device=device)
    with pytest.raises(ValueError, match="boolean-like"):
        G.generate_with_anchor_attention(model, p, steps=4, gen_length=4, block_length=4, mask_id=MASK,
                                         drop_non_anchor="perhaps", affix_end=2)
    with pytest.raises(ValueError, match="must not overlap"):
        G.generate_with_anchor_attention(model, p, steps=2, gen_length=2, block_length=2, mask_id=MASK,
                                         affix_start=0, affix_end=3, generation_start=2)
