"""The Dream entry point against an independent restatement of the reference's Dream model and decoding loop.

Nothing here routes both sides through the engine.  One side is ``acache_amd.generate_acache_dream`` on the paged
engine (HIP kernels, bf16).  The other side is written in this file in plain fp32 torch on the CPU from the
reference's module definitions, with the reference's parameter names:

* ``TorchDream`` restates ``dream/model/modeling_dream.py``: ``DreamRMSNorm`` (78-83), biased q/k/v projections and
  an unbiased output projection (340-343), the pre-RoPE dual cache whose rows the inputs overwrite (463-515), rotary
  tables and rotate-half application at absolute positions (164-170, 184-189, 525-561), grouped-query attention by
  repeating KV heads (296-305, 563-593), ``DreamMLP`` (291-292), the pre-norm residual layer (660-692), the final
  norm and the untied head (798, 945, 1016);
* ``reference_generate`` restates the loop of ``dream/generate_ACache.py:425-737`` for the case in which every
  affix token is an anchor (556-562), with that file's ``get_num_transfer_tokens`` (66-82) and
  ``get_transfer_index`` (85-139) at temperature 0.

The engine model is built from the same checkpoint-style state dict through ``dream.engine_model_from_checkpoint``,
so the mapping of the Qwen2-style parameter names (gate / up / down, q / k / v with biases) is checked too: a
swapped pair fails the logits comparison.
"""
import math
from types import SimpleNamespace

import pytest
import torch
import torch.nn.functional as F

from acache_amd import generate_acache_dream as GD

pytestmark = pytest.mark.gpu
MASK = 63
V, DM, H, HKV, HD, LAYERS, MLP = 64, 256, 4, 2, 64, 2, 128
THETA, EPS = 10000.0, 1e-6


def _checkpoint_state(seed):
    """Random weights under the reference's names, bf16-representable, as fp32 tensors on the CPU."""
    g = torch.Generator().manual_seed(seed)

    def w(*shape, std=0.08):
        return (torch.randn(*shape, generator=g) * std).to(torch.bfloat16).float()

    sd = {"model.embed_tokens.weight": w(V, DM), "model.norm.weight": (1 + w(DM, std=0.05)), "lm_head.weight": w(V, DM)}
    sd["lm_head.weight"][MASK].zero_()   # [MASK] is never the arg-max: the loops below then always terminate
    for i in range(LAYERS):
        p = f"model.layers.{i}."
        sd[p + "input_layernorm.weight"] = 1 + w(DM, std=0.05)
        sd[p + "post_attention_layernorm.weight"] = 1 + w(DM, std=0.05)
        for name, rows in (("q_proj", H * HD), ("k_proj", HKV * HD), ("v_proj", HKV * HD)):
            sd[p + f"self_attn.{name}.weight"] = w(rows, DM)
            sd[p + f"self_attn.{name}.bias"] = w(rows, std=0.2)
        sd[p + "self_attn.o_proj.weight"] = w(DM, H * HD)
        sd[p + "mlp.gate_proj.weight"] = w(MLP, DM)
        sd[p + "mlp.up_proj.weight"] = w(MLP, DM)
        sd[p + "mlp.down_proj.weight"] = w(DM, MLP)
    return {k: v.to(torch.bfloat16).float() for k, v in sd.items()}


class TorchDream:
    """fp32 restatement of the reference's DreamModel forward with its dual cache (see the module docstring)."""

    def __init__(self, sd):
        self.sd = sd
        self.inv_freq = 1.0 / (THETA ** (torch.arange(0, HD, 2, dtype=torch.float32) / HD))

    def _rms(self, x, weight):                                            # DreamRMSNorm.forward, 78-83
        variance = x.pow(2).mean(-1, keepdim=True)
        return weight * (x * torch.rsqrt(variance + EPS))

    def _rope(self, x, positions):                                        # 164-170, 184-189, apply at 549-561
        freqs = positions.float()[:, None] * self.inv_freq[None, :]
        emb = torch.cat((freqs, freqs), dim=-1)
        cos, sin = emb.cos()[None], emb.sin()[None]                       # [1, T, D] against x [heads, T, D]
        x1, x2 = x[..., : HD // 2], x[..., HD // 2:]
        return x * cos + torch.cat((-x2, x1), dim=-1) * sin

    def forward(self, tokens, positions, cache=None, replace_rows=None, probe=None):
        """tokens, positions: [T].  cache: per layer (k, v) [L, HKV * HD] before RoPE, rows at absolute positions
        0..L-1; the T inputs overwrite rows ``replace_rows`` (one to one).  Without a cache the inputs are the
        whole sequence.  ``probe(layer, q)`` sees every layer's queries before RoPE, ``[T, H, HD]``.
        Returns (logits [T, V], cache)."""
        sd = self.sd
        x = sd["model.embed_tokens.weight"][tokens]
        new_cache = []
        for i in range(LAYERS):
            p = f"model.layers.{i}."
            y = self._rms(x, sd[p + "input_layernorm.weight"])
            q = F.linear(y, sd[p + "self_attn.q_proj.weight"], sd[p + "self_attn.q_proj.bias"])
            if probe is not None:
                probe(i, q.view(-1, H, HD))
            k = F.linear(y, sd[p + "self_attn.k_proj.weight"], sd[p + "self_attn.k_proj.bias"])
            v = F.linear(y, sd[p + "self_attn.v_proj.weight"], sd[p + "self_attn.v_proj.bias"])
            if cache is None:
                keys, values, key_pos = k, v, positions
            else:                                                          # 463-515: rows replaced in the cache
                keys, values = cache[i][0].clone(), cache[i][1].clone()
                keys[replace_rows], values[replace_rows] = k, v
                key_pos = torch.arange(keys.shape[0])
            new_cache.append((keys, values))
            qh = self._rope(q.view(-1, H, HD).transpose(0, 1), positions)
            kh = self._rope(keys.view(-1, HKV, HD).transpose(0, 1), key_pos)
            vh = values.view(-1, HKV, HD).transpose(0, 1)
            kh = kh.repeat_interleave(H // HKV, dim=0)                     # repeat_kv, 296-305
            vh = vh.repeat_interleave(H // HKV, dim=0)
            att = torch.softmax(qh @ kh.transpose(1, 2) / math.sqrt(HD), dim=-1) @ vh   # 586-593, no mask
            x = x + F.linear(att.transpose(0, 1).reshape(-1, H * HD), sd[p + "self_attn.o_proj.weight"])
            y = self._rms(x, sd[p + "post_attention_layernorm.weight"])
            x = x + F.linear(F.silu(F.linear(y, sd[p + "mlp.gate_proj.weight"])) * F.linear(y, sd[p + "mlp.up_proj.weight"]),
                             sd[p + "mlp.down_proj.weight"])
        return F.linear(self._rms(x, sd["model.norm.weight"]), sd["lm_head.weight"]), new_cache


def _align(logits):                                                       # dream/generate_ACache.py:47-49
    return torch.cat([logits[:1], logits[:-1]], dim=0)


def _num_transfer_tokens(mask_block, steps):                              # dream/generate_ACache.py:66-82
    total = int(mask_block.sum())
    base, rem = divmod(total, steps)
    return [base + (1 if j < rem else 0) for j in range(steps)]


LOGIT_TOL, CONF_TOL = 0.1, 0.01   # gaps below these could be flipped by bf16 noise in the engine's logits


def _transfer_index(logits, mask_block, x_block, quota, threshold):      # dream/generate_ACache.py:85-139, T = 0
    """Returns (x0, transfer, margins); a margin is a decision's gap divided by the noise it has to withstand."""
    x0 = logits.argmax(-1)
    conf = torch.softmax(logits.double(), -1).gather(-1, x0[:, None])[:, 0]
    x0 = torch.where(mask_block, x0, x_block)
    conf = torch.where(mask_block, conf, torch.full_like(conf, torch.finfo(torch.float64).min))
    margins = []
    if threshold is not None:
        transfer = mask_block & (conf >= threshold)
        margins += [abs(float(c) - threshold) / CONF_TOL for c in conf[mask_block]]
        if not transfer.any() and int(mask_block.sum()) > 1:             # the forced pick decides: which row is best?
            ranked = conf.sort(descending=True).values
            margins.append(float(ranked[0] - ranked[1]) / CONF_TOL)
        transfer[conf.argmax()] = True
        transfer &= mask_block
    else:
        order = conf.sort(descending=True).indices
        transfer = torch.zeros_like(mask_block)
        transfer[order[:quota]] = True
        transfer &= mask_block
        if 0 < quota < int(mask_block.sum()):
            ranked = conf.sort(descending=True).values
            margins.append(float(ranked[quota - 1] - ranked[quota]) / CONF_TOL)
    top2 = logits.topk(2, dim=-1).values
    margins += [float(d) / LOGIT_TOL for d in (top2[:, 0] - top2[:, 1])[transfer]]
    return x0, transfer, margins


def reference_generate(model, prompt, steps, gen_length, block_length, threshold=None, generation_start=None):
    """dream/generate_ACache.py:486-735 with every affix token an anchor (556-562: no importance pass, so every
    position is recomputed at a block refresh).  Returns (x, nfe, smallest decision margin)."""
    num_blocks = gen_length // block_length
    spb = steps // num_blocks
    x = list(prompt)
    if generation_start is None:
        generation_start = len(prompt)
        x = x + [MASK] * gen_length
    else:
        x[generation_start:generation_start + gen_length] = [MASK] * gen_length
    x = torch.tensor(x)
    L = x.numel()
    every = torch.arange(L)
    margins = []
    logits, cache = model.forward(x, every)                               # 617-628: the initial forward
    logits, nfe = _align(logits), 1
    for nb in range(num_blocks):
        s = generation_start + nb * block_length
        e = s + block_length
        if nb > 0:                                                        # 655-675: block refresh
            logits, cache = model.forward(x, every, cache, every)
            logits, nfe = _align(logits), nfe + 1
        blk = logits[s:e]
        top2 = blk[0].topk(2).values
        margins.append(float(top2[0] - top2[1]) / LOGIT_TOL)
        x[s] = blk[0].argmax()                                            # 686-690: only the first token is committed
        quota = _num_transfer_tokens(x[s:e] == MASK, spb - 1) if threshold is None and spb > 1 else None   # 692-696
        for i in range(1, spb):                                           # 699-735: block-only refinement
            if (x[s:e] == MASK).sum() == 0:
                break
            out, cache = model.forward(x[s:e], torch.arange(s, e), cache, torch.arange(s, e))
            nfe += 1
            x0, transfer, m = _transfer_index(_align(out), x[s:e] == MASK, x[s:e], None if quota is None else quota[i - 1], threshold)
            margins += m
            x[s:e] = torch.where(transfer, x0, x[s:e])
    return x, nfe, min(margins)


def _engine_model(sd, device):
    from acache_amd.dream import engine_model_from_checkpoint

    from .test_generate_acache_host import CheckpointModelDouble
    hf_cfg = SimpleNamespace(vocab_size=V, hidden_size=DM, intermediate_size=MLP, num_hidden_layers=LAYERS,
                             num_attention_heads=H, num_key_value_heads=HKV, hidden_act="silu", max_position_embeddings=128,
                             rms_norm_eps=EPS, rope_theta=THETA, rope_scaling=None, use_sliding_window=False,
                             mask_token_id=MASK, tie_word_embeddings=False)
    theirs = {k: v.to(device=device, dtype=torch.bfloat16) for k, v in sd.items()}
    theirs["model.rotary_emb.inv_freq"] = torch.zeros(HD // 2, device=device)
    return engine_model_from_checkpoint(CheckpointModelDouble(hf_cfg, theirs)).eval()


def _engine_dense_logits(model, tokens):
    """Full-sequence forward of the engine model through the paged engine (no cache reuse)."""
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


def test_decoding_helpers_on_hand_computed_cases():
    # left shift (47-49): row i reads row i - 1, row 0 keeps its own
    x = torch.arange(12.0).view(1, 4, 3)
    assert GD._align_logits_for_dream(x)[0].tolist() == [[0, 1, 2], [0, 1, 2], [3, 4, 5], [6, 7, 8]]
    # quota over the steps that remain after the seeding step (692-696): 5 masks over 3 steps -> 2, 2, 1
    mask = torch.tensor([[True, True, False, True, True, True]])
    assert GD.get_num_transfer_tokens(mask, 3).tolist() == [[2, 2, 1]]
    assert _num_transfer_tokens(mask[0], 3) == [2, 2, 1]
    # first-token seeding takes the arg-max of the block's first (shifted) row at temperature 0 (686-690)
    conf, tok = GD.sample_tokens(torch.tensor([[0.0, 2.0, 1.0], [3.0, 0.0, 0.0]]), temperature=0.0)
    assert tok.tolist() == [1, 0] and abs(conf[0].item() - math.exp(2) / (1 + math.exp(2) + math.exp(1))) < 1e-6


@pytest.mark.parametrize("seed", [0, 1])
def test_engine_logits_match_the_restated_dream_forward(device, seed):
    sd = _checkpoint_state(seed)
    model = _engine_model(sd, device)
    g = torch.Generator().manual_seed(100 + seed)
    tokens = torch.randint(0, V - 1, (45,), generator=g).tolist() + [MASK] * 8
    want, _ = TorchDream(sd).forward(torch.tensor(tokens), torch.arange(len(tokens)))
    got = _engine_dense_logits(model, tokens).cpu()
    assert got.shape == want.shape
    # bf16 engine against an fp32 model: the rounding of two layers of bf16 activations shows in full (the
    # reference's own engine tests compare bf16 with bf16 at rtol = atol = 5e-2, tests/test_model_runner_acache.py:687).
    # Measured: mean 1.3e-2, largest 7.5e-2 on logits of magnitude up to 5.
    diff = (got - want).abs()
    assert diff.mean().item() <= 2e-2 and diff.max().item() <= 1.5e-1, (diff.mean().item(), diff.max().item())
    assert want.abs().max().item() > 1.0      # the comparison is not vacuous: logits of order one
    # ... and the bound has teeth: the same forward with one pair of projections exchanged (what a slip in the
    # checkpoint name mapping would do) or with the rotary halves the other way round is far outside it
    for a, b in (("mlp.gate_proj", "mlp.up_proj"), ("self_attn.k_proj", "self_attn.v_proj")):
        swapped = dict(sd)
        for key in sd:
            if a in key:
                swapped[key], swapped[key.replace(a, b)] = sd[key.replace(a, b)], sd[key]
        wrong, _ = TorchDream(swapped).forward(torch.tensor(tokens), torch.arange(len(tokens)))
        assert (got - wrong).abs().mean().item() > 10 * 2e-2, (a, b)
    shifted, _ = TorchDream(sd).forward(torch.tensor(tokens), torch.arange(len(tokens)) + 3)
    assert (shifted - want).abs().max().item() < 1e-3     # rotary positions are relative: a uniform offset changes nothing
    flipped = TorchDream(sd)
    flipped.inv_freq = -flipped.inv_freq                                  # the rotation the other way round ...
    wrong, _ = flipped.forward(torch.tensor(tokens), torch.arange(len(tokens)))
    assert (got - wrong).abs().mean().item() > 10 * 2e-2  # ... swaps left and right context: a different model
    nope = TorchDream(sd)
    nope._rope = lambda x, positions: x                                   # and so is no rotary at all
    wrong, _ = nope.forward(torch.tensor(tokens), torch.arange(len(tokens)))
    assert (got - wrong).abs().mean().item() > 10 * 2e-2


@pytest.mark.parametrize("placement", ["prefix", "infix", "suffix"])
@pytest.mark.parametrize("mode", ["quota", "threshold"])
def test_all_anchor_generation_equals_the_restated_loop(device, placement, mode):
    affix = list(range(20, 36))
    if placement == "prefix":
        prompt, kw = affix + [3, 4, 5], dict(affix_start=0, affix_end=16)
    elif placement == "infix":
        prompt, kw = [3, 4] + affix + [5, 6], dict(affix_start=2, affix_end=18)
    else:
        prompt, kw = [3, 4] + [MASK] * 8 + affix, dict(affix_start=10, affix_end=26, generation_start=2)
    threshold = 0.9 if mode == "threshold" else None
    # a seed whose every decision in the fp32 loop has a margin that bf16 noise cannot flip (arg-max gaps in logits,
    # confidence gaps at the quota / threshold boundary); the search is deterministic and runs on the CPU
    for seed in range(400):
        sd = _checkpoint_state(seed)
        want, nfe_want, margin = reference_generate(TorchDream(sd), prompt, steps=8, gen_length=8, block_length=4,
                                                    threshold=threshold, generation_start=kw.get("generation_start"))
        if margin > 1.0:
            break
    else:
        pytest.fail("no seed with comfortable decision margins")
    assert (want != MASK).all()
    model = _engine_model(sd, device)
    got, nfe = GD.generate_with_anchor_attention(
        model, torch.tensor([prompt], device=device), steps=8, gen_length=8, block_length=4, mask_id=MASK,
        anchor_ratio=1.0, threshold=threshold, **kw)
    assert got[0].cpu().tolist() == want.tolist()
    assert nfe == nfe_want                      # no importance pass is counted when every affix token is an anchor
    if mode == "quota":
        assert nfe == 8                         # per block of four: one refresh (seeds one token) + three quota steps


# --------------------------------------------------------------------------------------------------------------
# Anchor ratio below 1: the path that actually reuses the affix.  Restated from dream/generate_ACache.py:
#   the affix cache is the affix ALONE at positions 0..A-1, keys before RoPE (acache_eval_shared.py:599-609);
#   importance (183-344): one forward over the non-affix tokens against a cache that holds the frozen affix rows;
#     per layer, softmax over the AFFIX keys only of every query (rotated at their absolute positions), summed
#     over heads and over the [MASK] queries;
#   anchors (347-375): top-k by importance, ascending, plus affix_start;  k = min(ceil(ratio * A), A) (40-44, 552-553);
#   recomputed positions = anchors + every non-affix position; logits are shifted left in THAT compact order
#     (576-628); non-anchor affix rows keep the cached K/V for the whole run.

def reference_affix_cache(model, affix_tokens):
    _, cache = model.forward(torch.tensor(affix_tokens), torch.arange(len(affix_tokens)))
    return cache


def reference_importance(model, x, affix_cache, a0, A):
    L = x.numel()
    probe_pos = torch.cat([torch.arange(0, a0), torch.arange(a0 + A, L)])
    mask_q = (x[probe_pos] == MASK).float()
    cache = []
    for k, v in affix_cache:
        ck, cv = torch.zeros(L, HKV * HD), torch.zeros(L, HKV * HD)
        ck[a0:a0 + A], cv[a0:a0 + A] = k, v
        cache.append((ck, cv))
    importance = torch.zeros(A)

    def probe(layer, q):                                                  # 246-285
        q_rot = model._rope(q.transpose(0, 1), probe_pos)                 # [H, T, HD] at the queries' own positions
        k_rot = model._rope(affix_cache[layer][0].view(A, HKV, HD).transpose(0, 1), torch.arange(a0, a0 + A))
        k_rot = k_rot.repeat_interleave(H // HKV, dim=0)
        weights = torch.softmax(q_rot @ k_rot.transpose(1, 2) * HD ** -0.5, dim=-1)       # over affix keys only
        importance.add_((weights * mask_q[None, :, None]).sum(dim=1).sum(dim=0))

    model.forward(x[probe_pos], probe_pos, cache, probe_pos, probe=probe)
    return importance


def reference_generate_partial(model, prompt, a0, A, ratio, steps, gen_length, block_length, threshold=None):
    """Returns (x, nfe, anchors, smallest decision margin).  Tail generation (generation_start = len(prompt))."""
    num_blocks = gen_length // block_length
    spb = steps // num_blocks
    gen0 = len(prompt)
    x = torch.tensor(list(prompt) + [MASK] * gen_length)
    L = x.numel()
    affix_cache = reference_affix_cache(model, list(prompt[a0:a0 + A]))
    k = min(math.ceil(ratio * A), A)
    importance = reference_importance(model, x, affix_cache, a0, A)
    ranked = importance.sort(descending=True)
    anchors = (ranked.indices[:k].sort().values + a0)                     # 367-373 + 571
    margins = [float(ranked.values[k - 1] - ranked.values[k]) / (0.03 * float(ranked.values[k - 1]))]
    nfe = 1
    keep = torch.ones(L, dtype=torch.bool)
    keep[a0:a0 + A] = False
    keep[anchors] = True
    rec = keep.nonzero()[:, 0]                                            # recompute positions, ascending
    compact_of = {int(pos): i for i, pos in enumerate(rec)}
    cache = []
    for ck, cv in affix_cache:                                            # 612-626
        fk, fv = torch.zeros(L, HKV * HD), torch.zeros(L, HKV * HD)
        fk[a0:a0 + A], fv[a0:a0 + A] = ck, cv
        cache.append((fk, fv))
    logits, cache = model.forward(x[rec], rec, cache, rec)                # 630-640
    logits, nfe = _align(logits), nfe + 1
    for nb in range(num_blocks):
        s = gen0 + nb * block_length
        e = s + block_length
        if nb > 0:                                                        # 655-675
            logits, cache = model.forward(x[rec], rec, cache, rec)
            logits, nfe = _align(logits), nfe + 1
        c0 = compact_of[s]
        blk = logits[c0:c0 + block_length]
        top2 = blk[0].topk(2).values
        margins.append(float(top2[0] - top2[1]) / LOGIT_TOL)
        x[s] = blk[0].argmax()
        quota = _num_transfer_tokens(x[s:e] == MASK, spb - 1) if threshold is None and spb > 1 else None
        for i in range(1, spb):
            if (x[s:e] == MASK).sum() == 0:
                break
            out, cache = model.forward(x[s:e], torch.arange(s, e), cache, torch.arange(s, e))
            nfe += 1
            x0, transfer, m = _transfer_index(_align(out), x[s:e] == MASK, x[s:e], None if quota is None else quota[i - 1], threshold)
            margins += m
            x[s:e] = torch.where(transfer, x0, x[s:e])
    return x, nfe, anchors.tolist(), min(margins)


@pytest.mark.parametrize("threshold", [None, 0.03], ids=["quota", "threshold"])
@pytest.mark.parametrize("placement", ["prefix", "infix"])
def test_partial_ratio_generation_equals_the_restated_loop(device, placement, threshold):
    """Anchor ratio 0.25: importance pass, top-k anchors, frozen non-anchor affix rows, recompute of anchors and
    non-affix tokens at every block boundary.  Tokens and forward count must equal the restated reference loop, with
    the engine's own affix precompute and with the affix cache in Dream's layout handed in."""
    A = 24
    affix = [10 + (5 * i) % 40 for i in range(A)]
    if placement == "prefix":
        prompt, a0 = affix + [3, 4, 5, 6, 7], 0
    else:
        prompt, a0 = [3, 4, 5] + affix + [6, 7, 8], 3
    for seed in range(400):
        sd = _checkpoint_state(seed)
        ref = TorchDream(sd)
        want, nfe_want, anchors, margin = reference_generate_partial(ref, prompt, a0, A, 0.25, steps=8, gen_length=8,
                                                                    block_length=4, threshold=threshold)
        if margin > 1.0 and len(set(want[-8:].tolist())) >= 4:            # decisive and not one token eight times
            break
    else:
        pytest.fail("no seed with comfortable decision margins")
    assert len(anchors) == 6 and (want != MASK).all()
    # the frozen affix rows matter: recomputing the whole affix (every token an anchor) decodes other tokens
    everything, _, _ = reference_generate(ref, prompt, steps=8, gen_length=8, block_length=4, threshold=threshold,
                                          generation_start=None)
    assert everything.tolist() != want.tolist()
    model = _engine_model(sd, device)
    kw = dict(steps=8, gen_length=8, block_length=4, mask_id=MASK, anchor_ratio=0.25, affix_start=a0, affix_end=a0 + A,
              threshold=threshold)
    got, nfe = GD.generate_with_anchor_attention(model, torch.tensor([prompt], device=device), **kw)
    assert got[0].cpu().tolist() == want.tolist() and nfe == nfe_want
    # the same call with the reference-layout affix cache: [1, A, H_kv * D] per layer, keys before RoPE
    cache = tuple((k.to(device=device, dtype=torch.bfloat16)[None], v.to(device=device, dtype=torch.bfloat16)[None])
                  for k, v in reference_affix_cache(ref, affix))
    got2, nfe2 = GD.generate_with_anchor_attention(model, torch.tensor([prompt], device=device),
                                                   precomputed_affix_cache=cache, **kw)
    assert got2[0].cpu().tolist() == want.tolist() and nfe2 == nfe_want
    # and the importance values themselves (fp32 there, bf16 with the rotation on the queries here)
    x = torch.tensor([list(prompt) + [MASK] * 8], device=device)
    imp = GD.compute_attention_importance_cross_affix(model, x, cache, mask_id=MASK, affix_start=a0).cpu()[0]
    want_imp = reference_importance(ref, x[0].cpu(), reference_affix_cache(ref, affix), a0, A)
    torch.testing.assert_close(imp, want_imp, rtol=6e-2, atol=6e-2)
    assert abs(imp.sum().item() - want_imp.sum().item()) <= 1e-2 * want_imp.sum().item()
