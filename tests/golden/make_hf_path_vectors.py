"""Writes tests/golden/hf_path_vectors.pt: inputs and outputs of the reference's batch-1 HF path
(llada/generate_ACache.py) on a tiny random-init LLaDA model (2 layers, 2 heads of 128), computed on the CPU in fp32.

This is the one place where reference code is imported and run: the importance values of
``compute_attention_importance_cross_affix`` and the trajectory of ``generate_with_anchor_attention`` are
pinned by no golden vector, test or closed form inside the reference, so the only way to pin them is to record
what the reference itself returns.  The fixture holds data only: the model's weights (rounded to bf16 values so
that the engine, which computes in bf16, starts from the same numbers), the prompts, and the returned tensors.

    python tests/golden/make_hf_path_vectors.py        # needs /root/reference; run in the build container

The GPU tests that read the fixture: tests/test_gpu_generate_acache.py (``*_reference_fixture``).
"""
import sys
from pathlib import Path

import torch

REFERENCE = Path("/root/reference/llada")
OUT = Path(__file__).resolve().parent / "hf_path_vectors.pt"
MASK = 63


def main():
    sys.path.insert(0, str(REFERENCE))      # the module imports `generate` and `model` as top-level names
    import generate_ACache as R
    from model.configuration_llada import LLaDAConfig
    from model.modeling_llada import LLaDAModelLM

    torch.manual_seed(0)
    cfg = LLaDAConfig(
        d_model=256, n_heads=2, n_layers=2, mlp_hidden_size=128, vocab_size=64, embedding_size=64,
        mask_token_id=MASK, eos_token_id=0, pad_token_id=0, rope=True, rope_theta=10000.0, alibi=False,
        block_type="llama", activation_type="silu", layer_norm_type="rms", rms_norm_eps=1e-5,
        include_bias=False, include_qkv_bias=False, weight_tying=False, attention_dropout=0.0,
        residual_dropout=0.0, embedding_dropout=0.0, input_emb_norm=False, flash_attention=False,
        max_sequence_length=256, init_device="cpu", init_std=0.1, scale_logits=False)
    model = LLaDAModelLM(cfg, init_params=True).float().eval()
    with torch.no_grad():
        for p in model.parameters():          # bf16-representable weights, fp32 arithmetic
            p.copy_(p.to(torch.bfloat16).float())
    weights = {k: v.to(torch.bfloat16) for k, v in model.state_dict().items()}   # exact: the values are bf16 already

    g = torch.Generator().manual_seed(1)
    cases = []
    for name, (n_head, n_affix, n_tail) in {"prefix": (0, 24, 6), "infix": (5, 20, 4), "suffix": (12, 18, 0)}.items():
        head = torch.randint(2, MASK, (n_head,), generator=g)
        affix = torch.randint(2, MASK, (n_affix,), generator=g)
        tail = torch.randint(2, MASK, (n_tail,), generator=g)
        prompt = torch.cat([head, affix, tail]).unsqueeze(0)
        a0, a1 = n_head, n_head + n_affix
        gen_length, block_length, steps = 8, 4, 8
        kwargs = dict(steps=steps, gen_length=gen_length, block_length=block_length, temperature=0.0,
                      remasking="low_confidence", mask_id=MASK, affix_start=a0, affix_end=a1,
                      anchor_ratio=0.25, selection_mode="top")
        if name == "suffix":                  # generation window inside the prompt, right in front of the affix
            kwargs["generation_start"] = n_head - gen_length
        with torch.no_grad():
            # the affix alone, encoded once (acache_eval_shared.py:608-609)
            affix_cache = model(affix.unsqueeze(0), use_cache=True).past_key_values
            # the sequence the entry point scores: prompt plus the masked generation window (generate_ACache.py:380-402)
            if "generation_start" in kwargs:
                masked = prompt.clone()
                masked[:, n_head - gen_length:n_head] = MASK
            else:
                masked = torch.cat([prompt, torch.full((1, gen_length), MASK)], dim=1)
            importance = R.compute_attention_importance_cross_affix(model, masked, affix_cache, mask_id=MASK,
                                                                    affix_start=a0)
            x, nfe = R.generate_with_anchor_attention(model, prompt, precomputed_affix_cache=affix_cache, **kwargs)
        cases.append({"name": name, "prompt": prompt, "kwargs": {k: v for k, v in kwargs.items()},
                      "masked_input": masked, "importance": importance.float().clone(),
                      "affix_cache": [(k.clone(), v.clone()) for k, v in affix_cache],
                      "x": x.clone(), "nfe": int(nfe)})
        print(name, "nfe", nfe, "importance[:6]", [round(t, 3) for t in importance[0, :6].tolist()], "x", x[0].tolist())

    torch.save({"config": dict(d_model=256, n_heads=2, n_layers=2, mlp_hidden_size=128, vocab_size=64,
                               mask_token_id=MASK, rope_theta=10000.0, max_sequence_length=256, rms_norm_eps=1e-5),
                "weights": weights, "cases": cases}, OUT)
    print("wrote", OUT, OUT.stat().st_size, "bytes")


if __name__ == "__main__":
    main()
