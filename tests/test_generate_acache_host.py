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


def test_foreign_models_are_rejected_with_a_type_error():
    """The entry points keep the reference's signature but run on the paged engine: a model that is not built from
    this package's attention modules (an HF checkpoint model, say) is refused before any device work."""
    from acache_amd.generate_acache import generate_with_anchor_attention

    class Foreign(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.model = torch.nn.Linear(4, 4)
            self.config = object()

    prompt = torch.arange(2, 10).unsqueeze(0)
    with pytest.raises(TypeError, match="needs an acache_amd model"):
        generate_with_anchor_attention(Foreign(), prompt, steps=4, gen_length=4, block_length=4, mask_id=MASK,
                                       affix_start=0, affix_end=4)
