"""Affix-importance kernels against the oracle's fp32 restatement of nano-vdllm/model_runner.py:730-773.
Both score bf16 operands with fp32 accumulation and an fp32 softmax.  The oracle, like the reference, re-rotates
the cached keys and rounds them to bf16; the kernels rotate the queries by the opposite angle and round those
(the same product before rounding), and they sum in another order: 2e-3 relative, 1e-4 absolute."""
import pytest
import torch

from acache_amd import ops
from oracle import acache_oracle as O

pytestmark = pytest.mark.gpu


def _case(device, H, Hkv, D, A, mask_counts, shifts, slot0=0, dtype=torch.bfloat16, seed=0):
    g = torch.Generator().manual_seed(seed)
    S = slot0 + A + 7
    cos, sin = O.rope_table(max(shifts) + 2 if shifts else 4, D, 5e5)
    kc = (torch.randn(S, Hkv, D, generator=g) / D ** 0.25).to(dtype)
    Tq = sum(mask_counts) * 2 + 5
    q = (torch.randn(Tq, H, D, generator=g) / D ** 0.25).to(dtype)
    rows = torch.randperm(Tq, generator=g)[:sum(mask_counts)].sort().values.to(torch.int32)
    cu = torch.tensor([0] + torch.tensor(mask_counts).cumsum(0).tolist(), dtype=torch.int32)
    sh = torch.tensor(shifts, dtype=torch.int32) if shifts else None
    want = O.affix_importance(q, kc, rows, cu, A, affix_shifts=sh, cos=cos, sin=sin, affix_slot0=slot0)
    imp = torch.zeros(len(mask_counts), A + 3, dtype=torch.float32, device=device)
    args = dict(affix_shifts=None if sh is None else sh.to(device), rope_cos=cos.to(device) if shifts else None,
                rope_sin=sin.to(device) if shifts else None, affix_slot0=slot0)
    ops.affix_importance(imp, q.to(device), kc.to(device), rows.to(device), cu.to(device), A, max(mask_counts), **args)
    got = imp.cpu()
    assert torch.all(got[:, A:] == 0)                                     # padding columns untouched
    assert torch.allclose(got[:, :A], want, rtol=2e-3, atol=1e-4), (got[:, :A] - want).abs().max()
    return imp, want, (q, kc, rows, cu, args)


@pytest.mark.parametrize("H,Hkv,D", [(4, 4, 128), (8, 2, 128), (28, 4, 128), (4, 2, 64), (4, 4, 16), (4, 2, 32),
                                     (6, 2, 96), (4, 2, 160), (4, 4, 208), (2, 1, 256)])
def test_importance_matches_oracle(device, H, Hkv, D):
    _case(device, H, Hkv, D, A=203, mask_counts=[32, 0, 17, 64, 1], shifts=[0, 3, 40, 7, 0], slot0=5, seed=H)


def test_llada_shape_and_accumulation_over_layers(device):
    imp, want, (q, kc, rows, cu, args) = _case(device, 32, 32, 128, A=1000, mask_counts=[256, 200], shifts=[64, 255], seed=3)
    # a second call (the next layer) adds to the same buffer
    ops.affix_importance(imp, q.to(device), kc.to(device), rows.to(device), cu.to(device), 1000, 256, **args)
    assert torch.allclose(imp.cpu()[:, :1000], 2 * want, rtol=2e-3, atol=2e-4)
    # rows of the softmax sum to one
    assert torch.allclose(imp.cpu()[:, :1000].sum(1), 2 * torch.tensor([256.0 * 32, 200.0 * 32]), rtol=1e-4)


def test_no_relocation_f16_and_determinism(device):
    imp1, _, (q, kc, rows, cu, args) = _case(device, 8, 8, 128, A=130, mask_counts=[40, 9], shifts=None, dtype=torch.float16, seed=5)
    imp2 = torch.zeros_like(imp1)
    ops.affix_importance(imp2, q.to(device), kc.to(device), rows.to(device), cu.to(device), 130, 40, **args)
    assert torch.equal(imp1, imp2)                                        # no atomics: bit-identical reruns


def test_mask_rows_outside_q_are_absent_queries(device):
    """A stale or negative mask row must not be read: it counts as no query at all, with and without relocation."""
    for shifts in (None, [9, 2]):
        _, _, (q, kc, rows, cu, args) = _case(device, 8, 2, 128, A=90, mask_counts=[20, 6], shifts=shifts, seed=11)
        clean = torch.zeros(2, 90, dtype=torch.float32, device=device)
        ops.affix_importance(clean, q.to(device), kc.to(device), rows.to(device), cu.to(device), 90, 20, **args)
        # splice three invalid indices into the first request's rows
        bad = torch.cat([rows[:5], torch.tensor([-1, q.shape[0], 2 ** 30], dtype=torch.int32), rows[5:]])
        cu_bad = torch.tensor([0, 23, 29], dtype=torch.int32)
        got = torch.zeros_like(clean)
        ops.affix_importance(got, q.to(device), kc.to(device), bad.to(device), cu_bad.to(device), 90, 23, **args)
        assert torch.allclose(got, clean, rtol=1e-5, atol=1e-6)   # same rows, another tiling of them


def test_row_counts_beyond_the_declared_sizes_are_cut(device):
    """The prefix sums are device memory the host cannot check: a request that claims more mask rows than the
    index tensor holds, or than `max_mask_rows` says, is cut to what was declared."""
    _, _, (q, kc, rows, cu, args) = _case(device, 8, 2, 128, A=90, mask_counts=[20, 6], shifts=[9, 2], seed=12)
    clean = torch.zeros(2, 90, dtype=torch.float32, device=device)
    ops.affix_importance(clean, q.to(device), kc.to(device), rows.to(device), cu.to(device), 90, 20, **args)
    got = torch.zeros_like(clean)
    claims_too_many = torch.tensor([0, 20, 40], dtype=torch.int32, device=device)   # 26 rows exist
    ops.affix_importance(got, q.to(device), kc.to(device), rows.to(device), claims_too_many, 90, 20, **args)
    assert torch.equal(got, clean)
    # max_mask_rows = 6: the first request is scored on its first 6 rows only, the second is unchanged
    short = torch.zeros_like(clean)
    ops.affix_importance(short, q.to(device), kc.to(device), rows.to(device), cu.to(device), 90, 6, **args)
    first6 = torch.zeros_like(clean)
    cu6 = torch.tensor([0, 6, 6], dtype=torch.int32, device=device)
    ops.affix_importance(first6, q.to(device), kc.to(device), rows.to(device), cu6, 90, 6, **args)
    assert torch.equal(short[1], clean[1])
    assert torch.allclose(short[0], first6[0], rtol=1e-6, atol=1e-7)


def test_argument_errors(device):
    q = torch.zeros(4, 2, 128, dtype=torch.bfloat16, device=device)
    kc = torch.zeros(8, 2, 128, dtype=torch.bfloat16, device=device)
    imp = torch.zeros(1, 8, device=device)
    rows = torch.tensor([0, 1], dtype=torch.int32, device=device)
    cu = torch.tensor([0, 2], dtype=torch.int32, device=device)
    with pytest.raises(ValueError, match="outside"):
        ops.affix_importance(imp, q, kc, rows, cu, 8, 2, affix_slot0=4)
    with pytest.raises(ValueError, match="requires shifts and RoPE tables"):
        ops.affix_importance(imp, q, kc, rows, cu, 8, 2, affix_shifts=torch.zeros(1, dtype=torch.int32, device=device))
    with pytest.raises(AssertionError):
        ops.affix_importance(imp, q, kc, rows, cu, 8, 2, workspace=torch.empty(8, dtype=torch.uint8, device=device))
