"""acache_affix_importance_noalloc (scratch in a fixed device array inside the library) against
acache_affix_importance (caller workspace): the same kernels on the same inputs, so the results must be
bit-identical.  Two calls in a row share the array, the second on a smaller input."""
import pytest
import torch

from acache_amd import _lib, ops
from oracle import acache_oracle as O

pytestmark = pytest.mark.gpu


def _inputs(device, H, Hkv, D, A, mask_counts, shifts, seed):
    g = torch.Generator().manual_seed(seed)
    S = A + 9
    kc = (torch.randn(S, Hkv, D, generator=g) / D ** 0.25).to(torch.bfloat16).to(device)
    Tq = sum(mask_counts) + 11
    q = (torch.randn(Tq, H, D, generator=g) / D ** 0.25).to(torch.bfloat16).to(device)
    rows = torch.randperm(Tq, generator=g)[:sum(mask_counts)].sort().values.to(torch.int32).to(device)
    cu = torch.tensor([0] + torch.tensor(mask_counts).cumsum(0).tolist(), dtype=torch.int32, device=device)
    kw = {}
    if shifts is not None:
        cos, sin = O.rope_table(max(shifts) + 2, D, 5e5)
        kw = dict(affix_shifts=torch.tensor(shifts, dtype=torch.int32, device=device), rope_cos=cos.to(device),
                  rope_sin=sin.to(device))
    return q, kc, rows, cu, A, max(mask_counts), kw


def _both(device, *case):
    q, kc, rows, cu, A, max_rows, kw = _inputs(device, *case)
    B = cu.numel() - 1
    want = torch.zeros(B, A, dtype=torch.float32, device=device)
    got = torch.zeros(B, A, dtype=torch.float32, device=device)
    ops.affix_importance(want, q, kc, rows, cu, A, max_rows, **kw)
    before = torch.cuda.memory_allocated(device)
    ops.affix_importance(got, q, kc, rows, cu, A, max_rows, workspace="builtin", **kw)
    assert torch.cuda.memory_allocated(device) == before      # nothing came from torch's allocator either
    torch.cuda.synchronize(device)
    assert torch.equal(got, want)
    assert float(want.sum()) > 0
    return got


def test_two_calls_share_the_builtin_scratch(device):
    # LLaDA head geometry with relocation (the counter-rotated queries live in the scratch too), then a smaller
    # request batch without relocation: stale contents of the first call must not leak into the second
    _both(device, 32, 32, 128, 300, [64, 40, 7], [5, 0, 130], 1)
    _both(device, 8, 2, 128, 70, [9, 0, 3], None, 2)
    # and once more at the first shape: the array is reusable after a smaller call
    _both(device, 32, 32, 128, 300, [64, 40, 7], [5, 0, 130], 3)


def test_oversized_call_is_rejected_before_any_launch(device):
    lib = _lib.load()
    limit = lib.acache_affix_importance_noalloc_max_bytes()
    assert limit == 40 << 20
    q, kc, rows, cu, A, max_rows, kw = _inputs(device, 4, 4, 128, 50, [4], None, 4)
    imp = torch.zeros(1, A, dtype=torch.float32, device=device)
    # claim more mask rows than the array can keep statistics for: rejected from the sizes alone
    too_many = limit // (4 * 4) + 1   # 4 heads x one fp32 statistic per mask row
    rc = lib.acache_affix_importance_noalloc(
        imp.data_ptr(), q.data_ptr(), kc.data_ptr(), rows.data_ptr(), cu.data_ptr(), None, None, None, 0,
        float(128 ** -0.5), A, 0, 1, q.shape[0], too_many, 4, 4, 4, 128, 0, kc.shape[0], imp.stride(0), q.stride(0), q.stride(1),
        kc.stride(0), kc.stride(1), None)
    assert rc == -3 and b"built-in buffer" in lib.acache_last_error()
    torch.cuda.synchronize(device)
    assert float(imp.abs().sum()) == 0
