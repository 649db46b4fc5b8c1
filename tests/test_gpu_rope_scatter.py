"""Parity of the fused rotary + K/V scatter launch against the CPU oracle: bit-exact for bf16, fp16 and fp32."""
import pytest
import torch

from acache_amd import ops
from oracle import acache_oracle as O

pytestmark = pytest.mark.gpu


def _bits(t):
    return t.contiguous().view(torch.int16 if t.element_size() == 2 else torch.int32)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("H,H_kv,D", [(32, 32, 128), (28, 4, 128), (4, 2, 64), (4, 4, 16), (6, 2, 160), (3, 1, 96), (5, 5, 256)])
def test_rope_qk_scatter_bit_exact(device, dtype, H, H_kv, D):
    g = torch.Generator().manual_seed(0)
    N, NB, BS = 53, 5, 16
    cos, sin = O.rope_table(300, D, 5e5)
    q = torch.randn(N, H, D, generator=g).to(dtype)
    k = torch.randn(N, H_kv, D, generator=g).to(dtype)
    v = torch.randn(N, H_kv, D, generator=g).to(dtype)
    pos = torch.randint(0, 300, (N,), generator=g)
    pos[0], pos[1] = 0, 299
    slot = torch.randperm(NB * BS, generator=g)[:N].to(torch.int32)
    slot[[3, 17]] = -1
    kc = torch.randn(NB, BS, H_kv, D, generator=g).to(dtype)
    vc = torch.randn(NB, BS, H_kv, D, generator=g).to(dtype)
    ek, ev = kc.clone(), vc.clone()
    eq, ekr = O.rope_qk_scatter(q, k, v, pos, cos, sin, ek, ev, slot)
    gq, gk, gkc, gvc = q.to(device), k.to(device), kc.to(device), vc.to(device)
    ops.rope_qk_scatter(gq, gk, v.to(device), pos.to(device), cos.to(device), sin.to(device), gkc, gvc, slot.to(device))
    assert torch.equal(_bits(gq.cpu()), _bits(eq)), "rotated q"
    assert torch.equal(_bits(gk.cpu()), _bits(ekr)), "rotated k"
    assert torch.equal(_bits(gkc.cpu()), _bits(ek)), "k cache"
    assert torch.equal(_bits(gvc.cpu()), _bits(ev)), "v cache"


def test_rope_qk_scatter_on_views_of_a_fused_projection(device):
    """q, k, v as column slices of one [N, (H + 2 H_kv) D] projection; batched [B, L] positions flattened."""
    g = torch.Generator().manual_seed(1)
    B, L, H, H_kv, D = 3, 8, 8, 2, 128
    N = B * L
    cos, sin = O.rope_table(64, D, 1e4)
    fused = torch.randn(N, (H + 2 * H_kv) * D, generator=g).to(torch.bfloat16)
    q, k, v = fused[:, :H * D].view(N, H, D), fused[:, H * D:(H + H_kv) * D].view(N, H_kv, D), fused[:, (H + H_kv) * D:].view(N, H_kv, D)
    pos = (torch.tensor([5, 20, 40])[:, None] + torch.arange(L)[None, :]).reshape(-1)
    slot = torch.randperm(64, generator=g)[:N].to(torch.int32)
    kc = torch.zeros(4, 16, H_kv, D, dtype=torch.bfloat16)
    vc = torch.zeros_like(kc)
    ek, ev = kc.clone(), vc.clone()
    eq, ekr = O.rope_qk_scatter(q.contiguous(), k.contiguous(), v.contiguous(), pos, cos, sin, ek, ev, slot)
    dev_fused = fused.to(device)
    dq = dev_fused[:, :H * D].view(N, H, D)
    dk = dev_fused[:, H * D:(H + H_kv) * D].view(N, H_kv, D)
    dv = dev_fused[:, (H + H_kv) * D:].view(N, H_kv, D)
    gkc, gvc = kc.to(device), vc.to(device)
    ops.rope_qk_scatter(dq, dk, dv, pos.to(device), cos.to(device), sin.to(device), gkc, gvc, slot.to(device))
    assert torch.equal(_bits(dq.cpu()), _bits(eq)) and torch.equal(_bits(dk.cpu()), _bits(ekr))
    assert torch.equal(_bits(gkc.cpu()), _bits(ek)) and torch.equal(_bits(gvc.cpu()), _bits(ev))
    assert torch.equal(_bits(dv.cpu()), _bits(v))           # v itself is only read


def test_rope_only_and_out_of_table_positions(device):
    g = torch.Generator().manual_seed(2)
    N, H, D = 9, 4, 128
    cos, sin = O.rope_table(32, D, 1e4)
    q = torch.randn(N, H, D, generator=g).to(torch.bfloat16)
    k = torch.randn(N, H, D, generator=g).to(torch.bfloat16)
    pos = torch.tensor([0, 1, 31, 32, 1000, -1, 7, 8, 9])
    inside = (pos >= 0) & (pos < 32)
    eq, ek = q.clone(), k.clone()
    rq, rk = O.rope_qk_scatter(q[inside], k[inside], None, pos[inside], cos, sin)
    eq[inside], ek[inside] = rq, rk                          # rows outside the table stay as they are
    gq, gk = q.to(device), k.to(device)
    ops.rope_qk_scatter(gq, gk, None, pos.to(device), cos.to(device), sin.to(device))
    assert torch.equal(_bits(gq.cpu()), _bits(eq)) and torch.equal(_bits(gk.cpu()), _bits(ek))
    ops.rope_qk_scatter(gq[:0], gk[:0], None, pos[:0].to(device), cos.to(device), sin.to(device))   # empty: no launch
