"""Parity of the HIP relocate/RoPE/gather and materialise kernels against the CPU oracle.

Called through the package's ops, i.e. through the C ABI.  Bit-exact for bf16,
fp16-free here; fp32 rows bit-exact too (same separately-rounded fp32 products and sum).
"""
import pytest
import torch

from acache_amd import ops
from oracle import acache_oracle as O
from acache_amd.synthetic import ragged_relocation_batch

pytestmark = pytest.mark.gpu


def _bits(t):
    return t.contiguous().view(torch.int16) if t.element_size() == 2 else t.contiguous().view(torch.int32)


def test_reference_materialize_geometry_bit_exact(device):
    """tests/test_attention_kernels.py:127-165: L=2, 24 slots, Hkv=2, D=64, A=7, shift=5, dst=12, bf16, fp32 tables."""
    torch.manual_seed(0)
    L, S, H, D, A, shift, dst = 2, 24, 2, 64, 7, 5, 12
    k = torch.randn(L, S, H, D).to(torch.bfloat16)
    v = torch.randn_like(k)
    cos, sin = O.rope_table(S, D)
    ek, ev = k.clone(), v.clone()
    O.materialize_relocated_affix(ek, ev, cos, sin, dst, A, shift)
    gk, gv = k.to(device), v.to(device)
    ops.materialize_relocated_affix(gk, gv, cos.to(device), sin.to(device), dst, A, shift)
    torch.cuda.synchronize()
    assert torch.equal(_bits(gk.cpu()), _bits(ek))
    assert torch.equal(_bits(gv.cpu()), _bits(ev))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("H,D", [(32, 128), (4, 128), (2, 64), (3, 128)])
def test_relocate_gather_small_bit_exact(device, dtype, H, D):
    torch.manual_seed(1)
    L, S, T = 3, 300, 211
    cos, sin = O.rope_table(400, D, 5e5)
    k = torch.randn(L, S, H, D).to(dtype)
    v = torch.randn(L, S, H, D).to(dtype)
    slot = torch.randint(0, S, (T,), dtype=torch.int32)
    delta = torch.randint(-399, 400, (T,), dtype=torch.int32)
    delta[::4] = 0
    ek, ev = O.relocate_rope_gather(k, v, slot, delta, cos, sin)
    gk, gv = ops.relocate_rope_gather(k.to(device), v.to(device), slot.to(device), delta.to(device),
                                      cos.to(device), sin.to(device))
    torch.cuda.synchronize()
    assert torch.equal(_bits(gk.cpu()), _bits(ek))
    assert torch.equal(_bits(gv.cpu()), _bits(ev))


@pytest.mark.parametrize("dtype,H,D", [(torch.bfloat16, 2, 160), (torch.float16, 5, 96), (torch.float32, 3, 40),
                                       (torch.bfloat16, 1, 16), (torch.bfloat16, 4, 256), (torch.float32, 2, 72)])
def test_relocate_gather_other_head_dims_bit_exact(device, dtype, H, D):
    """Head dims other than 64 / 128 (the reference takes any width: acache_attention.py:100-101) go through the
    kernel with the row geometry in registers; same lane layout, same arithmetic, same bits.  Also the in-place
    materialise form and out-of-range rows."""
    torch.manual_seed(D)
    L, S, T = 2, 90, 77
    cos, sin = O.rope_table(128, D, 1e4)
    k = torch.randn(L, S, H, D).to(dtype)
    v = torch.randn(L, S, H, D).to(dtype)
    slot = torch.randint(0, S, (T,), dtype=torch.int32)
    delta = torch.randint(-127, 128, (T,), dtype=torch.int32)
    delta[::5] = 0
    ek, ev = O.relocate_rope_gather(k, v, slot, delta, cos, sin)
    gk, gv = ops.relocate_rope_gather(k.to(device), v.to(device), slot.to(device), delta.to(device),
                                      cos.to(device), sin.to(device))
    assert torch.equal(_bits(gk.cpu()), _bits(ek))
    assert torch.equal(_bits(gv.cpu()), _bits(ev))
    bad = slot.clone()
    bad[1], bad[2] = -1, S
    gk, gv = ops.relocate_rope_gather(k.to(device), v.to(device), bad.to(device), delta.to(device),
                                      cos.to(device), sin.to(device))
    assert torch.all(gk[:, 1:3] == 0) and torch.all(gv[:, 1:3] == 0)
    assert torch.equal(_bits(gk[:, 3:].cpu()), _bits(ek[:, 3:]))
    mk, mv = k.clone(), v.clone()
    O.materialize_relocated_affix(mk, mv, cos, sin, 40, 33, 21)
    dk, dv = k.to(device), v.to(device)
    ops.materialize_relocated_affix(dk, dv, cos.to(device), sin.to(device), 40, 33, 21)
    assert torch.equal(_bits(dk.cpu()), _bits(mk)) and torch.equal(_bits(dv.cpu()), _bits(mv))


def test_pure_gather_and_out_of_range_rows(device):
    torch.manual_seed(2)
    L, S, H, D, T = 2, 64, 4, 128, 40
    k = torch.randn(L, S, H, D).to(torch.bfloat16)
    v = torch.randn(L, S, H, D).to(torch.bfloat16)
    slot = torch.randint(0, S, (T,), dtype=torch.int32)
    gk, gv = ops.relocate_rope_gather(k.to(device), v.to(device), slot.to(device))
    assert torch.equal(_bits(gk.cpu()), _bits(k[:, slot.long()]))
    assert torch.equal(_bits(gv.cpu()), _bits(v[:, slot.long()]))
    # slots outside the cache and shifts beyond the table give zero rows, never a fault
    cos, sin = O.rope_table(16, D)
    bad_slot = slot.clone()
    bad_slot[3], bad_slot[7] = -1, S
    delta = torch.zeros(T, dtype=torch.int32)
    delta[5], delta[9] = 16, -99
    gk, gv = ops.relocate_rope_gather(k.to(device), v.to(device), bad_slot.to(device), delta.to(device),
                                      cos.to(device), sin.to(device))
    gk, gv = gk.cpu(), gv.cpu()
    for t in (3, 7, 5, 9):
        assert torch.all(gk[:, t] == 0) and torch.all(gv[:, t] == 0)
    ok = [t for t in range(T) if t not in (3, 7, 5, 9)]
    assert torch.equal(_bits(gk[:, ok]), _bits(k[:, slot[ok].long()]))


def test_empty_input(device):
    k = torch.zeros(2, 8, 2, 64, dtype=torch.bfloat16, device=device)
    gk, gv = ops.relocate_rope_gather(k, k.clone(), torch.zeros(0, dtype=torch.int32, device=device))
    assert gk.shape == (2, 0, 2, 64)


def test_cpu_reference_config_fp32_llada_layer_shape(device):
    """The fp32 configuration at its full size: 32 layers x 32 KV heads x 128, A = 512 affix rows moved to rows
    384..895 (shift +384, theta 5e5), identity block table, 256-token blocks, 384 private request rows in further
    blocks.  One launch over all layers on the device, checked bit for bit against the oracle four layers at a time."""
    g = torch.Generator().manual_seed(0)
    L, H, D, A, shift, BS = 32, 32, 128, 512, 384, 256
    nblocks = 4
    k = torch.randn(L, nblocks, BS, H, D, generator=g)
    v = torch.randn(L, nblocks, BS, H, D, generator=g)
    cos, sin = O.rope_table(896, D, 5e5)
    slot = torch.cat([torch.arange(2 * BS, 2 * BS + 384), torch.arange(A)]).to(torch.int32)
    delta = torch.cat([torch.zeros(384), torch.full((A,), shift)]).to(torch.int32)
    gk, gv = ops.relocate_rope_gather(k.to(device), v.to(device), slot.to(device), delta.to(device),
                                      cos.to(device), sin.to(device))
    assert gk.shape == (L, 896, H, D)
    gk, gv = gk.cpu(), gv.cpu()
    for l in range(0, L, 4):
        ek, ev = O.relocate_rope_gather(k[l:l + 4], v[l:l + 4], slot, delta, cos, sin)
        assert torch.equal(_bits(gk[l:l + 4]), _bits(ek)), f"keys, layers {l}..{l + 3}"
        assert torch.equal(_bits(gv[l:l + 4]), _bits(ev)), f"values, layers {l}..{l + 3}"
    # closed form: norms of (d, d+64) pairs survive the move
    n0 = gk[:, 384:, :, :64] ** 2 + gk[:, 384:, :, 64:] ** 2
    n1 = k.reshape(L, -1, H, D)[:, :A, :, :64] ** 2 + k.reshape(L, -1, H, D)[:, :A, :, 64:] ** 2
    torch.testing.assert_close(n0, n1, atol=1e-4, rtol=1e-5)


def test_ragged_batch_config_bit_exact_on_two_layers_and_properties_at_full_size(device):
    """The bf16 ragged configuration (16 requests, shuffled block tables, shifts in [-1200, 1200]) on 2 of
    the 32 layers against the oracle, then at more layers through properties that need no oracle."""
    w = ragged_relocation_batch(seed=0)
    H, D, BS = 32, 128, 256
    cos, sin = O.rope_table(1201, D, 5e5)
    g = torch.Generator().manual_seed(0)
    L = 2
    k = torch.randn(L, w["num_blocks"], BS, H, D, generator=g).to(torch.bfloat16)
    v = torch.randn(L, w["num_blocks"], BS, H, D, generator=g).to(torch.bfloat16)
    ek, ev = O.relocate_rope_gather(k, v, w["slot_map"], w["delta"], cos, sin)
    dk, dv = k.to(device), v.to(device)
    slot, delta = w["slot_map"].to(device), w["delta"].to(device)
    dcos, dsin = cos.to(device), sin.to(device)
    gk, gv = ops.relocate_rope_gather(dk, dv, slot, delta, dcos, dsin)
    assert torch.equal(_bits(gk.cpu()), _bits(ek))
    assert torch.equal(_bits(gv.cpu()), _bits(ev))

    # size-independent properties at the full 32 layers (the benchmark's launch), all on device:
    del k, v, ek, ev, dk, dv, gk, gv
    L = 32
    dk = torch.randn(L, w["num_blocks"], BS, H, D, device=device).to(torch.bfloat16)
    dv = torch.randn_like(dk)
    gk, gv = ops.relocate_rope_gather(dk, dv, slot, delta, dcos, dsin)
    flat_k = dk.view(L, -1, H, D)
    flat_v = dv.view(L, -1, H, D)
    # V and the unshifted rows are bit copies
    assert torch.equal(gv, flat_v[:, slot.long()])
    still = (delta == 0).nonzero().squeeze(1)
    assert torch.equal(gk[:, still], flat_k[:, slot[still].long()])
    # rotating back by -delta returns the cached key within 2 bf16 roundings
    scratch_slots = torch.arange(slot.numel(), dtype=torch.int32, device=device)
    bk, _ = ops.relocate_rope_gather(gk, gv, scratch_slots, -delta, dcos, dsin)
    for l in range(0, L, 8):                      # fp32 views of 8 layers at a time
        orig = flat_k[l:l + 8, slot.long()].float()
        err = (bk[l:l + 8].float() - orig).abs()
        assert err.max().item() <= 2 ** -7 * 1.5 * orig.abs().max().item()
        # pair norms are preserved up to bf16 rounding
        n0 = orig[..., :64] ** 2 + orig[..., 64:] ** 2
        rot = gk[l:l + 8].float()
        n1 = rot[..., :64] ** 2 + rot[..., 64:] ** 2
        assert ((n0 - n1).abs() <= 0.02 * n0 + 1e-3).all()
        del orig, err, n0, n1, rot
    # linearity of the rotation: rot(x) + rot(y) == rot(x + y) up to bf16 rounding of the three results
    x, y = flat_k[0, slot.long()].float(), flat_k[1, slot.long()].float()
    sk = (x + y).to(torch.bfloat16)[None]
    rs, _ = ops.relocate_rope_gather(sk, sk, scratch_slots, delta, dcos, dsin)
    lhs = gk[0].float() + gk[1].float()
    assert ((rs[0].float() - lhs).abs() <= 2 ** -6 * (x.abs() + y.abs()).amax(dim=-1, keepdim=True) + 1e-3).all()


def test_materialize_all_layers_llada_shape_matches_gather_form(device):
    """In-place form over all layers equals the gather form row for row (and rejects overlap)."""
    torch.manual_seed(3)
    L, H, D, BS = 4, 32, 128, 256
    A, shift = 1000, 137
    nblk = 9
    k = torch.randn(L, nblk * BS, H, D, device=device).to(torch.bfloat16)
    v = torch.randn_like(k)
    cos, sin = (t.to(device) for t in O.rope_table(2048, D, 5e5))
    dst = 4 * BS
    slot = torch.arange(A, dtype=torch.int32, device=device)
    delta = torch.full((A,), shift, dtype=torch.int32, device=device)
    ek, ev = ops.relocate_rope_gather(k, v, slot, delta, cos, sin)
    k0 = k.clone()
    ops.materialize_relocated_affix(k, v, cos, sin, dst, A, shift)
    assert torch.equal(k[:, dst:dst + A], ek) and torch.equal(v[:, dst:dst + A], ev)
    keep = torch.ones(nblk * BS, dtype=torch.bool, device=device)
    keep[dst:dst + A] = False
    assert torch.equal(k[:, keep], k0[:, keep])
    with pytest.raises(ValueError, match="overlap"):
        ops.materialize_relocated_affix(k, v, cos, sin, A - 1, A, shift)
    with pytest.raises(ValueError):
        ops.materialize_relocated_affix(k, v, cos, sin, nblk * BS - 10, A, shift)
