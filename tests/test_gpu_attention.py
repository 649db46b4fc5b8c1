"""Parity of the MFMA varlen attention against the CPU oracle (fp32 dense softmax attention).

Tolerance: 2e-2 absolute on bf16/fp16 outputs (fp32 accumulate), the bar this build commits to;
the reference's own tests use 5e-2 (nano-vdllm/tests/test_attention_kernels.py:291,368,422,476,546).
"""
import pytest
import torch

from acache_amd import ops
from acache_amd.synthetic import attention_batch
from oracle import acache_oracle as O

pytestmark = pytest.mark.gpu
ATOL = 2e-2


def _close(got, want, atol=ATOL):
    err = (got.float().cpu() - want.float()).abs().max().item()
    assert err <= atol, f"max abs err {err}"


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_reference_effective_kv_geometry(device, dtype):
    """tests/test_attention_kernels.py:479-546: 8 blocks of 8, H=4, Hkv=2, D=64, q=[5,3], kv=[9,6], random slot maps."""
    torch.manual_seed(0)
    H, Hkv, D = 4, 2, 64
    q = torch.randn(8, H, D).to(dtype)
    kc = torch.randn(8, 8, Hkv, D).to(dtype)
    vc = torch.randn(8, 8, Hkv, D).to(dtype)
    maps = torch.cat([torch.randperm(64)[:9], torch.randperm(64)[:6]]).to(torch.int32)
    cu_q = torch.tensor([0, 5, 8], dtype=torch.int32)
    cu_k = torch.tensor([0, 9, 15], dtype=torch.int32)
    want = O.acache_attention(q, kc, vc, cu_q, cu_k, maps)
    got = ops.acache_attention(q.to(device), kc.to(device), vc.to(device), cu_q.to(device), cu_k.to(device),
                               maps.to(device), D ** -0.5)
    _close(got, want)


@pytest.mark.parametrize("H,Hkv,D", [(4, 2, 128), (32, 32, 128), (28, 4, 128), (4, 4, 64), (6, 1, 64)])
def test_ragged_lengths_plain_mode(device, H, Hkv, D):
    torch.manual_seed(1)
    q_lens = [1, 16, 17, 0, 130, 64, 129, 33]
    kv_lens = [1, 63, 64, 40, 65, 300, 128, 0]
    S = 1024
    q = (torch.randn(sum(q_lens), H, D) / D ** 0.25).to(torch.bfloat16)
    kc = (torch.randn(S, Hkv, D) / D ** 0.25).to(torch.bfloat16)
    vc = torch.randn(S, Hkv, D).to(torch.bfloat16)
    slots = torch.cat([torch.randperm(S)[:n] for n in kv_lens]).to(torch.int32)
    cu_q = torch.tensor([0] + list(torch.tensor(q_lens).cumsum(0)), dtype=torch.int32)
    cu_k = torch.tensor([0] + list(torch.tensor(kv_lens).cumsum(0)), dtype=torch.int32)
    want = O.acache_attention(q, kc, vc, cu_q, cu_k, slots)
    got = ops.acache_attention(q.to(device), kc.view(S // 16, 16, Hkv, D).to(device),
                               vc.view(S // 16, 16, Hkv, D).to(device), cu_q.to(device), cu_k.to(device),
                               slots.to(device))
    _close(got, want)
    # the request without keys (last one) is written as zeros, not left uninitialised
    assert torch.all(got[cu_q[7]:cu_q[8]] == 0)


@pytest.mark.parametrize("B", [64, 65, 150])
def test_large_batches_on_both_sides_of_the_block_ordering_switch(device, B):
    """Up to 64 requests the workgroups walk the requests longest first; above that in batch order.  Many requests
    share a key count (ties in the ordering), some have no queries and some no keys."""
    g = torch.Generator().manual_seed(B)
    H, Hkv, D, S = 8, 8, 128, 2048
    q_lens = torch.randint(0, 40, (B,), generator=g).tolist()
    kv_lens = (torch.randint(0, 5, (B,), generator=g) * 48).tolist()     # 0, 48, ..., 192: plenty of ties
    q_lens[3], kv_lens[5] = 0, 0
    q = (torch.randn(sum(q_lens), H, D, generator=g) / D ** 0.25).to(torch.bfloat16)
    kc = (torch.randn(S, Hkv, D, generator=g) / D ** 0.25).to(torch.bfloat16)
    vc = torch.randn(S, Hkv, D, generator=g).to(torch.bfloat16)
    slots = torch.cat([torch.randperm(S, generator=g)[:n] for n in kv_lens]).to(torch.int32)
    cu_q = torch.tensor([0] + torch.tensor(q_lens).cumsum(0).tolist(), dtype=torch.int32)
    cu_k = torch.tensor([0] + torch.tensor(kv_lens).cumsum(0).tolist(), dtype=torch.int32)
    want = O.acache_attention(q, kc, vc, cu_q, cu_k, slots)
    got = ops.acache_attention(q.to(device), kc.view(S // 16, 16, Hkv, D).to(device),
                               vc.view(S // 16, 16, Hkv, D).to(device), cu_q.to(device), cu_k.to(device),
                               slots.to(device))
    _close(got, want)


def test_invariants_on_device(device):
    torch.manual_seed(2)
    H, Hkv, D, S = 8, 2, 128, 2048
    q = torch.randn(70, H, D, device=device).to(torch.bfloat16)
    kc = torch.randn(S, Hkv, D, device=device).to(torch.bfloat16)
    vc = torch.randn(S, Hkv, D, device=device).to(torch.bfloat16)
    slots = torch.randperm(S, device=device)[:777].to(torch.int32)
    cu_q = torch.tensor([0, 70], dtype=torch.int32, device=device)
    cu_k = torch.tensor([0, 777], dtype=torch.int32, device=device)
    out = ops.acache_attention(q, kc, vc, cu_q, cu_k, slots)
    # permuting the keys of a request does not change the result (up to summation order)
    perm = torch.randperm(777, device=device)
    out_p = ops.acache_attention(q, kc, vc, cu_q, cu_k, slots[perm])
    assert (out.float() - out_p.float()).abs().max().item() <= 1e-2
    # constant V rows -> every output row equals that row
    row = torch.randn(1, Hkv, D, device=device).to(torch.bfloat16)
    out_c = ops.acache_attention(q, kc, row.expand(S, -1, -1).contiguous(), cu_q, cu_k, slots)
    want = row[0].repeat_interleave(H // Hkv, 0)[None].expand(70, -1, -1)
    assert (out_c.float() - want.float()).abs().max().item() <= 1e-2
    # a duplicated request gives identical outputs (batch rows are independent)
    cu_q2 = torch.tensor([0, 70, 140], dtype=torch.int32, device=device)
    cu_k2 = torch.tensor([0, 777, 1554], dtype=torch.int32, device=device)
    out2 = ops.acache_attention(torch.cat([q, q]), kc, vc, cu_q2, cu_k2, torch.cat([slots, slots]))
    # every (request, query tile, head) unit walks its key tiles in the same order wherever the request sits in
    # the batch, so the two copies and the single-request call agree bit for bit
    assert torch.equal(out2[:70], out2[70:])
    assert torch.equal(out2[:70], out)
    # ... and the same call gives the same bits every time (fixed merge order, no atomics on data)
    again = ops.acache_attention(torch.cat([q, q]), kc, vc, cu_q2, cu_k2, torch.cat([slots, slots]))
    assert torch.equal(again, out2)
    # strided q (a slice of a fused qkv projection) is accepted
    qkv = torch.randn(70, 3, H, D, device=device).to(torch.bfloat16)
    out_s = ops.acache_attention(qkv[:, 0], kc, vc, cu_q, cu_k, slots)
    out_d = ops.acache_attention(qkv[:, 0].contiguous(), kc, vc, cu_q, cu_k, slots)
    assert torch.equal(out_s, out_d)


def test_key_side_equals_materialised_bitwise_reference_geometry(device):
    """tests/test_attention_kernels.py:168-234: key-side relocation == plain attention over the materialised copy."""
    torch.manual_seed(0)
    S, H, Hkv, D = 32, 4, 2, 64
    q_len, kv_len, a0, A, dst = 5, 13, 7, 3, 24
    q = torch.randn(q_len, H, D, device=device).to(torch.bfloat16)
    kc = torch.randn(1, S, Hkv, D, device=device).to(torch.bfloat16)
    vc = torch.randn_like(kc)
    cos, sin = (t.to(device) for t in O.rope_table(S, D))
    slots = list(range(A, A + kv_len))
    for local, pos in enumerate(range(a0, a0 + A)):
        slots[pos] = local
    cu_q = torch.tensor([0, q_len], dtype=torch.int32, device=device)
    cu_k = torch.tensor([0, kv_len], dtype=torch.int32, device=device)
    shifts = torch.tensor([a0], dtype=torch.int32, device=device)
    key_side = ops.acache_attention(q, kc[0].view(4, 8, Hkv, D), vc[0].view(4, 8, Hkv, D), cu_q, cu_k,
                                    torch.tensor(slots, dtype=torch.int32, device=device),
                                    shared_prefix_len=A, affix_shifts=shifts, rope_cos=cos, rope_sin=sin)
    want = O.acache_attention(q.cpu(), kc[0].cpu(), vc[0].cpu(), cu_q.cpu(), cu_k.cpu(), torch.tensor(slots),
                              shared_prefix_len=A, affix_shifts=shifts.cpu(), rope_cos=cos.cpu(), rope_sin=sin.cpu())
    _close(key_side, want)
    ops.materialize_relocated_affix(kc, vc, cos, sin, dst, A, a0)
    mslots = list(slots)
    for local, pos in enumerate(range(a0, a0 + A)):
        mslots[pos] = dst + local
    materialised = ops.acache_attention(q, kc[0].view(4, 8, Hkv, D), vc[0].view(4, 8, Hkv, D), cu_q, cu_k,
                                        torch.tensor(mslots, dtype=torch.int32, device=device))
    assert torch.equal(materialised, key_side)


def test_large_head_dim_matches_dense_reference(device):
    """tests/test_attention_kernels.py:237-291: head_dim 160 (not a power of two), fp16, 8 blocks of 8, H=4, Hkv=2,
    q=[3,2], kv=[7,5], random slot maps; tolerance 5e-2 there."""
    torch.manual_seed(0)
    H, Hkv, D = 4, 2, 160
    q = torch.randn(5, H, D).to(torch.float16)
    kc = torch.randn(8, 8, Hkv, D).to(torch.float16)
    vc = torch.randn_like(kc)
    maps = torch.cat([torch.randperm(64)[:7], torch.randperm(64)[:5]]).to(torch.int32)
    cu_q = torch.tensor([0, 3, 5], dtype=torch.int32)
    cu_k = torch.tensor([0, 7, 12], dtype=torch.int32)
    want = torch.cat([O.dense_attention_reference(q[a:b], kc.view(-1, Hkv, D)[maps[c:d].long()],
                                                  vc.view(-1, Hkv, D)[maps[c:d].long()], H, Hkv)
                      for (a, b), (c, d) in (((0, 3), (0, 7)), ((3, 5), (7, 12)))])
    got = ops.acache_attention(q.to(device), kc.to(device), vc.to(device), cu_q.to(device), cu_k.to(device),
                               maps.to(device))
    _close(got, want)


@pytest.mark.parametrize("D", [16, 32, 96, 160, 192, 256])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_other_head_dims_all_relocation_modes(device, D, dtype):
    """Every width that is a multiple of 16 up to 256 runs on the padded kernel: plain ragged batch, then an infix
    affix relocated on the key side and on the query side against the oracle, and key side == plain attention over
    the materialised copy, bit for bit."""
    g = torch.Generator().manual_seed(D)
    H, Hkv, S = 6, 2, 512
    q_lens = [1, 17, 0, 70, 64, 33]
    kv_lens = [1, 63, 40, 130, 0, 64]
    q = (torch.randn(sum(q_lens), H, D, generator=g) / D ** 0.25).to(dtype)
    kc = (torch.randn(S, Hkv, D, generator=g) / D ** 0.25).to(dtype)
    vc = torch.randn(S, Hkv, D, generator=g).to(dtype)
    slots = torch.cat([torch.randperm(S, generator=g)[:n] for n in kv_lens]).to(torch.int32)
    cu_q = torch.tensor([0] + torch.tensor(q_lens).cumsum(0).tolist(), dtype=torch.int32)
    cu_k = torch.tensor([0] + torch.tensor(kv_lens).cumsum(0).tolist(), dtype=torch.int32)
    dev = lambda t: None if t is None else t.to(device)
    want = O.acache_attention(q, kc, vc, cu_q, cu_k, slots)
    got = ops.acache_attention(dev(q), dev(kc.view(S // 16, 16, Hkv, D)), dev(vc.view(S // 16, 16, Hkv, D)),
                               dev(cu_q), dev(cu_k), dev(slots))
    _close(got, want)
    assert torch.all(got[cu_q[4]:cu_q[5]] == 0)            # the request without keys

    # infix affix: A shared rows cached at positions 0..A-1, read at a0..a0+A-1, every fifth one an anchor
    A, a0, tail, nq = 90, 37, 50, 45
    cos, sin = O.rope_table(256, D, 1e4)
    anchors = set(range(a0 + 2, a0 + A, 5))
    read, nxt = [], 128
    for pos in range(a0 + A + tail):
        if a0 <= pos < a0 + A and pos not in anchors:
            read.append(pos - a0)
        else:
            read.append(nxt)
            nxt += 1
    q1 = (torch.randn(nq, H, D, generator=g) / D ** 0.25).to(dtype)
    cu_q1 = torch.tensor([0, nq], dtype=torch.int32)
    cu_k1 = torch.tensor([0, len(read)], dtype=torch.int32)
    shifts = torch.tensor([a0], dtype=torch.int32)
    kc4, vc4 = dev(kc.view(S // 16, 16, Hkv, D)), dev(vc.view(S // 16, 16, Hkv, D))
    want = O.acache_attention(q1, kc, vc, cu_q1, cu_k1, torch.tensor(read, dtype=torch.int32), shared_prefix_len=A,
                              affix_shifts=shifts, rope_cos=cos, rope_sin=sin)
    key_side = ops.acache_attention(dev(q1), kc4, vc4, dev(cu_q1), dev(cu_k1),
                                    dev(torch.tensor(read, dtype=torch.int32)), shared_prefix_len=A,
                                    affix_shifts=dev(shifts), rope_cos=dev(cos), rope_sin=dev(sin))
    _close(key_side, want)
    packed, n_shared = O.attention_read_layout(read, 0, A, a0, True)
    query_side = ops.acache_attention(dev(q1), kc4, vc4, dev(cu_q1), dev(cu_k1),
                                      dev(torch.tensor(packed, dtype=torch.int32)), shared_prefix_len=A,
                                      shared_kv_lens=dev(torch.tensor([n_shared], dtype=torch.int32)),
                                      affix_shifts=dev(shifts), rope_cos=dev(cos), rope_sin=dev(sin))
    _close(query_side, want)
    # materialise the affix at slots 300.., then plain attention over the copy
    kl, vl = dev(kc)[None].clone(), dev(vc)[None].clone()
    ops.materialize_relocated_affix(kl, vl, dev(cos), dev(sin), 300, A, a0)
    mread = [300 + s if s < A else s for s in read]
    materialised = ops.acache_attention(dev(q1), kl[0].view(S // 16, 16, Hkv, D), vl[0].view(S // 16, 16, Hkv, D),
                                        dev(cu_q1), dev(cu_k1), dev(torch.tensor(mread, dtype=torch.int32)))
    assert torch.equal(materialised, key_side)


def test_query_side_relocation_reference_geometry(device):
    """tests/test_attention_kernels.py:294-368: keys cached post-RoPE at source positions, shared keys packed
    first, result compared with dense attention over keys rotated at their logical positions (fp16, tol 5e-2 there)."""
    torch.manual_seed(0)
    NB, BS, H, Hkv, D = 2, 8, 4, 2, 64
    q_len, kv_len, a0, shared = 3, 7, 3, 2
    dtype = torch.float16
    q1 = torch.randn(q_len, H, D).to(dtype)
    q = torch.cat([q1, q1])
    raw_k = torch.randn(kv_len, Hkv, D).to(dtype)
    vals = torch.randn_like(raw_k)
    kc = torch.zeros(NB * BS, Hkv, D, dtype=dtype)
    vc = torch.zeros_like(kc)
    cos, sin = O.rope_table(kv_len, D, dtype=dtype)
    mapping = []
    for pos in range(kv_len):
        if a0 <= pos < a0 + shared:
            src, slot = pos - a0, pos - a0
        else:
            src, slot = pos, shared + pos
        kc[slot] = O.apply_rope(raw_k[pos:pos + 1], cos[src:src + 1], sin[src:src + 1])[0]
        vc[slot] = vals[pos]
        mapping.append(slot)
    packed = [s for s in mapping if s < shared] + [s for s in mapping if s >= shared]
    dev = lambda t: t.to(device)
    out = ops.acache_attention(
        dev(q), dev(kc.view(NB, BS, Hkv, D)), dev(vc.view(NB, BS, Hkv, D)),
        dev(torch.tensor([0, q_len, 2 * q_len], dtype=torch.int32)),
        dev(torch.tensor([0, kv_len, 2 * kv_len], dtype=torch.int32)),
        dev(torch.tensor(packed * 2, dtype=torch.int32)),
        shared_prefix_len=shared, shared_kv_lens=dev(torch.tensor([shared, shared], dtype=torch.int32)),
        affix_shifts=dev(torch.tensor([a0, a0], dtype=torch.int32)), rope_cos=dev(cos), rope_sin=dev(sin))
    expected_k = O.apply_rope(raw_k, cos[:kv_len], sin[:kv_len])
    expected = O.dense_attention_reference(q1, expected_k, vals, H, Hkv)
    _close(out, torch.cat([expected, expected]), atol=5e-2)
    assert torch.equal(out[:q_len], out[q_len:])


@pytest.mark.parametrize("mode", ["key", "query"])
def test_relocation_modes_llada_shape(device, mode):
    """Infix affix of 300 shared rows moved by +77 / +130, two requests, 8 heads of the LLaDA layout, against the oracle."""
    torch.manual_seed(3)
    H, Hkv, D, BS = 8, 8, 128, 256
    A = 300
    starts, tails, q_lens = [77, 130], [200, 90], [90, 45]
    S = 6 * BS
    kc = (torch.randn(S, Hkv, D) / D ** 0.25).to(torch.bfloat16)
    vc = torch.randn(S, Hkv, D).to(torch.bfloat16)
    cos, sin = O.rope_table(1024, D, 5e5)
    reads, shared_lens = [], []
    next_private = 2 * BS
    for a0, tail in zip(starts, tails):
        L = a0 + A + tail
        read = []
        anchors = set(range(a0 + 5, a0 + A, 7))
        for pos in range(L):
            if a0 <= pos < a0 + A and pos not in anchors:
                read.append(pos - a0)
            else:
                read.append(next_private)
                next_private += 1
        if mode == "query":
            read, n_shared = O.attention_read_layout(read, 0, A, a0, True)
        else:
            n_shared = 0
        reads.append(read)
        shared_lens.append(n_shared)
    q = (torch.randn(sum(q_lens), H, D) / D ** 0.25).to(torch.bfloat16)
    cu_q = torch.tensor([0, q_lens[0], sum(q_lens)], dtype=torch.int32)
    cu_k = torch.tensor([0, len(reads[0]), len(reads[0]) + len(reads[1])], dtype=torch.int32)
    slots = torch.tensor(reads[0] + reads[1], dtype=torch.int32)
    shifts = torch.tensor(starts, dtype=torch.int32)
    skl = torch.tensor(shared_lens, dtype=torch.int32) if mode == "query" else None
    want = O.acache_attention(q, kc, vc, cu_q, cu_k, slots, shared_prefix_len=A, shared_kv_lens=skl,
                              affix_shifts=shifts, rope_cos=cos, rope_sin=sin)
    dev = lambda t: None if t is None else t.to(device)
    got = ops.acache_attention(dev(q), dev(kc.view(-1, BS, Hkv, D)), dev(vc.view(-1, BS, Hkv, D)), dev(cu_q),
                               dev(cu_k), dev(slots), shared_prefix_len=A, shared_kv_lens=dev(skl),
                               affix_shifts=dev(shifts), rope_cos=dev(cos), rope_sin=dev(sin))
    _close(got, want)


def test_anchor_recompute_config_against_oracle_on_a_head_subset(device):
    """The anchor-recompute configuration (batch 16, q = 20% anchors + 32, kv up to ~1700, shared affix slots +
    shuffled private blocks) with 4 of the 32 heads so the CPU oracle finishes in seconds."""
    w = attention_batch(seed=0)
    H = Hkv = 4
    D, BS = 128, 256
    g = torch.Generator().manual_seed(0)
    S = w["num_blocks"] * BS
    q = (torch.randn(int(w["cu_q"][-1]), H, D, generator=g) / D ** 0.5).to(torch.bfloat16)
    kc = (torch.randn(S, Hkv, D, generator=g) / D ** 0.5).to(torch.bfloat16)
    vc = (torch.randn(S, Hkv, D, generator=g) / D ** 0.5).to(torch.bfloat16)
    want = O.acache_attention(q, kc, vc, w["cu_q"], w["cu_k"], w["slot_map"])
    got = ops.acache_attention(q.to(device), kc.view(-1, BS, Hkv, D).to(device), vc.view(-1, BS, Hkv, D).to(device),
                               w["cu_q"].to(device), w["cu_k"].to(device), w["slot_map"].to(device))
    _close(got, want)


def test_anchor_recompute_config_full_size_against_library_attention_on_device(device):
    """All 32 heads of the anchor-recompute configuration (the benchmark's call): every request against
    F.scaled_dot_product_attention in fp32 on the gathered K/V (a library routine, independent of the oracle), plus
    the properties that need no reference: a duplicated batch gives the same bits, and permuting each request's
    key order changes the result by rounding only."""
    import torch.nn.functional as F
    w = attention_batch(seed=0)
    H = Hkv = 32
    D, BS = 128, 256
    g = torch.Generator(device=device).manual_seed(0)
    S = w["num_blocks"] * BS
    q = (torch.randn(int(w["cu_q"][-1]), H, D, generator=g, device=device) / D ** 0.5).to(torch.bfloat16)
    kc = (torch.randn(S, Hkv, D, generator=g, device=device) / D ** 0.5).to(torch.bfloat16)
    vc = (torch.randn(S, Hkv, D, generator=g, device=device) / D ** 0.5).to(torch.bfloat16)
    cu_q, cu_k, slots = w["cu_q"].to(device), w["cu_k"].to(device), w["slot_map"].to(device)
    kc4, vc4 = kc.view(-1, BS, Hkv, D), vc.view(-1, BS, Hkv, D)
    got = ops.acache_attention(q, kc4, vc4, cu_q, cu_k, slots)
    worst = 0.0
    for b in range(len(w["q_lens"])):
        q0, q1, k0, k1 = int(cu_q[b]), int(cu_q[b + 1]), int(cu_k[b]), int(cu_k[b + 1])
        idx = slots[k0:k1].long()
        want = F.scaled_dot_product_attention(q[q0:q1].float().transpose(0, 1), kc[idx].float().transpose(0, 1),
                                              vc[idx].float().transpose(0, 1)).transpose(0, 1)
        worst = max(worst, (got[q0:q1].float() - want).abs().max().item())
    assert worst <= ATOL, worst
    assert torch.equal(ops.acache_attention(q, kc4, vc4, cu_q, cu_k, slots), got)
    perm = torch.cat([int(cu_k[b]) + torch.randperm(int(cu_k[b + 1] - cu_k[b]), device=device)
                      for b in range(len(w["q_lens"]))])
    got_p = ops.acache_attention(q, kc4, vc4, cu_q, cu_k, slots[perm])
    assert (got_p.float() - got.float()).abs().max().item() <= 4e-3


def test_wide_slot_pitch_takes_the_64_bit_copy_addresses(device):
    """The copies address a compact cache (less than 4 GiB, slot pitch below 2^24 bytes) with 32-bit offsets from a
    scalar base and anything else with 64-bit addresses.  A cache whose slots lie 16 MiB apart takes the second
    form; its result must be the same bits as that of the same rows in a compact cache."""
    torch.manual_seed(5)
    H = Hkv = 8
    D, S = 128, 24
    pitch = 1 << 23   # elements: 16 MiB per slot
    q_lens, kv_lens = [70, 33], [S, S - 5]
    cu_q = torch.tensor([0, 70, 103], dtype=torch.int32, device=device)
    cu_k = torch.tensor([0, S, 2 * S - 5], dtype=torch.int32, device=device)
    slots = torch.cat([torch.randperm(S), torch.randperm(S)[:S - 5]]).to(torch.int32).to(device)
    q = (torch.randn(103, H, D, device=device) / D ** 0.5).to(torch.bfloat16)
    kc = (torch.randn(S, Hkv, D, device=device) / D ** 0.5).to(torch.bfloat16)
    vc = torch.randn(S, Hkv, D, device=device).to(torch.bfloat16)
    wide_k = torch.zeros(S * pitch, dtype=torch.bfloat16, device=device).as_strided((S, Hkv, D), (pitch, D, 1))
    wide_v = torch.zeros(S * pitch, dtype=torch.bfloat16, device=device).as_strided((S, Hkv, D), (pitch, D, 1))
    wide_k.copy_(kc)
    wide_v.copy_(vc)
    compact = ops.acache_attention(q, kc, vc, cu_q, cu_k, slots)
    wide = ops.acache_attention(q, wide_k, wide_v, cu_q, cu_k, slots)
    assert torch.equal(compact, wide)
    want = O.acache_attention(q.cpu(), kc.cpu(), vc.cpu(), cu_q.cpu(), cu_k.cpu(), slots.cpu())
    _close(compact, want)


def test_block_table_variants(device):
    """baseline_ragged_attention / baseline_decode_attention geometry of tests/test_attention_kernels.py:371-476,
    checked against dense attention over the un-paged K/V."""
    torch.manual_seed(4)
    H, Hkv, D, BS = 4, 2, 64, 8
    lengths = [7, 5]
    k = torch.randn(sum(lengths), Hkv, D).to(torch.float16)
    v = torch.randn_like(k)
    q = torch.randn(sum(lengths), H, D).to(torch.float16)
    nblk = [-(-n // BS) for n in lengths]
    perm = torch.randperm(sum(nblk))
    tables = torch.full((2, max(nblk)), -1, dtype=torch.int32)
    kc = torch.zeros(sum(nblk), BS, Hkv, D, dtype=torch.float16)
    vc = torch.zeros_like(kc)
    off = tok = 0
    for b, n in enumerate(lengths):
        tables[b, :nblk[b]] = perm[off:off + nblk[b]]
        for pos in range(n):
            kc[tables[b, pos // BS], pos % BS] = k[tok + pos]
            vc[tables[b, pos // BS], pos % BS] = v[tok + pos]
        off += nblk[b]
        tok += n
    cu = torch.tensor([0, lengths[0], sum(lengths)], dtype=torch.int32)
    want = torch.cat([O.dense_attention_reference(q[cu[b]:cu[b + 1]], k[cu[b]:cu[b + 1]], v[cu[b]:cu[b + 1]], H, Hkv)
                      for b in range(2)])
    got = ops.baseline_ragged_attention(q.to(device), kc.to(device), vc.to(device), cu.to(device), cu.to(device),
                                        tables.to(device), D ** -0.5)
    _close(got, want)
    # decode form: 4 queries per request against seqlens keys
    qd = torch.randn(2, 4, H, D).to(torch.float16)
    wantd = torch.stack([O.dense_attention_reference(qd[b], k[cu[b]:cu[b + 1]], v[cu[b]:cu[b + 1]], H, Hkv) for b in range(2)])
    gotd = ops.baseline_decode_attention(qd.to(device), kc.to(device), vc.to(device),
                                         torch.tensor(lengths, dtype=torch.int32, device=device), tables.to(device), D ** -0.5)
    assert gotd.shape == (2, 4, H, D)
    _close(gotd, wantd)


def test_relocation_argument_errors(device):
    q = torch.zeros(4, 2, 64, dtype=torch.bfloat16, device=device)
    kc = torch.zeros(2, 8, 2, 64, dtype=torch.bfloat16, device=device)
    cu = torch.tensor([0, 4], dtype=torch.int32, device=device)
    slots = torch.arange(4, dtype=torch.int32, device=device)
    shifts = torch.tensor([1], dtype=torch.int32, device=device)
    with pytest.raises(ValueError, match="requires shifts and RoPE tables"):
        ops.acache_attention(q, kc, kc, cu, cu, slots, shared_prefix_len=2, affix_shifts=shifts)
    cos = torch.ones(8, 64, device=device)
    with pytest.raises(ValueError, match="provided together"):
        ops.acache_attention(q, kc, kc, cu, cu, slots, rope_cos=cos)


@pytest.mark.parametrize("D", [64, 128])
def test_near_ties_among_large_scores(device, D):
    """The head-dim 64 / 128 kernels score q * scale * log2 e, rounded to the cache type once more, where the
    reference scales the fp32 product (acache_attention.py:439, 460, 499).  Here every query is aligned with TWO
    keys, so two scores of magnitude 30 compete and their difference (of order one) decides the output: the case in
    which an error relative to the score's size shows most.  Same bound as everywhere else."""
    g = torch.Generator().manual_seed(11)
    H, S, n_q, n_kv = 4, 512, 90, 300
    kc = torch.randn(S, H, D, generator=g)
    kc = (kc / kc.norm(dim=-1, keepdim=True)).to(torch.bfloat16)              # unit keys
    vc = torch.randn(S, H, D, generator=g).to(torch.bfloat16)
    slots = torch.randperm(S, generator=g)[:n_kv].to(torch.int32)
    first = slots[torch.randint(0, n_kv, (n_q,), generator=g)].long()
    second = slots[torch.randint(0, n_kv, (n_q,), generator=g)].long()
    # 30 / scale along both keys plus noise: both score ~30 (+- 1), every other key ~N(0, 1)
    q = ((kc[first].float() + kc[second].float()) * (30.0 * D ** 0.5) + torch.randn(n_q, H, D, generator=g)).to(torch.bfloat16)
    cu_q = torch.tensor([0, n_q], dtype=torch.int32)
    cu_k = torch.tensor([0, n_kv], dtype=torch.int32)
    want = O.acache_attention(q, kc.view(S // 16, 16, H, D), vc.view(S // 16, 16, H, D), cu_q, cu_k, slots)
    scores = torch.einsum("qhd,khd->hqk", q.float(), kc[slots.long()].float()) * D ** -0.5
    top2 = scores.topk(2, dim=-1).values
    assert top2[..., 1].median().item() > 25.0 and (top2[..., 0] - top2[..., 1]).median().item() < 3.0
    got = ops.acache_attention(q.to(device), kc.view(S // 16, 16, H, D).to(device), vc.view(S // 16, 16, H, D).to(device),
                               cu_q.to(device), cu_k.to(device), slots.to(device))
    _close(got, want)


def test_f16_queries_of_small_magnitude(device):
    """f16: queries of magnitude 1e-3 times the scale land near the bottom of the normal range when they are
    pre-scaled; keys of magnitude 1e2 keep the scores of order one, so lost query bits would show.  Same bound."""
    g = torch.Generator().manual_seed(12)
    H, Hkv, D, S, n_q, n_kv = 4, 2, 128, 512, 70, 260
    q = (torch.randn(n_q, H, D, generator=g) * 1e-3).to(torch.float16)
    kc = (torch.randn(S, Hkv, D, generator=g) * 1e2).to(torch.float16)
    vc = torch.randn(S, Hkv, D, generator=g).to(torch.float16)
    slots = torch.randperm(S, generator=g)[:n_kv].to(torch.int32)
    cu_q = torch.tensor([0, n_q], dtype=torch.int32)
    cu_k = torch.tensor([0, n_kv], dtype=torch.int32)
    want = O.acache_attention(q, kc.view(S // 16, 16, Hkv, D), vc.view(S // 16, 16, Hkv, D), cu_q, cu_k, slots)
    got = ops.acache_attention(q.to(device), kc.view(S // 16, 16, Hkv, D).to(device),
                               vc.view(S // 16, 16, Hkv, D).to(device), cu_q.to(device), cu_k.to(device), slots.to(device))
    assert (q.float().abs().max() * D ** -0.5 * 1.4427).item() < 1e-3      # pre-scaled values: a few 1e-4
    _close(got, want)
