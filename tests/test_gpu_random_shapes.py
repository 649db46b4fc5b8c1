"""Seeded random shapes through the C ABI against the CPU oracle: ragged batches with empty requests, every
relocation mode, MHA and GQA head layouts, tuned and padded head dims, slot maps with holes; and random gathers /
scatters / rotary scatters.  Each case is small enough for the oracle to finish in a fraction of a second."""
import os
import random

import pytest
import torch

from acache_amd import ops
from oracle import acache_oracle as O

pytestmark = pytest.mark.gpu
# more seeds on demand: ACACHE_RANDOM_CASES=400 python -m pytest tests/test_gpu_random_shapes.py -m gpu
CASES = int(os.environ.get("ACACHE_RANDOM_CASES", "24"))


def _bits(t):
    return t.contiguous().view(torch.int16 if t.element_size() == 2 else torch.int32)


@pytest.mark.parametrize("seed", range(CASES))
def test_attention_random_case(device, seed):
    rnd = random.Random(seed)
    g = torch.Generator().manual_seed(seed)
    D = rnd.choice([64, 128, 128, 128, 32, 96, 160])
    Hkv = rnd.choice([1, 2, 4, 8, 3])
    H = Hkv * rnd.choice([1, 1, 2, 7])
    dtype = rnd.choice([torch.bfloat16, torch.float16])
    B = rnd.randint(1, 7)
    mode = rnd.choice(["plain", "key", "query"])
    BS = rnd.choice([8, 16, 256])
    A = rnd.randint(1, 150) if mode != "plain" else 0              # shared affix rows cached at positions 0..A-1
    reads, q_lens, shifts, shared_lens = [], [], [], []
    next_private = -(-max(A, 1) // BS) * BS
    for b in range(B):
        head, tail = rnd.randint(0, 60), rnd.randint(0, 200)
        q_lens.append(rnd.choice([0, 1, 15, 16, 17, 33, 64, 65, 128, 129, 200]))
        if mode == "plain":
            n = rnd.choice([0, 1, 63, 64, 65, head + tail])
            read = list(range(next_private, next_private + n))
            next_private += n
            shared = 0
        else:
            anchors = set(rnd.sample(range(A), rnd.randint(0, A // 2)))
            read = []
            for pos in range(head + A + tail):
                if head <= pos < head + A and pos - head not in anchors:
                    read.append(pos - head)
                else:
                    read.append(next_private)
                    next_private += 1
            shared = 0
            if mode == "query":
                read, shared = O.attention_read_layout(read, 0, A, head, True)
        if read and rnd.random() < 0.3:                              # a hole: a slot outside the cache reads as zeros
            read[rnd.randrange(len(read))] = -1
        reads.append(read)
        shifts.append(head)
        shared_lens.append(shared)
    S = -(-(next_private + 1) // BS) * BS
    kc = (torch.randn(S, Hkv, D, generator=g) / D ** 0.25).to(dtype)
    vc = torch.randn(S, Hkv, D, generator=g).to(dtype)
    q = (torch.randn(sum(q_lens), H, D, generator=g) / D ** 0.25).to(dtype)
    cu_q = torch.tensor([0] + torch.tensor(q_lens).cumsum(0).tolist(), dtype=torch.int32)
    cu_k = torch.tensor([0] + torch.tensor([len(r) for r in reads]).cumsum(0).tolist(), dtype=torch.int32)
    slots = torch.tensor([s for r in reads for s in r], dtype=torch.int32)
    kw = {}
    if mode != "plain":
        cos, sin = O.rope_table(max(shifts) + A + 300, D, 1e4)
        kw = dict(shared_prefix_len=A, affix_shifts=torch.tensor(shifts, dtype=torch.int32), rope_cos=cos, rope_sin=sin)
        if mode == "query":
            kw["shared_kv_lens"] = torch.tensor(shared_lens, dtype=torch.int32)
    if sum(q_lens) == 0:
        return
    # the oracle gathers with plain indexing: point holes at a zero row appended to its copy of the cache
    o_slots = torch.where(slots < 0, torch.full_like(slots, S), slots)
    kz = torch.cat([kc, torch.zeros(1, Hkv, D, dtype=dtype)])
    vz = torch.cat([vc, torch.zeros(1, Hkv, D, dtype=dtype)])
    want = O.acache_attention(q, kz, vz, cu_q, cu_k, o_slots, **kw)
    dev = lambda t: t.to(device) if isinstance(t, torch.Tensor) else t
    got = ops.acache_attention(dev(q), dev(kc.view(S // BS, BS, Hkv, D)), dev(vc.view(S // BS, BS, Hkv, D)), dev(cu_q),
                               dev(cu_k), dev(slots), **{k: dev(v) for k, v in kw.items()})
    live = torch.cat([torch.full((n,), len(reads[b]) > 0) for b, n in enumerate(q_lens)])
    err = (got.float().cpu() - want.float())[live].abs().max().item() if live.any() else 0.0
    assert err <= 2e-2, (seed, mode, D, H, Hkv, dtype, err)
    assert torch.all(got.cpu()[~live] == 0)                         # requests without keys: zeros


@pytest.mark.parametrize("seed", range(max(CASES // 2, 1)))
def test_relocation_scatter_and_rotary_random_case(device, seed):
    rnd = random.Random(100 + seed)
    g = torch.Generator().manual_seed(100 + seed)
    dtype = rnd.choice([torch.bfloat16, torch.float16, torch.float32])
    D = rnd.choice([64, 128, 16, 48, 80, 256])
    H = rnd.randint(1, 9)
    L, S, T = rnd.randint(1, 4), rnd.randint(8, 300), rnd.randint(1, 260)
    cos, sin = O.rope_table(97, D, 5e5)
    k = torch.randn(L, S, H, D, generator=g).to(dtype)
    v = torch.randn(L, S, H, D, generator=g).to(dtype)
    slot = torch.randint(0, S, (T,), generator=g, dtype=torch.int32)
    delta = torch.randint(-96, 97, (T,), generator=g, dtype=torch.int32)
    delta[::3] = 0
    ek, ev = O.relocate_rope_gather(k, v, slot, delta, cos, sin)
    gk, gv = ops.relocate_rope_gather(k.to(device), v.to(device), slot.to(device), delta.to(device),
                                      cos.to(device), sin.to(device))
    assert torch.equal(_bits(gk.cpu()), _bits(ek)) and torch.equal(_bits(gv.cpu()), _bits(ev)), (seed, dtype, D, H)
    # scatter the gathered rows of layer 0 somewhere else and read them back
    dst = torch.randperm(S, generator=g)[:min(T, S)].to(torch.int32)
    dst[::5] = -1
    kc2, vc2 = torch.zeros(S, H, D, dtype=dtype), torch.zeros(S, H, D, dtype=dtype)
    rows = min(T, S)
    O.store_kvcache(ek[0, :rows], ev[0, :rows], kc2, vc2, dst)
    dk, dv = torch.zeros(S, 1, H, D, dtype=dtype, device=device), torch.zeros(S, 1, H, D, dtype=dtype, device=device)
    ops.store_kvcache(gk[0, :rows], gv[0, :rows], dk, dv, dst.to(device))
    assert torch.equal(_bits(dk.cpu().view(S, H, D)), _bits(kc2)) and torch.equal(_bits(dv.cpu().view(S, H, D)), _bits(vc2))
    # rotary + scatter of fresh rows
    Hq = H * rnd.choice([1, 2])
    N = rnd.randint(1, 70)
    q = torch.randn(N, Hq, D, generator=g).to(dtype)
    kk = torch.randn(N, H, D, generator=g).to(dtype)
    vv = torch.randn(N, H, D, generator=g).to(dtype)
    pos = torch.randint(0, 97, (N,), generator=g)
    sl = torch.randperm(S, generator=g)[:N].to(torch.int32) if N <= S else None
    if sl is None:
        return
    sl[::4] = -1
    ek3, ev3 = kc2.clone(), vc2.clone()
    eq, ekr = O.rope_qk_scatter(q, kk, vv, pos, cos, sin, ek3, ev3, sl)
    gq, gkk = q.to(device), kk.to(device)
    ops.rope_qk_scatter(gq, gkk, vv.to(device), pos.to(device), cos.to(device), sin.to(device), dk, dv, sl.to(device))
    assert torch.equal(_bits(gq.cpu()), _bits(eq)) and torch.equal(_bits(gkk.cpu()), _bits(ekr))
    assert torch.equal(_bits(dk.cpu().view(S, H, D)), _bits(ek3)) and torch.equal(_bits(dv.cpu().view(S, H, D)), _bits(ev3))
