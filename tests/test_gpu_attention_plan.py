"""acache_varlen_attn_planned: a dispatch plan changes the order the (request, query tile, head) units run in and
nothing else, so the planned call must give the bits of the unplanned one in every relocation mode, head layout and
dtype; against the CPU oracle it keeps the 2e-2 bound; a plan made for other lengths is harmless."""
import pytest
import torch

from acache_amd import ops
from acache_amd.synthetic import attention_batch
from oracle import acache_oracle as O

pytestmark = pytest.mark.gpu


def _batch(seed, B, H, Hkv, D, dtype, mode, device, A=200):
    """Ragged requests; in the relocation modes each holds A shared rows (slots 0..A-1): an infix after a0 private
    keys (key side), or in front of the private keys with the shift handed to the queries (query side)."""
    g = torch.Generator().manual_seed(seed)
    q_lens = torch.randint(1, 420, (B,), generator=g).tolist()
    tails = torch.randint(0, 1500, (B,), generator=g).tolist()
    starts = torch.randint(0, 60, (B,), generator=g).tolist()
    S = 256 * ((A + sum(starts) + sum(tails) + 255) // 256 + 1)
    reads, nxt = [], A
    for a0, tail in zip(starts, tails):
        private = list(range(nxt, nxt + a0 + tail))
        nxt += a0 + tail
        if mode == "plain":
            reads.append(private)
        elif mode == "key":
            reads.append(private[:a0] + list(range(A)) + private[a0:])
        else:
            reads.append(list(range(A)) + private)
    kv_lens = [len(r) for r in reads]
    cu = lambda lens: torch.tensor([0] + torch.tensor(lens).cumsum(0).tolist(), dtype=torch.int32)
    t = dict(q=(torch.randn(sum(q_lens), H, D, generator=g) / D ** 0.25).to(dtype),
             kc=(torch.randn(S, Hkv, D, generator=g) / D ** 0.25).to(dtype),
             vc=torch.randn(S, Hkv, D, generator=g).to(dtype),
             cu_q=cu(q_lens), cu_k=cu(kv_lens), slots=torch.tensor(sum(reads, []), dtype=torch.int32))
    kw = {}
    if mode != "plain":
        cos, sin = O.rope_table(4096, D, 5e5)
        kw = dict(shared_prefix_len=A, affix_shifts=torch.tensor(starts, dtype=torch.int32), rope_cos=cos, rope_sin=sin)
        if mode == "query":
            kw["shared_kv_lens"] = torch.full((B,), A, dtype=torch.int32)
    return t, kw


def _run(t, kw, device, plan=None):
    dev = lambda x: x.to(device) if torch.is_tensor(x) else x
    Hkv, D = t["kc"].shape[1:]
    return ops.acache_attention(dev(t["q"]), dev(t["kc"]).view(-1, 256, Hkv, D), dev(t["vc"]).view(-1, 256, Hkv, D),
                                dev(t["cu_q"]), dev(t["cu_k"]), dev(t["slots"]), **{k: dev(v) for k, v in kw.items()},
                                plan=plan)


@pytest.mark.parametrize("mode", ["plain", "key", "query"])
@pytest.mark.parametrize("H,Hkv,D,dtype", [(32, 8, 128, torch.bfloat16), (32, 32, 128, torch.bfloat16),
                                           (28, 4, 128, torch.float16), (8, 2, 64, torch.bfloat16),
                                           (12, 12, 64, torch.float16), (6, 1, 128, torch.bfloat16)])
def test_planned_call_gives_the_bits_of_the_unplanned_one(device, mode, H, Hkv, D, dtype):
    t, kw = _batch(H * 7 + Hkv, 14, H, Hkv, D, dtype, mode, device)
    # 8 slots per XCD puts every layout in the packing range (more units than slots, at most sixteen per slot)
    for slots in (8, None):
        plan = ops.attention_plan(t["cu_q"], t["cu_k"], H, Hkv, device, slots_per_xcd=slots)
        assert plan.shape[0] > 0 and plan.shape[0] % 8 == 0
        assert torch.equal(_run(t, kw, device, plan), _run(t, kw, device))


@pytest.mark.parametrize("B", [70, 150])
def test_more_than_64_requests(device, B):
    """Above 64 requests the unplanned kernel walks the requests in batch order; a plan orders any batch."""
    t, kw = _batch(B, B, 8, 8, 128, torch.bfloat16, "query", device, A=64)
    plan = ops.attention_plan(t["cu_q"], t["cu_k"], 8, 8, device)
    assert torch.equal(_run(t, kw, device, plan), _run(t, kw, device))


def test_planned_call_against_the_oracle(device):
    t, kw = _batch(5, 6, 4, 2, 128, torch.bfloat16, "key", device)
    plan = ops.attention_plan(t["cu_q"], t["cu_k"], 4, 2, device, slots_per_xcd=2)
    got = _run(t, kw, device, plan)
    want = O.acache_attention(t["q"], t["kc"], t["vc"], t["cu_q"], t["cu_k"], t["slots"], **kw)
    assert (got.float().cpu() - want.float()).abs().max().item() <= 2e-2


def test_benchmark_batch_all_heads(device):
    w = attention_batch(seed=0)
    H, D, BS = 32, 128, 256
    g = torch.Generator(device=device).manual_seed(0)
    q = (torch.randn(int(w["cu_q"][-1]), H, D, generator=g, device=device) / D ** 0.5).to(torch.bfloat16)
    kc = (torch.randn(w["num_blocks"], BS, H, D, generator=g, device=device) / D ** 0.5).to(torch.bfloat16)
    vc = (torch.randn(w["num_blocks"], BS, H, D, generator=g, device=device) / D ** 0.5).to(torch.bfloat16)
    cu_q, cu_k, slots = (w[k].to(device) for k in ("cu_q", "cu_k", "slot_map"))
    plan = ops.attention_plan(w["cu_q"], w["cu_k"], H, H, device)
    assert plan.shape == (1088, 2)
    assert torch.equal(ops.acache_attention(q, kc, vc, cu_q, cu_k, slots, plan=plan),
                       ops.acache_attention(q, kc, vc, cu_q, cu_k, slots))


def test_a_plan_for_other_lengths_is_harmless(device):
    """Entries that name a request, head or tile the call does not have are skipped: with a plan made for three
    requests, a call on the first two gives the result of the unplanned call."""
    t, kw = _batch(9, 3, 8, 8, 128, torch.bfloat16, "plain", device)
    plan = ops.attention_plan(t["cu_q"], t["cu_k"], 8, 8, device, slots_per_xcd=2)
    two = dict(t, cu_q=t["cu_q"][:3], cu_k=t["cu_k"][:3], q=t["q"][: int(t["cu_q"][2])],
               slots=t["slots"][: int(t["cu_k"][2])])
    assert torch.equal(_run(two, kw, device, plan), _run(two, kw, device))
    # sixteen heads in the plan, eight in the call
    plan16 = ops.attention_plan(two["cu_q"], two["cu_k"], 16, 8, device)
    assert torch.equal(_run(two, kw, device, plan16), _run(two, kw, device))
    with pytest.raises(Exception):
        ops.attention_plan([0, 5], [0, 5], 8, 3, device)                # 3 KV heads do not divide 8 heads


def test_other_head_dims_ignore_the_plan(device):
    t, kw = _batch(11, 5, 8, 8, 96, torch.bfloat16, "plain", device)
    plan = ops.attention_plan(t["cu_q"], t["cu_k"], 8, 8, device, slots_per_xcd=2)
    assert torch.equal(_run(t, kw, device, plan), _run(t, kw, device))
