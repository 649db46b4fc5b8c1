"""Parity of the HIP scatter and top-k kernels against the CPU oracle (bit/index exact)."""
import pytest
import torch

from acache_amd import ops
from oracle import acache_oracle as O
from acache_amd.synthetic import anchor_batch

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("H,D", [(4, 128), (32, 128), (2, 64)])
def test_store_kvcache_bit_exact_with_skips(device, dtype, H, D):
    torch.manual_seed(0)
    NB, BS, N = 6, 16, 37
    kc = torch.randn(NB, BS, H, D).to(dtype)
    vc = torch.randn(NB, BS, H, D).to(dtype)
    key = torch.randn(N, H, D).to(dtype)
    val = torch.randn(N, H, D).to(dtype)
    slot = torch.randperm(NB * BS)[:N].to(torch.int32)
    slot[[2, 11]] = -1
    ek, ev = kc.clone(), vc.clone()
    O.store_kvcache(key, val, ek, ev, slot)
    gk, gv = kc.to(device), vc.to(device)
    ops.store_kvcache(key.to(device), val.to(device), gk, gv, slot.to(device))
    assert torch.equal(gk.cpu(), ek) and torch.equal(gv.cpu(), ev)


def test_store_kvcache_strided_source(device):
    """key/value taken as slices of a fused qkv projection: token stride > H*D."""
    torch.manual_seed(1)
    N, H, D = 20, 4, 128
    qkv = torch.randn(N, 3 * H * D, device=device).to(torch.bfloat16)
    key = qkv[:, H * D:2 * H * D].view(N, H, D)
    val = qkv[:, 2 * H * D:].view(N, H, D)
    kc = torch.zeros(2, 32, H, D, dtype=torch.bfloat16, device=device)
    vc = torch.zeros_like(kc)
    slot = torch.randperm(64, device=device)[:N].to(torch.int32)
    ops.store_kvcache(key, val, kc, vc, slot)
    assert torch.equal(kc.view(-1, H, D)[slot.long()], key)
    assert torch.equal(vc.view(-1, H, D)[slot.long()], val)


def test_anchor_config_topk_then_scatter_all_layers(device):
    """GQA shape (28 layers here cut to 4, 4 KV heads, D=128), 16 infix requests, 5% ties, ratio 0.2:
    indices equal the oracle's, anchors land in the first K_b private slots, scatter is a bit copy."""
    w = anchor_batch(seed=0)
    B = len(w["A"])
    scores = torch.cat(w["scores"])
    cu_a = torch.tensor([0] + list(torch.tensor(w["A"]).cumsum(0)), dtype=torch.int32)
    cu_k = torch.tensor([0] + list(torch.tensor(w["K"]).cumsum(0)), dtype=torch.int32)
    offs = torch.tensor(w["affix_start"], dtype=torch.int32)
    got = ops.topk_anchors(scores.to(device), cu_a.to(device), cu_k.to(device), int(cu_k[-1]),
                           offsets=offs.to(device)).cpu()
    assert got.dtype == torch.int64
    for b in range(B):
        want = O.topk_anchors(w["scores"][b], w["K"][b], offset=w["affix_start"][b])
        assert got[cu_k[b]:cu_k[b + 1]].tolist() == want, f"request {b}"
        # value multiset equals torch.topk's (tie order aside)
        vals = torch.topk(w["scores"][b], w["K"][b]).values
        sel = w["scores"][b][got[cu_k[b]:cu_k[b + 1]] - w["affix_start"][b]]
        assert torch.equal(sel.sort(descending=True).values, vals.sort(descending=True).values)
    got32 = ops.topk_anchors(scores.to(device), cu_a.to(device), cu_k.to(device), int(cu_k[-1]),
                             offsets=offs.to(device), out_dtype=torch.int32).cpu()
    assert torch.equal(got32.long(), got)
    low = ops.topk_anchors(scores.to(device), cu_a.to(device), cu_k.to(device), int(cu_k[-1]), largest=False).cpu()
    for b in range(B):
        assert low[cu_k[b]:cu_k[b + 1]].tolist() == O.topk_anchors(w["scores"][b], w["K"][b], largest=False)

    # scatter the recomputed anchor rows of all layers into the first K_b private slots of each request
    L, H, D, BS = 28, 4, 128, 256                       # every layer of the Dream shape, one launch
    nblk = [-(-(k + r) // BS) for k, r in zip(w["K"], w["R"])]
    pool = torch.randperm(sum(nblk) + 8, generator=torch.Generator().manual_seed(1)) + 5
    slots, off = [], 0
    for b in range(B):
        bt = pool[off:off + nblk[b]]
        off += nblk[b]
        p = torch.arange(w["K"][b])
        slots.append(bt[p // BS] * BS + p % BS)
    slots = torch.cat(slots).to(torch.int32)
    S = (int(pool.max()) + 1) * BS
    N = slots.numel()
    g = torch.Generator().manual_seed(2)
    key = torch.randn(L, N, H, D, generator=g).to(torch.bfloat16)
    val = torch.randn(L, N, H, D, generator=g).to(torch.bfloat16)
    kc = torch.randn(L, S // BS, BS, H, D, generator=g).to(torch.bfloat16)
    vc = torch.randn(L, S // BS, BS, H, D, generator=g).to(torch.bfloat16)
    ek, ev = kc.clone(), vc.clone()
    for l in range(L):
        O.store_kvcache(key[l], val[l], ek[l], ev[l], slots)
    gk, gv = kc.to(device), vc.to(device)
    ops.kv_scatter_layers(key.to(device), val.to(device), gk, gv, slots.to(device))
    assert torch.equal(gk.cpu(), ek) and torch.equal(gv.cpu(), ev)
    # gather ∘ scatter = identity
    bk, bv = ops.relocate_rope_gather(gk, gv, slots.to(device))
    assert torch.equal(bk.cpu(), key) and torch.equal(bv.cpu(), val)


def test_topk_edge_cases(device):
    def run(rows, ks, largest=True):
        scores = torch.cat([torch.tensor(r, dtype=torch.float32) for r in rows]) if rows else torch.zeros(0)
        cu_a = torch.tensor([0] + list(torch.tensor([len(r) for r in rows]).cumsum(0)), dtype=torch.int32)
        cu_k = torch.tensor([0] + list(torch.tensor(ks).cumsum(0)), dtype=torch.int32)
        out = ops.topk_anchors(scores.to(device), cu_a.to(device), cu_k.to(device), int(cu_k[-1]), largest=largest).cpu()
        return [out[cu_k[i]:cu_k[i + 1]].tolist() for i in range(len(rows))]

    assert run([[0.5, 0.5, 0.1, 0.9]], [2]) == [[0, 3]]
    assert run([[0.5, 0.5, 0.1, 0.9]], [2], largest=False) == [[0, 2]]
    assert run([[1.0] * 700], [140]) == [list(range(140))]                 # all tied: lowest indices
    assert run([[0.0, -0.0, 1.0, -1.0]], [2], largest=False) == [[0, 3]]   # -0 == +0, lower index wins
    assert run([[3.0, 1.0], [2.0, 5.0, 4.0]], [0, 3]) == [[], [0, 1, 2]]   # K = 0 and K = A
    assert run([[1.0, 2.0]], [4]) == [[0, 1, -1, -1]]                      # K > A: clamped, tail filled with -1
    assert run([[float("nan"), 1.0, float("inf")]], [1]) == [[0]]          # NaN ranks first, as in torch.topk
    big = torch.randn(5000, generator=torch.Generator().manual_seed(3)).tolist()
    assert run([big], [777])[0] == O.topk_anchors(torch.tensor(big), 777)


@pytest.mark.parametrize("mode", ["top", "bottom", "random"])
def test_select_anchor_tokens_mirror(device, mode):
    torch.manual_seed(4)
    s = torch.rand(3, 50, device=device)
    out = ops.select_anchor_tokens(s, 7, mode)
    assert out.shape == (3, 7) and out.dtype == torch.int64
    assert torch.equal(out, out.sort(dim=-1).values)
    if mode != "random":
        for b in range(3):
            assert out[b].tolist() == O.topk_anchors(s[b].cpu(), 7, largest=(mode == "top"))
    with pytest.raises(ValueError):
        ops.select_anchor_tokens(s, -1)
    with pytest.raises(ValueError):
        ops.select_anchor_tokens(s, 3, "middle")
    assert ops.select_anchor_tokens(s, 99, "top").shape == (3, 50)
