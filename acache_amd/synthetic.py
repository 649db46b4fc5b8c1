"""Seeded synthetic inputs shaped like the benchmark configurations (used by bench.py and the tests)."""
from __future__ import annotations

import math

import numpy as np
import torch


def ragged_relocation_batch(seed=0, batch=16, affix=(600, 1200), request=(64, 256), block=256,
                            delta=(-1200, 1200), spare_blocks=4):
    """Per-request affix+request rows through shuffled block tables, per-request shifts on the affix rows.

    Returns dict(slot_map i32[T], delta i32[T], cu_seqlens i32[B+1], num_blocks, block_tables list, A, R).
    Layout per request: affix rows first (shifted by delta_b), then request rows (delta 0).
    """
    rng = np.random.default_rng(seed)
    A = rng.integers(affix[0], affix[1] + 1, batch)
    R = rng.integers(request[0], request[1] + 1, batch)
    lens = A + R
    nblk = -(-lens // block)
    total_blocks = int(nblk.sum()) + spare_blocks
    pool = rng.permutation(total_blocks)
    d = rng.integers(delta[0], delta[1] + 1, batch)
    slot_map, deltas, tables, off = [], [], [], 0
    for b in range(batch):
        bt = pool[off:off + nblk[b]]
        off += nblk[b]
        tables.append(bt.tolist())
        p = np.arange(lens[b])
        slot_map.append(bt[p // block] * block + p % block)
        deltas.append(np.where(p < A[b], d[b], 0))
    cu = np.concatenate([[0], np.cumsum(lens)])
    return dict(
        slot_map=torch.from_numpy(np.concatenate(slot_map).astype(np.int32)),
        delta=torch.from_numpy(np.concatenate(deltas).astype(np.int32)),
        cu_seqlens=torch.from_numpy(cu.astype(np.int32)),
        num_blocks=total_blocks, block_tables=tables, A=A.tolist(), R=R.tolist(), shifts=d.tolist(),
    )


def anchor_batch(seed=0, batch=16, affix=(600, 1200), request=(64, 256), ratio=0.2, tie_frac=0.05):
    """Ragged influence scores |N(0,1)| with injected exact ties, K_b = ceil(ratio*A_b), infix offsets."""
    g = torch.Generator().manual_seed(seed)
    rng = np.random.default_rng(seed)
    A = rng.integers(affix[0], affix[1] + 1, batch)
    R = rng.integers(request[0], request[1] + 1, batch)
    scores = []
    for a in A:
        s = torch.randn(int(a), generator=g).abs()
        n = max(int(tie_frac * a), 1)
        dst = torch.randperm(int(a), generator=g)[:n]
        src = torch.randint(0, int(a), (n,), generator=g)
        s[dst] = s[src]
        scores.append(s)
    K = [min(math.ceil(ratio * int(a)), int(a)) for a in A]
    starts = [int(rng.integers(0, r + 1)) for r in R]
    return dict(scores=scores, A=A.tolist(), R=R.tolist(), K=K, affix_start=starts)


def attention_batch(seed=0, batch=16, affix=(600, 1200), request=(64, 256), gen=256, block_q=32,
                    ratio=0.2, block=256, shared_affix=True):
    """q/kv lengths and a slot map of the anchor-recompute attention call.

    kv_b = A_b + R_b + gen; q_b = ceil(ratio*A_b) + block_q.  With ``shared_affix`` the non-anchor
    affix rows of every request read the shared slots ``[0, A_max)``; everything else reads private
    slots through shuffled block tables placed after the shared blocks.
    """
    rng = np.random.default_rng(seed)
    A = rng.integers(affix[0], affix[1] + 1, batch)
    R = rng.integers(request[0], request[1] + 1, batch)
    K = np.array([min(math.ceil(ratio * int(a)), int(a)) for a in A])
    q = K + block_q
    kv = A + R + gen
    shared_blocks = -(-int(A.max()) // block) if shared_affix else 0
    priv = (K + R + gen) if shared_affix else kv
    nblk = -(-priv // block)
    pool = shared_blocks + rng.permutation(int(nblk.sum()) + 2)
    slot_map, off = [], 0
    for b in range(batch):
        bt = pool[off:off + nblk[b]]
        off += nblk[b]
        p = np.arange(priv[b])
        pslots = bt[p // block] * block + p % block
        if shared_affix:
            anchors = np.sort(rng.choice(A[b], K[b], replace=False))
            read = np.empty(kv[b], dtype=np.int64)
            read[: A[b]] = np.arange(A[b])
            read[anchors] = pslots[: K[b]]
            read[A[b]:] = pslots[K[b]:]
        else:
            read = pslots
        slot_map.append(read)
    return dict(
        q_lens=q.tolist(), kv_lens=kv.tolist(),
        cu_q=torch.from_numpy(np.concatenate([[0], np.cumsum(q)]).astype(np.int32)),
        cu_k=torch.from_numpy(np.concatenate([[0], np.cumsum(kv)]).astype(np.int32)),
        slot_map=torch.from_numpy(np.concatenate(slot_map).astype(np.int32)),
        num_blocks=int(pool.max()) + 1,
    )
