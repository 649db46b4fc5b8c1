"""Device-side slot layout against the oracle's restatement of Sequence.finalize_slot_mapping
(nano-vdllm/sequence.py:169-202), which tests/test_host_layout.py pins on the reference's golden vectors: exact."""
import numpy as np
import pytest
import torch

from acache_amd import ops
from oracle import acache_oracle as O

pytestmark = pytest.mark.gpu


def _batch(seed, B, block_size, placement):
    rng = np.random.default_rng(seed)
    lengths, spans, anchors, tables = [], [], [], []
    pool = rng.permutation(4096).tolist()
    for b in range(B):
        A = int(rng.integers(0, 300))
        head = int(rng.integers(0, 120)) if placement != "prefix" else 0
        tail = int(rng.integers(1, 200)) if placement != "suffix" else 0
        n = head + A + tail
        if n == 0:
            n, tail = 1, 1
        K = int(rng.integers(0, A + 1)) if A else 0
        anc = sorted((head + rng.choice(A, K, replace=False)).tolist()) if K else []
        need = -(-(K + n - A) // block_size)
        tables.append([pool.pop() for _ in range(need)])
        lengths.append(n); spans.append((head, head + A)); anchors.append(anc)
    width = max(len(t) for t in tables) + 1
    bt = torch.full((B, width), -1, dtype=torch.int32)
    for b, t in enumerate(tables):
        bt[b, :len(t)] = torch.tensor(t, dtype=torch.int32)
    return lengths, spans, anchors, tables, bt


@pytest.mark.parametrize("placement", ["prefix", "infix", "suffix"])
@pytest.mark.parametrize("block_size", [8, 256])
def test_slot_layout_matches_finalize_slot_mapping(device, placement, block_size):
    lengths, spans, anchors, tables, bt = _batch(7, 19, block_size, placement)
    read, rpos, rslot, cu_len, cu_rec = ops.build_slot_layout(lengths, spans, anchors, bt.to(device), block_size,
                                                               shared_slot_offset=3)
    read, rpos, rslot = read.cpu().tolist(), rpos.cpu().tolist(), rslot.cpu().tolist()
    for b, (n, (s, e), anc, table) in enumerate(zip(lengths, spans, anchors, tables)):
        want_read, want_pos, want_slot = O.finalize_slot_mapping(n, s, e, anc, table, block_size, shared_slot_offset=3)
        assert read[cu_len[b]:cu_len[b + 1]] == want_read
        assert rpos[cu_rec[b]:cu_rec[b + 1]] == want_pos
        assert rslot[cu_rec[b]:cu_rec[b + 1]] == want_slot


def test_reference_golden_layout(device):
    """The layout the reference's own test fixes (tests/test_model_runner_acache.py:26-47 builds its read map from
    this geometry): prefix affix of 3 with anchor {1}, 3 request tokens, block size 8, block 1."""
    bt = torch.tensor([[1, -1]], dtype=torch.int32, device=device)
    read, rpos, rslot, _, _ = ops.build_slot_layout([6], [(0, 3)], [[1]], bt, 8)
    assert read.cpu().tolist() == [0, 8, 2, 9, 10, 11]
    assert rpos.cpu().tolist() == [1, 3, 4, 5] and rslot.cpu().tolist() == [8, 9, 10, 11]
