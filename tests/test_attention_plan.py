"""The host-side dispatch planner of the varlen attention (acache_varlen_attn_plan): every (request, query tile,
head) unit exactly once, each on the XCD that shares its KV head, padding marked, and a simulated makespan under the
planner's own cost model that never exceeds longest-first list scheduling.  Runs without a GPU."""
import heapq

import numpy as np
import pytest

from acache_amd import _lib
from acache_amd.synthetic import attention_batch

SLOTS = 64


def _plan(cu_q, cu_k, H, Hkv, slots=SLOTS):
    lib = _lib.load()
    cq, ck = np.asarray(cu_q, dtype=np.int32), np.asarray(cu_k, dtype=np.int32)
    B = cq.size - 1
    blocks = lib.acache_varlen_attn_plan(cq.ctypes.data, ck.ctypes.data, B, H, Hkv, slots, None, 0)
    assert blocks >= 0 and blocks % 8 == 0
    out = np.full((blocks, 2), 7, dtype=np.int32)
    if blocks:
        assert lib.acache_varlen_attn_plan(cq.ctypes.data, ck.ctypes.data, B, H, Hkv, slots, out.ctypes.data, blocks) == blocks
    return out


def _cost(rows, kv):      # the model the planner documents: a fixed part plus a term per 64-key tile
    return 290 + (kv + 63) // 64 * (100 if rows > 64 else 85 if rows > 32 else 60)


def _makespan(costs, slots):
    free_at = [0] * slots
    heapq.heapify(free_at)
    for c in costs:
        heapq.heappush(free_at, heapq.heappop(free_at) + c)
    return max(free_at)


def _check(cu_q, cu_k, H, Hkv, slots=SLOTS):
    plan = _plan(cu_q, cu_k, H, Hkv, slots)
    B, group = len(cu_q) - 1, H // Hkv
    want = {(b, t, h) for b in range(B) for t in range((cu_q[b + 1] - cu_q[b] + 127) // 128) for h in range(H)}
    live = plan[plan[:, 0] >= 0]
    got = [(int(b), int(y) & 0xFFFFF, int(y) >> 20) for b, y in live]
    assert len(got) == len(set(got)) and set(got) == want
    assert np.all(plan[plan[:, 0] < 0] == [-1, 0])                       # padding: request -1
    planned = lpt = 0
    for x in range(8):
        units = [(int(b), int(y) & 0xFFFFF, int(y) >> 20) for b, y in plan[x::8] if b >= 0]
        # KV head j may only appear on the XCDs that the interval [8 j / Hkv, 8 (j + 1) / Hkv) overlaps
        for j in {h // group for _, _, h in units}:
            assert min(8 * (j + 1), Hkv * (x + 1)) > max(8 * j, Hkv * x), (j, x)
        # all heads of a tile's group sit on the same XCD: they read the same K/V rows
        by_tile = {}
        for b, t, h in units:
            by_tile.setdefault((b, t, h // group), set()).add(h % group)
        assert all(len(v) == group for v in by_tile.values())
        costs = [_cost(min(128, cu_q[b + 1] - cu_q[b] - t * 128), cu_k[b + 1] - cu_k[b]) for b, t, _ in units]
        planned = max(planned, _makespan(costs, slots))
        lpt = max(lpt, _makespan(sorted(costs, reverse=True), slots))
    assert planned <= lpt
    return planned, lpt, plan


def test_benchmark_batch_is_packed_close_to_the_mean_load():
    w = attention_batch(seed=0)
    cu_q, cu_k = w["cu_q"].tolist(), w["cu_k"].tolist()
    planned, lpt, plan = _check(cu_q, cu_k, 32, 32)
    assert plan.shape[0] == 1088                                          # 34 tiles x 32 heads, nothing padded
    total = sum(_cost(min(128, cu_q[b + 1] - cu_q[b] - t * 128), cu_k[b + 1] - cu_k[b])
                for b in range(16) for t in range((cu_q[b + 1] - cu_q[b] + 127) // 128)) * 4
    assert planned <= 1.05 * total / SLOTS and lpt >= 1.15 * total / SLOTS      # 5080 against 5980, mean 4930
    _check(cu_q, cu_k, 32, 8)


@pytest.mark.parametrize("H,Hkv", [(32, 32), (32, 8), (28, 4), (8, 2), (6, 1), (12, 12), (36, 12), (5, 5), (16, 16)])
def test_every_unit_once_for_all_head_layouts(H, Hkv):
    rng = np.random.default_rng(H * 100 + Hkv)
    for B in (1, 2, 7, 33, 90):
        q = rng.integers(0, 500, B)
        k = q + rng.integers(0, 2500, B)
        q[rng.integers(0, B)] = 0
        _check([0] + np.cumsum(q).tolist(), [0] + np.cumsum(k).tolist(), H, Hkv)


def test_lists_outside_the_packing_range_are_longest_first():
    # 12 units per XCD on 64 slots (all start at once), and 1280 units per XCD on 2 slots (more than 16 per slot)
    big = [0] + [128 * 40 * (i + 1) for i in range(8)]
    big_k = [0] + list(np.cumsum([300 * (i + 1) for i in range(8)]))
    for cu_q, cu_k, slots in (([0, 32, 64, 96], [0, 900, 1100, 1500], 64), (big, big_k, 2)):
        plan = _check(cu_q, cu_k, 32, 32, slots=slots)[2]
        for x in range(8):
            kv = [cu_k[b + 1] - cu_k[b] for b, _ in plan[x::8] if b >= 0]
            assert kv == sorted(kv, reverse=True)


def test_empty_batches_and_argument_errors():
    lib = _lib.load()
    assert _plan([0], [0], 8, 8).shape == (0, 2)
    assert _plan([0, 0, 0], [0, 5, 9], 8, 8).shape == (0, 2)              # requests without queries
    cq = np.array([0, 200], dtype=np.int32)
    out = np.zeros((8, 2), dtype=np.int32)
    assert lib.acache_varlen_attn_plan(cq.ctypes.data, cq.ctypes.data, 1, 8, 8, 64, out.ctypes.data, 8) == -3
    assert b"blocks" in lib.acache_last_error()                           # the plan needs 16 blocks
    assert lib.acache_varlen_attn_plan(cq.ctypes.data, cq.ctypes.data, 1, 8, 3, 64, None, 0) == -3
    assert lib.acache_varlen_attn_plan(None, None, 1, 8, 8, 64, None, 0) == -1
    down = np.array([0, 200, 100], dtype=np.int32)
    assert lib.acache_varlen_attn_plan(down.ctypes.data, down.ctypes.data, 2, 8, 8, 64, None, 0) == -3
