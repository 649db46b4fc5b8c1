"""Logical request layout for affix-KV reuse: spans, anchor budget, slot maps.

Host-side mirror of the reference's ``Sequence`` (nano-vdllm/sequence.py:13-212):
same constructor arguments, attribute names, error messages and list-valued
results, so callers written against the reference keep working.  The slot-map
construction is vectorised with numpy because at batch 16 the per-token Python
loops of the reference dominate host time; the lists it returns are identical.

Vocabulary
----------
affix     span ``[affix_start, affix_end)`` shared by many requests
anchor    affix position whose K/V is recomputed per request (gets a private slot)
slot      flat index into the paged cache: ``block_id * cache_block_size + offset``
"""
from __future__ import annotations

import itertools
import math
from enum import Enum, auto

import numpy as np


class SequenceStatus(Enum):
    WAITING = auto()
    RUNNING = auto()
    FINISHED = auto()


class DeviceLayout:
    """Slot maps of one request as device tensors (views into the tensors the layout kernel filled for a whole
    admission batch), for an engine that never brings them to the host.

    ``anchors`` int32 ascending anchor positions; ``read`` int32 read slot per logical position; ``read_packed`` the
    same slots with the shared affix slots moved to the front (query-side relocation order) or ``None``;
    ``recompute_pos`` int64 / ``recompute_slots`` int32: the rows a cache refresh recomputes and where their K/V
    go; ``tokens`` int64 token ids, kept current by the engine as blocks are committed."""

    __slots__ = ("anchors", "read", "read_packed", "recompute_pos", "recompute_slots", "tokens")

    def __init__(self, anchors, read, read_packed, recompute_pos, recompute_slots, tokens):
        self.anchors, self.read, self.read_packed = anchors, read, read_packed
        self.recompute_pos, self.recompute_slots, self.tokens = recompute_pos, recompute_slots, tokens


def _host_mirror(name: str, fetch):
    """A list-valued attribute that may live on the device: read back (and kept) the first time the host asks."""
    slot = "_" + name

    def get(self):
        value = self.__dict__.get(slot)
        if value is None:
            value = fetch(self)
            self.__dict__[slot] = value
        return value

    def put(self, value):
        self.__dict__[slot] = value

    return property(get, put)


class Sequence:
    counter = itertools.count()

    # host lists of the reference; with a device layout attached they are fetched on first use only
    anchor_positions = _host_mirror(
        "anchor_positions", lambda s: (s.device_layout.anchors if s.device_layout is not None
                                       else s.pending_device_anchors).tolist())
    recompute_positions = _host_mirror("recompute_positions", lambda s: s.device_layout.recompute_pos.tolist())
    recompute_slot_mapping = _host_mirror("recompute_slot_mapping", lambda s: s.device_layout.recompute_slots.tolist())
    read_slot_map = _host_mirror("read_slot_map", lambda s: s.device_layout.read.tolist())

    def __init__(
        self,
        token_ids: list[int],
        block_length: int = 32,
        gen_length: int = 256,
        cache_block_size: int = 256,
        mask_id: int = 126336,
        prompt_affix_len: int = 0,
        prompt_affix_start: int | None = None,
        prompt_affix_end: int | None = None,
        generation_start: int | None = None,
    ):
        self.seq_id = next(Sequence.counter)
        self.status = SequenceStatus.WAITING
        self.token_ids = list(token_ids)
        self.num_prompt_tokens = len(self.token_ids)
        gen_length = int(gen_length)

        # Generation window: appended after the prompt, or an infill span inside it
        # (reference sequence.py:33-44).
        if generation_start is None:
            self.generation_start = self.num_prompt_tokens
            self.token_ids += [mask_id] * gen_length
        else:
            self.generation_start = int(generation_start)
            stop = self.generation_start + gen_length
            if not 0 <= self.generation_start <= stop <= self.num_prompt_tokens:
                raise ValueError(
                    "Infill generation span must be contained in the provided prompt."
                )
            self.token_ids[self.generation_start:stop] = [mask_id] * gen_length
        self.generation_end = self.generation_start + gen_length
        self.num_tokens = len(self.token_ids)

        # Declared affix span (reference sequence.py:46-59).
        a0 = 0 if prompt_affix_start is None else int(prompt_affix_start)
        a1 = a0 + int(prompt_affix_len) if prompt_affix_end is None else int(prompt_affix_end)
        if not 0 <= a0 <= a1 <= self.num_tokens:
            raise ValueError("Affix span must be contained in the logical sequence.")
        if self.generation_start < a1 and self.generation_end > a0:
            raise ValueError("Generation and affix spans must not overlap.")
        self.prompt_affix_start, self.prompt_affix_end = a0, a1
        self.prompt_affix_len = a1 - a0

        self.block_table: list[int] = []
        self.gen_length = gen_length
        self.block_length = block_length
        self.cache_block_size = cache_block_size
        self.current_block_idx = 0
        self.num_blocks_to_generate = -(-gen_length // block_length)

        self.acache_enabled = False
        self.device_layout: DeviceLayout | None = None
        self.pending_device_anchors = None   # anchors chosen on the device, before blocks are allocated
        self.affix_start, self.affix_end = a0, a1
        self.affix_len = 0
        self.anchor_positions: list[int] = []
        self.num_anchor_tokens = 0
        self.recompute_positions: list[int] = list(range(self.num_tokens))
        self.recompute_slot_mapping: list[int] = []
        self.read_slot_map: list[int] = []
        self.shared_slot_offset = 0
        self.relocated_affix_materialized = False

    # -- container protocol -------------------------------------------------
    def __len__(self):
        return self.num_tokens

    def __getitem__(self, key):
        return self.token_ids[key]

    # -- views --------------------------------------------------------------
    @property
    def is_finished(self):
        return self.status == SequenceStatus.FINISHED

    @property
    def prompt_token_ids(self):
        return self.token_ids[: self.num_prompt_tokens]

    @property
    def generated_token_ids(self):
        return self.token_ids[self.generation_start:self.generation_end]

    @property
    def prompt_affix_token_ids(self):
        return self.token_ids[self.prompt_affix_start:self.prompt_affix_end]

    @property
    def non_affix_positions(self):
        return [*range(self.affix_start), *range(self.affix_end, self.num_tokens)]

    # -- cache accounting (reference sequence.py:107-124) ---------------------
    @property
    def num_private_slots(self):
        if not self.acache_enabled:
            return self.num_tokens
        return self.num_anchor_tokens + self.num_tokens - self.affix_len

    @property
    def num_cache_blocks(self):
        return -(-self.num_private_slots // self.cache_block_size)

    @property
    def last_cache_block_num_tokens(self):
        return self.num_private_slots - (self.num_cache_blocks - 1) * self.cache_block_size

    def block(self, i):
        assert 0 <= i < self.num_cache_blocks
        bs = self.cache_block_size
        return self.token_ids[i * bs:(i + 1) * bs]

    # -- ACache layout --------------------------------------------------------
    def enable_acache(
        self,
        affix_len: int | None = None,
        anchor_ratio: float = 0.0,
        *,
        affix_start: int | None = None,
        affix_end: int | None = None,
    ):
        """Fix the affix span and the anchor budget ``K = min(ceil(ratio*A), A)``.

        ``ceil`` is evaluated on the Python double product exactly as the
        reference does (sequence.py:147), e.g. ``ceil(0.07 * 100) == 8`` because
        the binary64 product is 7.000000000000001.
        """
        a0 = self.prompt_affix_start if affix_start is None else int(affix_start)
        if affix_end is not None:
            a1 = int(affix_end)
        elif affix_len is not None:
            a1 = a0 + int(affix_len)
        else:
            a1 = self.prompt_affix_end
        self.affix_start, self.affix_end = a0, a1
        if not 0 <= a0 <= a1 <= self.num_tokens:
            raise ValueError("ACache affix span must be contained in the logical sequence.")
        self.affix_len = a1 - a0
        self.acache_enabled = self.affix_len > 0
        self.num_anchor_tokens = min(math.ceil(anchor_ratio * self.affix_len), self.affix_len)
        self.device_layout = None
        self.pending_device_anchors = None
        self.anchor_positions = []
        self.recompute_positions = list(range(self.num_tokens))
        self.recompute_slot_mapping = []
        self.read_slot_map = []
        self.relocated_affix_materialized = False

    def set_anchor_positions(self, anchor_positions: list[int]):
        """Record the chosen anchors (reference sequence.py:154-167)."""
        chosen = sorted({int(p) for p in anchor_positions})
        if not self.acache_enabled:
            self.anchor_positions = []
            self.num_anchor_tokens = 0
            self.recompute_positions = list(range(self.num_tokens))
            return
        assert all(self.affix_start <= p < self.affix_end for p in chosen)
        assert len(chosen) == min(self.num_anchor_tokens, self.affix_len)
        self.anchor_positions = chosen
        self.num_anchor_tokens = len(chosen)
        self.recompute_positions = sorted(chosen + self.non_affix_positions)

    def set_anchor_positions_on_device(self, anchors):
        """The engine's top-k left this request's ascending anchor positions in a device tensor (``None`` for a
        request without anchors); ``anchor_positions`` reads them back only if somebody asks."""
        assert self.acache_enabled
        self.pending_device_anchors = anchors
        self.anchor_positions = None if anchors is not None else []

    def attach_device_layout(self, layout: DeviceLayout, shared_slot_offset: int = 0):
        """The engine built this request's anchors and slot maps on the device (top-k and the layout kernel):
        adopt them without a read-back.  The four host lists are fetched from the tensors if anybody asks."""
        assert self.acache_enabled and layout.anchors.numel() == self.num_anchor_tokens
        self.device_layout = layout
        self.shared_slot_offset = shared_slot_offset
        for name in ("anchor_positions", "recompute_positions", "recompute_slot_mapping", "read_slot_map"):
            setattr(self, name, None)

    def private_slots(self) -> np.ndarray:
        """Slots owned by this request, block by block in ``block_table`` order."""
        n = self.num_private_slots
        if n == 0:
            return np.zeros(0, dtype=np.int64)
        bs = self.cache_block_size
        table = np.asarray(self.block_table[: self.num_cache_blocks], dtype=np.int64)
        slots = (table[:, None] * bs + np.arange(bs, dtype=np.int64)[None, :]).reshape(-1)[:n]
        assert slots.size == n
        return slots

    def finalize_slot_mapping(self, shared_slot_offset: int = 0):
        """Build ``read_slot_map`` and ``recompute_slot_mapping``.

        The first ``K`` private slots go to the anchors in ascending position
        order, the remaining ones to the non-affix positions in order; every
        other affix position reads the shared copy at
        ``shared_slot_offset + (pos - affix_start)`` (reference sequence.py:169-202).
        """
        self.shared_slot_offset = shared_slot_offset
        private = self.private_slots()

        if not self.acache_enabled:
            self.recompute_positions = list(range(self.num_tokens))
            self.recompute_slot_mapping = private.tolist()
            self.read_slot_map = private.tolist()
            return

        k = self.num_anchor_tokens
        dynamic = private[k:]
        assert dynamic.size == self.num_tokens - self.affix_len
        anchors = np.asarray(self.anchor_positions, dtype=np.int64)
        outside = np.asarray(self.non_affix_positions, dtype=np.int64)

        read = np.full(self.num_tokens, -1, dtype=np.int64)
        read[self.affix_start:self.affix_end] = shared_slot_offset + np.arange(self.affix_len)
        # zip() semantics of the reference: extra anchors beyond the private
        # slots available (never the case after allocate) are ignored.
        n_anchor = min(anchors.size, k)
        read[anchors[:n_anchor]] = private[:n_anchor]
        read[outside] = dynamic

        positions = np.concatenate([anchors[:n_anchor], outside])
        slots = np.concatenate([private[:n_anchor], dynamic])
        order = np.argsort(positions, kind="stable")
        self.recompute_positions = positions[order].tolist()
        self.recompute_slot_mapping = slots[order].tolist()
        self.read_slot_map = read.tolist()

    def block_query_start(self):
        """Index of the current block's first token among the recomputed rows (sequence.py:204-206 looks it up in
        the list; anchors all lie inside the affix, so the index follows from the spans alone)."""
        start = self.generation_start + self.current_block_idx * self.block_length
        if not self.acache_enabled or start < self.affix_start:
            return start
        anchors = self.num_anchor_tokens if self.device_layout is not None else len(self.anchor_positions)
        return start - self.affix_len + anchors

    def __getstate__(self):
        return (self.num_tokens, self.num_prompt_tokens, self.block_table)

    def __setstate__(self, state):
        self.num_tokens, self.num_prompt_tokens, self.block_table, self.token_ids = state
