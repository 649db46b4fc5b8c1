"""Waiting/running queues over a ``BlockManager``.

The reference's ``Scheduler`` (nano-vdllm/scheduler.py:8-71) is unreachable
code: nothing imports it and it calls ``BlockManager.can_append/may_append``
and ``Config.eos/kvcache_block_size``, none of which exist.  The real admission
logic lives in ``ModelRunner._collect_admissible_sequences``.  This class keeps
the same public surface (``add/schedule/preempt/postprocess/is_finished``) with
the admission half working against the block manager that does exist, so code
that constructs a ``Scheduler`` keeps running.
"""
from __future__ import annotations

from collections import deque

from .block_manager import BlockManager
from .config import Config
from .sequence import Sequence, SequenceStatus


class Scheduler:
    def __init__(self, config: Config):
        self.max_num_seqs = config.max_num_seqs
        self.max_num_batched_tokens = config.max_num_batched_tokens
        self.eos = getattr(config, "eos", -1)
        block_size = getattr(config, "kvcache_block_size", config.cache_block_size)
        self.block_manager = BlockManager(config.num_kvcache_blocks, block_size)
        self.waiting: deque[Sequence] = deque()
        self.running: deque[Sequence] = deque()

    def is_finished(self):
        return not self.waiting and not self.running

    def add(self, seq: Sequence):
        self.waiting.append(seq)

    def schedule(self) -> tuple[list[Sequence], bool]:
        """Admit waiting requests while blocks and the token budget allow.

        Returns ``(scheduled, True)`` for newly admitted requests, otherwise
        ``(running, False)``: diffusion decoding never grows a request, so the
        running set needs no per-step block appends.
        """
        limit = self.max_num_seqs if self.max_num_seqs > 0 else float("inf")
        admitted: list[Sequence] = []
        budget = self.max_num_batched_tokens
        while self.waiting and len(self.running) < limit:
            seq = self.waiting[0]
            if len(seq) > budget or not self.block_manager.can_allocate(seq):
                break
            self.block_manager.allocate(seq)
            budget -= len(seq)
            seq.status = SequenceStatus.RUNNING
            self.running.append(self.waiting.popleft())
            admitted.append(seq)
        if admitted:
            return admitted, True
        assert self.running
        return list(self.running), False

    def preempt(self, seq: Sequence):
        seq.status = SequenceStatus.WAITING
        self.block_manager.deallocate(seq)
        if seq in self.running:
            self.running.remove(seq)
        self.waiting.appendleft(seq)

    def postprocess(self, seqs: list[Sequence], finished: list[bool]) -> list[bool]:
        for seq, done in zip(seqs, finished):
            if done:
                seq.status = SequenceStatus.FINISHED
                self.block_manager.deallocate(seq)
                self.running.remove(seq)
        return list(finished)
