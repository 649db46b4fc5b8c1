"""Engine for block-wise masked-diffusion decoding with affix-KV reuse.

Mirror of the reference's ``ModelRunner`` (nano-vdllm/model_runner.py) for the LLaDA
path: same constructor, attribute names, method names/signatures and return
values for KV-cache allocation, shared-affix precompute, anchor selection,
relocation set-up, the ``prepare_*`` context builders and the two generation
loops.  What is re-designed:

* all device work goes through this package's HIP kernels (scatter, varlen
  attention, relocation, top-k); anchor top-k for a whole admission batch is one
  launch of the radix-select kernel instead of ``torch.topk`` + ``sort`` +
  ``tolist`` per request (model_runner.py:833-843);
* slot maps, positions and cu_seqlens are assembled with numpy in one pass per
  call instead of per-token Python loops (model_runner.py:1339-1359);
* the importance probe observes ``Attention`` through its ``probe`` hook instead
  of monkey-patching ``forward`` (model_runner.py:730-782);
* logits are computed only for the rows that are read (``logits_keep_indices``),
  which the reference does for its Dream path only (model_runner.py:2101-2104);
* the two generation loops share one implementation.

Not carried over: the dKV-cache schedules (model_runner.py:1725-2030) and the Dream
decoder-layer variants — neither is on the affix-KV reuse path measured here.
"""
from __future__ import annotations

import gc
import math
import sys
import time

import numpy as np
import torch

from . import ops
from .block_manager import BlockManager
from .checkpoint import engine_model_for
from .sequence import DeviceLayout, Sequence
from .utils import add_gumbel_noise, get_context, reset_context, set_context


class ModelRunner:
    def __init__(self, model, config):
        self.config = config
        # the reference's caller passes its own model class (model_runner.py:15-19); a model that is not built from
        # this package's blocks is taken over: same parameter tensors under the engine's decoder stack
        unwrapped = model.module if hasattr(model, "module") else model
        engine = engine_model_for(unwrapped)
        if engine is not unwrapped:
            model = engine
        self.model = model
        self.base_model = model.module if hasattr(model, "module") else model
        self.device = model.device
        self.kv_cache = None
        self.kv_cache_block_bytes = 0
        self.block_manager = None
        self.shared_prefix_len = 0
        self.shared_prefix_blocks = 0
        self.acache_ready = False
        self.shared_prefix_token_ids: tuple[int, ...] = ()
        self._affix_relocation_enabled = False
        self._affix_relocation_max_position = 0
        self._relocated_affix_slot_offset = None
        self.profile_timing = bool(getattr(config, "profile_timing", False))
        self.last_timing = {}
        self._decode_graph_warm = set()
        self._active_timing = None
        self._attention_plans = {}
        # two four-wave workgroups of the attention kernel fit a CU; an XCD holds an eighth of the CUs
        cus = torch.cuda.get_device_properties(self.device).multi_processor_count if self.device.type == "cuda" else 0
        self._workgroup_slots_per_xcd = 2 * max(1, cus // 8)
        # the merged projection weights exist before the cache is sized from free device memory
        if self.device.type == "cuda" and hasattr(self.base_model, "model"):
            with torch.no_grad():
                for block in self._llada_blocks():
                    if hasattr(block, "fuse_projections"):
                        block.fuse_projections()
        self.allocate_kv_cache()

    # ------------------------------------------------------------------ model access
    def _is_dream_model(self):
        return str(getattr(self.config, "model_type", "")).lower() == "dream"

    def _forward_model(self, input_ids, position_ids=None, compute_logits=True):
        return self.base_model.model.forward(
            input_ids=input_ids, position_ids=position_ids, compute_logits=compute_logits)

    def _llada_blocks(self):
        inner = self.base_model.model
        if hasattr(inner, "transformer") and "blocks" in inner.transformer:
            return list(inner.transformer["blocks"])
        if hasattr(inner, "layers"):
            return list(inner.layers)
        raise AttributeError("Unable to locate transformer blocks/layers on model.")

    def _attention_modules(self):
        return [m for m in self.model.modules() if hasattr(m, "k_cache") and hasattr(m, "v_cache")]

    def _attention_head_counts(self):
        first = self._attention_modules()[0]
        return first.num_heads, first.num_kv_heads

    # ------------------------------------------------------------------ timing (model_runner.py:80-140)
    def _profile_timing_enabled(self):
        return self.profile_timing

    def _new_timing(self, mode: str, num_prompts: int):
        if not self.profile_timing:
            return None
        return {"mode": mode, "num_prompts": int(num_prompts)}

    def _start_timing(self):
        if not self._profile_timing_enabled():
            return None
        if self.device.type == "cuda":
            torch.cuda.synchronize(self.device)
        return time.perf_counter()

    def _finish_timing(self, timing, key, start):
        if start is None or timing is None:
            return
        if self.device.type == "cuda":
            torch.cuda.synchronize(self.device)
        timing[key] = timing.get(key, 0.0) + (time.perf_counter() - start)

    def _add_timing_count(self, timing, key, value=1):
        if timing is None:
            return
        timing[key] = timing.get(key, 0) + int(value)

    def _record_kv_cache_usage(self, timing):
        if timing is None or self.block_manager is None:
            return
        bs = int(self.config.cache_block_size)
        used = len(self.block_manager.used_block_ids)
        cap = self.block_manager.num_blocks
        timing["kv_cache_block_size"] = bs
        timing["kv_cache_block_bytes"] = int(self.kv_cache_block_bytes)
        timing["kv_cache_slot_bytes"] = int(self.kv_cache_block_bytes // bs)
        for name, value in (("used_blocks", used), ("used_slots", used * bs),
                            ("used_bytes", used * self.kv_cache_block_bytes),
                            ("capacity_blocks", cap), ("capacity_slots", cap * bs),
                            ("capacity_bytes", cap * self.kv_cache_block_bytes)):
            key = f"kv_cache_peak_{name}"
            timing[key] = max(timing.get(key, 0), value)
        timing["kv_cache_peak_used_gb"] = timing["kv_cache_peak_used_bytes"] / 1024 ** 3
        timing["kv_cache_peak_capacity_gb"] = timing["kv_cache_peak_capacity_bytes"] / 1024 ** 3

    # ------------------------------------------------------------------ KV cache (model_runner.py:142-218)
    def _reset_acache_state(self):
        self.shared_prefix_len = 0
        self.shared_prefix_blocks = 0
        self.acache_ready = False
        self.shared_prefix_token_ids = ()
        self._affix_relocation_enabled = False
        self._affix_relocation_max_position = 0
        self._relocated_affix_slot_offset = None

    @staticmethod
    def _first_attr(obj, *names):
        for name in names:
            value = getattr(obj, name, None)
            if value is not None:
                return value
        return None

    def allocate_kv_cache(self, num_blocks: int | None = None):
        """``kv_cache[2, L, num_blocks, block, H_kv, D]`` bf16 with per-layer views bound to the attention modules."""
        config, hf = self.config, self.config.hf_config
        num_heads = self._first_attr(hf, "n_heads", "num_attention_heads")
        if num_heads is None:
            raise AttributeError("HF config must define n_heads or num_attention_heads.")
        num_kv_heads = self._first_attr(hf, "effective_n_kv_heads", "n_kv_heads", "num_key_value_heads") or num_heads
        hidden = self._first_attr(hf, "d_model", "hidden_size")
        if hidden is None:
            raise AttributeError("HF config must define d_model or hidden_size.")
        num_layers = self._first_attr(hf, "n_layers", "num_hidden_layers")
        if num_layers is None:
            raise AttributeError("HF config must define n_layers or num_hidden_layers.")
        head_dim = hidden // num_heads
        bs = config.cache_block_size
        self.kv_cache_block_bytes = 2 * num_layers * bs * num_kv_heads * head_dim * 2  # K and V, bf16

        if num_blocks is None and config.num_kvcache_blocks < 0:
            free, total = torch.cuda.mem_get_info()
            stats = torch.cuda.memory_stats()
            peak, current = stats["allocated_bytes.all.peak"], stats["allocated_bytes.all.current"]
            reserve = 0
            if config.enable_acache:
                reserve = int(max(float(config.acache_memory_reserve_gb), 0.0) * 1024 ** 3)
            available = total * config.gpu_memory_utilization - (total - free) - peak + current - reserve
            num_blocks = int(available // self.kv_cache_block_bytes)
        elif num_blocks is None:
            num_blocks = config.num_kvcache_blocks
        config.num_kvcache_blocks = int(num_blocks)
        assert config.num_kvcache_blocks >= 1, "Not enough GPU memory."

        if self.kv_cache is not None:
            # a resize: hand the old cache back before asking for the new one, or both are live at the peak
            for module in self._attention_modules():
                module.k_cache = module.v_cache = torch.empty(0, dtype=torch.bfloat16, device=self.device)
            self.kv_cache = None
            self._release_cached_device_memory()
        self.kv_cache = torch.empty(2, num_layers, config.num_kvcache_blocks, bs, num_kv_heads, head_dim,
                                    dtype=torch.bfloat16, device=self.device)
        self._reset_acache_state()
        for layer_id, module in enumerate(self._attention_modules()):
            module.k_cache = self.kv_cache[0, layer_id]
            module.v_cache = self.kv_cache[1, layer_id]
            module.use_reference_attention = self.config.use_reference_attention
            module.shared_prefix_len = 0
        self.block_manager = BlockManager(config.num_kvcache_blocks, bs)

    def _shared_affix_k(self, layer_idx: int):
        h, d = self.kv_cache.shape[-2:]
        return self.kv_cache[0, layer_idx].view(-1, h, d)[: self.shared_prefix_len]

    # ------------------------------------------------------------------ relocation set-up (231-341)
    def _configure_affix_relocation(self, seqs: list[Sequence]):
        uses_rope = bool(getattr(self.config.hf_config, "rope", True))
        required = uses_rope and any(seq.affix_start != 0 for seq in seqs)
        max_position = max((len(seq) for seq in seqs), default=0)
        if not required and not self._affix_relocation_enabled:
            return
        if required and self._affix_relocation_enabled and self._affix_relocation_max_position >= max_position:
            return
        for block in self._llada_blocks():
            attention, rotary = block.attn, block.rotary_emb
            attention.shared_prefix_len = self.shared_prefix_len if required else 0
            if not required or attention.relocation_rope_cos.shape[0] >= max_position:
                continue
            sin, cos = rotary.get_rotary_embedding(max_position, self.device)
            attention.relocation_rope_cos = cos
            attention.relocation_rope_sin = sin
        self._affix_relocation_enabled = required
        self._affix_relocation_max_position = max_position if required else 0

    def _attention_read_layout(self, seq, use_query_relocation: bool):
        """Read slots of one request; shared affix slots packed first for query-side relocation (275-282)."""
        if getattr(seq, "drop_non_anchor", False):
            # strict ablation of the HF path (llada/generate_ACache.py:478-491): the frozen affix rows are not
            # read at all; anchors and non-affix tokens live in private slots and keep their position ids
            slots = np.asarray(seq.read_slot_map, dtype=np.int64)
            frozen = (slots >= seq.shared_slot_offset) & (slots < seq.shared_slot_offset + self.shared_prefix_len)
            if self._relocated_affix_slot_offset is not None:
                lo = self._relocated_affix_slot_offset
                frozen |= (slots >= lo) & (slots < lo + self.shared_prefix_len)
            return slots[~frozen].tolist(), 0
        if not use_query_relocation or seq.affix_start == 0:
            return list(seq.read_slot_map), 0
        lo = seq.shared_slot_offset
        hi = lo + self.shared_prefix_len
        slots = np.asarray(seq.read_slot_map, dtype=np.int64)
        shared = (slots >= lo) & (slots < hi)
        return slots[shared].tolist() + slots[~shared].tolist(), int(shared.sum())

    def _use_query_side_affix_relocation(self, relocation_materialized: bool):
        return (self._affix_relocation_enabled and not relocation_materialized
                and self.config.max_num_seqs != 1)

    def _reserve_single_sequence_relocation_workspace(self, seq: Sequence, *, force: bool = False):
        """Pin the blocks right after the shared affix as the destination of its relocated copy (291-312)."""
        if (self.config.max_num_seqs != 1 and not force) or seq.affix_start == 0:
            return False
        bm = self.block_manager
        if self._relocated_affix_slot_offset is not None:
            if bm.can_allocate(seq):
                return True
            bm.release_prefix_tail(self.shared_prefix_blocks)
            self._relocated_affix_slot_offset = None
            return False
        need = self.shared_prefix_blocks
        if bm.num_free_blocks < need + seq.num_cache_blocks:
            return False
        end = self.shared_prefix_blocks + need
        if end > bm.num_blocks or not all(bm.is_free(i) for i in range(self.shared_prefix_blocks, end)):
            return False
        bm.reserve_prefix(end)
        self._relocated_affix_slot_offset = self.shared_prefix_blocks * self.config.cache_block_size
        self._record_kv_cache_usage(self._active_timing)
        return True

    def _materialize_single_sequence_affix(self, seq: Sequence):
        """Write the affix copy rotated by ``seq.affix_start`` into the workspace, all layers in one launch (314-341)."""
        if self._relocated_affix_slot_offset is None or seq.affix_start == 0:
            seq.relocated_affix_materialized = False
            return
        self._configure_affix_relocation([seq])
        start = self._start_timing()
        layers = self.kv_cache.shape[1]
        slots = self.kv_cache.shape[2] * self.kv_cache.shape[3]
        k_cache = self.kv_cache[0].view(layers, slots, *self.kv_cache.shape[-2:])
        v_cache = self.kv_cache[1].view_as(k_cache)
        attention = self._llada_blocks()[0].attn
        ops.materialize_relocated_affix(
            k_cache, v_cache, attention.relocation_rope_cos, attention.relocation_rope_sin,
            self._relocated_affix_slot_offset, seq.affix_len, seq.affix_start)
        lo, hi = seq.shared_slot_offset, seq.shared_slot_offset + seq.affix_len
        for local, pos in enumerate(range(seq.affix_start, seq.affix_end)):
            if lo <= seq.read_slot_map[pos] < hi:
                seq.read_slot_map[pos] = self._relocated_affix_slot_offset + local
        seq.relocated_affix_materialized = True
        self._finish_timing(self._active_timing, "affix_materialize", start)

    # ------------------------------------------------------------------ shared affix (474-541)
    def _resolve_declared_prefix_tokens(self, seqs: list[Sequence]) -> tuple[int, ...]:
        if not seqs:
            return ()
        affix_len = seqs[0].prompt_affix_len
        if affix_len <= 0:
            return ()
        tokens = tuple(seqs[0].prompt_affix_token_ids)
        for seq in seqs[1:]:
            if seq.prompt_affix_len != affix_len:
                raise ValueError("ACache requires the same explicit affix length for every sequence in the batch.")
            if tuple(seq.prompt_affix_token_ids) != tokens:
                raise ValueError("ACache requires identical explicit affix tokens for every sequence in the batch.")
        return tokens

    def _to_device(self, values, dtype):
        t = torch.as_tensor(np.asarray(values), dtype=dtype)
        if self.device.type == "cuda":
            t = t.pin_memory()
        return t.to(self.device, non_blocking=True)

    def _attention_plan(self, cu_q, cu_k):
        """Dispatch plan of the attention kernel for a refresh forward with these prefix sums (host values), or
        None where the order cannot matter: every layer of the forward shares it, and the refreshes of one batch
        repeat the same lengths, so the last few plans are kept."""
        if self.device.type != "cuda":
            return None
        cu_q, cu_k = np.asarray(cu_q, dtype=np.int32), np.asarray(cu_k, dtype=np.int32)
        heads, kv_heads = self._attention_head_counts()
        tiles = int(((np.diff(cu_q) + 127) // 128).sum())
        slots = self._workgroup_slots_per_xcd
        if tiles * heads <= 8 * slots:      # every unit starts at once
            return None
        key = (cu_q.tobytes(), cu_k.tobytes())
        plan = self._attention_plans.pop(key, None)
        if plan is None:
            plan = ops.attention_plan(cu_q, cu_k, heads, kv_heads, self.device, slots)
            if len(self._attention_plans) >= 8:
                self._attention_plans.pop(next(iter(self._attention_plans)))
        self._attention_plans[key] = plan   # most recently used last
        return plan

    def _precompute_shared_prefix(self, prefix_tokens: list[int]):
        """One forward of the affix alone at positions ``0..A-1``; its post-RoPE K/V land in slots ``0..A-1``."""
        n = len(prefix_tokens)
        if n == 0:
            return
        token_ids = tuple(prefix_tokens)
        if self.acache_ready and self.shared_prefix_token_ids == token_ids:
            return
        bs = self.config.cache_block_size
        shared_blocks = -(-n // bs)
        self.block_manager.reserve_prefix(shared_blocks)
        timing = self._active_timing
        self._record_kv_cache_usage(timing)
        start = self._start_timing()
        input_ids = self._to_device(prefix_tokens, torch.int64)
        positions = torch.arange(n, dtype=torch.int64, device=self.device)
        cu = self._to_device([0, n], torch.int32)
        slot_mapping = torch.arange(n, dtype=torch.int32, device=self.device)
        self._finish_timing(timing, "shared_prefix_prepare", start)
        set_context(True, cu, cu, None, n, n, slot_mapping, None, total_k=n)
        modules = self._attention_modules()
        saved = [m.use_reference_attention for m in modules]
        try:
            for m in modules:
                m.use_reference_attention = True  # attend over the fresh K/V rows, not through block tables
            start = self._start_timing()
            self._forward_model(input_ids=input_ids, position_ids=positions, compute_logits=False)
            self._finish_timing(timing, "shared_prefix_forward", start)
            self._add_timing_count(timing, "shared_prefix_forward_calls", 1)
        finally:
            for m, flag in zip(modules, saved):
                m.use_reference_attention = flag
            reset_context()
        self.shared_prefix_len = n
        self.shared_prefix_blocks = shared_blocks
        self.shared_prefix_token_ids = token_ids
        self.acache_ready = True

    # ------------------------------------------------------------------ anchor selection (543-845)
    def _compute_anchor_positions(self, seq: Sequence):
        return self._compute_anchor_positions_batch([seq])[0]

    def _finalize_anchor_selection_probe_layout(self, seq: Sequence, shared_slot_offset: int = 0):
        """Probe layout: anchor slots reserved but unused; queries = non-affix tokens, affix read from the shared copy."""
        private = seq.private_slots()
        dynamic = private[seq.num_anchor_tokens:]
        assert dynamic.size == seq.num_tokens - seq.affix_len
        read = np.full(seq.num_tokens, -1, dtype=np.int64)
        read[seq.affix_start:seq.affix_end] = shared_slot_offset + np.arange(seq.affix_len)
        outside = seq.non_affix_positions
        read[outside] = dynamic
        seq.shared_slot_offset = shared_slot_offset
        seq.recompute_positions = outside
        seq.recompute_slot_mapping = dynamic.tolist()
        seq.read_slot_map = read.tolist()

    def _compute_anchor_positions_batch(self, seqs: list[Sequence]):
        """Importance of every affix token for each request's [MASK] queries, then per-request top-k.

        The K highest (or lowest, ``selection_mode == 'bottom'``) importance indices,
        ascending, plus ``affix_start`` are the anchors (model_runner.py:833-843; ties go
        to the lower index).  One radix-select launch serves the whole batch.
        """
        chosen, counts = self._select_anchors_on_device(seqs)
        if chosen is None:
            return [[] for _ in seqs]
        flat, out, o = chosen.tolist(), [], 0
        for k in counts:
            out.append(flat[o:o + k])
            o += k
        return out

    def _select_anchors_on_device(self, seqs: list[Sequence]):
        """The same selection without the read-back: ``(anchors, counts)`` with ``anchors`` an int32 device tensor
        holding every request's ascending anchor positions back to back and ``counts`` the number per request
        (0 for a request without anchors); ``(None, counts)`` when no request has any."""
        counts = [0] * len(seqs)
        active = [(i, s) for i, s in enumerate(seqs) if s.acache_enabled and s.num_anchor_tokens > 0]
        if not active:
            return None, counts
        active_seqs = [s for _, s in active]
        affix_len = active_seqs[0].affix_len
        if affix_len <= 0:
            return None, counts
        if any(s.affix_len != affix_len for s in active_seqs):
            raise ValueError("Batched Anchor Selection requires a consistent explicit prefix affix length.")
        importance = self._compute_affix_importance(active_seqs)
        timing = self._active_timing
        start = self._start_timing()
        ks = [s.num_anchor_tokens for s in active_seqs]
        cu_k = np.concatenate([[0], np.cumsum(ks)])
        cu_a = np.arange(len(active_seqs) + 1) * affix_len
        chosen = ops.topk_anchors(
            importance.view(-1), self._to_device(cu_a, torch.int32), self._to_device(cu_k, torch.int32),
            int(cu_k[-1]), offsets=self._to_device([s.affix_start for s in active_seqs], torch.int32),
            largest=self.config.selection_mode != "bottom", out_dtype=torch.int32)
        for (i, _), k in zip(active, ks):
            counts[i] = k
        self._finish_timing(timing, "anchor_selection_topk", start)
        return chosen, counts

    def _compute_affix_importance(self, active_seqs: list[Sequence]) -> torch.Tensor:
        """fp32 ``[B, A]`` influence of every shared affix token on each request's [MASK] queries.

        Per layer and request: ``softmax(q_mask . K_affix^T * scale)`` over the affix keys only
        (the cached keys moved to the request's ``affix_start``), summed over heads and mask
        queries (model_runner.py:730-773).  Runs one probe forward over the non-affix tokens of
        the given requests; their layouts and block tables are restored afterwards.
        """
        affix_len = active_seqs[0].affix_len
        timing = self._active_timing
        start = self._start_timing()
        importance = torch.zeros(len(active_seqs), affix_len, device=self.device, dtype=torch.float32)
        saved, temp_allocated, workspace = [], [], False
        blocks = self._llada_blocks()
        try:
            for seq in active_seqs:
                saved.append((seq, list(seq.block_table), list(seq.anchor_positions), list(seq.recompute_positions),
                              list(seq.recompute_slot_mapping), list(seq.read_slot_map), seq.shared_slot_offset,
                              seq.relocated_affix_materialized))
                if not seq.block_table:
                    if len(active_seqs) == 1:
                        workspace = self._reserve_single_sequence_relocation_workspace(seq, force=True)
                    if not self.block_manager.can_allocate(seq):
                        raise torch.OutOfMemoryError("Not enough KV cache blocks for anchor-selection probe.")
                    self.block_manager.allocate(seq)
                    self._record_kv_cache_usage(timing)
                    temp_allocated.append(seq)
                seq.anchor_positions = []
                self._finalize_anchor_selection_probe_layout(seq)
                if workspace:
                    self._materialize_single_sequence_affix(seq)

            input_ids, position_ids, _ = self.prepare_caching_acache(active_seqs, use_query_relocation=False)
            cu_q = [0]
            for seq in active_seqs:
                cu_q.append(cu_q[-1] + len(seq.recompute_positions))
            # the [MASK] rows of every request among its probe queries, from the host's token lists (the same lists
            # input_ids was built from): no read-back of a device mask
            mask_positions = []
            for b, seq in enumerate(active_seqs):
                probe_tokens = np.asarray(seq.token_ids, dtype=np.int64)[np.asarray(seq.recompute_positions, dtype=np.int64)]
                mask_positions.append(np.nonzero(probe_tokens == self.config.mask_id)[0] + cu_q[b])
            self._add_timing_count(timing, "anchor_selection_query_tokens", int(input_ids.numel()))
            self._add_timing_count(timing, "anchor_selection_kv_tokens", sum(len(s) for s in active_seqs))
            self._finish_timing(timing, "anchor_selection_prepare", start)

            uses_rope = bool(getattr(self.config.hf_config, "rope", True))
            # one kernel pair per layer for the whole batch: softmax over the affix keys of every [MASK] query,
            # column sums over queries and heads added to `importance` (the reference loops over requests here)
            counts = [int(rows.size) for rows in mask_positions]
            probe_rows = self._to_device(np.concatenate(mask_positions) if mask_positions else np.zeros(0), torch.int32)
            probe_cu = self._to_device(np.concatenate([[0], np.cumsum(counts)]), torch.int32)
            shifts = [seq.affix_start if uses_rope else 0 for seq in active_seqs]
            probe_shifts = probe_cos = probe_sin = None
            if any(shifts):
                probe_shifts = self._to_device(shifts, torch.int32)
                probe_sin, probe_cos = blocks[0].rotary_emb.get_rotary_embedding(
                    max(self._affix_relocation_max_position, max(shifts) + 1), self.device)
            probe_scratch = torch.empty(
                max(16, ops.affix_importance_workspace_bytes(
                    sum(counts), len(active_seqs), blocks[0].attn.num_heads, blocks[0].attn.num_kv_heads,
                    blocks[0].attn.head_dim, affix_len, probe_shifts is not None)),
                dtype=torch.uint8, device=self.device)

            def make_probe(layer_idx, block):
                def probe(attention, q):
                    if sum(counts) == 0:
                        return
                    ops.affix_importance(
                        importance, q.reshape(-1, attention.num_heads, attention.head_dim), attention.k_cache,
                        probe_rows, probe_cu, affix_len, max(counts), attention.scale, probe_shifts, probe_cos,
                        probe_sin, affix_slot0=0, workspace=probe_scratch)
                return probe

            for layer_idx, block in enumerate(blocks):
                block.attn.probe = make_probe(layer_idx, block)
            start = self._start_timing()
            self._forward_model(input_ids=input_ids, position_ids=position_ids, compute_logits=False)
            self._finish_timing(timing, "anchor_selection_forward", start)
            self._add_timing_count(timing, "anchor_selection_forward_calls", 1)
            self._add_timing_count(timing, "anchor_selection_sequences", len(active_seqs))
        finally:
            for block in blocks:
                block.attn.probe = None
            reset_context()
            for seq in reversed(temp_allocated):
                if seq.block_table:
                    self.block_manager.deallocate(seq)
            for (seq, table, anchors, rpos, rslots, read, offset, materialized) in saved:
                seq.block_table = table
                seq.anchor_positions = anchors
                seq.recompute_positions = rpos
                seq.recompute_slot_mapping = rslots
                seq.read_slot_map = read
                seq.shared_slot_offset = offset
                seq.relocated_affix_materialized = materialized
            if workspace:
                self.block_manager.release_prefix_tail(self.shared_prefix_blocks)
                self._relocated_affix_slot_offset = None

        return importance

    # ------------------------------------------------------------------ admission (847-1003)
    def _prepare_acache(self, seqs: list[Sequence]):
        prefix = self._resolve_declared_prefix_tokens(seqs)
        if not prefix:
            return ()
        for seq in seqs:
            seq.enable_acache(len(prefix), self.config.anchor_ratio,
                              affix_start=seq.prompt_affix_start, affix_end=seq.prompt_affix_end)
        return prefix

    # KV-cache resize when admission runs out of device memory (model_runner.py:570-638, 862-955).  A resize
    # rebuilds the cache and the block manager, so it is only allowed while no request is in flight.
    def _blocks_for(self, prefix_len: int, private_blocks: int) -> int:
        return max(-(-prefix_len // self.config.cache_block_size) + private_blocks, 1)

    def _minimum_kv_cache_blocks_for_acache(self, seqs, prefix_len: int) -> int:
        """Shared affix plus one whole request: below this nothing can be served."""
        return self._blocks_for(prefix_len, max((s.num_cache_blocks for s in seqs), default=0))

    def _selection_kv_cache_blocks(self, seqs, prefix_len: int) -> int:
        """Shared affix plus the largest group of requests that one probe forward holds."""
        step = int(getattr(self.config, "anchor_selection_batch_size", 1) or 0) or max(len(seqs), 1)
        groups = (sum(s.num_cache_blocks for s in seqs[i:i + step]) for i in range(0, len(seqs), step))
        return self._blocks_for(prefix_len, max(groups, default=0))

    def _release_cached_device_memory(self):
        gc.collect()
        if self.device.type == "cuda":
            torch.cuda.empty_cache()

    def _shrink_kv_cache_for_acache(self, seqs, prefix_len: int, minimum_blocks: int | None = None) -> bool:
        """Give up to four blocks back to the allocator; False when the cache is already at its floor."""
        if self.kv_cache_block_bytes <= 0:
            return False
        floor = self._minimum_kv_cache_blocks_for_acache(seqs, prefix_len) if minimum_blocks is None else minimum_blocks
        have = int(self.config.num_kvcache_blocks)
        smaller = max(floor, have - 4)
        if smaller >= have:
            return False
        print(f"[acache] anchor selection OOM, shrinking KV cache blocks from {have} to {smaller} and retrying.")
        self.allocate_kv_cache(num_blocks=smaller)
        return True

    def _ensure_shared_prefix(self, prefix_token_ids, seqs, minimum_blocks: int | None = None):
        """Affix precompute that answers an out-of-memory error by shrinking the KV cache and trying again."""
        while True:
            try:
                self._precompute_shared_prefix(list(prefix_token_ids))
                return
            except torch.OutOfMemoryError as oom:
                failure = torch.OutOfMemoryError(str(oom))   # a fresh object: the original pins the failed frames
            self._release_cached_device_memory()
            if not self._shrink_kv_cache_for_acache(seqs, len(prefix_token_ids), minimum_blocks):
                raise failure

    def _select_anchor_positions_for_sequences(self, seqs, prefix_token_ids, allow_kv_cache_resize,
                                               minimum_blocks=None):
        # one request per probe forward by default, as the reference does (model_runner.py:873);
        # Config.anchor_selection_batch_size widens the probe (0: all admitted requests in one forward).
        # Out of memory: first halve the probe group, then (if allowed) shrink the KV cache, redo the affix
        # precompute that the new cache lost, and try the same group again.
        step = int(getattr(self.config, "anchor_selection_batch_size", 1) or 0) or len(seqs)
        done = 0
        while done < len(seqs):
            width = min(step, len(seqs) - done)
            while True:
                group = seqs[done:done + width]
                try:
                    if self._device_layouts():
                        chosen, counts = self._select_anchors_on_device(group)
                        at = 0
                        for seq, k in zip(group, counts):
                            if seq.acache_enabled:
                                seq.set_anchor_positions_on_device(chosen[at:at + k] if k else None)
                            else:
                                seq.set_anchor_positions([])
                            at += k
                    else:
                        for seq, anchors in zip(group, self._compute_anchor_positions_batch(group)):
                            seq.set_anchor_positions(anchors)
                    done += width
                    break
                except torch.OutOfMemoryError as oom:
                    failure = torch.OutOfMemoryError(str(oom))
                self._release_cached_device_memory()
                if width > 1:
                    width = max(width // 2, 1)
                    continue
                if not allow_kv_cache_resize or not self._shrink_kv_cache_for_acache(
                        seqs, len(prefix_token_ids), minimum_blocks):
                    raise failure
                self._ensure_shared_prefix(prefix_token_ids, seqs, minimum_blocks)

    def _prepare_admitted_sequences_for_acache(self, seqs, prefix_token_ids, allow_kv_cache_resize):
        if not seqs:
            return
        if self.acache_ready and self.shared_prefix_token_ids != prefix_token_ids:
            raise ValueError("ACache prefix mode requires a consistent shared prefix across active requests.")
        target = int(self.config.num_kvcache_blocks)
        floor = min(target, self._selection_kv_cache_blocks(seqs, len(prefix_token_ids)))
        try:
            if not self.acache_ready:
                if allow_kv_cache_resize:
                    self._ensure_shared_prefix(prefix_token_ids, seqs, floor)
                else:
                    self._precompute_shared_prefix(list(prefix_token_ids))
            self._select_anchor_positions_for_sequences(seqs, prefix_token_ids, allow_kv_cache_resize, floor)
        finally:
            # selection is over (or failed): serving goes on with the cache size the caller configured
            if allow_kv_cache_resize and self.config.num_kvcache_blocks != target:
                failed = sys.exc_info()[0] is not None
                self.allocate_kv_cache(num_blocks=target)
                if not failed:
                    self._ensure_shared_prefix(prefix_token_ids, seqs)

    def _finalize_sequence_layout(self, seq: Sequence):
        seq.finalize_slot_mapping()
        self._materialize_single_sequence_affix(seq)

    def _collect_admissible_sequences(self, prompts, next_prompt_idx, current_batch_size, max_num_seqs):
        admissible = []
        remaining = self.block_manager.num_free_blocks
        while next_prompt_idx < len(prompts) and current_batch_size + len(admissible) < max_num_seqs:
            seq = prompts[next_prompt_idx]
            if seq.num_cache_blocks > remaining:
                break
            admissible.append(seq)
            remaining -= seq.num_cache_blocks
            next_prompt_idx += 1
        return admissible, next_prompt_idx

    def _admit_sequences_with_acache(self, batched_prompts, new_prompts, prefix_token_ids, allow_kv_cache_resize):
        if not new_prompts:
            return 0
        self._prepare_admitted_sequences_for_acache(new_prompts, prefix_token_ids, allow_kv_cache_resize)
        self._reserve_single_sequence_relocation_workspace(new_prompts[0])
        admitted, on_device = 0, []
        for seq in new_prompts:
            if not self.block_manager.can_allocate(seq):
                break
            self.block_manager.allocate(seq)
            self._record_kv_cache_usage(self._active_timing)
            if self._device_layouts() and seq.acache_enabled:
                on_device.append(seq)
            else:
                self._finalize_sequence_layout(seq)
            batched_prompts.append(seq)
            admitted += 1
        if on_device:
            self._finalize_layouts_on_device(on_device)
        return admitted

    def _device_layouts(self) -> bool:
        """Slot maps and anchors stay on the device for batched serving.  The single-request mode
        (``max_num_seqs == 1``) edits its read map on the host when it materialises the relocated affix, and the
        HF-signature entry points run in that mode, so it keeps the host lists."""
        return self.device.type == "cuda" and self.config.max_num_seqs != 1

    def _finalize_layouts_on_device(self, seqs: list[Sequence]):
        """``finalize_slot_mapping`` for all newly admitted requests in one launch, fed by the anchors that the
        top-k launch left on the device (model_runner.py:833-843 reads them back with ``tolist`` and
        sequence.py:169-202 loops over tokens on the host).  Also prepares, once per request, what every later
        refresh would otherwise rebuild: the read map with the shared affix slots packed first (the order
        query-side relocation wants, model_runner.py:275-282) and a device copy of the token ids."""
        lengths = [len(s) for s in seqs]
        counts = [s.num_anchor_tokens for s in seqs]
        pending = [s.pending_device_anchors for s in seqs]
        assert all((p is not None and p.numel() == k) or k == 0 for p, k in zip(pending, counts))
        anchors = [p for p, k in zip(pending, counts) if k > 0]
        anchors = (torch.cat(anchors) if len(anchors) > 1 else anchors[0]) if anchors else \
            torch.zeros(0, dtype=torch.int32, device=self.device)
        tables = self.prepare_block_tables(seqs)
        read, rpos, rslot, cu_len, cu_rec = ops.build_slot_layout(
            lengths, [(s.affix_start, s.affix_end) for s in seqs], anchors, tables, self.config.cache_block_size,
            0, anchor_counts=counts)
        uses_rope = bool(getattr(self.config.hf_config, "rope", True))
        moved = [uses_rope and s.affix_start != 0 for s in seqs]
        packed = None
        if any(moved):
            # stable partition inside each request: shared affix slots (0 .. shared_prefix_len) first
            seg = np.repeat(np.arange(len(seqs), dtype=np.int64), lengths)
            flag = self._to_device(np.repeat(np.asarray(moved), lengths), torch.bool)
            private = ~((read >= 0) & (read < self.shared_prefix_len) & flag)
            order = torch.argsort(self._to_device(seg * 2, torch.int64) + private, stable=True)
            packed = read[order]
        tokens = self._to_device(np.concatenate([np.asarray(s.token_ids, dtype=np.int64) for s in seqs]), torch.int64)
        rpos64 = rpos.to(torch.int64)
        at = 0
        for b, seq in enumerate(seqs):
            lo, hi, r0, r1 = cu_len[b], cu_len[b + 1], cu_rec[b], cu_rec[b + 1]
            seq.attach_device_layout(DeviceLayout(
                anchors[at:at + counts[b]], read[lo:hi], packed[lo:hi] if moved[b] else None,
                rpos64[r0:r1], rslot[r0:r1], tokens[lo:hi]))
            seq.pending_device_anchors = None
            seq.relocated_affix_materialized = False
            at += counts[b]

    # ------------------------------------------------------------------ context builders (1004-1114, 1295-1471)
    def _select(self, seqs, active_indices):
        if active_indices is None:
            return list(seqs)
        if torch.is_tensor(active_indices):
            active_indices = active_indices.tolist()
        return [seqs[int(i)] for i in active_indices]

    def prepare_block_tables(self, seqs: list[Sequence]):
        width = max(len(seq.block_table) for seq in seqs)
        table = np.full((len(seqs), width), -1, dtype=np.int32)
        for i, seq in enumerate(seqs):
            table[i, : len(seq.block_table)] = seq.block_table
        return self._to_device(table, torch.int32)

    def prepare_caching(self, seqs, active_indices=None):
        """Full-recompute refresh: every token of every request is a query and is written to its block-table slot."""
        group = self._select(seqs, active_indices)
        block_tables = self.prepare_block_tables(group)
        lens = np.array([len(s) for s in group], dtype=np.int64)
        cu = np.concatenate([[0], np.cumsum(lens)])
        input_ids = np.concatenate([np.asarray(s.token_ids, dtype=np.int64) for s in group])
        positions = np.concatenate([np.arange(n, dtype=np.int64) for n in lens])
        slot_mapping = np.concatenate([s.private_slots() for s in group])
        generate_starts = cu[:-1] + np.array([s.generation_start for s in group])
        current = np.array([s.current_block_idx for s in group])
        cu_dev = self._to_device(cu, torch.int32)
        set_context(True, cu_dev, cu_dev, None, int(lens.max()), int(lens.max()),
                    self._to_device(slot_mapping, torch.int32), block_tables, total_k=int(cu[-1]),
                    attention_plan=self._attention_plan(cu, cu))
        return (self._to_device(input_ids, torch.int64), self._to_device(positions, torch.int64),
                self._to_device(generate_starts, torch.int32), self._to_device(current, torch.int32))

    def prepare_decoding(self, seqs, active_indices=None):
        """Block refinement on the full-recompute path: the current block's tokens against block-table K/V."""
        group = self._select(seqs, active_indices)
        block_length, bs = self.config.block_length, self.config.cache_block_size
        starts = np.array([s.generation_start + s.current_block_idx * block_length for s in group], dtype=np.int64)
        seqlens = np.array([len(s) for s in group], dtype=np.int64)
        positions = starts[:, None] + np.arange(block_length)[None, :]
        tables = [np.asarray(s.block_table, dtype=np.int64) for s in group]
        slot_mapping = np.concatenate([t[p // bs] * bs + p % bs for t, p in zip(tables, positions)])
        block_tables = self.prepare_block_tables(group)
        set_context(False, None, None, self._to_device(seqlens, torch.int32), None, None,
                    self._to_device(slot_mapping, torch.int32), block_tables, total_k=int(seqlens.sum()))
        return self._to_device(positions, torch.int64)

    def prepare_caching_acache(self, seqs, active_indices=None, use_query_relocation=None):
        """Cache refresh with affix reuse: queries = anchors + non-affix tokens; keys read through ``read_slot_map``."""
        group = self._select(seqs, active_indices)
        self._configure_affix_relocation(group)
        if use_query_relocation is None and all(s.device_layout is not None for s in group):
            return self._prepare_caching_from_device_layouts(group)
        relocation_materialized = all(getattr(s, "relocated_affix_materialized", False) for s in group)
        if use_query_relocation is None:
            use_query_relocation = self.config.max_num_seqs != 1
        use_query_relocation = (self._affix_relocation_enabled and not relocation_materialized
                                and bool(use_query_relocation))
        ids, pos, slots, reads = [], [], [], []
        shared_lens, shifts, block_starts = [], [], []
        cu_q, cu_k = [0], [0]
        for seq in group:
            q_pos = np.asarray(seq.recompute_positions, dtype=np.int64)
            assert len(seq.recompute_slot_mapping) == q_pos.size and len(seq.read_slot_map) == len(seq)
            ids.append(np.asarray(seq.token_ids, dtype=np.int64)[q_pos])
            pos.append(q_pos)
            slots.append(np.asarray(seq.recompute_slot_mapping, dtype=np.int64))
            layout, shared_len = self._attention_read_layout(seq, use_query_relocation)
            reads.append(np.asarray(layout, dtype=np.int64))
            shared_lens.append(shared_len)
            shifts.append(seq.affix_start if self._affix_relocation_enabled else 0)
            block_starts.append(cu_q[-1] + seq.block_query_start())
            cu_q.append(cu_q[-1] + q_pos.size)
            cu_k.append(cu_k[-1] + len(layout))
        kv_lens = np.diff(cu_k)
        set_context(
            True, self._to_device(cu_q, torch.int32), self._to_device(cu_k, torch.int32),
            self._to_device(kv_lens, torch.int32), int(np.diff(cu_q).max()), int(kv_lens.max()),
            self._to_device(np.concatenate(slots), torch.int32), None, True,
            self._to_device(np.concatenate(reads), torch.int32),
            self._to_device(shared_lens, torch.int32) if use_query_relocation else None,
            None if relocation_materialized else self._to_device(shifts, torch.int32),
            total_k=int(cu_k[-1]), attention_plan=self._attention_plan(cu_q, cu_k))
        return (self._to_device(np.concatenate(ids), torch.int64), self._to_device(np.concatenate(pos), torch.int64),
                self._to_device(block_starts, torch.int32))

    def _device_read_side(self, group):
        """Per request: the read map in the order attention wants it and the number of shared slots in front
        (the device twin of ``_attention_read_layout``); plus the metadata tensors both context builders share."""
        packed = self._affix_relocation_enabled   # batched serving never materialises: query-side relocation
        reads, shared_lens, cu_k = [], [], [0]
        for seq in group:
            layout = seq.device_layout
            if packed and layout.read_packed is not None:
                reads.append(layout.read_packed)
                shared_lens.append(seq.affix_len - seq.num_anchor_tokens)
            else:
                reads.append(layout.read)
                shared_lens.append(0)
            cu_k.append(cu_k[-1] + len(seq))
        shifts = [seq.affix_start if self._affix_relocation_enabled else 0 for seq in group]
        return packed, reads, shared_lens, shifts, cu_k

    def _context_metadata(self, *rows):
        """Several short int32 host lists in one pinned buffer and one copy; returns the device slices."""
        sizes = [len(r) for r in rows]
        flat = self._to_device(np.concatenate([np.asarray(r, dtype=np.int64) for r in rows]), torch.int32)
        out, at = [], 0
        for n in sizes:
            out.append(flat[at:at + n])
            at += n
        return out

    def _prepare_caching_from_device_layouts(self, group):
        """``prepare_caching_acache`` when the requests' slot maps live on the device: a few concatenations of
        per-request tensors and one small metadata copy; no per-token host work, no read-back."""
        packed, reads, shared_lens, shifts, cu_k = self._device_read_side(group)
        layouts = [s.device_layout for s in group]
        n_rec = [s.num_anchor_tokens + len(s) - s.affix_len for s in group]
        cu_q = [0] + list(np.cumsum(n_rec))
        block_starts = [cu_q[b] + s.block_query_start() for b, s in enumerate(group)]
        kv_lens = np.diff(cu_k)
        d_cu_q, d_cu_k, d_kv, d_shared, d_shifts, d_starts = self._context_metadata(
            cu_q, cu_k, kv_lens, shared_lens, shifts, block_starts)
        positions = torch.cat([l.recompute_pos for l in layouts])
        input_ids = torch.cat([l.tokens.index_select(0, l.recompute_pos) for l in layouts])
        set_context(
            True, d_cu_q, d_cu_k, d_kv, int(max(n_rec)), int(kv_lens.max()),
            torch.cat([l.recompute_slots for l in layouts]), None, True, torch.cat(reads),
            d_shared if packed else None, d_shifts, total_k=int(cu_k[-1]),
            attention_plan=self._attention_plan(cu_q, cu_k))
        return input_ids, positions, d_starts

    def _prepare_decoding_from_device_layouts(self, group):
        """``prepare_decoding_acache`` from the device layouts: the current block's slots are a slice of each
        request's read map."""
        block_length = self.config.block_length
        packed, reads, shared_lens, shifts, cu_k = self._device_read_side(group)
        starts = [s.generation_start + s.current_block_idx * block_length for s in group]
        kv_lens = np.diff(cu_k)
        cu_q = np.arange(len(group) + 1) * block_length
        d_cu_q, d_cu_k, d_kv, d_shared, d_shifts = self._context_metadata(cu_q, cu_k, kv_lens, shared_lens, shifts)
        slots = torch.cat([s.device_layout.read[b0:b0 + block_length] for s, b0 in zip(group, starts)])
        positions = np.asarray(starts, dtype=np.int64)[:, None] + np.arange(block_length)[None, :]
        set_context(
            False, d_cu_q, d_cu_k, d_kv, block_length, int(kv_lens.max()), slots, None, True, torch.cat(reads),
            d_shared if packed else None, d_shifts, total_k=int(cu_k[-1]))
        return self._to_device(positions, torch.int64)

    def prepare_decoding_acache(self, seqs, active_indices=None):
        """Block refinement with affix reuse: the current block's tokens against the same read slot maps."""
        group = self._select(seqs, active_indices)
        block_length = self.config.block_length
        self._configure_affix_relocation(group)
        if all(s.device_layout is not None for s in group):
            return self._prepare_decoding_from_device_layouts(group)
        relocation_materialized = all(getattr(s, "relocated_affix_materialized", False) for s in group)
        use_query_relocation = self._use_query_side_affix_relocation(relocation_materialized)
        starts, slots, reads, shared_lens, shifts, cu_k = [], [], [], [], [], [0]
        for seq in group:
            start = seq.generation_start + seq.current_block_idx * block_length
            starts.append(start)
            slots.append(np.asarray(seq.read_slot_map[start:start + block_length], dtype=np.int64))
            layout, shared_len = self._attention_read_layout(seq, use_query_relocation)
            reads.append(np.asarray(layout, dtype=np.int64))
            shared_lens.append(shared_len)
            shifts.append(seq.affix_start if self._affix_relocation_enabled else 0)
            cu_k.append(cu_k[-1] + len(layout))
        kv_lens = np.diff(cu_k)
        positions = np.asarray(starts, dtype=np.int64)[:, None] + np.arange(block_length)[None, :]
        cu_q = np.arange(len(group) + 1) * block_length
        set_context(
            False, self._to_device(cu_q, torch.int32), self._to_device(cu_k, torch.int32),
            self._to_device(kv_lens, torch.int32), block_length, int(kv_lens.max()),
            self._to_device(np.concatenate(slots), torch.int32), None, True,
            self._to_device(np.concatenate(reads), torch.int32),
            self._to_device(shared_lens, torch.int32) if use_query_relocation else None,
            None if relocation_materialized else self._to_device(shifts, torch.int32),
            total_k=int(cu_k[-1]))
        return self._to_device(positions, torch.int64)

    # ------------------------------------------------------------------ generation (1473-1723, 2032-2277)
    @torch.inference_mode()
    def generate_with_dual_cache(self, prompts: list[Sequence]):
        """Full affix recompute baseline: every refresh re-encodes the whole request."""
        return self._generate(prompts, None, "dual_cache")

    @torch.inference_mode()
    def generate_with_acache(self, prompts: list[Sequence]):
        """Block-wise denoising with the shared affix K/V reused and only anchors recomputed."""
        timing = self._new_timing("acache", len(prompts))
        previous = self._active_timing
        self._active_timing = timing
        start = self._start_timing()
        prefix = self._prepare_acache(prompts)
        self._finish_timing(timing, "acache_metadata", start)
        self._active_timing = previous
        if not prefix:
            return self.generate_with_dual_cache(prompts)
        return self._generate(prompts, prefix, "acache", timing)

    def _generate(self, prompts, prefix, mode, timing=None):
        cfg = self.config
        device, model = self.device, self.model
        mask_id, block_length = cfg.mask_id, cfg.block_length
        temperature, remasking, threshold = cfg.temperature, cfg.remasking, cfg.threshold
        step = cfg.recompute_batch_size
        assert step > 0, "recompute_batch_size must be larger than 0"
        max_num_seqs = cfg.max_num_seqs if cfg.max_num_seqs > 0 else len(prompts)
        use_acache = prefix is not None
        dream = self._is_dream_model()
        if timing is None:
            timing = self._new_timing(mode, len(prompts))
        self.last_timing = timing or {}
        previous = self._active_timing
        self._active_timing = timing
        total_start = self._start_timing()

        # Positions index the model's rotary table, and the kernels clamp an out-of-table row for memory safety only
        # (it would come back unrotated).  The table has no hard limit: like the reference's, which builds it for
        # position_ids.max() + 1 (nano-vdllm/model/modeling_llada.py:910), it grows to the longest request here,
        # on the host, where the lengths are known.
        longest = max((len(seq) for seq in prompts), default=0)
        core = getattr(self.base_model, "model", None)
        if core is not None and hasattr(core, "config"):
            core.rope_positions = max(int(getattr(core, "rope_positions", 0)), longest)

        total_nfe = 0
        results = [None] * len(prompts)
        index_of = {seq.seq_id: i for i, seq in enumerate(prompts)}
        next_idx = 0
        batch: list[Sequence] = []

        def admit(allow_resize):
            nonlocal next_idx
            start = self._start_timing()
            if use_acache:
                fresh, next_idx = self._collect_admissible_sequences(prompts, next_idx, len(batch), max_num_seqs)
                admitted = self._admit_sequences_with_acache(batch, fresh, prefix, allow_resize)
                next_idx -= len(fresh) - admitted
            else:
                while (next_idx < len(prompts) and len(batch) < max_num_seqs
                       and self.block_manager.can_allocate(prompts[next_idx])):
                    self.block_manager.allocate(prompts[next_idx])
                    self._record_kv_cache_usage(timing)
                    batch.append(prompts[next_idx])
                    next_idx += 1
            self._finish_timing(timing, "scheduler", start)

        admit(True)
        batch_size = len(batch)
        if batch_size == 0 and prompts:
            budget = "ACache KV-cache budget" if use_acache else "KV-cache budget"
            raise RuntimeError(f"No requests could be admitted under the current {budget}.")
        working = torch.full((batch_size, block_length), mask_id, dtype=torch.int64, device=device)
        offsets = torch.arange(block_length, device=device)
        committed_rows = torch.zeros(1, dtype=torch.int32, device=device)   # rows that committed a token in a step

        def refresh(rows: torch.Tensor):
            """Cache refresh of the listed batch rows, ``recompute_batch_size`` requests per forward."""
            nonlocal total_nfe
            for i in range(0, len(rows), step):
                part = rows[i:i + step]
                start = self._start_timing()
                if use_acache:
                    input_ids, positions, block_starts = self.prepare_caching_acache(batch, part)
                    keep = block_starts.unsqueeze(1) + offsets
                else:
                    input_ids, positions, gen_starts, current = self.prepare_caching(batch, part)
                    keep = gen_starts.unsqueeze(1) + block_length * current.unsqueeze(1) + offsets
                if dream:
                    # Dream reads token i from the hidden state of the row in front of it (the first row of a
                    # request keeps its own): model_runner.py:63-66
                    group = self._select(batch, part)
                    if use_acache:
                        first = block_starts - self._to_device([s.block_query_start() for s in group], torch.int32)
                    else:
                        first = gen_starts - self._to_device([s.generation_start for s in group], torch.int32)
                    keep = torch.maximum(keep, first.unsqueeze(1) + 1) - 1
                self._finish_timing(timing, "cache_prepare", start)
                start = self._start_timing()
                logits = model(input_ids, position_ids=positions, logits_keep_indices=keep.flatten().long()).logits
                self._finish_timing(timing, "cache_forward", start)
                self._add_timing_count(timing, "cache_forward_calls", 1)
                self._add_timing_count(timing, "cache_forward_nfe", len(part))
                self._add_timing_count(timing, "cache_forward_tokens", int(input_ids.numel()))
                start = self._start_timing()
                logits = logits.view(len(part), block_length, -1)
                if dream:
                    # a refresh commits only the first token of the block (model_runner.py:68-78, 1548-1552)
                    working[part, 0] = self._sample_dream_seed_tokens(logits[:, 0])
                else:
                    working[part] = self._commit_from_logits(logits, working[part], temperature, remasking, threshold,
                                                             committed_rows)
                self._finish_timing(timing, "cache_update", start)
            total_nfe += len(rows)

        refresh(torch.arange(batch_size, device=device))

        last_active = None
        refreshed = adjusted = False
        decoding_positions = None
        decode_graph = None
        stalled = None   # device flag of the last refinement step: it left every [MASK] of its rows in place
        stalled_steps = 0
        # At temperature 0 the forward is deterministic: one step without a committed token would repeat for ever.
        # With sampling the next step draws other tokens, so only a run of such steps is taken as no progress.
        stall_limit = 1 if temperature == 0 else 8
        while batch:
            if stalled is not None:
                stalled_steps = stalled_steps + 1 if bool(stalled) else 0
                if stalled_steps >= stall_limit:
                    err = RuntimeError(
                        "Refinement step committed no token: the model predicts the mask token at every position "
                        "still masked in the active blocks, so block-wise decoding cannot make progress.")
                    err.partial_results = results   # requests that had finished before the loop gave up
                    raise err
            stalled = None
            has_mask = (working == mask_id).any(dim=1)
            done = ~has_mask
            if done.any():
                start = self._start_timing()
                done_rows = torch.where(done)[0]
                finished = []
                for row in done_rows.tolist():
                    seq = batch[row]
                    begin = seq.generation_start + seq.current_block_idx * block_length
                    seq.token_ids[begin:begin + block_length] = working[row].tolist()
                    if seq.device_layout is not None:
                        seq.device_layout.tokens[begin:begin + block_length] = working[row]
                    seq.current_block_idx += 1
                    if seq.current_block_idx >= seq.num_blocks_to_generate:
                        self.block_manager.deallocate(seq)
                        finished.append(row)
                        results[index_of[seq.seq_id]] = seq.generated_token_ids
                working[done_rows] = mask_id
                if finished:
                    adjusted = True
                    gone = set(finished)
                    batch[:] = [s for i, s in enumerate(batch) if i not in gone]
                    self._finish_timing(timing, "scheduler", start)
                    admit(len(batch) == 0)
                    start = self._start_timing()
                    survivors = torch.tensor([i for i in range(batch_size) if i not in gone],
                                             dtype=torch.int64, device=device)
                    kept = working[survivors]
                    batch_size = len(batch)
                    working = torch.full((batch_size, block_length), mask_id, dtype=torch.int64, device=device)
                    working[: len(survivors)] = kept
                self._finish_timing(timing, "scheduler", start)

                fresh_rows = torch.where((working == mask_id).all(dim=1))[0]
                if len(fresh_rows) > 0:
                    refreshed = True
                    refresh(fresh_rows)
                    continue

            if adjusted:
                adjusted = False
                has_mask = (working == mask_id).any(dim=1)
            active = torch.where(has_mask)[0]
            if len(active) > 0:
                if last_active is None or len(active) < len(last_active) or refreshed:
                    refreshed = False
                    last_active = active
                    start = self._start_timing()
                    decoding_positions = (self.prepare_decoding_acache if use_acache else self.prepare_decoding)(
                        batch, active)
                    decode_graph = None  # new slot maps and positions: the captured launches are stale
                    self._finish_timing(timing, "decode_prepare", start)
                start = self._start_timing()
                if cfg.decode_hip_graph:
                    if decode_graph is None:
                        decode_graph = self._capture_decode_graph(working[active], decoding_positions)
                        self._add_timing_count(timing, "decode_graph_captures", 1)
                    graph, graph_tokens, logits = decode_graph
                    graph_tokens.copy_(working[active])
                    graph.replay()
                else:
                    logits = model(working[active], position_ids=decoding_positions).logits
                if dream:  # block-local shift: position i is predicted by the row in front of it (56-61)
                    logits = torch.cat([logits[:, :1], logits[:, :-1]], dim=1)
                self._finish_timing(timing, "decode_forward", start)
                self._add_timing_count(timing, "decode_forward_calls", 1)
                self._add_timing_count(timing, "decode_forward_nfe", len(active))
                self._add_timing_count(timing, "decode_forward_tokens", len(active) * block_length)
                start = self._start_timing()
                committed_rows.zero_()
                working[active] = self._commit_from_logits(logits, working[active], temperature, remasking, threshold,
                                                           committed_rows)
                stalled = committed_rows == 0     # read at the top of the loop
                self._finish_timing(timing, "decode_update", start)
                total_nfe += len(active)

        reset_context()
        self._finish_timing(timing, "total", total_start)
        if timing is not None:
            timing["total_nfe"] = int(total_nfe)
        self._active_timing = previous
        return results, total_nfe

    def _capture_decode_graph(self, tokens, positions):
        """Record one block-refinement forward (``tokens`` ``[n, block_length]`` at ``positions``, attention
        metadata from the current ``Context``) into a HIP graph.  Returns ``(graph, token buffer, logits buffer)``:
        copy the step's tokens into the buffer, replay, read the logits.  Every launch of the forward — library
        GEMMs, the fused rotary + scatter, attention — is recorded from the stream it is enqueued on; nothing in
        it synchronises with the host.  The first forward of a new shape runs eagerly on a side stream first so
        that library handles and workspaces exist before the capture."""
        static_tokens = tokens.clone()
        shape = (tuple(tokens.shape), len(self._llada_blocks()))
        if shape not in self._decode_graph_warm:
            side = torch.cuda.Stream(device=self.device)
            side.wait_stream(torch.cuda.current_stream(self.device))
            with torch.cuda.stream(side):
                self.model(static_tokens, position_ids=positions)
            torch.cuda.current_stream(self.device).wait_stream(side)
            self._decode_graph_warm.add(shape)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            logits = self.model(static_tokens, position_ids=positions).logits
        return graph, static_tokens, logits

    def _sample_dream_seed_tokens(self, logits):
        """First token of a freshly refreshed block: arg-max, or a categorical draw at temperature > 0."""
        temperature = float(self.config.temperature)
        if temperature > 0:
            return torch.distributions.Categorical(probs=torch.softmax(logits.float() / temperature, dim=-1)).sample()
        return logits.argmax(dim=-1)

    # ------------------------------------------------------------------ token transfer (2279-2314)
    def _commit_from_logits(self, logits, current_blocks, temperature, remasking, threshold, committed_rows):
        """``current_blocks`` with this step's picks written in, by the rule of ``get_transfer_index``.  With
        confidence-based remasking and logits the confidence kernel takes, proposal, confidence and commit are
        two or three launches; otherwise the tensor formulation.  ``committed_rows`` counts rows that committed.
        ``current_blocks`` is the caller's own copy (the result of indexing the working blocks) and may be
        written in place."""
        fused = (remasking == "low_confidence" and logits.is_cuda and logits.is_contiguous()
                 and logits.data_ptr() % 16 == 0 and (logits.shape[-1] * logits.element_size()) % 16 == 0)
        if not fused:
            x0, transfer = self.get_transfer_index(logits, temperature, remasking,
                                                   current_blocks == self.config.mask_id, current_blocks, threshold)
            committed_rows += transfer.any(dim=1).sum().to(torch.int32)
            return torch.where(transfer, x0, current_blocks)
        if temperature == 0:
            x0, x0_p = ops.argmax_confidence(logits)
        else:
            x0 = torch.argmax(add_gumbel_noise(logits, temperature=temperature), dim=-1)
            _, x0_p = ops.argmax_confidence(logits, picks=x0)
        out = current_blocks if current_blocks.is_contiguous() else current_blocks.contiguous()
        ops.commit_tokens(out, x0.view_as(out).contiguous(), x0_p.view_as(out).contiguous(), committed_rows,
                          self.config.mask_id, threshold)
        return out

    def get_transfer_index(self, logits, temperature, remasking, mask_index, x, threshold=0.9):
        """Pick the tokens to commit: confidence >= threshold among masked positions, at least one per row."""
        fused = (logits.is_cuda and logits.stride(-1) == 1 and logits.data_ptr() % 16 == 0
                 and (logits.shape[-1] * logits.element_size()) % 16 == 0 and logits.is_contiguous())
        if remasking == "low_confidence" and fused:
            # one streaming pass per row: arg-max token and exp(logit - logsumexp) together
            if temperature == 0:
                x0, x0_p = ops.argmax_confidence(logits)
            else:
                x0 = torch.argmax(add_gumbel_noise(logits, temperature=temperature), dim=-1)
                _, x0_p = ops.argmax_confidence(logits, picks=x0)
        elif remasking == "low_confidence":
            x0 = torch.argmax(add_gumbel_noise(logits, temperature=temperature), dim=-1)
            flat = logits.reshape(-1, logits.shape[-1])
            picks = x0.reshape(-1)
            conf = torch.empty(picks.shape, dtype=torch.float32, device=logits.device)
            for lo in range(0, flat.shape[0], 64):  # bounded fp32 temporaries over the vocabulary
                rows = flat[lo:lo + 64].float()
                chosen = rows.gather(-1, picks[lo:lo + 64, None]).squeeze(-1)
                conf[lo:lo + 64] = torch.exp(chosen - torch.logsumexp(rows, dim=-1))
            x0_p = conf.view_as(x0)
        elif remasking == "random":
            x0 = torch.argmax(add_gumbel_noise(logits, temperature=temperature), dim=-1)
            x0_p = torch.rand(x0.shape, device=x0.device)
        else:
            raise NotImplementedError(remasking)
        x0 = torch.where(mask_index, x0, x)
        # A position whose prediction is [MASK] itself cannot be committed: writing it changes nothing, and when it
        # is the row's forced pick the same forward repeats for ever (the reference's rule, model_runner.py:2279-2314,
        # never terminates there).  Such positions are left out of the pick; writing [MASK] over [MASK] is a no-op,
        # so wherever the reference's loop terminates the committed tokens are the same.
        committable = mask_index & (x0 != self.config.mask_id)
        confidence = torch.where(committable, x0_p, torch.full_like(x0_p, -math.inf))
        transfer = (confidence >= threshold) & committable
        # a row with committable positions and none above the threshold commits its most confident one
        stuck = committable.any(dim=1) & ~transfer.any(dim=1)
        forced = torch.zeros_like(transfer).scatter_(1, confidence.argmax(dim=1, keepdim=True), stuck.unsqueeze(1))
        return x0, transfer | forced
