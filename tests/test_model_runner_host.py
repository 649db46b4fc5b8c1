"""ModelRunner host logic that needs no GPU (golden vectors of the reference's CPU tests,
nano-vdllm/tests/test_model_runner_acache.py:26-61 and 106-124, plus admission failure)."""
from types import SimpleNamespace

import pytest
import torch

from acache_amd import Config, Sequence
from acache_amd.llada import LLaDAConfig, LLaDAModelLM
from acache_amd.model_runner import ModelRunner


def test_attention_read_layout_packs_shared_slots_for_query_relocation():
    runner = object.__new__(ModelRunner)
    runner.shared_prefix_len = 3
    seq = SimpleNamespace(affix_start=2, shared_slot_offset=0, read_slot_map=[8, 9, 0, 10, 2, 11])
    assert runner._attention_read_layout(seq, True) == ([0, 2, 8, 9, 10, 11], 2)


def test_attention_read_layout_keeps_logical_order_for_key_relocation():
    runner = object.__new__(ModelRunner)
    runner.shared_prefix_len = 3
    seq = SimpleNamespace(affix_start=2, shared_slot_offset=0, read_slot_map=[8, 9, 0, 10, 2, 11])
    assert runner._attention_read_layout(seq, False) == ([8, 9, 0, 10, 2, 11], 0)


@pytest.mark.parametrize(
    ("max_num_seqs", "relocation_materialized", "expected"),
    [(0, False, True), (16, False, True), (1, False, False), (0, True, False)],
)
def test_query_side_relocation_treats_zero_as_unlimited_batching(max_num_seqs, relocation_materialized, expected):
    runner = object.__new__(ModelRunner)
    runner._affix_relocation_enabled = True
    runner.config = SimpleNamespace(max_num_seqs=max_num_seqs)
    assert runner._use_query_side_affix_relocation(relocation_materialized) is expected


def test_profile_timing_helpers_are_noop_when_disabled(monkeypatch):
    runner = object.__new__(ModelRunner)
    runner.profile_timing = False
    runner.device = SimpleNamespace(type="cuda")
    monkeypatch.setattr(torch.cuda, "synchronize",
                        lambda *a, **k: pytest.fail("CUDA sync should not run when profile_timing is disabled"))
    monkeypatch.setattr("acache_amd.model_runner.time.perf_counter",
                        lambda: pytest.fail("perf_counter should not run when profile_timing is disabled"))
    assert runner._new_timing("dual_cache", 1) is None
    assert runner._start_timing() is None
    runner._finish_timing(None, "total", None)
    runner._add_timing_count(None, "calls")


def _tiny_runner(**overrides):
    cfg = LLaDAConfig(vocab_size=64, d_model=128, n_heads=2, n_layers=1, mlp_hidden_size=64,
                      max_sequence_length=64, mask_token_id=63)
    model = LLaDAModelLM(cfg).to(torch.bfloat16).eval()
    serve = Config(hf_config=cfg, mask_id=63, recompute_batch_size=2, gen_length=4, block_length=4,
                   cache_block_size=8, num_kvcache_blocks=2, temperature=0.0, threshold=0.0,
                   enable_acache=True, anchor_ratio=0.5)
    for k, v in overrides.items():
        setattr(serve, k, v)
    return ModelRunner(model, serve)


def test_kv_cache_layout_and_block_bytes_on_cpu():
    runner = _tiny_runner()
    assert runner.kv_cache.shape == (2, 1, 2, 8, 2, 64) and runner.kv_cache.dtype == torch.bfloat16
    assert runner.kv_cache_block_bytes == 2 * 1 * 8 * 2 * 64 * 2
    attn = runner._llada_blocks()[0].attn
    assert attn.k_cache.data_ptr() == runner.kv_cache[0, 0].data_ptr()
    assert attn.v_cache.data_ptr() == runner.kv_cache[1, 0].data_ptr()
    assert len(runner.block_manager.free_block_ids) == 2


def test_block_exhaustion_stops_admission_with_runtime_error():
    """Failure handling that a host test can force: no request fits the KV budget (model_runner.py:1511-1512, 2080-2081)."""
    runner = _tiny_runner(num_kvcache_blocks=1)
    runner.allocate_kv_cache(1)
    seqs = [Sequence(list(range(2, 14)), gen_length=4, cache_block_size=8, block_length=4, mask_id=63)]  # 16 tokens -> 2 blocks
    with pytest.raises(RuntimeError, match="No requests could be admitted"):
        runner.generate_with_dual_cache(seqs)


def test_inconsistent_affix_is_rejected_before_any_device_work():
    runner = _tiny_runner()
    a = Sequence([2, 3, 4, 5], gen_length=4, cache_block_size=8, block_length=4, mask_id=63, prompt_affix_len=2)
    b = Sequence([2, 9, 4, 5], gen_length=4, cache_block_size=8, block_length=4, mask_id=63, prompt_affix_len=2)
    c = Sequence([2, 3, 4, 5], gen_length=4, cache_block_size=8, block_length=4, mask_id=63, prompt_affix_len=3)
    with pytest.raises(ValueError, match="identical explicit affix tokens"):
        runner.generate_with_acache([a, b])
    with pytest.raises(ValueError, match="same explicit affix length"):
        runner._prepare_acache([a, c])
    assert runner._prepare_acache([a]) == (2, 3) and a.num_anchor_tokens == 1


def test_collect_admissible_sequences_respects_free_blocks():
    runner = _tiny_runner(num_kvcache_blocks=3)
    runner.allocate_kv_cache(3)
    seqs = [Sequence(list(range(2, 14)), gen_length=4, cache_block_size=8, block_length=4, mask_id=63) for _ in range(3)]
    got, nxt = runner._collect_admissible_sequences(seqs, 0, 0, 8)
    assert got == seqs[:1] and nxt == 1            # 2 blocks each, 3 free -> one request
    got, nxt = runner._collect_admissible_sequences(seqs, 0, 0, 0)
    assert got == [] and nxt == 0


class _StubForward:
    """Stands in for the model in the generation loop: returns logits from a rule over the tokens it is shown, so
    the loop's control flow runs on the CPU without any attention kernel."""

    def __init__(self, rule, vocab=64):
        self.rule, self.vocab, self.calls = rule, vocab, 0

    def __call__(self, input_ids, position_ids=None, logits_keep_indices=None):
        self.calls += 1
        if logits_keep_indices is not None:      # cache refresh: one logit row per kept position
            tokens = input_ids[logits_keep_indices]
        else:                                    # block refinement: [requests, block_length]
            tokens = input_ids
        picks = self.rule(tokens)
        logits = torch.zeros(*tokens.shape, self.vocab)
        logits.scatter_(-1, picks.unsqueeze(-1), 4.0)
        return SimpleNamespace(logits=logits)


def _stub_requests(n=2):
    return [Sequence([2 + i, 3, 4, 5], gen_length=8, cache_block_size=8, block_length=4, mask_id=63) for i in range(n)]


def test_refinement_loop_raises_when_a_step_commits_nothing():
    """A head that answers [MASK] everywhere can never fill a block: the loop must stop with an error instead of
    repeating the same forward (the reference's loop, model_runner.py:1554-1723, has no such bound)."""
    runner = _tiny_runner(num_kvcache_blocks=8, enable_acache=False, threshold=0.9)
    runner.allocate_kv_cache(8)
    runner.model = _StubForward(lambda tokens: torch.full_like(tokens, 63))
    with pytest.raises(RuntimeError, match="committed no token"):
        runner.generate_with_dual_cache(_stub_requests())
    assert runner.model.calls <= 3   # one refresh forward, one refinement forward, no spin


def test_with_sampling_one_step_without_a_commit_is_not_the_end():
    """temperature > 0: a step in which every draw is [MASK] may be followed by one that commits tokens (the
    reference keeps looping, model_runner.py:2242-2271); only a run of such steps is given up on, and the error then
    carries the requests that had finished."""
    runner = _tiny_runner(num_kvcache_blocks=8, enable_acache=False, threshold=0.9, temperature=0.5)
    runner.allocate_kv_cache(8)
    state = {"refinements": 0}

    def rule(tokens):
        if tokens.dim() == 2:                    # refinement forward: every other one answers [MASK] everywhere
            state["refinements"] += 1
            if state["refinements"] % 2 == 1:
                return torch.full_like(tokens, 63)
        return torch.full_like(tokens, 7)

    stub = _StubForward(rule)
    stub_call = stub.__call__

    def peaked(*args, **kwargs):                 # refinement: a head so peaked that the Gumbel draw is its arg-max
        out = stub_call(*args, **kwargs)
        if kwargs.get("logits_keep_indices") is None:
            out.logits = out.logits * 50.0       # (a block refresh stays below the threshold: one forced token per row)
        return out

    runner.model = peaked
    torch.manual_seed(0)
    out, nfe = runner.generate_with_dual_cache(_stub_requests())
    assert all(len(o) == 8 and 63 not in o for o in out)
    assert state["refinements"] >= 2
    # a head that never answers anything else is still given up on, after a bounded number of steps
    runner2 = _tiny_runner(num_kvcache_blocks=8, enable_acache=False, threshold=0.9, temperature=0.5)
    runner2.allocate_kv_cache(8)
    always = _StubForward(lambda tokens: torch.full_like(tokens, 63))
    always_call = always.__call__

    def peaked_mask(*args, **kwargs):
        out = always_call(*args, **kwargs)
        out.logits = out.logits * 50.0
        return out

    runner2.model = peaked_mask
    with pytest.raises(RuntimeError, match="committed no token") as info:
        runner2.generate_with_dual_cache(_stub_requests())
    assert always.calls <= 1 + 8 + 1 and hasattr(info.value, "partial_results")


def test_forced_pick_skips_positions_that_predict_the_mask_token():
    """Column 0 answers [MASK] until the rest of its block is filled, with the same confidence as every other
    position; the forced one-token-per-step pick must take the other positions first and the run must finish."""
    runner = _tiny_runner(num_kvcache_blocks=8, enable_acache=False, threshold=0.99)
    runner.allocate_kv_cache(8)

    def rule(tokens):
        picks = torch.full_like(tokens, 7)
        flat = tokens.reshape(-1, 4)
        others_masked = (flat[:, 1:] == 63).any(dim=1)
        picks.view(-1, 4)[others_masked, 0] = 63
        return picks

    runner.model = _StubForward(rule)
    out, nfe = runner.generate_with_dual_cache(_stub_requests())
    assert out == [[7] * 8, [7] * 8]
    assert nfe == 2 * 2 * 4          # one token per request and step: 4 steps for each of 2 blocks of 2 requests


def test_out_of_memory_at_admission_shrinks_retries_and_restores(capsys):
    """Host logic of the resize path (model_runner.py:592-638, 862-955) with the two device steps stubbed: the
    probe fails once with an out-of-memory error, the cache loses four blocks, the affix precompute is redone for
    the new cache, the same request is retried, and the configured size is back afterwards."""
    runner = _tiny_runner(num_kvcache_blocks=12)
    runner.allocate_kv_cache(12)
    seqs = [Sequence([2, 3, 4, 5 + i], gen_length=4, cache_block_size=8, block_length=4, mask_id=63,
                     prompt_affix_len=2) for i in range(2)]
    prefix = runner._prepare_acache(seqs)
    log = []

    def precompute(tokens):
        log.append(("affix", int(runner.config.num_kvcache_blocks)))
        runner.shared_prefix_len, runner.shared_prefix_blocks = len(tokens), 1
        runner.shared_prefix_token_ids, runner.acache_ready = tuple(tokens), True

    def probe(batch):
        log.append(("probe", int(runner.config.num_kvcache_blocks)))
        if sum(1 for what, _ in log if what == "probe") == 2:
            raise torch.OutOfMemoryError("forced by the test")
        return [[1] for _ in batch]

    runner._precompute_shared_prefix = precompute
    runner._compute_anchor_positions_batch = probe
    runner._prepare_admitted_sequences_for_acache(seqs, prefix, allow_kv_cache_resize=True)
    assert log == [("affix", 12), ("probe", 12), ("probe", 12), ("affix", 8), ("probe", 8), ("affix", 12)]
    assert "from 12 to 8" in capsys.readouterr().out
    assert runner.kv_cache.shape[2] == 12 and runner.block_manager.num_blocks == 12 and runner.acache_ready
    assert [s.anchor_positions for s in seqs] == [[1], [1]]

    # the floor: shared affix block + the one request a probe holds = 2 blocks; at the floor the error surfaces
    runner.allocate_kv_cache(2)
    log.clear()
    runner._compute_anchor_positions_batch = lambda batch: (_ for _ in ()).throw(torch.OutOfMemoryError("always"))
    with pytest.raises(torch.OutOfMemoryError):
        runner._prepare_admitted_sequences_for_acache(seqs, prefix, allow_kv_cache_resize=True)
    assert runner.kv_cache.shape[2] == 2
    # without permission to resize nothing is shrunk
    runner.allocate_kv_cache(12)
    with pytest.raises(torch.OutOfMemoryError):
        runner._prepare_admitted_sequences_for_acache(seqs, prefix, allow_kv_cache_resize=False)
    assert runner.kv_cache.shape[2] == 12


def test_requests_longer_than_the_configured_length_grow_the_rotary_table():
    """The reference's rotary table grows with the positions it is asked for (nano-vdllm/model/modeling_llada.py:910);
    the engine does the same on the host before the first forward instead of leaving out-of-table rows unrotated."""
    from acache_amd.rope import rope_table

    runner = _tiny_runner(num_kvcache_blocks=16, enable_acache=False)
    runner.allocate_kv_cache(16)
    core = runner.base_model.model
    assert core.config.max_sequence_length == 64
    seen = {}

    def forward(input_ids, position_ids=None, logits_keep_indices=None):
        seen["rows"] = max(core.config.max_sequence_length, int(getattr(core, "rope_positions", 0)))
        tokens = input_ids[logits_keep_indices] if logits_keep_indices is not None else input_ids
        logits = torch.zeros(*tokens.shape, 64)
        logits[..., 7] = 9.0
        return SimpleNamespace(logits=logits)

    runner.model = forward
    long_request = Sequence(list(range(2, 62)), gen_length=8, cache_block_size=8, block_length=4, mask_id=63)  # 68 > 64
    out, _ = runner.generate_with_dual_cache([long_request])
    assert out == [[7] * 8] and seen["rows"] == 68
    # the rotary module hands out as many rows as it is asked for, equal to the closed-form table
    sin, cos = core.transformer["blocks"][0].rotary_emb.get_rotary_embedding(68, torch.device("cpu"))
    want_cos, want_sin = rope_table(68, 64, core.config.rope_theta)
    assert sin.shape[0] == 68 and torch.equal(cos, want_cos) and torch.equal(sin, want_sin)


def test_model_runner_takes_over_a_checkpoint_model_object():
    """``ModelRunner(model, config)`` with the model class of another package (the reference's caller passes its
    own, model_runner.py:15-19): the runner runs the engine model built around the same parameter tensors."""
    from .test_generate_acache_host import CheckpointModelDouble, _fixture_weights, _llada_checkpoint_config

    weights = _fixture_weights()
    checkpoint_model = CheckpointModelDouble(_llada_checkpoint_config(), weights)
    serve = Config(hf_config=checkpoint_model.config, mask_id=63, recompute_batch_size=2, gen_length=4, block_length=4,
                   cache_block_size=8, num_kvcache_blocks=2, temperature=0.0, threshold=0.0)
    runner = ModelRunner(checkpoint_model, serve)
    assert isinstance(runner.model, LLaDAModelLM) and runner.base_model is runner.model
    q = runner._llada_blocks()[0].q_proj.weight
    assert q.data_ptr() == weights["model.transformer.blocks.0.q_proj.weight"].data_ptr()
    assert runner.kv_cache.shape == (2, 2, 2, 8, 2, 128)      # [K/V, layers, blocks, block size, KV heads, head dim]
    with pytest.raises(TypeError, match="checkpoint model object"):
        ModelRunner(object(), serve)
