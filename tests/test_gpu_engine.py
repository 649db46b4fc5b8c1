"""Engine integration on the GPU with a tiny random-init LLaDA-shaped model.

Mirrors the invariants of the reference's engine tests
(nano-vdllm/tests/test_model_runner_acache.py:305-430, 470-590, 605-687): shared-affix
precompute state, batched == single anchor selection, ratio-1.0 ACache logits equal
full-recompute logits for prefix / infix / suffix placement (tolerance 5e-2 there and here),
and end-to-end generation for mixed layouts.  Head dim is 64 unless a test says otherwise.
"""
import pytest
import torch

from acache_amd import Config, Sequence
from acache_amd.llada import LLaDAConfig, LLaDAModelLM
from acache_amd.model_runner import ModelRunner
from acache_amd.utils import reset_context

pytestmark = pytest.mark.gpu


def _model(device, seed=0, layers=2, d_model=256):
    torch.manual_seed(seed)
    cfg = LLaDAConfig(vocab_size=64, d_model=d_model, n_heads=4, n_layers=layers, mlp_hidden_size=128,
                      max_sequence_length=64, mask_token_id=63, rope_theta=10000.0)
    model = LLaDAModelLM(cfg, init_std=0.08).to(device=device, dtype=torch.bfloat16).eval()
    return cfg, model


def _serve(cfg, **kw):
    base = dict(hf_config=cfg, mask_id=63, recompute_batch_size=2, gen_length=4, block_length=4,
                cache_block_size=8, num_kvcache_blocks=8, temperature=0.0, threshold=0.0,
                enable_acache=True, anchor_ratio=0.25, selection_mode="top", use_reference_attention=False)
    base.update(kw)
    return Config(**base)


def test_prepare_acache_tiny_model(device):
    cfg, model = _model(device)
    runner = ModelRunner(model, _serve(cfg))
    Sequence([1], gen_length=1, cache_block_size=8, block_length=1, mask_id=63)  # advance the global counter
    seqs = [
        Sequence([2, 3, 4, 5], gen_length=4, cache_block_size=8, block_length=4, mask_id=63, prompt_affix_len=2),
        Sequence([2, 3, 4, 6], gen_length=4, cache_block_size=8, block_length=4, mask_id=63, prompt_affix_len=2),
    ]
    assert runner.kv_cache.shape[2] == 8
    prefix = runner._prepare_acache(seqs)
    assert prefix == (2, 3)
    with torch.inference_mode():
        runner._prepare_admitted_sequences_for_acache(seqs, prefix, allow_kv_cache_resize=True)
    assert runner.shared_prefix_len == 2 and runner.shared_prefix_blocks == 1
    assert runner.shared_prefix_token_ids == (2, 3)
    assert all(len(s.anchor_positions) == 1 and 0 <= s.anchor_positions[0] < 2 for s in seqs)
    # the probe left no temporary state behind
    assert all(not s.block_table for s in seqs)
    assert runner.block_manager.used_block_ids == {0}


def test_admission_out_of_memory_shrinks_the_cache_and_restores_it(device, capsys):
    """An out-of-memory error in the anchor probe gives four KV blocks back, redoes the affix precompute in the
    smaller cache, retries the same request, and ends with the configured cache size and a valid shared affix
    (model_runner.py:592-638, 862-955).  The error is raised from the host; no allocation is actually refused."""
    cfg, model = _model(device)

    def requests():
        return [Sequence([2, 3, 4, 5 + i], gen_length=4, cache_block_size=8, block_length=4, mask_id=63,
                         prompt_affix_len=2) for i in range(2)]

    def admit(fail_on, allow):
        runner = ModelRunner(model, _serve(cfg, num_kvcache_blocks=12))
        seqs = requests()
        prefix = runner._prepare_acache(seqs)
        real, sizes = runner._select_anchors_on_device, []

        def probe(batch):
            sizes.append(int(runner.config.num_kvcache_blocks))
            if len(sizes) == fail_on:
                raise torch.OutOfMemoryError("forced by the test")
            return real(batch)

        runner._select_anchors_on_device = probe
        with torch.inference_mode():
            runner._prepare_admitted_sequences_for_acache(seqs, prefix, allow_kv_cache_resize=allow)
        return runner, seqs, sizes

    plain, plain_seqs, sizes = admit(0, True)
    assert sizes == [12, 12]
    runner, seqs, sizes = admit(2, True)
    assert sizes == [12, 12, 8]                      # second request: failed at 12 blocks, retried at 8
    assert "shrinking KV cache blocks from 12 to 8" in capsys.readouterr().out
    assert runner.config.num_kvcache_blocks == 12 and runner.kv_cache.shape[2] == 12
    assert runner.acache_ready and runner.shared_prefix_token_ids == (2, 3)
    assert runner.block_manager.used_block_ids == {0} and runner.block_manager.num_free_blocks == 11
    assert [s.anchor_positions for s in seqs] == [s.anchor_positions for s in plain_seqs]
    attn = runner._llada_blocks()[0].attn
    assert attn.k_cache.data_ptr() == runner.kv_cache[0, 0].data_ptr()
    assert torch.equal(runner._shared_affix_k(0), plain._shared_affix_k(0))
    with pytest.raises(torch.OutOfMemoryError):
        admit(1, False)


def test_batched_anchor_selection_matches_single_sequence_selection(device):
    cfg, model = _model(device)
    serve = _serve(cfg, anchor_ratio=0.5)
    runner = ModelRunner(model, serve)
    affix = [2, 3, 9, 11, 17, 21]
    seqs = [
        Sequence(affix + [4, 5], gen_length=4, cache_block_size=8, block_length=4, mask_id=63, prompt_affix_len=6),
        Sequence(affix + [7, 8], gen_length=4, cache_block_size=8, block_length=4, mask_id=63, prompt_affix_len=6),
    ]
    with torch.inference_mode():
        runner._precompute_shared_prefix(affix)
        for s in seqs:
            s.enable_acache(6, serve.anchor_ratio)
        single = [runner._compute_anchor_positions(s) for s in seqs]
        batched = runner._compute_anchor_positions_batch(seqs)
    assert batched == single
    assert all(len(a) == 3 and a == sorted(a) and all(0 <= p < 6 for p in a) for a in single)


@pytest.mark.parametrize(
    ("tokens", "affix_start", "affix_end", "generation_start"),
    [
        ([2, 3, 4, 5], 0, 2, None),
        ([4, 2, 3, 5], 1, 3, None),
        ([4, 63, 63, 2, 3], 3, 5, 1),
        (list(range(2, 22)), 5, 16, None),        # longer infix affix, crosses a cache block
    ],
)
@pytest.mark.parametrize("max_num_seqs", [4, 1])
@pytest.mark.parametrize("d_model", [256, 64, 384])
def test_full_recomputation_matches_baseline_for_all_affix_layouts(device, tokens, affix_start, affix_end,
                                                                   generation_start, max_num_seqs, d_model):
    """anchor_ratio = 1.0: every affix token is recomputed, so refresh logits must equal the full-recompute
    baseline.  max_num_seqs = 4 exercises query-side relocation, 1 the materialised / key-side path.  d_model 64
    is the reference tests' own tiny configuration (4 heads of 16); 384 gives heads of 96."""
    cfg, model = _model(device, seed=7, d_model=d_model)

    def serve(enable):
        return _serve(cfg, recompute_batch_size=1, gen_length=2, block_length=2, max_num_seqs=max_num_seqs,
                      enable_acache=enable, anchor_ratio=1.0, num_kvcache_blocks=12)

    def make():
        return Sequence(tokens, gen_length=2, block_length=2, cache_block_size=8, mask_id=63,
                        prompt_affix_start=affix_start, prompt_affix_end=affix_end, generation_start=generation_start)

    with torch.inference_mode():
        base = ModelRunner(model, serve(False))
        bseq = make()
        base.block_manager.allocate(bseq)
        bseq.finalize_slot_mapping()
        ids, pos, _, _ = base.prepare_caching([bseq])
        base_logits = model(ids, position_ids=pos).logits.float()
        reset_context()

        ac = ModelRunner(model, serve(True))
        aseq = make()
        affix_tokens = ac._prepare_acache([aseq])
        ac._precompute_shared_prefix(list(affix_tokens))
        aseq.set_anchor_positions(list(range(affix_start, affix_end)))
        ac._reserve_single_sequence_relocation_workspace(aseq)
        ac.block_manager.allocate(aseq)
        ac._finalize_sequence_layout(aseq)
        ids, pos, _ = ac.prepare_caching_acache([aseq])
        ac_logits = model(ids, position_ids=pos).logits.float()
        reset_context()
    assert aseq.recompute_positions == list(range(len(aseq)))
    torch.testing.assert_close(ac_logits, base_logits, rtol=5e-2, atol=5e-2)


@pytest.mark.parametrize("max_num_seqs", [4, 1])
def test_full_recomputation_matches_baseline_at_llada_head_geometry(device, max_num_seqs):
    """The same invariant at the real attention geometry: 32 heads of 128 (d_model 4096), 256-token cache blocks,
    a 300-token infix affix that crosses a cache block, a 32-token generation block; two layers keep it small.
    Exercises the head-dim-128 attention, fused rotary + scatter and relocation kernels inside the engine."""
    torch.manual_seed(11)
    mask = 511
    cfg = LLaDAConfig(vocab_size=512, d_model=4096, n_heads=32, n_layers=2, mlp_hidden_size=512,
                      max_sequence_length=1024, mask_token_id=mask, rope_theta=500000.0)
    model = LLaDAModelLM(cfg, init_std=0.02).to(device=device, dtype=torch.bfloat16).eval()
    g = torch.Generator().manual_seed(5)
    draw = lambda n: torch.randint(2, 500, (n,), generator=g).tolist()
    head, affix, tail = draw(40), draw(300), draw(30)
    tokens, a0, a1 = head + affix + tail, 40, 340

    def serve(enable):
        return Config(hf_config=cfg, mask_id=mask, recompute_batch_size=1, gen_length=32, block_length=32,
                      cache_block_size=256, num_kvcache_blocks=10, temperature=0.0, threshold=0.0,
                      enable_acache=enable, anchor_ratio=1.0, selection_mode="top", max_num_seqs=max_num_seqs)

    def make():
        return Sequence(tokens, gen_length=32, block_length=32, cache_block_size=256, mask_id=mask,
                        prompt_affix_start=a0, prompt_affix_end=a1)

    with torch.inference_mode():
        base = ModelRunner(model, serve(False))
        bseq = make()
        base.block_manager.allocate(bseq)
        bseq.finalize_slot_mapping()
        ids, pos, _, _ = base.prepare_caching([bseq])
        base_logits = model(ids, position_ids=pos).logits.float()
        reset_context()

        ac = ModelRunner(model, serve(True))
        aseq = make()
        affix_tokens = ac._prepare_acache([aseq])
        ac._precompute_shared_prefix(list(affix_tokens))
        aseq.set_anchor_positions(list(range(a0, a1)))
        ac._reserve_single_sequence_relocation_workspace(aseq)
        ac.block_manager.allocate(aseq)
        ac._finalize_sequence_layout(aseq)
        ids, pos, _ = ac.prepare_caching_acache([aseq])
        ac_logits = model(ids, position_ids=pos).logits.float()
        reset_context()
    assert ac.shared_prefix_blocks == 2 and aseq.recompute_positions == list(range(len(aseq)))
    assert float(base_logits.abs().max()) > 0.5          # the comparison is not between two all-zero tensors
    torch.testing.assert_close(ac_logits, base_logits, rtol=5e-2, atol=5e-2)


@pytest.mark.parametrize("max_num_seqs", [4, 1])
def test_partial_anchor_refresh_matches_dense_recompute_of_the_same_layout(device, max_num_seqs):
    """anchor_ratio < 1: refresh logits must equal a dense forward in which the non-anchor affix keys are the
    cached shared keys moved to the request's positions — the semantics of affix reuse, for any relocation mode."""
    cfg, model = _model(device, seed=3)
    tokens = [5, 6, 7] + list(range(20, 32)) + [8, 9]      # affix = 12 tokens at positions 3..14
    a0, a1 = 3, 15
    with torch.inference_mode():
        outs = {}
        for mode in ("acache", "oracle_layout"):
            runner = ModelRunner(model, _serve(cfg, recompute_batch_size=1, gen_length=4, block_length=4,
                                               max_num_seqs=max_num_seqs if mode == "acache" else 1,
                                               anchor_ratio=0.5, num_kvcache_blocks=16))
            seq = Sequence(tokens, gen_length=4, block_length=4, cache_block_size=8, mask_id=63,
                           prompt_affix_start=a0, prompt_affix_end=a1)
            prefix = runner._prepare_acache([seq])
            runner._precompute_shared_prefix(list(prefix))
            seq.set_anchor_positions([3, 5, 8, 9, 12, 14])
            if mode == "acache":
                runner._reserve_single_sequence_relocation_workspace(seq)
            else:
                runner._reserve_single_sequence_relocation_workspace(seq, force=True)  # always materialise
            runner.block_manager.allocate(seq)
            runner._finalize_sequence_layout(seq)
            ids, pos, _ = runner.prepare_caching_acache([seq])
            outs[mode] = model(ids, position_ids=pos).logits.float()
            reset_context()
    torch.testing.assert_close(outs["acache"], outs["oracle_layout"], rtol=5e-2, atol=5e-2)


def test_generate_with_acache_mixed_layouts_and_result_order(device):
    cfg, model = _model(device)
    serve = _serve(cfg, recompute_batch_size=1, max_num_seqs=1, anchor_ratio=0.5)
    runner = ModelRunner(model, serve)
    seqs = [
        Sequence([2, 3, 4, 5], gen_length=4, cache_block_size=8, block_length=4, mask_id=63, prompt_affix_len=2),
        Sequence([2, 3, 4, 6], gen_length=4, cache_block_size=8, block_length=4, mask_id=63, prompt_affix_len=2),
        Sequence([4, 10, 11, 12, 13, 2, 3], gen_length=4, generation_start=1, cache_block_size=8, block_length=4,
                 mask_id=63, prompt_affix_start=5, prompt_affix_end=7),
    ]
    calls = []
    real = runner._compute_anchor_positions_batch

    def spy(batch):
        calls.append(len(batch))
        return real(batch)

    runner._compute_anchor_positions_batch = spy
    generated, nfe = runner.generate_with_acache(seqs)
    assert calls == [1, 1, 1]                      # anchor selection stays per request
    assert len(generated) == 3 and all(g is not None and len(g) == 4 for g in generated)
    assert seqs[2].token_ids[5:] == [2, 3]         # the suffix affix is untouched
    assert nfe >= 3
    assert runner.block_manager.used_block_ids == set(runner.block_manager.reserved_block_ids)


@pytest.mark.parametrize("ratio", [0.0, 0.5, 1.0])
def test_generate_batched_threshold_loop_matches_dual_cache_token_counts(device, ratio):
    """Batch of 4 with infix placement, two blocks per request, threshold 0.9 (forced single-token steps with
    random weights): both loops terminate, fill every masked position and report consistent NFE."""
    cfg, model = _model(device, seed=1)
    affix = list(range(20, 30))

    def make(i):
        toks = [2 + i] + affix + [40 + i, 41 + i]
        return Sequence(toks, gen_length=8, block_length=4, cache_block_size=8, mask_id=63,
                        prompt_affix_start=1, prompt_affix_end=11)

    serve = _serve(cfg, recompute_batch_size=2, max_num_seqs=0, gen_length=8, block_length=4,
                   num_kvcache_blocks=32, threshold=0.9, anchor_ratio=ratio)
    ac = ModelRunner(model, serve)
    out, nfe = ac.generate_with_acache([make(i) for i in range(4)])
    assert len(out) == 4 and all(len(g) == 8 for g in out)
    base = ModelRunner(model, _serve(cfg, recompute_batch_size=2, max_num_seqs=0, gen_length=8, block_length=4,
                                     num_kvcache_blocks=32, threshold=0.9, enable_acache=False))
    out_b, nfe_b = base.generate_with_dual_cache([make(i) for i in range(4)])
    assert all(len(g) == 8 for g in out_b)
    assert 8 <= nfe <= 4 * 8 + 8 and 8 <= nfe_b <= 4 * 8 + 8
    if ratio == 1.0:
        agree = sum(a == b for g, h in zip(out, out_b) for a, b in zip(g, h))
        assert agree >= 24, f"only {agree}/32 tokens agree with full recompute at ratio 1.0"


@pytest.mark.parametrize("use_acache", [True, False])
def test_hip_graph_replay_of_refinement_steps_gives_the_same_tokens(device, use_acache):
    """The captured refinement forward is replayed for every step of a block, with the engine's eager work (token
    transfer, scheduling, the next block's refresh) between replays; every run must commit exactly the tokens of the
    eager loop, and the graph must be re-captured when the attention metadata changes."""
    cfg, model = _model(device, seed=3)
    affix = list(range(20, 30))

    def make(i):
        return Sequence([2 + i] + affix + [40 + i, 41 + i], gen_length=16, block_length=8, cache_block_size=8,
                        mask_id=63, prompt_affix_start=1, prompt_affix_end=11)

    def run(graph):
        serve = _serve(cfg, recompute_batch_size=2, max_num_seqs=0, gen_length=16, block_length=8,
                       num_kvcache_blocks=48, threshold=0.9, anchor_ratio=0.5, enable_acache=use_acache,
                       decode_hip_graph=graph)
        runner = ModelRunner(model, serve)
        seqs = [make(i) for i in range(3)]
        out, nfe = (runner.generate_with_acache if use_acache else runner.generate_with_dual_cache)(seqs)
        return out, nfe, runner.last_timing

    eager, nfe_eager, _ = run(False)
    for _ in range(2):   # twice: the second run captures without the eager warm-up forward
        replayed, nfe_graph, timing = run(True)
        assert replayed == eager and nfe_graph == nfe_eager
        assert all(63 not in g for g in replayed)


@pytest.mark.parametrize("d_model", [256, 64])
@pytest.mark.parametrize("placement", ["prefix", "infix"])
def test_batched_probe_at_admission_selects_the_same_anchors(device, placement, d_model):
    """Config.anchor_selection_batch_size = 0 probes all admitted requests in one forward instead of one forward
    per request (the reference's choice, model_runner.py:873): same anchors, same generated tokens."""
    cfg, model = _model(device, seed=3, d_model=d_model)
    affix = list(range(20, 32))

    def make(i):
        if placement == "prefix":
            return Sequence(affix + [40 + i, 41 + i, 42 + i][: 2 + i % 2], gen_length=4, block_length=4,
                            cache_block_size=8, mask_id=63, prompt_affix_len=len(affix))
        return Sequence([2 + i] * (1 + i % 3) + affix + [40 + i], gen_length=4, block_length=4, cache_block_size=8,
                        mask_id=63, prompt_affix_start=1 + i % 3, prompt_affix_end=1 + i % 3 + len(affix))

    results = []
    for probe_batch in (1, 0, 3):
        runner = ModelRunner(model, _serve(cfg, recompute_batch_size=2, max_num_seqs=0, num_kvcache_blocks=40,
                                           anchor_ratio=0.4, anchor_selection_batch_size=probe_batch))
        calls = []
        real = runner._select_anchors_on_device      # batched serving keeps the anchors on the device

        def spy(batch, real=real, calls=calls):
            calls.append(len(batch))
            return real(batch)

        runner._select_anchors_on_device = spy
        seqs = [make(i) for i in range(5)]
        out, _ = runner.generate_with_acache(seqs)
        assert all(s.device_layout is not None for s in seqs)
        results.append(([list(s.anchor_positions) for s in seqs], out))   # read back on demand
        assert calls == {1: [1] * 5, 0: [5], 3: [3, 2]}[probe_batch]
    assert results[0] == results[1] == results[2]
    assert all(len(a) == 5 for a in results[0][0])          # ceil(0.4 * 12) anchors per request


@pytest.mark.parametrize("ratio,expected_anchors", [(0.4, 5), (0.0, 0), (1.0, 12)])
def test_device_layouts_equal_the_host_layouts(device, ratio, expected_anchors):
    """Batched serving keeps anchors and slot maps on the device.  What the layout launch produced for the admitted
    requests must be, list for list, what ``Sequence.finalize_slot_mapping`` builds on the host from the same
    anchors and block tables, and the packed read order must be the host's query-relocation order.  Prefix, infix
    and suffix placement (generation window in front of the affix); no anchors, some, and all of the affix."""
    cfg, model = _model(device, seed=3)
    affix = list(range(20, 32))

    def make(i):
        if i == 4:   # suffix: [head, window of 4 masks, affix]
            return Sequence([2, 3] + [63] * 4 + affix, gen_length=4, block_length=4, cache_block_size=8, mask_id=63,
                            prompt_affix_start=6, prompt_affix_end=6 + len(affix), generation_start=2)
        if i % 2:
            return Sequence(affix + [40 + i, 41 + i], gen_length=4, block_length=4, cache_block_size=8, mask_id=63,
                            prompt_affix_len=len(affix))
        return Sequence([2 + i] * (1 + i) + affix + [40 + i], gen_length=4, block_length=4, cache_block_size=8,
                        mask_id=63, prompt_affix_start=1 + i, prompt_affix_end=1 + i + len(affix))

    runner = ModelRunner(model, _serve(cfg, max_num_seqs=0, num_kvcache_blocks=48, anchor_ratio=ratio))
    seqs = [make(i) for i in range(5)]
    with torch.inference_mode():
        prefix = runner._prepare_acache(seqs)
        batch = []
        assert runner._admit_sequences_with_acache(batch, seqs, prefix, True) == 5
    for seq in seqs:
        layout = seq.device_layout
        assert layout is not None and layout.anchors.dtype == torch.int32
        twin = Sequence(seq.token_ids[: seq.num_prompt_tokens], gen_length=4, block_length=4, cache_block_size=8,
                        mask_id=63, prompt_affix_start=seq.affix_start, prompt_affix_end=seq.affix_end,
                        generation_start=seq.generation_start if seq.generation_start < seq.affix_start else None)
        twin.enable_acache(len(affix), ratio, affix_start=seq.affix_start, affix_end=seq.affix_end)
        twin.set_anchor_positions(layout.anchors.tolist())
        twin.block_table = list(seq.block_table)
        twin.finalize_slot_mapping()
        assert seq.anchor_positions == twin.anchor_positions and len(twin.anchor_positions) == expected_anchors
        assert seq.read_slot_map == twin.read_slot_map
        assert seq.recompute_positions == twin.recompute_positions
        assert seq.recompute_slot_mapping == twin.recompute_slot_mapping
        assert seq.block_query_start() == twin.recompute_positions.index(twin.generation_start)
        assert layout.tokens.tolist() == seq.token_ids
        want, shared = runner._attention_read_layout(twin, True)
        if seq.affix_start:
            assert layout.read_packed.tolist() == want and shared == seq.affix_len - seq.num_anchor_tokens
        else:
            assert layout.read_packed is None and shared == 0


def test_merged_projections_keep_the_state_dict_and_follow_parameter_updates(device):
    """q / k / v (and gate / up) run as one GEMM whose weight the separate projections' parameters are views of:
    same state-dict names and shapes, loading new weights afterwards takes effect, and a hooked projection falls
    back to its own forward call."""
    cfg, model = _model(device, seed=5)
    ids = torch.randint(2, 60, (2, 12), device=device)
    pos = torch.arange(12, device=device).expand(2, 12)
    runner = ModelRunner(model, _serve(cfg, enable_acache=False))      # gives the attention modules a cache

    def forward():
        seqs = [Sequence(ids[i].tolist(), gen_length=4, cache_block_size=8, block_length=4, mask_id=63) for i in range(2)]
        for s in seqs:
            runner.block_manager.allocate(s)
            s.finalize_slot_mapping()
        with torch.inference_mode():
            flat_ids, flat_pos, _, _ = runner.prepare_caching(seqs)
            out = model(flat_ids, position_ids=flat_pos).logits.float()
        reset_context()
        for s in seqs:
            runner.block_manager.deallocate(s)
        return out

    keys_before = {k: tuple(v.shape) for k, v in model.state_dict().items()}
    merged = forward()
    block = model.model.transformer["blocks"][0]
    w_qkv = block._fused["qkv"][0]
    assert block.q_proj.weight.data_ptr() == w_qkv.data_ptr()          # parameters alias the merged weight
    assert {k: tuple(v.shape) for k, v in model.state_dict().items()} == keys_before
    # a hooked projection is called on its own: same result up to GEMM rounding
    seen = []
    hook = block.k_proj.register_forward_hook(lambda m, i, o: seen.append(tuple(o.shape)))
    separate = forward()
    hook.remove()
    assert seen and seen[0][-1] == cfg.d_model
    torch.testing.assert_close(separate, merged, rtol=2e-2, atol=2e-2)
    # new weights loaded through the usual interface are what the merged GEMM uses
    state = {k: (torch.randn_like(v) * 0.08 if v.dim() > 1 else v.clone()) for k, v in model.state_dict().items()}
    model.load_state_dict(state)
    assert block.q_proj.weight.data_ptr() == w_qkv.data_ptr()
    assert torch.equal(w_qkv[: cfg.d_model], state["model.transformer.blocks.0.q_proj.weight"])
    changed = forward()
    assert (changed - merged).abs().max().item() > 1e-2
    hook = block.k_proj.register_forward_hook(lambda m, i, o: None)
    torch.testing.assert_close(forward(), changed, rtol=2e-2, atol=2e-2)
    hook.remove()


def test_request_longer_than_the_configured_length_is_served(device):
    """The rotary table grows with the request (the reference builds it for position_ids.max() + 1,
    nano-vdllm/model/modeling_llada.py:910): a request past ``max_sequence_length`` generates the tokens that the
    same weights generate under a configuration whose table was long enough from the start."""
    import copy

    cfg, model = _model(device, seed=3)
    assert cfg.max_sequence_length == 64
    wide_cfg = copy.deepcopy(cfg)
    wide_cfg.max_sequence_length = 256
    wide = LLaDAModelLM(wide_cfg, init_std=0.08).to(device=device, dtype=torch.bfloat16).eval()
    wide.load_state_dict(model.state_dict())
    prompt = [2 + (7 * i) % 50 for i in range(90)]

    def run(m, c):
        runner = ModelRunner(m, _serve(c, num_kvcache_blocks=32, gen_length=8, anchor_ratio=0.25, threshold=0.9))
        seq = Sequence(list(prompt), gen_length=8, cache_block_size=8, block_length=4, mask_id=63,
                       prompt_affix_start=10, prompt_affix_end=50)
        return runner.generate_with_acache([seq])

    got, nfe = run(model, cfg)
    want, nfe_want = run(wide, wide_cfg)
    assert got == want and nfe == nfe_want and 63 not in got[0]


@pytest.mark.parametrize("use_acache", [True, False])
def test_refresh_forwards_run_under_a_dispatch_plan_and_give_the_same_tokens(device, use_acache):
    """With more attention units than workgroup slots a refresh forward carries a dispatch plan in its context
    (one per distinct set of lengths, reused by later refreshes); the generated tokens equal those of a runner
    that never plans."""
    cfg, model = _model(device, seed=1)
    affix = list(range(20, 30))

    def make(i):
        toks = [2 + i] + affix + [40 + i, 41 + i]
        return Sequence(toks, gen_length=8, block_length=4, cache_block_size=8, mask_id=63,
                        prompt_affix_start=1, prompt_affix_end=11)

    def generate(plans):
        serve = _serve(cfg, recompute_batch_size=2, max_num_seqs=0, gen_length=8, block_length=4,
                       num_kvcache_blocks=32, threshold=0.9, anchor_ratio=0.5, enable_acache=use_acache)
        runner = ModelRunner(model, serve)
        seen = []
        if plans:
            runner._workgroup_slots_per_xcd = 0        # any number of units counts as more than the slots
            real = runner._attention_plan

            def spy(cu_q, cu_k):
                plan = real(cu_q, cu_k)
                seen.append(plan)
                return plan

            runner._attention_plan = spy
        else:
            runner._attention_plan = lambda cu_q, cu_k: None
        seqs = [make(i) for i in range(4)]
        out, _ = runner.generate_with_acache(seqs) if use_acache else runner.generate_with_dual_cache(seqs)
        return out, seen, runner

    planned, seen, runner = generate(True)
    assert seen and all(p is not None and p.shape[0] % 8 == 0 and p.shape[0] > 0 for p in seen)
    assert len({p.data_ptr() for p in seen}) < len(seen)      # later refreshes of the same lengths reuse a plan
    assert len(runner._attention_plans) <= 8
    unplanned, _, _ = generate(False)
    assert planned == unplanned
