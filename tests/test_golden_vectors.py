"""The reference's own fixtures for this path (tests/golden/reference_vectors.json, transcribed from its CPU and GPU
tests) against the oracle, the host classes and — on a GPU — the kernels."""
import json
from pathlib import Path
from types import SimpleNamespace

import pytest
import torch

from acache_amd import BlockManager, Sequence
from acache_amd.model_runner import ModelRunner
from oracle import acache_oracle as O

G = json.loads((Path(__file__).parent / "golden" / "reference_vectors.json").read_text())


def test_fixture_file_is_what_the_script_writes():
    import importlib.util
    spec = importlib.util.spec_from_file_location("make_vectors", Path(__file__).parent / "golden" / "make_vectors.py")
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    assert json.loads(json.dumps(mod.VECTORS)) == G


def test_attention_read_layout_golden():
    v = G["attention_read_layout"]
    for key, query in (("query_relocation", True), ("key_relocation", False)):
        want = (v[key]["slots"], v[key]["shared_len"])
        assert O.attention_read_layout(v["read_slot_map"], v["shared_slot_offset"], v["shared_prefix_len"],
                                       v["affix_start"], query) == want
        runner = object.__new__(ModelRunner)
        runner.shared_prefix_len = v["shared_prefix_len"]
        runner._relocated_affix_slot_offset = None
        seq = SimpleNamespace(affix_start=v["affix_start"], shared_slot_offset=v["shared_slot_offset"],
                              read_slot_map=list(v["read_slot_map"]))
        assert runner._attention_read_layout(seq, query) == want


def test_query_side_relocation_truth_table_golden():
    for case in G["use_query_side_relocation"]["cases"]:
        runner = object.__new__(ModelRunner)
        runner._affix_relocation_enabled = True
        runner.config = SimpleNamespace(max_num_seqs=case["max_num_seqs"])
        assert runner._use_query_side_affix_relocation(case["relocation_materialized"]) is case["expected"]


def test_span_layouts_golden():
    v = G["affix_span_layouts"]
    for case in v["cases"]:
        seq = Sequence(case["tokens"], gen_length=v["gen_length"], block_length=v["block_length"],
                       cache_block_size=v["cache_block_size"], mask_id=v["mask_id"],
                       prompt_affix_start=case["affix_start"], prompt_affix_end=case["affix_end"],
                       generation_start=case["generation_start"])
        seq.enable_acache(anchor_ratio=v["anchor_ratio"])
        anchor = case["affix_end"] - 1
        seq.set_anchor_positions([anchor])
        seq.block_table = list(range(v["first_block"], v["first_block"] + seq.num_cache_blocks))
        seq.finalize_slot_mapping(shared_slot_offset=0)
        assert seq.recompute_positions == sorted([anchor] + seq.non_affix_positions)
        assert seq.read_slot_map[case["affix_start"]] == 0
        assert seq.read_slot_map[anchor] != anchor - case["affix_start"]
        assert all(slot >= 0 for slot in seq.read_slot_map)
        # the oracle's restatement gives the same three lists
        read, rpos, rslot = O.finalize_slot_mapping(len(seq), case["affix_start"], case["affix_end"], [anchor],
                                                    seq.block_table, v["cache_block_size"])
        assert (read, rpos, rslot) == (seq.read_slot_map, seq.recompute_positions, seq.recompute_slot_mapping)


def test_suffix_layout_and_prefix_release_golden():
    v = G["suffix_layout"]
    seq = Sequence(v["tokens"], gen_length=v["gen_length"], block_length=v["block_length"], mask_id=v["mask_id"],
                   prompt_affix_start=v["affix_start"], prompt_affix_end=v["affix_end"],
                   generation_start=v["generation_start"])
    assert seq.token_ids == v["token_ids"]
    assert seq.generated_token_ids == v["generated_token_ids"]
    assert seq.prompt_affix_token_ids == v["prompt_affix_token_ids"]
    r = G["release_prefix_tail"]
    bm = BlockManager(num_blocks=r["num_blocks"], cache_block_size=r["cache_block_size"])
    bm.reserve_prefix(r["reserve"])
    bm.release_prefix_tail(r["release_from"])
    assert bm.reserved_block_ids == set(r["reserved"]) and bm.used_block_ids == set(r["used"])
    assert set(bm.free_block_ids) == set(r["free"])


def _materialize_case():
    v = G["materialize_geometry"]
    g = torch.Generator().manual_seed(0)
    shape = (v["num_layers"], v["num_slots"], v["num_kv_heads"], v["head_dim"])
    k = torch.randn(shape, generator=g).to(torch.bfloat16)
    val = torch.randn(shape, generator=g).to(torch.bfloat16)
    cos, sin = O.rope_table(v["rope_rows"], v["head_dim"], v["rope_base"])
    return v, k, val, cos, sin


def test_materialize_geometry_oracle():
    v, k, val, cos, sin = _materialize_case()
    n, s, d = v["affix_len"], v["affix_shift"], v["dst_slot"]
    src_k, src_v = k[:, :n].clone(), val[:, :n].clone()
    O.materialize_relocated_affix(k, val, cos, sin, d, n, s)
    want = O.apply_rope(src_k.reshape(-1, v["num_kv_heads"], v["head_dim"]), cos[s].expand(src_k.shape[0] * n, -1),
                        sin[s].expand(src_k.shape[0] * n, -1)).view_as(src_k)
    assert torch.equal(k[:, d:d + n].view(torch.int16), want.view(torch.int16))
    assert torch.equal(val[:, d:d + n].view(torch.int16), src_v.view(torch.int16))


@pytest.mark.gpu
def test_materialize_geometry_kernel(device):
    from acache_amd import ops
    v, k, val, cos, sin = _materialize_case()
    n, s, d = v["affix_len"], v["affix_shift"], v["dst_slot"]
    ek, ev = k.clone(), val.clone()
    O.materialize_relocated_affix(ek, ev, cos, sin, d, n, s)
    gk, gv = k.to(device), val.to(device)
    ops.materialize_relocated_affix(gk, gv, cos.to(device), sin.to(device), d, n, s)
    assert torch.equal(gk.cpu().view(torch.int16), ek.view(torch.int16))
    assert torch.equal(gv.cpu().view(torch.int16), ev.view(torch.int16))
