"""Writes tests/golden/reference_vectors.json: the inputs and expected outputs that the reference's own CPU tests
hold for the host layout of this path, transcribed as data (nothing of the reference is imported or executed).

    python tests/golden/make_vectors.py
"""
import json
from pathlib import Path

VECTORS = {
    "attention_read_layout": {
        "source": "nano-vdllm/tests/test_model_runner_acache.py:26-47",
        "shared_prefix_len": 3,
        "affix_start": 2,
        "shared_slot_offset": 0,
        "read_slot_map": [8, 9, 0, 10, 2, 11],
        "query_relocation": {"slots": [0, 2, 8, 9, 10, 11], "shared_len": 2},
        "key_relocation": {"slots": [8, 9, 0, 10, 2, 11], "shared_len": 0},
    },
    "use_query_side_relocation": {
        "source": "nano-vdllm/tests/test_model_runner_acache.py:50-61",
        "cases": [
            {"max_num_seqs": 0, "relocation_materialized": False, "expected": True},
            {"max_num_seqs": 16, "relocation_materialized": False, "expected": True},
            {"max_num_seqs": 1, "relocation_materialized": False, "expected": False},
            {"max_num_seqs": 0, "relocation_materialized": True, "expected": False},
        ],
    },
    "affix_span_layouts": {
        "source": "nano-vdllm/tests/test_sequence_spans.py:11-45",
        "gen_length": 2, "block_length": 2, "cache_block_size": 4, "mask_id": 99, "anchor_ratio": 0.5,
        "first_block": 2,
        "cases": [
            {"tokens": [10, 11, 12], "affix_start": 0, "affix_end": 2, "generation_start": None},
            {"tokens": [10, 20, 21, 11], "affix_start": 1, "affix_end": 3, "generation_start": None},
            {"tokens": [10, 99, 99, 20, 21], "affix_start": 3, "affix_end": 5, "generation_start": 1},
        ],
        "expect": "anchor = affix_end - 1; recompute_positions == sorted([anchor] + non_affix_positions); "
                  "read_slot_map[affix_start] == 0; read_slot_map[anchor] != anchor - affix_start; all slots >= 0",
    },
    "suffix_layout": {
        "source": "nano-vdllm/tests/test_sequence_spans.py:48-58",
        "tokens": [10, 50, 51, 20, 21], "gen_length": 2, "block_length": 2, "mask_id": 99,
        "affix_start": 3, "affix_end": 5, "generation_start": 1,
        "token_ids": [10, 99, 99, 20, 21], "generated_token_ids": [99, 99], "prompt_affix_token_ids": [20, 21],
    },
    "release_prefix_tail": {
        "source": "nano-vdllm/tests/test_sequence_spans.py:76-84",
        "num_blocks": 8, "cache_block_size": 4, "reserve": 5, "release_from": 2,
        "reserved": [0, 1], "used": [0, 1], "free": [2, 3, 4, 5, 6, 7],
    },
    "materialize_geometry": {
        "source": "nano-vdllm/tests/test_attention_kernels.py:127-165 (bit-exact: rtol = atol = 0)",
        "num_layers": 2, "num_slots": 24, "num_kv_heads": 2, "head_dim": 64, "affix_len": 7, "affix_shift": 5,
        "dst_slot": 12, "dtype": "bfloat16", "rope_base": 10000.0, "rope_rows": 24,
        "expect": "k_cache[:, dst:dst+affix_len] == apply_rope(k_cache[:, :affix_len], cos[shift], sin[shift]) and "
                  "v_cache[:, dst:dst+affix_len] == v_cache[:, :affix_len], both bit for bit",
    },
}

if __name__ == "__main__":
    out = Path(__file__).with_name("reference_vectors.json")
    out.write_text(json.dumps(VECTORS, indent=1) + "\n")
    print("wrote", out)
