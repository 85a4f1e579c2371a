"""Writes the golden-vector fixtures. The literals below are the parametrisations of the
reference's tests (file:line in README.md); the script imports nothing from the reference."""

import json
from pathlib import Path

HERE = Path(__file__).resolve().parent

segments = {
    "find_segments": [
        {"adapter_indices": [0, 0, 0, 1, 1, 2, 2, 2, 2, 2, 1, 1], "segments": [0, 3, 5, 10, 12], "segment_indices": [0, 1, 2, 1]},
        {"adapter_indices": [], "segments": [0], "segment_indices": []},
        {"adapter_indices": [0], "segments": [0, 1], "segment_indices": [0]},
        {"adapter_indices": [1], "segments": [0, 1], "segment_indices": [1]},
    ],
    "concat_segments": [
        {
            "batches": [[[0, 1, 4, 7, 8], [2, 1, 2, 1]], [[0, 2, 5], [1, 2]]],
            "segments": [0, 1, 4, 7, 10, 13],
            "segment_indices": [2, 1, 2, 1, 2],
        },
        {
            "batches": [[[0, 1, 4, 7], [2, 1, 2]], [[0, 2, 5], [1, 2]]],
            "segments": [0, 1, 4, 7, 9, 12],
            "segment_indices": [2, 1, 2, 1, 2],
        },
    ],
}

lora_batch = {
    "prefill": {
        "h": 1024,
        "rank_sets": [[8, 16], [32, 64]],
        "adapter_indices": [0, 0, 1, 1, 0, 0, 1, 1],
        "adapter_list": [0, 1, 0, 1],
        "adapter_segments": [0, 2, 4, 6, 8],
        "segment_indices": [0, 1, 0, 1],
        "min_rank_custom": 16,
        "entries_per_rank_group": 2,
    },
    "decode": [
        {
            "lora_ranks": [8, 8, 16],
            "adapter_indices": [0, 0, 1, 1, 0, 0, 1, 1, 2, 2],
            "expected": {
                "8": {"num_ptrs": 4, "indices": [0, 0, 1, 1, 0, 0, 1, 1, -1, -1]},
                "16": {"num_ptrs": 1, "indices": [-1, -1, -1, -1, -1, -1, -1, -1, 0, 0]},
            },
        },
        {
            "lora_ranks": [4, 8, 16],
            "adapter_indices": [0, 0, 1, 1, 0, 0, 1, 1, 2, 2],
            "expected": {
                "4": {"num_ptrs": 2, "indices": [0, 0, -1, -1, 0, 0, -1, -1, -1, -1]},
                "8": {"num_ptrs": 2, "indices": [-1, -1, 0, 0, -1, -1, 0, 0, -1, -1]},
                "16": {"num_ptrs": 1, "indices": [-1, -1, -1, -1, -1, -1, -1, -1, 0, 0]},
            },
        },
    ],
    "no_lora_segments": {
        "lora_adapter": 1,
        "lora_rank": 16,
        "adapter_indices": [0, 0, 0, 0],
        "adapter_list": [0],
        "adapter_segments": [0, 4],
        "segment_indices": [0],
    },
}

sgmv_kat = {
    "seed": 42,
    "B": 3,
    "H": 1024,
    "nlayers": 2,
    "layer_idx": 0,
    "dtype": "float16",
    "lora_ranks": [8, 16, 32, 64, 128],
    "segments": [[[0, 2], [1, 3]], [[0, -1], [1, -1]]],
    "rtol": 1e-2,
    "atol": 1e-3,
    "pad_rank": {"world_sizes": [1, 2, 4, 8], "lora_ranks": [8, 16, 32, 64, 128], "bs": 8, "h": 1024},
    "tmp_bytes_per_problem": 60,
    "shrink_tmp_bytes": 8388608,
}

for name, obj in (("segments", segments), ("lora_batch", lora_batch), ("sgmv_kat", sgmv_kat)):
    (HERE / f"{name}.json").write_text(json.dumps(obj, indent=1) + "\n")
    print("wrote", name)
