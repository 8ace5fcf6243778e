"""Writes tests/golden/reference_cases.json.

The fixture holds *data only*: the case tables (mesh shapes, placements, tensor shapes, seeds) and
the literal known-answer vectors of the reference's own tests for this path, transcribed by reading
them (the reference was not imported or run):

  tests/test_self_copy_bucket.py:51-63            self-copy known answers
  tests/test_communication_cpu.py:42-49,122-137   11 mesh pairs, 4-D meshes, _StridedShard target
  tests/test_communication_symmetric_mesh.py:41-45,116-121
  tests/test_communication_replicate_shard.py:330-431   10 reshard cases (slice-view, Partial)
  tests/test_communication_replicate_shard.py:306-311   fp32 Partial -> bf16 Replicate
  tests/test_partial_chunk_reduce.py:146-176      21 Partial reduce cases

Placements are encoded as strings: "R", "S<dim>", "SS<dim>/<split_factor>", "P<op>".
"""

import json
import os

CASES = {
    "self_copy": [
        {"name": "single_entry", "tensor": [1, 2, 3, 4, 0, 0, 0, 0], "copies": [[0, 4]], "bucket_size": 1,
         "expect_tail": [1, 2, 3, 4], "tail_from": 4},
        {"name": "bundled", "tensor": [1, 2, 3, 4, 5, 6, 7, 8, 0, 0, 0, 0, 0, 0, 0, 0], "copies": [[0, 8], [4, 12]],
         "bucket_size": 262144, "expect_tail": [1, 2, 3, 4, 5, 6, 7, 8], "tail_from": 8, "expect_buckets": 1,
         "expect_chunks_in_bucket": 2},
    ],
    "communication_cpu": {
        "tensor_shape": [64, 64], "dtype": "float32", "seed": 0,
        "source_placements": ["R", "R", "S0", "S1"],
        "target_placements": ["R", "SS1/2", "R", "S1"],
        "bucket_sizes": [1, 262144],
        "mesh_pairs": [
            [[4, 1, 1, 1], [4, 1, 1, 1]], [[2, 2, 1, 1], [2, 1, 1, 2]], [[2, 2, 1, 1], [2, 1, 2, 1]],
            [[2, 1, 2, 1], [2, 1, 1, 2]], [[2, 1, 1, 2], [1, 1, 2, 2]], [[1, 2, 2, 1], [1, 2, 1, 2]],
            [[1, 2, 1, 2], [1, 1, 2, 2]], [[1, 1, 2, 2], [2, 1, 1, 2]], [[4, 1, 1, 1], [1, 1, 1, 4]],
            [[1, 4, 1, 1], [1, 1, 4, 1]], [[1, 1, 4, 1], [1, 1, 1, 4]],
        ],
    },
    "symmetric_mesh": {"tensor_shape": [64, 64], "dtype": "float32", "seed": 0, "mesh": [4], "placements": ["S1"]},
    "reshard": [
        {"src_mesh": [1, 2, 2], "src": ["R", "S0", "S0"], "tgt_mesh": [4], "tgt": ["S0"], "shape": [8, 16, 32], "slice_view": False},
        {"src_mesh": [2, 2], "src": ["R", "S0"], "tgt_mesh": [2, 2], "tgt": ["R", "S0"], "shape": [8, 16], "slice_view": False},
        {"src_mesh": [1, 4], "src": ["R", "R"], "tgt_mesh": [2, 2], "tgt": ["R", "S0"], "shape": [8, 16], "slice_view": False},
        {"src_mesh": [1, 2, 2], "src": ["R", "S0", "S0"], "tgt_mesh": [4], "tgt": ["S0"], "shape": [8, 16, 32], "slice_view": True},
        {"src_mesh": [2, 2], "src": ["S0", "S0"], "tgt_mesh": [4], "tgt": ["S0"], "shape": [8, 16, 32], "slice_view": True},
        {"src_mesh": [4], "src": ["Psum"], "tgt_mesh": [4], "tgt": ["R"], "shape": [8, 16], "slice_view": False},
        {"src_mesh": [4], "src": ["Pavg"], "tgt_mesh": [4], "tgt": ["S0"], "shape": [8, 16], "slice_view": False},
        {"src_mesh": [2, 2], "src": ["S0", "Psum"], "tgt_mesh": [4], "tgt": ["S0"], "shape": [8, 16], "slice_view": False},
        {"src_mesh": [2, 2], "src": ["Psum", "Psum"], "tgt_mesh": [4], "tgt": ["R"], "shape": [8, 16], "slice_view": False},
        {"src_mesh": [2, 3], "src": ["Psum", "Psum"], "tgt_mesh": [2], "tgt": ["R"], "shape": [8, 16], "slice_view": False},
    ],
    "reshard_bucket_sizes": [1, 268435456],
    "partial_mixed_dtype": {"src_mesh": [4], "tgt_mesh": [4], "shape": [8, 16], "source_dtype": "float32",
                            "transfer_dtype": "bfloat16", "scale": 1000.0, "seed_base": 1000},
    "partial_chunk_reduce": [
        [[4], ["Psum"], [8, 16], "fp32", False], [[4], ["Pavg"], [8, 16], "fp32", False],
        [[4], ["Pmax"], [8, 16], "fp32", False], [[4], ["Pmin"], [8, 16], "fp32", False],
        [[2, 2], ["R", "Psum"], [8, 16], "fp32", False], [[2, 2], ["Psum", "R"], [8, 16], "fp32", False],
        [[2, 2], ["S0", "Psum"], [8, 16], "fp32", False], [[2, 2], ["Psum", "S0"], [8, 16], "fp32", False],
        [[2, 2], ["S1", "Psum"], [8, 16], "fp32", False], [[2, 2], ["Psum", "Psum"], [8, 16], "fp32", False],
        [[2, 2], ["Pavg", "Pavg"], [8, 16], "fp32", False],
        [[1, 2, 2], ["R", "Psum", "S0"], [8, 16], "fp32", False],
        [[2, 2, 2], ["S0", "Psum", "R"], [16, 32], "fp32", False],
        [[4], ["Psum"], [64, 64], "fp16", False], [[4], ["Psum"], [64, 64], "bf16", False],
        [[4], ["Pavg"], [64, 64], "fp16", False],
        [[4], ["Psum"], [8, 16], "fp32", True], [[2, 2], ["S0", "Psum"], [8, 16], "fp32", True],
        [[4], ["Psum"], [8, 16], "fp32", False], [[4], ["Psum"], [10, 13], "fp32", False],
        [[4], ["Psum"], [3, 5], "fp32", False],
    ],
    "partial_tolerances": {"fp32": [1e-5, 1e-5], "fp16": [5e-3, 5e-3], "bf16": [5e-2, 5e-2]},
}

if __name__ == "__main__":
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "reference_cases.json")
    with open(path, "w") as f:
        json.dump(CASES, f, indent=1)
    print(path)
