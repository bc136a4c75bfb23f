"""Writes tests/golden/reference_vectors.json.

Each entry restates, as data, a known answer that the reference's own tests hold
for a function on the attention path (file:line of the test is recorded in the
entry).  Where the reference's test states its expected values as literals they
are copied as literals; where it states them as a closed form over literal
inputs (the hand-composed attention head), the closed form is evaluated here in
float64 from those inputs.  Nothing from the reference is imported or run.
"""
import json
import math
import os


def attention_head(query, key, value):
    """Closed form used by crates/incin-backends/tests/tensor_parallel_reference.rs:250-262
    and crates/incin/tests/tp2_network.rs:354-366: sequence length 2, head width 1, scale 1."""
    out = []
    for qi in query:
        logits = [qi * key[0], qi * key[1]]
        mx = max(logits)
        ex = [math.exp(l - mx) for l in logits]
        out.append((ex[0] * value[0] + ex[1] * value[1]) / (ex[0] + ex[1]))
    return out


def main():
    heads = [([1.0, 2.0], [1.0, -1.0], [3.0, 5.0]), ([0.5, -0.5], [2.0, 1.0], [7.0, 11.0])]
    vectors = {
        "attention_heads": {
            "source": "crates/incin-backends/tests/tensor_parallel_reference.rs:133-135,250-270 (tol 1e-6); "
                      "crates/incin/tests/tp2_network.rs:339-366 (tol 1e-4)",
            "scale": 1.0,
            "tol": 1e-6,
            "cases": [{"q": q, "k": k, "v": v, "expected": attention_head(q, k, v)} for q, k, v in heads],
        },
        "sdpa_ones": {
            "source": "crates/incin/tests/medium_priority_ops_tests.rs:57-67 (asserts dims only; uniform softmax "
                      "of equal logits makes every output element 1)",
            "shape": [1, 2, 4],
            "expected_dims": [1, 2, 4],
            "expected_value": 1.0,
            "tol": 1e-6,
        },
        "softmax": {
            "source": "crates/incin/tests/tensor_ops.rs:69-88; crates/incin-backends/src/cpu/ops/elementwise.rs:1578-1642",
            "cases": [
                {"x": [1000.0, 1000.0, 1000.0], "expected": [1 / 3, 1 / 3, 1 / 3], "tol": 1e-4},
                {"x": [-1000.0, 0.0, 1000.0], "expected": [0.0, 0.0, 1.0], "tol": 1e-4},
                {"x": [0.0, 0.0, 0.0], "expected": [1 / 3, 1 / 3, 1 / 3], "tol": 1e-4},
            ],
            "rows_sum_to_one": [[1.0, 2.0, 3.0], [4.0, 5.0, 6.0]],
            "rows_sum_tol": 1e-5,
            "monotonic": [1.0, 2.0, 3.0],
        },
        "log_softmax": {
            "source": "crates/incin-backends/src/cpu/ops/elementwise.rs:1697-1712",
            "x": [1000.0, 1000.0, 1000.0],
            "expected": [-math.log(3.0)] * 3,
            "tol": 1e-4,
        },
        "matmul": {
            "source": "crates/incin-backends/src/cpu/ops/matmul.rs:677-724; "
                      "crates/incin-backends/src/external/conformance.rs:396-398",
            "cases": [
                {"lhs": [[1, 2, 3], [4, 5, 6]],
                 "rhs": [[7, 8, 9, 10], [11, 12, 13, 14], [15, 16, 17, 18]],
                 "expected": [[74, 80, 86, 92], [173, 188, 203, 218]]},
                {"lhs": [[1, 2, 3], [4, 5, 6]],
                 "rhs": [[7, 8], [9, 10], [11, 12]],
                 "expected": [[58, 64], [139, 154]]},
            ],
        },
        "batch_broadcast_shapes": {
            "source": "crates/incin-backends/src/cpu/ops/matmul.rs:839-858,1327-1355",
            "cases": [
                {"lhs": [1, 3, 4], "rhs": [2, 4, 5], "out": [2, 3, 5]},
                {"lhs": [2, 1, 3, 4], "rhs": [1, 5, 4, 6], "out": [2, 5, 3, 6]},
            ],
        },
        "tolerance_profiles": {
            "source": "crates/incin-backends/src/external/conformance.rs:73-82",
            "F32_ACCUMULATED": {"abs": 1e-5, "rel": 1e-5},
        },
    }
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "reference_vectors.json")
    with open(path, "w") as f:
        json.dump(vectors, f, indent=1)
    print("wrote", path)


if __name__ == "__main__":
    main()
