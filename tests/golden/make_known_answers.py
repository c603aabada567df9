"""Writes tests/golden/known_answers.json: small input/expected-output vectors that pin the oracle.

Nothing here imports the reference or the oracle.  Each vector is either literal data published
with the algorithm (the worked example in the docstring of vLLM's ``moe_align_block_size``, made
0-indexed), a case whose answer is fixed by arithmetic (rounding ties), or the expected output of a
known-answer test held by the reference, recomputed with that test's own plain loop
(``tests/unit/train/models/test_moe.py:83-109``, ``score_before_experts=False`` branch).
"""

import json
from pathlib import Path


def align_docstring_example():
    # 4 tokens, top-3, experts 0..4 (expert 0 unused), block 4.
    topk_ids = [[2, 3, 4], [1, 2, 4], [1, 3, 4], [1, 2, 3]]
    P = 12
    return {
        "topk_ids": topk_ids,
        "block_size": 4,
        "num_experts": 5,
        "sorted_token_ids_prefix": [3, 6, 9, P, 0, 4, 10, P, 1, 7, 11, P, 2, 5, 8, P],
        "expert_ids_prefix": [1, 2, 3, 4],
        "num_tokens_post_padded": 16,
        "sentinel": P,
    }


def quant_ties():
    # absmax 127 -> scale exactly 1.0, so x*inv == x and the .5 values are exact ties.
    return {
        "x": [127.0, 2.5, -2.5, 0.5, -0.5, 1.5, -1.5, 126.5],
        "q_half_away": [127, 3, -3, 1, -1, 2, -2, 127],
        "q_half_even_WRONG": [127, 2, -2, 0, 0, 2, -2, 126],
        "scale": 1.0,
        "zero_row_scale": 1e-10 / 127.0,
    }


def dispatcher_known_answer():
    x = [[float(3 * t + c) for c in range(3)] for t in range(4)]
    scores = [[0.2, 0.8], [0.4, 0.6], [0.7, 0.3], [0.9, 0.1]]
    selected = [[0, 1], [1, 2], [2, 0], [1, 0]]
    expected = [[0.0] * 3 for _ in range(4)]
    for token in range(4):
        for route in range(2):
            score = scores[token][route]
            expert_scale = selected[token][route] + 1
            for c in range(3):
                expected[token][c] += (x[token][c] ** 2) * expert_scale * score
    return {"x": x, "scores": scores, "selected": selected, "num_experts": 3, "expected": expected}


def routed_experts_payloads():
    # The two payloads held by the reference's own tests (tests/unit/inference/test_serving_tokens.py:46-60):
    # a [2, 2, 2] int64 array travels as its uint8 bytes, and "AQID" is base64 of the bytes 1, 2, 3.
    return {
        "array": [[[1, 2], [3, 4]], [[5, 6], [7, 8]]],
        "array_bytes": [1, 2, 3, 4, 5, 6, 7, 8],
        "array_base64": "AQIDBAUGBwg=",
        "compact": {"data": "AQID", "shape": [1, 1, 3], "start": 0, "dtype": "uint8"},
        "compact_ids": [[[1, 2, 3]]],
    }


def weight_quant_ties():
    # absmax 127 -> scale exactly 1.0: the quotient is the value itself and .5 values are exact ties,
    # which the weight quantiser (and the dense activation quantiser) round to even.
    return {
        "w": [127.0, 0.5, 1.5, 2.5, -0.5, -1.5, -2.5, -127.0, 3.5, 126.5, 0.0, 0.25, 0.75, -0.75, 64.5, -64.5],
        "q_half_even": [127, 0, 2, 2, 0, -2, -2, -127, 4, 126, 0, 0, 1, -1, 64, -64],
        "scale": 1.0,
        "zero_row_scale": 1e-12,
    }


def router_ties():
    # selection on the raw logits (top-k softmax router): descending value, equal values by ascending index;
    # with four groups of two and one group kept, equal group maxima go to the lower group.
    return {
        "logits": [1.0, 3.0, 3.0, 0.0, 3.0, 2.0, 2.0, -1.0],
        "top5_ids": [1, 2, 4, 5, 6],
        "grouped_logits": [5.0, 0.0, 5.0, 0.0, 4.0, 4.0, 1.0, 1.0],
        "grouped_num_groups": 4,
        "grouped_topk_groups": 1,
        "grouped_top2_ids": [0, 1],
    }


def main():
    out = {
        "align_docstring_example": align_docstring_example(),
        "quant_ties": quant_ties(),
        "dispatcher_known_answer": dispatcher_known_answer(),
        "routed_experts_payloads": routed_experts_payloads(),
        "weight_quant_ties": weight_quant_ties(),
        "router_ties": router_ties(),
    }
    path = Path(__file__).resolve().parent / "known_answers.json"
    path.write_text(json.dumps(out, indent=1) + "\n")
    print(path)


if __name__ == "__main__":
    main()
