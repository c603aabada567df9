"""Pins the oracle's router and routed-experts record (CPU only)."""

import base64
import math

import numpy as np
import pytest
import torch


def brute_force_route(logits, k, score_func, renormalize, route_scale, bias, num_groups, topk_groups, group_top2):
    """One token at a time in Python floats."""
    out_w, out_ids = [], []
    for row in logits.tolist():
        E = len(row)
        if score_func == "softmax":
            mx = max(row)
            ex = [math.exp(x - mx) for x in row]
            tot = sum(ex)
            scores = [e / tot for e in ex]
        elif score_func == "sigmoid":
            scores = [1.0 / (1.0 + math.exp(-x)) for x in row]
        else:
            scores = list(row)
        sel = [s + (bias[i] if bias is not None else 0.0) for i, s in enumerate(scores)]
        eligible = set(range(E))
        if num_groups > 1:
            per = E // num_groups
            gscore = []
            for g in range(num_groups):
                vals = sorted(sel[g * per:(g + 1) * per], reverse=True)
                gscore.append(vals[0] + vals[1] if group_top2 else vals[0])
            keep = sorted(range(num_groups), key=lambda g: (-gscore[g], g))[:topk_groups]
            eligible = {e for g in keep for e in range(g * per, (g + 1) * per)}
        ids = sorted(eligible, key=lambda e: (-sel[e], e))[:k]
        w = [scores[e] for e in ids]
        if score_func == "topk_softmax":
            mx = max(w)
            ex = [math.exp(x - mx) for x in w]
            w = [e / sum(ex) for e in ex]
        if renormalize:
            tot = sum(w) + 1e-20
            w = [x / tot for x in w]
        out_w.append([x * route_scale for x in w])
        out_ids.append(ids)
    return out_w, out_ids


CASES = [
    dict(E=8, k=2, score_func="softmax", renormalize=True, route_scale=1.0, bias=False, G=1, KG=1, top2=False),
    dict(E=8, k=3, score_func="softmax", renormalize=False, route_scale=2.5, bias=False, G=1, KG=1, top2=False),
    dict(E=16, k=4, score_func="sigmoid", renormalize=True, route_scale=1.0, bias=True, G=1, KG=1, top2=False),
    dict(E=16, k=4, score_func="topk_softmax", renormalize=False, route_scale=1.0, bias=False, G=1, KG=1, top2=False),
    dict(E=16, k=4, score_func="topk_softmax", renormalize=True, route_scale=0.5, bias=True, G=1, KG=1, top2=False),
    dict(E=32, k=4, score_func="sigmoid", renormalize=True, route_scale=2.5, bias=True, G=4, KG=2, top2=True),
    dict(E=32, k=6, score_func="softmax", renormalize=True, route_scale=1.0, bias=False, G=8, KG=3, top2=False),
    dict(E=24, k=5, score_func="sigmoid", renormalize=False, route_scale=1.0, bias=True, G=3, KG=2, top2=True),
]


@pytest.mark.parametrize("case", CASES, ids=lambda c: f"{c['score_func']}-E{c['E']}k{c['k']}G{c['G']}")
def test_router_matches_brute_force(oracle, case):
    g = torch.Generator().manual_seed(case["E"] * 7 + case["k"])
    logits = torch.randn(13, case["E"], generator=g, dtype=torch.float32) * 2.0
    bias = torch.randn(case["E"], generator=g, dtype=torch.float32) * 0.3 if case["bias"] else None
    w, ids = oracle.route_topk(logits, case["k"], case["score_func"], case["renormalize"], case["route_scale"], bias,
                               case["G"], case["KG"], case["top2"])
    # float32 inputs evaluated in float64 Python floats: the selection can only differ from the
    # float32 one where two candidates are closer than float32 resolution, which this seed avoids
    bw, bids = brute_force_route(logits.double(), case["k"], case["score_func"], case["renormalize"],
                                 case["route_scale"], None if bias is None else bias.double().tolist(), case["G"],
                                 case["KG"], case["top2"])
    assert ids.tolist() == bids
    torch.testing.assert_close(w.double(), torch.tensor(bw, dtype=torch.float64), rtol=2e-6, atol=1e-9)
    assert w.dtype == torch.float32 and ids.dtype == torch.int32


def test_equal_values_go_to_the_lowest_index(oracle):
    logits = torch.tensor([[1.0, 3.0, 3.0, 0.0, 3.0, 2.0, 2.0, -1.0]])
    _, ids = oracle.route_topk(logits, 5, "topk_softmax", False)
    assert ids.tolist() == [[1, 2, 4, 5, 6]]
    # equal group scores: the lower group wins
    logits = torch.tensor([[5.0, 0.0, 5.0, 0.0, 4.0, 4.0, 1.0, 1.0]])
    _, ids = oracle.route_topk(logits, 2, "topk_softmax", False, num_groups=4, topk_groups=1)
    assert ids.tolist() == [[0, 1]]


def test_router_closed_forms(oracle):
    g = torch.Generator().manual_seed(3)
    logits = torch.randn(64, 128, generator=g)
    w, ids = oracle.route_topk(logits, 8, "softmax", True)
    torch.testing.assert_close(w.sum(1), torch.ones(64), rtol=0, atol=2e-6)
    assert bool((w[:, :-1] >= w[:, 1:]).all())  # descending
    assert all(len(set(r)) == 8 for r in ids.tolist())
    # the older restatements of the two routers agree
    w2, ids2 = oracle.softmax_topk(logits, 8)
    assert torch.equal(ids, ids2) and torch.allclose(w, w2, rtol=1e-6, atol=0)
    bias = torch.randn(256, generator=g) * 0.1
    logits = torch.randn(40, 256, generator=g)
    w, ids = oracle.route_topk(logits, 8, "sigmoid", True, 2.5, bias, 8, 4, True)
    w2, ids2 = oracle.grouped_topk(logits, bias, 8, 8, 4, True, 2.5)
    assert torch.equal(ids, ids2) and torch.allclose(w, w2, rtol=1e-6, atol=0)
    assert all(len({e // 32 for e in r}) <= 4 for r in ids.tolist())
    # one group of everything = no groups
    a = oracle.route_topk(logits, 8, "sigmoid", True, 1.0, bias, 1, 1, True)
    b = oracle.route_topk(logits, 8, "sigmoid", True, 1.0, bias)
    assert torch.equal(a[1], b[1]) and torch.equal(a[0], b[0])
    # the bias steers the selection only: weights of the chosen experts are the unbiased scores
    w, ids = oracle.route_topk(logits, 8, "sigmoid", False, 1.0, bias)
    assert torch.equal(w, torch.sigmoid(logits).gather(1, ids.long()))
    w0, ids0 = oracle.route_topk(logits, 8, "sigmoid", False, 1.0, None)
    assert not torch.equal(ids, ids0)
    # topk_softmax: weights are the softmax of the selected logits
    w, ids = oracle.route_topk(logits, 8, "topk_softmax", False)
    torch.testing.assert_close(w, torch.softmax(logits.gather(1, ids.long()), dim=-1))


def test_routed_experts_record_reference_payloads(oracle):
    # tests/unit/inference/test_serving_tokens.py:46-60 of the reference
    arr = np.array([[[1, 2], [3, 4]], [[5, 6], [7, 8]]], dtype=np.int64)
    enc = oracle.serialize_routed_experts(arr)
    assert enc["shape"] == [2, 2, 2] and enc["dtype"] == "uint8" and enc["start"] == 0
    dec = np.frombuffer(base64.b64decode(enc["data"]), dtype=np.uint8).reshape(enc["shape"])
    np.testing.assert_array_equal(dec, arr)
    assert oracle.serialize_routed_experts(np.array([[[1, 2, 3]]]))["data"] == "AQID"
    wide = oracle.serialize_routed_experts(np.array([[[1, 511]]]), start=4)
    assert wide["dtype"] == "uint16" and wide["start"] == 4
    assert np.frombuffer(base64.b64decode(wide["data"]), dtype=np.uint16).tolist() == [1, 511]
    assert oracle.serialize_routed_experts(None) is None


def test_golden_vectors(oracle, golden):
    g = golden["router_ties"]
    _, ids = oracle.route_topk(torch.tensor([g["logits"]]), 5, "topk_softmax", False)
    assert ids.tolist() == [g["top5_ids"]]
    _, ids = oracle.route_topk(torch.tensor([g["grouped_logits"]]), 2, "topk_softmax", False,
                               num_groups=g["grouped_num_groups"], topk_groups=g["grouped_topk_groups"])
    assert ids.tolist() == [g["grouped_top2_ids"]]
    r = golden["routed_experts_payloads"]
    enc = oracle.serialize_routed_experts(np.array(r["array"], dtype=np.int64))
    assert enc["data"] == r["array_base64"] and list(base64.b64decode(enc["data"])) == r["array_bytes"]
    assert oracle.serialize_routed_experts(np.array(r["compact_ids"])) == r["compact"]
