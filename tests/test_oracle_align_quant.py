"""Pins the oracle's moe_align_block_size and per_token_quant_int8 (CPU only)."""

import math

import numpy as np
import pytest
import torch
from hypothesis import given, settings
from hypothesis import strategies as st


# ---------------------------------------------------------------- moe_align_block_size
def brute_force_align(ids, B, E):
    """Slot-by-slot construction with plain Python lists."""
    flat = [int(v) for row in ids for v in row]
    P = len(flat)
    sorted_ids, expert_ids = [], []
    for e in range(E):
        members = [t for t in range(P) if flat[t] == e]
        while len(members) % B:
            members.append(P)
        sorted_ids += members
        expert_ids += [e] * (len(members) // B)
    return sorted_ids, expert_ids


def check_align_invariants(ids, B, E, sorted_ids, expert_ids, npp):
    flat = ids.reshape(-1).to(torch.int64)
    P = flat.numel()
    npp = int(npp)
    counts = torch.bincount(flat, minlength=E)
    assert npp % B == 0 and npp <= P + E * (B - 1)
    assert npp == int(((counts + B - 1) // B * B).sum())
    used = sorted_ids[:npp].to(torch.int64)
    real = used[used < P]
    assert torch.equal(torch.sort(real)[0], torch.arange(P))  # every pair exactly once
    assert bool((sorted_ids[npp:] == P).all()) and bool((expert_ids[npp // B :] == -1).all())
    for j in range(npp // B):
        seg = used[j * B : (j + 1) * B]
        e = int(expert_ids[j])
        valid = seg[seg < P]
        assert bool((flat[valid] == e).all())
        assert bool((valid[1:] > valid[:-1]).all())  # ascending inside a block
        assert bool((seg[len(valid) :] == P).all())  # padding only at the end
    # closed form: stable argsort + exclusive cumsum of padded counts
    order = torch.argsort(flat, stable=True)
    starts = torch.cumsum((counts + B - 1) // B * B, 0) - (counts + B - 1) // B * B
    pos = 0
    for e in range(E):
        c = int(counts[e])
        assert torch.equal(used[int(starts[e]) : int(starts[e]) + c], order[pos : pos + c])
        pos += c


def test_align_upstream_docstring_example(oracle, golden):
    g = golden["align_docstring_example"]
    ids = torch.tensor(g["topk_ids"], dtype=torch.int32)
    s, e, npp = oracle.moe_align_block_size(ids, g["block_size"], g["num_experts"])
    assert int(npp) == g["num_tokens_post_padded"]
    assert s[: int(npp)].tolist() == g["sorted_token_ids_prefix"]
    assert e[: int(npp) // g["block_size"]].tolist() == g["expert_ids_prefix"]
    assert s.numel() == 12 + 5 * 3 and bool((s[int(npp) :] == g["sentinel"]).all())


@settings(max_examples=60, deadline=None)
@given(
    M=st.integers(0, 40), k=st.integers(1, 4), E=st.integers(1, 9), B=st.sampled_from([1, 2, 4, 16]), seed=st.integers(0, 10**6)
)
def test_align_matches_brute_force(M, k, E, B, seed):
    import importlib

    oracle = importlib.import_module("oracle.moe_i8_oracle")
    g = torch.Generator().manual_seed(seed)
    ids = torch.randint(0, E, (M, k), generator=g, dtype=torch.int32)
    s, e, npp = oracle.moe_align_block_size(ids, B, E)
    bs, be = brute_force_align(ids.tolist(), B, E)
    assert int(npp) == len(bs)
    assert s[: len(bs)].tolist() == bs and e[: len(be)].tolist() == be
    check_align_invariants(ids, B, E, s, e, npp)


@pytest.mark.parametrize(
    "case", ["unused_experts", "empty", "one_expert", "exact_multiple", "uniform_128x8", "zipf"]
)
def test_align_edge_cases(oracle, case, gen):
    B, E = 64, 128
    if case == "unused_experts":  # reference tests/unit/train/models/test_moe.py:115-125
        ids, E, B = torch.tensor([[0], [2]], dtype=torch.int32), 3, 16
    elif case == "empty":  # reference test_moe.py:126-132
        ids = torch.zeros((0, 8), dtype=torch.int32)
    elif case == "one_expert":
        ids = torch.full((100, 1), 7, dtype=torch.int32)
    elif case == "exact_multiple":
        ids = torch.arange(4, dtype=torch.int32).repeat_interleave(64).reshape(-1, 1)
        E = 4
    elif case == "uniform_128x8":
        ids = torch.stack([torch.randperm(E, generator=gen)[:8] for _ in range(300)]).to(torch.int32)
    else:
        p = torch.arange(1, E + 1, dtype=torch.float32) ** -1.2
        ids = torch.multinomial(p.expand(500, E), 8, generator=gen).to(torch.int32)
    s, e, npp = oracle.moe_align_block_size(ids, B, E)
    check_align_invariants(ids, B, E, s, e, npp)
    if case == "empty":
        assert int(npp) == 0 and s.numel() == E * (B - 1)
    if case == "exact_multiple":
        assert int(npp) == ids.numel() and bool((s[: int(npp)] < ids.numel()).all())


# ---------------------------------------------------------------- per_token_quant_int8
def test_quant_tie_vector(oracle, golden):
    g = golden["quant_ties"]
    x = torch.tensor([g["x"]], dtype=torch.bfloat16)
    q, s = oracle.per_token_quant_int8(x)
    assert q[0].tolist() == g["q_half_away"]
    assert q[0].tolist() != g["q_half_even_WRONG"]
    assert float(s[0, 0]) == g["scale"]


def test_round_half_away_is_c_roundf(oracle):
    xs = [0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 0.49999997, -0.49999997, 126.5, 3.0, -0.0, 8388609.0]
    got = oracle.round_half_away(torch.tensor(xs, dtype=torch.float32)).tolist()
    want = [float(math.floor(abs(v) + 0.5)) * (1 if v >= 0 else -1) for v in np.float32(xs).astype(float)]
    assert got == want


def test_quant_zero_row_and_invariants(oracle, gen, golden):
    x = torch.randn((64, 256), generator=gen).to(torch.bfloat16)
    x[3] = 0
    q, s = oracle.per_token_quant_int8(x)
    assert q.dtype == torch.int8 and s.shape == (64, 1) and s.dtype == torch.float32
    assert bool((q[3] == 0).all())
    assert float(s[3, 0]) == pytest.approx(golden["quant_ties"]["zero_row_scale"], rel=1e-6)
    qi = q.to(torch.int32)
    assert int(qi.abs().max()) <= 127
    nz = [r for r in range(64) if r != 3]
    assert bool((qi[nz].abs().amax(dim=1) == 127).all())
    err = (x.float() - qi.float() * s).abs()
    assert bool((err <= s / 2 * (1 + 1e-5)).all())


def test_quant_matches_elementwise_python(oracle, gen):
    """Element by element in numpy float32 scalars with C-style rounding."""
    x = (torch.randn((400, 256), generator=gen) * 3).to(torch.bfloat16)
    q, s = oracle.per_token_quant_int8(x)
    xf = x.float().numpy()
    double_rounded = 0
    for r in range(xf.shape[0]):
        absmax = max(np.float32(np.abs(xf[r]).max()), np.float32(1e-10))
        inv = np.float32(127.0) / absmax  # one IEEE division
        assert np.float32(s[r, 0]) == absmax / np.float32(127.0)
        y = (xf[r] * inv).astype(np.float32).astype(np.float64)
        want = np.copysign(np.floor(np.abs(y) + 0.5), y).astype(np.int64)
        assert np.array_equal(q[r].numpy().astype(np.int64), want)
        inv2 = np.float32(np.float32(1.0) / absmax) * np.float32(127.0)  # reciprocal-then-multiply
        y2 = (xf[r] * inv2).astype(np.float32).astype(np.float64)
        double_rounded += int((np.copysign(np.floor(np.abs(y2) + 0.5), y2).astype(np.int64) != want).sum())
    # the input is large enough that the two-rounding variant is distinguishable
    assert double_rounded > 0
