"""Pins the oracle's per-output-channel weight quantiser and the kernel weight layout (CPU only)."""

import numpy as np
import torch


def brute_force_row(row_bf16):
    """One row in numpy float32, element by element: scale = max(absmax / 127, 1e-12), q = rint(x / scale)."""
    x = row_bf16.to(torch.float32).numpy()
    absmax = np.float32(0.0)
    for v in x:
        absmax = max(absmax, np.float32(abs(v)))
    scale = max(np.float32(absmax / np.float32(127.0)), np.float32(1e-12))
    q = [int(min(127.0, max(-127.0, float(np.rint(np.float32(v) / scale))))) for v in x]
    return q, float(scale)


def test_ties_round_to_even_and_extremes_hit_127(oracle):
    # absmax 127 -> scale exactly 1 -> the quotient is the value itself
    w = torch.tensor([[127.0, 0.5, 1.5, 2.5, -0.5, -1.5, -2.5, -127.0, 3.5, 126.5, 0.0, 0.25, 0.75, -0.75, 64.5, -64.5]],
                     dtype=torch.bfloat16)
    q, s = oracle.quantize_weights_per_channel(w)
    assert s.tolist() == [1.0]
    assert q.tolist() == [[127, 0, 2, 2, 0, -2, -2, -127, 4, 126, 0, 0, 1, -1, 64, -64]]
    # half-away rounding (the activation rule) would differ on this vector
    away = oracle.round_half_away(w.float())
    assert not torch.equal(away.to(torch.int8), q)


def test_zero_row_and_tiny_row(oracle):
    w = torch.zeros(3, 16, dtype=torch.bfloat16)
    w[1, 3] = 2.0 ** -100  # absmax / 127 below the clamp
    w[2, 5] = -3.0
    q, s = oracle.quantize_weights_per_channel(w)
    assert s[0].item() == np.float32(1e-12) and bool((q[0] == 0).all())
    assert s[1].item() == np.float32(1e-12) and bool((q[1] == 0).all())
    assert q[2, 5].item() == -127 and s[2].item() == np.float32(3.0) / np.float32(127.0)


def test_brute_force_and_error_bound(oracle):
    g = torch.Generator().manual_seed(5)
    w = (torch.randn(40, 64, generator=g) * torch.logspace(-4, 2, 40)[:, None]).to(torch.bfloat16)
    q, s = oracle.quantize_weights_per_channel(w)
    for r in range(w.shape[0]):
        qb, sb = brute_force_row(w[r])
        assert q[r].tolist() == qb and s[r].item() == sb
    wf = w.float()
    assert bool((q.abs().amax(dim=1) == 127).all())  # the largest element of a row maps to +-127
    # reconstruction within half a step (plus the float32 rounding of a quotient of size <= 127)
    s64 = s.double()[:, None]
    assert bool(((q.double() * s64 - wf.double()).abs() <= s64 * (0.5 + 127 * 2.0 ** -23)).all())
    # sign symmetry: quantising -w negates q and keeps the scale
    qn, sn = oracle.quantize_weights_per_channel(-w)
    assert torch.equal(qn, -q) and torch.equal(sn, s)


def test_kernel_layout_matches_reference_conversion_shapes(oracle):
    # shapes asserted by the reference's conversion test (tests/unit/train/models/
    # test_glm_moe_dsa_conversion.py:47-50): E=2, I=3, H=6 -> w13 (2, 6, 6), w2 (2, 6, 3)
    g = torch.Generator().manual_seed(1)
    gate = torch.randn(2, 3, 6, generator=g).to(torch.bfloat16)
    up = torch.randn(2, 3, 6, generator=g).to(torch.bfloat16)
    down = torch.randn(2, 6, 3, generator=g).to(torch.bfloat16)
    w13, s13, w2, s2 = oracle.quantize_expert_weights(gate, up, down)
    assert w13.shape == (2, 6, 6) and s13.shape == (2, 6) and w13.dtype == torch.int8 and s13.dtype == torch.float32
    assert w2.shape == (2, 6, 3) and s2.shape == (2, 6)
    # gate rows first, then up rows, each quantised on its own row scale
    qg, sg = oracle.quantize_weights_per_channel(gate)
    qu, su = oracle.quantize_weights_per_channel(up)
    assert torch.equal(w13[:, :3], qg) and torch.equal(w13[:, 3:], qu)
    assert torch.equal(s13[:, :3], sg) and torch.equal(s13[:, 3:], su)


def test_quantised_layer_tracks_the_bf16_layer(oracle):
    from _util import inputs_mod

    inputs = inputs_mod()
    # end to end: weights quantised by this rule drive the int8 layer close to the fp32 layer on the
    # same bf16 weights
    shape = inputs.SHAPES["toy"]
    g = torch.Generator().manual_seed(9)
    E, I, H = shape.E_total, shape.I, shape.H
    gate = (torch.randn(E, I, H, generator=g) * H ** -0.5).to(torch.bfloat16)
    up = (torch.randn(E, I, H, generator=g) * H ** -0.5).to(torch.bfloat16)
    down = (torch.randn(E, H, I, generator=g) * I ** -0.5).to(torch.bfloat16)
    w13, s13, w2, s2 = oracle.quantize_expert_weights(gate, up, down)
    x = torch.randn(24, H, generator=g).to(torch.bfloat16)
    tw, ids = inputs.route(shape, 24, g)
    got = oracle.fused_experts(x, w13, w2, tw, ids, s13, s2).float()
    ones13, ones2 = torch.ones(E, 2 * I), torch.ones(E, H)
    # dequant_fp32_moe with unit scales on the unquantised weights = the fp32 layer
    want = oracle.dequant_fp32_moe(x, torch.cat([gate, up], 1).float(), down.float(), tw, ids, ones13, ones2).float()
    rel = (got - want).norm() / want.norm()
    assert rel < 0.05, rel


def test_golden_tie_vector(oracle, golden):
    g = golden["weight_quant_ties"]
    q, s = oracle.quantize_weights_per_channel(torch.tensor([g["w"]], dtype=torch.bfloat16))
    assert q.tolist() == [g["q_half_even"]] and s.tolist() == [g["scale"]]
    qd, sd = oracle.scaled_int8_quant(torch.tensor([g["w"]], dtype=torch.bfloat16))
    assert qd.tolist() == [g["q_half_even"]] and sd.tolist() == [[g["scale"]]]
    _, z = oracle.quantize_weights_per_channel(torch.zeros(1, 8, dtype=torch.bfloat16))
    assert z.item() == np.float32(g["zero_row_scale"])
