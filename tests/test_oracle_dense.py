"""Pins the oracle's dense W8A8 functions (CPU only)."""

import numpy as np
import torch


def test_scaled_quant_rounds_ties_to_even(oracle):
    x = torch.tensor([[127.0, 0.5, 1.5, 2.5, -0.5, -1.5, -2.5, -127.0, 3.5, 126.5, 0.0, 0.25, 0.75, -0.75, 64.5, -64.5]],
                     dtype=torch.bfloat16)
    q, s = oracle.scaled_int8_quant(x)
    assert s.tolist() == [[1.0]]
    assert q.tolist() == [[127, 0, 2, 2, 0, -2, -2, -127, 4, 126, 0, 0, 1, -1, 64, -64]]
    qa, sa = oracle.per_token_quant_int8(x)  # the MoE quantiser: ties away from zero
    assert qa.tolist() == [[127, 1, 2, 3, -1, -2, -3, -127, 4, 127, 0, 0, 1, -1, 65, -65]] and torch.equal(s, sa)


def test_scaled_quant_brute_force(oracle):
    g = torch.Generator().manual_seed(2)
    x = (torch.randn(20, 48, generator=g) * torch.logspace(-3, 2, 20)[:, None]).to(torch.bfloat16)
    x[3] = 0
    q, s = oracle.scaled_int8_quant(x)
    for r in range(x.shape[0]):
        row = x[r].float().numpy()
        absmax = max(np.float32(np.abs(row).max()), np.float32(1e-10))
        inv = np.float32(127.0) / absmax
        want = [int(np.rint(np.float32(v) * inv)) for v in row]
        assert q[r].tolist() == want and s[r].item() == np.float32(absmax / np.float32(127.0))


def test_linear_against_float64(oracle):
    g = torch.Generator().manual_seed(4)
    x = torch.randn(9, 128, generator=g).to(torch.bfloat16)
    w = torch.randint(-127, 128, (40, 128), generator=g, dtype=torch.int8)
    ws = torch.rand(40, generator=g) * 0.01 + 0.001
    out = oracle.w8a8_linear(x, w, ws)
    q, a = oracle.scaled_int8_quant(x)
    want = (q.double() @ w.double().t()) * a.double() * ws.double().reshape(1, -1)
    assert out.dtype == torch.bfloat16 and out.shape == (9, 40)
    # one bf16 rounding of an fp32 product chain
    assert bool(((out.double() - want).abs() <= want.abs() * 2.0 ** -8 + 1e-30).all())
    # against the unquantised product: the activation quantisation error only (weights are exact)
    full = x.double() @ (w.double() * ws.double().reshape(-1, 1)).t()
    assert float((out.double() - full).norm() / full.norm()) < 0.02


def test_mlp_is_the_moe_layer_with_one_expert(oracle):
    # a dense gated MLP = an MoE layer whose single expert every token visits with weight 1; the two
    # differ only in how activation ties round, so on bf16 random data they agree to rounding noise
    g = torch.Generator().manual_seed(6)
    H, I, M = 128, 64, 33
    x = torch.randn(M, H, generator=g).to(torch.bfloat16)
    w13 = torch.randint(-127, 128, (2 * I, H), generator=g, dtype=torch.int8)
    w2 = torch.randint(-127, 128, (H, I), generator=g, dtype=torch.int8)
    s13 = torch.rand(2 * I, generator=g) * 0.004 + 0.001
    s2 = torch.rand(H, generator=g) * 0.004 + 0.001
    dense = oracle.w8a8_mlp(x, w13, s13, w2, s2)
    moe = oracle.fused_experts(x, w13[None], w2[None], torch.ones(M, 1), torch.zeros(M, 1, dtype=torch.int32),
                               s13[None], s2[None])
    assert float((dense.float() - moe.float()).norm() / moe.float().norm()) < 5e-3
    fp32 = oracle.dequant_fp32_moe(x, w13[None], w2[None], torch.ones(M, 1), torch.zeros(M, 1, dtype=torch.int32),
                                   s13[None], s2[None])
    assert float((dense.float() - fp32).norm() / fp32.norm()) < 3e-2
