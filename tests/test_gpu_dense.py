"""GPU parity: dense W8A8 quantiser (bit-exact), linear (bit-exact) and gated MLP through the C-ABI against the
CPU oracle."""

import pytest
import torch

from _util import bf16_ulp_diff, rel_err

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _weights(n, k, g):
    w = torch.randint(-127, 128, (n, k), generator=g, dtype=torch.int8)
    s = torch.rand(n, generator=g) * 0.008 + 0.002
    return w, s


def test_scaled_quant_tie_vector_and_rows(pra, oracle):
    x = torch.tensor([[127.0, 0.5, 1.5, 2.5, -0.5, -1.5, -2.5, -127.0, 3.5, 126.5, 0.0, 0.25, 0.75, -0.75, 64.5, -64.5]],
                     dtype=torch.bfloat16)
    q, s, azp = pra.scaled_int8_quant(x.to(DEV))
    assert azp is None and s.cpu().tolist() == [[1.0]]
    assert q.cpu().tolist() == [[127, 0, 2, 2, 0, -2, -2, -127, 4, 126, 0, 0, 1, -1, 64, -64]]
    g = torch.Generator().manual_seed(1)
    for rows, cols in [(1, 8), (37, 768), (64, 2048), (5, 4104), (3, 9000 // 8 * 8)]:
        x = (torch.randn(rows, cols, generator=g) * torch.logspace(-2, 2, rows)[:, None]).to(torch.bfloat16)
        q, s, _ = pra.scaled_int8_quant(x.to(DEV))
        qo, so = oracle.scaled_int8_quant(x)
        assert torch.equal(q.cpu(), qo) and torch.equal(s.cpu(), so)
    with pytest.raises(NotImplementedError):
        pra.scaled_int8_quant(x.to(DEV), scale=torch.ones(1, device=DEV))


@pytest.mark.parametrize("variant", ["auto", "stream", "tile_wide", "tile_deep", "tile_ring", "narrow"])
@pytest.mark.parametrize("M,N,K", [(1, 64, 256), (7, 128, 512), (64, 1536, 2048), (200, 2048, 768), (1000, 512, 1024)])
def test_linear_is_bit_exact(pra, oracle, variant, M, N, K):
    g = torch.Generator().manual_seed(M + N)
    x = torch.randn(M, K, generator=g).to(torch.bfloat16)
    w, s = _weights(N, K, g)
    try:
        out = pra.apply_int8_linear(x.to(DEV), w.to(DEV), s.to(DEV), gemm_variant=variant)
    except pra._abi.MoeI8Error as e:
        if e.code == pra._abi.EUNSUPPORTED:
            pytest.skip(str(e))
        raise
    ref = oracle.w8a8_linear(x, w, s)
    assert torch.equal(out.cpu(), ref)


def test_linear_accepts_the_transposed_view_and_batched_input(pra, oracle):
    g = torch.Generator().manual_seed(3)
    x = torch.randn(4, 6, 256, generator=g).to(torch.bfloat16)
    w, s = _weights(128, 256, g)
    wd = w.to(DEV)
    out = pra.apply_int8_linear(x.to(DEV), wd.t(), s.to(DEV))  # [K, N] view, as vLLM holds it for scaled_mm
    assert out.shape == (4, 6, 128) and torch.equal(out.cpu(), oracle.w8a8_linear(x, w, s))
    with pytest.raises(NotImplementedError):
        pra.apply_int8_linear(x.to(DEV), wd, s.to(DEV), bias=torch.zeros(128, device=DEV))
    with pytest.raises(ValueError):
        pra.apply_int8_linear(x.to(DEV)[..., :128].contiguous(), wd, s.to(DEV))


@pytest.mark.parametrize("variant", ["auto", "stream", "tile_wide", "tile_deep", "tile_ring", "narrow"])
@pytest.mark.parametrize("M,H,I", [(1, 256, 128), (50, 2048, 768), (300, 4096, 1408), (2048, 2048, 768)])
def test_gated_mlp(pra, oracle, variant, M, H, I):
    g = torch.Generator().manual_seed(M + I)
    x = torch.randn(M, H, generator=g).to(torch.bfloat16)
    w13, s13 = _weights(2 * I, H, g)
    w2, s2 = _weights(H, I, g)
    s13, s2 = s13 * 0.3, s2 * 0.3
    try:
        out = pra.w8a8_mlp(x.to(DEV), w13.to(DEV), s13.to(DEV), w2.to(DEV), s2.to(DEV), gemm_variant=variant)
    except pra._abi.MoeI8Error as e:
        if e.code == pra._abi.EUNSUPPORTED:
            pytest.skip(str(e))
        raise
    ref = oracle.w8a8_mlp(x, w13, s13, w2, s2)
    assert rel_err(out.cpu(), ref) < 1e-2
    # the same MLP as an MoE layer with one expert (only tie rounding differs)
    moe = pra.fused_experts(x.to(DEV), w13.to(DEV)[None], w2.to(DEV)[None], torch.ones(M, 1, device=DEV),
                            torch.zeros(M, 1, dtype=torch.int32, device=DEV), use_int8_w8a8=True,
                            per_channel_quant=True, w1_scale=s13.to(DEV)[None], w2_scale=s2.to(DEV)[None],
                            gemm_variant=variant)
    assert rel_err(out.cpu(), moe.cpu()) < 5e-3


@pytest.mark.parametrize("m", [1, 7, 16])
@pytest.mark.parametrize("H,I", [(2048, 768), (256, 128), (4096, 1024)])
def test_gated_mlp_of_a_few_rows_equals_the_rows_of_a_larger_call(pra, H, I, m):
    """Up to 16 rows the MLP runs as three launches (the down GEMM quantises its own input, ties to
    even); rows are independent, so the result must be, bit for bit, what the same rows give inside a
    larger call that takes the five-launch path."""
    g = torch.Generator().manual_seed(m + I)
    x = torch.randn(96, H, generator=g).to(torch.bfloat16).to(DEV)
    w13, s13 = _weights(2 * I, H, g)
    w2, s2 = _weights(H, I, g)
    args = (w13.to(DEV), (s13 * 0.3).to(DEV), w2.to(DEV), (s2 * 0.3).to(DEV))
    big = pra.w8a8_mlp(x, *args)
    small = pra.w8a8_mlp(x[:m].contiguous(), *args)
    assert torch.equal(small, big[:m]), int((small != big[:m]).sum())


def test_caller_owned_workspace_for_the_dense_ops(pra):
    """``workspace=`` of ``apply_int8_linear`` and ``w8a8_mlp``: the caller's buffer is used (bit-equal to the
    default call, also when the buffer starts out as garbage) and one that is too small is refused."""
    g = torch.Generator().manual_seed(11)
    M, H, I = 70, 512, 256
    x = torch.randn(M, H, generator=g).to(torch.bfloat16).to(DEV)
    w13, s13 = _weights(2 * I, H, g)
    w2, s2 = _weights(H, I, g)
    args = (w13.to(DEV), (s13 * 0.3).to(DEV), w2.to(DEV), (s2 * 0.3).to(DEV))
    lib = pra._abi.load()
    need = max(lib.moe_i8_dense_workspace_bytes(M, H, I), lib.moe_i8_dense_workspace_bytes(M, H, 0))
    ws = torch.full((need,), 0xA5, dtype=torch.uint8, device=DEV)
    want = pra.w8a8_mlp(x, *args)
    assert torch.equal(pra.w8a8_mlp(x, *args, workspace=ws), want)
    lin = pra.apply_int8_linear(x, args[0], args[1])
    ws.fill_(0x3C)
    assert torch.equal(pra.apply_int8_linear(x, args[0], args[1], workspace=ws), lin)
    with pytest.raises(ValueError):
        pra.w8a8_mlp(x, *args, workspace=ws[:64])
    with pytest.raises(ValueError):
        pra.apply_int8_linear(x, args[0], args[1], workspace=ws[:64])
