"""GPU parity for the grouped int8 GEMMs through the C-ABI: int32 accumulators bit-exact, the down
epilogue bit-exact, the SiLU-gated epilogue to within bf16 rounding noise (the only difference is
the last bits of exp and of the reciprocal before two bf16 roundings)."""

import pytest
import torch

from _util import bf16_ulp_diff, inputs_mod

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
VARIANTS = ["stream", "tile_wide", "tile_deep", "tile_ring", "narrow"]


def _problem(oracle, E, k, H, I, M, seed, B=64, routing="softmax"):
    im = inputs_mod()
    shape = im.LayerShape("t", E=E, k=k, H=H, I=I, routing=routing)
    inp = im.make_inputs(shape, M, seed=seed)
    st = oracle.fused_experts_staged(inp.hidden_states, inp.w1, inp.w2, inp.topk_weights, inp.topk_ids,
                                     inp.w1_scale, inp.w2_scale, B)
    return inp, st


def _routing_on_gpu(pra, inp, B):
    return pra.moe_align_block_size(inp.topk_ids.to(DEV), B, inp.w1.shape[0])


def _skip_if_unsupported(pra, fn):
    try:
        return fn()
    except pra._abi.MoeI8Error as exc:
        if exc.code == pra._abi.EUNSUPPORTED:
            pytest.skip(str(exc))
        raise


def _none_if_unsupported(pra, fn):
    try:
        return fn()
    except pra._abi.MoeI8Error as exc:
        if exc.code == pra._abi.EUNSUPPORTED:
            return None
        raise


def _unpack(shape):
    return shape if len(shape) == 7 else (*shape, "softmax")


def _shape_id(shape):
    return "-".join(str(v) for v in shape)


SHAPES = [
    # E, k, H, I, M, B
    (4, 2, 128, 64, 5, 16),
    (8, 2, 256, 192, 96, 64),
    (8, 2, 1024, 2816, 256, 64),     # toy layer of the baseline
    (128, 8, 2048, 768, 16, 64),     # Qwen3-30B-A3B decode
    (128, 8, 2048, 768, 300, 64),
    (16, 4, 1408, 448, 200, 32),     # K = 22 * 64: exercises the unroll tail
    (3, 1, 64, 64, 700, 128),        # one 16-channel tile, block 128
    (32, 8, 512, 320, 64, 64),
    (8, 2, 512, 512, 300, 128),      # block 128: two 64-row tiles per block
    (5, 3, 640, 1024, 150, 64),
    (4, 2, 512, 192, 100, 64),       # three gate_up channel tiles of the narrow family, down too short for it
    (4, 2, 192, 512, 100, 64),       # down with a partial last channel tile
    (6, 2, 1024, 512, 900, 64, "zipf"),  # skewed: experts with many blocks and experts with none
]


@pytest.mark.parametrize("variant", VARIANTS)
@pytest.mark.parametrize("shape", SHAPES, ids=_shape_id)
def test_int32_accumulators_bit_exact(pra, oracle, variant, shape):
    E, k, H, I, M, B, routing = _unpack(shape)
    inp, st = _problem(oracle, E, k, H, I, M, seed=E + M, B=B, routing=routing)
    s, e, npp = _routing_on_gpu(pra, inp, B)
    P = M * k
    # a family may support one of the two GEMM shapes of a layer and not the other
    acc1 = _none_if_unsupported(pra, lambda: pra.gemm_acc_i32(
        st["x_q"].to(DEV), inp.w1.to(DEV), s, e, npp, k, B, P, variant))
    if acc1 is not None:
        assert torch.equal(acc1.cpu(), st["acc1"]), int((acc1.cpu() != st["acc1"]).sum())
    acc2 = _none_if_unsupported(pra, lambda: pra.gemm_acc_i32(
        st["h_q"].to(DEV), inp.w2.to(DEV), s, e, npp, 1, B, P, variant))
    if acc2 is not None:
        assert torch.equal(acc2.cpu(), st["acc2"]), int((acc2.cpu() != st["acc2"]).sum())
    if acc1 is None and acc2 is None:
        pytest.skip("family supports neither GEMM of this shape")


@pytest.mark.parametrize("variant", VARIANTS)
def test_accumulators_extreme_values(pra, oracle, variant):
    """All operands at +-127 with K=7168: the largest magnitude the path can produce."""
    E, k, H, N, M, B = 2, 1, 7168, 64, 40, 64
    a = torch.full((M, H), 127, dtype=torch.int8)
    a[::2] = -127
    w = torch.full((E, N, H), -127, dtype=torch.int8)
    w[1, ::3] = 127
    ids = (torch.arange(M, dtype=torch.int32) % E).reshape(M, 1)
    s, e, npp = pra.moe_align_block_size(ids.to(DEV), B, E)
    acc = _skip_if_unsupported(pra, lambda: pra.gemm_acc_i32(a.to(DEV), w.to(DEV), s, e, npp, 1, B, M, variant))
    want = oracle.grouped_int_gemm(a, w, ids, 1)
    assert int(want.abs().max()) == 127 * 127 * 7168
    assert torch.equal(acc.cpu(), want)


@pytest.mark.parametrize("variant", VARIANTS)
@pytest.mark.parametrize("shape", SHAPES, ids=_shape_id)
def test_down_gemm_epilogue_bit_exact(pra, oracle, variant, shape):
    E, k, H, I, M, B, routing = _unpack(shape)
    inp, st = _problem(oracle, E, k, H, I, M, seed=E + M + 1, B=B, routing=routing)
    s, e, npp = _routing_on_gpu(pra, inp, B)
    out = _skip_if_unsupported(pra, lambda: pra.gemm_down(
        st["h_q"].to(DEV), st["a2_scale"].to(DEV), inp.w2.to(DEV), inp.w2_scale.to(DEV),
        inp.topk_weights.to(DEV), s, e, npp, B, variant))
    want = st["cache3"].reshape(M * k, H)
    assert torch.equal(out.cpu(), want), int((out.cpu() != want).sum())


@pytest.mark.parametrize("shape", SHAPES + [(8, 2, 256, 1024, 130, 64), (8, 2, 128, 1000 // 64 * 64, 70, 16)],
                         ids=_shape_id)
def test_down_gemm_that_quantises_its_own_activations(pra, oracle, shape):
    # bf16 activations in, the second per-token quantisation inside the kernel: the same bits as
    # quantise-then-GEMM (and so as the oracle)
    E, k, H, I, M, B, routing = _unpack(shape)
    inp, st = _problem(oracle, E, k, H, I, M, seed=E + M + 3, B=B, routing=routing)
    s, e, npp = _routing_on_gpu(pra, inp, B)
    args = (st["cache2"].to(DEV), inp.w2.to(DEV), inp.w2_scale.to(DEV), inp.topk_weights.to(DEV), s, e, npp, B)
    if I > 1024:
        with pytest.raises(pra._abi.MoeI8Error) as info:
            pra.gemm_down_bf16(*args)
        assert info.value.code == pra._abi.EUNSUPPORTED
        return
    out = pra.gemm_down_bf16(*args)
    want = st["cache3"].reshape(M * k, H)
    assert torch.equal(out.cpu(), want), int((out.cpu() != want).sum())
    two_step = pra.gemm_down(*pra.per_token_quant_int8(st["cache2"].to(DEV)), inp.w2.to(DEV), inp.w2_scale.to(DEV),
                             inp.topk_weights.to(DEV), s, e, npp, B, "stream")
    assert torch.equal(out, two_step)


@pytest.mark.parametrize("variant", VARIANTS)
@pytest.mark.parametrize("shape", SHAPES, ids=_shape_id)
def test_gate_up_silu_within_bf16_rounding(pra, oracle, variant, shape):
    E, k, H, I, M, B, routing = _unpack(shape)
    inp, st = _problem(oracle, E, k, H, I, M, seed=E + M + 2, B=B, routing=routing)
    s, e, npp = _routing_on_gpu(pra, inp, B)
    act = _skip_if_unsupported(pra, lambda: pra.gemm_gate_up_silu(
        st["x_q"].to(DEV), st["a1_scale"].to(DEV), inp.w1.to(DEV), inp.w1_scale.to(DEV), s, e, npp,
        k, B, M * k, variant))
    # identical except where an fp32 value sits within a few ulp of a bf16 rounding boundary: then
    # one bf16 step (two when the silu step is then doubled by the product's own rounding)
    d = bf16_ulp_diff(act, st["cache2"])
    assert int(d.max()) <= 2, int(d.max())
    assert float((d > 0).float().mean()) < 3e-3, float((d > 0).float().mean())
    assert float((d > 1).float().mean()) < 2e-4, float((d > 1).float().mean())


@pytest.mark.parametrize("variant", VARIANTS)
def test_gemm_is_deterministic(pra, oracle, variant):
    inp, st = _problem(oracle, 16, 4, 512, 256, 333, seed=7)
    s, e, npp = _routing_on_gpu(pra, inp, 64)
    args = (st["x_q"].to(DEV), st["a1_scale"].to(DEV), inp.w1.to(DEV), inp.w1_scale.to(DEV), s, e, npp, 4, 64, 333 * 4)
    first = _skip_if_unsupported(pra, lambda: pra.gemm_gate_up_silu(*args, variant))
    for _ in range(3):
        assert torch.equal(first, pra.gemm_gate_up_silu(*args, variant))


# The GEMM shapes of the GLM-4.5-Air and DeepSeek-V3 layers (many channel tiles, long reductions):
# int32 accumulators of every family that accepts the shape, all rows against each other on the
# device and a few hundred sampled rows against the oracle's exact integer product.
REAL_GEMM_SHAPES = [
    # E, N, K, rows per expert (about), row_div
    (8, 2 * 1408, 4096, 300, 8),   # GLM-4.5-Air gate_up
    (8, 4096, 1408, 300, 1),       # GLM-4.5-Air down
    (4, 4096, 7168, 400, 8),       # DeepSeek-V3 gate_up
    (4, 7168, 2048, 400, 1),       # DeepSeek-V3 down
]


@pytest.mark.parametrize("E,N,K,rows,row_div", REAL_GEMM_SHAPES, ids=lambda v: str(v))
def test_int32_accumulators_at_real_gemm_shapes(pra, oracle, E, N, K, rows, row_div):
    g = torch.Generator().manual_seed(N + K)
    P = E * rows
    M = (P + row_div - 1) // row_div
    a = torch.randint(-127, 128, (M, K), generator=g, dtype=torch.int8)
    w = torch.randint(-127, 128, (E, N, K), generator=g, dtype=torch.int8)
    ids = torch.randint(0, E, (P, 1), generator=g, dtype=torch.int32)
    s, e, npp = pra.moe_align_block_size(ids.to(DEV), 64, E)
    a_d, w_d = a.to(DEV), w.to(DEV)
    got = {}
    for variant in VARIANTS:
        acc = _none_if_unsupported(pra, lambda: pra.gemm_acc_i32(a_d, w_d, s, e, npp, row_div, 64, P, variant))
        if acc is not None:
            got[variant] = acc
    assert "stream" in got and len(got) >= 2, sorted(got)
    for variant, acc in got.items():
        assert torch.equal(acc, got["stream"]), variant
    sel = torch.randperm(P, generator=g)[:256]
    want = oracle.grouped_int_gemm(a[sel // row_div], w, ids[sel], 1)
    assert torch.equal(got["stream"][sel.to(DEV)].cpu(), want)
