"""The entry point that allocates nothing (``moe_i8_fused_experts_static``): same result as
``moe_i8_fused_experts`` with a caller-owned workspace, through the C-ABI, on two calls in a row
(the second with a smaller batch, so it runs over what the first left in the static array), and a
clear error beyond the array's size."""

import pytest
import torch

from _util import inputs_mod

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _call(pra, inp, static: bool):
    abi = pra._abi
    lib = abi.load()
    M, H = inp.hidden_states.shape
    E, N1, _ = inp.w1.shape
    I = N1 // 2
    k = inp.topk_ids.shape[1]
    ids = inp.topk_ids.to(torch.int32).contiguous()
    tw = inp.topk_weights.to(torch.float32).contiguous()
    out = torch.empty_like(inp.hidden_states)
    stream = torch.cuda.current_stream().cuda_stream
    p = lambda t: t.data_ptr()
    head = (p(inp.hidden_states), p(inp.w1), p(inp.w2), p(tw), p(ids), p(inp.w1_scale), p(inp.w2_scale), p(out),
            M, k, E, H, I, 64)
    if static:
        rc = lib.moe_i8_fused_experts_static(*head, abi.GEMM_AUTO, stream)
    else:
        need = lib.moe_i8_workspace_bytes(M, k, E, H, I, 64)
        ws = torch.empty(need, dtype=torch.uint8, device=DEV)
        rc = lib.moe_i8_fused_experts(*head, p(ws), need, abi.GEMM_AUTO, stream)
    torch.cuda.synchronize()
    return rc, out


def test_static_scratch_matches_workspace_entry_twice(pra):
    im = inputs_mod()
    for M, seed in [(192, 11), (24, 12)]:  # the second call is smaller than the first
        inp = im.make_inputs("qwen3-30b-a3b", M, seed=seed).to(DEV)
        rc_ws, want = _call(pra, inp, static=False)
        rc_st, got = _call(pra, inp, static=True)
        assert rc_ws == 0 and rc_st == 0, pra._abi.load().moe_i8_last_error()
        assert torch.equal(got, want), f"M={M}"  # same kernels, same arithmetic: bit-identical


def test_static_scratch_rejects_oversize(pra):
    abi = pra._abi
    lib = abi.load()
    im = inputs_mod()
    shape = im.SHAPES["qwen3-30b-a3b"]
    M = 2048
    assert lib.moe_i8_workspace_bytes(M, shape.k, shape.E_total, shape.H, shape.I, 64) > abi.STATIC_SCRATCH_BYTES
    inp = im.make_inputs("qwen3-30b-a3b", M, seed=3).to(DEV)
    rc, _ = _call(pra, inp, static=True)
    assert rc == abi.EWORKSPACE
    assert b"static array" in lib.moe_i8_last_error()
