"""The entry point that allocates nothing (``moe_i8_fused_experts_static``): same result as
``moe_i8_fused_experts`` with a caller-owned workspace, through the C-ABI, on two calls in a row
(the second with a smaller batch, so it runs over what the first left in the static array), and a
clear error beyond the array's size; and the property the entry exists for: after its first call on a
device it can be recorded into a HIP graph (a capture fails on any allocation, free or synchronisation) and
the replay follows changed inputs."""

import copy

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


def test_static_scratch_call_can_be_captured_and_replayed(pra):
    abi = pra._abi
    lib = abi.load()
    im = inputs_mod()
    M = 48
    inp = im.make_inputs("qwen3-30b-a3b", M, seed=21).to(DEV)
    fresh = im.make_inputs("qwen3-30b-a3b", M, seed=22).to(DEV)
    other = copy.copy(inp)  # the same weights, another batch and routing
    other.hidden_states, other.topk_ids, other.topk_weights = fresh.hidden_states, fresh.topk_ids, fresh.topk_weights
    rc, want_first = _call(pra, inp, static=False)
    assert rc == 0
    rc, want_second = _call(pra, other, static=False)
    assert rc == 0
    assert not torch.equal(want_first, want_second)
    rc, warm = _call(pra, inp, static=True)  # first call on the device: looks up the array's address
    assert rc == 0 and torch.equal(warm, want_first)

    H = inp.hidden_states.shape[1]
    E, N1, _ = inp.w1.shape
    k = inp.topk_ids.shape[1]
    x = inp.hidden_states.clone()
    ids = inp.topk_ids.to(torch.int32).contiguous()
    tw = inp.topk_weights.to(torch.float32).contiguous()
    out = torch.zeros_like(x)
    p = lambda t: t.data_ptr()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        rc = lib.moe_i8_fused_experts_static(p(x), p(inp.w1), p(inp.w2), p(tw), p(ids), p(inp.w1_scale),
                                             p(inp.w2_scale), p(out), M, k, E, H, N1 // 2, 64, abi.GEMM_AUTO,
                                             torch.cuda.current_stream().cuda_stream)
    assert rc == 0, lib.moe_i8_last_error()
    for i in range(2):
        out.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, want_first), i
        _call(pra, other, static=False)  # eager work of the program between the replays
    x.copy_(other.hidden_states)
    ids.copy_(other.topk_ids.to(torch.int32))
    tw.copy_(other.topk_weights.to(torch.float32))
    out.zero_()
    torch.cuda.synchronize()
    graph.replay()
    torch.cuda.synchronize()
    assert torch.equal(out, want_second)
