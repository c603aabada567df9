"""GPU parity for the whole layer through ``fused_experts``: within 1e-2 relative of the CPU oracle
on identical seeded inputs (the tolerance the task states for bf16 outputs), on every baseline
configuration; the largest ones are checked on sampled tokens, which is exact because the layer is
independent per token."""

import pytest
import torch

from _util import bf16_ulp_diff, inputs_mod, rel_err, subset_problem

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
TOL = 1e-2  # relative, bf16 output vs the oracle's fused_experts


def _run(pra, inp, **kw):
    out = pra.fused_experts(*inp.fused_experts_args(), **inp.fused_experts_kwargs(), **kw)
    torch.cuda.synchronize()
    return out


def _check_against_oracle(pra, oracle, shape_name, M, seed, variant="auto"):
    im = inputs_mod()
    inp = im.make_inputs(shape_name, M, seed=seed)
    out = _run(pra, inp.to(DEV), gemm_variant=variant)
    want = oracle.fused_experts(inp.hidden_states, inp.w1, inp.w2, inp.topk_weights, inp.topk_ids,
                                inp.w1_scale, inp.w2_scale, 64)
    assert out.shape == want.shape and out.dtype == torch.bfloat16
    err = rel_err(out, want)
    assert err < TOL, err
    # elementwise: almost everything identical, nothing further than a few bf16 steps of the row scale
    d = (out.float().cpu() - want.float()).abs()
    assert float(d.max()) <= 0.02 * float(want.float().abs().max()), float(d.max())
    return err


@pytest.mark.parametrize("variant", ["stream", "auto"])
@pytest.mark.parametrize("shape_name,M", [
    ("toy", 256), ("toy", 1), ("qwen3-30b-a3b", 16), ("qwen3-30b-a3b", 128), ("qwen3-30b-a3b", 1024),
    ("qwen3-30b-a3b", 2048), ("glm-4.5-air", 32),
])
def test_fused_experts_matches_oracle(pra, oracle, shape_name, M, variant):
    _check_against_oracle(pra, oracle, shape_name, M, seed=M, variant=variant)


@pytest.mark.parametrize("shape_name,M,weights_on_device", [
    ("qwen3-30b-a3b", 8192, False), ("qwen3-30b-a3b", 65536, True), ("glm-4.5-air", 512, False), ("glm-4.5-air", 4096, False),
    ("deepseek-v3", 8, True), ("deepseek-v3", 64, True), ("deepseek-v3", 2048, True), ("deepseek-v3", 16384, True),
])
def test_fused_experts_full_size_sampled_tokens(pra, oracle, shape_name, M, weights_on_device):
    im = inputs_mod()
    inp = im.make_inputs(shape_name, M, seed=M + 1, device=DEV, weights_on_device=weights_on_device)
    out = _run(pra, inp)
    assert bool(torch.isfinite(out.float()).all())
    g = torch.Generator().manual_seed(0)
    # tokens the oracle recomputes: as many as keep the experts they use (copied to the host) within a few GB
    weight_bytes = inp.w1.numel() + inp.w2.numel()
    sel = torch.randperm(M, generator=g)[: min(M, 256 if weight_bytes < (3 << 30) else 32)].sort()[0]
    sub = subset_problem(inp, sel)
    want = oracle.fused_experts(sub["hidden_states"], sub["w1"], sub["w2"], sub["topk_weights"], sub["topk_ids"],
                                sub["w1_scale"], sub["w2_scale"], 64)
    err = rel_err(out[sel.to(DEV)], want)
    assert err < TOL, err


def test_inplace_and_workspace_argument(pra, oracle):
    im = inputs_mod()
    inp = im.make_inputs("toy", 64, seed=5).to(DEV)
    ref = _run(pra, inp)
    x = inp.hidden_states.clone()
    ws = torch.empty((pra.workspace_bytes(64, 2, 8, 1024, 2816, 64),), dtype=torch.uint8, device=DEV)
    out = pra.fused_experts(x, inp.w1, inp.w2, inp.topk_weights, inp.topk_ids, inplace=True, workspace=ws,
                            **inp.fused_experts_kwargs())
    assert out.data_ptr() == x.data_ptr() and torch.equal(out, ref)
    with pytest.raises(ValueError, match="workspace too small"):
        pra.fused_experts(*inp.fused_experts_args(), workspace=ws[:1024], **inp.fused_experts_kwargs())
    # int64 ids and [E, N, 1] scales as vLLM passes them
    out2 = pra.fused_experts(inp.hidden_states, inp.w1, inp.w2, inp.topk_weights, inp.topk_ids.to(torch.int64),
                             use_int8_w8a8=True, per_channel_quant=True, w1_scale=inp.w1_scale.unsqueeze(-1),
                             w2_scale=inp.w2_scale.unsqueeze(-1))
    assert torch.equal(out2, ref)


def test_empty_batch_and_bad_shapes(pra):
    im = inputs_mod()
    inp = im.make_inputs("toy", 4, seed=1).to(DEV)
    empty = pra.fused_experts(inp.hidden_states[:0], inp.w1, inp.w2, inp.topk_weights[:0], inp.topk_ids[:0],
                              **inp.fused_experts_kwargs())
    assert empty.shape == (0, 1024)
    with pytest.raises(ValueError):
        pra.fused_experts(inp.hidden_states[:, :512].contiguous(), inp.w1, inp.w2, inp.topk_weights, inp.topk_ids,
                          **inp.fused_experts_kwargs())
    with pytest.raises(ValueError):
        pra.fused_experts(inp.hidden_states, inp.w1, inp.w2, inp.topk_weights[:2], inp.topk_ids,
                          **inp.fused_experts_kwargs())


def test_layer_is_deterministic_and_stream_safe(pra):
    im = inputs_mod()
    inp = im.make_inputs("qwen3-30b-a3b", 64, seed=2).to(DEV)
    first = _run(pra, inp)
    for _ in range(3):
        assert torch.equal(first, _run(pra, inp))
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        other = pra.fused_experts(*inp.fused_experts_args(), **inp.fused_experts_kwargs())
    side.synchronize()
    assert torch.equal(first, other)


def test_block_size_does_not_change_the_result(pra):
    im = inputs_mod()
    inp = im.make_inputs("toy", 100, seed=3).to(DEV)
    ref = _run(pra, inp, block_size_m=64)
    for B in (16, 32, 128):
        assert torch.equal(ref, _run(pra, inp, block_size_m=B))


@pytest.mark.parametrize("M", [16, 512, 1024, 2048])  # streaming, narrow-tile, deep and wide LDS-tile GEMM families
def test_hip_graph_replay(pra, M):
    """The call records no allocation, memset or synchronisation, so it can be captured and replayed."""
    im = inputs_mod()
    inp = im.make_inputs("qwen3-30b-a3b", M, seed=4).to(DEV)
    eager = _run(pra, inp)
    ws = torch.empty((pra.workspace_bytes(M, 8, 128, 2048, 768, 64),), dtype=torch.uint8, device=DEV)
    static_x = inp.hidden_states.clone()
    out = torch.empty_like(static_x)
    kw = dict(workspace=ws, **inp.fused_experts_kwargs())
    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):
        pra.fused_experts(static_x, inp.w1, inp.w2, inp.topk_weights, inp.topk_ids, **kw)
    torch.cuda.current_stream().wait_stream(s)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out.copy_(pra.fused_experts(static_x, inp.w1, inp.w2, inp.topk_weights, inp.topk_ids, **kw))
    for i in range(3):
        out.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, eager), i
        assert torch.equal(_run(pra, inp), eager)
    # another batch copied into the captured input tensors: the replay must follow it (kernels that ran
    # eagerly during the capture instead of being recorded would leave the old result in place)
    other = im.make_inputs("qwen3-30b-a3b", M, seed=44).to(DEV)
    static_x.copy_(other.hidden_states)
    inp.topk_weights.copy_(other.topk_weights)
    inp.topk_ids.copy_(other.topk_ids)
    want = pra.fused_experts(other.hidden_states, inp.w1, inp.w2, other.topk_weights, other.topk_ids,
                             **inp.fused_experts_kwargs())
    assert not torch.equal(want, eager)
    out.zero_()
    torch.cuda.synchronize()
    graph.replay()
    torch.cuda.synchronize()
    assert torch.equal(out, want)


def test_decode_mix_sequence_reuses_workspace(pra, oracle):
    """Continuous-batching decode: layers with independently seeded weights called back to back with
    a batch size that changes every step, one shared workspace; every step is checked on sampled
    tokens (the layer is independent per token)."""
    im = inputs_mod()
    shape = im.SHAPES["qwen3-30b-a3b"]
    layers = [im.make_inputs(shape, 256, seed=100 + i).to(DEV) for i in range(3)]
    ws = torch.empty((pra.workspace_bytes(256, shape.k, shape.E, shape.H, shape.I, 64),), dtype=torch.uint8, device=DEV)
    g = torch.Generator().manual_seed(7)
    for step in range(12):
        M = int(torch.randint(1, 257, (1,), generator=g))
        layer = layers[step % len(layers)]
        tw, ids = im.route(shape, M, g)
        x = layer.hidden_states[:M].contiguous()
        out = pra.fused_experts(x, layer.w1, layer.w2, tw.to(DEV), ids.to(DEV), workspace=ws,
                                **layer.fused_experts_kwargs())
        sel = torch.randperm(M, generator=g)[: min(M, 3)].sort()[0]
        probe = type(layer)(shape, x, layer.w1, layer.w2, layer.w1_scale, layer.w2_scale, tw, ids)
        sub = subset_problem(probe, sel)
        want = oracle.fused_experts(sub["hidden_states"], sub["w1"], sub["w2"], sub["topk_weights"], sub["topk_ids"],
                                    sub["w1_scale"], sub["w2_scale"], 64)
        err = rel_err(out[sel.to(DEV)], want)
        assert err < TOL, (step, M, err)


@pytest.mark.parametrize("E,k,H,I,M,B", [
    (128, 8, 2048, 768, 1, 64), (128, 8, 2048, 768, 16, 64), (128, 8, 2048, 768, 48, 64),
    (8, 2, 256, 128, 12, 16), (16, 3, 512, 256, 16, 64), (24, 4, 320, 1024, 18, 32), (64, 6, 1024, 512, 32, 64),
    (4, 1, 64, 64, 12, 16), (2, 2, 2048, 64, 3, 128), (8, 8, 192, 192, 3, 64),
])
def test_small_batch_layer_equals_the_chain_of_its_stages(pra, E, k, H, I, M, B):
    """With a handful of rows per expert the layer merges launches (moe_align with the first
    quantisation, the second quantisation with the down GEMM).  The result must equal, bit for bit,
    the six stand-alone stages called one after the other — on skewed routing too, where one block
    holds several 16-row passes — and must not depend on what the workspace held."""
    im = inputs_mod()
    for routing in ("softmax", "zipf"):
        shape = im.LayerShape("s", E=E, k=k, H=H, I=I, routing=routing)
        inp = im.make_inputs(shape, M, seed=M + E).to(DEV)
        P = M * k
        x_q, a1 = pra.per_token_quant_int8(inp.hidden_states)
        s, e, npp = pra.moe_align_block_size(inp.topk_ids, B, E)
        act = pra.gemm_gate_up_silu(x_q, a1, inp.w1, inp.w1_scale, s, e, npp, k, B, P, "stream")
        h_q, a2 = pra.per_token_quant_int8(act)
        down = pra.gemm_down(h_q, a2, inp.w2, inp.w2_scale, inp.topk_weights, s, e, npp, B, "stream")
        want = torch.empty(M, H, dtype=torch.bfloat16, device=DEV)
        pra.moe_sum(down.view(M, k, H), want)
        ws = torch.empty((pra.workspace_bytes(M, k, E, H, I, B),), dtype=torch.uint8, device=DEV)
        for fill in (0, 0xFF, 0x5A):
            ws.fill_(fill)
            out = pra.fused_experts(*inp.fused_experts_args(), **inp.fused_experts_kwargs(), block_size_m=B,
                                    workspace=ws, gemm_variant="stream")
            torch.cuda.synchronize()
            same = bool(torch.equal(out, want))
            assert same, (routing, fill, int((out != want).sum()))


# Whole-output checks at full size.  The sampled-token comparison above sees 6 rows; a tile
# scheduler that dropped or duplicated a tile elsewhere would leave finite stale rows there.  The
# streaming family uses none of the tiled families' scheduling code (one workgroup per block and
# channel group, no persistent loop, no tile list), so bit-equality of the complete outputs of two
# families over every row is a check of all of them.  The families share one SiLU definition and
# the same integer accumulators, so the layer output is bit-identical by construction.
FULL_SIZE = [
    ("qwen3-30b-a3b", 8192), ("glm-4.5-air", 4096), ("deepseek-v3", 2048), ("deepseek-v3", 16384),
]


@pytest.mark.parametrize("shape_name,M", FULL_SIZE)
def test_full_size_whole_output_equal_across_families(pra, shape_name, M):
    im = inputs_mod()
    inp = im.make_inputs(shape_name, M, seed=M + 7, device=DEV, weights_on_device=True)
    stream = _run(pra, inp, gemm_variant="stream")
    assert bool(torch.isfinite(stream.float()).all())
    # what the library picks by itself, and both geometries of the LDS-tiled family
    for variant in ("auto", "tile_wide", "tile_deep", "tile_ring"):
        tiled = _run(pra, inp, gemm_variant=variant)
        differing = int((tiled != stream).sum())
        assert differing == 0, f"{variant}: {differing} of {tiled.numel()} elements differ between the families"
        del tiled
    # and stage by stage on the device: the down GEMM of the tiled family against the streaming one
    P = M * inp.topk_ids.shape[1]
    x_q, a1 = pra.per_token_quant_int8(inp.hidden_states)
    E = inp.w1.shape[0]
    s, e, npp = pra.moe_align_block_size(inp.topk_ids, 64, E)
    act = pra.gemm_gate_up_silu(x_q, a1, inp.w1, inp.w1_scale, s, e, npp, inp.topk_ids.shape[1], 64, P, "stream")
    h_q, a2 = pra.per_token_quant_int8(act)
    d_auto = pra.gemm_down(h_q, a2, inp.w2, inp.w2_scale, inp.topk_weights, s, e, npp, 64, "auto")
    d_stream = pra.gemm_down(h_q, a2, inp.w2, inp.w2_scale, inp.topk_weights, s, e, npp, 64, "stream")
    assert torch.equal(d_auto, d_stream)


def test_capture_never_allocates_the_default_workspace(pra):
    """Under HIP graph capture the default workspace is never created or grown: a capture that finds
    none raises, one that finds a reserved buffer replays correctly after a larger eager call."""
    im = inputs_mod()
    inp = im.make_inputs("qwen3-30b-a3b", 32, seed=5).to(DEV)
    big = im.make_inputs("qwen3-30b-a3b", 256, seed=6).to(DEV)
    eager = _run(pra, inp)
    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream):
        graph = torch.cuda.CUDAGraph()
        with pytest.raises(RuntimeError, match="reserve_workspace"):
            with torch.cuda.graph(graph, stream=stream):
                pra.fused_experts(*inp.fused_experts_args(), **inp.fused_experts_kwargs())
    torch.cuda.synchronize()
    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream):
        shape = im.SHAPES["qwen3-30b-a3b"]
        pra.reserve_workspace(256, shape.k, shape.E_total, shape.H, shape.I)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            out = pra.fused_experts(*inp.fused_experts_args(), **inp.fused_experts_kwargs())
        for _ in range(3):
            graph.replay()
            torch.cuda.synchronize()
            assert torch.equal(out, eager)
            # eager work at the reserved size on the same stream between replays: same buffer, no regrowth
            pra.fused_experts(*big.fused_experts_args(), **big.fused_experts_kwargs())
            torch.cuda.synchronize()


def test_captured_graph_survives_a_larger_eager_call(pra):
    """A graph captured against the default workspace keeps replaying correctly after an eager call on the
    same stream has needed a larger one: the buffer the graph holds stays allocated (it is retired, not
    freed) and is not handed to anything else."""
    im = inputs_mod()
    api = pra.api
    shape = im.SHAPES["qwen3-30b-a3b"]
    inp = im.make_inputs(shape, 32, seed=15).to(DEV)
    big = im.make_inputs(shape, 256, seed=16).to(DEV)
    eager = _run(pra, inp)
    eager_big = _run(pra, big)
    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream):
        reserved = pra.reserve_workspace(32, shape.k, shape.E_total, shape.H, shape.I)
        key = (reserved.device.index, stream.cuda_stream)
        assert api._workspaces[key] is reserved
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            out = pra.fused_experts(*inp.fused_experts_args(), **inp.fused_experts_kwargs())
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, eager)
        # larger than reserved, same stream, eager: the cache entry grows by replacement ...
        got_big = pra.fused_experts(*big.fused_experts_args(), **big.fused_experts_kwargs())
        torch.cuda.synchronize()
        assert torch.equal(got_big, eager_big)
        grown = api._workspaces[key]
        assert grown is not reserved and grown.numel() > reserved.numel()
        # ... and the captured buffer is still referenced, so the allocator cannot hand it out again
        assert any(t is reserved for t in api._retired_workspaces)
        fill = [torch.full((reserved.numel(),), 0x5A, dtype=torch.uint8, device=DEV) for _ in range(4)]
        assert all(f.data_ptr() != reserved.data_ptr() for f in fill)
        for _ in range(3):
            out.zero_()
            graph.replay()
            torch.cuda.synchronize()
            assert torch.equal(out, eager)
            assert all(bool((f == 0x5A).all()) for f in fill)  # the replay wrote nothing outside its own buffer
            assert torch.equal(pra.fused_experts(*big.fused_experts_args(), **big.fused_experts_kwargs()), eager_big)
            torch.cuda.synchronize()


def test_apply_adapter_and_out_keyword_on_device(pra, oracle):
    """The modular-kernel adapter (``Int8W8A8HipExperts.apply(output, hidden_states, w1, w2, topk_weights,
    topk_ids, ...)``) and the ``out=`` keyword of ``fused_experts`` on device tensors: the caller's tensor is
    written, bit-equal to the plain call, within tolerance of the oracle; ``out`` may alias the input."""
    im = inputs_mod()
    for name, M in (("toy", 100), ("qwen3-30b-a3b", 48)):
        inp = im.make_inputs(name, M, seed=31).to(DEV)
        plain = _run(pra, inp)
        cpu = inp.to("cpu")
        want = oracle.fused_experts(cpu.hidden_states, cpu.w1, cpu.w2, cpu.topk_weights, cpu.topk_ids,
                                    cpu.w1_scale, cpu.w2_scale, 64)
        assert rel_err(plain, want) < TOL
        # out=
        out = torch.full_like(inp.hidden_states, float("nan"))
        ret = pra.fused_experts(*inp.fused_experts_args(), out=out, **inp.fused_experts_kwargs())
        assert ret is out and torch.equal(out, plain)
        # the adapter: output first, vLLM's keyword names, its two workspaces ignored
        experts = pra.vllm_plugin.Int8W8A8HipExperts(inp.w1_scale, inp.w2_scale)
        output = torch.full_like(inp.hidden_states, float("nan"))
        before = output.data_ptr()
        junk = torch.empty(16, device=DEV)
        experts.apply(output, inp.hidden_states, inp.w1, inp.w2, inp.topk_weights, inp.topk_ids, activation="silu",
                      global_num_experts=inp.w1.shape[0], expert_map=None, a1q_scale=None, a2_scale=None,
                      workspace13=junk, workspace2=junk, expert_tokens_meta=None, apply_router_weight_on_input=False)
        assert output.data_ptr() == before and torch.equal(output, plain)
        assert rel_err(output, want) < TOL
        with pytest.raises(NotImplementedError):
            experts.apply(output, inp.hidden_states, inp.w1, inp.w2, inp.topk_weights, inp.topk_ids,
                          expert_map=torch.arange(inp.w1.shape[0], device=DEV))
        # in place: out is the input tensor
        x = inp.hidden_states.clone()
        ret = pra.fused_experts(x, *inp.fused_experts_args()[1:], out=x, **inp.fused_experts_kwargs())
        assert ret is x and torch.equal(x, plain)
        # wrong shape or dtype of out is refused before anything runs
        with pytest.raises(ValueError):
            pra.fused_experts(*inp.fused_experts_args(), out=out[:, :-8], **inp.fused_experts_kwargs())
        with pytest.raises(ValueError):
            pra.fused_experts(*inp.fused_experts_args(), out=out.float(), **inp.fused_experts_kwargs())


# The LDS-tiled family builds its tile list inside the kernel; inside fused_experts (expert ids known to
# ascend) from per-expert runs, two experts per thread.  Routings that stress that list: more than 512
# experts with most of them absent, a single expert holding every row (dozens of tiles of one expert,
# i.e. several groups of eight), one row per expert, and both block sizes.  The streaming family has no
# tile list, so bit-equality of the complete outputs is the check.
@pytest.mark.parametrize("E,k,M,B,routing", [
    (640, 2, 700, 64, "softmax"),     # > 512 experts: both slots of a thread, many absent experts
    (1024, 1, 300, 64, "softmax"),    # the largest expert count the library takes, most experts absent
    (8, 1, 3000, 64, "one_hot"),      # one expert holds all 3000 rows
    (8, 1, 3000, 128, "one_hot"),
    (40, 4, 10, 128, "softmax"),      # one row per expert at most
    (16, 2, 1100, 128, "zipf"),
])
@pytest.mark.parametrize("variant", ["tile_wide", "tile_deep", "tile_ring"])
def test_tile_list_edge_routings(pra, E, k, M, B, routing, variant):
    im = inputs_mod()
    shape = im.LayerShape("edge", E=E, k=k, H=512, I=512, routing="softmax" if routing == "one_hot" else routing)
    inp = im.make_inputs(shape, M, seed=E + M).to(DEV)
    if routing == "one_hot":
        inp.topk_ids.fill_(3)
    want = _run(pra, inp, gemm_variant="stream", block_size_m=B)
    got = _run(pra, inp, gemm_variant=variant, block_size_m=B)
    differing = int((got != want).sum())
    assert differing == 0, f"{differing} of {got.numel()} elements differ"
