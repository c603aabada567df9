"""GPU parity (bit-exact): per-output-channel weight quantisation into the kernel layout through the
C-ABI against the CPU oracle, and the quantised weights driving the layer."""

import pytest
import torch

from _util import inputs_mod, rel_err

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _weights(E, I, H, seed, spread=True):
    g = torch.Generator().manual_seed(seed)
    gate = torch.randn(E, I, H, generator=g) * H ** -0.5
    up = torch.randn(E, I, H, generator=g) * H ** -0.5
    down = torch.randn(E, H, I, generator=g) * I ** -0.5
    if spread:  # row magnitudes over several decades, some rows exactly zero
        gate *= torch.logspace(-3, 1, I)[None, :, None]
        down[:, ::7] = 0.0
    return gate.to(torch.bfloat16), up.to(torch.bfloat16), down.to(torch.bfloat16)


def test_tie_vector(pra, oracle):
    w = torch.tensor([[127.0, 0.5, 1.5, 2.5, -0.5, -1.5, -2.5, -127.0, 3.5, 126.5, 0.0, 0.25, 0.75, -0.75, 64.5, -64.5]],
                     dtype=torch.bfloat16)
    q, s = pra.quantize_weights_per_channel(w.to(DEV))
    assert q.cpu().tolist() == [[127, 0, 2, 2, 0, -2, -2, -127, 4, 126, 0, 0, 1, -1, 64, -64]]
    assert s.cpu().tolist() == [1.0]


@pytest.mark.parametrize("rows,cols", [(1, 8), (5, 24), (64, 512), (33, 520), (7, 768), (16, 2048), (9, 4096),
                                       (3, 8192), (2, 8200), (4, 16384)])
def test_rows_match_oracle(pra, oracle, rows, cols):
    g = torch.Generator().manual_seed(rows * 131 + cols)
    w = (torch.randn(rows, cols, generator=g) * torch.logspace(-6, 3, rows)[:, None]).to(torch.bfloat16)
    if rows > 2:
        w[1] = 0.0
        w[2] = 0.0
        w[2, cols // 2] = 2.0 ** -100
    q, s = pra.quantize_weights_per_channel(w.to(DEV))
    qo, so = oracle.quantize_weights_per_channel(w)
    assert torch.equal(q.cpu(), qo) and torch.equal(s.cpu(), so)


@pytest.mark.parametrize("shape_name", ["toy", "qwen3-30b-a3b"])
def test_expert_weights_layout_and_values(pra, oracle, shape_name):
    shape = inputs_mod().SHAPES[shape_name]
    E = min(shape.E_total, 16)
    gate, up, down = _weights(E, shape.I, shape.H, seed=3)
    w13, s13, w2, s2 = pra.quantize_expert_weights(gate.to(DEV), up.to(DEV), down.to(DEV))
    o13, os13, o2, os2 = oracle.quantize_expert_weights(gate, up, down)
    assert w13.shape == (E, 2 * shape.I, shape.H) and w2.shape == (E, shape.H, shape.I)
    assert torch.equal(w13.cpu(), o13) and torch.equal(s13.cpu(), os13)
    assert torch.equal(w2.cpu(), o2) and torch.equal(s2.cpu(), os2)


def test_in_place_update_of_engine_parameters(pra, oracle):
    # a policy step changes the trainer weights; the engine's tensors are overwritten where they lie
    shape = inputs_mod().SHAPES["toy"]
    E, I, H = shape.E_total, shape.I, shape.H
    g0 = [t.to(DEV) for t in _weights(E, I, H, seed=10, spread=False)]
    params = pra.quantize_expert_weights(*g0)
    ptrs = [t.data_ptr() for t in params]
    new = _weights(E, I, H, seed=11, spread=False)
    again = pra.quantize_expert_weights(*[t.to(DEV) for t in new], out=params)
    assert [t.data_ptr() for t in again] == ptrs
    want = oracle.quantize_expert_weights(*new)
    for got, ref in zip(params, want):
        assert torch.equal(got.cpu(), ref)
    # and the layer on the updated parameters equals the oracle's layer on the oracle's parameters
    im = inputs_mod()
    x = torch.randn(48, H, generator=torch.Generator().manual_seed(2)).to(torch.bfloat16)
    tw, ids = im.route(shape, 48, torch.Generator().manual_seed(3))
    out = pra.fused_experts(x.to(DEV), params[0], params[2], tw.to(DEV), ids.to(DEV), use_int8_w8a8=True,
                            per_channel_quant=True, w1_scale=params[1], w2_scale=params[3])
    ref = oracle.fused_experts(x, want[0], want[2], tw, ids, want[1], want[3])
    assert rel_err(out.cpu(), ref) < 1e-2


def test_full_size_properties(pra):
    # Qwen3-30B-A3B layer at full size (E=128): properties that need no CPU pass over 600 MB
    shape = inputs_mod().SHAPES["qwen3-30b-a3b"]
    E, I, H = shape.E_total, shape.I, shape.H
    g = torch.Generator(device=DEV).manual_seed(4)
    gate = (torch.randn(E, I, H, generator=g, device=DEV) * 0.02).to(torch.bfloat16)
    up = (torch.randn(E, I, H, generator=g, device=DEV) * 0.02).to(torch.bfloat16)
    down = (torch.randn(E, H, I, generator=g, device=DEV) * 0.02).to(torch.bfloat16)
    w13, s13, w2, s2 = pra.quantize_expert_weights(gate, up, down)
    for w, q, s in ((gate, w13[:, :I], s13[:, :I]), (up, w13[:, I:], s13[:, I:]), (down, w2, s2)):
        wf = w.float()
        absmax = wf.abs().amax(-1)
        # tensor / tensor: a true division (tensor / python-float multiplies by a rounded reciprocal)
        same_scale = torch.equal(s, (absmax / torch.full_like(absmax, 127.0)).clamp(min=1e-12))
        assert same_scale
        hits_127 = bool((q.abs().amax(-1) == 127).all())
        assert hits_127
        s64 = s.double()[..., None]
        half_step = bool(((q.double() * s64 - wf.double()).abs() <= s64 * (0.5 + 127 * 2.0 ** -23)).all())
        assert half_step
    # negation symmetry and idempotence on the dequantised weights' grid
    w13n, s13n, _, _ = pra.quantize_expert_weights(-gate, -up, down)
    negated = torch.equal(w13n, -w13) and torch.equal(s13n, s13)
    assert negated


def test_argument_errors(pra):
    w = torch.zeros(4, 16, dtype=torch.bfloat16, device=DEV)
    with pytest.raises(NotImplementedError):
        pra.quantize_weights_per_channel(w.float())
    with pytest.raises(ValueError):
        pra.quantize_weights_per_channel(torch.zeros(4, 12, dtype=torch.bfloat16, device=DEV))
    with pytest.raises(ValueError):
        pra.quantize_weights_per_channel(w.cpu())
    with pytest.raises(ValueError):
        pra.quantize_expert_weights(w.view(1, 4, 16), w.view(1, 4, 16), w.view(1, 4, 16))


def test_policy_update_hook_writes_layer_parameters_in_place(pra, oracle):
    """``load_quantized_expert_weights`` (the int8 counterpart of the reference's in-place
    ``param.copy_`` loop, src/prime_rl/inference/vllm/worker/weight_transfer.py:97-134): the four
    parameters of the named layer are rewritten at their addresses, the layer's output afterwards is
    the oracle's on the re-quantised weights, another layer in the same dict is untouched, and a
    missing name or a wrong shape raises before anything is written."""
    im = inputs_mod()
    shape = im.SHAPES["toy"]
    E, I, H = shape.E_total, shape.I, shape.H
    old = pra.quantize_expert_weights(*[t.to(DEV) for t in _weights(E, I, H, seed=20, spread=False)])
    other = pra.quantize_expert_weights(*[t.to(DEV) for t in _weights(E, I, H, seed=21, spread=False)])
    names = ("w13_weight", "w13_weight_scale", "w2_weight", "w2_weight_scale")
    params = {}
    for layer, tensors, nested in (("model.layers.0.mlp.experts", old, ".routed_experts"),
                                   ("model.layers.1.mlp.experts", other, "")):
        for name, t in zip(names, tensors):
            if name.endswith("_scale"):
                t = t.unsqueeze(-1).contiguous()  # the engine keeps [E, N, 1]
            params[f"{layer}{nested}.{name}"] = torch.nn.Parameter(t, requires_grad=False)
    ptrs = {k: v.data_ptr() for k, v in params.items()}
    before_other = {k: v.detach().clone() for k, v in params.items() if ".layers.1." in k}
    new = _weights(E, I, H, seed=22, spread=False)
    written = pra.load_quantized_expert_weights(params, "model.layers.0.mlp.experts", *[t.to(DEV) for t in new])
    assert written == [f"model.layers.0.mlp.experts.routed_experts.{n}" for n in names]
    assert {k: v.data_ptr() for k, v in params.items()} == ptrs
    for k, v in before_other.items():
        assert torch.equal(params[k], v)
    want = oracle.quantize_expert_weights(*new)
    got = [params[f"model.layers.0.mlp.experts.routed_experts.{n}"] for n in names]
    assert torch.equal(got[0].cpu(), want[0]) and torch.equal(got[1].cpu().squeeze(-1), want[1])
    assert torch.equal(got[2].cpu(), want[2]) and torch.equal(got[3].cpu().squeeze(-1), want[3])
    x = torch.randn(40, H, generator=torch.Generator().manual_seed(5)).to(torch.bfloat16)
    tw, ids = im.route(shape, 40, torch.Generator().manual_seed(6))
    out = pra.fused_experts(x.to(DEV), got[0], got[2], tw.to(DEV), ids.to(DEV), use_int8_w8a8=True,
                            per_channel_quant=True, w1_scale=got[1], w2_scale=got[3])
    ref = oracle.fused_experts(x, want[0], want[2], tw, ids, want[1], want[3])
    assert rel_err(out.cpu(), ref) < 1e-2
    # a worker that holds a subset of the experts takes its rows of the trainer's tensors
    sub = torch.tensor([5, 1, 6], device=DEV)
    small = {f"l.{n}": torch.nn.Parameter(t[:3].clone(), requires_grad=False) for n, t in zip(names, old)}
    pra.load_quantized_expert_weights(small, "l", *[t.to(DEV) for t in new], source_indices=sub)
    assert torch.equal(small["l.w13_weight"].cpu(), want[0][[5, 1, 6]])
    assert torch.equal(small["l.w2_weight_scale"].cpu(), want[3][[5, 1, 6]])
    # errors come before any write
    snapshot = got[0].detach().clone()
    with pytest.raises(ValueError, match="not found in model"):
        pra.load_quantized_expert_weights(params, "model.layers.7.mlp.experts", *[t.to(DEV) for t in new])
    with pytest.raises(ValueError, match="shape mismatches"):
        pra.load_quantized_expert_weights(params, "model.layers.0.mlp.experts",
                                          *[t[:4].to(DEV) for t in new])
    assert torch.equal(got[0], snapshot)


def test_model_level_weight_update_from_a_name_tensor_stream(pra, oracle):
    """``load_weights_kernel_int8``, the int8 counterpart of the reference's ``load_weights_kernel``
    (src/prime_rl/inference/vllm/worker/weight_transfer.py:97-134), on a two-layer stand-in model: one layer's
    experts arrive under the trainer's names (gate_proj / up_proj / down_proj), the other's in kernel format
    (bf16 w13_weight / w2_weight) and interleaved with other tensors; the engine nests one layer's parameters
    under ``routed_experts`` and keeps the other flat.  Every parameter is rewritten at its address with the
    oracle's bits; tensors that are not expert weights are copied; bad names and shapes are all reported in
    ONE error after everything valid has been written."""
    im = inputs_mod()
    shape = im.SHAPES["toy"]
    E, I, H = shape.E_total, shape.I, shape.H
    names = ("w13_weight", "w13_weight_scale", "w2_weight", "w2_weight_scale")
    params = {}
    for layer, nested, seed in ((0, ".routed_experts", 30), (1, "", 31)):
        old = pra.quantize_expert_weights(*[t.to(DEV) for t in _weights(E, I, H, seed=seed, spread=False)])
        for name, t in zip(names, old):
            if name.endswith("_scale") and layer == 0:
                t = t.unsqueeze(-1).contiguous()
            params[f"model.layers.{layer}.mlp.experts{nested}.{name}"] = torch.nn.Parameter(t, requires_grad=False)
        params[f"model.layers.{layer}.input_layernorm.weight"] = torch.nn.Parameter(
            torch.zeros(H, dtype=torch.bfloat16, device=DEV), requires_grad=False)
    ptrs = {k: v.data_ptr() for k, v in params.items()}
    new0 = _weights(E, I, H, seed=32, spread=False)
    new1 = _weights(E, I, H, seed=33, spread=True)
    norm = torch.randn(H, generator=torch.Generator().manual_seed(3)).to(torch.bfloat16)

    def stream():
        yield "model.layers.0.mlp.experts.gate_proj", new0[0].to(DEV)
        yield "model.layers.1.mlp.experts.w2_weight", new1[2].to(DEV)           # kernel format, bf16 payload
        yield "model.layers.0.input_layernorm.weight", norm.to(DEV)
        yield "model.layers.0.mlp.experts.down_proj", new0[2].to(DEV)
        yield "model.layers.1.mlp.experts.w13_weight", torch.cat([new1[0], new1[1]], dim=1).to(DEV)
        yield "model.layers.0.mlp.experts.up_proj", new0[1].to(DEV)
        yield "model.layers.1.input_layernorm.weight", (norm * 2).to(DEV)

    class Model:  # enough of a module: named_parameters()
        def named_parameters(self):
            return iter(params.items())

    result = pra.load_weights_kernel_int8(Model(), stream())
    assert sorted(result["quantized_layers"]) == ["model.layers.0.mlp.experts", "model.layers.1.mlp.experts"]
    assert sorted(result["loaded"]) == sorted(params)
    assert {k: v.data_ptr() for k, v in params.items()} == ptrs
    for layer, nested, new in ((0, ".routed_experts", new0), (1, "", new1)):
        want = oracle.quantize_expert_weights(*new)
        got = [params[f"model.layers.{layer}.mlp.experts{nested}.{n}"].cpu() for n in names]
        assert torch.equal(got[0], want[0]) and torch.equal(got[1].reshape(want[1].shape), want[1])
        assert torch.equal(got[2], want[2]) and torch.equal(got[3].reshape(want[3].shape), want[3])
    assert torch.equal(params["model.layers.0.input_layernorm.weight"].cpu(), norm)
    assert torch.equal(params["model.layers.1.input_layernorm.weight"].cpu(), norm * 2)
    # the layer computes with the new weights
    x = torch.randn(24, H, generator=torch.Generator().manual_seed(5)).to(torch.bfloat16)
    tw, ids = im.route(shape, 24, torch.Generator().manual_seed(6))
    l1 = [params[f"model.layers.1.mlp.experts.{n}"] for n in names]
    out = pra.fused_experts(x.to(DEV), l1[0], l1[2], tw.to(DEV), ids.to(DEV), use_int8_w8a8=True,
                            per_channel_quant=True, w1_scale=l1[1], w2_scale=l1[3])
    want1 = oracle.quantize_expert_weights(*new1)
    assert rel_err(out.cpu(), oracle.fused_experts(x, want1[0], want1[2], tw, ids, want1[1], want1[3])) < 1e-2

    # a stream with several faults: everything valid is still written, one error names all the rest
    newer = _weights(E, I, H, seed=34, spread=False)

    def faulty():
        yield "model.layers.1.mlp.experts.gate_proj", newer[0].to(DEV)
        yield "model.layers.9.mlp.experts.gate_proj", newer[0].to(DEV)          # a layer the model does not have ...
        yield "model.layers.9.mlp.experts.up_proj", newer[1].to(DEV)
        yield "model.layers.9.mlp.experts.down_proj", newer[2].to(DEV)
        yield "model.layers.0.mlp.experts.gate_proj", newer[0][:4].to(DEV)      # ... wrong expert count ...
        yield "model.layers.0.mlp.experts.up_proj", newer[1][:4].to(DEV)
        yield "model.layers.0.mlp.experts.down_proj", newer[2][:4].to(DEV)
        yield "model.layers.1.mlp.experts.up_proj", newer[1].to(DEV)
        yield "model.norm.weight", norm.to(DEV)                                  # ... an unknown plain tensor ...
        yield "model.layers.0.input_layernorm.weight", norm[:-8].to(DEV)        # ... a plain tensor of the wrong shape
        yield "model.layers.1.mlp.experts.down_proj", newer[2].to(DEV)
        yield "model.layers.0.mlp.experts.w13_weight", torch.cat([newer[0], newer[1]], dim=1).to(DEV)  # never completed

    layer0_before = params["model.layers.0.mlp.experts.routed_experts.w13_weight"].detach().clone()
    with pytest.raises(ValueError) as err:
        pra.load_weights_kernel_int8(params, faulty())
    msg = str(err.value)
    assert "shape mismatches" in msg and "not found in model" in msg
    for fragment in ("model.layers.9.mlp.experts.w13_weight", "model.norm.weight", "model.layers.0.input_layernorm.weight",
                     "model.layers.0.mlp.experts.routed_experts.w13_weight", "incomplete expert group"):
        assert fragment in msg, fragment
    assert torch.equal(params["model.layers.0.mlp.experts.routed_experts.w13_weight"], layer0_before)
    want = oracle.quantize_expert_weights(*newer)
    assert torch.equal(params["model.layers.1.mlp.experts.w13_weight"].cpu(), want[0])   # the valid layer was written
    assert {k: v.data_ptr() for k, v in params.items()} == ptrs
