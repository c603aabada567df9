"""GPU parity: router top-k (ids exact, weights to 1e-5 relative) and the routed-experts record through the
C-ABI against the CPU oracle."""

import base64

import numpy as np
import pytest
import torch

from _util import inputs_mod

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
RTOL = 1e-5  # fp32 exp / division on two different implementations


def _selection_values(logits, score_func, bias):
    lf = logits.float()
    s = torch.softmax(lf, 1) if score_func == "softmax" else torch.sigmoid(lf) if score_func == "sigmoid" else lf
    return s if bias is None else s + bias.reshape(1, -1)


def _check(pra, oracle, logits, k, score_func="softmax", renormalize=True, route_scale=1.0, bias=None, G=1, KG=1,
           top2=False):
    w, ids = pra.route_topk(logits.to(DEV), k, score_func=score_func, renormalize=renormalize,
                            route_scale=route_scale, selection_bias=None if bias is None else bias.to(DEV),
                            num_expert_group=G, topk_group=KG, group_score_top2=top2)
    torch.cuda.synchronize()
    wo, ido = oracle.route_topk(logits, k, score_func, renormalize, route_scale, bias, G, KG, top2)
    w, ids = w.cpu(), ids.cpu()
    same = (ids == ido).all(dim=1)
    if not bool(same.all()):
        # the device exp differs from the host's in the last bits, so two experts whose selection
        # values agree to float32 resolution may swap: accept a row only if the chosen values do
        sel = _selection_values(logits, score_func, bias)
        rows = torch.nonzero(~same).flatten()
        assert rows.numel() <= max(1, logits.shape[0] // 500), f"{rows.numel()} rows differ"
        got = sel[rows].gather(1, ids[rows].long())
        want = sel[rows].gather(1, ido[rows].long())
        torch.testing.assert_close(got, want, rtol=1e-6, atol=1e-9)
    good = same
    torch.testing.assert_close(w[good], wo[good], rtol=RTOL, atol=1e-9)
    assert all(len(set(r)) == k for r in ids.tolist())
    return w, ids


@pytest.mark.parametrize("E,k", [(8, 2), (60, 6), (64, 8), (128, 8), (160, 6), (256, 8), (384, 8), (512, 10), (1024, 16)])
@pytest.mark.parametrize("score_func", ["softmax", "sigmoid", "topk_softmax"])
def test_ungrouped_routers(pra, oracle, E, k, score_func):
    g = torch.Generator().manual_seed(E + k)
    logits = torch.randn(257, E, generator=g) * 2.0
    _check(pra, oracle, logits, k, score_func, renormalize=True)
    _check(pra, oracle, logits, k, score_func, renormalize=False, route_scale=2.5,
           bias=torch.randn(E, generator=g) * 0.2)


@pytest.mark.parametrize("E,k,G,KG", [(256, 8, 8, 4), (128, 8, 1, 1), (64, 6, 8, 3), (32, 4, 4, 2), (512, 8, 16, 4),
                                      (1024, 8, 8, 2), (16, 2, 8, 2)])
@pytest.mark.parametrize("top2", [True, False])
def test_grouped_routers(pra, oracle, E, k, G, KG, top2):
    g = torch.Generator().manual_seed(E * 3 + G)
    logits = torch.randn(130, E, generator=g) * 1.5
    bias = torch.randn(E, generator=g) * 0.1
    _, ids = _check(pra, oracle, logits, k, "sigmoid", True, 2.5, bias, G, KG, top2)
    assert all(len({e // (E // G) for e in r}) <= KG for r in ids.tolist())
    _check(pra, oracle, logits, k, "softmax", False, 1.0, None, G, KG, top2)


def test_equal_values_go_to_the_lowest_index(pra):
    logits = torch.tensor([[1.0, 3.0, 3.0, 0.0, 3.0, 2.0, 2.0, -1.0]], device=DEV)
    _, ids = pra.route_topk(logits, 5, score_func="topk_softmax", renormalize=False)
    assert ids.cpu().tolist() == [[1, 2, 4, 5, 6]]
    logits = torch.tensor([[5.0, 0.0, 5.0, 0.0, 4.0, 4.0, 1.0, 1.0]], device=DEV)
    _, ids = pra.route_topk(logits, 2, score_func="topk_softmax", renormalize=False, num_expert_group=4, topk_group=1)
    assert ids.cpu().tolist() == [[0, 1]]
    # all equal: first k indices, uniform weights
    w, ids = pra.route_topk(torch.zeros(3, 128, device=DEV), 8)
    assert ids.cpu().tolist() == [list(range(8))] * 3
    torch.testing.assert_close(w.cpu(), torch.full((3, 8), 0.125))


@pytest.mark.parametrize("shape_name,M", [("qwen3-30b-a3b", 16), ("qwen3-30b-a3b", 8192), ("glm-4.5-air", 4096),
                                          ("deepseek-v3", 64), ("deepseek-v3", 16384)])
def test_baseline_shapes_match_the_workload_generator(pra, oracle, shape_name, M):
    # the routing of the benchmark workloads, now from the device router
    im = inputs_mod()
    shape = im.SHAPES[shape_name]
    g = torch.Generator().manual_seed(M)
    logits = torch.randn(M, shape.E, generator=g)
    if shape.routing == "grouped":
        bias = torch.randn(shape.E, generator=g) * 0.1
        w, ids = _check(pra, oracle, logits, shape.k, "sigmoid", True, 1.0, bias, shape.n_group, shape.topk_group, True)
    else:
        w, ids = _check(pra, oracle, logits, shape.k, "softmax", True)
    torch.testing.assert_close(w.sum(1), torch.ones(M), rtol=0, atol=5e-6)
    # size-independent properties at full size: descending selection, ids in range and distinct
    assert int(ids.min()) >= 0 and int(ids.max()) < shape.E
    s = torch.sort(ids, dim=1)[0]
    assert bool((s[:, 1:] != s[:, :-1]).all())


def test_vllm_entry_points(pra, oracle):
    g = torch.Generator().manual_seed(8)
    x = torch.zeros(33, 64, dtype=torch.bfloat16, device=DEV)
    logits = torch.randn(33, 256, generator=g)
    w, ids = pra.fused_topk(x, logits.to(DEV), 8, True)
    wo, ido = oracle.softmax_topk(logits, 8)
    assert torch.equal(ids.cpu(), ido)
    torch.testing.assert_close(w.cpu(), wo, rtol=RTOL, atol=1e-9)
    bias = torch.randn(256, generator=g) * 0.1
    w, ids = pra.grouped_topk(x, logits.to(DEV), 8, True, 8, 4, "sigmoid", 2.5, bias.to(DEV))
    wo, ido = oracle.grouped_topk(logits, bias, 8, 8, 4, True, 2.5)
    assert torch.equal(ids.cpu(), ido)
    torch.testing.assert_close(w.cpu(), wo, rtol=RTOL, atol=1e-9)
    with pytest.raises(ValueError):
        pra.fused_topk(x[:5], logits.to(DEV), 8, True)
    with pytest.raises(NotImplementedError):
        pra.route_topk(logits.to(DEV), 8, score_func="tanh")
    with pytest.raises(NotImplementedError):
        pra.route_topk(logits.to(DEV).half(), 8)
    with pytest.raises(pra._abi.MoeI8Error):
        pra.route_topk(logits.to(DEV), 8, num_expert_group=3)  # 256 % 3
    with pytest.raises(pra._abi.MoeI8Error):
        pra.route_topk(logits.to(DEV), 65)


@pytest.mark.parametrize("E,dtype", [(128, torch.uint8), (256, torch.uint8), (512, torch.uint16)])
def test_routed_experts_record(pra, oracle, E, dtype):
    # three layers route the same 50 tokens; each launch fills its slice of the [seq, layers, k] record
    M, L, k = 50, 3, 8
    g = torch.Generator().manual_seed(E)
    record = torch.full((M, L, k), 7, dtype=dtype, device=DEV)
    all_ids = []
    for layer in (2, 0, 1):
        logits = torch.randn(M, E, generator=g)
        _, ids = pra.route_topk(logits.to(DEV), k, routed_experts_out=(record, layer))
        _, ido = oracle.route_topk(logits, k)
        assert torch.equal(ids.cpu(), ido)
        all_ids.append((layer, ido))
    want = np.zeros((M, L, k), dtype=np.int64)
    for layer, ido in all_ids:
        want[:, layer, :] = ido.numpy()
    payload = pra.routed_experts_payload(record, start=5)
    ref = oracle.serialize_routed_experts(want, start=5)
    if E <= 256:
        assert payload == ref  # byte for byte the reference's wire form
    else:
        assert payload["dtype"] == "uint16" == ref["dtype"] and payload["data"] == ref["data"]
    dec = np.frombuffer(base64.b64decode(payload["data"]), dtype=payload["dtype"]).reshape(payload["shape"])
    np.testing.assert_array_equal(dec, want)
    with pytest.raises(ValueError):
        pra.route_topk(torch.zeros(M, E, device=DEV), k, routed_experts_out=(record, 3))
    if E > 256:
        small = torch.zeros((M, L, k), dtype=torch.uint8, device=DEV)
        with pytest.raises(pra._abi.MoeI8Error):
            pra.route_topk(torch.zeros(M, E, device=DEV), k, routed_experts_out=(small, 0))


def test_router_feeds_the_layer(pra, oracle):
    # router -> fused_experts on the device equals oracle router -> oracle layer
    im = inputs_mod()
    shape = im.SHAPES["toy"]
    inp = im.make_inputs(shape, 40, seed=21)
    logits = torch.randn(40, shape.E, generator=torch.Generator().manual_seed(5))
    w, ids = pra.route_topk(logits.to(DEV), shape.k)
    wo, ido = oracle.route_topk(logits, shape.k)
    assert torch.equal(ids.cpu(), ido)
    d = inp.to(DEV)
    out = pra.fused_experts(d.hidden_states, d.w1, d.w2, w, ids, use_int8_w8a8=True, per_channel_quant=True,
                            w1_scale=d.w1_scale, w2_scale=d.w2_scale)
    ref = oracle.fused_experts(inp.hidden_states, inp.w1, inp.w2, wo, ido, inp.w1_scale, inp.w2_scale)
    from _util import rel_err
    assert rel_err(out.cpu(), ref) < 1e-2


def test_fused_moe_from_router_logits(pra, oracle):
    # vLLM fused_moe = routing + experts: softmax router on the toy shape, grouped sigmoid router on a
    # DeepSeek-like one, both against oracle router -> oracle layer
    from _util import rel_err

    im = inputs_mod()
    shape = im.SHAPES["toy"]
    inp = im.make_inputs(shape, 33, seed=4)
    d = inp.to(DEV)
    logits = torch.randn(33, shape.E, generator=torch.Generator().manual_seed(6))
    record = torch.zeros(33, 2, shape.k, dtype=torch.uint8, device=DEV)
    out = pra.fused_moe(d.hidden_states, d.w1, d.w2, logits.to(DEV), shape.k, True, use_int8_w8a8=True,
                        per_channel_quant=True, w1_scale=d.w1_scale, w2_scale=d.w2_scale,
                        routed_experts_out=(record, 1))
    wo, ido = oracle.route_topk(logits, shape.k)
    ref = oracle.fused_experts(inp.hidden_states, inp.w1, inp.w2, wo, ido, inp.w1_scale, inp.w2_scale)
    assert rel_err(out.cpu(), ref) < 1e-2
    assert torch.equal(record[:, 1, :].cpu().to(torch.int32), ido) and int(record[:, 0, :].abs().sum()) == 0
    gshape = im.LayerShape("g", E=64, k=6, H=256, I=128)
    ginp = im.make_inputs(gshape, 21, seed=5)
    gd = ginp.to(DEV)
    glogits = torch.randn(21, 64, generator=torch.Generator().manual_seed(7))
    bias = torch.randn(64, generator=torch.Generator().manual_seed(8)) * 0.1
    out = pra.fused_moe(gd.hidden_states, gd.w1, gd.w2, glogits.to(DEV), 6, True, use_grouped_topk=True,
                        num_expert_group=8, topk_group=3, use_int8_w8a8=True, per_channel_quant=True,
                        w1_scale=gd.w1_scale, w2_scale=gd.w2_scale, scoring_func="sigmoid",
                        routed_scaling_factor=2.5, e_score_correction_bias=bias.to(DEV))
    wo, ido = oracle.grouped_topk(glogits, bias, 6, 8, 3, True, 2.5)
    ref = oracle.fused_experts(ginp.hidden_states, ginp.w1, ginp.w2, wo, ido, ginp.w1_scale, ginp.w2_scale)
    assert rel_err(out.cpu(), ref) < 1e-2
