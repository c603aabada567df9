"""The vLLM plugin shim against a stand-in ``vllm`` module tree (vLLM itself is not installable here):
environment gate, idempotence through the marker attribute (the reference's pattern,
``src/prime_rl/inference/patches.py:57-58``), rebinding in modules that imported the name
(``patches.py:227-231``), fall-through for calls this library does not handle, keyword filtering, and
the ``apply``-shaped adapter.  No GPU: the HIP entry is replaced by a recorder."""

import sys
import types

import pytest
import torch


class _FakeCudaBf16:
    """Enough of a tensor for the dispatch decision."""
    is_cuda = True
    dtype = torch.bfloat16


def _install_fake_vllm(monkeypatch):
    calls = []

    def original_fused_experts(hidden_states, w1, w2, topk_weights, topk_ids, *args, **kwargs):
        calls.append(("original", kwargs))
        return "original"

    names = ["vllm", "vllm.model_executor", "vllm.model_executor.layers", "vllm.model_executor.layers.fused_moe",
             "vllm.model_executor.layers.fused_moe.fused_moe", "vllm.model_executor.layers.fused_moe.layer",
             "vllm.model_executor.layers.quantization"]
    mods = {n: types.ModuleType(n) for n in names}
    mods["vllm.model_executor.layers.fused_moe.fused_moe"].fused_experts = original_fused_experts
    # two modules that did `from ...fused_moe import fused_experts` at import time, one that did not
    mods["vllm.model_executor.layers.fused_moe"].fused_experts = original_fused_experts
    mods["vllm.model_executor.layers.fused_moe.layer"].fused_experts = original_fused_experts
    mods["vllm.model_executor.layers.quantization"].fused_experts = lambda *a, **k: "unrelated"
    for n, m in mods.items():
        monkeypatch.setitem(sys.modules, n, m)
    return mods, original_fused_experts, calls


@pytest.fixture
def plugin(pra, monkeypatch):
    hip_calls = []

    def hip_fused_experts(hidden_states, w1, w2, topk_weights, topk_ids, inplace=False, activation="silu",
                          apply_router_weight_on_input=False, use_int8_w8a8=False, per_channel_quant=False,
                          global_num_experts=-1, expert_map=None, w1_scale=None, w2_scale=None, a1_scale=None,
                          a2_scale=None, block_shape=None, *, workspace=None):
        hip_calls.append(dict(use_int8_w8a8=use_int8_w8a8, w1_scale=w1_scale, global_num_experts=global_num_experts))
        tag = w1_scale if isinstance(w1_scale, str) else ""
        if tag == "unsupported-shape":
            raise NotImplementedError("shape")
        if tag == "rejected-by-validation":
            raise ValueError("w2 must be [E, H, I]")
        if tag == "launch-failed":
            raise RuntimeError("launch")
        return "hip"

    monkeypatch.setattr(pra.api, "fused_experts", hip_fused_experts)
    return pra.vllm_plugin, hip_calls


def test_register_is_gated_by_the_environment(plugin, monkeypatch):
    vp, _ = plugin
    mods, original, _ = _install_fake_vllm(monkeypatch)
    monkeypatch.delenv(vp.ENV_FLAG, raising=False)
    assert vp.register() is False
    monkeypatch.setenv(vp.ENV_FLAG, "0")
    assert vp.register() is False
    assert mods[vp.FUSED_MOE_MODULE].fused_experts is original


def test_register_rebinds_every_importer_once(plugin, monkeypatch):
    vp, _ = plugin
    mods, original, _ = _install_fake_vllm(monkeypatch)
    monkeypatch.setenv(vp.ENV_FLAG, "1")
    assert vp.register() is True
    patched = mods[vp.FUSED_MOE_MODULE].fused_experts
    assert patched is not original and getattr(patched, vp._MARK) is True and patched.__wrapped__ is original
    assert mods["vllm.model_executor.layers.fused_moe"].fused_experts is patched
    assert mods["vllm.model_executor.layers.fused_moe.layer"].fused_experts is patched
    # a different function that happens to carry the same name is left alone
    assert mods["vllm.model_executor.layers.quantization"].fused_experts() == "unrelated"
    # second call: the marker makes it a no-op, nothing is wrapped twice
    assert vp.register() is False
    assert mods[vp.FUSED_MOE_MODULE].fused_experts is patched


def test_dispatch_and_fall_through(plugin, monkeypatch):
    vp, hip_calls = plugin
    mods, _, calls = _install_fake_vllm(monkeypatch)
    monkeypatch.setenv(vp.ENV_FLAG, "1")
    vp.register()
    fe = mods[vp.FUSED_MOE_MODULE].fused_experts
    x = _FakeCudaBf16()
    int8 = dict(use_int8_w8a8=True, per_channel_quant=True, w1_scale="s1", w2_scale="s2")
    # the int8 W8A8 call, with the other mode flags a flat-signature caller passes along
    assert fe(x, 1, 2, 3, 4, **int8, use_fp8_w8a8=False, use_int8_w8a16=False, w1_zp=None, allow_deep_gemm=False,
              global_num_experts=8) == "hip"
    assert hip_calls[-1] == dict(use_int8_w8a8=True, w1_scale="s1", global_num_experts=8)
    # everything else goes to the original, arguments untouched
    for other in (dict(use_fp8_w8a8=True), dict(expert_map="map"), dict(block_shape=[128, 128]),
                  dict(apply_router_weight_on_input=True), dict(activation="gelu"), dict(per_channel_quant=False),
                  dict(some_future_flag=True)):
        n = len(hip_calls)
        assert fe(x, 1, 2, 3, 4, **{**int8, **other}) == "original"
        assert len(hip_calls) == n and calls[-1][1] == {**int8, **other}
    assert fe(x, 1, 2, 3, 4, use_int8_w8a8=False) == "original"
    cpu = types.SimpleNamespace(is_cuda=False, dtype=torch.bfloat16)
    assert fe(cpu, 1, 2, 3, 4, **int8) == "original"
    fp16 = types.SimpleNamespace(is_cuda=True, dtype=torch.float16)
    assert fe(fp16, 1, 2, 3, 4, **int8) == "original"
    # positional extras (an older signature) are not guessed at
    assert fe(x, 1, 2, 3, 4, True, **int8) == "original"
    # a shape the library rejects falls through instead of failing the forward pass
    assert fe(x, 1, 2, 3, 4, **{**int8, "w1_scale": "unsupported-shape"}) == "original"


def test_tensor_valued_keywords_fall_through_without_being_evaluated(plugin, monkeypatch):
    """An expert map, a bias or zero points arrive as tensors: the dispatch decides on their presence and never
    asks for their truth value (ambiguous for more than one element, a device sync for one)."""
    vp, hip_calls = plugin
    mods, _, calls = _install_fake_vllm(monkeypatch)
    monkeypatch.setenv(vp.ENV_FLAG, "1")
    vp.register()
    fe = mods[vp.FUSED_MOE_MODULE].fused_experts
    x = _FakeCudaBf16()
    int8 = dict(use_int8_w8a8=True, per_channel_quant=True, w1_scale=torch.ones(8, 4), w2_scale=torch.ones(8, 4))

    class NoTruth(torch.Tensor):
        def __bool__(self):
            raise AssertionError("the dispatch evaluated a tensor")

        def __eq__(self, other):
            raise AssertionError("the dispatch compared a tensor")

        __hash__ = None

    for other in (dict(expert_map=torch.arange(8)), dict(w1_bias=torch.zeros(8, 4)), dict(w1_zp=torch.zeros(1)),
                  dict(some_future_tensor=torch.zeros(3)), dict(expert_map=torch.arange(8).as_subclass(NoTruth)),
                  dict(unknown=torch.zeros(2).as_subclass(NoTruth))):
        n = len(hip_calls)
        assert fe(x, 1, 2, 3, 4, **{**int8, **other}) == "original"
        assert len(hip_calls) == n
    # tensor-valued scales on the handled path are not evaluated either
    n = len(hip_calls)
    scales = dict(w1_scale=torch.ones(8, 4).as_subclass(NoTruth), w2_scale=torch.ones(8, 4).as_subclass(NoTruth))
    assert fe(x, 1, 2, 3, 4, **{**int8, **scales}, expert_map=None, w1_bias=None) == "hip"
    assert len(hip_calls) == n + 1


def test_rejected_shapes_fall_through_and_runtime_errors_do_not(plugin, monkeypatch):
    vp, hip_calls = plugin
    mods, _, calls = _install_fake_vllm(monkeypatch)
    monkeypatch.setenv(vp.ENV_FLAG, "1")
    vp.register()
    fe = mods[vp.FUSED_MOE_MODULE].fused_experts
    int8 = dict(use_int8_w8a8=True, per_channel_quant=True, w1_scale="s1", w2_scale="s2")

    def meta(*shape, dtype=torch.int8):
        return torch.empty(shape, dtype=dtype, device="meta")

    class X:
        is_cuda = True
        dtype = torch.bfloat16
        shape = (5, 128)

    ok = (X(), meta(4, 256, 128), meta(4, 128, 128))
    assert fe(*ok, 3, 4, **int8) == "hip"
    n = len(hip_calls)
    # decided from the shapes alone, before the HIP entry is called
    for w1, w2 in ((meta(4, 256, 96), meta(4, 96, 128)),       # hidden size not a multiple of 64 (and != x)
                   (meta(4, 200, 128), meta(4, 128, 100)),     # intermediate size not a multiple of 64
                   (meta(4, 256, 128), meta(4, 128, 64)),      # w2 does not match w1
                   (meta(2000, 256, 128), meta(2000, 128, 128))):  # more experts than the kernels index
        assert fe(X(), w1, w2, 3, 4, **int8) == "original"
    assert fe(*ok, 3, 4, **int8, global_num_experts=16) == "original"  # would need an expert map
    assert fe(*ok, 3, 4, **{**int8, "w1_scale": None}) == "original"
    assert len(hip_calls) == n
    # the entry's own validation may still reject: ValueError falls through like NotImplementedError
    assert fe(*ok, 3, 4, **{**int8, "w1_scale": "rejected-by-validation"}) == "original"
    # anything raised while the HIP path runs is a real failure and surfaces
    with pytest.raises(RuntimeError, match="launch"):
        fe(*ok, 3, 4, **{**int8, "w1_scale": "launch-failed"})


def test_apply_adapter_forwards_to_the_flat_entry(pra, monkeypatch):
    seen = {}

    def fake(hidden_states, w1, w2, topk_weights, topk_ids, **kw):
        seen.update(kw, hidden_states=hidden_states)
        return kw["out"]

    monkeypatch.setattr(pra.api, "fused_experts", fake)
    experts = pra.vllm_plugin.Int8W8A8HipExperts("s1", "s2", block_size_m=64)
    out = object()
    assert experts.apply(out, "x", "w1", "w2", "tw", "ids", activation="silu", global_num_experts=128,
                         expert_map=None, a1q_scale=None, a2_scale=None, workspace13="ws13", workspace2="ws2",
                         expert_tokens_meta=None, apply_router_weight_on_input=False) is out
    assert seen["use_int8_w8a8"] is True and seen["per_channel_quant"] is True and seen["out"] is out
    assert seen["w1_scale"] == "s1" and seen["w2_scale"] == "s2" and seen["global_num_experts"] == 128
    assert not experts.supports_expert_map()
    with pytest.raises(NotImplementedError, match="a1q_scale"):
        experts.apply(out, "x_q", "w1", "w2", "tw", "ids", a1q_scale="already quantised")


def test_default_workspace_cache_is_bounded(pra, monkeypatch):
    api = pra.api
    monkeypatch.setattr(api, "_workspaces", type(api._workspaces)())
    monkeypatch.setattr(api, "_pinned_workspaces", set())
    monkeypatch.setattr(api, "_retired_workspaces", [])
    made = []
    real_empty = torch.empty

    def fake_empty(shape, dtype=None, device=None):
        t = real_empty(shape, dtype=dtype)  # CPU stand-in
        made.append(t)
        return t

    monkeypatch.setattr(api.torch, "empty", fake_empty)
    dev = torch.device("cuda", 0)
    for stream in range(api._MAX_CACHED_WORKSPACES + 5):
        api._workspace(dev, stream, 1024)
    assert len(api._workspaces) == api._MAX_CACHED_WORKSPACES
    # the most recent streams stay; a hit does not allocate
    n = len(made)
    assert api._workspace(dev, api._MAX_CACHED_WORKSPACES + 4, 512) is made[-1]
    assert len(made) == n


def test_pinned_workspaces_are_never_freed(pra, monkeypatch):
    """A buffer handed out by reserve_workspace or under capture may sit in a captured graph: growing the
    cache entry retires it to a keep-alive list instead of dropping it, and eviction passes it over."""
    api = pra.api
    monkeypatch.setattr(api, "_workspaces", type(api._workspaces)())
    monkeypatch.setattr(api, "_pinned_workspaces", set())
    monkeypatch.setattr(api, "_retired_workspaces", [])
    real_empty = torch.empty
    monkeypatch.setattr(api.torch, "empty", lambda shape, dtype=None, device=None: real_empty(shape, dtype=dtype))
    capturing = [False]
    monkeypatch.setattr(api, "_capturing", lambda device: capturing[0])
    dev = torch.device("cuda", 0)
    reserved = api._workspace(dev, 7, 1000, pin=True)
    assert api._workspace(dev, 7, 800) is reserved
    grown = api._workspace(dev, 7, 5000)  # eager call above the reserved size
    assert grown is not reserved and grown.numel() >= 5000
    assert any(t is reserved for t in api._retired_workspaces)  # still allocated for graphs that hold it
    # a buffer first used under capture is pinned from then on
    plain = api._workspace(dev, 8, 1000)
    capturing[0] = True
    assert api._workspace(dev, 8, 900) is plain
    with pytest.raises(RuntimeError, match="reserve_workspace"):
        api._workspace(dev, 8, 2000)
    capturing[0] = False
    bigger = api._workspace(dev, 8, 2000)
    assert bigger is not plain and any(t is plain for t in api._retired_workspaces)
    # eviction only ever drops buffers no capture has seen
    pinned = api._workspace(dev, 9, 64, pin=True)
    for stream in range(100, 100 + 2 * api._MAX_CACHED_WORKSPACES):
        api._workspace(dev, stream, 64)
    assert api._workspaces[(0, 9)] is pinned
    assert len(api._workspaces) <= api._MAX_CACHED_WORKSPACES


def test_experts_selection_hook(pra, monkeypatch):
    """``register_experts_selection`` against a stand-in quantisation-method class: gated by the environment,
    idempotent, returns the HIP experts for an eligible layer and defers to the original for an expert map, static
    activation scales, another dtype, or a shape the kernels do not take."""
    vp = pra.vllm_plugin
    module_name, class_name = vp.MODULAR_METHODS[0]
    parts = module_name.split(".")
    for i in range(1, len(parts) + 1):
        name = ".".join(parts[:i])
        if name not in sys.modules:
            monkeypatch.setitem(sys.modules, name, types.ModuleType(name))

    class Method:
        static_input_scales = False

        def select_gemm_impl(self, prepare_finalize, layer):
            return "original experts"

    monkeypatch.setattr(sys.modules[module_name], class_name, Method, raising=False)

    def layer(**over):
        base = dict(w13_weight=torch.empty(4, 256, 128, dtype=torch.int8, device="meta"),
                    w2_weight=torch.empty(4, 128, 128, dtype=torch.int8, device="meta"),
                    w13_weight_scale="s13", w2_weight_scale="s2", expert_map=None, activation="silu")
        base.update(over)
        return types.SimpleNamespace(**base)

    monkeypatch.delenv(vp.ENV_FLAG, raising=False)
    assert vp.register_experts_selection() is False
    assert Method().select_gemm_impl(None, layer()) == "original experts"
    monkeypatch.setenv(vp.ENV_FLAG, "1")
    assert vp.register_experts_selection() is True
    assert vp.register_experts_selection() is False  # the marker: nothing is wrapped twice
    experts = Method().select_gemm_impl("prepare/finalize", layer())
    assert isinstance(experts, vp.Int8W8A8HipExperts) and experts.w1_scale == "s13" and experts.w2_scale == "s2"
    for other in (dict(expert_map=torch.arange(4)), dict(activation="gelu"), dict(w13_input_scale=torch.ones(1)),
                  dict(w13_weight=torch.empty(4, 256, 128, dtype=torch.float8_e4m3fn, device="meta")),
                  dict(w13_weight=torch.empty(4, 200, 128, dtype=torch.int8, device="meta")),
                  dict(w2_weight_scale=None)):
        assert Method().select_gemm_impl(None, layer(**other)) == "original experts", other
    static = Method()
    static.static_input_scales = True
    assert static.select_gemm_impl(None, layer()) == "original experts"
    # another quantisation method can be named through the environment
    other_mod = types.ModuleType("vllm_standin_quant")

    class Other(Method):
        pass

    Other.select_gemm_impl = lambda self, prepare_finalize, layer: "other original"
    other_mod.Other = Other
    monkeypatch.setitem(sys.modules, "vllm_standin_quant", other_mod)
    monkeypatch.setenv(vp.ENV_METHODS, "vllm_standin_quant:Other")
    assert vp.register_experts_selection() is True
    assert isinstance(Other().select_gemm_impl(None, layer()), vp.Int8W8A8HipExperts)
    assert Other().select_gemm_impl(None, layer(expert_map="map")) == "other original"
