"""Host-side checks that need no GPU: the C-ABI library loads, exports every symbol the header
declares, validates its arguments with error codes (no launch happens), and the Python wrappers
raise instead of falling back."""

import ctypes
import re
from pathlib import Path

import pytest
import torch

ROOT = Path(__file__).resolve().parent.parent


def _declared_symbols():
    text = (ROOT / "include" / "moe_i8.h").read_text()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(moe_i8_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol(pra):
    lib = pra._abi.load()
    declared = _declared_symbols()
    assert len(declared) >= 12
    assert sorted(pra._abi.SIGNATURES) == declared
    for name in declared:
        assert getattr(lib, name) is not None
    assert lib.moe_i8_version() >= 1


def test_capacity_and_workspace_formulas(pra):
    lib = pra._abi.load()
    assert lib.moe_i8_sorted_capacity(12, 5, 4) == 12 + 5 * 3
    assert lib.moe_i8_sorted_capacity(128, 128, 64) == 128 * 64  # fewer pairs than experts: P*B
    assert lib.moe_i8_sorted_capacity(65536, 128, 64) == 65536 + 128 * 63
    assert lib.moe_i8_sorted_capacity(0, 8, 64) == 0
    assert lib.moe_i8_align_workspace_bytes(1024, 128, 64) == 0
    big = lib.moe_i8_align_workspace_bytes(131072, 256, 64)
    assert big == 4 * (2 * 128 * 256 + 257)
    ws = lib.moe_i8_workspace_bytes(16, 8, 128, 2048, 768, 64)
    P = 128
    assert ws >= 16 * 2048 + P * 768 * 3 + P * 2048 * 2 and ws % 256 == 0
    assert lib.moe_i8_workspace_bytes(16, 8, 128, 2048, 768, 48) == -1


def test_c_abi_rejects_bad_arguments_without_launching(pra):
    abi = pra._abi
    lib = abi.load()
    buf = (ctypes.c_int32 * 1024)()
    p = ctypes.cast(buf, ctypes.c_void_p)
    err = lambda: lib.moe_i8_last_error().decode()
    # align: null outputs, bad block size, too many experts, capacity too small
    assert lib.moe_i8_align_block_size(p, 8, 4, 64, None, 260, p, 5, p, None, 0, None) == abi.EINVAL
    assert lib.moe_i8_align_block_size(p, 8, 4, 48, p, 260, p, 5, p, None, 0, None) == abi.EINVAL
    assert "block_size" in err()
    assert lib.moe_i8_align_block_size(p, 8, 2000, 64, p, 10**6, p, 10**5, p, None, 0, None) == abi.EINVAL
    assert lib.moe_i8_align_block_size(p, 8, 4, 64, p, 10, p, 5, p, None, 0, None) == abi.EWORKSPACE
    assert lib.moe_i8_align_block_size(p, 20000, 4, 64, p, 20000 + 4 * 63, p, 400, p, None, 0, None) == abi.EWORKSPACE
    assert "workspace" in err()
    # quant: dtype, cols, stride, alignment
    assert lib.moe_i8_quant_rows(p, 7, 4, 64, 64, None, 1, 4, p, p, None) == abi.EUNSUPPORTED
    assert lib.moe_i8_quant_rows(p, 0, 4, 60, 64, None, 1, 4, p, p, None) == abi.EINVAL
    assert lib.moe_i8_quant_rows(p, 0, 4, 64, 32, None, 1, 4, p, p, None) == abi.EINVAL
    assert lib.moe_i8_quant_rows(None, 0, 4, 64, 64, None, 1, 4, p, p, None) == abi.EINVAL
    assert lib.moe_i8_quant_rows(p, 0, 4, 64, 64, None, 1, 0, p, p, None) == abi.OK  # zero rows: no-op
    # router: expert / top-k limits, groups that do not tile, capture that does not fit
    rt = lambda E=128, k=8, score=0, G=1, KG=1, cap=None, cdt=0, stride=0, off=0: lib.moe_i8_route_topk(
        p, 4, E, k, score, None, G, KG, 0, 1, 1.0, p, p, cap, cdt, stride, off, None)
    assert rt(E=2000) == abi.EINVAL and rt(k=0) == abi.EINVAL and rt(k=65, E=128) == abi.EINVAL
    assert rt(score=5) == abi.EINVAL and rt(G=3) == abi.EINVAL
    assert rt(E=192, G=4, KG=1) == abi.EUNSUPPORTED  # 48-expert groups = 12 lanes of 4: not a power of two
    assert rt(G=8, KG=9) == abi.EINVAL and rt(G=8, KG=1, k=17) == abi.EINVAL
    assert rt(E=512, cap=p, cdt=1, stride=8) == abi.EINVAL and "uint8" in err()
    assert rt(cap=p, cdt=1, stride=8, off=1) == abi.EINVAL and rt(cap=None, cdt=2, stride=8) == abi.EINVAL
    # weight quant: dtype, cols, row groups that do not tile / do not fit
    assert lib.moe_i8_quant_weights(p, 7, 4, 64, 0, 0, 0, p, p, None) == abi.EUNSUPPORTED
    assert lib.moe_i8_quant_weights(p, 0, 4, 60, 0, 0, 0, p, p, None) == abi.EINVAL
    assert lib.moe_i8_quant_weights(p, 0, 4, 64, 3, 6, 0, p, p, None) == abi.EINVAL
    assert lib.moe_i8_quant_weights(p, 0, 4, 64, 2, 4, 3, p, p, None) == abi.EINVAL
    assert "row groups" in err()
    assert lib.moe_i8_quant_weights(p, 0, 4, 64, 2, 4, 2, None, p, None) == abi.EINVAL
    assert lib.moe_i8_quant_weights(p, 0, 0, 64, 0, 0, 0, p, p, None) == abi.OK
    # gemm: K not multiple of 64, N not multiple of 16, unknown variant, null
    base = dict(num_pairs=8, top_k=2, E=4, H=128, I=64, B=64, cap=8 + 4 * 63)
    call = lambda H=128, I=64, variant=0, x=p: lib.moe_i8_gemm_gate_up_silu(
        x, p, p, p, p, p, p, base["num_pairs"], 2, 4, H, I, 64, base["cap"], p, variant, None
    )
    assert call(H=96) == abi.EINVAL
    assert call(I=24) == abi.EINVAL
    assert call(variant=9) == abi.EINVAL
    # a family demanded for a shape it does not handle: refused before anything is launched
    assert call(H=128, variant=abi.GEMM_TILE) == abi.EUNSUPPORTED and "tile" in err()
    assert call(H=384, variant=abi.GEMM_NARROW) == abi.EUNSUPPORTED and "narrow" in err()
    assert call(x=None) == abi.EINVAL
    assert lib.moe_i8_gemm_down(p, p, p, p, p, p, p, p, 8, 4, 128, 100, 64, 260, p, 0, None) == abi.EINVAL
    assert lib.moe_i8_gemm_acc_i32(p, p, p, p, p, 8, 0, 4, 128, 128, 64, 260, p, 0, None) == abi.EINVAL
    # sum / fused driver
    assert lib.moe_i8_sum(p, p, 4, 0, 64, None) == abi.EINVAL
    assert lib.moe_i8_sum(p, p, 4, 2, 20, None) == abi.EINVAL
    assert lib.moe_i8_sum(None, None, 0, 2, 64, None) == abi.OK
    assert lib.moe_i8_fused_experts(p, p, p, p, p, p, p, p, 4, 2, 4, 128, 64, 64, None, 0, 0, None) == abi.EINVAL
    assert lib.moe_i8_fused_experts(p, p, p, p, p, p, p, p, 4, 2, 4, 100, 64, 64, p, 1 << 30, 0, None) == abi.EINVAL


def test_python_wrappers_refuse_cpu_tensors_and_unsupported_modes(pra):
    x = torch.zeros((4, 128), dtype=torch.bfloat16)
    w1 = torch.zeros((2, 128, 128), dtype=torch.int8)
    w2 = torch.zeros((2, 128, 64), dtype=torch.int8)
    tw = torch.ones((4, 1))
    ids = torch.zeros((4, 1), dtype=torch.int32)
    s1, s2 = torch.ones((2, 128)), torch.ones((2, 128))
    kw = dict(use_int8_w8a8=True, per_channel_quant=True, w1_scale=s1, w2_scale=s2)
    with pytest.raises(ValueError, match="GPU tensor"):
        pra.fused_experts(x, w1, w2, tw, ids, **kw)
    with pytest.raises(ValueError, match="GPU tensor"):
        pra.moe_align_block_size(ids, 64, 2)
    with pytest.raises(ValueError, match="GPU tensor"):
        pra.per_token_quant_int8(x)
    with pytest.raises(NotImplementedError):
        pra.fused_experts(x, w1, w2, tw, ids, w1_scale=s1, w2_scale=s2)  # not int8
    with pytest.raises(NotImplementedError):
        pra.fused_experts(x, w1, w2, tw, ids, **{**kw, "per_channel_quant": False})
    with pytest.raises(NotImplementedError):
        pra.fused_experts(x, w1, w2, tw, ids, activation="gelu", **kw)
    with pytest.raises(NotImplementedError):
        pra.fused_experts(x, w1, w2, tw, ids, expert_map=torch.zeros(2), **kw)
    with pytest.raises(NotImplementedError):
        pra.fused_experts(x, w1, w2, tw, ids, block_shape=[128, 128], **kw)
    with pytest.raises(NotImplementedError):
        pra.fused_experts(x, w1, w2, tw, ids, apply_router_weight_on_input=True, **kw)
    with pytest.raises(NotImplementedError):
        pra.moe_align_block_size(ids, 64, 2, expert_map=torch.zeros(2))


def test_widened_wrappers_refuse_cpu_tensors_and_unsupported_modes(pra):
    x = torch.zeros((4, 128), dtype=torch.bfloat16)
    logits = torch.zeros((4, 8))
    w = torch.zeros((8, 128), dtype=torch.int8)
    ws = torch.ones(8)
    for call in (
        lambda: pra.route_topk(logits, 2),
        lambda: pra.fused_topk(x, logits, 2, True),
        lambda: pra.grouped_topk(x, logits, 2, True, 2, 1),
        lambda: pra.quantize_weights_per_channel(x),
        lambda: pra.quantize_expert_weights(x.view(1, 4, 128), x.view(1, 4, 128), x.view(1, 128, 4)),
        lambda: pra.scaled_int8_quant(x),
        lambda: pra.apply_int8_linear(x, w, ws),
        lambda: pra.w8a8_mlp(x, w, ws, w, ws),
        lambda: pra.moe_sum(torch.zeros(4, 2, 128, dtype=torch.bfloat16), x),
    ):
        with pytest.raises(ValueError, match="GPU tensor"):
            call()
    with pytest.raises(ValueError, match="tokens mismatch"):
        pra.fused_topk(x[:2], logits, 2, True)
    with pytest.raises(ValueError, match="Unsupported scoring"):
        pra.grouped_topk(x, logits, 2, True, 2, 1, "tanh")
    with pytest.raises(NotImplementedError):
        pra.scaled_int8_quant(x, scale=torch.ones(1))
    with pytest.raises(NotImplementedError):
        pra.apply_int8_linear(x, w, ws, input_scale=torch.ones(1))
    with pytest.raises(NotImplementedError):
        pra.fused_moe(x, w, w, logits, 2, True, custom_routing_function=lambda *a: None)
    with pytest.raises(ValueError, match="record must be"):
        pra.routed_experts_payload(torch.zeros(4, 2, dtype=torch.uint8))
    # the wire form of a record needs no GPU: field for field the reference's dictionary
    rec = torch.tensor([[[1, 2, 3]]], dtype=torch.uint8)
    assert pra.routed_experts_payload(rec) == {"data": "AQID", "shape": [1, 1, 3], "start": 0, "dtype": "uint8"}


def test_fused_experts_signature_is_vllms(pra):
    import inspect

    params = list(inspect.signature(pra.fused_experts).parameters)
    assert params[:5] == ["hidden_states", "w1", "w2", "topk_weights", "topk_ids"]
    for name in ("inplace", "activation", "apply_router_weight_on_input", "use_int8_w8a8", "per_channel_quant",
                 "global_num_experts", "expert_map", "w1_scale", "w2_scale", "a1_scale", "a2_scale", "block_shape"):
        assert name in params
    assert list(inspect.signature(pra.moe_align_block_size).parameters) == [
        "topk_ids", "block_size", "num_experts", "expert_map", "pad_sorted_ids"]
    assert list(inspect.signature(pra.moe_sum).parameters) == ["input", "output"]


def test_vllm_plugin_is_noop_without_vllm(pra, monkeypatch):
    monkeypatch.setenv(pra.vllm_plugin.ENV_FLAG, "1")
    assert pra.vllm_plugin.register() is False
    monkeypatch.setenv(pra.vllm_plugin.ENV_FLAG, "0")
    assert pra.vllm_plugin.register() is False


def test_missing_library_fails_loudly(pra, monkeypatch, tmp_path):
    monkeypatch.setattr(pra._abi, "_lib", None)
    monkeypatch.setattr(pra._abi, "LIB_PATH", tmp_path / "libmoe_i8.so")
    with pytest.raises(ImportError, match="no CPU or PyTorch fallback"):
        pra._abi.load()


def test_header_is_plain_c_and_a_c_client_links(pra, tmp_path):
    """include/moe_i8.h compiles as C99 and a C program linked against the library gets the documented
    sizes and argument errors (no GPU needed for any of these calls)."""
    import shutil
    import subprocess

    gcc = shutil.which("gcc")
    if gcc is None:
        pytest.skip("no gcc")
    root = ROOT
    lib = pra._abi.LIB_PATH
    exe = tmp_path / "abi_check"
    cmd = [gcc, "-std=c99", "-Wall", "-Werror", "-pedantic", "-I", str(root / "include"),
           str(root / "tests" / "c" / "abi_check.c"), "-o", str(exe), str(lib), f"-Wl,-rpath,{lib.parent}",
           "-Wl,-rpath,/opt/rocm/lib"]
    subprocess.run(cmd, check=True, capture_output=True, text=True)
    run = subprocess.run([str(exe)], capture_output=True, text=True, timeout=120)
    assert run.returncode == 0 and run.stdout.strip() == "ok", run.stdout + run.stderr


# Which kernel the library picks by itself at every benchmark point (shape, tokens) and how many launches a
# layer call makes there.  These are the kernels the committed measurements were taken on: a retune of the
# hand-over points between the GEMM families must change this table knowingly.
_PLAN = [
    ("toy", 256, "tile_deep", "tile_deep", 5),
    ("qwen3-30b-a3b", 1, "stream", "stream", 4),
    ("qwen3-30b-a3b", 16, "stream", "stream", 4),
    ("qwen3-30b-a3b", 17, "narrow", "narrow", 5),   # more than 16 tokens: a block may need a second streaming pass
    ("qwen3-30b-a3b", 128, "narrow", "narrow", 5),
    ("qwen3-30b-a3b", 256, "narrow", "narrow", 5),
    ("qwen3-30b-a3b", 512, "narrow", "narrow", 5),
    ("qwen3-30b-a3b", 640, "narrow", "narrow", 5),
    ("qwen3-30b-a3b", 704, "tile_deep", "tile_deep", 5),
    ("qwen3-30b-a3b", 1024, "tile_deep", "tile_deep", 5),
    ("qwen3-30b-a3b", 8192, "tile_wide", "tile_wide", 7),
    ("glm-4.5-air", 16, "stream", "stream", 5),
    ("glm-4.5-air", 32, "narrow", "narrow", 5),     # the shared expert holds every token: 32 rows in one block
    ("glm-4.5-air", 512, "tile_deep", "tile_deep", 5),
    ("glm-4.5-air", 4096, "tile_wide", "tile_wide", 7),
    ("deepseek-v3", 8, "stream", "stream", 5),
    ("deepseek-v3", 64, "narrow", "narrow", 5),
    ("deepseek-v3", 2048, "tile_deep", "tile_deep", 6),
    ("deepseek-v3", 16384, "tile_wide", "tile_wide", 7),
]


@pytest.mark.parametrize("shape_name,M,gate_up,down,launches", _PLAN)
def test_kernel_choice_at_the_benchmark_points(pra, shape_name, M, gate_up, down, launches):
    shape = pra.inputs.SHAPES[shape_name]
    k = shape.k + (1 if shape.shared_expert else 0)
    plan = pra.layer_plan(M, k, shape.E_total, shape.H, shape.I)
    assert plan == {"gate_up": gate_up, "down": down, "launches": launches}


def test_layer_plan_follows_a_demanded_family_and_rejects_what_it_cannot_run(pra):
    abi = pra._abi
    assert pra.layer_plan(8192, 8, 128, 2048, 768, gemm_variant="stream") == {
        "gate_up": "stream", "down": "stream", "launches": 7}
    assert pra.layer_plan(1024, 8, 128, 2048, 768, gemm_variant="tile_wide")["gate_up"] == "tile_wide"
    assert pra.layer_plan(1024, 8, 128, 2048, 768, gemm_variant="tile")["gate_up"] == "tile_deep"
    # the ring pipeline runs only where it is demanded
    assert pra.layer_plan(8192, 8, 128, 2048, 768, gemm_variant="tile_ring") == {
        "gate_up": "tile_ring", "down": "tile_ring", "launches": 7}
    with pytest.raises(abi.MoeI8Error) as e:  # the tiled families take blocks of 64 or 128 rows only
        pra.layer_plan(1024, 8, 128, 2048, 768, block_size=16, gemm_variant="tile_wide")
    assert e.value.code == abi.EUNSUPPORTED
    with pytest.raises(abi.MoeI8Error):
        pra.layer_plan(0, 8, 128, 2048, 768)
    with pytest.raises(abi.MoeI8Error):
        pra.layer_plan(16, 8, 128, 2048, 700)
    # output pointers are optional
    assert abi.load().moe_i8_layer_plan(16, 8, 128, 2048, 768, 64, abi.GEMM_AUTO, None, None, None) == abi.OK
