"""Host side of the gfx950 INT8 W8A8 fused-MoE path, with vLLM's call signatures.

``fused_experts`` keeps the flat signature of vLLM 0.28.0's
``vllm.model_executor.layers.fused_moe.fused_experts`` (the function the reference's rollout
engine reaches through the ``quantization`` pass-through,
``packages/prime-rl-configs/src/prime_rl/configs/inference.py:108-109``), and
``moe_align_block_size`` / ``per_token_quant_int8`` / ``moe_sum`` keep the names and returns of the
pieces it is made of.  Everything runs in hand-written HIP kernels behind the C-ABI of
``libmoe_i8.so``; torch only supplies device memory and the current stream.  There is no CPU or
eager fallback: without the built library, or off a GPU, these functions raise.
"""

from __future__ import annotations

import threading
from collections import OrderedDict

import torch

from . import _abi

__all__ = [
    "fused_experts",
    "fused_moe",
    "moe_align_block_size",
    "per_token_quant_int8",
    "quantize_weights_per_channel",
    "quantize_expert_weights",
    "load_quantized_expert_weights",
    "moe_sum",
    "fused_topk",
    "grouped_topk",
    "route_topk",
    "routed_experts_payload",
    "scaled_int8_quant",
    "apply_int8_linear",
    "w8a8_mlp",
    "gemm_gate_up_silu",
    "gemm_down",
    "gemm_down_bf16",
    "gemm_acc_i32",
    "workspace_bytes",
    "reserve_workspace",
    "sorted_capacity",
    "DEFAULT_BLOCK_SIZE_M",
]

DEFAULT_BLOCK_SIZE_M = 64
_VARIANTS = {
    "auto": _abi.GEMM_AUTO, "stream": _abi.GEMM_STREAM, "tile": _abi.GEMM_TILE, "narrow": _abi.GEMM_NARROW,
    "tile_wide": _abi.GEMM_TILE_WIDE, "tile_deep": _abi.GEMM_TILE_DEEP, "tile_ring": _abi.GEMM_TILE_RING,
}
# Default workspaces, one per (device, stream) that has called without a caller-owned one: a small
# LRU (a process has a handful of forward streams) guarded by a lock.  Entries are only ever created or
# grown outside HIP graph capture (a capture that finds no entry large enough raises instead of
# allocating), and an entry that a capture used or reserve_workspace made is never freed: when it is
# outgrown it is retired to a keep-alive list, and eviction skips it.
_MAX_CACHED_WORKSPACES = 16
_workspaces: "OrderedDict[tuple[int, int], torch.Tensor]" = OrderedDict()
_pinned_workspaces: "set[tuple[int, int]]" = set()  # keys whose buffer a capture or reserve_workspace handed out
_retired_workspaces: "list[torch.Tensor]" = []      # outgrown pinned buffers, kept allocated
_workspaces_lock = threading.Lock()


def _ptr(t: torch.Tensor | None) -> int | None:
    return None if t is None else t.data_ptr()


def _stream(t: torch.Tensor) -> int:
    return torch.cuda.current_stream(t.device).cuda_stream


def _require_gpu(name: str, t: torch.Tensor) -> None:
    if not isinstance(t, torch.Tensor):
        raise TypeError(f"{name} must be a torch.Tensor")
    if not t.is_cuda:
        raise ValueError(f"{name} must be a GPU tensor (this path has no CPU implementation)")
    if not t.is_contiguous():
        raise ValueError(f"{name} must be contiguous")


def _variant(v: str | int) -> int:
    if isinstance(v, int):
        return v
    try:
        return _VARIANTS[v]
    except KeyError:
        raise ValueError(f"gemm variant must be one of {sorted(_VARIANTS)}") from None


def _block_size(block_size: int) -> int:
    if block_size not in (16, 32, 64, 128):
        raise ValueError("block_size must be 16, 32, 64 or 128")
    return int(block_size)


def _as_i32_ids(topk_ids: torch.Tensor) -> torch.Tensor:
    if topk_ids.dtype == torch.int32:
        return topk_ids
    if topk_ids.dtype in (torch.int64, torch.int16, torch.uint8):
        return topk_ids.to(torch.int32)
    raise ValueError(f"topk_ids must be an integer tensor, got {topk_ids.dtype}")


def sorted_capacity(num_pairs: int, num_experts: int, block_size: int) -> int:
    """Length of ``sorted_token_ids``: ``min(P + E*(B-1), P*B)`` as upstream sizes it."""
    return int(_abi.load().moe_i8_sorted_capacity(num_pairs, num_experts, block_size))


def workspace_bytes(m: int, top_k: int, num_experts: int, hidden: int, inter: int, block_size: int) -> int:
    n = int(_abi.load().moe_i8_workspace_bytes(m, top_k, num_experts, hidden, inter, block_size))
    if n < 0:
        raise ValueError("invalid shape for workspace_bytes")
    return n


_KERNEL_NAMES = {_abi.GEMM_STREAM: "stream", _abi.GEMM_NARROW: "narrow", _abi.GEMM_TILE_WIDE: "tile_wide",
                 _abi.GEMM_TILE_DEEP: "tile_deep", _abi.GEMM_TILE_RING: "tile_ring"}


def layer_plan(m: int, top_k: int, num_experts: int, hidden: int, inter: int,
               block_size: int = 64, gemm_variant: str | int = "auto") -> dict:
    """Which GEMM kernel ``fused_experts`` runs for each projection of a layer of this shape and how many
    kernel launches one call makes: ``{"gate_up": name, "down": name, "launches": n}``.  Decided on the host
    from the sizes alone (no GPU needed), by the same code the driver uses."""
    import ctypes

    gu, dn, n = ctypes.c_int(), ctypes.c_int(), ctypes.c_int()
    _abi.check(_abi.load().moe_i8_layer_plan(m, top_k, num_experts, hidden, inter, block_size, _variant(gemm_variant),
                                             ctypes.byref(gu), ctypes.byref(dn), ctypes.byref(n)))
    return {"gate_up": _KERNEL_NAMES[gu.value], "down": _KERNEL_NAMES[dn.value], "launches": n.value}


# --------------------------------------------------------------------------------------------- #
def moe_align_block_size(
    topk_ids: torch.Tensor,
    block_size: int,
    num_experts: int,
    expert_map: torch.Tensor | None = None,
    pad_sorted_ids: bool = False,
) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """vLLM ``moe_align_block_size``: returns ``(sorted_token_ids, expert_ids, num_tokens_post_padded)``.

    ``sorted_token_ids`` holds flat pair indices ``m*k + j`` grouped by expert in ascending order
    (the reference's stable sort, ``trainer/distributed/token_dispatcher.py:145``), each expert
    padded to a multiple of ``block_size`` with the sentinel ``topk_ids.numel()``; the unused tail
    is all sentinel and unused ``expert_ids`` are ``-1``.
    """
    if expert_map is not None:
        raise NotImplementedError("expert_map (expert parallelism) is not supported on this path")
    _require_gpu("topk_ids", topk_ids)
    block_size = _block_size(block_size)
    if not 1 <= num_experts <= _abi.MAX_EXPERTS:
        raise ValueError(f"num_experts must be in [1, {_abi.MAX_EXPERTS}]")
    lib = _abi.load()
    ids = _as_i32_ids(topk_ids)
    P = ids.numel()
    cap = sorted_capacity(P, num_experts, block_size)
    if pad_sorted_ids:
        cap = (cap + block_size - 1) // block_size * block_size
    dev = ids.device
    sorted_ids = torch.empty((cap,), dtype=torch.int32, device=dev)
    expert_ids = torch.empty(((cap + block_size - 1) // block_size,), dtype=torch.int32, device=dev)
    npp = torch.empty((1,), dtype=torch.int32, device=dev)
    ws_bytes = int(lib.moe_i8_align_workspace_bytes(P, num_experts, block_size))
    ws = torch.empty((max(ws_bytes, 1),), dtype=torch.uint8, device=dev)
    _abi.check(
        lib.moe_i8_align_block_size(
            _ptr(ids), P, num_experts, block_size, _ptr(sorted_ids), cap, _ptr(expert_ids),
            expert_ids.numel(), _ptr(npp), _ptr(ws), ws_bytes, _stream(ids),
        )
    )
    return sorted_ids, expert_ids, npp


def per_token_quant_int8(x: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
    """vLLM ``per_token_quant_int8``: ``(x_q int8 like x, scales fp32 [..., 1])``, fp32 arithmetic,
    ``scale = max(absmax, 1e-10) / 127``, rounding half away from zero."""
    _require_gpu("x", x)
    if x.dtype != torch.bfloat16:
        raise NotImplementedError(f"only bfloat16 activations are supported, got {x.dtype}")
    cols = x.shape[-1]
    if cols % 8 or cols == 0:
        raise ValueError("last dimension must be a positive multiple of 8")
    rows = x.numel() // cols
    q = torch.empty(x.shape, dtype=torch.int8, device=x.device)
    scale = torch.empty((*x.shape[:-1], 1), dtype=torch.float32, device=x.device)
    _abi.check(
        _abi.load().moe_i8_quant_rows(
            _ptr(x), _abi.DTYPE_BF16, rows, cols, cols, None, 1, rows, _ptr(q), _ptr(scale), _stream(x)
        )
    )
    return q, scale


def _quant_weights_into(w, q, scale, rows_per_group=0, out_rows_per_group=0, out_row_offset=0) -> None:
    cols = w.shape[-1]
    rows = w.numel() // cols if cols else 0
    _abi.check(
        _abi.load().moe_i8_quant_weights(
            _ptr(w), _abi.DTYPE_BF16, rows, cols, rows_per_group, out_rows_per_group, out_row_offset,
            _ptr(q), _ptr(scale), _stream(w),
        )
    )


def _check_bf16_weight(name: str, w: torch.Tensor, ndim_min: int = 2) -> None:
    _require_gpu(name, w)
    if w.dtype != torch.bfloat16:
        raise NotImplementedError(f"only bfloat16 weights are supported, got {w.dtype} for {name}")
    if w.dim() < ndim_min:
        raise ValueError(f"{name} must have at least {ndim_min} dimensions")
    if w.shape[-1] == 0 or w.shape[-1] % 8:
        raise ValueError(f"last dimension of {name} must be a positive multiple of 8")


def quantize_weights_per_channel(
    w: torch.Tensor, out: tuple[torch.Tensor, torch.Tensor] | None = None
) -> tuple[torch.Tensor, torch.Tensor]:
    """Symmetric per-output-channel int8 quantisation of bf16 ``w [..., N, K]``: the reference's
    blockwise weight quantiser (``src/prime_rl/trainer/models/fp8.py:33-36``) with one whole row as
    the block and ``qmax = 127`` — ``scale = max(absmax / 127, 1e-12)``, ``q = rint(w / scale)``
    clamped to ±127.  Returns ``(q int8 like w, scale fp32 [..., N])``; with ``out=(q, scale)`` the
    result is written into those tensors (an in-place update of engine parameters, as
    ``src/prime_rl/inference/vllm/worker/weight_transfer.py:97-134`` does with ``param.copy_``)."""
    _check_bf16_weight("w", w)
    if out is None:
        q = torch.empty(w.shape, dtype=torch.int8, device=w.device)
        scale = torch.empty(w.shape[:-1], dtype=torch.float32, device=w.device)
    else:
        q, scale = out
        _require_gpu("out[0]", q)
        _require_gpu("out[1]", scale)
        if q.dtype != torch.int8 or q.shape != w.shape:
            raise ValueError("out[0] must be int8 with the shape of w")
        if scale.dtype != torch.float32 or scale.numel() != w.numel() // w.shape[-1]:
            raise ValueError("out[1] must be fp32 with one element per row of w")
    _quant_weights_into(w, q, scale)
    return q, scale


def quantize_expert_weights(
    gate_proj: torch.Tensor,
    up_proj: torch.Tensor,
    down_proj: torch.Tensor,
    out: tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor] | None = None,
) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    """Trainer expert weights → the int8 kernel layout ``fused_experts`` reads, in three launches and
    with no concatenated bf16 intermediate.

    ``gate_proj, up_proj`` bf16 ``[E, I, H]`` and ``down_proj`` bf16 ``[E, H, I]`` (``w1, w3, w2`` of
    ``src/prime_rl/trainer/models/glm_moe_dsa/converting_glm_moe_dsa.py:97-125``) → ``w13 int8
    [E, 2I, H]`` (gate rows first, as ``torch.cat([w1, w3], dim=1)`` there), ``w13_scale fp32
    [E, 2I]``, ``w2 int8 [E, H, I]``, ``w2_scale fp32 [E, H]``.  ``out=(w13, w13_scale, w2,
    w2_scale)`` overwrites the parameters of a running engine in place.
    """
    _check_bf16_weight("gate_proj", gate_proj, 3)
    _check_bf16_weight("up_proj", up_proj, 3)
    _check_bf16_weight("down_proj", down_proj, 3)
    if gate_proj.dim() != 3 or gate_proj.shape != up_proj.shape:
        raise ValueError("gate_proj and up_proj must both be [E, I, H]")
    E, I, H = gate_proj.shape
    if down_proj.shape != (E, H, I):
        raise ValueError(f"down_proj must be [E, H, I] = {(E, H, I)}, got {tuple(down_proj.shape)}")
    dev = gate_proj.device
    if out is None:
        w13 = torch.empty((E, 2 * I, H), dtype=torch.int8, device=dev)
        s13 = torch.empty((E, 2 * I), dtype=torch.float32, device=dev)
        w2 = torch.empty((E, H, I), dtype=torch.int8, device=dev)
        s2 = torch.empty((E, H), dtype=torch.float32, device=dev)
    else:
        w13, s13, w2, s2 = out
        for name, t, dtype, numel in (
            ("w13", w13, torch.int8, E * 2 * I * H),
            ("w13_scale", s13, torch.float32, E * 2 * I),
            ("w2", w2, torch.int8, E * H * I),
            ("w2_scale", s2, torch.float32, E * H),
        ):
            _require_gpu(name, t)
            if t.dtype != dtype or t.numel() != numel:
                raise ValueError(f"out tensor {name} must be {dtype} with {numel} elements")
        if w13.shape != (E, 2 * I, H) or w2.shape != (E, H, I):
            raise ValueError("out weights must be w13 [E, 2I, H] and w2 [E, H, I]")
    _quant_weights_into(gate_proj, w13, s13, I, 2 * I, 0)
    _quant_weights_into(up_proj, w13, s13, I, 2 * I, I)
    _quant_weights_into(down_proj, w2, s2)
    return w13, s13, w2, s2


_EXPERT_PARAM_SUFFIXES = ("w13_weight", "w13_weight_scale", "w2_weight", "w2_weight_scale")


def _resolve_expert_params(params: dict, prefix: str, E: int, I: int, H: int):
    """The four int8 parameters of the layer ``prefix`` as ``(names, views, missing, mismatches)``: looked up
    as ``{prefix}.{name}`` or, as the pinned vLLM nests them, ``{prefix}.routed_experts.{name}``
    (``src/prime_rl/inference/vllm/worker/weight_transfer.py:76-82``); ``views`` are the parameters' tensors
    in the shapes the quantiser writes (scales may be kept as ``[E, N]`` or ``[E, N, 1]``)."""
    want = {"w13_weight": (E, 2 * I, H), "w13_weight_scale": (E, 2 * I), "w2_weight": (E, H, I),
            "w2_weight_scale": (E, H)}
    names, views, missing, mismatches = {}, {}, [], []
    for suffix in _EXPERT_PARAM_SUFFIXES:
        for name in (f"{prefix}.{suffix}", f"{prefix}.routed_experts.{suffix}"):
            if name in params:
                break
        else:
            missing.append(f"{prefix}.{suffix}")
            continue
        param = params[name]
        t = param.data if isinstance(param, torch.nn.Parameter) else param
        shape = tuple(t.shape)
        if shape == want[suffix]:
            views[suffix] = t
        elif suffix.endswith("_scale") and shape == want[suffix] + (1,):
            views[suffix] = t.view(want[suffix])
        else:
            mismatches.append(f"{name}: param={list(shape)} != received={list(want[suffix])}")
            continue
        names[suffix] = name
    return names, views, missing, mismatches


@torch.no_grad()
def load_quantized_expert_weights(
    params: dict,
    prefix: str,
    w1: torch.Tensor,
    w3: torch.Tensor,
    w2: torch.Tensor,
    source_indices: torch.Tensor | None = None,
) -> list[str]:
    """Policy update of one int8 W8A8 MoE layer of a running engine: quantise the trainer's bf16
    ``w1`` (gate) ``[E, I, H]``, ``w3`` (up) ``[E, I, H]`` and ``w2`` (down) ``[E, H, I]`` and write
    ``w13_weight``, ``w13_weight_scale``, ``w2_weight``, ``w2_weight_scale`` of that layer in place, so
    the addresses the engine (and any captured graph) holds stay valid.

    The int8 counterpart of the reference's kernel-format weight transfer
    (``src/prime_rl/inference/vllm/worker/weight_transfer.py:97-134``): ``params`` is
    ``dict(model.named_parameters())``; the four tensors are looked up as ``{prefix}.{name}`` or, as the
    pinned vLLM nests them, ``{prefix}.routed_experts.{name}`` (``weight_transfer.py:76-82``); a missing
    name or a shape that does not match raises ``ValueError`` naming it, as the reference does, before
    anything is written; ``source_indices`` selects the experts local to this worker from the trainer's
    tensors the way ``tensor[source_indices]`` does there (``:120-125``).  Scales may be ``[E, N]`` or
    ``[E, N, 1]``.  Returns the names written.
    """
    if source_indices is not None:
        idx = source_indices.to(device=w1.device, dtype=torch.long)
        w1, w3, w2 = w1[idx].contiguous(), w3[idx].contiguous(), w2[idx].contiguous()
    if w1.dim() != 3 or w1.shape != w3.shape or w2.dim() != 3:
        raise ValueError("w1 and w3 must be [E, I, H] and w2 [E, H, I]")
    E, I, H = w1.shape
    names, views, missing, mismatches = _resolve_expert_params(params, prefix, E, I, H)
    if missing:
        raise ValueError(f"int8 expert weight update: {len(missing)} parameters not found in model: {missing}")
    if tuple(w2.shape) != (E, H, I):
        mismatches.append(f"{names.get('w2_weight', prefix + '.w2_weight')}: param={[E, H, I]} != received={list(w2.shape)}")
    if mismatches:
        raise ValueError(f"int8 expert weight update had {len(mismatches)} shape mismatches: {mismatches}")
    quantize_expert_weights(
        w1, w3, w2, out=(views["w13_weight"], views["w13_weight_scale"], views["w2_weight"], views["w2_weight_scale"])
    )
    return [names[suffix] for suffix in _EXPERT_PARAM_SUFFIXES]


# incoming names of routed-expert weights -> (role, layer prefix).  Trainer format
# (``src/prime_rl/trainer/models/glm_moe_dsa/converting_glm_moe_dsa.py:97-99``): ``...experts.gate_proj``,
# ``...experts.up_proj``, ``...experts.down_proj``; kernel format with bf16 payload (``:123-125``):
# ``...experts.w13_weight`` (gate rows, then up rows) and ``...experts.w2_weight``.
_EXPERT_ROLE_SUFFIXES = (
    (".experts.gate_proj", "w1"), (".experts.up_proj", "w3"), (".experts.down_proj", "w2"),
    (".experts.routed_experts.w13_weight", "w13"), (".experts.routed_experts.w2_weight", "w2"),
    (".experts.w13_weight", "w13"), (".experts.w2_weight", "w2"),
)


def _expert_role(name: str):
    for suffix, role in _EXPERT_ROLE_SUFFIXES:
        if name.endswith(suffix):
            return role, name[: len(name) - len(suffix)] + ".experts"
    return None, None


@torch.no_grad()
def load_weights_kernel_int8(model, state_iter, expert_source_indices: dict | None = None) -> dict:
    """Policy update of a whole int8 W8A8 model from the trainer's ``(name, tensor)`` stream: the int8
    counterpart of the reference's ``load_weights_kernel``
    (``src/prime_rl/inference/vllm/worker/weight_transfer.py:97-134``).

    ``model`` is the engine's module (its ``named_parameters()`` are used) or such a dict.  bf16
    routed-expert weights are collected per layer — ``w1``/``w3``/``w2`` under the trainer's names, or
    ``w13_weight``/``w2_weight`` in kernel format — and, once a layer is complete, quantised per output
    channel and written in place into that layer's ``w13_weight``, ``w13_weight_scale``, ``w2_weight``,
    ``w2_weight_scale`` (flat or nested under ``routed_experts``).  Every other tensor is copied in place
    into the parameter of the same name (tried flat, then with the ``routed_experts`` nesting), exactly as
    the reference does; that includes weights that arrive already quantised.  ``expert_source_indices``
    maps a module-name prefix to the experts local to this worker (``weight_transfer.py:76-95,120-125``).

    Nothing raises midway: names that are not in the model, tensors whose shapes do not match and expert
    groups that never became complete are collected, everything else is written, and ONE ``ValueError``
    at the end lists them all (mismatches first, as the reference orders its two errors).  Returns
    ``{"loaded": [...names written...], "quantized_layers": [...prefixes...]}``.
    """
    params = dict(model.named_parameters()) if hasattr(model, "named_parameters") else dict(model)
    expert_source_indices = expert_source_indices or {}
    loaded, layers, skipped, mismatches = [], [], [], []
    pending: dict[str, dict[str, tuple[str, torch.Tensor]]] = {}

    def local_experts(prefix: str, t: torch.Tensor) -> torch.Tensor:
        for module_name, idx in expert_source_indices.items():
            if prefix.startswith(f"{module_name}.") or prefix == module_name:
                return t[idx.to(device=t.device, dtype=torch.long)].contiguous()
        return t

    def flush(prefix: str, group: dict) -> None:
        w2 = local_experts(prefix, group["w2"][1])
        if "w13" in group:
            w13 = local_experts(prefix, group["w13"][1])
            if w13.dim() != 3 or w13.shape[1] % 2 or w2.dim() != 3:
                mismatches.append(f"{group['w13'][0]}: received={list(w13.shape)} is not [E, 2I, H]")
                return
            E, I, H = w13.shape[0], w13.shape[1] // 2, w13.shape[2]
        else:
            w1, w3 = local_experts(prefix, group["w1"][1]), local_experts(prefix, group["w3"][1])
            if w1.dim() != 3 or w1.shape != w3.shape or w2.dim() != 3:
                mismatches.append(f"{group['w1'][0]}: received={list(w1.shape)} / {list(w3.shape)} are not two [E, I, H]")
                return
            E, I, H = w1.shape
        names, views, missing, bad = _resolve_expert_params(params, prefix, E, I, H)
        if tuple(w2.shape) != (E, H, I):
            bad.append(f"{group['w2'][0]}: param={[E, H, I]} != received={list(w2.shape)}")
        if missing or bad:
            skipped.extend(missing)
            mismatches.extend(bad)
            return
        out = (views["w13_weight"], views["w13_weight_scale"], views["w2_weight"], views["w2_weight_scale"])
        if "w13" in group:
            quantize_weights_per_channel(w13.contiguous(), out=out[:2])
            quantize_weights_per_channel(w2.contiguous(), out=out[2:])
        else:
            quantize_expert_weights(w1.contiguous(), w3.contiguous(), w2.contiguous(), out=out)
        loaded.extend(names[suffix] for suffix in _EXPERT_PARAM_SUFFIXES)
        layers.append(prefix)

    for name, tensor in state_iter:
        role, prefix = _expert_role(name)
        if role is not None and tensor.dtype == torch.bfloat16:
            group = pending.setdefault(prefix, {})
            group[role] = (name, tensor)
            if "w2" in group and ("w13" in group or ("w1" in group and "w3" in group)):
                flush(prefix, pending.pop(prefix))
            continue
        target = name
        if target not in params and ".experts." in name and ".routed_experts." not in name:
            head, _, tail = name.rpartition(".experts.")
            target = f"{head}.experts.routed_experts.{tail}"
        if target not in params:
            skipped.append(name)
            continue
        param = params[target]
        if tuple(param.shape) != tuple(tensor.shape):
            prefix_of = target.rpartition(".")[0]
            tensor = local_experts(prefix_of, tensor) if expert_source_indices else tensor
            if tuple(param.shape) != tuple(tensor.shape):
                mismatches.append(f"{target}: param={list(param.shape)} != received={list(tensor.shape)}")
                continue
        param.copy_(tensor)
        loaded.append(target)
    for prefix, group in pending.items():
        skipped.extend(f"{n} (incomplete expert group of {prefix}: got {sorted(group)})" for n, _ in group.values())
    if mismatches or skipped:
        parts = []
        if mismatches:
            parts.append(f"{len(mismatches)} shape mismatches: {mismatches}")
        if skipped:
            parts.append(f"skipped {len(skipped)} weights not found in model: {skipped}")
        raise ValueError("int8 kernel weight transfer had " + "; ".join(parts))
    return {"loaded": loaded, "quantized_layers": layers}


def moe_sum(input: torch.Tensor, output: torch.Tensor) -> None:
    """vLLM ``ops.moe_sum``: ``output[m] = sum_j input[m, j]`` for bf16 ``[M, k, H]`` → ``[M, H]``."""
    _require_gpu("input", input)
    _require_gpu("output", output)
    if input.dtype != torch.bfloat16 or output.dtype != torch.bfloat16:
        raise NotImplementedError("only bfloat16 is supported")
    if input.dim() != 3 or output.shape != (input.shape[0], input.shape[2]):
        raise ValueError("expected input [M, k, H] and output [M, H]")
    M, k, H = input.shape
    if H % 8:
        raise ValueError("hidden size must be a multiple of 8")
    _abi.check(_abi.load().moe_i8_sum(_ptr(input), _ptr(output), M, k, H, _stream(input)))


# --------------------------------------------------------------------------------------------- #
_SCORE_FUNCS = {
    "softmax": _abi.SCORE_SOFTMAX,
    "sigmoid": _abi.SCORE_SIGMOID,
    "topk_softmax": _abi.SCORE_TOPK_SOFTMAX,
}


def route_topk(
    gating_output: torch.Tensor,
    topk: int,
    *,
    score_func: str = "softmax",
    renormalize: bool = True,
    route_scale: float = 1.0,
    selection_bias: torch.Tensor | None = None,
    num_expert_group: int = 1,
    topk_group: int = 1,
    group_score_top2: bool = False,
    routed_experts_out: tuple[torch.Tensor, int] | None = None,
) -> tuple[torch.Tensor, torch.Tensor]:
    """The reference router after its gate GEMM (``TokenChoiceTopKRouter.forward``,
    ``src/prime_rl/trainer/models/layers/moe.py:261-307``) in one launch: fp32 scores
    (``score_func`` ∈ softmax / sigmoid / topk_softmax), a bias that only steers the selection,
    optional group pre-selection, top-k in descending order (equal values by ascending index),
    ``route_norm`` (``renormalize``: divide by sum + 1e-20) and ``route_scale``.

    ``gating_output`` fp32 ``[M, E]`` → ``(topk_weights fp32 [M, topk], topk_ids int32 [M, topk])``.
    ``routed_experts_out=(record, layer)`` also writes the ids into ``record[:, layer, :]`` of a
    uint8 / uint16 ``[M, layers, topk]`` tensor, the compact routed-experts record of
    ``src/prime_rl/inference/vllm/routed_experts.py:11-33``.
    """
    _require_gpu("gating_output", gating_output)
    if gating_output.dtype != torch.float32:
        raise NotImplementedError(f"router logits must be float32, got {gating_output.dtype}")
    if gating_output.dim() != 2:
        raise ValueError("gating_output must be [M, E]")
    if score_func not in _SCORE_FUNCS:
        raise NotImplementedError(f"Unknown score function {score_func}")
    M, E = gating_output.shape
    if selection_bias is not None:
        _require_gpu("selection_bias", selection_bias)
        if selection_bias.dtype != torch.float32 or selection_bias.numel() != E:
            raise ValueError("selection_bias must be float32 with one element per expert")
    capture, capture_dtype, stride, offset = None, 0, 0, 0
    if routed_experts_out is not None:
        record, layer = routed_experts_out
        _require_gpu("routed_experts_out[0]", record)
        if record.dtype not in (torch.uint8, torch.uint16):
            raise ValueError("the routed-experts record must be uint8 or uint16")
        if record.dim() != 3 or record.shape[0] != M or record.shape[2] != topk:
            raise ValueError(f"the routed-experts record must be [M, layers, topk] = [{M}, *, {topk}]")
        if not 0 <= layer < record.shape[1]:
            raise ValueError("layer index outside the routed-experts record")
        capture, capture_dtype = record, 1 if record.dtype == torch.uint8 else 2
        stride, offset = record.shape[1] * topk, layer * topk
    weights = torch.empty((M, topk), dtype=torch.float32, device=gating_output.device)
    ids = torch.empty((M, topk), dtype=torch.int32, device=gating_output.device)
    _abi.check(
        _abi.load().moe_i8_route_topk(
            _ptr(gating_output), M, E, topk, _SCORE_FUNCS[score_func], _ptr(selection_bias), num_expert_group,
            topk_group, int(group_score_top2), int(renormalize), float(route_scale), _ptr(weights), _ptr(ids),
            _ptr(capture), capture_dtype, stride, offset, _stream(gating_output),
        )
    )
    return weights, ids


def fused_topk(
    hidden_states: torch.Tensor,
    gating_output: torch.Tensor,
    topk: int,
    renormalize: bool,
    *,
    routed_experts_out: tuple[torch.Tensor, int] | None = None,
) -> tuple[torch.Tensor, torch.Tensor]:
    """vLLM ``fused_topk``: softmax over all experts, top-k, optional renormalisation.
    ``hidden_states`` is only checked for its token count, as upstream."""
    if hidden_states.shape[0] != gating_output.shape[0]:
        raise ValueError("Number of tokens mismatch")
    return route_topk(gating_output, topk, score_func="softmax", renormalize=renormalize,
                      routed_experts_out=routed_experts_out)


def grouped_topk(
    hidden_states: torch.Tensor,
    gating_output: torch.Tensor,
    topk: int,
    renormalize: bool,
    num_expert_group: int = 0,
    topk_group: int = 0,
    scoring_func: str = "softmax",
    routed_scaling_factor: float = 1.0,
    e_score_correction_bias: torch.Tensor | None = None,
    *,
    routed_experts_out: tuple[torch.Tensor, int] | None = None,
) -> tuple[torch.Tensor, torch.Tensor]:
    """vLLM ``grouped_topk`` (DeepSeek-style): with a correction bias a group scores the sum of its
    two largest biased scores, without one its largest score; the ``topk_group`` best of
    ``num_expert_group`` groups stay eligible; weights are the unbiased scores."""
    if hidden_states.shape[0] != gating_output.shape[0]:
        raise ValueError("Number of tokens mismatch")
    if scoring_func not in ("softmax", "sigmoid"):
        raise ValueError(f"Unsupported scoring function: {scoring_func}")
    return route_topk(
        gating_output, topk, score_func=scoring_func, renormalize=renormalize, route_scale=routed_scaling_factor,
        selection_bias=e_score_correction_bias, num_expert_group=max(num_expert_group, 1),
        topk_group=max(topk_group, 1), group_score_top2=e_score_correction_bias is not None,
        routed_experts_out=routed_experts_out,
    )


def routed_experts_payload(record: torch.Tensor, start: int = 0) -> dict:
    """The wire form of a routed-experts record ``[seq_len, layers, topk]`` (uint8 / uint16), field
    for field what ``serialize_routed_experts`` builds
    (``src/prime_rl/inference/vllm/routed_experts.py:27-33``): base64 of the raw bytes, shape, start
    and dtype name.  The record is already compact on the GPU, so this is one copy to the host."""
    import base64

    if record.dim() != 3 or record.dtype not in (torch.uint8, torch.uint16):
        raise ValueError("record must be a uint8 or uint16 [seq_len, layers, topk] tensor")
    host = record.contiguous().cpu().numpy()
    return {
        "data": base64.b64encode(memoryview(host)).decode("ascii"),
        "shape": list(host.shape),
        "start": start,
        "dtype": host.dtype.name,
    }


def scaled_int8_quant(
    input: torch.Tensor, scale: torch.Tensor | None = None, azp: torch.Tensor | None = None, symmetric: bool = True
) -> tuple[torch.Tensor, torch.Tensor, None]:
    """vLLM ``ops.scaled_int8_quant`` in its dynamic per-token symmetric form: ``(q int8 like input,
    scales fp32 [..., 1], None)``, ``q = rint(x * (127 / absmax))`` with ties to even (the dense-layer
    quantiser; ``per_token_quant_int8`` of the MoE path rounds ties away from zero)."""
    if scale is not None or azp is not None or not symmetric:
        raise NotImplementedError("only dynamic per-token symmetric quantisation is supported")
    _require_gpu("input", input)
    if input.dtype != torch.bfloat16:
        raise NotImplementedError(f"only bfloat16 activations are supported, got {input.dtype}")
    cols = input.shape[-1]
    if cols % 8 or cols == 0:
        raise ValueError("last dimension must be a positive multiple of 8")
    rows = input.numel() // cols
    q = torch.empty(input.shape, dtype=torch.int8, device=input.device)
    scales = torch.empty((*input.shape[:-1], 1), dtype=torch.float32, device=input.device)
    _abi.check(
        _abi.load().moe_i8_scaled_int8_quant(_ptr(input), _abi.DTYPE_BF16, rows, cols, cols, _ptr(q), _ptr(scales),
                                             _stream(input))
    )
    return q, scales, None


def _dense_weight(name: str, w: torch.Tensor, scale: torch.Tensor) -> torch.Tensor:
    """Accept the weight as [N, K] contiguous or as vLLM holds it for scaled_mm, the [K, N] transposed view."""
    if not isinstance(w, torch.Tensor) or not w.is_cuda:
        raise ValueError(f"{name} must be a GPU tensor (this path has no CPU implementation)")
    if w.dtype != torch.int8 or w.dim() != 2:
        raise ValueError(f"{name} must be a 2-d int8 tensor")
    if not w.is_contiguous():
        if not w.t().is_contiguous():
            raise ValueError(f"{name} must be [N, K] contiguous or the transposed view of such a tensor")
        w = w.t()
    _require_gpu(f"{name}_scale", scale)
    if scale.dtype != torch.float32 or scale.numel() != w.shape[0]:
        raise ValueError(f"{name}_scale must be float32 with one element per output channel")
    return w


def _dense_workspace(x: torch.Tensor, k: int, inter: int, workspace: torch.Tensor | None = None) -> torch.Tensor:
    """Workspace of the dense entry points: the caller's (``moe_i8_dense_workspace_bytes`` bytes, needed
    under graph capture unless one was cached earlier) or the cached per-(device, stream) one."""
    m = x.numel() // k
    need = _abi.load().moe_i8_dense_workspace_bytes(m, k, inter)
    if workspace is None:
        return _workspace(x.device, _stream(x), need)
    _require_gpu("workspace", workspace)
    if workspace.numel() * workspace.element_size() < need:
        raise ValueError(f"workspace too small: need {need} bytes")
    return workspace


def apply_int8_linear(
    input: torch.Tensor,
    weight: torch.Tensor,
    weight_scale: torch.Tensor,
    input_scale: torch.Tensor | None = None,
    input_zero_point: torch.Tensor | None = None,
    azp_adj: torch.Tensor | None = None,
    bias: torch.Tensor | None = None,
    *,
    gemm_variant: str | int = "auto",
    workspace: torch.Tensor | None = None,
) -> torch.Tensor:
    """vLLM's dense W8A8 int8 linear (dynamic per-token symmetric activations, per-channel weights):
    ``scaled_int8_quant`` then ``cutlass_scaled_mm``; ``out = bf16((acc * a_scale) * w_scale)``.
    ``weight`` int8 is ``[N, K]`` contiguous or its ``[K, N]`` transposed view."""
    if input_scale is not None or input_zero_point is not None or azp_adj is not None:
        raise NotImplementedError("static or asymmetric activation quantisation is not supported")
    if bias is not None:
        raise NotImplementedError("bias is not supported")
    _require_gpu("input", input)
    if input.dtype != torch.bfloat16:
        raise NotImplementedError(f"only bfloat16 activations are supported, got {input.dtype}")
    w = _dense_weight("weight", weight, weight_scale)
    n, k = w.shape
    if input.shape[-1] != k:
        raise ValueError(f"input has {input.shape[-1]} features, weight expects {k}")
    m = input.numel() // k
    out = torch.empty((*input.shape[:-1], n), dtype=torch.bfloat16, device=input.device)
    ws = _dense_workspace(input, k, 0, workspace)
    _abi.check(
        _abi.load().moe_i8_w8a8_linear(_ptr(input), _ptr(w), _ptr(weight_scale), _ptr(out), m, n, k, _ptr(ws),
                                       ws.numel() * ws.element_size(), _variant(gemm_variant), _stream(input))
    )
    return out


def w8a8_mlp(
    x: torch.Tensor,
    w13: torch.Tensor,
    w13_scale: torch.Tensor,
    w2: torch.Tensor,
    w2_scale: torch.Tensor,
    *,
    gemm_variant: str | int = "auto",
    workspace: torch.Tensor | None = None,
) -> torch.Tensor:
    """Dense gated MLP ``down(silu(gate(x)) * up(x))`` in W8A8 (the shared expert the reference adds to the
    routed output, ``src/prime_rl/trainer/models/layers/moe.py:453-462``; ``FeedForward.forward``,
    ``src/prime_rl/trainer/models/layers/mlp.py:29-32``): ``w13`` int8 ``[2I, H]`` gate rows first, ``w2``
    int8 ``[H, I]``, per-channel scales; both activations quantised per token with ties to even."""
    _require_gpu("x", x)
    if x.dtype != torch.bfloat16:
        raise NotImplementedError(f"only bfloat16 activations are supported, got {x.dtype}")
    w13 = _dense_weight("w13", w13, w13_scale)
    w2 = _dense_weight("w2", w2, w2_scale)
    two_i, h = w13.shape
    if two_i % 2 or w2.shape != (h, two_i // 2) or x.shape[-1] != h:
        raise ValueError("expected x [*, H], w13 [2I, H], w2 [H, I]")
    m = x.numel() // h
    out = torch.empty_like(x)
    ws = _dense_workspace(x, h, two_i // 2, workspace)
    _abi.check(
        _abi.load().moe_i8_w8a8_mlp(_ptr(x), _ptr(w13), _ptr(w13_scale), _ptr(w2), _ptr(w2_scale), _ptr(out), m, h,
                                    two_i // 2, _ptr(ws), ws.numel() * ws.element_size(), _variant(gemm_variant), _stream(x))
    )
    return out


def _check_routing(sorted_token_ids, expert_ids, num_tokens_post_padded):
    for name, t in (
        ("sorted_token_ids", sorted_token_ids),
        ("expert_ids", expert_ids),
        ("num_tokens_post_padded", num_tokens_post_padded),
    ):
        _require_gpu(name, t)
        if t.dtype != torch.int32:
            raise ValueError(f"{name} must be int32")


def _check_weights(name: str, w: torch.Tensor, scale: torch.Tensor) -> torch.Tensor:
    _require_gpu(name, w)
    if w.dtype != torch.int8 or w.dim() != 3:
        raise ValueError(f"{name} must be int8 [E, N, K]")
    _require_gpu(name + "_scale", scale)
    if scale.dtype != torch.float32:
        raise ValueError(f"{name}_scale must be float32")
    E, N, _ = w.shape
    if scale.numel() != E * N:
        raise NotImplementedError(f"{name}_scale must be per output channel, [E, N] or [E, N, 1]")
    return scale.reshape(E, N)


def gemm_gate_up_silu(
    x_q, a_scale, w1, w1_scale, sorted_token_ids, expert_ids, num_tokens_post_padded,
    top_k: int, block_size: int, num_pairs: int, variant: str | int = "auto",
) -> torch.Tensor:
    """Grouped gate_up GEMM on int8 MFMA with scale epilogue and fused SiLU·mul → bf16 ``[P, I]``."""
    _require_gpu("x_q", x_q)
    _check_routing(sorted_token_ids, expert_ids, num_tokens_post_padded)
    w1_scale = _check_weights("w1", w1, w1_scale)
    E, N, H = w1.shape
    if x_q.dtype != torch.int8 or x_q.dim() != 2 or x_q.shape[1] != H:
        raise ValueError("x_q must be int8 [M, H]")
    if N % 2:
        raise ValueError("w1 must stack gate and up: [E, 2I, H]")
    a_scale = a_scale.reshape(-1)
    out = torch.empty((num_pairs, N // 2), dtype=torch.bfloat16, device=x_q.device)
    _abi.check(
        _abi.load().moe_i8_gemm_gate_up_silu(
            _ptr(x_q), _ptr(a_scale), _ptr(w1), _ptr(w1_scale), _ptr(sorted_token_ids),
            _ptr(expert_ids), _ptr(num_tokens_post_padded), num_pairs, top_k, E, H, N // 2,
            _block_size(block_size), sorted_token_ids.numel(), _ptr(out), _variant(variant),
            _stream(x_q),
        )
    )
    return out


def gemm_down(
    h_q, a_scale, w2, w2_scale, topk_weights, sorted_token_ids, expert_ids,
    num_tokens_post_padded, block_size: int, variant: str | int = "auto",
) -> torch.Tensor:
    """Grouped down GEMM on int8 MFMA, scales and routed weight in the epilogue → bf16 ``[P, H]``."""
    _require_gpu("h_q", h_q)
    _check_routing(sorted_token_ids, expert_ids, num_tokens_post_padded)
    w2_scale = _check_weights("w2", w2, w2_scale)
    E, H, I = w2.shape
    if h_q.dtype != torch.int8 or h_q.dim() != 2 or h_q.shape[1] != I:
        raise ValueError("h_q must be int8 [P, I]")
    P = h_q.shape[0]
    tw = topk_weights.reshape(-1)
    if tw.dtype != torch.float32 or tw.numel() != P:
        raise ValueError("topk_weights must be float32 with one entry per pair")
    a_scale = a_scale.reshape(-1)
    out = torch.empty((P, H), dtype=torch.bfloat16, device=h_q.device)
    _abi.check(
        _abi.load().moe_i8_gemm_down(
            _ptr(h_q), _ptr(a_scale), _ptr(w2), _ptr(w2_scale), _ptr(tw), _ptr(sorted_token_ids),
            _ptr(expert_ids), _ptr(num_tokens_post_padded), P, E, H, I, _block_size(block_size),
            sorted_token_ids.numel(), _ptr(out), _variant(variant), _stream(h_q),
        )
    )
    return out


def gemm_down_bf16(
    act, w2, w2_scale, topk_weights, sorted_token_ids, expert_ids, num_tokens_post_padded, block_size: int
) -> torch.Tensor:
    """The down GEMM of the streaming family with the second ``per_token_quant_int8`` folded in: ``act`` is
    the bf16 ``[P, I]`` output of the gate_up GEMM; the result equals quantising it and calling ``gemm_down``."""
    _require_gpu("act", act)
    _check_routing(sorted_token_ids, expert_ids, num_tokens_post_padded)
    w2_scale = _check_weights("w2", w2, w2_scale)
    E, H, I = w2.shape
    if act.dtype != torch.bfloat16 or act.dim() != 2 or act.shape[1] != I:
        raise ValueError("act must be bfloat16 [P, I]")
    P = act.shape[0]
    tw = topk_weights.reshape(-1)
    if tw.dtype != torch.float32 or tw.numel() != P:
        raise ValueError("topk_weights must be float32 with one entry per pair")
    out = torch.empty((P, H), dtype=torch.bfloat16, device=act.device)
    _abi.check(
        _abi.load().moe_i8_gemm_down_bf16(
            _ptr(act), _ptr(w2), _ptr(w2_scale), _ptr(tw), _ptr(sorted_token_ids), _ptr(expert_ids),
            _ptr(num_tokens_post_padded), P, E, H, I, _block_size(block_size), sorted_token_ids.numel(), _ptr(out),
            _stream(act),
        )
    )
    return out


def gemm_acc_i32(
    a_q, w, sorted_token_ids, expert_ids, num_tokens_post_padded, row_div: int, block_size: int,
    num_pairs: int, variant: str | int = "auto",
) -> torch.Tensor:
    """Raw int32 accumulators ``acc[t, n] = Σ_K a_q[t // row_div, K]·w[e_t, n, K]`` → int32 ``[P, N]``
    (rows of pairs whose expert id is out of range are left zero)."""
    _require_gpu("a_q", a_q)
    _require_gpu("w", w)
    _check_routing(sorted_token_ids, expert_ids, num_tokens_post_padded)
    E, N, K = w.shape
    if a_q.dtype != torch.int8 or w.dtype != torch.int8 or a_q.shape[-1] != K:
        raise ValueError("a_q int8 [*, K] and w int8 [E, N, K] expected")
    out = torch.zeros((num_pairs, N), dtype=torch.int32, device=a_q.device)
    _abi.check(
        _abi.load().moe_i8_gemm_acc_i32(
            _ptr(a_q), _ptr(w), _ptr(sorted_token_ids), _ptr(expert_ids),
            _ptr(num_tokens_post_padded), num_pairs, row_div, E, N, K, _block_size(block_size),
            sorted_token_ids.numel(), _ptr(out), _variant(variant), _stream(a_q),
        )
    )
    return out


# --------------------------------------------------------------------------------------------- #
def _capturing(device: torch.device) -> bool:
    return bool(torch.cuda.is_available() and torch.cuda.is_current_stream_capturing())


def _workspace(device: torch.device, stream: int, nbytes: int, pin: bool = False) -> torch.Tensor:
    """Default workspace of a (device, stream).  A buffer that ``reserve_workspace`` allocated, or that a
    call made under graph capture used, is *pinned*: a captured graph may hold its address, so it is never
    replaced in place or evicted; when a later eager call needs more, the pinned buffer moves to a keep-alive
    list (it stays allocated for the life of the process) and a larger one takes its place in the cache.
    Only buffers that no capture has seen are freed, when the cache is over its size or they are outgrown."""
    key = (device.index if device.index is not None else torch.cuda.current_device(), stream)
    with _workspaces_lock:
        ws = _workspaces.get(key)
        capturing = _capturing(device)
        if ws is not None and ws.numel() >= nbytes:
            _workspaces.move_to_end(key)
            if pin or capturing:
                _pinned_workspaces.add(key)
            return ws
        if capturing:
            raise RuntimeError(
                f"this call needs a {nbytes}-byte workspace while the stream is being captured into a graph and "
                "none of that size was allocated for it beforehand: pass workspace=, or call reserve_workspace() "
                "(or run the largest batch once eagerly on this stream) before capturing"
            )
        if ws is not None and key in _pinned_workspaces:
            _retired_workspaces.append(ws)  # a graph may replay on it: keep it allocated
            _pinned_workspaces.discard(key)
        ws = torch.empty((max(nbytes, 256),), dtype=torch.uint8, device=device)
        _workspaces[key] = ws
        _workspaces.move_to_end(key)
        if pin:
            _pinned_workspaces.add(key)
        if len(_workspaces) > _MAX_CACHED_WORKSPACES:
            for old_key in [k for k in _workspaces if k not in _pinned_workspaces and k != key]:
                if len(_workspaces) <= _MAX_CACHED_WORKSPACES:
                    break
                del _workspaces[old_key]
        return ws


def reserve_workspace(max_tokens: int, top_k: int, num_experts: int, hidden: int, inter: int, device=None,
                      block_size_m: int = DEFAULT_BLOCK_SIZE_M) -> torch.Tensor:
    """Allocate now (outside any graph capture) the default workspace that ``fused_experts`` calls on the
    current stream of ``device`` use for up to ``max_tokens`` tokens of this layer shape, so that captured
    calls find it.  The tensor stays allocated for the life of the process (graphs captured against it stay
    valid whatever later calls need); it is also returned."""
    device = torch.device("cuda", torch.cuda.current_device()) if device is None else torch.device(device)
    stream = torch.cuda.current_stream(device).cuda_stream
    return _workspace(device, stream, workspace_bytes(max_tokens, top_k, num_experts, hidden, inter, block_size_m),
                      pin=True)


def fused_experts(
    hidden_states: torch.Tensor,
    w1: torch.Tensor,
    w2: torch.Tensor,
    topk_weights: torch.Tensor,
    topk_ids: torch.Tensor,
    inplace: bool = False,
    activation: str = "silu",
    apply_router_weight_on_input: bool = False,
    use_int8_w8a8: bool = False,
    per_channel_quant: bool = False,
    global_num_experts: int = -1,
    expert_map: torch.Tensor | None = None,
    w1_scale: torch.Tensor | None = None,
    w2_scale: torch.Tensor | None = None,
    a1_scale: torch.Tensor | None = None,
    a2_scale: torch.Tensor | None = None,
    block_shape: list[int] | None = None,
    *,
    block_size_m: int = DEFAULT_BLOCK_SIZE_M,
    gemm_variant: str | int = "auto",
    workspace: torch.Tensor | None = None,
    out: torch.Tensor | None = None,
) -> torch.Tensor:
    """Drop-in for vLLM ``fused_experts`` on the INT8 W8A8 path (per-channel weight scales, dynamic
    per-token activation scales, SiLU-gated experts, routed weight applied after the experts).

    ``a1_scale`` / ``a2_scale`` are accepted for signature compatibility and ignored: with
    per-token dynamic quantisation upstream recomputes them too.  The keyword-only arguments are
    extensions: the moe_align block size (64, as the baseline pins it), the GEMM kernel family, an
    optional caller-owned workspace of ``workspace_bytes(...)`` bytes and an optional bf16 ``[M, H]``
    tensor to write the result into.  Without ``workspace`` a cached per-(device, stream) buffer is
    used; it is never allocated or grown while the stream is being captured (see ``reserve_workspace``).

    ``topk_ids`` must lie in ``[0, E)`` (there is no expert map on this path, and a pair routed
    nowhere would leave its row of the intermediate buffer unwritten) and the ``k`` experts of one
    token must be distinct, as every router produces them: the kernels size their work on an expert
    holding at most one row per token.
    """
    if not use_int8_w8a8:
        raise NotImplementedError("this library implements only the use_int8_w8a8=True path")
    if not per_channel_quant:
        raise NotImplementedError("int8 W8A8 MoE requires per_channel_quant=True (channel-wise weights)")
    if activation != "silu":
        raise NotImplementedError(f"activation {activation!r} is not supported (only 'silu')")
    if apply_router_weight_on_input:
        raise NotImplementedError("apply_router_weight_on_input=True is not supported")
    if expert_map is not None:
        raise NotImplementedError("expert_map (expert parallelism) is not supported on this path")
    if block_shape is not None:
        raise NotImplementedError("block-wise quantisation (block_shape) is not supported")
    if w1_scale is None or w2_scale is None:
        raise ValueError("w1_scale and w2_scale are required for use_int8_w8a8")
    _require_gpu("hidden_states", hidden_states)
    if hidden_states.dtype != torch.bfloat16:
        raise NotImplementedError(f"only bfloat16 hidden_states are supported, got {hidden_states.dtype}")
    if hidden_states.dim() != 2:
        raise ValueError("hidden_states must be [M, H]")
    w1_scale = _check_weights("w1", w1, w1_scale)
    w2_scale = _check_weights("w2", w2, w2_scale)
    M, H = hidden_states.shape
    E, N1, K1 = w1.shape
    if K1 != H:
        raise ValueError(f"hidden size mismatch: hidden_states {H} vs w1 {K1}")
    if N1 % 2:
        raise ValueError("w1 must stack gate and up: [E, 2I, H]")
    I = N1 // 2
    if tuple(w2.shape) != (E, H, I):
        raise ValueError(f"w2 must be [E, H, I] = {(E, H, I)}, got {tuple(w2.shape)}")
    if global_num_experts not in (-1, E):
        raise NotImplementedError("global_num_experts != local expert count needs expert_map")
    if E > _abi.MAX_EXPERTS:
        raise ValueError(f"at most {_abi.MAX_EXPERTS} experts are supported")
    if H % 64 or I % 64:
        raise ValueError("hidden and intermediate sizes must be multiples of 64")
    if topk_weights.shape != topk_ids.shape or topk_ids.dim() != 2 or topk_ids.shape[0] != M:
        raise ValueError("topk_weights and topk_ids must both be [M, k]")
    _require_gpu("topk_ids", topk_ids)
    _require_gpu("topk_weights", topk_weights)
    block_size_m = _block_size(block_size_m)
    k = topk_ids.shape[1]
    if out is not None:
        _require_gpu("out", out)
        if out.shape != hidden_states.shape or out.dtype != torch.bfloat16:
            raise ValueError("out must be bfloat16 with the shape of hidden_states")
    else:
        out = hidden_states if inplace else torch.empty_like(hidden_states)
    if M == 0:
        return out
    ids = _as_i32_ids(topk_ids)
    tw = topk_weights if topk_weights.dtype == torch.float32 else topk_weights.to(torch.float32)
    lib = _abi.load()
    need = workspace_bytes(M, k, E, H, I, block_size_m)
    stream = _stream(hidden_states)
    if workspace is None:
        workspace = _workspace(hidden_states.device, stream, need)
    else:
        _require_gpu("workspace", workspace)
        if workspace.numel() * workspace.element_size() < need:
            raise ValueError(f"workspace too small: need {need} bytes")
    _abi.check(
        lib.moe_i8_fused_experts(
            _ptr(hidden_states), _ptr(w1), _ptr(w2), _ptr(tw), _ptr(ids), _ptr(w1_scale),
            _ptr(w2_scale), _ptr(out), M, k, E, H, I, block_size_m, _ptr(workspace),
            workspace.numel() * workspace.element_size(), _variant(gemm_variant), stream,
        )
    )
    return out


def fused_moe(
    hidden_states: torch.Tensor,
    w1: torch.Tensor,
    w2: torch.Tensor,
    gating_output: torch.Tensor,
    topk: int,
    renormalize: bool,
    inplace: bool = False,
    activation: str = "silu",
    use_grouped_topk: bool = False,
    num_expert_group: int | None = None,
    topk_group: int | None = None,
    custom_routing_function=None,
    use_int8_w8a8: bool = False,
    per_channel_quant: bool = False,
    global_num_experts: int = -1,
    expert_map: torch.Tensor | None = None,
    w1_scale: torch.Tensor | None = None,
    w2_scale: torch.Tensor | None = None,
    a1_scale: torch.Tensor | None = None,
    a2_scale: torch.Tensor | None = None,
    block_shape: list[int] | None = None,
    *,
    scoring_func: str = "softmax",
    routed_scaling_factor: float = 1.0,
    e_score_correction_bias: torch.Tensor | None = None,
    routed_experts_out: tuple[torch.Tensor, int] | None = None,
    block_size_m: int = DEFAULT_BLOCK_SIZE_M,
    gemm_variant: str | int = "auto",
    workspace: torch.Tensor | None = None,
) -> torch.Tensor:
    """vLLM ``fused_moe``: routing from the router logits (``fused_topk``, or ``grouped_topk`` with
    ``use_grouped_topk``) followed by ``fused_experts`` — the router launch and the layer's launches on the
    current stream.  ``gating_output`` must be float32 (the reference runs its router in fp32,
    ``src/prime_rl/trainer/models/layers/moe.py:262-269``)."""
    if custom_routing_function is not None:
        raise NotImplementedError("custom_routing_function is not supported")
    if gating_output.dtype != torch.float32:
        gating_output = gating_output.float()
    if use_grouped_topk:
        if not num_expert_group or not topk_group:
            raise ValueError("use_grouped_topk needs num_expert_group and topk_group")
        topk_weights, topk_ids = grouped_topk(
            hidden_states, gating_output, topk, renormalize, num_expert_group, topk_group, scoring_func,
            routed_scaling_factor, e_score_correction_bias, routed_experts_out=routed_experts_out,
        )
    else:
        if scoring_func != "softmax" or e_score_correction_bias is not None or routed_scaling_factor != 1.0:
            topk_weights, topk_ids = route_topk(
                gating_output, topk, score_func=scoring_func, renormalize=renormalize,
                route_scale=routed_scaling_factor, selection_bias=e_score_correction_bias,
                routed_experts_out=routed_experts_out,
            )
        else:
            topk_weights, topk_ids = fused_topk(hidden_states, gating_output, topk, renormalize,
                                                routed_experts_out=routed_experts_out)
    return fused_experts(
        hidden_states, w1, w2, topk_weights, topk_ids, inplace=inplace, activation=activation,
        use_int8_w8a8=use_int8_w8a8, per_channel_quant=per_channel_quant, global_num_experts=global_num_experts,
        expert_map=expert_map, w1_scale=w1_scale, w2_scale=w2_scale, a1_scale=a1_scale, a2_scale=a2_scale,
        block_shape=block_shape, block_size_m=block_size_m, gemm_variant=gemm_variant, workspace=workspace,
    )
