"""CPU oracle for the INT8 W8A8 fused-MoE layer.  TEST INFRASTRUCTURE ONLY.

This module is the checker, never the product: only ``tests/``,
``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` may
import it.  It restates, on the CPU with torch, the algorithm that the
reference's rollout engine runs for an int8-quantised MoE layer.  That
arithmetic is not in the reference tree: it lives in the pinned third-party
dependency vLLM 0.28.0 (reference ``pyproject.toml:58``, ``uv.lock:8107-8109``),
selected only through the ``quantization`` pass-through
(``packages/prime-rl-configs/src/prime_rl/configs/inference.py:108-109``).
Each function therefore restates vLLM's published algorithm and is anchored on
the closest statement of the same semantics that IS in the reference tree.

Pinning status (what independent evidence each function is checked against in
``tests/test_oracle_*.py``):

* ``moe_align_block_size``   pinned: upstream docstring known answer; closed form
  (bincount / cumsum / stable argsort as in the reference's
  ``trainer/distributed/token_dispatcher.py:139-145``); brute force; invariants.
* ``per_token_quant_int8``   pinned: tie vector, zero row, error-bound invariants,
  element-wise brute force in Python floats.
* ``grouped_int_gemm``       pinned: brute-force triple loop; ``torch._int_mm``
  versus float64 matmul (two library routines).
* ``silu_and_mul``           pinned: ``F.silu(g) * u`` in torch bf16, the
  reference's own activation (``trainer/models/layers/activations.py:29-34``).
* ``moe_sum`` / combine      pinned: the reference's dispatcher known answer
  (``tests/unit/train/models/test_moe.py:83-109``) and closed form.
* ``quantize_weights_per_channel`` / ``quantize_expert_weights``  layout pinned by the
  shapes the reference's conversion test asserts
  (``tests/unit/train/models/test_glm_moe_dsa_conversion.py:47-50,65-68``) and by ``torch.cat``;
  arithmetic pinned by a tie vector, zero rows, the half-step error bound and an element-wise
  brute force in numpy float32.  Parity unpinned against an int8 checkpoint producer: the
  reference tree quantises weights to FP8 only (``trainer/models/fp8.py:5-41``); the int8
  rule here is that function with qmax = 127, a whole row as the block and the integer grid.
* ``route_topk``             pinned: element-wise brute force in Python floats (math.exp, sorted by
  (-value, index)); closed forms (weights of the softmax router sum to 1 after renormalisation,
  a selection bias changes which experts are chosen but not the weights of those chosen, the
  grouped router only returns experts of ``topk_groups`` groups, one group = the ungrouped router);
  agreement with the older ``softmax_topk`` / ``grouped_topk`` restatements.  Order among exactly
  equal selection values is this build's rule (ascending index); ``torch.topk`` leaves it open.
* ``serialize_routed_experts`` pinned: the two payloads of the reference's own tests
  (``tests/unit/inference/test_serving_tokens.py:46-60``: a 2x2x2 int64 array round-trips as uint8;
  ``"AQID"`` is bytes 1,2,3 of shape [1,1,3]) and the uint16 switch above 255.
* ``scaled_int8_quant`` / ``w8a8_linear`` / ``w8a8_mlp``  pinned: tie vector (even, and different from the
  half-away quantiser on it), numpy float32 brute force; the linear against a float64 matmul of the
  dequantised operands; the MLP against the MoE layer with one expert that every token visits (which
  differs only in the rounding of ties) and against the fp32 MLP.  Parity unpinned at the vLLM
  boundary (``scaled_int8_quant`` / ``cutlass_scaled_mm`` are not in the reference tree).
* ``fused_experts`` (whole)  parity unpinned at the vLLM boundary: no test or
  fixture in the reference touches int8 ``fused_experts``.  Pinned only against
  ``native_w8a8_moe`` (an independent per-expert formulation) and against the
  dequantised fp32 MLP, both to a tolerance.
"""

from __future__ import annotations

import math

import numpy as np
import torch

__all__ = [
    "round_half_away",
    "per_token_quant_int8",
    "moe_align_block_size",
    "grouped_int_gemm",
    "scale_epilogue",
    "silu_and_mul",
    "moe_sum",
    "fused_experts_staged",
    "fused_experts",
    "native_w8a8_moe",
    "dequant_fp32_moe",
    "softmax_topk",
    "grouped_topk",
    "quantize_weights_per_channel",
    "quantize_expert_weights",
    "route_topk",
    "serialize_routed_experts",
    "scaled_int8_quant",
    "w8a8_linear",
    "w8a8_mlp",
]


# --------------------------------------------------------------------------- #
# R1 / R5: per-token dynamic symmetric int8 quantisation
# --------------------------------------------------------------------------- #
def round_half_away(x: torch.Tensor) -> torch.Tensor:
    """Round to nearest, ties away from zero (C ``roundf``); ``torch.round`` is ties-to-even."""
    t = torch.trunc(x)
    return t + torch.sign(x) * ((x - t).abs() >= 0.5).to(x.dtype)


def per_token_quant_int8(x: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
    """vLLM ``per_token_quant_int8`` (``quantization/utils/int8_utils.py``), all in fp32:
    ``absmax = max(max|x|, 1e-10)``; ``scale = absmax / 127``;
    ``q = round_half_away(x * (127 / absmax))``.  Returns ``(q int8, scale fp32 [..., 1])``.
    In-tree analogue (FP8, different clamp): ``trainer/models/kernels/fp8_utils.py:186-201``.
    """
    xf = x.to(torch.float32)
    absmax = xf.abs().amax(dim=-1, keepdim=True).clamp_min(1e-10) if xf.shape[-1] else xf.new_full(
        (*xf.shape[:-1], 1), 1e-10
    )
    scale = absmax / 127.0
    # tensor / tensor is one correctly rounded IEEE division; `127.0 / absmax` on a torch tensor is
    # evaluated as reciprocal-then-multiply (two roundings) and flips near-tie elements.
    inv = torch.full_like(absmax, 127.0) / absmax
    q = round_half_away(xf * inv).to(torch.int8)
    return q, scale


# --------------------------------------------------------------------------- #
# R2: moe_align_block_size
# --------------------------------------------------------------------------- #
def moe_align_block_size(
    topk_ids: torch.Tensor, block_size: int, num_experts: int
) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """vLLM ``moe_align_block_size`` with the stable (ascending flat index) order inside
    each expert segment, i.e. the reference's ``argsort(stable=True)``
    (``trainer/distributed/token_dispatcher.py:145``) plus per-expert padding to a multiple
    of ``block_size`` (``token_dispatcher.py:107-121``).

    Returns ``sorted_token_ids`` int32 ``[P + E*(B-1)]`` (unused slots = ``P``),
    ``expert_ids`` int32 ``[ceil(EM/B)]`` (unused blocks = ``-1``) and
    ``num_tokens_post_padded`` int32 ``[1]``.
    """
    flat = topk_ids.reshape(-1).to(torch.int64).numpy()
    P, E, B = int(flat.size), int(num_experts), int(block_size)
    EM = P + E * (B - 1)
    sorted_ids = np.full(EM, P, dtype=np.int32)
    expert_ids = np.full((EM + B - 1) // B, -1, dtype=np.int32)
    cursor = 0
    for e in range(E):
        idx = np.nonzero(flat == e)[0]  # ascending flat index == stable order
        n = idx.size
        padded = (n + B - 1) // B * B
        sorted_ids[cursor : cursor + n] = idx
        expert_ids[cursor // B : (cursor + padded) // B] = e
        cursor += padded
    return (
        torch.from_numpy(sorted_ids),
        torch.from_numpy(expert_ids),
        torch.tensor([cursor], dtype=torch.int32),
    )


# --------------------------------------------------------------------------- #
# R3 / R6: grouped integer GEMM (exact int32 accumulators) and fp32 epilogue
# --------------------------------------------------------------------------- #
def _int_mm(a: torch.Tensor, b_t: torch.Tensor) -> torch.Tensor:
    """Exact ``a[m,K] @ b_t[n,K].T`` → int32 for int8 operands."""
    if a.shape[0] == 0:
        return torch.zeros((0, b_t.shape[0]), dtype=torch.int32)
    return torch._int_mm(a.contiguous(), b_t.t())


def grouped_int_gemm(
    a_q: torch.Tensor, w: torch.Tensor, topk_ids: torch.Tensor, rows_per_token: int
) -> torch.Tensor:
    """``acc[t, n] = sum_K a_q[t // rows_per_token, K] * w[e_t, n, K]`` with ``e_t = topk_ids.flat[t]``.

    ``rows_per_token = k`` for the gate_up GEMM (A row is the token's row) and ``1`` for the
    down GEMM (A row is the pair's own row).  The grouped-GEMM contract ``x[start:end] @ W[e]``
    is the reference's ``tests/unit/train/models/test_moe.py:60-66``; weights are ``[E, N, K]``
    (``inference/vllm/gpt_oss_weight_loading.py:93-104``).  Exact int32, no padding rows.
    """
    flat = topk_ids.reshape(-1).to(torch.int64)
    P = flat.numel()
    acc = torch.zeros((P, w.shape[1]), dtype=torch.int32)
    for e in torch.unique(flat).tolist():
        t = torch.nonzero(flat == e).squeeze(1)
        acc[t] = _int_mm(a_q[t // rows_per_token], w[e])
    return acc


def scale_epilogue(
    acc: torch.Tensor,
    a_scale_rows: torch.Tensor,
    w_scale: torch.Tensor,
    topk_ids: torch.Tensor,
    row_weight: torch.Tensor | None,
    out_dtype: torch.dtype,
) -> torch.Tensor:
    """fp32 epilogue of vLLM's ``fused_moe_kernel``: ``float(acc) * a_scale[row] * w_scale[e, n]``
    (then ``* topk_weight[row]`` for the down GEMM, ``MUL_ROUTED_WEIGHT``), evaluated left to
    right in fp32 and rounded once to ``out_dtype``.  Weight-after-experts in fp32 then cast is
    also the reference's convention (``trainer/distributed/token_dispatcher.py:159-160``).
    """
    flat = topk_ids.reshape(-1).to(torch.int64)
    y = acc.to(torch.float32) * a_scale_rows.reshape(-1, 1).to(torch.float32)
    y = y * w_scale.reshape(w_scale.shape[0], -1)[flat]
    if row_weight is not None:
        y = y * row_weight.reshape(-1, 1).to(torch.float32)
    return y.to(out_dtype)


# --------------------------------------------------------------------------- #
# R4: SiLU-gated activation with bf16 rounding points
# --------------------------------------------------------------------------- #
def silu_and_mul(c: torch.Tensor) -> torch.Tensor:
    """vLLM ``silu_and_mul``: ``h = dtype(float(dtype(silu_f32(g))) * float(u))`` with
    ``g = c[:, :I]``, ``u = c[:, I:]`` and ``silu(x) = x / (1 + exp(-x))`` in fp32.
    Same two roundings as ``F.silu(gate) * up`` in bf16
    (``trainer/models/layers/activations.py:29-34``).
    """
    I = c.shape[-1] // 2
    g = c[..., :I].to(torch.float32)
    u = c[..., I:].to(torch.float32)
    s = (g / (1.0 + torch.exp(-g))).to(c.dtype)
    return (s.to(torch.float32) * u).to(c.dtype)


# --------------------------------------------------------------------------- #
# R7: top-k combine
# --------------------------------------------------------------------------- #
def moe_sum(c3: torch.Tensor) -> torch.Tensor:
    """vLLM ``moe_sum``: ``out[m] = sum_j c3[m, j]``.  For k in {2,3,4} upstream's kernel adds
    sequentially in the activation dtype (one rounding per add); any other k goes through
    ``at::sum_out`` (fp32 accumulation, one rounding; restated here as j-ascending fp32 adds).
    Reference analogue: ``scatter_add`` into zeros (``token_dispatcher.py:162-165``).
    """
    M, k, H = c3.shape
    if k in (2, 3, 4):
        out = c3[:, 0].clone()
        for j in range(1, k):
            out = out + c3[:, j]  # rounds to c3.dtype after every add
        return out
    acc = torch.zeros((M, H), dtype=torch.float32)
    for j in range(k):
        acc = acc + c3[:, j].to(torch.float32)
    return acc.to(c3.dtype)


# --------------------------------------------------------------------------- #
# R0: the whole layer, stage by stage
# --------------------------------------------------------------------------- #
def fused_experts_staged(
    hidden_states: torch.Tensor,
    w1: torch.Tensor,
    w2: torch.Tensor,
    topk_weights: torch.Tensor,
    topk_ids: torch.Tensor,
    w1_scale: torch.Tensor,
    w2_scale: torch.Tensor,
    block_size: int = 64,
) -> dict[str, torch.Tensor]:
    """vLLM ``fused_experts_impl`` for ``use_int8_w8a8=True, per_channel_quant=True`` with
    dynamic per-token activation scales, returning every intermediate:
    quant → align → gate_up GEMM → SiLU·mul → quant → down GEMM (× top-k weight) → sum.
    """
    M, H = hidden_states.shape
    E, N1, _ = w1.shape
    k = topk_ids.shape[1]
    dt = hidden_states.dtype
    st: dict[str, torch.Tensor] = {}
    st["x_q"], st["a1_scale"] = per_token_quant_int8(hidden_states)
    st["sorted_token_ids"], st["expert_ids"], st["num_tokens_post_padded"] = moe_align_block_size(
        topk_ids, block_size, E
    )
    st["acc1"] = grouped_int_gemm(st["x_q"], w1, topk_ids, k)
    a1_rows = st["a1_scale"].reshape(-1).repeat_interleave(k)
    st["cache1"] = scale_epilogue(st["acc1"], a1_rows, w1_scale, topk_ids, None, dt)
    st["cache2"] = silu_and_mul(st["cache1"])
    st["h_q"], st["a2_scale"] = per_token_quant_int8(st["cache2"])
    st["acc2"] = grouped_int_gemm(st["h_q"], w2, topk_ids, 1)
    st["cache3"] = scale_epilogue(
        st["acc2"], st["a2_scale"], w2_scale, topk_ids, topk_weights.reshape(-1), dt
    ).reshape(M, k, H)
    st["out"] = moe_sum(st["cache3"])
    return st


def fused_experts(hidden_states, w1, w2, topk_weights, topk_ids, w1_scale, w2_scale, block_size=64):
    return fused_experts_staged(
        hidden_states, w1, w2, topk_weights, topk_ids, w1_scale, w2_scale, block_size
    )["out"]


# --------------------------------------------------------------------------- #
# Independent formulations used to pin the whole layer and as the CPU baseline
# --------------------------------------------------------------------------- #
def native_w8a8_moe(hidden_states, w1, w2, topk_weights, topk_ids, w1_scale, w2_scale):
    """The torch-native W8A8 MoE that upstream vLLM uses as its own test oracle
    (``torch_w8a8_per_column_moe``): per-token quant, per-expert masked loop,
    ``A.float() @ W.float().T``, ``a_scale * C * w_scale``, ``F.silu(g) * u`` in the
    activation dtype, re-quant, second matmul, top-k weight applied in the activation dtype,
    sum over k.  This is "the reference's torch CPU path" that ``bench.py`` times.
    """
    M, H = hidden_states.shape
    E = w1.shape[0]
    k = topk_ids.shape[1]
    dt = hidden_states.dtype
    a_q, a_s = per_token_quant_int8(hidden_states)
    a_q = a_q.repeat_interleave(k, dim=0)
    a_s = a_s.repeat_interleave(k, dim=0)
    flat = topk_ids.reshape(-1).to(torch.int64)
    out = torch.zeros((M * k, w2.shape[1]), dtype=dt)
    for e in range(E):
        mask = flat == e
        if not bool(mask.any()):
            continue
        c = a_q[mask].to(torch.float32) @ w1[e].to(torch.float32).t()
        c = (a_s[mask] * c * w1_scale[e].reshape(1, -1)).to(dt)
        I = c.shape[1] // 2
        act = torch.nn.functional.silu(c[:, :I]) * c[:, I:]
        act_q, act_s = per_token_quant_int8(act)
        d = act_q.to(torch.float32) @ w2[e].to(torch.float32).t()
        out[mask] = (act_s * d * w2_scale[e].reshape(1, -1)).to(dt)
    return (out.view(M, k, -1) * topk_weights.view(M, k, 1).to(dt)).sum(dim=1)


def dequant_fp32_moe(hidden_states, w1, w2, topk_weights, topk_ids, w1_scale, w2_scale):
    """Unquantised fp32 MLP with dequantised weights: sanity bound for the quantised layer,
    written as the reference's own per-expert loop (``tests/unit/train/models/test_moe.py:164-181``)."""
    M, H = hidden_states.shape
    k = topk_ids.shape[1]
    x = hidden_states.to(torch.float32)
    out = torch.zeros((M, H), dtype=torch.float32)
    for e in torch.unique(topk_ids).tolist():
        tok, slot = torch.nonzero(topk_ids == e, as_tuple=True)
        wg = w1[e].to(torch.float32) * w1_scale[e].reshape(-1, 1)
        wd = w2[e].to(torch.float32) * w2_scale[e].reshape(-1, 1)
        c = x[tok] @ wg.t()
        I = c.shape[1] // 2
        hmid = torch.nn.functional.silu(c[:, :I]) * c[:, I:]
        out.index_add_(0, tok, (hmid @ wd.t()) * topk_weights[tok, slot].reshape(-1, 1))
    return out


# --------------------------------------------------------------------------- #
# Routing used by the synthetic workloads (restated from the reference's router)
# --------------------------------------------------------------------------- #
def softmax_topk(logits: torch.Tensor, k: int, renormalize: bool = True, score_func: str = "softmax"):
    """fp32 softmax (or sigmoid) → top-k → gather scores → renormalise:
    ``trainer/models/layers/moe.py:254-298`` (score in fp32, ``route_norm`` with ``+1e-20``)."""
    lf = logits.to(torch.float32)
    scores = torch.softmax(lf, dim=1) if score_func == "softmax" else torch.sigmoid(lf)
    _, ids = torch.topk(scores, k=k, dim=1)
    w = scores.gather(1, ids)
    if renormalize:
        w = w / (w.sum(dim=-1, keepdim=True) + 1e-20)
    return w.to(torch.float32), ids.to(torch.int32)


def grouped_topk(
    logits: torch.Tensor,
    bias: torch.Tensor,
    k: int,
    num_groups: int,
    topk_groups: int,
    renormalize: bool = True,
    routed_scaling_factor: float = 1.0,
):
    """DeepSeek-V3 style grouped top-k: ``s = sigmoid(logits)``; ``s' = s + bias`` (bias affects
    selection only, as ``moe.py:276-284``); group score = sum of the top-2 ``s'`` in each group;
    keep ``topk_groups`` groups; top-k of the masked ``s'``; weights = unbiased ``s`` gathered,
    renormalised, times ``routed_scaling_factor``.  No in-tree implementation exists
    (``tests/unit/train/models/test_glm4_moe.py:31`` uses one group); this follows the published
    DeepSeek-V3 router.
    """
    M, E = logits.shape
    s = torch.sigmoid(logits.to(torch.float32))
    sb = s + bias.to(torch.float32).reshape(1, E)
    gs = sb.view(M, num_groups, E // num_groups).topk(2, dim=-1)[0].sum(dim=-1)
    gidx = gs.topk(topk_groups, dim=-1)[1]
    gmask = torch.zeros_like(gs).scatter_(1, gidx, 1.0)
    mask = gmask.unsqueeze(-1).expand(M, num_groups, E // num_groups).reshape(M, E)
    masked = sb.masked_fill(mask == 0, float("-inf"))
    ids = masked.topk(k, dim=-1)[1]
    w = s.gather(1, ids)
    if renormalize:
        w = w / (w.sum(dim=-1, keepdim=True) + 1e-20)
    w = w * routed_scaling_factor
    return w.to(torch.float32), ids.to(torch.int32)


# --------------------------------------------------------------------------- #
# Weight (re)quantisation into the kernel layout
# --------------------------------------------------------------------------- #
def quantize_weights_per_channel(w: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
    """Symmetric per-output-channel int8 quantisation of ``w [..., N, K]`` (one scale per row).

    The reference's ``quantize_to_fp8_blockwise`` (``trainer/models/fp8.py:33-36``) with the block
    widened to one whole row, ``qmax = 127`` and the integer grid: ``scale = (absmax / 127)
    .clamp(min=1e-12)``; ``q = (w.float() / scale).clamp(-127, 127)`` rounded to nearest, ties to
    even (what the cast to the quantised type does there).  Returns ``(q int8, scale fp32 [..., N])``.
    """
    wf = w.to(torch.float32)
    absmax = wf.abs().amax(dim=-1, keepdim=True)
    scale = (absmax / 127.0).clamp(min=1e-12)
    q = torch.round(wf / scale).clamp(-127, 127).to(torch.int8)
    return q, scale.squeeze(-1)


def quantize_expert_weights(gate_proj: torch.Tensor, up_proj: torch.Tensor, down_proj: torch.Tensor):
    """Trainer expert weights → the four tensors ``fused_experts`` consumes.

    ``gate_proj, up_proj [E, I, H]``, ``down_proj [E, H, I]`` (the reference's ``w1, w3, w2``) →
    ``w13 int8 [E, 2I, H]`` with gate rows first (``torch.cat([w1, w3], dim=1)``,
    ``trainer/models/glm_moe_dsa/converting_glm_moe_dsa.py:97-104``), ``w13_scale fp32 [E, 2I]``,
    ``w2 int8 [E, H, I]``, ``w2_scale fp32 [E, H]``.
    """
    w13, s13 = quantize_weights_per_channel(torch.cat([gate_proj, up_proj], dim=1))
    w2, s2 = quantize_weights_per_channel(down_proj)
    return w13, s13, w2, s2


# --------------------------------------------------------------------------- #
# Router (restated from the reference) and the routed-experts record
# --------------------------------------------------------------------------- #
def route_topk(
    logits: torch.Tensor,
    k: int,
    score_func: str = "softmax",
    renormalize: bool = True,
    route_scale: float = 1.0,
    selection_bias: torch.Tensor | None = None,
    num_groups: int = 1,
    topk_groups: int = 1,
    group_top2: bool = False,
):
    """``TokenChoiceTopKRouter.forward`` after the gate GEMM (``trainer/models/layers/moe.py:261-307``):
    scores in fp32 (:262-269), bias for selection only (:281-283), top-k (:284-289), gather of the
    unbiased scores (:290), softmax over the selected for ``topk_softmax`` (:292-293), ``route_norm``
    with ``+1e-20`` (:302-304), ``route_scale`` (:305); plus the group pre-selection of the published
    DeepSeek routers (group score = largest, or sum of the two largest, selection value).  Order:
    descending selection value, equal values by ascending index (a stable sort)."""
    lf = logits.to(torch.float32)
    M, E = lf.shape
    if score_func == "softmax":
        scores = torch.softmax(lf, dim=1)
    elif score_func == "sigmoid":
        scores = torch.sigmoid(lf)
    elif score_func == "topk_softmax":
        scores = lf
    else:
        raise NotImplementedError(f"Unknown score function {score_func}")
    sel = scores if selection_bias is None else scores + selection_bias.to(torch.float32).reshape(1, E)
    if num_groups > 1:
        per = E // num_groups
        grouped = sel.view(M, num_groups, per)
        gs = grouped.topk(2, dim=-1)[0].sum(dim=-1) if group_top2 else grouped.amax(dim=-1)
        gorder = torch.sort(gs, dim=-1, descending=True, stable=True)[1][:, :topk_groups]
        gmask = torch.zeros((M, num_groups), dtype=torch.bool).scatter_(1, gorder, True)
        sel = sel.masked_fill(~gmask.unsqueeze(-1).expand(M, num_groups, per).reshape(M, E), float("-inf"))
    ids = torch.sort(sel, dim=1, descending=True, stable=True)[1][:, :k]
    w = scores.gather(1, ids)
    if score_func == "topk_softmax":
        w = torch.softmax(w, dim=-1)
    if renormalize:
        w = w / (w.sum(dim=-1, keepdim=True) + 1e-20)
    w = w * route_scale
    return w.to(torch.float32), ids.to(torch.int32)


def serialize_routed_experts(routed_experts, start: int = 0):
    """``serialize_routed_experts`` of ``inference/vllm/routed_experts.py:11-33``: a 3-d integer array
    ``[seq_len, layers, topk]`` becomes base64 of its uint8 bytes (uint16 when an id exceeds 255)
    with ``shape``, ``start`` and ``dtype``."""
    import base64

    if routed_experts is None:
        return None
    array = np.asarray(routed_experts)
    assert array.ndim == 3 and np.issubdtype(array.dtype, np.integer)
    dtype = np.uint8
    if array.size:
        assert array.min() >= 0
        if array.max() > 255:
            assert array.max() <= 65535
            dtype = np.uint16
    compact = np.ascontiguousarray(array.astype(dtype, copy=False))
    return {
        "data": base64.b64encode(memoryview(compact)).decode("ascii"),
        "shape": list(compact.shape),
        "start": start,
        "dtype": np.dtype(dtype).name,
    }


# --------------------------------------------------------------------------- #
# Dense W8A8 (shared experts, dense MLPs)
# --------------------------------------------------------------------------- #
def scaled_int8_quant(x: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
    """vLLM ``scaled_int8_quant`` (dynamic, per token, symmetric): as ``per_token_quant_int8`` but the
    product ``x * (127 / absmax)`` is rounded to nearest with ties to even."""
    xf = x.to(torch.float32)
    absmax = xf.abs().amax(dim=-1, keepdim=True).clamp_min(1e-10)
    inv = torch.full_like(absmax, 127.0) / absmax
    return torch.round(xf * inv).to(torch.int8), absmax / 127.0


def w8a8_linear(x: torch.Tensor, w: torch.Tensor, w_scale: torch.Tensor) -> torch.Tensor:
    """``bf16((acc * a_scale) * w_scale)`` with ``acc = x_q @ w.T`` in int32; ``w`` int8 ``[N, K]``."""
    q, a = scaled_int8_quant(x.reshape(-1, x.shape[-1]))
    acc = _int_mm(q, w).to(torch.float32)
    out = ((acc * a) * w_scale.reshape(1, -1)).to(torch.bfloat16)
    return out.reshape(*x.shape[:-1], w.shape[0])


def w8a8_mlp(x, w13, w13_scale, w2, w2_scale) -> torch.Tensor:
    """``down(silu(gate(x)) * up(x))`` (``trainer/models/layers/mlp.py:29-32``) with both linears W8A8 and the
    activation evaluated on bf16 values as ``silu_and_mul`` does."""
    c = w8a8_linear(x, w13, w13_scale)
    return w8a8_linear(silu_and_mul(c), w2, w2_scale)
