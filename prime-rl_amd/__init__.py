"""gfx950-native INT8 W8A8 fused-MoE path (drop-in for vLLM's ``fused_experts``).

The directory name carries a hyphen, so import it through the top-level ``prime_rl_amd`` module
(``import prime_rl_amd``), which aliases this package and its submodules.
"""

from . import _abi, inputs  # noqa: F401
from .api import (  # noqa: F401
    DEFAULT_BLOCK_SIZE_M,
    apply_int8_linear,
    fused_experts,
    fused_moe,
    fused_topk,
    layer_plan,
    grouped_topk,
    route_topk,
    routed_experts_payload,
    scaled_int8_quant,
    w8a8_mlp,
    gemm_acc_i32,
    gemm_down,
    gemm_down_bf16,
    gemm_gate_up_silu,
    moe_align_block_size,
    moe_sum,
    per_token_quant_int8,
    quantize_expert_weights,
    load_quantized_expert_weights,
    load_weights_kernel_int8,
    reserve_workspace,
    quantize_weights_per_channel,
    sorted_capacity,
    workspace_bytes,
)
from . import api, build, vllm_plugin  # noqa: F401

__all__ = [
    "fused_experts",
    "fused_moe",
    "layer_plan",
    "moe_align_block_size",
    "per_token_quant_int8",
    "quantize_weights_per_channel",
    "quantize_expert_weights",
    "load_quantized_expert_weights",
    "load_weights_kernel_int8",
    "reserve_workspace",
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
    "sorted_capacity",
    "DEFAULT_BLOCK_SIZE_M",
]
