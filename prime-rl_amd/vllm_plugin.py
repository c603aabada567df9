"""vLLM general-plugin shim: installs this library's ``fused_experts`` for INT8 W8A8 MoE layers.

Installed the way the reference installs its own patches: a zero-argument function named by a
``[project.entry-points."vllm.general_plugins"]`` entry (reference ``pyproject.toml:49-50``) that
vLLM runs in every process, spawned workers included (``src/prime_rl/inference/patches.py:4-11``).
It is idempotent through a marker attribute (``patches.py:57-58``), gated by an environment
variable because workers are spawned without config objects
(``src/prime_rl/inference/vllm/worker/__init__.py:12-22``), and rebinds the name in every module
that imported it with ``from ... import fused_experts`` (``patches.py:227-231``).

Without vLLM installed ``register()`` is a no-op.  It cannot be exercised offline; it is kept thin
and makes no parity claim of its own.
"""

from __future__ import annotations

import importlib
import os
import sys

ENV_FLAG = "PRIME_MOE_I8_HIP"
_MARK = "_prime_moe_i8_hip_patched"


def _wrap(original):
    from .api import fused_experts as hip_fused_experts

    def fused_experts(hidden_states, w1, w2, topk_weights, topk_ids, *args, **kwargs):
        use_hip = (
            kwargs.get("use_int8_w8a8", False)
            and kwargs.get("per_channel_quant", False)
            and kwargs.get("expert_map") is None
            and kwargs.get("block_shape") is None
            and kwargs.get("activation", "silu") == "silu"
            and not kwargs.get("apply_router_weight_on_input", False)
            and not args
            and hidden_states.is_cuda
            and str(hidden_states.dtype) == "torch.bfloat16"
        )
        if use_hip:
            return hip_fused_experts(hidden_states, w1, w2, topk_weights, topk_ids, **kwargs)
        return original(hidden_states, w1, w2, topk_weights, topk_ids, *args, **kwargs)

    setattr(fused_experts, _MARK, True)
    fused_experts.__wrapped__ = original
    return fused_experts


def register() -> bool:
    """Entry point for ``vllm.general_plugins``. Returns True when a patch was applied."""
    if os.environ.get(ENV_FLAG, "0") != "1":
        return False
    try:
        fm = importlib.import_module("vllm.model_executor.layers.fused_moe.fused_moe")
    except ImportError:
        return False
    original = getattr(fm, "fused_experts", None)
    if original is None or getattr(original, _MARK, False):
        return False
    patched = _wrap(original)
    fm.fused_experts = patched
    for mod in list(sys.modules.values()):
        if mod is None or not getattr(mod, "__name__", "").startswith("vllm."):
            continue
        if getattr(mod, "fused_experts", None) is original:
            mod.fused_experts = patched
    return True
