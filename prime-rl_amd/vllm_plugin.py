"""vLLM general-plugin shim: installs this library's ``fused_experts`` for INT8 W8A8 MoE layers.

Installed the way the reference installs its own patches: a zero-argument function named by a
``[project.entry-points."vllm.general_plugins"]`` entry (reference ``pyproject.toml:49-50``) that
vLLM runs in every process, spawned workers included (``src/prime_rl/inference/patches.py:4-11``).
It is idempotent through a marker attribute (``patches.py:57-58``), gated by an environment
variable because workers are spawned without config objects
(``src/prime_rl/inference/vllm/worker/__init__.py:12-22``), and rebinds the name in every module
that imported it with ``from ... import fused_experts`` (``patches.py:227-231``).

Two surfaces are covered:

* the flat ``fused_experts(hidden_states, w1, w2, topk_weights, topk_ids, ..., use_int8_w8a8=True, ...)``
  function: calls this library handles go to the HIP path, everything else (another quantisation
  mode, an expert map, a bias, a keyword this library does not know, a shape it rejects — decided from
  the shapes before the call, and again if the entry's own validation raises ``ValueError`` or
  ``NotImplementedError``) falls through to the original.  Errors raised while the HIP path runs
  (a failed launch, a capture without a reserved workspace) are not swallowed;
* the modular-kernel surface the pinned vLLM selects kernels through (``FusedMoE`` is a factory
  returning a ``MoERunner``, reference ``src/prime_rl/inference/vllm/worker/weight_transfer.py:76-82``;
  the choice of experts implementation goes through ``FusedMoEConfig``, ``patches.py:740-757``):
  ``Int8W8A8HipExperts`` has the ``apply(output, hidden_states, w1, w2, topk_weights, topk_ids, ...)``
  shape of an experts implementation and forwards to the same C-ABI driver;
  ``register_experts_selection()`` makes the int8 W8A8 quantisation method's ``select_gemm_impl`` return
  it for layers this library can take.

Nothing here allocates under HIP graph capture: a call made while the stream is capturing uses a
workspace that was allocated beforehand for that (device, stream) by ``reserve_workspace`` or by an
earlier eager call of at least the same size, and raises otherwise.

Without vLLM installed ``register()`` is a no-op.  vLLM itself cannot be run offline; the
rebinding, marker and fall-through logic is exercised against a stand-in module tree in the CPU tests.
"""

from __future__ import annotations

import importlib
import inspect
import os
import sys

ENV_FLAG = "PRIME_MOE_I8_HIP"
_MARK = "_prime_moe_i8_hip_patched"
FUSED_MOE_MODULE = "vllm.model_executor.layers.fused_moe.fused_moe"
# keywords of vLLM's flat signature that select another code path when truthy: the HIP path is only
# taken when all of them are absent or falsy
_OTHER_MODE_FLAGS = (
    "use_fp8_w8a8", "use_int8_w8a16", "use_int4_w4a16", "use_mxfp4_w4a4", "use_nvfp4_w4a4", "ocp_mx_scheme",
    "w1_zp", "w2_zp", "w1_bias", "w2_bias", "allow_deep_gemm", "allow_cutlass_block_scaled_grouped_gemm",
    "apply_router_weight_on_input", "expert_map", "block_shape",
)


def _accepted_keywords(fn) -> frozenset:
    return frozenset(
        name for name, p in inspect.signature(fn).parameters.items()
        if p.kind in (inspect.Parameter.POSITIONAL_OR_KEYWORD, inspect.Parameter.KEYWORD_ONLY)
    )


def _present(value) -> bool:
    """A keyword counts as set unless it is None or False.  Decided by identity only: the value may be a
    tensor (an expert map, a bias, zero points), whose truth value is ambiguous or forces a device sync."""
    return value is not None and value is not False


def _shapes_eligible(hidden_states, w1, w2, kwargs) -> bool:
    """The argument checks of the HIP entry that depend on shapes only, made up front so that a layer this
    library cannot take goes to the original instead of failing the forward pass.  Objects without shapes
    (nothing to check) pass; the entry validates again."""
    try:
        s1, s2, sx = tuple(w1.shape), tuple(w2.shape), tuple(hidden_states.shape)
    except (AttributeError, TypeError):
        return True
    if len(sx) != 2 or len(s1) != 3 or len(s2) != 3:
        return False
    experts, n1, hidden = s1
    if n1 % 2 or sx[1] != hidden or s2 != (experts, hidden, n1 // 2):
        return False
    if experts > 1024 or hidden % 64 or (n1 // 2) % 64:
        return False
    gne = kwargs.get("global_num_experts", -1)
    return gne in (-1, experts)


def _handles(hidden_states, w1, w2, kwargs, accepted) -> bool:
    if kwargs.get("use_int8_w8a8", False) is not True or kwargs.get("per_channel_quant", False) is not True:
        return False
    if kwargs.get("activation", "silu") != "silu":
        return False
    if any(_present(kwargs.get(flag)) for flag in _OTHER_MODE_FLAGS):
        return False
    # a keyword this library has never heard of may change the meaning of the call
    if any(k not in accepted and k not in _OTHER_MODE_FLAGS and _present(v) for k, v in kwargs.items()):
        return False
    if kwargs.get("w1_scale") is None or kwargs.get("w2_scale") is None:
        return False
    if not (bool(getattr(hidden_states, "is_cuda", False)) and str(getattr(hidden_states, "dtype", "")) == "torch.bfloat16"):
        return False
    return _shapes_eligible(hidden_states, w1, w2, kwargs)


def _wrap(original, hip_fused_experts=None):
    if hip_fused_experts is None:
        from .api import fused_experts as hip_fused_experts
    accepted = _accepted_keywords(hip_fused_experts)
    signature = inspect.signature(hip_fused_experts)

    def fused_experts(hidden_states, w1, w2, topk_weights, topk_ids, *args, **kwargs):
        if not args and _handles(hidden_states, w1, w2, kwargs, accepted):
            forwarded = {k: v for k, v in kwargs.items() if k in accepted}
            try:
                signature.bind(hidden_states, w1, w2, topk_weights, topk_ids, **forwarded)
            except TypeError:
                bound = False  # the call does not fit the HIP entry's signature: not ours
            else:
                bound = True
            if bound:
                try:
                    return hip_fused_experts(hidden_states, w1, w2, topk_weights, topk_ids, **forwarded)
                except (NotImplementedError, ValueError):
                    pass  # a mode or shape the entry's own validation rejects: the original handles it
        return original(hidden_states, w1, w2, topk_weights, topk_ids, *args, **kwargs)

    setattr(fused_experts, _MARK, True)
    fused_experts.__wrapped__ = original
    return fused_experts


def _register_flat() -> bool:
    try:
        fm = importlib.import_module(FUSED_MOE_MODULE)
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


# Where the engine picks the experts implementation of an int8 W8A8 MoE layer: the quantisation method's
# ``select_gemm_impl(prepare_finalize, layer)`` returns the object whose ``apply`` the modular kernel calls.
# (Class and module names as vLLM publishes them for channel-wise int8 compressed-tensors checkpoints; override
# with PRIME_MOE_I8_HIP_METHOD="module:Class[,module:Class...]" for another quantisation method.)
MODULAR_METHODS = (
    ("vllm.model_executor.layers.quantization.compressed_tensors.compressed_tensors_moe",
     "CompressedTensorsW8A8Int8MoEMethod"),
)
ENV_METHODS = "PRIME_MOE_I8_HIP_METHOD"


def _layer_eligible(method, layer) -> bool:
    """Channel-wise int8 weights with dynamic per-token activation scales, SiLU, every expert local."""
    w13, w2 = getattr(layer, "w13_weight", None), getattr(layer, "w2_weight", None)
    s13, s2 = getattr(layer, "w13_weight_scale", None), getattr(layer, "w2_weight_scale", None)
    if w13 is None or w2 is None or s13 is None or s2 is None:
        return False
    if str(getattr(w13, "dtype", "")) != "torch.int8" or str(getattr(w2, "dtype", "")) != "torch.int8":
        return False
    if getattr(layer, "expert_map", None) is not None or getattr(layer, "_expert_map", None) is not None:
        return False
    if getattr(layer, "activation", "silu") != "silu":
        return False
    if getattr(method, "static_input_scales", False) is True:
        return False
    if getattr(layer, "w13_input_scale", None) is not None or getattr(layer, "w2_input_scale", None) is not None:
        return False
    probe = type("x", (), {"shape": (1, w13.shape[-1])})()
    return _shapes_eligible(probe, w13, w2, {})


def _wrap_select_gemm_impl(original):
    def select_gemm_impl(self, prepare_finalize, layer, *args, **kwargs):
        if _layer_eligible(self, layer):
            return Int8W8A8HipExperts(layer.w13_weight_scale, layer.w2_weight_scale)
        return original(self, prepare_finalize, layer, *args, **kwargs)

    setattr(select_gemm_impl, _MARK, True)
    select_gemm_impl.__wrapped__ = original
    return select_gemm_impl


def register_experts_selection() -> bool:
    """Put ``Int8W8A8HipExperts`` where the engine selects a MoE layer's experts implementation, the way the
    reference steers that selection by patching a class of the pinned vLLM in every process
    (``src/prime_rl/inference/patches.py:740-757``, gated by an environment variable as in
    ``src/prime_rl/inference/vllm/worker/__init__.py:12-22``): ``select_gemm_impl`` of the int8 W8A8 MoE
    quantisation method returns the HIP experts for layers this library can take and defers to the original
    otherwise.  Idempotent; returns True when at least one class was patched.  Exercised on the CPU against a
    stand-in class; which class the pinned vLLM uses can only be confirmed on a machine that has it, hence the
    override variable."""
    if os.environ.get(ENV_FLAG, "0") != "1":
        return False
    targets = list(MODULAR_METHODS)
    override = os.environ.get(ENV_METHODS, "")
    if override:
        targets = [tuple(item.split(":", 1)) for item in override.split(",") if ":" in item]
    patched_any = False
    for module_name, class_name in targets:
        try:
            cls = getattr(importlib.import_module(module_name), class_name, None)
        except ImportError:
            continue
        original = getattr(cls, "select_gemm_impl", None) if cls is not None else None
        if original is None or getattr(original, _MARK, False):
            continue
        cls.select_gemm_impl = _wrap_select_gemm_impl(original)
        patched_any = True
    return patched_any


def register() -> bool:
    """Entry point for ``vllm.general_plugins``. Returns True when a patch was applied: the flat
    ``fused_experts`` function is rebound and the experts selection of the modular-kernel path is steered."""
    if os.environ.get(ENV_FLAG, "0") != "1":
        return False
    flat = _register_flat()
    modular = register_experts_selection()
    return flat or modular


def reserve_workspace(max_tokens: int, top_k: int, num_experts: int, hidden: int, inter: int, device=None,
                      block_size_m: int = 64):
    """Allocate, before any graph capture, the workspace calls on the current stream of `device` will use
    for batches of up to `max_tokens` tokens.  Returns the tensor (the cache keeps it alive)."""
    from . import api

    return api.reserve_workspace(max_tokens, top_k, num_experts, hidden, inter, device=device,
                                 block_size_m=block_size_m)


class Int8W8A8HipExperts:
    """Experts implementation with the ``apply`` shape of vLLM's modular MoE kernels
    (``TritonExperts.apply(output, hidden_states, w1, w2, topk_weights, topk_ids, activation,
    global_num_experts, expert_map, a1q_scale, a2_scale, workspace13, workspace2, ...)``) for channel-wise
    int8 weights with dynamic per-token activation scales (what ``int8_w8a8_moe_quant_config(w1_scale,
    w2_scale, per_act_token_quant=True)`` describes).  ``apply`` writes the layer's result into ``output``.

    The activation quantisation runs inside the library, so ``hidden_states`` is the bf16 input and an
    ``a1q_scale`` handed over by a prepare step that has already quantised is refused (that pairing
    would quantise twice).  vLLM's two workspace tensors are not used: the library's own workspace
    holds its intermediates.
    """

    def __init__(self, w1_scale, w2_scale, block_size_m: int = 64, gemm_variant: str = "auto"):
        self.w1_scale = w1_scale
        self.w2_scale = w2_scale
        self.block_size_m = block_size_m
        self.gemm_variant = gemm_variant

    def supports_expert_map(self) -> bool:
        return False

    def supports_chunking(self) -> bool:
        return True

    def apply(self, output, hidden_states, w1, w2, topk_weights, topk_ids, activation="silu",
              global_num_experts=-1, expert_map=None, a1q_scale=None, a2_scale=None, workspace13=None,
              workspace2=None, expert_tokens_meta=None, apply_router_weight_on_input=False, **_unused):
        from . import api

        if a1q_scale is not None:
            raise NotImplementedError("hidden_states must be the unquantised bf16 input (a1q_scale is None)")
        result = api.fused_experts(
            hidden_states, w1, w2, topk_weights, topk_ids, inplace=False, activation=activation,
            apply_router_weight_on_input=apply_router_weight_on_input, use_int8_w8a8=True, per_channel_quant=True,
            global_num_experts=global_num_experts, expert_map=expert_map, w1_scale=self.w1_scale,
            w2_scale=self.w2_scale, block_size_m=self.block_size_m, gemm_variant=self.gemm_variant, out=output,
        )
        return result
