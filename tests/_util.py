"""Helpers shared by the GPU parity tests."""

import importlib

import torch


def inputs_mod():
    return importlib.import_module("prime_rl_amd").inputs


def rel_err(got: torch.Tensor, want: torch.Tensor) -> float:
    """mean|Δ| / mean|want| — the measure upstream's own int8 MoE test uses."""
    got, want = got.float().cpu(), want.float().cpu()
    return float((got - want).abs().mean() / want.abs().mean().clamp_min(1e-30))


def bf16_ulp_diff(got: torch.Tensor, want: torch.Tensor) -> torch.Tensor:
    """Distance in bf16 representable steps (sign-magnitude bit patterns mapped to a line).
    Magnitudes below 2^-100 count as zero: whether a product that small is flushed is not a
    property of the algorithm."""
    def key(t):
        t = t.cpu().contiguous()
        t = torch.where(t.float().abs() < 2.0 ** -100, torch.zeros_like(t), t)
        b = t.view(torch.int16).to(torch.int32) & 0xFFFF
        return torch.where(b >= 0x8000, 0x8000 - b, b)
    return (key(got) - key(want)).abs()


def subset_problem(inp, token_idx: torch.Tensor):
    """The layer is independent per token: restrict a (possibly GPU-resident, huge) problem to a few
    tokens and the experts they use, remap expert ids, and return CPU tensors for the oracle."""
    token_idx = token_idx.cpu()
    ids = inp.topk_ids.cpu()[token_idx].to(torch.int64)
    used = torch.unique(ids)
    remap = torch.full((int(inp.w1.shape[0]),), -1, dtype=torch.int64)
    remap[used] = torch.arange(used.numel())
    dev_used = used.to(inp.w1.device)
    return dict(
        hidden_states=inp.hidden_states.cpu()[token_idx],
        w1=inp.w1[dev_used].cpu(),
        w2=inp.w2[dev_used].cpu(),
        topk_weights=inp.topk_weights.cpu()[token_idx],
        topk_ids=remap[ids].to(torch.int32),
        w1_scale=inp.w1_scale[dev_used].cpu(),
        w2_scale=inp.w2_scale[dev_used].cpu(),
    )
