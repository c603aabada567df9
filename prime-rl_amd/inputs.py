"""Seeded synthetic workloads for the INT8 MoE layer: shapes, weights, activations and routing.

Data is drawn on the CPU from one ``torch.Generator`` so that a CPU checker and the GPU path see
identical bits, then moved to the requested device.  For layers whose weights would not be worth
holding twice (tens of GB) the int8 weights can be drawn on the device instead
(``weights_on_device=True``); such workloads are only checked through sampled rows.

Routing follows the reference's router (``trainer/models/layers/moe.py:254-298``): scores in fp32,
top-k, gather the unbiased scores, renormalise with ``+1e-20``.
"""

from __future__ import annotations

import dataclasses
import math

import torch

__all__ = ["LayerShape", "SHAPES", "MoEInputs", "make_inputs", "route", "algorithmic_bytes", "algorithmic_ops"]


@dataclasses.dataclass(frozen=True)
class LayerShape:
    name: str
    E: int  # routed experts
    k: int  # routed experts per token
    H: int  # hidden size
    I: int  # expert intermediate size
    routing: str = "softmax"  # softmax | zipf | grouped
    shared_expert: bool = False  # one always-on expert appended as id E with weight 1.0
    n_group: int = 1
    topk_group: int = 1

    @property
    def E_total(self) -> int:
        return self.E + (1 if self.shared_expert else 0)

    @property
    def k_total(self) -> int:
        return self.k + (1 if self.shared_expert else 0)


SHAPES = {
    "toy": LayerShape("toy", E=8, k=2, H=1024, I=2816),
    "qwen3-30b-a3b": LayerShape("qwen3-30b-a3b", E=128, k=8, H=2048, I=768),
    "glm-4.5-air": LayerShape("glm-4.5-air", E=128, k=8, H=4096, I=1408, routing="zipf", shared_expert=True),
    "deepseek-v3": LayerShape("deepseek-v3", E=256, k=8, H=7168, I=2048, routing="grouped", n_group=8, topk_group=4),
}


@dataclasses.dataclass
class MoEInputs:
    shape: LayerShape
    hidden_states: torch.Tensor  # bf16 [M, H]
    w1: torch.Tensor  # int8 [E', 2I, H]
    w2: torch.Tensor  # int8 [E', H, I]
    w1_scale: torch.Tensor  # fp32 [E', 2I]
    w2_scale: torch.Tensor  # fp32 [E', H]
    topk_weights: torch.Tensor  # fp32 [M, k']
    topk_ids: torch.Tensor  # int32 [M, k']

    def to(self, device) -> "MoEInputs":
        return dataclasses.replace(
            self, **{f.name: getattr(self, f.name).to(device) for f in dataclasses.fields(self) if f.name != "shape"}
        )

    def fused_experts_args(self) -> tuple:
        return (self.hidden_states, self.w1, self.w2, self.topk_weights, self.topk_ids)

    def fused_experts_kwargs(self) -> dict:
        return dict(use_int8_w8a8=True, per_channel_quant=True, w1_scale=self.w1_scale, w2_scale=self.w2_scale)


def _renorm(w: torch.Tensor) -> torch.Tensor:
    return w / (w.sum(dim=-1, keepdim=True) + 1e-20)


def route(shape: LayerShape, M: int, gen: torch.Generator) -> tuple[torch.Tensor, torch.Tensor]:
    """Router outputs ``(topk_weights fp32 [M, k'], topk_ids int32 [M, k'])`` for ``M`` tokens."""
    E, k = shape.E, shape.k
    logits = torch.randn((M, E), generator=gen, dtype=torch.float32)
    if shape.routing == "softmax":
        scores = torch.softmax(logits, dim=1)
        ids = torch.topk(scores, k, dim=1)[1]
        w = _renorm(scores.gather(1, ids))
    elif shape.routing == "zipf":
        # expert popularity p_e ∝ rank^-1.2 under a fixed random permutation of the ranks
        ranks = torch.randperm(E, generator=gen).to(torch.float32) + 1.0
        scores = torch.softmax(logits + (-1.2) * torch.log(ranks).reshape(1, E), dim=1)
        ids = torch.topk(scores, k, dim=1)[1]
        w = _renorm(scores.gather(1, ids))
    elif shape.routing == "grouped":
        bias = torch.randn((E,), generator=gen, dtype=torch.float32) * 0.1
        s = torch.sigmoid(logits)
        sb = s + bias.reshape(1, E)
        per = E // shape.n_group
        group_score = sb.view(M, shape.n_group, per).topk(2, dim=-1)[0].sum(dim=-1)
        keep = group_score.topk(shape.topk_group, dim=-1)[1]
        gmask = torch.zeros((M, shape.n_group), dtype=torch.bool).scatter_(1, keep, True)
        mask = gmask.unsqueeze(-1).expand(M, shape.n_group, per).reshape(M, E)
        ids = sb.masked_fill(~mask, float("-inf")).topk(k, dim=-1)[1]
        w = _renorm(s.gather(1, ids))
    else:
        raise ValueError(shape.routing)
    ids = ids.to(torch.int32)
    w = w.to(torch.float32)
    if shape.shared_expert:
        ids = torch.cat([ids, torch.full((M, 1), E, dtype=torch.int32)], dim=1)
        w = torch.cat([w, torch.ones((M, 1), dtype=torch.float32)], dim=1)
    return w.contiguous(), ids.contiguous()


def make_inputs(
    shape: LayerShape | str,
    M: int,
    seed: int = 0,
    device: str | torch.device = "cpu",
    weights_on_device: bool = False,
) -> MoEInputs:
    """Weights uniform in [-127, 127], channel scales U(0.002, 0.01), activations N(0, 1) in bf16."""
    if isinstance(shape, str):
        shape = SHAPES[shape]
    gen = torch.Generator(device="cpu").manual_seed(seed)
    Et, H, I = shape.E_total, shape.H, shape.I
    w1_scale = torch.empty((Et, 2 * I), dtype=torch.float32).uniform_(0.002, 0.01, generator=gen)
    w2_scale = torch.empty((Et, H), dtype=torch.float32).uniform_(0.002, 0.01, generator=gen)
    x = torch.randn((M, H), generator=gen, dtype=torch.float32).to(torch.bfloat16)
    tw, ids = route(shape, M, gen)
    if weights_on_device:
        dgen = torch.Generator(device=device).manual_seed(seed)
        w1 = torch.randint(-127, 128, (Et, 2 * I, H), generator=dgen, dtype=torch.int8, device=device)
        w2 = torch.randint(-127, 128, (Et, H, I), generator=dgen, dtype=torch.int8, device=device)
    else:
        w1 = torch.randint(-127, 128, (Et, 2 * I, H), generator=gen, dtype=torch.int8)
        w2 = torch.randint(-127, 128, (Et, H, I), generator=gen, dtype=torch.int8)
    inp = MoEInputs(shape, x, w1, w2, w1_scale, w2_scale, tw, ids)
    return inp.to(device)


def algorithmic_bytes(shape: LayerShape, M: int, topk_ids: torch.Tensor) -> int:
    """HBM bytes one layer call has to move: int8 weights and fp32 channel scales of the experts
    that are actually routed to, bf16 activations in and out, routing ids and weights."""
    n_act = int(torch.unique(topk_ids).numel())
    return n_act * (3 * shape.I * shape.H + 4 * (2 * shape.I + shape.H)) + 4 * M * shape.H + 8 * M * topk_ids.shape[1]


def algorithmic_ops(shape: LayerShape, M: int) -> int:
    """int8 multiply-accumulate operations (2 per MAC) of one layer call, padding rows excluded."""
    return 6 * M * shape.k_total * shape.I * shape.H
