"""A routed feed-forward: every token runs a few of many small gated feed-forwards."""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from ..ops import kernels
from ..ops.linear import Linear
from .base import FeedForward, StepContext
from .registry import register_part
from .spec import ParamSpec

# the gate's activation is g sigmoid(ACT_ALPHA g)
ACT_ALPHA = 1.702


@register_part("feed_forward", "routed_experts")
class RoutedExperts(FeedForward):
    """Router: z = x Wr^T in float32, scores s = sigmoid(z); a token's ``top`` experts are those with the largest
    scores, its weights their scores as they are (not renormalised).

    Expert e on a row r: g = min(Wg_e r, limit), u = clamp(Wu_e r, -limit, limit), y = g sigmoid(alpha g) (u + 1),
    out = Wd_e y; no biases.  The weight scales the expert's INPUT: a token's output is sum_e expert_e(s_e x).

    The checkpoint holds every expert's three matrices apart (``expert_names`` with the expert's number filled in); they
    are stacked at load: gate_up [E, 2 F, D], down [E, D, F].  Everything a step decides (which experts, which rows) is
    decided on the device."""
    graph_safe_prompts = True

    def __init__(self, hidden_size: int, expert_size: int, num_experts: int, top: int, limit: float,
                 act_alpha: float = ACT_ALPHA, router_name: str = "router",
                 expert_names: tuple = ("e{}.gate", "e{}.up", "e{}.down"), act_dtype: torch.dtype = torch.bfloat16):
        if not 1 <= top <= min(num_experts, kernels.MOE_MAX_TOP):
            raise ValueError(f"{top} experts per token of {num_experts} (at most {kernels.MOE_MAX_TOP})")
        if not limit > 0:
            raise ValueError(f"the experts' limit must be positive, got {limit}")
        self.hidden_size, self.expert_size, self.num_experts, self.top = hidden_size, expert_size, num_experts, top
        self.limit, self.act_alpha = float(limit), float(act_alpha)
        self.router_name, self.expert_names = router_name, tuple(expert_names)
        self.act_dtype = act_dtype
        self.router: Optional[Linear] = None
        self.gate_up: Optional[Linear] = None       # [E * 2 F, D]: as a matrix, so that reports count its bytes
        self.down: Optional[Linear] = None          # [E * D, F]

    def param_specs(self) -> List[ParamSpec]:
        D, F = self.hidden_size, self.expert_size
        g, u, d = self.expert_names
        out = [ParamSpec(self.router_name, (self.num_experts, D))]
        for e in range(self.num_experts):
            out += [ParamSpec(g.format(e), (F, D)), ParamSpec(u.format(e), (F, D)), ParamSpec(d.format(e), (D, F))]
        return out

    def load(self, tensors: Dict[str, torch.Tensor], device, dtype) -> None:
        g, u, d = self.expert_names
        E = self.num_experts
        self.router = Linear(tensors[self.router_name].float().to(device))      # routed in float32 in both engines
        ws = [tensors[n.format(e)] for e in range(E) for n in (g, u)]
        wdt = torch.float32 if dtype == torch.float32 or any(w.dtype == torch.float32 for w in ws) else torch.bfloat16
        self.gate_up = Linear(torch.cat([w.to(wdt) for w in ws], dim=0).to(device))
        self.down = Linear(torch.cat([tensors[d.format(e)].to(wdt) for e in range(E)], dim=0).to(device))

    def weight_bytes(self) -> int:
        # what a step of one token streams: the router and ``top`` experts
        per = (self.gate_up.weight.numel() + self.down.weight.numel()) * self.gate_up.weight.element_size() // self.num_experts
        return self.router.weight.numel() * 4 + self.top * per

    def flops(self, tokens: int, pairs: int) -> float:
        D, F = self.hidden_size, self.expert_size
        return 2.0 * tokens * (self.num_experts * D + self.top * 3 * F * D)

    def forward(self, x: torch.Tensor, ctx: StepContext) -> torch.Tensor:
        E, F, D = self.num_experts, self.expert_size, self.hidden_size
        experts, weights = kernels.moe_router(x, self.router.weight, self.top)
        gate_up = self.gate_up.weight.view(E, 2 * F, D)
        down = self.down.weight.view(E, D, F)
        if x.dtype != gate_up.dtype:
            x = x.to(gate_up.dtype)
        if kernels.moe_fast_ok(x, gate_up, down):
            # few rows stream their experts' matrices; many are sorted by expert and go to the matrix cores.  The
            # second gives one float32 slab a slot: the next norm adds them up
            return kernels.moe_experts(x, gate_up, down, experts, weights, self.limit, self.act_alpha)
        return kernels.moe_experts_plain(x, gate_up, down, experts, weights, self.limit, self.act_alpha)

    def graph_variant(self, ctx: StepContext) -> tuple:
        return (("routed_experts", kernels.moe_grouped_rows(ctx.num_tokens, self.top)),)
