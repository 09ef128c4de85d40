"""Learned absolute positions on the residual stream."""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from ..ops import kernels
from .base import StepContext, StreamPart
from .registry import register_part
from .spec import ParamSpec


@register_part("stream", "learned_positions")
class LearnedPositions(StreamPart):
    """resid[t] += table[position of t], in float32; the table has one row per position a request can reach
    (``max_positions``), and a step that would read beyond it is refused where the engine is built
    (``ModelSpec.max_position``)."""
    graph_safe_prompts = True

    def __init__(self, size: int, max_positions: int, name: str = "weight", act_dtype: torch.dtype = torch.bfloat16):
        self.size, self.max_positions, self.name = size, max_positions, name
        self.table: Optional[torch.Tensor] = None

    def param_specs(self) -> List[ParamSpec]:
        return [ParamSpec(self.name, (self.max_positions, self.size))]

    def load(self, tensors: Dict[str, torch.Tensor], device, dtype) -> None:
        self.table = tensors[self.name].to(device).contiguous()

    def weight_bytes(self) -> int:
        return 0                     # a step reads one row a token, not the table

    def forward(self, resid: torch.Tensor, ctx: StepContext) -> torch.Tensor:
        return kernels.add_rows(resid, self.table, ctx.positions[:ctx.num_tokens])
