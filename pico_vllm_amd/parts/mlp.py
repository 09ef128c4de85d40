"""Dense feed-forwards: SwiGLU, squared ReLU, and none at all."""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from ..ops.linear import Linear
from .base import FeedForward, StepContext
from .registry import register_part
from .spec import ParamSpec


@register_part("feed_forward", "swiglu_mlp")
class SwiGLUMLP(FeedForward):
    """down( silu(gate) * up ), [gate; up] = x Wgu^T, no biases
    (pico_vllm/model.py:309-318; gate rows first, weights.py:58).  The
    checkpoint holds gate_proj and up_proj separately; they are concatenated
    at load so one GEMM makes both."""

    takes_deferred_norm = True      # Linear.swiglu runs or fuses it
    graph_safe_prompts = True

    def __init__(self, hidden_size: int, intermediate_size: int, act_dtype: torch.dtype = torch.bfloat16,
                 names: tuple = ("gate_proj.weight", "up_proj.weight", "down_proj.weight")):
        # names: the three matrices' names behind the part's prefix (gate, up, down)
        self.hidden_size, self.intermediate_size = hidden_size, intermediate_size
        self.names = tuple(names)
        self.gate_up: Optional[Linear] = None
        self.down: Optional[Linear] = None

    def param_specs(self) -> List[ParamSpec]:
        H, I = self.hidden_size, self.intermediate_size
        g, u, d = self.names
        return [ParamSpec(g, (I, H)), ParamSpec(u, (I, H)), ParamSpec(d, (H, I))]

    def load(self, tensors: Dict[str, torch.Tensor], device, dtype) -> None:
        g, u = tensors[self.names[0]], tensors[self.names[1]]
        wdt = torch.float32 if torch.float32 in (g.dtype, u.dtype) else g.dtype
        self.gate_up = Linear(torch.cat([g.to(wdt), u.to(wdt)], dim=0).to(device))
        self.down = Linear(tensors[self.names[2]].to(device))

    def forward(self, x: torch.Tensor, ctx: StepContext) -> torch.Tensor:
        return self.down.partial(self.gate_up.swiglu(x))


@register_part("feed_forward", "relu2_mlp")
class Relu2MLP(FeedForward):
    """down( relu(up x)^2 ), no biases.  ``names``: the two matrices' names behind the part's prefix."""
    graph_safe_prompts = True

    def __init__(self, hidden_size: int, intermediate_size: int, up_name: str = "up", down_name: str = "down",
                 act_dtype: torch.dtype = torch.bfloat16):
        self.hidden_size, self.intermediate_size = hidden_size, intermediate_size
        self.up_name, self.down_name = up_name, down_name
        self.up: Optional[Linear] = None
        self.down: Optional[Linear] = None

    def param_specs(self) -> List[ParamSpec]:
        H, I = self.hidden_size, self.intermediate_size
        return [ParamSpec(self.up_name, (I, H)), ParamSpec(self.down_name, (H, I))]

    def load(self, tensors: Dict[str, torch.Tensor], device, dtype) -> None:
        self.up = Linear(tensors[self.up_name].to(device))
        self.down = Linear(tensors[self.down_name].to(device))

    def forward(self, x: torch.Tensor, ctx: StepContext) -> torch.Tensor:
        return self.down.partial(self.up.relu2(x))


@register_part("feed_forward", "none")
class NoFeedForward(FeedForward):
    """A layer without a feed-forward: contributes nothing (``forward`` returns None, which an arrangement that
    allows it takes as "no delta")."""
    graph_safe_prompts = True

    def __init__(self, act_dtype: torch.dtype = torch.bfloat16):
        pass

    def forward(self, x, ctx):
        return None
