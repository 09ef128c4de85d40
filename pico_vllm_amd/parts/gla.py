"""Gated linear attention: a recurrent mixer that keeps a matrix per head and request instead of keys and values."""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from ..ops import kernels
from ..ops.linear import Linear
from .base import Mixer, StepContext
from .registry import register_part
from .spec import CacheSpec, ParamSpec


@register_part("mixer", "gated_linear_attention")
class GatedLinearAttention(Mixer):
    """q = x Wq^T dk^(-1/2), k = x Wk^T (heads x dk), v = x Wv^T, g = x Wg^T (heads x dv), and a decay per key channel,

      alpha = sigmoid(z)^(1 / tau),   z = (x Wa1^T) Wa2^T + b        (heads x dk; Wa1 projects to a few dimensions)

    Per head the state S [dk, dv] goes from token to token:  S_t = diag(alpha_t) S_(t-1) + k_t v_t^T,  o_t = S_t^T q_t.
    Every head's o is RMS-normed over its dv entries with one weight [dv] for all heads, the heads side by side are
    multiplied by silu(g), and the output matrix follows.

    The state is float32, starts at zero for a new request and lives in the request's state slot; decays (as logarithms
    log sigmoid(z) / tau), the recurrence and the head norm are float32 in both engines.  One product makes q, k, v, g
    and x Wa1^T.  ``names``: the tensors' names behind the part's prefix."""

    graph_safe_prompts = True

    # In the bfloat16 engine a step with a prompt portion cuts its sequences into chunks of this many tokens that run
    # side by side (``kernels.gla_scan``); decided from the step's shape alone.  The 32-bit engine walks every sequence
    # whole, so that its sums do not depend on how a prompt was cut.
    CHUNK, CHUNKED_FROM = 64, 128

    NAMES = {"q": "q", "k": "k", "v": "v", "g": "g", "o": "o", "norm": "norm", "a1": "a1", "a2": "a2", "a2_bias": "a2.b"}

    def __init__(self, hidden_size: int, num_heads: int, key_dim: int, value_dim: int, tau: float, rank: int, norm_eps: float,
                 names: Optional[Dict[str, str]] = None, act_dtype: torch.dtype = torch.bfloat16):
        if not 1 <= key_dim <= kernels.GLA_MAX_KEY_DIM:
            raise ValueError(f"key size {key_dim} outside what the recurrence kernel takes (1 to {kernels.GLA_MAX_KEY_DIM})")
        if not (tau > 0 and rank >= 1 and value_dim >= 1 and num_heads >= 1):
            raise ValueError("tau must be positive; rank, value size and heads at least 1")
        self.hidden_size, self.heads, self.dk, self.dv = hidden_size, num_heads, key_dim, value_dim
        self.tau, self.rank, self.norm_eps = float(tau), int(rank), float(norm_eps)
        self.names = dict(self.NAMES, **(names or {}))
        self.act_dtype = act_dtype
        self.proj: Optional[Linear] = None               # rows [q | k | v | g | a1]
        self.o: Optional[Linear] = None
        self.a2: Optional[torch.Tensor] = None
        self.a2_bias: Optional[torch.Tensor] = None
        self.norm_weight: Optional[torch.Tensor] = None
        hk, hv = num_heads * key_dim, num_heads * value_dim
        self.q_col, self.k_col, self.v_col, self.g_col, self.a_col = 0, hk, 2 * hk, 2 * hk + hv, 2 * hk + 2 * hv

    def cache_spec(self) -> CacheSpec:
        return CacheSpec("state", state_shape=(self.heads, self.dk, self.dv), state_dtype="float32")

    def flops(self, tokens: int, pairs: int) -> float:
        # the products, the low-rank decay, and per token and head the state's update and its read
        return super().flops(tokens, pairs) + tokens * self.heads * self.dk * (2.0 * self.rank + 5.0 * self.dv)

    def param_specs(self) -> List[ParamSpec]:
        H, n = self.hidden_size, self.names
        hk, hv = self.heads * self.dk, self.heads * self.dv
        return [ParamSpec(n["q"], (hk, H)), ParamSpec(n["k"], (hk, H)), ParamSpec(n["v"], (hv, H)),
                ParamSpec(n["g"], (hv, H)), ParamSpec(n["o"], (H, hv)), ParamSpec(n["norm"], (self.dv,), role="norm"),
                ParamSpec(n["a1"], (self.rank, H)), ParamSpec(n["a2"], (hk, self.rank)),
                ParamSpec(n["a2_bias"], (hk,), role="bias")]

    def load(self, tensors: Dict[str, torch.Tensor], device, dtype) -> None:
        n = self.names
        ws = [tensors[n[x]] for x in ("q", "k", "v", "g", "a1")]
        wdt = torch.float32 if any(w.dtype == torch.float32 for w in ws) else ws[0].dtype
        self.proj = Linear(torch.cat([t.to(wdt) for t in ws], dim=0).to(device))
        self.o = Linear(tensors[n["o"]].to(device))
        self.a2 = tensors[n["a2"]].to(device=device, dtype=wdt).contiguous()
        self.a2_bias = tensors[n["a2_bias"]].to(device=device, dtype=torch.float32).contiguous()
        self.norm_weight = tensors[n["norm"]].to(device=device, dtype=torch.float32).contiguous()

    def weight_bytes(self) -> int:
        return super().weight_bytes() + self.a2.numel() * self.a2.element_size()

    def forward(self, x: torch.Tensor, ctx: StepContext, cache) -> torch.Tensor:
        return self.o.partial(self.mix(x, ctx, cache))

    def forward_into(self, x: torch.Tensor, ctx: StepContext, cache, resid: torch.Tensor) -> None:
        """resid += the mixer's output: with few rows the sum is the epilogue of the output projection."""
        self.o.add_into(self.mix(x, ctx, cache), resid)

    def mix(self, x: torch.Tensor, ctx: StepContext, cache) -> torch.Tensor:
        """The normed and gated heads' outputs [T, H dv] in front of the output projection."""
        y = self.proj(x)                                   # [T, q | k | v | g | a1]
        chunked = self.act_dtype == torch.bfloat16 and not ctx.all_decode and ctx.num_tokens >= self.CHUNKED_FROM
        # a whole walk makes its decays itself (the same arithmetic, one launch less); chunks need them beforehand
        log_decay = kernels.gla_decay(y, self.a_col, self.a2, self.a2_bias, self.tau) if chunked else None
        o = kernels.gla_scan(y, self.q_col, self.k_col, self.v_col, log_decay, ctx.cu_seqlens, ctx.state_slots, cache.state,
                             ctx.num_seqs, self.heads, self.dk, self.dv, self.dk ** -0.5, chunk=self.CHUNK if chunked else 0,
                             decay_from=(self.a_col, self.a2, self.a2_bias, self.tau))
        return kernels.gla_out(o, y, self.g_col, self.norm_weight, self.norm_eps, self.heads, self.dv)
