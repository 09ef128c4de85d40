"""Grouped-query attention whose positions enter through the scores: a linear distance penalty per head, a query
temperature that grows with the position, an optional sliding window, keys and values of different sizes, and values
mixed with those of an earlier layer."""
from __future__ import annotations

import dataclasses
from typing import Dict, List, Optional

import torch

from ..ops import kernels
from ..ops.linear import Linear
from .base import Mixer, StepContext
from .registry import register_part
from .spec import CacheSpec, PageTensor, ParamSpec

# the penalty's slopes fall from 2^(-span / H) to 2^(-span) over the H heads
SLOPE_SPAN = 8.0


def kv_page_tensors(num_kv_heads: int, key_dim: int, value_dim: int):
    """A page keeps a token's key contiguous ([kv heads, page, key size]) and, of every value dimension, the page's
    tokens ([kv heads, value size, page]): the matrix-core kernels contract the values over keys."""
    return (PageTensor("k", (num_kv_heads, "page", key_dim)), PageTensor("v", (num_kv_heads, value_dim, "page")))


@register_part("mixer", "distance_bias_attention")
class DistanceBiasAttention(Mixer):
    """q, k, v = x Wq^T + bq, x Wk^T + bk, x Wv^T + bv (one product); no rotation.

      score_ij = (q_i . k_j) scale temp(i) - slope_h (i - j)      for keys j <= i, and i - j < window if there is one
      temp(i)  = 1 + temp_coef ln(floor((i + 1) / temp_every) + 1)   (temp_every = 0: 1)
      slope_h  = 2^(-slope_span (h + 1) / H)                         (slope_span = 0: none)

    softmax over the visible keys, then o = a Wo^T + bo.  Query head h reads kv head h // (H / G).

    ``value_mix``: "source" keeps this layer's values of the step's tokens for later layers (under ``mix_key`` in the
    step's shared record); "mix" replaces v by (1 - lambda) v + lambda v_source before it is stored, lambda a learned
    scalar.  The mixed value is what the cache holds.  A "source" layer may own a lambda tensor it never uses
    (``unused_mix_tensor``), as checkpoints of designs that give every such layer one do.

    Keys and values of the new tokens are stored first and attention reads old and new alike from the cache, so a
    prompt cut into portions equals the whole prompt.  ``names``: the tensors' names behind the part's prefix."""

    graph_safe_prompts = True

    NAMES = {"q": "q", "k": "k", "v": "v", "o": "o", "q_bias": "q.b", "k_bias": "k.b", "v_bias": "v.b", "o_bias": "o.b",
             "mix": "vmix"}

    def __init__(self, hidden_size: int, num_heads: int, num_kv_heads: int, key_dim: int, value_dim: int, scale: float,
                 window: int = 0, temp_coef: float = 0.0, temp_every: int = 0, slope_span: float = SLOPE_SPAN,
                 proj_bias: bool = True, out_bias: bool = True, value_mix: Optional[str] = None,
                 mix_key: str = "value_mix", unused_mix_tensor: bool = False, names: Optional[Dict[str, str]] = None,
                 act_dtype: torch.dtype = torch.bfloat16):
        if num_heads % num_kv_heads:
            raise ValueError(f"{num_heads} query heads are not a multiple of {num_kv_heads} kv heads")
        if not (1 <= key_dim <= 1024 and 1 <= value_dim <= 256):
            raise ValueError(f"key size {key_dim} (1 to 1024) or value size {value_dim} (1 to 256) outside what the kernels take")
        if window < 0 or temp_every < 0 or slope_span < 0:
            raise ValueError("window, temperature interval and slope span must not be negative")
        if value_mix not in (None, "source", "mix"):
            raise ValueError(f"value_mix is None, 'source' or 'mix', got {value_mix!r}")
        self.hidden_size, self.nq, self.nkv, self.dk, self.dv = hidden_size, num_heads, num_kv_heads, key_dim, value_dim
        self.scale, self.window = float(scale), int(window)
        self.temp_coef, self.temp_every, self.slope_span = float(temp_coef), int(temp_every), float(slope_span)
        self.proj_bias, self.out_bias, self.value_mix, self.mix_key = proj_bias, out_bias, value_mix, mix_key
        self.unused_mix_tensor = unused_mix_tensor
        self.names = dict(self.NAMES, **(names or {}))
        self.act_dtype = act_dtype
        self.qkv: Optional[Linear] = None
        self.o: Optional[Linear] = None
        self.mix = 0.0
        self.fast = None                                 # matrix-core kernels, chosen at load
        self.k_col = self.nq * self.dk
        self.v_col = self.k_col + self.nkv * self.dk

    def cache_spec(self) -> CacheSpec:
        return CacheSpec("paged_kv", window=self.window, page_tensors=kv_page_tensors(self.nkv, self.dk, self.dv))

    def flops(self, tokens: int, pairs: int) -> float:
        return super().flops(tokens, pairs) + 2.0 * self.nq * (self.dk + self.dv) * pairs

    def param_specs(self) -> List[ParamSpec]:
        H, nq, nkv, dk, dv, n = self.hidden_size, self.nq, self.nkv, self.dk, self.dv, self.names
        out = [ParamSpec(n["q"], (nq * dk, H)), ParamSpec(n["k"], (nkv * dk, H)), ParamSpec(n["v"], (nkv * dv, H)),
               ParamSpec(n["o"], (H, nq * dv))]
        if self.proj_bias:
            out += [ParamSpec(n["q_bias"], (nq * dk,), role="bias"), ParamSpec(n["k_bias"], (nkv * dk,), role="bias"),
                    ParamSpec(n["v_bias"], (nkv * dv,), role="bias")]
        if self.out_bias:
            out.append(ParamSpec(n["o_bias"], (H,), role="bias"))
        if self.value_mix == "mix" or (self.value_mix == "source" and self.unused_mix_tensor):
            out.append(ParamSpec(n["mix"], (), role="bias"))
        return out

    def load(self, tensors: Dict[str, torch.Tensor], device, dtype) -> None:
        n = self.names
        ws = [tensors[n[x]] for x in "qkv"]
        wdt = torch.float32 if any(w.dtype == torch.float32 for w in ws) else ws[0].dtype
        b = None
        if self.proj_bias:
            b = torch.cat([tensors[n[x + "_bias"]].float() for x in "qkv"], dim=0).to(device)
        self.qkv = Linear(torch.cat([t.to(wdt) for t in ws], dim=0).to(device), b)
        self.o = Linear(tensors[n["o"]].to(device), tensors[n["o_bias"]].float().to(device) if self.out_bias else None)
        if self.value_mix == "mix":
            self.mix = float(tensors[n["mix"]].float().item())
        if self.act_dtype == torch.bfloat16:
            from ..ops import attention_bias_fast
            self.fast = attention_bias_fast.choose(self)

    def graph_variant(self, ctx: StepContext) -> tuple:
        own = (("distance_bias_attention",) + self.fast.plan(ctx),) if self.fast is not None else ()
        return own + super().graph_variant(ctx)

    def forward(self, x: torch.Tensor, ctx: StepContext, cache) -> torch.Tensor:
        return self.o(self.attend(x, ctx, cache))

    def forward_into(self, x: torch.Tensor, ctx: StepContext, cache, resid: torch.Tensor) -> None:
        """resid += the mixer's output: with few rows the sum is the epilogue of the output projection."""
        self.o.add_into(self.attend(x, ctx, cache), resid)

    def attend(self, x: torch.Tensor, ctx: StepContext, cache) -> torch.Tensor:
        """The heads' outputs [T, H dv] in front of the output projection."""
        bt = ctx.block_tables[cache.group]
        if getattr(cache, "read_only", False):
            # another run's keys and values: nothing is stored, every token's slot reads as "none"
            if "no_slots" not in ctx.shared:
                ctx.shared["no_slots"] = torch.full_like(ctx.slot_mapping[cache.group], -1)
            ctx = dataclasses.replace(ctx, slot_mapping=[ctx.shared["no_slots"]] * len(ctx.slot_mapping))
        qkv = self.qkv(x)                                  # [T, H dk + G dk + G dv]
        v_first = None
        if self.value_mix == "mix":
            try:
                v_first = ctx.shared[("value_mix", self.mix_key)]
            except KeyError:
                raise RuntimeError(f"no earlier layer of this step kept values under {self.mix_key!r}") from None
        elif self.value_mix == "source":
            ctx.shared[("value_mix", self.mix_key)] = qkv[:, self.v_col:]
        kernels.kv_mix_store(qkv, self.k_col, self.v_col, ctx.slot_mapping[cache.group], cache.k, cache.v,
                             self.nkv, self.dk, self.dv, v_first, self.mix)
        if self.fast is not None and cache.k.dtype == torch.bfloat16:
            a = self.fast(qkv, cache, bt, ctx)
        else:
            a = kernels.attn_bias_plain(qkv, cache.k, cache.v, bt, ctx.positions, ctx.token_seq, self.nq, self.nkv,
                                        self.dk, self.dv, self.scale, self.window, self.temp_coef, self.temp_every,
                                        self.slope_span)
        return a
