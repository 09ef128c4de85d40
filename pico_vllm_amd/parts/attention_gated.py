"""Grouped-query attention with an output gate, a cap on the scores, a sliding window that keeps a request's first
positions, keys and values of different sizes, a position encoding of its own choice, and optionally another layer's
keys and values."""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from ..ops import kernels
from ..ops.linear import Linear
from .attention_bias import kv_page_tensors
from .base import Mixer, StepContext
from .registry import build_part, register_part
from .spec import CacheSpec, ParamSpec, PartSpec


@register_part("mixer", "gated_attention")
class GatedAttention(Mixer):
    """q, k, v, g = x Wq^T, x Wk^T, x Wv^T, x Wg^T (one product); the position encoding on q and k;

      score_ij = (q_i . k_j) scale,   then score <- softcap tanh(score / softcap)      (softcap = 0: as it is)
      key j is seen by query i iff j <= i and (no window, or i - j < window, or j < keep_first)

    softmax over the seen keys; the heads' outputs, side by side, times sigmoid(g); then o = a Wo^T.  Query head h reads
    kv head h // (H / G).  Kept first positions keep their true positions (for the rotation).

    ``own_kv`` False: the layer has no Wk and Wv; it is run with another layer's cache (``cache.read_only``), whose keys
    (encoded as that layer stored them) and values it attends over with its own queries, mask and gate.
    ``cache_window`` / ``cache_keep_first``: what the cache has to keep, the layer's own mask or a wider one when other
    layers with other masks read the same cache (a layer and its readers name the same, so their cache needs are equal).

    Keys and values of the new tokens are stored first and attention reads old and new alike from the cache, so a
    prompt cut into portions equals the whole prompt.  ``names``: the tensors' names behind the part's prefix."""

    graph_safe_prompts = True

    NAMES = {"q": "q", "k": "k", "v": "v", "g": "g", "o": "o"}

    def __init__(self, hidden_size: int, num_heads: int, num_kv_heads: int, key_dim: int, value_dim: int, scale: float,
                 position: PartSpec, softcap: float = 0.0, window: int = 0, keep_first: int = 0, gated: bool = True,
                 own_kv: bool = True, cache_window: Optional[int] = None, cache_keep_first: Optional[int] = None,
                 names: Optional[Dict[str, str]] = None, act_dtype: torch.dtype = torch.bfloat16):
        if num_heads % num_kv_heads:
            raise ValueError(f"{num_heads} query heads are not a multiple of {num_kv_heads} kv heads")
        if not (1 <= key_dim <= 1024 and 1 <= value_dim <= 256):
            raise ValueError(f"key size {key_dim} (1 to 1024) or value size {value_dim} (1 to 256) outside what the kernels take")
        if window < 0 or keep_first < 0 or softcap < 0:
            raise ValueError("window, kept first positions and the cap must not be negative")
        self.hidden_size, self.nq, self.nkv, self.dk, self.dv = hidden_size, num_heads, num_kv_heads, key_dim, value_dim
        self.scale, self.softcap, self.window, self.keep_first = float(scale), float(softcap), int(window), int(keep_first)
        self.gated, self.own_kv = bool(gated), bool(own_kv)
        self.cache_window = self.window if cache_window is None else int(cache_window)
        self.cache_keep_first = self.keep_first if cache_keep_first is None else int(cache_keep_first)
        if self.cache_window and (not self.window or self.window > self.cache_window or self.keep_first > self.cache_keep_first):
            raise ValueError("the cache would keep less than this layer's mask reads")
        # what the attention kernels of this package call these (no distance penalty, no query temperature)
        self.temp_coef, self.temp_every, self.slope_span = 0.0, 0, 0.0
        self.names = dict(self.NAMES, **(names or {}))
        self.act_dtype = act_dtype
        self.position = build_part("position", position, act_dtype=act_dtype)
        self.proj: Optional[Linear] = None               # rows [q | k | v | g] (own_kv) or [q | g]
        self.o: Optional[Linear] = None
        self.fast = None                                 # matrix-core kernel, chosen at load
        # a gate's columns start on 8 bytes for the matrix-core kernel: q, k, v blocks are padded to multiples of 4
        self.q_col = 0
        nqk = self.nq * self.dk
        if self.own_kv:
            self.k_col = nqk
            self.v_col = self.k_col + self.nkv * self.dk
            self.g_col = self.v_col + self.nkv * self.dv
        else:
            self.k_col = self.v_col = 0
            self.g_col = nqk

    def cache_spec(self) -> CacheSpec:
        return CacheSpec("paged_kv", window=self.cache_window, keep_first=self.cache_keep_first if self.cache_window else 0,
                         page_tensors=kv_page_tensors(self.nkv, self.dk, self.dv))

    def flops(self, tokens: int, pairs: int) -> float:
        return super().flops(tokens, pairs) + 2.0 * self.nq * (self.dk + self.dv) * pairs

    def _blocks(self) -> List[tuple]:
        """(name, rows) of the matrices that make the one product, in row order."""
        out = [("q", self.nq * self.dk)]
        if self.own_kv:
            out += [("k", self.nkv * self.dk), ("v", self.nkv * self.dv)]
        if self.gated:
            out.append(("g", self.nq * self.dv))
        return out

    def param_specs(self) -> List[ParamSpec]:
        H, n = self.hidden_size, self.names
        out = [ParamSpec(n[x], (rows, H)) for x, rows in self._blocks()]
        out.append(ParamSpec(n["o"], (H, self.nq * self.dv)))
        return out + [ParamSpec("position." + p.name, p.shape, p.role, p.std) for p in self.position.param_specs()]

    def load(self, tensors: Dict[str, torch.Tensor], device, dtype) -> None:
        n = self.names
        ws = [tensors[n[x]] for x, _ in self._blocks()]
        wdt = torch.float32 if any(w.dtype == torch.float32 for w in ws) else ws[0].dtype
        self.proj = Linear(torch.cat([t.to(wdt) for t in ws], dim=0).to(device))
        self.o = Linear(tensors[n["o"]].to(device))
        self.position.load({k[len("position."):]: v for k, v in tensors.items() if k.startswith("position.")}, device, dtype)
        if self.act_dtype == torch.bfloat16 and (not self.gated or self.g_col % 4 == 0):
            from ..ops import attention_bias_fast
            self.fast = attention_bias_fast.choose(self)

    def graph_variant(self, ctx: StepContext) -> tuple:
        own = (("gated_attention",) + self.fast.plan(ctx),) if self.fast is not None else ()
        return own + super().graph_variant(ctx)

    def forward(self, x: torch.Tensor, ctx: StepContext, cache) -> torch.Tensor:
        return self.o.partial(self.attend(x, ctx, cache))

    def forward_into(self, x: torch.Tensor, ctx: StepContext, cache, resid: torch.Tensor) -> None:
        """resid += the mixer's output: with few rows the sum is the epilogue of the output projection."""
        self.o.add_into(self.attend(x, ctx, cache), resid)

    def attend(self, x: torch.Tensor, ctx: StepContext, cache) -> torch.Tensor:
        """The gated heads' outputs [T, H dv] in front of the output projection."""
        reads_other = bool(getattr(cache, "read_only", False))
        if reads_other == self.own_kv:
            raise RuntimeError("a layer with keys and values of its own runs on its own cache, one without on another layer's")
        bt = ctx.block_tables[cache.group]
        y = self.proj(x)                                   # [T, q | k | v | g]
        self.position.rotate_store(y, self.q_col, self.k_col, self.v_col, ctx, cache, self.nq, self.nkv, self.dk, self.dv,
                                   store=self.own_kv)
        gate = y[:, self.g_col:] if self.gated else None
        if self.fast is not None and cache.k.dtype == torch.bfloat16:
            return self.fast(y, cache, bt, ctx, gate=gate)
        return kernels.attn_bias_plain(y, cache.k, cache.v, bt, ctx.positions, ctx.token_seq, self.nq, self.nkv, self.dk,
                                       self.dv, self.scale, self.window, softcap=self.softcap, keep_first=self.keep_first,
                                       gate=gate)
