"""Rotate-half rotary position encoding."""
from __future__ import annotations

import torch

from ..ops import kernels
from .base import DeferredNorm, PositionEncoding
from .registry import register_part


@register_part("position", "rotary_half")
class RotaryHalf(PositionEncoding):
    """Pairs (j, j + rotary_dim/2) are rotated by position * theta^(-2j/rotary_dim)
    (pico_vllm/model.py:80-86,116-123).  Angles, cosines and sines are float32
    and are computed inside the kernel from the position, so there is no table
    whose length bounds the sequence (the reference keeps a [131072, d] table)."""

    graph_safe_prompts = True

    def __init__(self, rotary_dim: int, theta: float, act_dtype: torch.dtype = torch.bfloat16):
        if rotary_dim % 2:
            raise ValueError(f"rotary_dim must be even, got {rotary_dim}")
        self.rotary_dim, self.theta = rotary_dim, theta
        self.inv_freq = None

    def load(self, tensors, device, dtype) -> None:
        d = self.rotary_dim
        # same float32 arithmetic as pico_vllm/model.py:80-82
        inv = 1.0 / (self.theta ** (torch.arange(0, d, 2).float() / d))
        self.inv_freq = inv.to(device).contiguous()

    def table(self, ctx) -> torch.Tensor:
        """cos and sin of every token's angles, [T, rotary_dim / 2, 2]; the first layer of a step
        that asks computes them, the others find them in ``ctx.shared``."""
        key = ("rotary_half", self.rotary_dim, self.theta)
        if key not in ctx.shared:
            ctx.shared[key] = kernels.rope_table(ctx.positions[:ctx.num_tokens], self.inv_freq)
        return ctx.shared[key]

    def rotate_and_store(self, qkv, ctx, kv, block_table, nq, nkv, d) -> None:
        kernels.rope_kv_store(qkv, self.table(ctx), ctx.slot_mapping[kv.group], kv.k, kv.v, nq, nkv, d, self.rotary_dim)

    takes_deferred_norm = True

    def project_rotate_store(self, x, linear, ctx, kv, block_table, nq, nkv, d) -> torch.Tensor:
        fusable = (self.rotary_dim == d and d % 32 == 0 and kv.k.dtype == torch.bfloat16
                   and kv.k.shape[2] & (kv.k.shape[2] - 1) == 0)
        if isinstance(x, DeferredNorm):
            # one token: the norm in front rides on the same kernel
            if fusable and x.kind == "rms" and kernels.skinny_norm_ok(x.resid_in, x.delta, linear.weight):
                q, x.resid = kernels.gemm_skinny_rope_norm(x.resid_in, x.delta, x.weight, x.eps, linear.weight, linear.bias_f32,
                                                           self.table(ctx), ctx.slot_mapping[kv.group], kv.k, kv.v, nq, nkv, d)
                return q
            x = x.run()
        # few tokens in bfloat16: projection, bias, rotation and cache store are one weight-streaming kernel
        if fusable and kernels.skinny_ok(x, linear.weight):
            return kernels.gemm_skinny_rope(x, linear.weight, linear.bias_f32, self.table(ctx), ctx.slot_mapping[kv.group],
                                            kv.k, kv.v, nq, nkv, d)
        return super().project_rotate_store(x, linear, ctx, kv, block_table, nq, nkv, d)


def scaled_frequencies(rotary_dim: int, base: float, scaling=None):
    """(frequencies of the rotary_dim / 2 pairs as float64 list, factor on cosine and sine).

    Plain: f_i = base^(-2i / rotary_dim), factor 1.  ``scaling`` = (factor s, original length L, fast, slow) stretches
    the slow pairs for contexts longer than L: the pair that turns exactly r times within L positions has the
    (real-valued) index d(r) = rotary_dim ln(L / (2 pi r)) / (2 ln base); with lo = max(floor(d(fast)), 0),
    hi = min(ceil(d(slow)), rotary_dim - 1) and ramp_i = clamp((i - lo) / max(hi - lo, 0.001), 0, 1) the frequency is
    f_i / s * ramp_i + f_i * (1 - ramp_i), and cosine and sine are multiplied by 0.1 ln s + 1."""
    import math
    half = rotary_dim // 2
    f = [base ** (-2.0 * i / rotary_dim) for i in range(half)]
    if not scaling:
        return f, 1.0
    s, L, fast, slow = (float(x) for x in scaling)

    def index_of(turns: float) -> float:
        return rotary_dim * math.log(L / (2.0 * math.pi * turns)) / (2.0 * math.log(base))
    lo = max(math.floor(index_of(fast)), 0)
    hi = min(math.ceil(index_of(slow)), rotary_dim - 1)
    out = []
    for i in range(half):
        ramp = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
        out.append(f[i] / s * ramp + f[i] * (1.0 - ramp))
    return out, 0.1 * math.log(s) + 1.0


@register_part("position", "rotary_pairs")
class RotaryPairs(PositionEncoding):
    """Neighbouring entries (2i, 2i + 1) of the first ``rotary_dim`` entries of every head are turned by
    position * f_i; the rest of the head passes unchanged.  Frequencies, optionally scaled for long contexts, as
    ``scaled_frequencies`` gives them.  Angles, cosines and sines are float32, computed on the device from the position
    once a step for all layers that turn alike.  Keys and values may differ in size: the mixer says where q, k and v
    stand in a row and how large they are (``rotate_store``)."""

    graph_safe_prompts = True

    def __init__(self, rotary_dim: int, base: float, scaling=None, act_dtype: torch.dtype = torch.bfloat16):
        if rotary_dim % 2 or rotary_dim < 2:
            raise ValueError(f"rotary_dim must be even and positive, got {rotary_dim}")
        self.rotary_dim, self.base = rotary_dim, float(base)
        self.scaling = tuple(float(x) for x in scaling) if scaling else None
        freqs, self.magnitude = scaled_frequencies(rotary_dim, self.base, self.scaling)
        self._freqs = torch.tensor(freqs, dtype=torch.float64).to(torch.float32)
        self.inv_freq = None

    def load(self, tensors, device, dtype) -> None:
        self.inv_freq = self._freqs.to(device).contiguous()

    def table(self, ctx) -> torch.Tensor:
        key = ("rotary_pairs", self.rotary_dim, self.base, self.scaling)
        if key not in ctx.shared:
            ctx.shared[key] = kernels.rope_table(ctx.positions[:ctx.num_tokens], self.inv_freq, self.magnitude)
        return ctx.shared[key]

    def rotate_store(self, x, q_col, k_col, v_col, ctx, kv, nq, nkv, dk, dv, store: bool = True) -> None:
        """Turn the queries of ``x`` in place (columns q_col ..) and, with ``store``, turn the keys (k_col ..) and write
        them and the values (v_col ..) into the pages of ``kv``."""
        if store:
            kernels.rope_pairs_store(x, q_col, k_col, v_col, self.table(ctx), self.rotary_dim, ctx.slot_mapping[kv.group],
                                     kv.k, kv.v, nq, nkv, dk, dv)
        else:
            kernels.rope_pairs_store(x, q_col, 0, 0, self.table(ctx), self.rotary_dim, None, None, None, nq, nkv, dk, dv)


@register_part("position", "none")
class NoPosition(PositionEncoding):
    """No position encoding: keys and values are stored as they are."""
    graph_safe_prompts = True

    def __init__(self, act_dtype: torch.dtype = torch.bfloat16):
        pass

    def rotate_and_store(self, qkv, ctx, kv, block_table, nq, nkv, d) -> None:
        kernels.rope_kv_store(qkv, None, ctx.slot_mapping[kv.group], kv.k, kv.v, nq, nkv, d, 0)

    def rotate_store(self, x, q_col, k_col, v_col, ctx, kv, nq, nkv, dk, dv, store: bool = True) -> None:
        """Keys and values of different sizes, stored as they are (see ``RotaryPairs.rotate_store``)."""
        if store:
            kernels.rope_pairs_store(x, q_col, k_col, v_col, None, 0, ctx.slot_mapping[kv.group], kv.k, kv.v, nq, nkv, dk, dv)
