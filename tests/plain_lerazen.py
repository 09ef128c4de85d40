"""A plain, slow implementation of the Lerazen decoder: whole sequences, no cache, one function per mechanism,
float64 by default.  It shares no code with the engine; the tests compare the engine with it.

A model is (config, tensors): ``config`` is what config.json holds, ``tensors`` maps checkpoint names to torch
tensors.  Notation: n tokens, width D, query heads H, key/value heads G, query/key size dk, value size dv.
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional

import torch


def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """x / sqrt(mean(x^2) + eps) * weight over the last axis."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * weight


def embed_tokens(tokens, embed: torch.Tensor, pos: torch.Tensor, first_position: int = 0) -> torch.Tensor:
    """Row of the token plus the learned row of its position (positions count from ``first_position``)."""
    ids = torch.as_tensor(list(tokens), dtype=torch.long)
    places = torch.arange(first_position, first_position + len(ids))
    return embed[ids] + pos[places]


def head_slopes(heads: int) -> torch.Tensor:
    """Slope of head h (0-based) of the distance penalty: 2^(-8 (h + 1) / heads)."""
    return torch.tensor([2.0 ** (-8.0 * (h + 1) / heads) for h in range(heads)], dtype=torch.float64)


def query_temperature(position: int, coef: float, every: int) -> float:
    """1 + coef ln(floor((p + 1) / every) + 1)."""
    return 1.0 + coef * math.log((position + 1) // every + 1)


def visible(i: int, j: int, window: Optional[int]) -> bool:
    """Query i sees key j: never the future, and with a window only the last ``window`` positions, itself included."""
    return 0 <= i - j and (window is None or i - j < window)


def attention_scores(q: torch.Tensor, k: torch.Tensor, scale: float, slopes: torch.Tensor,
                     window: Optional[int]) -> torch.Tensor:
    """Softmax weights [H, n, n] from q [n, H, dk] and k [n, G, dk]: (q . k) scale - slope_h (i - j) over visible keys."""
    n, H, _ = q.shape
    G = k.shape[1]
    out = torch.zeros(H, n, n, dtype=q.dtype)
    for h in range(H):
        g = h // (H // G)
        for i in range(n):
            js = [j for j in range(n) if visible(i, j, window)]
            s = torch.stack([(q[i, h] * k[j, g]).sum() * scale - slopes[h].to(q.dtype) * (i - j) for j in js])
            out[h, i, js] = torch.softmax(s, 0)
    return out


def attention_scores_fast(q, k, scale, slopes, window):
    """The same as ``attention_scores`` with matrix operations (for sequences of hundreds of tokens)."""
    n, H, _ = q.shape
    G = k.shape[1]
    kk = k.repeat_interleave(H // G, dim=1)                       # head h reads group h // (H / G)
    s = torch.einsum("ihd,jhd->hij", q, kk) * scale
    i = torch.arange(n)[:, None]
    j = torch.arange(n)[None, :]
    dist = (i - j)
    s = s - slopes.to(q.dtype)[:, None, None] * dist.to(q.dtype)
    ok = dist >= 0
    if window is not None:
        ok = ok & (dist < window)
    s = s.masked_fill(~ok, float("-inf"))
    return torch.softmax(s, -1)


def attention_mixer(h: torch.Tensor, w: Dict[str, torch.Tensor], m: dict, v_first: Optional[torch.Tensor],
                    first_position: int = 0, fast: bool = True):
    """The attention mixer on normed rows h [n, D].  ``w``: the mixer's tensors by their names behind 'mix.'.
    ``v_first``: the values [n, G, dv] of the first value-mixing layer, or None if this layer is that one (or
    mixes nothing).  Returns (output [n, D], the values this layer attends over)."""
    n = h.shape[0]
    H, G, dk, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (h @ w["q"].T + w["q.b"]).view(n, H, dk)
    k = (h @ w["k"].T + w["k.b"]).view(n, G, dk)
    v = (h @ w["v"].T + w["v.b"]).view(n, G, dv)
    qt = m.get("q_temp")
    if qt:
        t = torch.tensor([query_temperature(first_position + i, qt["coef"], qt["every"]) for i in range(n)], dtype=h.dtype)
        q = q * t[:, None, None]
    if m.get("v_mix") and v_first is not None:
        lam = w["vmix"].to(h.dtype)
        v = (1 - lam) * v + lam * v_first
    window = (m.get("mask") or {}).get("size")
    f = attention_scores_fast if fast else attention_scores
    p = f(q, k, m["scale"], head_slopes(H), window)               # [H, n, n]
    vv = v.repeat_interleave(H // G, dim=1)                       # [n, H, dv]
    a = torch.einsum("hij,jhd->ihd", p, vv).reshape(n, H * dv)
    return a @ w["o"].T + w["o.b"], v


def dense_ff(h: torch.Tensor, w: Dict[str, torch.Tensor]) -> torch.Tensor:
    """down(relu(up h)^2)."""
    return torch.relu(h @ w["up"].T) ** 2 @ w["down"].T


def expert_ff(x: torch.Tensor, gate: torch.Tensor, up: torch.Tensor, down: torch.Tensor, limit: float) -> torch.Tensor:
    """g = min(gate x, limit); u = clamp(up x, -limit, limit); down(g sigmoid(1.702 g) (u + 1))."""
    g = torch.clamp(x @ gate.T, max=limit)
    u = torch.clamp(x @ up.T, -limit, limit)
    return (g * torch.sigmoid(1.702 * g) * (u + 1)) @ down.T


def route(h: torch.Tensor, router: torch.Tensor, top: int):
    """(experts [n, top], weights [n, top]): the ``top`` largest sigmoid scores of every token, as they are."""
    s = torch.sigmoid(h @ router.T)
    weights, experts = torch.topk(s, top, dim=-1)
    return experts, weights


def router_margins(h: torch.Tensor, router: torch.Tensor, top: int) -> torch.Tensor:
    """How far every token's choice is from being another: the gap between its last chosen and its first rejected
    router logit, in units of the logits' spread (infinite where every expert is chosen)."""
    z = h @ router.T
    if top >= z.shape[-1]:
        return torch.full((h.shape[0],), float("inf"), dtype=h.dtype)
    s, _ = torch.sort(z, -1, descending=True)
    return (s[:, top - 1] - s[:, top]) / z.std()


def moe_ff(h: torch.Tensor, w: Dict[str, torch.Tensor], mlp: dict) -> torch.Tensor:
    """Sum over a token's chosen experts of expert(weight * h)."""
    experts, weights = route(h, w["router"], mlp["router"]["top"])
    out = torch.zeros_like(h)
    for i in range(h.shape[0]):
        for e, s in zip(experts[i].tolist(), weights[i]):
            out[i] += expert_ff(s * h[i], w[f"e{e}.gate"], w[f"e{e}.up"], w[f"e{e}.down"], mlp["expert"]["limit"])
    return out


def _sub(tensors: Dict[str, torch.Tensor], prefix: str, dtype) -> Dict[str, torch.Tensor]:
    return {k[len(prefix):]: v.to(dtype) for k, v in tensors.items() if k.startswith(prefix)}


def forward(config: dict, tensors: Dict[str, torch.Tensor], tokens, dtype=torch.float64, layers_out: Optional[List] = None,
            fast: bool = True, margins_out: Optional[List] = None) -> torch.Tensor:
    """Logits [n, vocab] of one whole sequence.  ``layers_out``: a list that receives the residual stream after every
    layer; ``margins_out``: one that receives ``router_margins`` of every routed layer."""
    eps = config["norm"]["eps"]
    x = embed_tokens(tokens, tensors["embed"].to(dtype), tensors["pos"].to(dtype))
    v_first = None
    for i, layer in enumerate(config["layers"]):
        if layer["type"] != "attention":
            raise ValueError(f"unknown mixer {layer['type']!r}")
        h = rms_norm(x, tensors[f"l{i}.norm1"].to(dtype), eps)
        m = layer["mixer"]
        a, v = attention_mixer(h, _sub(tensors, f"l{i}.mix.", dtype), m, v_first if m.get("v_mix") else None, fast=fast)
        if m.get("v_mix") and v_first is None:
            v_first = v
        delta = a
        mlp = layer.get("mlp")
        if mlp:
            w = _sub(tensors, f"l{i}.mlp.", dtype)
            if mlp["kind"] == "moe" and margins_out is not None:
                margins_out.append(router_margins(h, w["router"], mlp["router"]["top"]))
            delta = delta + (dense_ff(h, w) if mlp["kind"] == "dense" else moe_ff(h, w, mlp))
        x = x + delta
        if layers_out is not None:
            layers_out.append(x.clone())
    x = rms_norm(x, tensors["final.norm"].to(dtype), eps)
    return x @ tensors["head"].to(dtype).T


def random_model(config: dict, seed: int = 0, std: float = 0.08, bias_std: float = 0.05) -> Dict[str, torch.Tensor]:
    """Random tensors (bfloat16, as a checkpoint holds them) for ``config``, by the names the design gives them."""
    g = torch.Generator().manual_seed(seed)

    def mat(*shape, s=std):
        return (torch.randn(*shape, generator=g) * s).to(torch.bfloat16)

    D, V = config["width"], config["vocab"]
    t = {"embed": mat(V, D, s=1.0), "pos": mat(config["max_positions"], D, s=0.3),
         "final.norm": (1 + 0.1 * torch.randn(D, generator=g)).to(torch.bfloat16), "head": mat(V, D, s=D ** -0.5)}
    for i, layer in enumerate(config["layers"]):
        m = layer["mixer"]
        H, G, dk, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        p = f"l{i}."
        t[p + "norm1"] = (1 + 0.1 * torch.randn(D, generator=g)).to(torch.bfloat16)
        t[p + "mix.q"], t[p + "mix.q.b"] = mat(H * dk, D, s=D ** -0.5), mat(H * dk, s=bias_std)
        t[p + "mix.k"], t[p + "mix.k.b"] = mat(G * dk, D, s=D ** -0.5), mat(G * dk, s=bias_std)
        t[p + "mix.v"], t[p + "mix.v.b"] = mat(G * dv, D, s=D ** -0.5), mat(G * dv, s=bias_std)
        t[p + "mix.o"], t[p + "mix.o.b"] = mat(D, H * dv, s=(H * dv) ** -0.5), mat(D, s=bias_std)
        if m.get("v_mix"):
            t[p + "mix.vmix"] = torch.tensor(0.2 + 0.6 * torch.rand((), generator=g).item()).to(torch.bfloat16)
        mlp = layer.get("mlp")
        if mlp and mlp["kind"] == "dense":
            t[p + "mlp.up"], t[p + "mlp.down"] = mat(mlp["ff"], D, s=D ** -0.5), mat(D, mlp["ff"], s=mlp["ff"] ** -0.5)
        elif mlp:
            F = mlp["expert"]["ff"]
            t[p + "mlp.router"] = mat(mlp["router"]["experts"], D, s=2 * D ** -0.5)
            for e in range(mlp["router"]["experts"]):
                t[p + f"mlp.e{e}.gate"], t[p + f"mlp.e{e}.up"] = mat(F, D, s=D ** -0.5), mat(F, D, s=D ** -0.5)
                t[p + f"mlp.e{e}.down"] = mat(D, F, s=F ** -0.5)
    return t
