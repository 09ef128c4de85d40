"""A plain, slow implementation of the Nasedra decoder: whole sequences, no cache, one function per mechanism,
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


def silu(z: torch.Tensor) -> torch.Tensor:
    return z * torch.sigmoid(z)


# ---------------------------------------------------------------------------------------------------------------
# rotation
# ---------------------------------------------------------------------------------------------------------------
def rotation_frequencies(rot: dict):
    """(frequencies [dims / 2], factor on cosine and sine).  Plain: f_i = base^(-2i / dims), factor 1.  With a scaling
    record (factor s, original length L, fast, slow): a frequency that turns more than ``fast`` times in L keeps its
    value, one that turns fewer than ``slow`` times is divided by s, and between the two the mix is linear in the
    index of the pair; cosine and sine are multiplied by 0.1 ln s + 1."""
    dims, base = rot["dims"], float(rot["base"])
    half = dims // 2
    f = [base ** (-2.0 * i / dims) for i in range(half)]
    sc = rot.get("scaling")
    if not sc:
        return torch.tensor(f, dtype=torch.float64), 1.0
    s, L = float(sc["factor"]), float(sc["original"])

    def pair_index(turns: float) -> float:          # the (real-valued) pair that turns ``turns`` times in L positions
        return dims * math.log(L / (2.0 * math.pi * turns)) / (2.0 * math.log(base))
    lo = max(math.floor(pair_index(float(sc["fast"]))), 0)
    hi = min(math.ceil(pair_index(float(sc["slow"]))), dims - 1)
    out = []
    for i in range(half):
        ramp = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
        out.append(f[i] / s * ramp + f[i] * (1.0 - ramp))
    return torch.tensor(out, dtype=torch.float64), 0.1 * math.log(s) + 1.0


def rotate_pairs(x: torch.Tensor, positions: torch.Tensor, rot: dict) -> torch.Tensor:
    """x [n, heads, d]: neighbours (2i, 2i + 1) of the first ``dims`` entries of every head are turned by
    position * f_i; the rest passes."""
    f, mag = rotation_frequencies(rot)
    dims = rot["dims"]
    ang = positions.to(torch.float64)[:, None] * f[None, :]                   # [n, dims / 2]
    c, s = (torch.cos(ang) * mag).to(x.dtype)[:, None, :], (torch.sin(ang) * mag).to(x.dtype)[:, None, :]
    out = x.clone()
    a, b = x[..., 0:dims:2], x[..., 1:dims:2]
    out[..., 0:dims:2] = a * c - b * s
    out[..., 1:dims:2] = b * c + a * s
    return out


# ---------------------------------------------------------------------------------------------------------------
# attention
# ---------------------------------------------------------------------------------------------------------------
def visible(i: int, j: int, window: Optional[int], keep_first: int) -> bool:
    """Query i sees key j: never the future; with a window the last ``window`` positions (itself included) and the
    first ``keep_first`` positions of the sequence."""
    if j > i:
        return False
    return window is None or i - j < window or j < keep_first


def visibility_matrix(positions: torch.Tensor, window: Optional[int], keep_first: int) -> torch.Tensor:
    """``visible`` for all pairs at once, [queries, keys] (the tests check it against ``visible`` pair by pair)."""
    i, j = positions[:, None], positions[None, :]
    ok = j <= i
    if window is not None:
        ok = ok & ((i - j < window) | (j < keep_first))
    return ok


def capped(s: torch.Tensor, cap: Optional[float]) -> torch.Tensor:
    return s if not cap else cap * torch.tanh(s / cap)


def attention_keys_values(h: torch.Tensor, w: Dict[str, torch.Tensor], m: dict, positions: torch.Tensor):
    """Rotated keys [n, G, dk] and values [n, G, dv] of a layer that has projections of its own."""
    n = h.shape[0]
    G, dk, dv = m["kv_heads"], m["dim"], m["vdim"]
    k = (h @ w["k"].T).view(n, G, dk)
    v = (h @ w["v"].T).view(n, G, dv)
    if m.get("rot"):
        k = rotate_pairs(k, positions, m["rot"])
    return k, v


def attention_mixer(h: torch.Tensor, w: Dict[str, torch.Tensor], m: dict, k: torch.Tensor, v: torch.Tensor,
                    positions: torch.Tensor) -> torch.Tensor:
    """Attention on normed rows h [n, D] over keys k [n, G, dk] (rotated) and values v [n, G, dv], which are this
    layer's own or another layer's.  Gate: the heads' outputs times sigmoid(Wg h), then the output matrix."""
    n = h.shape[0]
    H, G, dk, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (h @ w["q"].T).view(n, H, dk)
    if m.get("rot"):
        q = rotate_pairs(q, positions, m["rot"])
    mask = m.get("mask") or {}
    window, keep = mask.get("size"), int(mask.get("keep_first", 0))
    out = torch.zeros(n, H, dv, dtype=h.dtype)
    ok = visibility_matrix(positions, window, keep)
    for hd in range(H):
        g = hd // (H // G)
        s = capped((q[:, hd] @ k[:, g].T) * m["scale"], m.get("softcap"))
        p = torch.softmax(s.masked_fill(~ok, float("-inf")), -1)
        out[:, hd] = p @ v[:, g]
    a = out.reshape(n, H * dv)
    if "g" in w:
        a = a * torch.sigmoid(h @ w["g"].T)
    return a @ w["o"].T


# ---------------------------------------------------------------------------------------------------------------
# gated linear attention
# ---------------------------------------------------------------------------------------------------------------
def gla_decay(h: torch.Tensor, w: Dict[str, torch.Tensor], m: dict) -> torch.Tensor:
    """alpha [n, H, dk] = sigmoid(W_a2 (W_a1 h) + b)^(1 / tau), a decay per key channel."""
    z = (h @ w["a1"].T) @ w["a2"].T + w["a2.b"]
    return torch.sigmoid(z).pow(1.0 / m["tau"]).view(h.shape[0], m["heads"], m["dim"])


def gla_recurrence(q, k, v, alpha, state=None):
    """Token by token: S <- diag(alpha_t) S + k_t v_t^T, o_t = S^T q_t.  q, k, alpha [n, H, dk]; v [n, H, dv];
    state [H, dk, dv] (None: zeros).  Returns (o [n, H, dv], the state after the last token)."""
    n, H, dk = q.shape
    dv = v.shape[-1]
    S = torch.zeros(H, dk, dv, dtype=q.dtype) if state is None else state.clone()
    o = torch.zeros(n, H, dv, dtype=q.dtype)
    for t in range(n):
        S = alpha[t][:, :, None] * S + k[t][:, :, None] * v[t][:, None, :]
        o[t] = torch.einsum("hkv,hk->hv", S, q[t])
    return o, S


def gla_cancellation(q, k, v, alpha) -> torch.Tensor:
    """[n]: over the heads the smallest |o_t| / (|q_t| |S_t|), how much of the state's size survives the sum over key
    channels.  The head norm divides by |o_t|: where almost everything cancels (the first token of a sequence whose
    query is nearly orthogonal to its key, say) a rounding of q or k decides the output's sign."""
    n, H, dk = q.shape
    S = torch.zeros(H, dk, v.shape[-1], dtype=q.dtype)
    out = torch.zeros(n, dtype=q.dtype)
    for t in range(n):
        S = alpha[t][:, :, None] * S + k[t][:, :, None] * v[t][:, None, :]
        o = torch.einsum("hkv,hk->hv", S, q[t])
        out[t] = (o.norm(dim=-1) / (q[t].norm(dim=-1) * S.flatten(1).norm(dim=-1) + 1e-300)).min()
    return out


def gla_mixer(h: torch.Tensor, w: Dict[str, torch.Tensor], m: dict, eps: float, cancel_out: Optional[List] = None) -> torch.Tensor:
    n = h.shape[0]
    H, dk, dv = m["heads"], m["dim"], m["vdim"]
    q = (h @ w["q"].T).view(n, H, dk) * dk ** -0.5
    k = (h @ w["k"].T).view(n, H, dk)
    v = (h @ w["v"].T).view(n, H, dv)
    o, _ = gla_recurrence(q, k, v, gla_decay(h, w, m))
    if cancel_out is not None:
        cancel_out.append(gla_cancellation(q, k, v, gla_decay(h, w, m)))
    o = rms_norm(o, w["norm"], eps).reshape(n, H * dv)          # every head by itself, one weight for all heads
    return (o * silu(h @ w["g"].T)) @ w["o"].T


# ---------------------------------------------------------------------------------------------------------------
# feed-forwards
# ---------------------------------------------------------------------------------------------------------------
def gated_mlp(h: torch.Tensor, gate: torch.Tensor, up: torch.Tensor, down: torch.Tensor) -> torch.Tensor:
    return (silu(h @ gate.T) * (h @ up.T)) @ down.T


def route(h: torch.Tensor, router: torch.Tensor, correction: Optional[torch.Tensor], top: int, scale: float):
    """(chosen [n, top], weights [n, top]).  Scores: softmax of the router's logits over all its outputs.  The ``top``
    largest of score + correction are chosen (the lowest index among equals); the weights are the chosen scores
    (without the correction) over their sum, times ``scale``."""
    s = torch.softmax(h @ router.T, -1)
    choice = s if correction is None else s + correction
    n, E = s.shape
    chosen = torch.zeros(n, top, dtype=torch.long)
    for t in range(n):
        left = list(range(E))
        for k in range(top):
            best = max(left, key=lambda e: (float(choice[t, e]), -e))
            chosen[t, k] = best
            left.remove(best)
    ws = torch.gather(s, 1, chosen)
    return chosen, ws / (ws.sum(-1, keepdim=True) + 1e-20) * scale


def route_margin(h: torch.Tensor, router: torch.Tensor, correction: Optional[torch.Tensor], top: int) -> torch.Tensor:
    """[n]: how far the last chosen output lies in front of the first rejected one, as a fraction of the larger of
    their two scores (a small value: rounding may choose the other)."""
    s = torch.softmax(h @ router.T, -1)
    choice = s if correction is None else s + correction
    if top >= s.shape[1]:
        return torch.full((s.shape[0],), float("inf"), dtype=s.dtype)
    order = torch.argsort(choice, dim=-1, descending=True, stable=True)
    a, b = order[:, top - 1:top], order[:, top:top + 1]
    gap = torch.gather(choice, 1, a) - torch.gather(choice, 1, b)
    return (gap / (torch.maximum(torch.gather(s, 1, a), torch.gather(s, 1, b)) + 1e-9))[:, 0]


def routed_mlp(h: torch.Tensor, w: Dict[str, torch.Tensor], f: dict) -> torch.Tensor:
    """Experts e0 .. e(E-1) are gated feed-forwards; the router's outputs E .. E + identity - 1 stand for experts that
    hand their input on unchanged.  A shared expert, if there is one, runs for every token."""
    r = f["router"]
    E, ident = r["experts"], int(r.get("identity", 0))
    chosen, ws = route(h, w["router"], w.get("correction"), r["top"], float(r.get("scale", 1.0)))
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e, wt in zip(chosen[t].tolist(), ws[t]):
            if e >= E:
                assert e < E + ident
                out[t] += wt * h[t]
            else:
                out[t] += wt * gated_mlp(h[t:t + 1], w[f"e{e}.gate"], w[f"e{e}.up"], w[f"e{e}.down"])[0]
    if f.get("shared"):
        out = out + gated_mlp(h, w["shared.gate"], w["shared.up"], w["shared.down"])
    return out


def feed_forward(h, w, f):
    if f is None:
        return torch.zeros_like(h)
    if f["kind"] == "dense":
        return gated_mlp(h, w["gate"], w["up"], w["down"])
    return routed_mlp(h, w, f)


# ---------------------------------------------------------------------------------------------------------------
# the model
# ---------------------------------------------------------------------------------------------------------------
def sub(tensors: Dict[str, torch.Tensor], prefix: str) -> Dict[str, torch.Tensor]:
    return {k[len(prefix):]: v for k, v in tensors.items() if k.startswith(prefix)}


def forward(config: dict, tensors: Dict[str, torch.Tensor], tokens, dtype=torch.float64, layers_out: Optional[List] = None,
            margins_out: Optional[List] = None):
    """Logits [n, vocab] of a whole sequence from position 0.  ``layers_out``: a list that gets the residual stream
    after every layer; ``margins_out``: one that gets ``route_margin`` of every routed layer and four times
    ``gla_cancellation`` of every recurrent layer (a value below about 0.08 of either kind: rounding to bfloat16 may
    decide what the position computes)."""
    t = {k: v.to(dtype) if v.is_floating_point() else v for k, v in tensors.items()}
    ids = torch.as_tensor(list(tokens), dtype=torch.long)
    n = len(ids)
    positions = torch.arange(n)
    eps = float(config["norm"]["eps"])
    x = t["embed"][ids] * float((config.get("embedding") or {}).get("scale", 1.0))
    kept = {}                                                                      # layer -> its keys and values
    for i, layer in enumerate(config["layers"]):
        p = f"l{i}."
        m = layer["mixer"]
        w = sub(t, p + "mix.")
        h1 = rms_norm(x, t[p + "norm1"], eps)
        h2 = rms_norm(x, t[p + "norm2"], eps)
        if layer["type"] == "attention":
            if m.get("kv_from") is not None:
                k, v = kept[int(m["kv_from"])]
            else:
                k, v = kept[i] = attention_keys_values(h1, w, m, positions)
            a = attention_mixer(h1, w, m, k, v, positions)
        elif layer["type"] == "gla":
            cancel = [] if margins_out is not None else None
            a = gla_mixer(h1, w, m, eps, cancel)
            if cancel:
                margins_out.append(4.0 * cancel[0])
        else:
            raise ValueError(layer["type"])
        f = layer.get("mlp")
        if margins_out is not None and f is not None and f["kind"] == "moe":
            margins_out.append(route_margin(h2, t[p + "mlp.router"], t.get(p + "mlp.correction"), f["router"]["top"]))
        x = x + (a + feed_forward(h2, sub(t, p + "mlp."), f))
        if layers_out is not None:
            layers_out.append(x.clone())
    return rms_norm(x, t["final.norm"], eps) @ t["head"].T


# ---------------------------------------------------------------------------------------------------------------
# random models
# ---------------------------------------------------------------------------------------------------------------
def tensor_shapes(config: dict, rank: int = 16) -> Dict[str, tuple]:
    """Names and shapes of a checkpoint.  ``rank``: the inner size of the decay's two matrices, which config.json does
    not hold (a reader takes it from the tensors' shapes)."""
    D, V = config["width"], config["vocab"]
    out = {"embed": (V, D)}
    for i, layer in enumerate(config["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        out[p + "norm1"] = (D,)
        out[p + "norm2"] = (D,)
        H, dk, dv = m["heads"], m["dim"], m["vdim"]
        if layer["type"] == "attention":
            G = m["kv_heads"]
            out[p + "mix.q"] = (H * dk, D)
            if m.get("kv_from") is None:
                out[p + "mix.k"] = (G * dk, D)
                out[p + "mix.v"] = (G * dv, D)
            out[p + "mix.g"] = (H * dv, D)
            out[p + "mix.o"] = (D, H * dv)
        else:
            r = rank
            out.update({p + "mix.q": (H * dk, D), p + "mix.k": (H * dk, D), p + "mix.v": (H * dv, D),
                        p + "mix.g": (H * dv, D), p + "mix.o": (D, H * dv), p + "mix.norm": (dv,),
                        p + "mix.a1": (r, D), p + "mix.a2": (H * dk, r), p + "mix.a2.b": (H * dk,)})
        f = layer.get("mlp")
        if f is None:
            continue
        if f["kind"] == "dense":
            out.update({p + "mlp.gate": (f["ff"], D), p + "mlp.up": (f["ff"], D), p + "mlp.down": (D, f["ff"])})
        else:
            r, F = f["router"], f["expert"]["ff"]
            for e in range(r["experts"]):
                out.update({p + f"mlp.e{e}.gate": (F, D), p + f"mlp.e{e}.up": (F, D), p + f"mlp.e{e}.down": (D, F)})
            n_out = r["experts"] + int(r.get("identity", 0))
            out[p + "mlp.router"] = (n_out, D)
            out[p + "mlp.correction"] = (n_out,)
            if f.get("shared"):
                S = f["shared"]["ff"]
                out.update({p + "mlp.shared.gate": (S, D), p + "mlp.shared.up": (S, D), p + "mlp.shared.down": (D, S)})
    out["final.norm"] = (D,)
    out["head"] = (V, D)
    return out


def random_model(config: dict, seed: int = 0, dtype=torch.bfloat16, rank: int = 16) -> Dict[str, torch.Tensor]:
    """Random tensors of a size that keeps every mechanism alive: scores of a few units, routers that disagree, decays
    spread between fast and slow."""
    g = torch.Generator().manual_seed(seed)
    D = config["width"]
    out = {}
    for name, shape in tensor_shapes(config, rank).items():
        last = name.rsplit(".", 1)[-1]
        if "norm" in last:
            t = 1.0 + 0.2 * (torch.rand(shape, generator=g) - 0.5)
        elif name.endswith("a2.b"):
            t = 1.0 + 2.0 * torch.randn(shape, generator=g)
        elif last == "correction":
            t = 0.05 * torch.randn(shape, generator=g)
        elif last == "embed":
            t = torch.randn(shape, generator=g) / float((config.get("embedding") or {}).get("scale", 1.0))
        elif last == "router":
            t = torch.randn(shape, generator=g) * 6.0 / math.sqrt(shape[-1])       # peaked scores: few close calls
        elif last == "a2":
            t = torch.randn(shape, generator=g) * 2.0 / math.sqrt(shape[-1])
        elif last in ("q", "k"):
            t = torch.randn(shape, generator=g) * 1.5 / math.sqrt(shape[-1])
        else:
            t = torch.randn(shape, generator=g) / math.sqrt(shape[-1])
        out[name] = t.to(dtype)
    return out
