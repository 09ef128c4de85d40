"""The Nasedra decoder as a typed configuration and a model description.

config.json gives every size and every constant that differs between models of the design:

  architecture "Nasedra", vocab, width, norm.eps, embedding.scale,
  layers: a list; each entry has type (its mixer), mixer (the mixer's sizes) and mlp (its feed-forward, or null)
    type "attention": heads, kv_heads, dim, vdim, scale, softcap, mask.size / mask.keep_first (or no mask),
                      rot.dims / rot.base / rot.scaling.{factor, original, fast, slow} (or no rot, or no scaling),
                      kv_from (the layer whose keys and values this one reads; it then has no k and v matrices)
    type "gla":       heads, dim, vdim, tau; the inner size of the decay's two matrices is the shape of '<layer>.mix.a1'
    mlp kind "dense": ff;  kind "moe": expert.ff, router.experts / top / identity / scale, shared.ff (or no shared)

The model: token row times embedding.scale; layers of the parallel arrangement with two norms (the mixer reads norm1(x),
the feed-forward norm2(x), both of the same x); a final norm; the output matrix.  Tensor names: embed, l<i>.norm1,
l<i>.norm2, l<i>.mix.*, l<i>.mlp.*, final.norm, head.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Dict, Optional, Tuple

from ..parts.spec import LayerSpec, ModelSpec, PartSpec, RunEntry
from .lerazen import _int, _num
from .model_config import ConfigError
from .registry import register_architecture

DEFAULT_DECAY_RANK = 32      # where neither a checkpoint nor the configuration says (a model yet to be written)


@dataclass(frozen=True)
class RotationConfig:
    dims: int
    base: float
    scaling: Optional[Tuple[float, float, float, float]]    # factor, original length, fast, slow

    @classmethod
    def from_dict(cls, d: Dict[str, Any], where: str, head_dim: int) -> "RotationConfig":
        dims = _int(d, "dims", where, least=2)
        if dims % 2 or dims > head_dim:
            raise ConfigError(f"{where}: dims must be even and at most the head size {head_dim}, got {dims}")
        base = _num(d, "base", where)
        if not base > 1:
            raise ConfigError(f"{where}: base must be larger than 1")
        sc = d.get("scaling")
        scaling = None
        if sc:
            w = where + ".scaling"
            scaling = (_num(sc, "factor", w), _num(sc, "original", w), _num(sc, "fast", w), _num(sc, "slow", w))
            if not (scaling[0] > 0 and scaling[1] > 0 and scaling[2] > 0 and scaling[3] > 0):
                raise ConfigError(f"{w}: factor, original, fast and slow must be positive")
        return cls(dims, base, scaling)


@dataclass(frozen=True)
class AttentionConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    softcap: float         # 0: none
    window: int            # 0: none
    keep_first: int
    rot: Optional[RotationConfig]
    kv_from: Optional[int]
    gated: bool = True     # False: a checkpoint without the gate's matrix

    @classmethod
    def from_dict(cls, d: Dict[str, Any], where: str, gated: bool = True) -> "AttentionConfig":
        mask = d.get("mask") or {}
        dim = _int(d, "dim", where)
        kv_from = d.get("kv_from")
        if kv_from is not None and (isinstance(kv_from, bool) or not isinstance(kv_from, int) or kv_from < 0):
            raise ConfigError(f"{where}: kv_from must name a layer, got {kv_from!r}")
        cfg = cls(heads=_int(d, "heads", where), kv_heads=_int(d, "kv_heads", where), dim=dim, vdim=_int(d, "vdim", where),
                  scale=_num(d, "scale", where), softcap=_num(d, "softcap", where) if d.get("softcap") is not None else 0.0,
                  window=_int(mask, "size", where + ".mask") if mask.get("size") is not None else 0,
                  keep_first=_int(mask, "keep_first", where + ".mask", least=0) if mask.get("keep_first") is not None else 0,
                  rot=RotationConfig.from_dict(d["rot"], where + ".rot", dim) if d.get("rot") else None, kv_from=kv_from,
                  gated=gated)
        if cfg.heads % cfg.kv_heads:
            raise ConfigError(f"{where}: {cfg.heads} heads are not a multiple of {cfg.kv_heads} kv_heads")
        if cfg.softcap < 0:
            raise ConfigError(f"{where}: softcap must not be negative")
        return cfg


@dataclass(frozen=True)
class GLAConfig:
    heads: int
    dim: int
    vdim: int
    tau: float
    rank: int

    @classmethod
    def from_dict(cls, d: Dict[str, Any], where: str, rank: int) -> "GLAConfig":
        cfg = cls(heads=_int(d, "heads", where), dim=_int(d, "dim", where), vdim=_int(d, "vdim", where),
                  tau=_num(d, "tau", where), rank=rank)
        if not cfg.tau > 0:
            raise ConfigError(f"{where}: tau must be positive")
        return cfg


@dataclass(frozen=True)
class FeedForwardConfig:
    kind: str              # "dense" or "moe"
    ff: int
    experts: int = 0
    top: int = 0
    identity: int = 0
    scale: float = 1.0
    shared_ff: int = 0     # 0: no shared expert
    correction: bool = True    # False: a checkpoint without the choice's correction vector

    @classmethod
    def from_dict(cls, d: Dict[str, Any], where: str, correction: bool = True) -> "FeedForwardConfig":
        kind = d.get("kind")
        if kind == "dense":
            return cls("dense", _int(d, "ff", where))
        if kind == "moe":
            ex, ro, sh = d.get("expert") or {}, d.get("router") or {}, d.get("shared") or {}
            cfg = cls("moe", _int(ex, "ff", where + ".expert"), _int(ro, "experts", where + ".router"),
                      _int(ro, "top", where + ".router"),
                      _int(ro, "identity", where + ".router", least=0) if ro.get("identity") is not None else 0,
                      _num(ro, "scale", where + ".router") if ro.get("scale") is not None else 1.0,
                      _int(sh, "ff", where + ".shared") if sh else 0, correction)
            if cfg.top > cfg.experts + cfg.identity:
                raise ConfigError(f"{where}: top {cfg.top} of {cfg.experts + cfg.identity} router outputs")
            return cfg
        raise ConfigError(f"{where}: mlp kind {kind!r} is not known (dense, moe)")


@dataclass(frozen=True)
class NasedraLayer:
    type: str              # "attention" or "gla"
    mixer: Any             # AttentionConfig or GLAConfig
    mlp: Optional[FeedForwardConfig]


@dataclass(frozen=True)
class NasedraConfig:
    vocab: int
    width: int
    norm_eps: float
    embed_scale: float
    layers: Tuple[NasedraLayer, ...]
    eos_token_id: Optional[int] = None

    @classmethod
    def from_dict(cls, d: Dict[str, Any], shapes: Optional[Dict[str, tuple]] = None) -> "NasedraConfig":
        norm = d.get("norm") or {}
        raw_layers = d.get("layers")
        if not isinstance(raw_layers, list):
            raise ConfigError("config.json lacks the list 'layers'")
        layers = []
        for i, l in enumerate(raw_layers):
            where = f"layers[{i}]"
            if not isinstance(l.get("mixer"), dict):
                raise ConfigError(f"{where} lacks 'mixer'")
            # tensors that a checkpoint may leave out (a gate, a correction of the choice) are taken as it has them
            has = (lambda name: True) if shapes is None else (lambda name: name in shapes)
            if l.get("type") == "attention":
                mixer = AttentionConfig.from_dict(l["mixer"], where + ".mixer", gated=has(f"l{i}.mix.g"))
            elif l.get("type") == "gla":
                # the inner size of the decay's matrices: the checkpoint's shape; else a key of the mixer (a model that
                # is yet to be written); else the usual one
                name = f"l{i}.mix.a1"
                if shapes is not None and name in shapes and len(shapes[name]) == 2:
                    rank = int(shapes[name][0])
                elif l["mixer"].get("rank") is not None:
                    rank = _int(l["mixer"], "rank", where + ".mixer")
                else:
                    rank = DEFAULT_DECAY_RANK
                mixer = GLAConfig.from_dict(l["mixer"], where + ".mixer", rank)
            else:
                raise ConfigError(f"{where}: mixer type {l.get('type')!r} is not known (attention, gla)")
            mlp = l.get("mlp")
            layers.append(NasedraLayer(l["type"], mixer,
                                       FeedForwardConfig.from_dict(mlp, where + ".mlp", has(f"l{i}.mlp.correction")) if mlp else None))
        for i, l in enumerate(layers):
            if l.type != "attention" or l.mixer.kv_from is None:
                continue
            j, where = l.mixer.kv_from, f"layers[{i}].mixer"
            if j >= i or layers[j].type != "attention" or layers[j].mixer.kv_from is not None:
                raise ConfigError(f"{where}: kv_from must name an earlier attention layer with keys and values of its own, got {j}")
            o, m = layers[j].mixer, l.mixer
            if (o.kv_heads, o.dim, o.vdim) != (m.kv_heads, m.dim, m.vdim):
                raise ConfigError(f"{where}: layer {j}'s keys and values do not have this layer's sizes")
        eps = _num(norm, "eps", "norm")
        if not eps > 0:
            raise ConfigError("norm.eps must be positive")
        emb = d.get("embedding") or {}
        eos = d.get("eos_token_id")
        return cls(vocab=_int(d, "vocab", "config.json"), width=_int(d, "width", "config.json"), norm_eps=eps,
                   embed_scale=_num(emb, "scale", "embedding") if emb.get("scale") is not None else 1.0,
                   layers=tuple(layers), eos_token_id=eos if isinstance(eos, int) and not isinstance(eos, bool) else None)


def _cache_extent(cfg: NasedraConfig, owner: int) -> Tuple[int, int]:
    """(window, kept first positions) that the cache of layer ``owner`` has to serve: its own mask and those of the
    layers that read its keys and values.  A window of 0 (none) wins; else the largest; the most kept positions."""
    users = [cfg.layers[owner].mixer] + [l.mixer for l in cfg.layers if l.type == "attention" and l.mixer.kv_from == owner]
    if any(u.window == 0 for u in users):
        return 0, 0
    return max(u.window for u in users), max(u.keep_first for u in users)


def nasedra_spec(cfg: NasedraConfig) -> ModelSpec:
    norm = PartSpec("rms_norm", {"size": cfg.width, "eps": cfg.norm_eps, "weight_name": ""})
    layers, run_order = [], []
    for i, l in enumerate(cfg.layers):
        m = l.mixer
        if l.type == "attention":
            owner = i if m.kv_from is None else m.kv_from
            cache_window, cache_keep = _cache_extent(cfg, owner)
            position = PartSpec("none", {})
            if m.rot is not None:
                position = PartSpec("rotary_pairs", {"rotary_dim": m.rot.dims, "base": m.rot.base, "scaling": m.rot.scaling})
            mixer = PartSpec("gated_attention", {
                "hidden_size": cfg.width, "num_heads": m.heads, "num_kv_heads": m.kv_heads, "key_dim": m.dim,
                "value_dim": m.vdim, "scale": m.scale, "softcap": m.softcap, "window": m.window, "keep_first": m.keep_first,
                "gated": m.gated,
                "position": position, "own_kv": m.kv_from is None, "cache_window": cache_window,
                "cache_keep_first": cache_keep})
            run_order.append(RunEntry(i, cache_of=m.kv_from))
        else:
            mixer = PartSpec("gated_linear_attention", {
                "hidden_size": cfg.width, "num_heads": m.heads, "key_dim": m.dim, "value_dim": m.vdim, "tau": m.tau,
                "rank": m.rank, "norm_eps": cfg.norm_eps})
            run_order.append(RunEntry(i))
        if l.mlp is None:
            ff = PartSpec("none", {})
        elif l.mlp.kind == "dense":
            ff = PartSpec("swiglu_mlp", {"hidden_size": cfg.width, "intermediate_size": l.mlp.ff,
                                         "names": ("gate", "up", "down")})
        else:
            ff = PartSpec("softmax_routed_experts", {
                "hidden_size": cfg.width, "expert_size": l.mlp.ff, "num_experts": l.mlp.experts, "top": l.mlp.top,
                "identity": l.mlp.identity, "scale": l.mlp.scale, "shared_size": l.mlp.shared_ff,
                "correction_name": "correction" if l.mlp.correction else None})
        layers.append(LayerSpec(prefix=f"l{i}", block="parallel_two_norms",
                                slots={"norm1": ("norm1", norm), "mixer": ("mix", mixer), "norm2": ("norm2", norm),
                                       "ff": ("mlp", ff)}))
    return ModelSpec(
        hidden_size=cfg.width, vocab_size=cfg.vocab, embed_name="embed", layers=layers, run_order=run_order,
        final_norm=norm, final_norm_name="final.norm", head_name="head", eos_token_id=cfg.eos_token_id,
        embed_scale=cfg.embed_scale)


def nasedra_sizes(cfg: NasedraConfig) -> dict:
    """The sizes of a configuration as a flat record (of its first layer of every kind)."""
    out = {"layers": len(cfg.layers), "hidden": cfg.width, "vocab": cfg.vocab, "tied": False}
    for l in cfg.layers:
        m = l.mixer
        if l.type == "attention":
            out.setdefault("q_heads", m.heads)
            out.setdefault("kv_heads", m.kv_heads)
            out.setdefault("head_dim", m.dim)
            out.setdefault("value_dim", m.vdim)
            out.setdefault("window", m.window)
        else:
            out.setdefault("gla_heads", m.heads)
            out.setdefault("gla_key_dim", m.dim)
            out.setdefault("gla_value_dim", m.vdim)
        if l.mlp is not None and l.mlp.kind == "dense":
            out.setdefault("intermediate", l.mlp.ff)
        elif l.mlp is not None:
            out.setdefault("experts", l.mlp.experts)
            out.setdefault("top", l.mlp.top)
            out.setdefault("expert_size", l.mlp.ff)
    return out


def nasedra_with_layers(raw: dict, layers: int) -> dict:
    """The same kinds of layers, ``layers`` of them: the list cut, or repeated from its start (a layer that reads
    another's keys and values keeps its distance to that layer)."""
    have = raw["layers"]
    out = []
    for i in range(layers):
        src = i % len(have)
        l = dict(have[src])
        if l.get("type") == "attention" and l["mixer"].get("kv_from") is not None:
            l["mixer"] = dict(l["mixer"], kv_from=i - (src - l["mixer"]["kv_from"]))
        out.append(l)
    return dict(raw, layers=out if have else [])


register_architecture("Nasedra", NasedraConfig.from_dict, nasedra_spec, nasedra_sizes, nasedra_with_layers,
                      reads_shapes=True)
