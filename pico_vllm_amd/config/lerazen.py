"""The Lerazen decoder as a typed configuration and a model description.

config.json gives every size and every constant that differs between models of the design:

  architecture "Lerazen", vocab, width, max_positions, norm.eps,
  layers: a list; each entry has type (its mixer), mixer (the mixer's sizes) and mlp (its feed-forward, or null)
    type "attention": mixer = heads, kv_heads, dim, vdim, scale, mask.size (or no mask), q_temp.coef / q_temp.every
                      (or no q_temp), v_mix
    mlp kind "dense": ff;  kind "moe": expert.ff, expert.limit, router.experts, router.top

The model: token row + learned position row; layers of the parallel arrangement (one norm, mixer and feed-forward both
read it); a final norm; the output matrix.  Tensor names: embed, pos, l<i>.norm1, l<i>.mix.*, l<i>.mlp.*, final.norm, head.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Dict, Optional, Tuple

from ..parts.spec import LayerSpec, ModelSpec, PartSpec, RunEntry
from .model_config import ConfigError
from .registry import register_architecture


def _int(d: Dict[str, Any], key: str, where: str, least: int = 1) -> int:
    if key not in d:
        raise ConfigError(f"{where} lacks {key!r}")
    v = d[key]
    if isinstance(v, bool) or not isinstance(v, int) or v < least:
        raise ConfigError(f"{where}: {key} must be an integer of at least {least}, got {v!r}")
    return v


def _num(d: Dict[str, Any], key: str, where: str) -> float:
    if key not in d:
        raise ConfigError(f"{where} lacks {key!r}")
    v = d[key]
    if isinstance(v, bool) or not isinstance(v, (int, float)):
        raise ConfigError(f"{where}: {key} must be a number, got {v!r}")
    return float(v)


@dataclass(frozen=True)
class AttentionConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    window: int            # 0: none
    temp_coef: float
    temp_every: int        # 0: no query temperature
    v_mix: bool

    @classmethod
    def from_dict(cls, d: Dict[str, Any], where: str) -> "AttentionConfig":
        mask, qt = d.get("mask") or {}, d.get("q_temp") or {}
        cfg = cls(heads=_int(d, "heads", where), kv_heads=_int(d, "kv_heads", where), dim=_int(d, "dim", where),
                  vdim=_int(d, "vdim", where), scale=_num(d, "scale", where),
                  window=_int(mask, "size", where + ".mask") if mask else 0,
                  temp_coef=_num(qt, "coef", where + ".q_temp") if qt else 0.0,
                  temp_every=_int(qt, "every", where + ".q_temp") if qt else 0,
                  v_mix=bool(d.get("v_mix", False)))
        if cfg.heads % cfg.kv_heads:
            raise ConfigError(f"{where}: {cfg.heads} heads are not a multiple of {cfg.kv_heads} kv_heads")
        return cfg


@dataclass(frozen=True)
class FeedForwardConfig:
    kind: str              # "dense" or "moe"
    ff: int
    experts: int = 0
    top: int = 0
    limit: float = 0.0

    @classmethod
    def from_dict(cls, d: Dict[str, Any], where: str) -> "FeedForwardConfig":
        kind = d.get("kind")
        if kind == "dense":
            return cls("dense", _int(d, "ff", where))
        if kind == "moe":
            ex, ro = d.get("expert") or {}, d.get("router") or {}
            cfg = cls("moe", _int(ex, "ff", where + ".expert"), _int(ro, "experts", where + ".router"),
                      _int(ro, "top", where + ".router"), _num(ex, "limit", where + ".expert"))
            if cfg.top > cfg.experts:
                raise ConfigError(f"{where}: top {cfg.top} of {cfg.experts} experts")
            if not cfg.limit > 0:
                raise ConfigError(f"{where}: the experts' limit must be positive")
            return cfg
        raise ConfigError(f"{where}: mlp kind {kind!r} is not known (dense, moe)")


@dataclass(frozen=True)
class LerazenLayer:
    type: str
    mixer: AttentionConfig
    mlp: Optional[FeedForwardConfig]


@dataclass(frozen=True)
class LerazenConfig:
    vocab: int
    width: int
    max_positions: int
    norm_eps: float
    layers: Tuple[LerazenLayer, ...]
    eos_token_id: Optional[int] = None

    @classmethod
    def from_dict(cls, d: Dict[str, Any]) -> "LerazenConfig":
        norm = d.get("norm") or {}
        raw_layers = d.get("layers")
        if not isinstance(raw_layers, list):
            raise ConfigError("config.json lacks the list 'layers'")
        layers = []
        for i, l in enumerate(raw_layers):
            where = f"layers[{i}]"
            if l.get("type") != "attention":
                raise ConfigError(f"{where}: mixer type {l.get('type')!r} is not known (attention)")
            if not isinstance(l.get("mixer"), dict):
                raise ConfigError(f"{where} lacks 'mixer'")
            mlp = l.get("mlp")
            layers.append(LerazenLayer("attention", AttentionConfig.from_dict(l["mixer"], where + ".mixer"),
                                       FeedForwardConfig.from_dict(mlp, where + ".mlp") if mlp else None))
        eps = _num(norm, "eps", "norm")
        if not eps > 0:
            raise ConfigError("norm.eps must be positive")
        mixing = [l.mixer for l in layers if l.mixer.v_mix]
        if any((m.kv_heads, m.vdim) != (mixing[0].kv_heads, mixing[0].vdim) for m in mixing):
            raise ConfigError("layers that mix values must have the same kv_heads and vdim")
        eos = d.get("eos_token_id")
        return cls(vocab=_int(d, "vocab", "config.json"), width=_int(d, "width", "config.json"),
                   max_positions=_int(d, "max_positions", "config.json"), norm_eps=eps, layers=tuple(layers),
                   eos_token_id=eos if isinstance(eos, int) and not isinstance(eos, bool) else None)


def lerazen_spec(cfg: LerazenConfig) -> ModelSpec:
    norm = PartSpec("rms_norm", {"size": cfg.width, "eps": cfg.norm_eps, "weight_name": ""})
    layers, mixing_seen = [], False
    for i, l in enumerate(cfg.layers):
        m = l.mixer
        value_mix = None
        if m.v_mix:
            value_mix = "mix" if mixing_seen else "source"      # the first such layer gives, the later ones take
            mixing_seen = True
        mixer = PartSpec("distance_bias_attention", {
            "hidden_size": cfg.width, "num_heads": m.heads, "num_kv_heads": m.kv_heads, "key_dim": m.dim,
            "value_dim": m.vdim, "scale": m.scale, "window": m.window, "temp_coef": m.temp_coef,
            "temp_every": m.temp_every, "value_mix": value_mix, "unused_mix_tensor": True})
        if l.mlp is None:
            ff = PartSpec("none", {})
        elif l.mlp.kind == "dense":
            ff = PartSpec("relu2_mlp", {"hidden_size": cfg.width, "intermediate_size": l.mlp.ff})
        else:
            ff = PartSpec("routed_experts", {"hidden_size": cfg.width, "expert_size": l.mlp.ff,
                                             "num_experts": l.mlp.experts, "top": l.mlp.top, "limit": l.mlp.limit})
        layers.append(LayerSpec(prefix=f"l{i}", block="parallel",
                                slots={"norm1": ("norm1", norm), "mixer": ("mix", mixer), "ff": ("mlp", ff)}))
    return ModelSpec(
        hidden_size=cfg.width, vocab_size=cfg.vocab, embed_name="embed", layers=layers,
        run_order=[RunEntry(i) for i in range(len(layers))],
        final_norm=norm, final_norm_name="final.norm", head_name="head", eos_token_id=cfg.eos_token_id,
        max_position=cfg.max_positions,
        # a checkpoint may hold a mixing scalar for a layer that does not mix: it is not used
        ignored_tensors=tuple(f"l{i}.mix.vmix" for i, l in enumerate(cfg.layers) if not l.mixer.v_mix),
        before_layers=(("", PartSpec("learned_positions", {"size": cfg.width, "max_positions": cfg.max_positions,
                                                           "name": "pos"})),),
    )


def lerazen_sizes(cfg: LerazenConfig) -> dict:
    """The sizes of a configuration as a flat record (of its first layer and its first routed layer)."""
    out = {"layers": len(cfg.layers), "hidden": cfg.width, "vocab": cfg.vocab, "tied": False}
    if cfg.layers:
        m = cfg.layers[0].mixer
        out.update(q_heads=m.heads, kv_heads=m.kv_heads, head_dim=m.dim, value_dim=m.vdim, window=m.window)
    for l in cfg.layers:
        if l.mlp is not None and l.mlp.kind == "dense":
            out.setdefault("intermediate", l.mlp.ff)
        elif l.mlp is not None:
            out.setdefault("experts", l.mlp.experts)
            out.setdefault("top", l.mlp.top)
            out.setdefault("expert_size", l.mlp.ff)
    return out


def lerazen_with_layers(raw: dict, layers: int) -> dict:
    """The same kinds of layers, ``layers`` of them: the list cut, or repeated from its start."""
    have = raw["layers"]
    return dict(raw, layers=[have[i % len(have)] for i in range(layers)] if have else [])


register_architecture("Lerazen", LerazenConfig.from_dict, lerazen_spec, lerazen_sizes, lerazen_with_layers)
