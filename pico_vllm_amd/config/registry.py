"""One registry from an architecture's name (``architectures[0]`` of
config.json, or its ``architecture``) to its typed configuration and its model description.

The reference has no registry: its entry script imports the one model class
directly (pico_vllm/run_single.py:2,10-11).
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Callable, Dict, Optional

from .model_config import ConfigError, read_config_json


@dataclass(frozen=True)
class Architecture:
    name: str
    config_from_dict: Callable[[Dict[str, Any]], Any]   # raw config.json -> typed config
    build_spec: Callable[[Any], Any]                     # typed config -> parts.spec.ModelSpec
    # for reports and measurements, so that the programs that make them read no architecture's keys:
    sizes: Optional[Callable[[Any], Dict[str, Any]]] = None          # typed config -> flat {name: number} of its sizes
    with_layers: Optional[Callable[[Dict[str, Any], int], Dict[str, Any]]] = None   # raw config, n -> the same layer sizes, n layers
    # True: config_from_dict takes a second argument, {tensor name: shape} of the checkpoint (or None where there is
    # none yet), for sizes that config.json leaves to the tensors
    reads_shapes: bool = False


_ARCHITECTURES: Dict[str, Architecture] = {}


def register_architecture(name: str, config_from_dict, build_spec, sizes=None, with_layers=None,
                          reads_shapes: bool = False) -> Architecture:
    arch = Architecture(name, config_from_dict, build_spec, sizes, with_layers, reads_shapes)
    _ARCHITECTURES[name] = arch
    return arch


def known_architectures():
    return sorted(_ARCHITECTURES)


def resolve_architecture(raw_config: Dict[str, Any]) -> Architecture:
    names = raw_config.get("architectures")
    if not names and isinstance(raw_config.get("architecture"), str):
        names = [raw_config["architecture"]]
    if not names:
        raise ConfigError("config.json has no 'architectures' entry; known architectures: "
                          + ", ".join(known_architectures()))
    name = names[0]
    if name not in _ARCHITECTURES:
        raise ConfigError(f"architecture {name!r} is not registered; known architectures: "
                          + ", ".join(known_architectures()))
    return _ARCHITECTURES[name]


def load_model_description(model_dir: str):
    """(architecture, typed config, ModelSpec) of a model folder."""
    raw = read_config_json(model_dir)
    arch = resolve_architecture(raw)
    if arch.reads_shapes:
        cfg = arch.config_from_dict(raw, checkpoint_shapes(model_dir))
    else:
        cfg = arch.config_from_dict(raw)
    return arch, cfg, arch.build_spec(cfg)


def checkpoint_shapes(model_dir: str) -> Dict[str, tuple]:
    """{tensor name: shape} from the headers of the folder's safetensors files (no tensor is read)."""
    from ..weights.safetensors_io import SafetensorsFile, list_safetensors
    out: Dict[str, tuple] = {}
    for path in list_safetensors(model_dir):
        with SafetensorsFile(path) as sf:
            for name, (_, shape) in sf.entries.items():
                out[name] = tuple(shape)
    return out
