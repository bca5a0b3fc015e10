"""Architectures: a name -> (typed configuration, model description) table, and
the one decoder class that runs any description."""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Callable, Mapping, Optional, Tuple

from ..config import ConfigError, read_config_json
from ..parts.spec import ModelSpec
from ..registry import Registry, UnknownName


@dataclass(frozen=True)
class Architecture:
    name: str
    read_config: Callable[[Mapping[str, Any]], Any]   # config.json dict -> typed configuration
    describe: Callable[[Any], ModelSpec]               # typed configuration -> ModelSpec
    # (config.json dict, tensor name -> shape of the stored tensors) -> config.json dict in which the sizes that the
    # file leaves out are filled in from the shapes; None: the design's config.json names every size
    sizes_from_tensors: Optional[Callable[[Mapping[str, Any], Mapping[str, Tuple[int, ...]]], Mapping[str, Any]]] = None


ARCHITECTURES: Registry = Registry("architecture")


def architecture_of(config_json: Mapping[str, Any]) -> Architecture:
    """By `architectures[0]`, then by `architecture`, then by `model_type`."""
    names = list(config_json.get("architectures") or [])
    candidates = names[:1] + [config_json[k] for k in ("architecture", "model_type")
                              if isinstance(config_json.get(k), str) and config_json[k]]
    for n in candidates:
        if n in ARCHITECTURES:
            return ARCHITECTURES.get(n)
    if not candidates:
        raise ConfigError("config.json names no architecture (keys 'architectures', 'architecture' and 'model_type' are all absent)")
    raise ConfigError(f"config.json names architecture {candidates!r}; known: {', '.join(ARCHITECTURES.names())}")


def describe_model(config_json: Mapping[str, Any],
                   tensor_shapes: Optional[Mapping[str, Tuple[int, ...]]] = None) -> Tuple[Architecture, Any, ModelSpec]:
    """`tensor_shapes` (of a model folder's stored tensors): a design whose config.json may leave sizes to the shapes
    gets them filled in before the configuration is read."""
    arch = architecture_of(config_json)
    if tensor_shapes is not None and arch.sizes_from_tensors is not None:
        config_json = arch.sizes_from_tensors(config_json, tensor_shapes)
    cfg = arch.read_config(config_json)
    spec = arch.describe(cfg)
    spec.validate()
    return arch, cfg, spec


from . import gulidra, lesarax, llama, risizen, seredra  # noqa: E402,F401  (they register themselves)
from .decoder import DecoderModel, load_model  # noqa: E402

__all__ = ["ARCHITECTURES", "Architecture", "architecture_of", "describe_model", "DecoderModel", "load_model"]
