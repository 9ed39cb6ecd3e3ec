"""One registry from an architecture's name to its configuration class and model builder.

The reference resolves a lowercase substring of ``model_type`` /
``architectures[0]`` to one of a fixed list and dispatches with a ``match``
(crates/infer-protocol/src/config.rs:420-492,
crates/infer-worker/src/bin/worker_main.rs:778-855).  Here the key is the exact
``architectures[0]`` string (``model_type`` as a fallback alias), and anything can
be registered from outside the package.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Callable, Dict, Optional, Type

from .model_config import ConfigError, ModelConfig, read_config_json


@dataclass(frozen=True)
class ArchitectureEntry:
    name: str
    config_cls: Type[ModelConfig]
    # builder(config) -> rustinfer_amd.models.DecoderModel (weights not yet loaded)
    builder: Callable[[ModelConfig], Any]


_ARCHITECTURES: Dict[str, ArchitectureEntry] = {}
_MODEL_TYPE_ALIASES: Dict[str, str] = {}


def register_architecture(name: str, config_cls: Type[ModelConfig],
                          builder: Callable[[ModelConfig], Any],
                          model_type: Optional[str] = None, replace: bool = False) -> None:
    if name in _ARCHITECTURES and not replace:
        raise ValueError(f"architecture {name!r} is already registered")
    _ARCHITECTURES[name] = ArchitectureEntry(name, config_cls, builder)
    if model_type is not None:
        _MODEL_TYPE_ALIASES[model_type] = name


def unregister_architecture(name: str) -> None:
    _ARCHITECTURES.pop(name, None)
    for k in [k for k, v in _MODEL_TYPE_ALIASES.items() if v == name]:
        del _MODEL_TYPE_ALIASES[k]


def registered_architectures():
    return sorted(_ARCHITECTURES)


def resolve_architecture(config_dict: Dict[str, Any], where: str = "config.json") -> ArchitectureEntry:
    """Pick the registry entry for a parsed config.json."""
    _ensure_builtin()
    archs = config_dict.get("architectures")
    hint = None
    if isinstance(archs, list) and archs and isinstance(archs[0], str):
        hint = archs[0]
        if hint in _ARCHITECTURES:
            return _ARCHITECTURES[hint]
    mt = config_dict.get("model_type")
    if isinstance(mt, str):
        if mt in _MODEL_TYPE_ALIASES:
            return _ARCHITECTURES[_MODEL_TYPE_ALIASES[mt]]
        hint = hint or mt
    shown = hint if hint else "<missing architectures/model_type>"
    raise ConfigError(
        f"{where}: unsupported architecture {shown}; registered: "
        f"{', '.join(registered_architectures())}")


def load_model_config(model_dir: str):
    """Read ``model_dir/config.json`` -> (registry entry, typed config)."""
    d = read_config_json(model_dir)
    entry = resolve_architecture(d, where=f"{model_dir}/config.json")
    return entry, entry.config_cls.from_dict(d, where=f"{model_dir}/config.json")


_builtin_done = False


def _ensure_builtin() -> None:
    global _builtin_done
    if _builtin_done:
        return
    _builtin_done = True
    from ..models import llama  # noqa: F401  (registers LlamaForCausalLM)
