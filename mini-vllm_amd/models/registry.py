"""One registry from an architecture's name (``architectures[0]`` of config.json) to what the
engine needs to serve it.

Reference: minivllm/models/models/__init__.py:4-11 maps the name to a model class and
minivllm/models/loader.py:9-15 raises ``ValueError("Model architecture ... is not
supported.")`` for an unknown one. Here the entry is an ``Architecture``: the typed config
class, a function from the config to a ``ModelPlan`` (the layers as data), and the map from
the plan's logical tensor names to the names on disk.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Callable, Dict, FrozenSet, List, Type

from ..config.model_config import ConfigError, ModelConfig, architecture_name, read_config_json
from ..parts.plan import ModelPlan, TensorLocation


@dataclass(frozen=True)
class Architecture:
    name: str
    config_class: Type[ModelConfig]
    plan: Callable[[ModelConfig], ModelPlan]
    tensor_name: Callable[[ModelConfig, TensorLocation], str]
    # names that may be present in the model folder without being used (e.g. a stored copy of
    # a tied output head)
    ignorable: Callable[[ModelConfig], FrozenSet[str]] = lambda config: frozenset()


_ARCHITECTURES: Dict[str, Architecture] = {}


def register_architecture(arch: Architecture, replace: bool = False) -> Architecture:
    if arch.name in _ARCHITECTURES and not replace:
        raise ValueError(f"architecture {arch.name!r} is already registered")
    _ARCHITECTURES[arch.name] = arch
    return arch


def unregister_architecture(name: str) -> None:
    _ARCHITECTURES.pop(name, None)


def get_architecture(name: str) -> Architecture:
    try:
        return _ARCHITECTURES[name]
    except KeyError:
        raise ConfigError(f"Model architecture {name} is not supported "
                          f"(registered: {sorted(_ARCHITECTURES)})") from None


def registered_architectures() -> List[str]:
    return sorted(_ARCHITECTURES)


def config_from_dict(d: Dict[str, Any], where: str = "config.json"):
    """(Architecture, typed config) selected by ``architectures[0]``."""
    arch = get_architecture(architecture_name(d, where))
    return arch, arch.config_class.from_dict(d, where)


def load_config(model_dir: str):
    return config_from_dict(read_config_json(model_dir), where=f"{model_dir}/config.json")
