"""One registry from an architecture's name to its configuration class and model builder.

The reference maps config.json's "model_type" to an enum and matches on it where the
configuration is parsed and where the model is loaded
(core/src/model_executor/models/model_factory.rs:44-50, :285-332, :155-266). Here one table
holds both; an architecture is added by one ``register_architecture`` call and nothing else
in the package names it.
"""
from dataclasses import dataclass
from typing import Any, Callable, Dict, Tuple

from .model_config import ArchConfig, ConfigError, read_config_json


@dataclass(frozen=True)
class Architecture:
    name: str                                   # config.json "architectures"[0]
    model_type: str                             # config.json "model_type" (fallback key)
    config_class: type                          # ArchConfig subclass with from_dict / to_dict
    build_spec: Callable[[Any], Any]            # config -> parts.spec.ModelSpec
    tolerated_tensors: Tuple[str, ...] = ()     # checkpoint names that may be present and are ignored


_ARCHITECTURES: Dict[str, Architecture] = {}
_builtin_loaded = False


def _load_builtin() -> None:
    """Import the package's own architectures once, so that they are registered before a lookup."""
    global _builtin_loaded
    if not _builtin_loaded:
        _builtin_loaded = True
        from .. import models  # noqa: F401


def register_architecture(name: str, model_type: str, config_class: type,
                          build_spec: Callable[[Any], Any],
                          tolerated_tensors: Tuple[str, ...] = (), replace: bool = False) -> Architecture:
    if name in _ARCHITECTURES and not replace:
        raise ValueError("architecture %r is already registered" % name)
    arch = Architecture(name, model_type, config_class, build_spec, tuple(tolerated_tensors))
    _ARCHITECTURES[name] = arch
    return arch


def unregister_architecture(name: str) -> None:
    _ARCHITECTURES.pop(name, None)


def registered_architectures() -> Tuple[str, ...]:
    _load_builtin()
    return tuple(sorted(_ARCHITECTURES))


def get_architecture(name: str) -> Architecture:
    _load_builtin()
    try:
        return _ARCHITECTURES[name]
    except KeyError:
        raise ConfigError("architecture %r is not supported; registered: %s"
                          % (name, ", ".join(registered_architectures()) or "(none)"))


def resolve_architecture(config_dict: Dict[str, Any]) -> Architecture:
    """The architecture that a config.json names: "architectures"[0], else "model_type"
    (case-insensitive, as the reference's strum enum, model_factory.rs:44-50)."""
    _load_builtin()
    archs = config_dict.get("architectures")
    if isinstance(archs, (list, tuple)) and archs:
        return get_architecture(str(archs[0]))
    mt = config_dict.get("model_type")
    if isinstance(mt, str):
        for a in _ARCHITECTURES.values():
            if a.model_type.lower() == mt.lower():
                return a
        raise ConfigError("model_type %r is not supported; registered architectures: %s"
                          % (mt, ", ".join(registered_architectures()) or "(none)"))
    raise ConfigError("config.json names neither 'architectures' nor 'model_type'")


def load_model_config(folder: str) -> Tuple[Architecture, ArchConfig]:
    """Read ``folder``/config.json and parse it with the class its architecture registered."""
    d = read_config_json(folder)
    arch = resolve_architecture(d)
    return arch, arch.config_class.from_dict(d)
