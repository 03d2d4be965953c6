"""One registry from an architecture's name (``model_type`` in config.json) to
its configuration class and the function that turns a configuration into a
ModelSpec.  The reference matches on ``model_type`` in its entry points
(infernum-examples/examples/generate.rs:128-144,263-291), with "llama" as the
default when the key is absent.
"""
from __future__ import annotations

from typing import Any, Callable, Dict, List, Mapping, Tuple

from .base import ConfigError, UnsupportedModelError, read_config_json

_ARCHITECTURES: Dict[str, Tuple[Any, Callable[..., Any]]] = {}
DEFAULT_MODEL_TYPE = "llama"


def register_architecture(model_type: str, config_cls: Any, spec_builder: Callable[..., Any],
                          replace: bool = False) -> None:
    """``config_cls.from_dict(raw, where)`` reads config.json; ``spec_builder(config)`` gives the ModelSpec."""
    if model_type in _ARCHITECTURES and not replace and _ARCHITECTURES[model_type] != (config_cls, spec_builder):
        raise ValueError(f"architecture {model_type!r} is registered already")
    _ARCHITECTURES[model_type] = (config_cls, spec_builder)


def registered_architectures() -> List[str]:
    return sorted(_ARCHITECTURES)


def resolve_architecture(model_type: str) -> Tuple[Any, Callable[..., Any]]:
    try:
        return _ARCHITECTURES[model_type]
    except KeyError:
        raise UnsupportedModelError(
            f'Unsupported model_type: "{model_type}". Supported: {", ".join(registered_architectures())}') from None


def config_from_dict(raw: Mapping[str, Any], where: str = "config.json") -> Any:
    model_type = raw.get("model_type", DEFAULT_MODEL_TYPE)
    if not isinstance(model_type, str):
        raise ConfigError(f"{where}: 'model_type' must be a string")
    config_cls, _ = resolve_architecture(model_type)
    return config_cls.from_dict(raw, where)


def load_config(model_dir: str) -> Any:
    """Read ``model_dir/config.json`` with the configuration class of its model_type."""
    return config_from_dict(read_config_json(model_dir), where=str(model_dir))


def model_spec_for(config: Any, **kw: Any) -> Any:
    _, builder = resolve_architecture(config.model_type)
    return builder(config, **kw)
