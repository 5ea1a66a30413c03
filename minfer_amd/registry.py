"""One registry from an architecture's name (config.json `architectures[0]`) to its
configuration class, which in turn describes the model.

The reference selects its model by the architecture string of the file it loads and answers
an unknown one with `Unsupported architecture: '<x>'` (src/models/mod.rs:74-87 of
yusiwen/minfer); here an unknown name is an error that also lists the registered names.
"""
from __future__ import annotations

from typing import Any, Dict

from .config.base import ConfigError, architecture_name, read_config_json

_ARCHITECTURES: Dict[str, Any] = {}


def register_architecture(name: str, config_class: Any) -> None:
    """`config_class.from_dict(raw)` must return an object with `model_spec()` and
    `to_dict()`; see `minfer_amd.config.qwen2.Qwen2Config`."""
    for attr in ("from_dict", "model_spec"):
        if not hasattr(config_class, attr):
            raise TypeError(f"configuration class for {name!r} lacks {attr}()")
    _ARCHITECTURES[name] = config_class


def registered_architectures():
    return sorted(_ARCHITECTURES)


def config_from_dict(raw: Dict[str, Any]):
    name = architecture_name(raw)
    if name not in _ARCHITECTURES:
        raise ConfigError(f"Unsupported architecture: {name!r}; registered: "
                          f"{', '.join(registered_architectures()) or '(none)'}")
    return _ARCHITECTURES[name].from_dict(raw)


def load_config(folder_or_file: str):
    return config_from_dict(read_config_json(folder_or_file))


def _register_builtin() -> None:
    from .config.qwen2 import ARCHITECTURE, Qwen2Config
    register_architecture(ARCHITECTURE, Qwen2Config)


_register_builtin()
