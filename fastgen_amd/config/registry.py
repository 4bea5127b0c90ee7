"""One registry from the architecture name in ``config.json`` to the code
that reads its configuration and lays its layers out.

The reference matches ``config["architectures"]`` against one-element lists
and raises ``RuntimeError("Unsupported model type ...")`` otherwise
(``fastgen/utils/loading.py:236-244``).
"""

from __future__ import annotations

from typing import Any, Dict, Mapping, Protocol

from .layout import ModelLayout
from .model_args import ConfigError, architecture_name


class Architecture(Protocol):
    """What an architecture has to offer to be served.

    ``parse`` turns the keys of ``config.json`` into a typed record,
    ``layout`` turns that record into parts and a run order, and
    ``to_hf_config`` writes the record back as ``config.json`` keys (used
    by the random-weights mode).
    """

    name: str

    def parse(self, config: Mapping[str, Any]) -> Any: ...

    def layout(self, args: Any) -> ModelLayout: ...

    def to_hf_config(self, args: Any) -> dict: ...


_ARCHITECTURES: Dict[str, Architecture] = {}


def register_architecture(arch: Architecture, *, replace: bool = False) -> Architecture:
    if arch.name in _ARCHITECTURES and not replace:
        raise ValueError(f"architecture {arch.name!r} is already registered")
    _ARCHITECTURES[arch.name] = arch
    return arch


def unregister_architecture(name: str) -> None:
    _ARCHITECTURES.pop(name, None)


def get_architecture(name_or_config: str | Mapping[str, Any]) -> Architecture:
    if isinstance(name_or_config, str):
        name = name_or_config
    else:
        name = architecture_name(name_or_config)
    if name not in _ARCHITECTURES:
        raise ConfigError(
            f"Unsupported model type {name!r}; registered architectures:"
            f" {sorted(_ARCHITECTURES)}"
        )
    return _ARCHITECTURES[name]


def registered_architectures() -> list[str]:
    return sorted(_ARCHITECTURES)
