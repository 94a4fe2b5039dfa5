"""One registry from the architecture name in config.json to everything that builds
its model: the typed configuration, the layer plan and the checkpoint's tensor names.

The reference accepts exactly one name through a constant (atomserve/config.py:11,
34-38); here the same check is a table lookup, so another architecture is one more
`register_architecture` call and no change elsewhere.
"""

import json
import os
from dataclasses import dataclass
from typing import Any, Callable

from atomserve_amd.config.model_config import ConfigError


@dataclass(frozen=True)
class Architecture:
    """name:           the string in config.json's `architectures`
    parse_config:   raw config.json dict -> typed configuration (validates)
    build_plan:     typed configuration -> parts.plan.ModelPlan (layers as data)
    checkpoint_map: typed configuration -> {plan tensor name: [checkpoint names to stack]}
    checkpoint_shapes: typed configuration -> {checkpoint name: (shape, "matrix" | "vector")},
                    in the order in which random weights are drawn
    ignored:        typed configuration -> checkpoint names that may be present and unused
    """

    name: str
    parse_config: Callable[[dict], Any]
    build_plan: Callable[[Any], Any]
    checkpoint_map: Callable[[Any], dict]
    checkpoint_shapes: Callable[[Any], dict]
    ignored: Callable[[Any], set] = lambda config: set()


_ARCHITECTURES: dict[str, Architecture] = {}


def register_architecture(arch: Architecture, replace: bool = False) -> Architecture:
    if arch.name in _ARCHITECTURES and not replace:
        raise ValueError(f"architecture {arch.name!r} is already registered")
    _ARCHITECTURES[arch.name] = arch
    return arch


def supported_architectures() -> list[str]:
    _load_builtin()
    return sorted(_ARCHITECTURES)


def architecture_for(raw: dict) -> Architecture:
    """The registered architecture that config.json names, or a ConfigError listing what is."""
    _load_builtin()
    names = raw.get("architectures") or []
    if len(names) != 1 or names[0] not in _ARCHITECTURES:
        raise ConfigError(
            f"atomserve_amd only supports {', '.join(sorted(_ARCHITECTURES))}; "
            f"config.json names {names}"
        )
    return _ARCHITECTURES[names[0]]


def load_model_config(model_dir: str) -> tuple[Architecture, Any]:
    """Read `<model_dir>/config.json`; returns (architecture, typed configuration)."""
    path = os.path.join(model_dir, "config.json")
    if not os.path.isfile(path):
        raise FileNotFoundError(f"no config.json in {model_dir}")
    with open(path) as f:
        raw = json.load(f)
    arch = architecture_for(raw)
    return arch, arch.parse_config(raw)


def _load_builtin() -> None:
    # Imported lazily: the model modules import parts, which import this package.
    import atomserve_amd.models.qwen3  # noqa: F401
