"""One registry from an architecture's name (config.json ``architectures[0]``)
to the pair (hyper-parameter class, function that lays out the model).

The reference registers one torch class per architecture
(src/csrc/pybinding.cc:53-80) and picks hyper-parameters by model name
(src/examples/lib/common_gpt_hyper_params.h:105-130).  Here the name in
config.json selects both, and another architecture is one more
``register_architecture`` call."""
from __future__ import annotations

import json
import os
from dataclasses import dataclass
from typing import Any, Callable, Dict, Optional

from .hyper_param import ConfigError


@dataclass(frozen=True)
class Architecture:
    name: str
    hyper_param_cls: Any                     # has from_dict(dict) and to_config_dict()
    build_spec: Callable[[Any], Any]         # hyper param -> parts.spec.ModelSpec
    short_name: str = ""                     # e.g. "opt": prefix of reference-style model names
    presets: Optional[Callable[..., Any]] = None   # (model name, **overrides) -> hyper param, for named sizes


_ARCHITECTURES: Dict[str, Architecture] = {}


def register_architecture(name: str, hyper_param_cls, build_spec, short_name: str = "",
                          presets: Optional[Callable[..., Any]] = None) -> None:
    """``presets(model_name, **overrides)`` (optional) returns the hyper-parameters of a named size
    (``<short_name>_<size>``) for runs that have no config.json."""
    _ARCHITECTURES[name] = Architecture(name, hyper_param_cls, build_spec, short_name, presets)


def hyper_param_by_name(model_name: str, **overrides):
    """Hyper-parameters of a reference-style model name (``opt_1.3b``): the family before the
    first ``_`` or ``-`` selects the architecture, whose ``presets`` know its sizes
    (src/examples/lib/common_gpt_hyper_params.h:105-130 looks names up the same way).  Raises
    KeyError with the valid names."""
    _ensure_builtin()
    family = model_name.lower().replace("-", "_").split("_")[0]
    for arch in _ARCHITECTURES.values():
        if arch.short_name and arch.short_name == family and arch.presets is not None:
            return arch.presets(model_name, **overrides)
    families = sorted(a.short_name for a in _ARCHITECTURES.values() if a.short_name and a.presets is not None)
    raise KeyError(f"invalid model name {model_name!r}: no registered architecture has sizes named "
                   f"{family}_*; families: {' '.join(families)}")


def registered_architectures():
    _ensure_builtin()
    return sorted(_ARCHITECTURES)


def _ensure_builtin() -> None:
    # the built-in architecture registers itself on import
    from ..models import opt  # noqa: F401


def resolve_architecture(name: str) -> Architecture:
    _ensure_builtin()
    if name not in _ARCHITECTURES:
        raise ConfigError(
            f"unknown architecture {name!r}; registered: {sorted(_ARCHITECTURES)}")
    return _ARCHITECTURES[name]


def read_config(model_dir: str) -> Dict[str, Any]:
    path = os.path.join(model_dir, "config.json")
    if not os.path.isfile(path):
        raise ConfigError(f"{model_dir!r} has no config.json")
    with open(path, "r", encoding="utf-8") as f:
        return json.load(f)


def hyper_param_from_dir(model_dir: str):
    """(architecture, typed hyper-parameters) of the model in ``model_dir``."""
    cfg = read_config(model_dir)
    archs = cfg.get("architectures")
    if archs:
        arch = resolve_architecture(archs[0])
    else:
        # no class name: fall back to the family name ("model_type": "opt")
        _ensure_builtin()
        family = str(cfg.get("model_type", "")).lower()
        matches = [a for a in _ARCHITECTURES.values() if a.short_name and a.short_name == family]
        if not matches:
            raise ConfigError("config.json names no architecture: neither 'architectures' nor a known "
                              f"'model_type' (registered: {sorted(_ARCHITECTURES)})")
        arch = matches[0]
        cfg = dict(cfg, architectures=[arch.name])
    return arch, arch.hyper_param_cls.from_dict(cfg)
