"""One registry from architecture name to model, plus named models.

Architectures: config.json's `architectures[0]` -> (config parser, model builder).
Named models: the reference's short name / `family/short` resolution
(engine/models/_registry.py:194-263), each backed by a config.json shipped as data
under config/presets, so no size stands in code.
"""

from __future__ import annotations

import json
from collections import defaultdict
from dataclasses import dataclass
from pathlib import Path
from typing import Any, Callable

_PRESET_DIR = Path(__file__).parent / "presets"


@dataclass(frozen=True)
class Architecture:
    name: str
    parse_config: Callable[[dict], Any]      # raw config.json dict -> typed config
    build_spec: Callable[[Any], Any]         # typed config -> models.spec.ModelSpec


_ARCHITECTURES: dict[str, Architecture] = {}
_MODEL_PRESETS: dict[str, Path] = {}
_MODEL_FAMILY: dict[str, str] = {}
_FAMILY_MODELS: dict[str, list[str]] = defaultdict(list)


def register_architecture(name: str, *, parse_config, build_spec) -> None:
    if name in _ARCHITECTURES:
        raise ValueError(f"Architecture {name} already registered.")
    _ARCHITECTURES[name] = Architecture(name, parse_config, build_spec)


def _ensure_registered() -> None:
    # importing the models package registers the built-in architecture(s)
    import tokensprint_amd.models  # noqa: F401


def get_architecture(name: str) -> Architecture:
    _ensure_registered()
    if name not in _ARCHITECTURES:
        raise ValueError(
            f"Unsupported architecture '{name}'. Registered: {sorted(_ARCHITECTURES)}")
    return _ARCHITECTURES[name]


def architecture_names() -> list[str]:
    _ensure_registered()
    return sorted(_ARCHITECTURES)


def register_named_model(family: str, name: str, preset: Path) -> None:
    """engine/models/_registry.py:130-151: duplicates are rejected."""
    if name in _MODEL_PRESETS:
        raise ValueError(f"Model {name} already registered.")
    _MODEL_PRESETS[name] = Path(preset)
    _MODEL_FAMILY[name] = family
    _FAMILY_MODELS[family].append(name)


def _register_presets() -> None:
    if _MODEL_PRESETS:
        return
    index = json.loads((_PRESET_DIR / "index.json").read_text())
    for family, names in index.items():
        for name in names:
            register_named_model(family, name, _PRESET_DIR / f"{name}.json")


def resolve_model_name(model_name: str) -> str:
    """Short name, or `family/short` when the short name belongs to that family."""
    _register_presets()
    if model_name in _MODEL_PRESETS:
        return model_name
    if "/" in model_name:
        family, short = model_name.split("/", 1)
        if short in _MODEL_PRESETS and _MODEL_FAMILY.get(short) == family:
            return short
    available = ", ".join(sorted(all_registered_repo_ids()))
    raise ValueError(f"Unsupported model_name '{model_name}'. Available models: [{available}]")


def model_is_registered(model_name: str) -> bool:
    try:
        resolve_model_name(model_name)
        return True
    except ValueError:
        return False


def get_model_family(model: str) -> str:
    return _MODEL_FAMILY[resolve_model_name(model)]


def get_model_repo_id(model: str) -> str:
    name = resolve_model_name(model)
    return f"{_MODEL_FAMILY[name]}/{name}"


def get_models_from_family(family: str, newest_first: bool = True) -> list[str]:
    _register_presets()
    models = list(_FAMILY_MODELS[family])
    return models[::-1] if newest_first else models


def all_registered_models(newest_first: bool = True) -> list[str]:
    _register_presets()
    models = list(_MODEL_PRESETS)
    return models[::-1] if newest_first else models


def all_registered_repo_ids(newest_first: bool = True) -> list[str]:
    return [f"{_MODEL_FAMILY[n]}/{n}" for n in all_registered_models(newest_first)]


def load_named_config(model_name: str) -> dict:
    """The raw config.json dict of a named model."""
    name = resolve_model_name(model_name)
    return json.loads(_MODEL_PRESETS[name].read_text())
