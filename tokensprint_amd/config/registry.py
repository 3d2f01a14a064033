"""One registry from architecture name to model, plus named models.

Architectures: config.json's `architectures[0]` -> (config parser, model builder).
Named models: the reference's short name / `family/short` resolution
(engine/models/_registry.py:194-263), each backed by a config.json shipped as data
under config/presets, so no size stands in code.
"""

from __future__ import annotations

import json
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


@dataclass(frozen=True)
class NamedModel:
    """A model known by name: `short` alone or `family/short` (its repository id)."""

    family: str
    short: str
    preset: Path                             # a config.json kept as data

    @property
    def repo_id(self) -> str:
        return f"{self.family}/{self.short}"


_NAMED: dict[str, NamedModel] = {}           # short name -> model, in order of registration
_presets_read = False


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


# ------------------------------------------------------------------ named models
# Behaviour of engine/models/_registry.py:130-151,194-263: a short name is unique over
# all families, `family/short` names the same model, an unknown name is an error that
# lists what there is.  Kept here as one table and one lookup.


def register_named_model(family: str, name: str, preset: Path) -> None:
    if name in _NAMED:
        raise ValueError(f"Model {name} already registered.")
    _NAMED[name] = NamedModel(family, name, Path(preset))


def _named() -> dict[str, NamedModel]:
    global _presets_read
    if not _presets_read:
        _presets_read = True
        for family, names in json.loads((_PRESET_DIR / "index.json").read_text()).items():
            for name in names:
                if name not in _NAMED:
                    register_named_model(family, name, _PRESET_DIR / f"{name}.json")
    return _NAMED


def lookup(model_name: str) -> NamedModel:
    """The model `model_name` means, given as `short` or as `family/short`."""
    table = _named()
    family, _, short = model_name.rpartition("/")
    found = table.get(short)
    if found is None or (family and family != found.family):
        known = ", ".join(sorted(m.repo_id for m in table.values()))
        raise ValueError(f"Unsupported model_name '{model_name}'. Available models: [{known}]")
    return found


def resolve_model_name(model_name: str) -> str:
    return lookup(model_name).short


def model_is_registered(model_name: str) -> bool:
    try:
        lookup(model_name)
    except ValueError:
        return False
    return True


def get_model_family(model: str) -> str:
    return lookup(model).family


def get_model_repo_id(model: str) -> str:
    return lookup(model).repo_id


def models_by_family() -> dict[str, list[NamedModel]]:
    """Every named model under its family, families and models in order of registration."""
    out: dict[str, list[NamedModel]] = {}
    for m in _named().values():
        out.setdefault(m.family, []).append(m)
    return out


def get_models_from_family(family: str, newest_first: bool = True) -> list[str]:
    names = [m.short for m in models_by_family().get(family, [])]
    return names[::-1] if newest_first else names


def all_registered_models(newest_first: bool = True) -> list[str]:
    names = list(_named())
    return names[::-1] if newest_first else names


def all_registered_repo_ids(newest_first: bool = True) -> list[str]:
    return [_NAMED[n].repo_id for n in all_registered_models(newest_first)]


def load_named_config(model_name: str) -> dict:
    """The raw config.json dict of a named model."""
    return json.loads(lookup(model_name).preset.read_text())
