"""One registry from an architecture's name to its configuration class.

The reference keeps a table of registry rows and scans it by name
(`src/compat/architecture.cpp:415-426`); an unknown name is refused with the
list of the supported ones (`src/compat/architecture.cpp:578-585`). Here a
row is a configuration class with `from_json(dict)` and `plan()`; the model
itself is always the generic decoder built from the plan.
"""

from __future__ import annotations

import inspect
import json
import os
from typing import Callable, Dict, List

from ..errors import InvalidModel, Unsupported

_ARCHITECTURES: Dict[str, type] = {}
_MODEL_TYPES: Dict[str, str] = {}


def register_architecture(name: str, config_cls: type, model_types: List[str] = ()) -> None:
    """Registers `config_cls` under config.json's `architectures[0]` name and,
    optionally, under `model_type` values that mean the same architecture."""
    _ARCHITECTURES[name] = config_cls
    for mt in model_types:
        _MODEL_TYPES[mt] = name


def supported_architectures() -> str:
    return ",".join(sorted(_ARCHITECTURES))


def find_architecture(name: str) -> type:
    cls = _ARCHITECTURES.get(name)
    if cls is None:
        raise Unsupported(
            f"architecture '{name}' is not supported yet (supported: {supported_architectures()})"
        )
    return cls


def architecture_name_of(raw: dict) -> str:
    archs = raw.get("architectures")
    if isinstance(archs, list) and archs and isinstance(archs[0], str):
        return archs[0]
    arch = raw.get("architecture")
    if isinstance(arch, str):
        return arch
    mt = raw.get("model_type")
    if isinstance(mt, str):
        if mt in _MODEL_TYPES:
            return _MODEL_TYPES[mt]
        raise Unsupported(
            f"architecture '{mt}' is not supported yet (supported: {supported_architectures()})"
        )
    raise InvalidModel("not a model folder: config.json has neither 'architectures' nor 'architecture' nor 'model_type'")


def config_from_dict(raw: dict, shapes=None):
    """Typed configuration for a parsed config.json. `shapes` (tensor name -> shape, of the weights file beside it) goes
    to configuration classes that read sizes from tensors' shapes (`from_json(raw, shapes=)`)."""
    if not isinstance(raw, dict):
        raise InvalidModel("config.json must hold a JSON object")
    cls = find_architecture(architecture_name_of(raw))
    if shapes is not None and "shapes" in inspect.signature(cls.from_json).parameters:
        return cls.from_json(raw, shapes=shapes)
    return cls.from_json(raw)


def load_config(model_dir: str):
    path = os.path.join(model_dir, "config.json")
    if not os.path.isfile(path):
        raise InvalidModel(f"not a model folder: '{path}' is missing")
    try:
        with open(path, "r", encoding="utf-8") as f:
            raw = json.load(f)
    except json.JSONDecodeError as e:
        raise InvalidModel(f"config.json is not valid JSON: {e}") from None
    shapes = None
    weights = os.path.join(model_dir, "model.safetensors")
    if os.path.isfile(weights):
        from ..weights.safetensors_io import SafetensorsFile

        shapes = {name: e.shape for name, e in SafetensorsFile(weights).entries.items()}
    return config_from_dict(raw, shapes)
