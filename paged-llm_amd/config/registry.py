"""One table from the architecture name in config.json to the code that builds the model.

The reference accepts exactly one name (pagedllm/model/loader.py:14,24-30); here the name
selects an ``Architecture``: how to read the typed configuration, and how to turn it into a
``ModelSpec`` (the list of layers and their parts).  Another architecture is one more
``register_architecture`` call (the modules of ``models/`` make theirs when that package is imported); nothing
else in the engine names a model.
"""

from __future__ import annotations

import json
import os
from dataclasses import dataclass
from typing import Any, Callable


@dataclass(frozen=True)
class Architecture:
    name: str
    read_config: Callable[[dict], Any]        # config.json dict -> typed configuration
    build_spec: Callable[[Any], Any]          # typed configuration -> ModelSpec


ARCHITECTURES: dict[str, Architecture] = {}


def register_architecture(arch: Architecture) -> None:
    ARCHITECTURES[arch.name] = arch


def lookup_architecture(hf_config: dict) -> Architecture:
    from .. import models  # noqa: F401  (importing the package registers the architectures it ships)
    names = hf_config.get("architectures") or []
    for n in names:
        if n in ARCHITECTURES:
            return ARCHITECTURES[n]
    raise ValueError(f"unsupported architecture {names}; registered: {sorted(ARCHITECTURES)}")


def read_config_json(model_dir: str) -> dict:
    path = os.path.join(model_dir, "config.json")
    if not os.path.isfile(path):
        raise FileNotFoundError(f"{path} not found: a model folder holds config.json and *.safetensors")
    with open(path) as f:
        return json.load(f)
