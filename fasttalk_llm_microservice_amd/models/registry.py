"""Architecture registry: which configuration parser and which model class serve a
checkpoint directory or a registry name.

An architecture registers (a) how its ``config.json`` is recognised and parsed and
(b) a factory for its model class.  ``resolve_config`` is what the engine calls with
``EngineConfig.model`` / ``EngineConfig.weights``; ``build_model`` is what the model
runner calls.  Llama-3 (HF ``config.json``) is the default architecture; a
``config.json`` with an ``"architecture"`` key picks its architecture by that name.
"""
from __future__ import annotations

import dataclasses
import json
import os
from typing import Any, Callable, Dict, Optional


@dataclasses.dataclass
class Architecture:
    name: str
    # parsed config.json dict -> bool
    matches: Callable[[dict], bool]
    # (config.json dict, checkpoint dir name) -> config object
    parse: Callable[[dict, str], Any]
    # (cfg, device, dtype, comm, max_model_len, quantization) -> model
    build: Callable[..., Any]
    # registry names of this architecture (random-init shapes): name -> config object
    presets: Dict[str, Any] = dataclasses.field(default_factory=dict)


ARCHITECTURES: Dict[str, Architecture] = {}


def register(arch: Architecture):
    ARCHITECTURES[arch.name.lower()] = arch


_loaded = False


def _ensure_loaded():
    global _loaded
    if _loaded:
        return
    _loaded = True
    from . import bagasun, fufipel, kerarax, llama_arch, nulazen  # noqa: F401  (each registers itself)


def architecture_of(cfg) -> Architecture:
    _ensure_loaded()
    name = getattr(cfg, "architecture", "llama").lower()
    return ARCHITECTURES[name]


def config_from_dir(path: str):
    """The configuration object of a checkpoint directory (``config.json``)."""
    _ensure_loaded()
    with open(os.path.join(path, "config.json")) as f:
        c = json.load(f)
    name = os.path.basename(os.path.normpath(path)) or "model"
    # an explicit architecture name wins; Llama (HF layout) is the default
    for arch in ARCHITECTURES.values():
        if arch.name != "llama" and arch.matches(c):
            return arch.parse(c, name)
    return ARCHITECTURES["llama"].parse(c, name)


def preset(name: str) -> Optional[Any]:
    _ensure_loaded()
    low = name.strip().lower()
    for arch in ARCHITECTURES.values():
        if low in arch.presets:
            return arch.presets[low]
    return None


def build_model(cfg, device, dtype, comm, max_model_len: int, quantization: Optional[str] = None):
    return architecture_of(cfg).build(cfg, device, dtype, comm, max_model_len, quantization)
