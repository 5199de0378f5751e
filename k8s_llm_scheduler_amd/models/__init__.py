"""Model registry: a preset name, ``<preset>@L<n>``, or a checkpoint directory / config.json resolves to a
configuration, and a configuration to the model class that runs it.  A config.json names its design in
``architecture`` (this framework's own designs) or ``architectures`` (HuggingFace checkpoints)."""

from __future__ import annotations

import json
from pathlib import Path


def _architecture(c: dict) -> str:
    a = c.get("architecture") or (c.get("architectures") or [""])[0] or c.get("model_type", "")
    return str(a)


def load_config(name_or_path: str):
    """The configuration object of a preset or checkpoint."""
    from . import nukizen, putulorn, rupatar, semanex
    from .config import get_config

    designs = (putulorn, rupatar, nukizen, semanex)
    for d in designs:
        if name_or_path in d.PRESETS:
            return d.PRESETS[name_or_path]
    p = Path(name_or_path)
    if p.is_dir():
        p = p / "config.json"
    if p.is_file():
        c = json.loads(p.read_text())
        for d in designs:
            if _architecture(c) == d.ARCHITECTURE:
                return d.config_from_json(c, p.parent.name or d.ARCHITECTURE.lower())
    return get_config(name_or_path)


def model_class(cfg):
    """The model class of a configuration object."""
    from .config import LlamaConfig
    from .llama import LlamaModel
    from .nukizen import NukizenConfig, NukizenModel
    from .putulorn import PutulornConfig, PutulornModel
    from .rupatar import RupatarConfig, RupatarModel
    from .semanex import SemanexConfig, SemanexModel

    if isinstance(cfg, PutulornConfig):
        return PutulornModel
    if isinstance(cfg, RupatarConfig):
        return RupatarModel
    if isinstance(cfg, NukizenConfig):
        return NukizenModel
    if isinstance(cfg, SemanexConfig):
        return SemanexModel
    if isinstance(cfg, LlamaConfig):
        return LlamaModel
    raise TypeError(f"no model class for {type(cfg).__name__}")
