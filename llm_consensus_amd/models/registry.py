"""Model registry: which configuration reader and model class serve a checkpoint directory.

A checkpoint names its family in ``config.json``: Hugging Face checkpoints by ``model_type``
(llama, qwen2, mistral, mixtral -> ``TransformerModel``), hybrid decoders by ``architecture``
(Nidozen, Telurax, Surevik -> ``HybridModel``). ``resolve(path)`` returns the family entry; ``loader.load_model``
and ``loader.build_model`` go through it, so the engine, the back ends and the command-line
tools take either kind of directory.
"""
from __future__ import annotations

import json
from dataclasses import dataclass
from pathlib import Path
from typing import Callable, Dict, Tuple


@dataclass(frozen=True)
class Family:
    name: str
    read_config: Callable[[str], object]          # checkpoint dir -> configuration
    load: Callable[..., object]                   # (path, device, **kw) -> model with weights
    kernel_groups: Tuple[str, ...]                # source groups of the kernel library it needs (build_native.py)


# the designs models/hybrid.py serves (its ``DESIGNS``), named here so that finding a checkpoint's
# family does not import the model code
HYBRID_DESIGNS = ("Nidozen", "Telurax", "Surevik", "Gizilorn")

_FAMILIES: Dict[str, Family] = {}
_BY_KEY: Dict[Tuple[str, str], str] = {}          # (config key, value) -> family name


def register(family: Family, keys) -> None:
    _FAMILIES[family.name] = family
    for k in keys:
        _BY_KEY[k] = family.name


def family_of(config: dict) -> Family:
    for key in ("architecture", "model_type"):
        name = _BY_KEY.get((key, str(config.get(key))))
        if name is not None:
            return _FAMILIES[name]
    known = sorted(f"{k}={v}" for k, v in _BY_KEY)
    raise ValueError(f"no model family for this config.json (architecture={config.get('architecture')!r}, "
                     f"model_type={config.get('model_type')!r}); known: {', '.join(known)}")


def resolve(path: str) -> Family:
    p = Path(path)
    p = p / "config.json" if p.is_dir() else p
    return family_of(json.loads(p.read_text()))


def _register_builtin() -> None:
    from . import config as tcfg

    def load_transformer(path, device, **kw):
        from .loader import load_transformer as f

        return f(path, device, **kw)

    def load_hybrid(path, device, **kw):
        from .loader import load_hybrid as f

        return f(path, device, **kw)

    def hybrid_config(path):
        from .hybrid import config_from_path

        return config_from_path(path)

    register(Family("transformer", tcfg.from_hf_config, load_transformer, ("base", "transformer")),
             [("model_type", t) for t in tcfg.SUPPORTED_MODEL_TYPES])
    register(Family("hybrid", hybrid_config, load_hybrid, ("base", "hybrid")),
             [("architecture", a) for a in HYBRID_DESIGNS])


_register_builtin()
