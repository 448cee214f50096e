"""Architecture registry: which config reader, model class and weight loader
serve a checkpoint directory, chosen by its config.json.

A family registers under the names it answers to in config.json —
"architectures": [...] (HF layout) or "architecture": "..." — and provides
`load(path, device, dtype, **kw) -> model`.  Named built-in configs of every
family live in CONFIGS (models/__init__.py); a config object builds its own
model through `build_model(device, dtype)`.
"""
from __future__ import annotations

import json
from pathlib import Path
from typing import Callable

_LOADERS: dict[str, Callable] = {}


def register_architecture(names, load: Callable) -> None:
    for n in ([names] if isinstance(names, str) else names):
        _LOADERS[n] = load


def architecture_of(path: str) -> str:
    c = json.loads((Path(path) / "config.json").read_text())
    if isinstance(c.get("architecture"), str):
        return c["architecture"]
    archs = c.get("architectures") or []
    if archs:
        return archs[0]
    raise ValueError(f"{path}/config.json names no architecture")


def registered() -> list[str]:
    return sorted(_LOADERS)


def load_model(path: str, device="cpu", dtype=None, **kw):
    """Build the model a checkpoint directory describes and load its
    weights.  Raises KeyError for an architecture no family registered."""
    import torch
    arch = architecture_of(path)
    if arch not in _LOADERS:
        raise KeyError(f"no model family registered for architecture "
                       f"{arch!r} (known: {', '.join(registered())})")
    return _LOADERS[arch](path, device=device,
                          dtype=dtype or torch.bfloat16, **kw)


def build_model(cfg, device="cpu", dtype=None):
    """Random-weight model for a config object of any family."""
    import torch
    dtype = dtype or torch.bfloat16
    if hasattr(cfg, "build_model"):
        return cfg.build_model(device=device, dtype=dtype)
    from .llama import LlamaForCausalLM
    return LlamaForCausalLM(cfg, device=device, dtype=dtype)


def _load_llama(path, device="cpu", dtype=None, **kw):
    from .checkpoint import config_from_dir, load_checkpoint
    from .llama import LlamaForCausalLM
    cfg = config_from_dir(path)
    if kw.get("max_position"):
        cfg.max_position = kw["max_position"]
    model = LlamaForCausalLM(cfg, device=device, dtype=dtype)
    return load_checkpoint(model, path).eval()


def _load_reperax(path, device="cpu", dtype=None, **kw):
    from .hybrid import load_reperax
    return load_reperax(path, device=device, dtype=dtype,
                        max_position=kw.get("max_position"))


def _load_zudisun(path, device="cpu", dtype=None, **kw):
    from .zudisun import load_zudisun
    return load_zudisun(path, device=device, dtype=dtype,
                        max_position=kw.get("max_position"))


def _load_fugevik(path, device="cpu", dtype=None, **kw):
    from .fugevik import load_fugevik
    return load_fugevik(path, device=device, dtype=dtype,
                        max_position=kw.get("max_position"))


def _load_vabedra(path, device="cpu", dtype=None, **kw):
    from .vabedra import load_vabedra
    return load_vabedra(path, device=device, dtype=dtype,
                        max_position=kw.get("max_position"))


register_architecture(["LlamaForCausalLM", "MistralForCausalLM",
                       "MixtralForCausalLM"], _load_llama)
register_architecture("Reperax", _load_reperax)
register_architecture("Zudisun", _load_zudisun)
register_architecture("Fugevik", _load_fugevik)
register_architecture("Vabedra", _load_vabedra)
