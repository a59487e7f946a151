"""Model registry with the reference's contract (tybok/registry.py:33-149): ``@register(name)``,
lazy backend import, ``detect_model_type`` from ``config.json``'s ``type`` field, keyword
filtering for closed-signature engines and loud rejection of flags a backend does not implement.
"""

from __future__ import annotations

import importlib
import inspect
import json
import os
from typing import TYPE_CHECKING, Any

if TYPE_CHECKING:
    from .base import PolicyEngine

_REGISTRY: dict[str, type["PolicyEngine"]] = {}
BACKENDS = ("pi05", "smolvla")


def register(name: str):
    def deco(cls):
        if name in _REGISTRY:
            raise ValueError(f"engine '{name}' already registered")
        _REGISTRY[name] = cls
        return cls

    return deco


def _ensure_backends() -> None:
    for name in BACKENDS:
        importlib.import_module(f"{__package__}.policies.{name}.engine")


def available() -> list[str]:
    _ensure_backends()
    return sorted(_REGISTRY)


def shipped_models() -> list[str]:
    return sorted(BACKENDS)


def detect_model_type(checkpoint_dir: str) -> str:
    with open(os.path.join(checkpoint_dir, "config.json"), "r", encoding="utf-8") as f:
        mtype = json.load(f).get("type")
    if not mtype:
        raise ValueError(f"checkpoint {checkpoint_dir} has no 'type' field in config.json")
    return mtype


def _engine_kwargs(cls, kwargs: dict[str, Any]) -> dict[str, Any]:
    params = inspect.signature(cls.__init__).parameters
    if any(p.kind is inspect.Parameter.VAR_KEYWORD for p in params.values()):
        return kwargs
    accepted = {n for n, p in params.items() if p.kind in (p.POSITIONAL_OR_KEYWORD, p.KEYWORD_ONLY)}
    return {k: v for k, v in kwargs.items() if k in accepted}


def reject_unsupported_flags(cls, model_type: str, kwargs: dict[str, Any]) -> None:
    """``cls._UNSUPPORTED_FLAGS`` maps a flag to its inert value; any other value was requested."""
    for flag, inert in (getattr(cls, "_UNSUPPORTED_FLAGS", None) or {}).items():
        if flag in kwargs and kwargs[flag] != inert:
            raise NotImplementedError(f"--{flag.replace('_', '-')} is not supported by the {model_type} backend")


def create_engine(checkpoint_dir: str, model_type: str | None = None, device: str = "auto", **kwargs: Any):
    if model_type is None:
        model_type = detect_model_type(checkpoint_dir)
    _ensure_backends()
    cls = _REGISTRY.get(model_type)
    if cls is None:
        raise ValueError(f"unknown model type {model_type!r}; available: {available()}")
    reject_unsupported_flags(cls, model_type, kwargs)
    return cls(checkpoint_dir, device=device, **_engine_kwargs(cls, kwargs))
