"""Model-name -> engine-class table with the behaviour of the reference's registry
(tybok/registry.py:33-149): backends announce themselves with ``@register(name)`` and are imported on
first use; ``create_engine`` reads the model name from the checkpoint's ``config.json`` (``"type"``)
when it is not given, drops keywords a closed-signature engine does not take, and refuses -- loudly --
any flag the chosen backend declares it does not implement.
"""

from __future__ import annotations

import importlib
import inspect
import json
import os
from typing import TYPE_CHECKING, Any, Callable

if TYPE_CHECKING:
    from .base import PolicyEngine

BACKENDS = ("pi05", "smolvla")
_ENGINES: dict[str, type["PolicyEngine"]] = {}


def register(name: str) -> Callable[[type], type]:
    """Class decorator: make ``cls`` the engine of model type ``name`` (a name can be taken once)."""

    def bind(cls: type) -> type:
        if _ENGINES.setdefault(name, cls) is not cls:
            raise ValueError(f"engine '{name}' already registered")
        return cls

    return bind


def _load_backends() -> None:
    for backend in BACKENDS:
        importlib.import_module(f"{__package__}.policies.{backend}.engine")


def available() -> list[str]:
    """Model types with a registered engine (imports the shipped backends)."""
    _load_backends()
    return sorted(_ENGINES)


def shipped_models() -> list[str]:
    return sorted(BACKENDS)


def detect_model_type(checkpoint_dir: str) -> str:
    """The ``"type"`` field of ``<checkpoint_dir>/config.json``."""
    with open(os.path.join(checkpoint_dir, "config.json"), encoding="utf-8") as handle:
        model_type = json.load(handle).get("type")
    if not model_type:
        raise ValueError(f"checkpoint {checkpoint_dir} has no 'type' field in config.json")
    return model_type


def _accepted_keywords(cls: type, kwargs: dict[str, Any]) -> dict[str, Any]:
    """``kwargs`` restricted to what ``cls.__init__`` names, unless it takes ``**kwargs`` itself."""
    named, open_ended = set(), False
    for pname, param in inspect.signature(cls.__init__).parameters.items():
        if param.kind is inspect.Parameter.VAR_KEYWORD:
            open_ended = True
        elif param.kind in (inspect.Parameter.POSITIONAL_OR_KEYWORD, inspect.Parameter.KEYWORD_ONLY):
            named.add(pname)
    return dict(kwargs) if open_ended else {k: v for k, v in kwargs.items() if k in named}


def reject_unsupported_flags(cls: type, model_type: str, kwargs: dict[str, Any]) -> None:
    """``cls._UNSUPPORTED_FLAGS`` maps each flag the backend does not implement to the value that
    leaves it off; a request carrying any other value for such a flag is an error, not a silent no-op."""
    declared = getattr(cls, "_UNSUPPORTED_FLAGS", None) or {}
    for flag, off_value in declared.items():
        if kwargs.get(flag, off_value) != off_value:
            raise NotImplementedError(f"--{flag.replace('_', '-')} is not supported by the {model_type} backend")


def create_engine(checkpoint_dir: str, model_type: str | None = None, device: str = "auto", **kwargs: Any):
    """Build the engine for ``checkpoint_dir`` (model type from its ``config.json`` unless given)."""
    model_type = model_type or detect_model_type(checkpoint_dir)
    _load_backends()
    try:
        cls = _ENGINES[model_type]
    except KeyError:
        raise ValueError(f"unknown model type {model_type!r}; available: {sorted(_ENGINES)}") from None
    reject_unsupported_flags(cls, model_type, kwargs)
    return cls(checkpoint_dir, device=device, **_accepted_keywords(cls, kwargs))
