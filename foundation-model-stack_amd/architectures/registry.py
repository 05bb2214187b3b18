"""One registry from an architecture's name to what builds it, and from
(architecture, variant) to a configuration.

The calls mirror the reference's (fms/models/__init__.py:31-69): registering a
name twice raises KeyError, asking for an unknown name raises KeyError.
"""

from __future__ import annotations

import dataclasses
from typing import Callable, Dict, List, Tuple, Type

from ..config import ModelConfig
from ..parts import ModelSpec


@dataclasses.dataclass
class Architecture:
    name: str
    config_class: Type[ModelConfig]
    build_spec: Callable[[ModelConfig], ModelSpec]  # configuration -> which parts, in which order
    hf_architectures: Tuple[str, ...] = ()  # names in a config.json's "architectures" that mean this one
    from_hf_dict: Callable[[dict], ModelConfig] = None  # config.json (Hugging Face keys) -> configuration
    to_hf_dict: Callable[[ModelConfig], dict] = None
    hf_tensor_layout: Callable[[ModelConfig], list] = None  # names/shapes/inits of a Hugging Face checkpoint
    detect_source: Callable[[list], str] = None  # a checkpoint's tensor names -> the name of its source (adapter)


_architectures: Dict[str, Architecture] = {}
_variants: Dict[str, Dict[str, Callable[..., ModelConfig]]] = {}


def register_architecture(arch: Architecture) -> None:
    if arch.name in _architectures:
        raise KeyError(f"architecture {arch.name!r} is already registered")
    _architectures[arch.name] = arch
    _variants.setdefault(arch.name, {})


def get_architecture(name: str) -> Architecture:
    if name not in _architectures:
        raise KeyError(f"{name} is not registered; known architectures: {list_models()}")
    return _architectures[name]


def architecture_for_hf(hf_name: str) -> Architecture:
    for arch in _architectures.values():
        if hf_name in arch.hf_architectures:
            return arch
    known = sorted(n for a in _architectures.values() for n in a.hf_architectures)
    raise KeyError(f"config.json names architecture {hf_name!r}, which this library does not have; it has {known}")


def register_model(architecture: str, variant: str, factory: Callable[..., ModelConfig]) -> None:
    """`factory(**overrides)` returns the variant's configuration (fms/models/__init__.py:31-48)."""
    variants = _variants.setdefault(architecture, {})
    if variant in variants:
        raise KeyError(f"Variant {variant} already registered for architecture {architecture}")
    variants[variant] = factory


def list_models() -> List[str]:
    return sorted(_variants)


def list_variants(architecture: str) -> List[str]:
    if architecture not in _variants:
        raise KeyError(f"{architecture} is not registered. See `models.list_models()` for available architectures")
    return sorted(_variants[architecture])


def variant_config(architecture: str, variant: str, **overrides) -> ModelConfig:
    if architecture not in _variants:
        raise KeyError(f"{architecture} is not registered. See `models.list_models()` for available architectures")
    if variant not in _variants[architecture]:
        raise KeyError(f'{variant} is not a registered variant of {architecture}. See `models.list_variants("{architecture}")`')
    return _variants[architecture][variant](**overrides)
