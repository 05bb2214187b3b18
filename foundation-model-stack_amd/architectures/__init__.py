from . import llama  # noqa: F401  (registers the architecture, its adapters and variants)
from .registry import (
    Architecture,
    architecture_for_hf,
    get_architecture,
    list_models,
    list_variants,
    register_architecture,
    register_model,
    variant_config,
)

__all__ = [
    "Architecture", "architecture_for_hf", "get_architecture", "list_models", "list_variants",
    "register_architecture", "register_model", "variant_config",
]
