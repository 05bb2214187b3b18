"""fms_amd: a Llama library for one AMD MI355X — configuration, weights, parts, a paged
sequence cache, one ragged step function on hand-written gfx950 kernels, sampling and a
generation loop.  Importing the package touches no GPU; the kernel library is compiled
(if no built copy is found) and loaded when the first kernel is called."""

from . import architectures as _architectures  # noqa: F401  (fills the registries)
from .architectures import list_models, list_variants, register_architecture, register_model
from .config import LLaMAConfig, ModelConfig
from .models import LLaMA, from_config, get_model, write_model_folder

__all__ = [
    "LLaMA", "LLaMAConfig", "ModelConfig", "from_config", "get_model", "write_model_folder", "list_models", "list_variants",
    "register_architecture", "register_model", "generate", "generate_requests", "pad_input_ids", "Engine",
]


def __getattr__(name):
    # the generation loop and the engine are imported on first use
    if name in ("generate", "generate_requests", "logits", "pad_input_ids", "truncate_after_eos", "trim_prefix"):
        from . import generation

        return getattr(generation, name)
    if name == "Engine":
        from .engine import Engine

        return Engine
    raise AttributeError(name)
