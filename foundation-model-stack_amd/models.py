"""``get_model``: from an architecture name (or a model folder) to a model on the GPU.

The call follows the reference's (fms/models/__init__.py:298-503):
``get_model(architecture, variant, model_path=..., source=..., device_type=..., data_type=..., **overrides)``,
with the special architectures ``"hf_pretrained"`` (configuration and weights from a folder
with config.json and safetensors) and ``"hf_configured"`` (configuration only).  Without a
path the weights are random, from ``random_seed``.
"""

from __future__ import annotations

import json
import logging
import os
from typing import Optional, Union

import torch

from .architectures import architecture_for_hf, get_architecture, variant_config
from .config import ModelConfig
from .engine.model import DecoderModel
from .weights import Checkpoint, init_random, load_checkpoint, random_tensor, write_safetensors

logger = logging.getLogger(__name__)

_DTYPES = {
    "fp32": torch.float32, "float32": torch.float32, "float": torch.float32,
    "bf16": torch.bfloat16, "bfloat16": torch.bfloat16,
}


def resolve_dtype(data_type) -> Optional[torch.dtype]:
    if data_type is None or isinstance(data_type, torch.dtype):
        if data_type not in (None, torch.float32, torch.bfloat16):
            raise ValueError(f"models run in float32 or bfloat16, not {data_type}")
        return data_type
    try:
        return _DTYPES[str(data_type).lower()]
    except KeyError:
        # fms/models/__init__.py:352-356: an unknown dtype string is a ValueError
        raise ValueError(f"Unknown data type {data_type!r}; use one of {sorted(_DTYPES)}") from None


def read_model_folder_config(model_path: str):
    """(architecture, configuration) of a folder's config.json, chosen by what config.json says."""
    cfg_file = os.path.join(model_path, "config.json")
    if not os.path.isfile(cfg_file):
        raise FileNotFoundError(f"Can't find the requested checkpoint data at {model_path}: no config.json")
    with open(cfg_file, "r", encoding="utf-8") as f:
        raw = json.load(f)
    if raw.get("architectures"):
        arch = architecture_for_hf(raw["architectures"][0])
        return arch, arch.from_hf_dict(raw)
    if raw.get("architecture"):
        arch = get_architecture(raw["architecture"])
        return arch, arch.config_class.from_dict(raw)
    raise ValueError(f"{cfg_file} names no architecture (neither 'architectures' nor 'architecture')")


def _gpu_device(device_type) -> torch.device:
    device = torch.device(device_type if ":" in str(device_type) or device_type != "cuda" else "cuda:0")
    if device.type != "cuda":
        raise RuntimeError("fms_amd models run on the GPU only (device_type='cuda'); there is no CPU path")
    if not torch.cuda.is_available():  # before anything is allocated: the message is this library's, not the runtime's
        raise RuntimeError("fms_amd models run on an AMD GPU, and this machine shows none to PyTorch "
                           "(torch.cuda.is_available() is False); there is no CPU path")
    return device


def get_model(
    architecture: str,
    variant: Optional[str] = None,
    model_path: Optional[str] = None,
    source: Optional[str] = None,
    device_type: str = "cuda",
    data_type: Union[None, str, torch.dtype] = None,
    distributed_strategy: Optional[str] = None,
    checkpoint_sharding: Optional[str] = None,
    group=None,
    random_seed: int = 0,
    **kwargs,
) -> DecoderModel:
    """The reference's get_model (fms/models/__init__.py:298-309) on this library: architecture and variant from
    the registry (or "hf_pretrained"/"hf_configured" and a model folder), weights from `model_path` named as
    `source` says, on the GPU, in `data_type` (the checkpoint's type if none is given); further keyword arguments
    override fields of the configuration.  distributed_strategy, checkpoint_sharding and group are the reference's
    parameters for several GPUs: this library runs on one, so anything but None is refused."""
    if distributed_strategy is not None or checkpoint_sharding is not None or group is not None:
        raise NotImplementedError("fms_amd runs a model on one GPU: distributed_strategy, checkpoint_sharding and group must be None")
    dtype = resolve_dtype(data_type)
    if architecture in ("hf_pretrained", "hf_configured"):
        # fms/models/__init__.py:88-98: the folder may come as `variant` or as `model_path`, not both
        if variant is not None and model_path is not None:
            raise ValueError(f"{architecture} takes the model folder either as variant or as model_path, not both")
        if source is not None:
            raise ValueError(f"source must be None for {architecture}: the folder's layout is the Hugging Face one")
        folder = model_path if model_path is not None else variant
        if folder is None:
            raise ValueError(f"{architecture} needs a model folder")
        arch, config = read_model_folder_config(folder)
        config = config.updated(**kwargs) if kwargs else config
        model_path = folder if architecture == "hf_pretrained" else None
        source = "hf" if model_path else None
    else:
        arch = get_architecture(architecture)
        if variant is None:
            raise KeyError(f"a variant of {architecture} is needed")
        config = variant_config(architecture, variant, **kwargs)

    device = _gpu_device(device_type)

    ckpt_dtype = None
    if model_path is not None:
        ckpt = Checkpoint(model_path, source)
        try:
            names = ckpt.keys()
            if source is None:
                if arch.detect_source is None:
                    raise ValueError(f"architecture {arch.name} cannot tell a checkpoint's source from its tensor names: pass source=")
                source = arch.detect_source(names)
            floats = [ckpt.stored_dtype(n) for n in names if ckpt.stored_dtype(n).is_floating_point]
            if floats:
                ckpt_dtype = torch.float32 if all(d in (torch.float32, torch.float64) for d in floats) else torch.bfloat16
        finally:
            ckpt.close()
    if dtype is None:
        # the reference keeps the checkpoint's type unless one is given (fms/utils/serialization.py:679-687)
        dtype = ckpt_dtype or torch.float32

    model = DecoderModel(arch.build_spec(config), dtype, config=config)
    model.architecture = arch.name
    if model_path is not None:
        load_checkpoint(model, model_path, arch.name, source, device, forced_dtype=data_type is not None)
    else:
        init_random(model, random_seed, device)
    model.finalize_all(device)
    return model


def from_config(config: ModelConfig, architecture: str = "llama", data_type: Union[None, str, torch.dtype] = "bfloat16",
                device_type: str = "cuda", random_seed: int = 0, **kwargs) -> DecoderModel:
    """A model of `config` with random weights (keyword arguments replace fields of the configuration): what the
    reference's `LLaMA(config, **kwargs)` followed by `reset_parameters()` gives (fms/models/llama.py:362-394),
    with this library's random-weights rule (every tensor a function of the seed and its name)."""
    arch = get_architecture(architecture)
    if not isinstance(config, arch.config_class):
        raise TypeError(f"architecture {architecture} is configured by {arch.config_class.__name__}, not {type(config).__name__}")
    config = config.updated(**kwargs) if kwargs else config
    dtype = resolve_dtype(data_type) or torch.float32
    device = _gpu_device(device_type)
    model = DecoderModel(arch.build_spec(config), dtype, config=config)
    model.architecture = arch.name
    init_random(model, random_seed, device)
    model.finalize_all(device)
    return model


def LLaMA(config=None, **kwargs) -> DecoderModel:
    """The reference's constructor by its name: `LLaMA(config)` or `LLaMA(emb_dim=..., nlayers=...)`, random weights;
    `data_type`, `device_type` and `random_seed` as in from_config."""
    from .config import LLaMAConfig

    return from_config(config if config is not None else LLaMAConfig(), "llama", **kwargs)


def write_model_folder(
    folder: str,
    config: ModelConfig,
    seed: int,
    architecture: str = "llama",
    data_type: Union[str, torch.dtype] = "bfloat16",
    std: float = 0.02,
    norm_std: float = 0.0,
) -> str:
    """Random-weights mode: write config.json and model.safetensors (Hugging Face layout) from a
    configuration and a seed.  Every tensor is a function of (seed, its name): N(0, std) for
    matrices, ones (+ N(0, norm_std)) for norm scales.  Tensors are produced one at a time."""
    arch = get_architecture(architecture)
    dtype = resolve_dtype(data_type)
    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w", encoding="utf-8") as f:
        json.dump(arch.to_hf_dict(config), f, indent=1)
    layout = arch.hf_tensor_layout(config)
    inits = {name: (shape, init) for name, shape, init in layout}

    def produce(name):
        shape, init = inits[name]
        return random_tensor(name, shape, init, seed, std, norm_std, dtype=dtype)

    write_safetensors(os.path.join(folder, "model.safetensors"), [(n, s, dtype) for n, s, _ in layout], produce)
    return folder
