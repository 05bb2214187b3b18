from .adapters import extend_adapter, get_adapted, get_adapter, list_sources, register_adapter, register_adapter_step
from .checkpoint import Checkpoint, find_files
from .loader import WeightsError, init_random, kept_dtype, load_checkpoint, random_tensor
from .safetensors_io import SafetensorsFile, write_safetensors

__all__ = [
    "extend_adapter", "get_adapted", "get_adapter", "list_sources", "register_adapter", "register_adapter_step", "Checkpoint", "find_files",
    "WeightsError", "init_random", "kept_dtype", "load_checkpoint", "random_tensor", "SafetensorsFile",
    "write_safetensors",
]
