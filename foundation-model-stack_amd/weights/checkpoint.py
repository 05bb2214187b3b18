"""Finding the files of a checkpoint and reading their tensors by name.

File discovery follows fms/utils/serialization.py:378-419: a path may be a
file or a folder; in a folder ``*.safetensors`` files are taken first (an
``hf`` folder's ``consolidated.safetensors`` is skipped), then ``*.pth``/``*.bin``
/``*.pt``; no file at all is an error that names the path.  Several files act as
one mapping (the reference chains them, :434-464).
"""

from __future__ import annotations

import glob
import os
from typing import Dict, List, Optional, Tuple

import torch

from .safetensors_io import SafetensorsFile


class Checkpoint:
    """name -> tensor over one or several files; tensors are read when asked for."""

    def __init__(self, path: str, source: Optional[str] = None):
        self.path = path
        self.files = find_files(path, source)
        self._st: List[SafetensorsFile] = []
        self._loaded: Dict[str, torch.Tensor] = {}
        self._where: Dict[str, SafetensorsFile] = {}
        for f in self.files:
            if f.endswith(".safetensors"):
                st = SafetensorsFile(f)
                self._st.append(st)
                for name in st.keys():
                    self._where.setdefault(name, st)
            else:
                # weights_only: nothing from the file is executed
                state = torch.load(f, map_location="cpu", mmap=True, weights_only=True)
                if isinstance(state, dict) and "model_state" in state:
                    state = state["model_state"]
                for name, t in state.items():
                    self._loaded.setdefault(name, t)

    def keys(self) -> List[str]:
        return list(self._where) + [k for k in self._loaded if k not in self._where]

    def stored_dtype(self, name: str) -> torch.dtype:
        return self._where[name].dtype(name) if name in self._where else self._loaded[name].dtype

    def stored_shape(self, name: str) -> Tuple[int, ...]:
        return self._where[name].shape(name) if name in self._where else tuple(self._loaded[name].shape)

    def read(self, name: str) -> torch.Tensor:
        return self._where[name].read(name) if name in self._where else self._loaded[name]

    def close(self) -> None:
        for st in self._st:
            st.close()


def find_files(path: str, source: Optional[str] = None) -> List[str]:
    path = os.path.expanduser(str(path))
    if os.path.isfile(path):
        return [path]
    if os.path.isdir(path):
        if source == "meta":
            patterns = ["*.pth", "*.safetensors"]
        elif source == "hf":
            patterns = ["*.safetensors", "*.bin", "*.pt"]
        else:
            patterns = ["*.safetensors", "*.pth", "*.bin"]
        for pattern in patterns:
            files = sorted(glob.glob(os.path.join(path, pattern)))
            if source == "hf":
                files = [f for f in files if os.path.basename(f) != "consolidated.safetensors"]
            if files:
                return files
    else:
        files = sorted(glob.glob(path))
        if files:
            return files
    raise FileNotFoundError(f"Can't find the requested checkpoint data at {path}")
