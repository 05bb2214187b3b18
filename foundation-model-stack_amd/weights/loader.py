"""Filling a model's parameters: from a checkpoint by tensor name, or at random from a seed.

Kept types.  With a type asked for (``data_type``), floating tensors are cast
to it, as the reference does (fms/utils/serialization.py:679-687,
tests/models/test_getmodel_datatype.py:58-90); only norm scales and shifts
(parameters of kind "scale") that the file stores in 32-bit stay 32-bit: the
norm kernels compute in 32-bit and read either type.  With no type asked for,
the model runs in the checkpoint's type, and in a bfloat16 model a tensor that
the file stores in 32-bit stays 32-bit.  Integer tensors become int32.  Every problem of a checkpoint — tensors the model lacks,
tensors the model has and the checkpoint lacks, wrong shapes — is collected and
raised as one error.  (The reference warns about unused keys and leaves missing
ones uninitialised, fms/utils/serialization.py:604-608, fms/models/__init__.py:494-501;
here both are errors.)
"""

from __future__ import annotations

import hashlib
import re
from typing import Dict, List, Optional

import torch

from .adapters import get_adapter
from .checkpoint import Checkpoint


class WeightsError(ValueError):
    def __init__(self, missing, unexpected, wrong_shapes, where=""):
        self.missing, self.unexpected, self.wrong_shapes = sorted(missing), sorted(unexpected), list(wrong_shapes)
        lines = [f"the checkpoint {where} does not fit the model:"]
        if self.missing:
            lines.append(f"  missing tensors ({len(self.missing)}): " + ", ".join(self.missing))
        if self.unexpected:
            lines.append(f"  unexpected tensors ({len(self.unexpected)}): " + ", ".join(self.unexpected))
        if self.wrong_shapes:
            lines.append(f"  wrong shapes ({len(self.wrong_shapes)}): " + ", ".join(
                f"{n} is {tuple(got)}, the model has {tuple(want)}" for n, got, want in self.wrong_shapes))
        super().__init__("\n".join(lines))


def kept_dtype(stored: torch.dtype, kind: str, model_dtype: torch.dtype, forced: bool = False) -> torch.dtype:
    """The type in which a checkpoint tensor is kept on the device.  forced: the caller asked for model_dtype."""
    if kind == "int" or not stored.is_floating_point:
        return torch.int32
    if stored in (torch.float32, torch.float64) and model_dtype == torch.bfloat16 and (kind == "scale" or not forced):
        return torch.float32  # stored in 32-bit and nobody asked otherwise: it stays so
    return model_dtype


_LAYER = re.compile(r"(^|\.)(\d+)\.")


def _layer_groups(names: List[str]) -> List[List[str]]:
    """Names that share a layer index go together, all others form one group
    (fms/utils/serialization.py:467-492), so that fusing steps see what they need."""
    groups: Dict[str, List[str]] = {}
    for name in names:
        m = _LAYER.search(name)
        key = name[: m.end()] if m else ""
        groups.setdefault(key, []).append(name)
    return [groups[k] for k in sorted(groups)]


def load_checkpoint(model, path: str, architecture: str, source: Optional[str], device, verbose: bool = False,
                    forced_dtype: bool = False) -> None:
    """Bind every parameter of `model` from the checkpoint at `path`; one WeightsError lists all that is wrong.
    forced_dtype: the model's type was asked for by the caller, so floating tensors are cast to it."""
    ckpt = Checkpoint(path, source)
    try:
        adapter = get_adapter(architecture, source)
        expected = {full: (spec, part, local) for full, spec, part, local in model.named_specs()}
        bound, unexpected, wrong = set(), [], []
        for group in _layer_groups(ckpt.keys()):
            partial = adapter({name: ckpt.read(name) for name in group}, model_config=model.config)
            for name, tensor in partial.items():
                if name not in expected:
                    unexpected.append(name)
                    continue
                spec, part, local = expected[name]
                if tuple(tensor.shape) != spec.shape:
                    wrong.append((name, tuple(tensor.shape), spec.shape))
                    continue
                dtype = kept_dtype(tensor.dtype, spec.kind, model.dtype, forced_dtype)
                part.bind(local, tensor.to(dtype).contiguous().to(device))
                bound.add(name)
            del partial
        for alias, target in model.tied.items():
            if alias not in bound and target in bound:
                spec, part, local = expected[alias]
                tspec, tpart, tlocal = expected[target]
                part.bind(local, tpart.w[tlocal])
                bound.add(alias)
            elif alias in bound and target not in bound:
                spec, part, local = expected[target]
                aspec, apart, alocal = expected[alias]
                part.bind(local, apart.w[alocal])
                bound.add(target)
        misshapen = {n for n, _, _ in wrong}
        missing = [n for n in expected if n not in bound and n not in misshapen]
        if missing or unexpected or wrong:
            raise WeightsError(missing, unexpected, wrong, where=f"at {path}")
    finally:
        ckpt.close()


def _seed_for(seed: int, name: str) -> int:
    digest = hashlib.sha256(f"{seed}:{name}".encode()).digest()
    return int.from_bytes(digest[:8], "little") & 0x7FFFFFFFFFFFFFFF


def random_tensor(name: str, shape, init: str, seed: int, std: float = 0.02, norm_std: float = 0.0,
                  device="cpu", dtype=torch.float32) -> torch.Tensor:
    """The tensor that random-weights mode gives `name`: N(0, std) for matrices, ones (plus
    N(0, norm_std) if asked) for norm scales, zeros for biases; a function of (seed, name) only."""
    gen = torch.Generator(device=device)
    gen.manual_seed(_seed_for(seed, name))
    if init == "normal":
        t = torch.randn(shape, generator=gen, device=device, dtype=torch.float32) * std
    elif init == "ones":
        t = torch.ones(shape, device=device, dtype=torch.float32)
        if norm_std:
            t = t + torch.randn(shape, generator=gen, device=device, dtype=torch.float32) * norm_std
    elif init == "zeros":
        t = torch.zeros(shape, device=device, dtype=torch.float32)
    else:
        raise ValueError(f"unknown init {init!r}")
    return t.to(dtype)


def init_random(model, seed: int, device, std: float = 0.02, norm_std: float = 0.0) -> None:
    """Random weights straight into the model (no file): every tensor a function of (seed, its name).

    The reference initialises with trunc_normal(0, 0.02) for linears and norm scales of one
    (fms/modules/attention.py:689-692, feedforward.py:269-283, layernorm.py:50-54); here the
    embedding and the head use the same 0.02.
    """
    expected = {full: (spec, part, local) for full, spec, part, local in model.named_specs()}
    for full, (spec, part, local) in expected.items():
        if full in model.tied:
            continue
        dtype = torch.int32 if spec.kind == "int" else model.dtype
        part.bind(local, random_tensor(full, spec.shape, spec.init, seed, std, norm_std, device=device, dtype=dtype))
    for alias, target in model.tied.items():
        spec, part, local = expected[alias]
        tspec, tpart, tlocal = expected[target]
        part.bind(local, tpart.w[tlocal])
