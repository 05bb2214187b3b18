"""Adapters: from the tensor names and layouts of a checkpoint source to the model's own.

An adapter is a list of named steps, each a function from a partial state dict
(the tensors of one layer, or all tensors outside the layers) to another, run in
order; the reference composes its adapters the same way
(fms/utils/serialization.py:27-101).  Steps are registered per architecture.
"""

from __future__ import annotations

import re
from typing import Callable, Dict, List, Mapping, Optional, Tuple

import torch

Step = Callable[..., Mapping[str, torch.Tensor]]

_steps: Dict[str, Dict[str, Step]] = {}
_adapters: Dict[str, Dict[str, List[str]]] = {}


def register_adapter_step(architecture: str, name: str, step: Step) -> None:
    steps = _steps.setdefault(architecture, {})
    if name in steps:
        raise KeyError(f"adapter step {name!r} of {architecture!r} is already registered")
    steps[name] = step


def register_adapter(architecture: str, source: str, step_names: List[str]) -> None:
    sources = _adapters.setdefault(architecture, {})
    if source in sources:
        raise KeyError(f"adapter {source!r} of {architecture!r} is already registered")
    missing = [s for s in step_names if s not in _steps.get(architecture, {})]
    if missing:
        raise KeyError(f"adapter {source!r} of {architecture!r} names unknown steps {missing}")
    sources[source] = list(step_names)


def extend_adapter(architecture: str, source: str, step_names: List[str]) -> None:
    """Further steps behind those a source already has (fms/utils/serialization.py:104-148): the source must be
    registered, and so must the steps."""
    if source not in _adapters.get(architecture, {}):
        raise KeyError(f"adapter {source!r} of {architecture!r} must be registered before it is extended")
    missing = [s for s in step_names if s not in _steps.get(architecture, {})]
    if missing:
        raise KeyError(f"adapter {source!r} of {architecture!r} is extended by unknown steps {missing}")
    _adapters[architecture][source] = _adapters[architecture][source] + list(step_names)


def list_sources(architecture: str) -> List[str]:
    return sorted(_adapters.get(architecture, {}))


def get_adapter(architecture: str, source: Optional[str]) -> Step:
    """The composed steps of a source; None or 'fms' is the identity (fms/utils/serialization.py:273-289)."""
    if source in (None, "fms"):
        return lambda sd, **kw: sd
    try:
        names = _adapters[architecture][source]
    except KeyError:
        raise KeyError(f"no adapter from source {source!r} for architecture {architecture!r}; known: {list_sources(architecture)}") from None
    steps = [_steps[architecture][n] for n in names]

    def run(sd, **kw):
        for step in steps:
            sd = step(sd, **kw)
        return sd

    return run


def get_adapted(architecture: str, source: Optional[str], state_dict: Mapping[str, torch.Tensor],
                adapter_kwargs: Optional[Mapping] = None) -> Mapping[str, torch.Tensor]:
    """A state dict in the model's own names and layouts (fms/utils/serialization.py:292-317); an empty one is
    handed back as it is.  Steps that need the model's sizes read them from adapter_kwargs["model_config"]."""
    if not len(state_dict):
        return state_dict
    return get_adapter(architecture, source)(state_dict, **dict(adapter_kwargs or {}))


# ---- steps shared by decoder architectures -----------------------------------
def rename_step(replacements: List[Tuple[str, str]]) -> Step:
    compiled = [(re.compile(p), r) for p, r in replacements]

    def step(sd, **kw):
        out = {}
        for name, t in sd.items():
            for pattern, repl in compiled:
                name = pattern.sub(repl, name)
            out[name] = t
        return out

    return step


def fuse_attention_step(sd, **kw):
    """query, key, value -> qkv_fused = cat([q, k, v]) for weights and biases (fms/utils/serialization.py:173-227)."""
    out = dict(sd)
    for name in list(sd):
        m = re.match(r"(.*\.in_proj)\.query\.(weight|bias)$", name)
        if not m:
            continue
        prefix, kind = m.groups()
        parts = [f"{prefix}.{which}.{kind}" for which in ("query", "key", "value")]
        if all(p in sd for p in parts):
            out[f"{prefix}.qkv_fused.{kind}"] = torch.cat([sd[p] for p in parts], dim=0)
            for p in parts:
                del out[p]
    return out


def fuse_glu_step(sd, **kw):
    """wg, w1 -> wg1_fused = cat([wg, w1]): the gate comes first (fms/utils/serialization.py:230-270)."""
    out = dict(sd)
    for name in list(sd):
        m = re.match(r"(.*)\.wg\.(weight|bias)$", name)
        if not m:
            continue
        prefix, kind = m.groups()
        up = f"{prefix}.w1.{kind}"
        if up in sd:
            out[f"{prefix}.wg1_fused.{kind}"] = torch.cat([sd[name], sd[up]], dim=0)
            del out[name], out[up]
    return out
