"""What every part of a model has in common: declared parameters, children,
and the registries from which a configuration picks parts by name.

A part knows its own sizes and constants (they are constructor arguments) and
nothing about the model it sits in.  Parameters are declared with a shape and
are bound to device tensors by the loader, by full dotted name.
"""

from __future__ import annotations

import dataclasses
from typing import Callable, Dict, Iterator, List, Optional, Tuple

import torch


@dataclasses.dataclass(frozen=True)
class ParamSpec:
    shape: Tuple[int, ...]
    init: str = "normal"  # "normal" (std 0.02), "ones", "zeros": what random-weights mode writes
    # "float": the model's type; "scale": a norm's scale or shift, which stays 32-bit if the file stores it so;
    # "int": int32
    kind: str = "float"


class Part:
    """Base of mixers, feed-forwards, norms, position encodings, blocks and models."""

    def __init__(self) -> None:
        self._specs: Dict[str, ParamSpec] = {}
        self._children: Dict[str, "Part"] = {}
        self.w: Dict[str, Optional[torch.Tensor]] = {}

    # ---- declaration ----------------------------------------------------
    def declare(self, name: str, shape, init: str = "normal", kind: str = "float") -> None:
        self._specs[name] = ParamSpec(tuple(int(s) for s in shape), init, kind)
        self.w[name] = None

    def add_child(self, name: str, part: "Part") -> "Part":
        self._children[name] = part
        return part

    def children(self) -> Dict[str, "Part"]:
        return dict(self._children)

    def named_specs(self, prefix: str = "") -> Iterator[Tuple[str, ParamSpec, "Part", str]]:
        """(full name, spec, owning part, local name) of every parameter below this part."""
        for local, spec in self._specs.items():
            yield prefix + local, spec, self, local
        for name, child in self._children.items():
            yield from child.named_specs(prefix + name + ".")

    def walk(self) -> Iterator["Part"]:
        yield self
        for child in self._children.values():
            yield from child.walk()

    def bind(self, local: str, tensor: torch.Tensor) -> None:
        spec = self._specs[local]
        if tuple(tensor.shape) != spec.shape:
            raise ValueError(f"{local}: shape {tuple(tensor.shape)} does not match {spec.shape}")
        self.w[local] = tensor

    def finalize(self, device: torch.device, dtype: torch.dtype) -> None:
        """Called once after all parameters are bound: build tables, check what was bound."""


class NormedRows:
    """The input of a branch whose norm is left to the branch's first product: `rows` hold the stream times
    the norm's weight in the activation type, `row_norm` what the product needs to divide by the rows' root
    mean square (kernels.ops.RowNorm).  Only parts that say `accepts_normed_rows` ever see one."""

    def __init__(self, rows: torch.Tensor, row_norm):
        self.rows, self.row_norm = rows, row_norm

    @property
    def shape(self):
        return self.rows.shape

    @property
    def dtype(self):
        return self.rows.dtype


class BranchOutput:
    """A branch's output that is still one product away: linear(x).  Whoever holds the residual stream
    decides whether that product also adds to the stream (ResidualStream.add_branch) or just runs."""

    def __init__(self, x: torch.Tensor, linear: "Part"):
        self.x, self.linear = x, linear

    def value(self) -> torch.Tensor:
        return self.linear.forward(self.x)


def split_normed(x):
    """(rows, row_norm) of a branch input, whether the norm was applied (row_norm None) or left to the product."""
    return (x.rows, x.row_norm) if isinstance(x, NormedRows) else (x, None)


class Mixer(Part):
    """A part that mixes information along the sequence.  It says what it needs of the cache:
    keys and values in pages (``kv_need``), fixed-size memory per sequence (``state_need``), or nothing."""

    def kv_need(self):
        return None

    def state_need(self):
        return None

    def check_step(self, max_position: int) -> None:
        """Raise if a token at `max_position` cannot be processed (for instance beyond a position table)."""

    def prefill_qblock(self, n_tokens: int, dtype) -> int:
        """If the mixer wants the tokens of a multi-token step cut into blocks (that never span two
        sequences), the block size; the step's batch then carries them in `qblocks[size]`.  0: no."""
        return 0

    def forward(self, x: torch.Tensor, batch, cache) -> torch.Tensor:
        raise NotImplementedError

    # optional, for kernels that fuse across the boundary of the part --------
    def accepts_normed_rows(self, rows: int, dtype, batch) -> bool:
        """True if forward_branch takes a NormedRows for a step of this shape."""
        return False

    def forward_branch(self, x, batch, cache):
        """Like forward, but may return a BranchOutput and may be given a NormedRows (if it says so)."""
        return self.forward(x, batch, cache)


class FeedForward(Part):
    """A part that maps every token on its own: [T, width] -> [T, width]."""

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        raise NotImplementedError

    def accepts_normed_rows(self, rows: int, dtype) -> bool:
        return False

    def forward_branch(self, x):
        return self.forward(x)


# --------------------------------------------------------------------------
# registries: category -> kind -> constructor
# --------------------------------------------------------------------------
CATEGORIES = ("mixer", "feed_forward", "norm", "position", "block", "embedding", "head")
_registry: Dict[str, Dict[str, Callable[..., Part]]] = {c: {} for c in CATEGORIES}


def register_part(category: str, kind: str, constructor: Callable[..., Part], replace: bool = False) -> None:
    if category not in _registry:
        raise KeyError(f"unknown part category {category!r}; categories are {CATEGORIES}")
    if kind in _registry[category] and not replace:
        raise KeyError(f"{category} {kind!r} is already registered")
    _registry[category][kind] = constructor


def unregister_part(category: str, kind: str) -> None:
    _registry[category].pop(kind, None)


def list_parts(category: str) -> List[str]:
    return sorted(_registry[category])


def part_attribute(category: str, kind: str, name: str, default=None):
    """An attribute of the registered constructor (a class attribute of the part), or `default`: what a part says
    about itself before it is built."""
    try:
        constructor = _registry[category][kind]
    except KeyError:
        raise KeyError(f"no {category} named {kind!r}; registered: {list_parts(category)}") from None
    return getattr(constructor, name, default)


def make_part(category: str, kind: str, **kwargs) -> Part:
    try:
        constructor = _registry[category][kind]
    except KeyError:
        raise KeyError(f"no {category} named {kind!r}; registered: {list_parts(category)}") from None
    return constructor(**kwargs)
