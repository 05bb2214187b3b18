"""Choosing the next token from logits, the way the reference's generate does
(fms/utils/generation.py:316-328): greedy argmax, or logits / temperature, keep
the top_k largest (ties at the threshold survive), softmax, one multinomial draw.

The draw is an inverse CDF in index order at a uniform number that is a pure
function of (request seed, how many tokens the request has drawn), so a request
samples the same tokens alone and in any batch.
"""

from __future__ import annotations

import dataclasses
from typing import List, Optional, Sequence

import torch

from ..kernels import ops

_MASK = (1 << 64) - 1


@dataclasses.dataclass
class SamplingParams:
    do_sample: bool = True
    temperature: float = 1.0
    top_k: int = 10

    def __post_init__(self):
        if self.do_sample and not self.temperature > 0:
            raise ValueError(f"temperature {self.temperature} must be positive when sampling (use do_sample=False for greedy)")
        if self.top_k is not None and self.top_k < 0:
            raise ValueError("top_k cannot be negative")


def uniform(seed: int, counter: int) -> float:
    """The number in [0, 1) that the kernel draws for (seed, counter): splitmix64, top 24 bits."""
    z = (seed + (counter + 1) * 0x9E3779B97F4A7C15) & _MASK
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & _MASK
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & _MASK
    z = z ^ (z >> 31)
    return (z >> 40) / 16777216.0


def _mix(z: int) -> int:
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & _MASK
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & _MASK
    return z ^ (z >> 31)


def request_seed(seed: int, request_index: int) -> int:
    """A seed of its own for each request of a call (mixed, so that neighbouring requests and
    neighbouring counters do not meet); it fits a signed 64-bit integer."""
    return _mix((_mix(seed & _MASK) + 0xD1342543DE82EF95 * (request_index + 1)) & _MASK) >> 1


def choose(
    logits: torch.Tensor,
    params: SamplingParams,
    seeds: Optional[Sequence[int]] = None,
    counters: Optional[Sequence[int]] = None,
) -> torch.Tensor:
    """int32 token per row of float32 logits [rows, vocab] (a device tensor)."""
    rng = None
    if params.do_sample:
        if seeds is None or counters is None or len(seeds) != logits.shape[0]:
            raise ValueError("sampling needs a seed and a counter per row")
        rng = torch.tensor([[int(s), int(c)] for s, c in zip(seeds, counters)], dtype=torch.int64).reshape(-1, 2).to(logits.device)
    return ops.sample(logits, params.do_sample, params.temperature, params.top_k or 0, rng)
