"""Helpers for callers written against the reference's rectangular batches.

The engine never sees padding; these build and undo the padded tensors that the
reference's scripts pass around.  Their results are fixed by the reference's tests
(tests/utils/test_generate.py:139-198, 281-323).
"""

from __future__ import annotations

from typing import List, Optional

import torch


def pad_input_ids(input_ids_list: List[torch.Tensor], min_pad_length: int = 0, is_causal_mask: bool = True,
                  padding_side: str = "left", position_ids_offset: int = 0, pad_token_id: int = 0):
    """Prompts of unequal lengths as one [B, S] tensor, S = max(longest prompt, min_pad_length), with the
    additive mask [B, S, S] and the position_ids [B, S] that the reference's models take
    (fms/utils/generation.py:16-109): a query sees the keys of its own kind (real or padding) at or before
    itself (any key of its kind when is_causal_mask is False); real tokens count from position_ids_offset,
    padding places hold position_ids_offset.  The real lengths and the side are returned too, which is what
    ``generate`` reads."""
    if padding_side not in ("left", "right"):
        raise NotImplementedError("padding_side must be 'right' or left'")
    lengths = [int(p.numel()) for p in input_ids_list]
    width = max(lengths + [int(min_pad_length)])
    device = input_ids_list[0].device
    rows = len(input_ids_list)
    input_ids = torch.full((rows, width), pad_token_id, dtype=torch.long, device=device)
    position_ids = torch.full((rows, width), position_ids_offset, dtype=torch.long, device=device)
    real = torch.zeros(rows, width, dtype=torch.bool, device=device)
    for b, (prompt, n) in enumerate(zip(input_ids_list, lengths)):
        first = width - n if padding_side == "left" else 0
        input_ids[b, first : first + n] = prompt
        position_ids[b, first : first + n] += torch.arange(n, device=device)
        real[b, first : first + n] = True
    visible = real[:, :, None] == real[:, None, :]  # [B, query, key]
    if is_causal_mask:
        place = torch.arange(width, device=device)
        visible &= place[None, :, None] >= place[None, None, :]
    mask = torch.zeros(rows, width, width, device=device).masked_fill_(~visible, float("-inf"))
    return input_ids, {"mask": mask, "position_ids": position_ids, "lengths": lengths, "padding_side": padding_side}


def truncate_after_eos(result: torch.Tensor, eos_token_id: Optional[int]) -> torch.Tensor:
    """A 1-D result up to and including its first eos token (fms/utils/generation.py:372-387)."""
    if eos_token_id is None:
        return result
    hits = (result == eos_token_id).nonzero()
    return result if hits.numel() == 0 else result[: int(hits[0]) + 1]


def trim_prefix(result: torch.Tensor, pad_token_id: int = 0) -> torch.Tensor:
    """A 1-D result without its leading run of pad tokens; a result that is nothing but pad tokens stays
    as it is (fms/utils/generation.py:390-413)."""
    leading = int(torch.cumsum((result != pad_token_id).to(torch.int64), 0).eq(0).sum())
    return result if leading in (0, result.numel()) else result[leading:]
