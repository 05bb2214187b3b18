"""The index data of one step: which tokens, of which sequences, at which
positions, reading which pages.  Built on the host, sent to the device in one
copy, and handed to every part."""

from __future__ import annotations

import dataclasses
from typing import Dict, List, Optional, Sequence

import numpy as np
import torch

from ..cache import SequenceCache


@dataclasses.dataclass
class StepBatch:
    n_tokens: int
    n_seqs: int
    slots: List[int]  # cache slot of each sequence of the step
    q_lens: List[int]  # tokens each sequence brings
    starts: List[int]  # position of each sequence's first token
    is_decode: bool  # every sequence brings exactly one token
    max_context: int  # longest sequence after this step (host value)
    context_bound: int  # what the decode attention is launched for: max_context or a rounder number above it
    token_ids: torch.Tensor  # int32 [T]
    positions: torch.Tensor  # int32 [T]
    seq_of_token: torch.Tensor  # int32 [T], index into the rows of the block tables (-1: padding row)
    slot_ids: torch.Tensor  # int32 [B], row of each sequence in the state tensors
    seq_starts: torch.Tensor  # int32 [B + 1], offsets of the sequences in the token arrays
    block_tables: Dict[int, torch.Tensor]  # group index -> int32 [B, pages]
    # query blocks for the prefill attention kernel: block size -> (first token, length) of each block
    qblocks: Dict[int, tuple] = dataclasses.field(default_factory=dict)
    logit_rows: Optional[torch.Tensor] = None  # int32 [n_wanted] token indices whose logits are wanted
    n_logit_rows: int = 0
    # decode steps: the token rows from the longest context to the shortest (int32 [T]).  A kernel whose blocks
    # take a sequence each hands out the long ones first, so that none of them is left to run alone at the end.
    rows_by_length: Optional[torch.Tensor] = None
    # Rows of the logits that the caller asked for: the first n_wanted of the n_logit_rows that are computed (a
    # decode step padded to a row bucket computes a row for every padding token as well, as a captured step does).
    n_wanted: int = 0


def build_batch(
    cache: SequenceCache,
    slots: Sequence[int],
    tokens: Sequence[Sequence[int]],
    starts: Sequence[int],
    want: Sequence[Sequence[int]],
    device,
    qblock_sizes: Sequence[int] = (),
    pad_rows_to: int = 0,
) -> StepBatch:
    """Index arrays of a step.  `starts[b]` is what cache.extend(slot, len(tokens[b])) returned.
    qblock_sizes: the block sizes in which mixers want the step's tokens cut (blocks never span sequences).
    pad_rows_to: a decode step (one token a sequence) is filled up to this many token rows with padding rows
    (sequence -1, which every kernel skips), so that it has the shape of the captured step of that many rows:
    the same kernels then run with the same launch, and give the same bits."""
    B = len(slots)
    q_lens = [len(t) for t in tokens]
    T = sum(q_lens)
    # arrays, not Python loops over tokens: a prompt of thousands of tokens is prepared while the GPU waits
    lens = np.asarray(q_lens, dtype=np.int64)
    first = np.asarray(list(starts), dtype=np.int64)
    offsets = np.concatenate([[0], np.cumsum(lens)])
    seq_of_token = np.repeat(np.arange(B, dtype=np.int64), lens)
    flat_ids = np.concatenate([np.asarray(t, dtype=np.int64) for t in tokens]) if B else np.zeros(0, dtype=np.int64)
    positions = np.arange(T, dtype=np.int64) - offsets[:-1][seq_of_token] + first[seq_of_token]
    seq_starts = offsets
    rows: List[int] = []
    sizes = sorted(set(int(s) for s in qblock_sizes if s))
    qb_start: Dict[int, List[int]] = {s: [] for s in sizes}
    qb_len: Dict[int, List[int]] = {s: [] for s in sizes}
    for b in range(B):
        base = int(offsets[b])
        for w in want[b]:
            if not 0 <= w < q_lens[b]:
                raise IndexError(f"wanted place {w} is outside the {q_lens[b]} tokens of sequence {b}")
            rows.append(base + w)
        for size in sizes:
            for off in range(0, q_lens[b], size):
                qb_start[size].append(base + off)
                qb_len[size].append(min(size, q_lens[b] - off))
    tables = {g: cache.block_table(g, slots) for g in range(len(cache.groups))}

    # one host buffer, one copy
    is_decode = all(n == 1 for n in q_lens)
    by_length = np.argsort(-positions, kind="stable") if is_decode else []
    n_wanted = len(rows)
    pad = pad_rows_to - T if is_decode and B and pad_rows_to > T else 0
    if pad:
        filler = np.zeros(pad, dtype=np.int64)
        flat_ids = np.concatenate([flat_ids, filler])
        positions = np.concatenate([positions, filler])
        seq_of_token = np.concatenate([seq_of_token, filler - 1])
        by_length = np.concatenate([by_length, np.arange(T, T + pad)])
        if rows == list(range(T)):  # every sequence's token is wanted: the padding rows' too, as in a captured step
            rows = rows + list(range(T, T + pad))
        T += pad
    parts = [flat_ids, positions, seq_of_token, list(slots), seq_starts, rows, by_length]
    for size in sizes:
        parts += [qb_start[size], qb_len[size]]
    lengths = [len(p) for p in parts]
    table_sizes = {g: t.numel() for g, t in tables.items()}
    total = sum(lengths) + sum(table_sizes.values())
    host = torch.empty(total, dtype=torch.int32, pin_memory=torch.cuda.is_available())
    off = 0
    spans = []
    for p, n in zip(parts, lengths):
        if n:
            host[off : off + n] = torch.from_numpy(np.asarray(p).astype(np.int32, copy=False))
        spans.append((off, n))
        off += n
    table_spans = {}
    for g, t in tables.items():
        host[off : off + t.numel()] = t.reshape(-1)
        table_spans[g] = (off, t.shape)
        off += t.numel()
    dev = host.to(device, non_blocking=True)

    def span(i):
        o, n = spans[i]
        return dev[o : o + n]

    return StepBatch(
        n_tokens=T,
        n_seqs=B,
        slots=list(slots),
        q_lens=q_lens,
        starts=list(starts),
        is_decode=is_decode,
        max_context=max(s + n for s, n in zip(starts, q_lens)),
        context_bound=max(s + n for s, n in zip(starts, q_lens)),
        token_ids=span(0),
        positions=span(1),
        seq_of_token=span(2),
        slot_ids=span(3),
        seq_starts=span(4),
        block_tables={g: dev[o : o + shape[0] * shape[1]].view(shape) for g, (o, shape) in table_spans.items()},
        qblocks={size: (span(7 + 2 * i), span(8 + 2 * i)) for i, size in enumerate(sizes)},
        logit_rows=span(5),
        n_logit_rows=len(rows),
        rows_by_length=span(6) if is_decode else None,
        n_wanted=n_wanted,
    )
