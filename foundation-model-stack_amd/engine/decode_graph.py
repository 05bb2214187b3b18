"""Decode steps as a captured HIP graph.

One decode step of a batch is some hundred small launches; replaying them as a
graph takes the launch cost and the host's work out of the step.  A graph is
captured for a fixed number of rows (the batch padded up to a bucket; padding
rows carry sequence -1 and are skipped by the kernels) and a fixed upper bound
of the context length (it sizes the split of the attention kernel).  Its index
data lives in static device buffers: the sampled tokens are written where the
next step reads its input, positions advance on the device, and the host only
writes a block-table row when a sequence gets a new page.

No memset is recorded into a graph (fill kernels only), and a graph is only
used when every part of the model says it can be captured.
"""

from __future__ import annotations

import gc

from typing import List, Optional, Sequence, Tuple

import torch

from ..cache import pages_for
from ..kernels import ops
from .batch import StepBatch

ROW_BUCKETS = (1, 2, 4, 8, 12, 16, 20, 24, 32, 40, 48, 56, 64, 80, 96, 112, 128, 160, 192, 256)
CONTEXT_BUCKET = 2048  # the smallest context bound of a graph; larger ones double
CONTEXT_HEADROOM = 256  # a new graph is captured for a bound this far beyond the longest context


def row_bucket(n: int) -> int:
    for b in ROW_BUCKETS:
        if n <= b:
            return b
    return -(-n // 64) * 64


def context_bucket(n: int, limit: int) -> int:
    """The context bound of the graph captured for contexts of up to n tokens: a power of two times 2048,
    at most `limit`.  The decode attention deals every sequence's own pages out over its splits, so a bound
    well above the contexts costs little, and doubling keeps the number of captures small."""
    bound = CONTEXT_BUCKET
    while bound < n:
        bound *= 2
    return min(bound, max(limit, 1))


class DecodeGraph:
    def __init__(self, engine, rows: int, max_context: int, sampling):
        self.engine, self.rows, self.max_context, self.sampling = engine, rows, max_context, sampling
        dev = engine.device
        cache = engine.cache
        self.table_width = pages_for(cache.max_seq_len)
        self.tokens = torch.zeros(rows, dtype=torch.int32, device=dev)
        self.positions = torch.zeros(rows, dtype=torch.int32, device=dev)
        self.seq_of_token = torch.full((rows,), -1, dtype=torch.int32, device=dev)
        self.slot_ids = torch.zeros(rows, dtype=torch.int32, device=dev)
        self.seq_starts = torch.arange(rows + 1, dtype=torch.int32, device=dev)
        self.logit_rows = torch.arange(rows, dtype=torch.int32, device=dev)
        self.rows_by_length = torch.arange(rows, dtype=torch.int32, device=dev)
        self.tables = {g: torch.zeros(rows, self.table_width, dtype=torch.int32, device=dev) for g in range(len(cache.groups))}
        self.rng = torch.zeros(rows, 2, dtype=torch.int64, device=dev)
        self.batch = StepBatch(
            n_tokens=rows, n_seqs=rows, slots=[], q_lens=[1] * rows, starts=[0] * rows, is_decode=True,
            max_context=max_context, context_bound=max_context, token_ids=self.tokens, positions=self.positions, seq_of_token=self.seq_of_token,
            slot_ids=self.slot_ids, seq_starts=self.seq_starts, block_tables=self.tables,
            logit_rows=self.logit_rows, n_logit_rows=rows, rows_by_length=self.rows_by_length,
        )
        # what the static buffers currently describe
        self.slots: Tuple[int, ...] = ()
        self.next_tokens: Optional[List[int]] = None  # tokens now in self.tokens (the last step's choices)
        self.n_pages: List[int] = []
        self.stamps: List[int] = []  # the cache's stamp of every sequence after the last replay
        self.graph: Optional[torch.cuda.CUDAGraph] = None
        self.logits: Optional[torch.Tensor] = None
        self.chosen = torch.empty(8, rows, dtype=torch.int32, device=dev)  # [steps, rows]: the tokens of replays that are waited for together

    def _run(self) -> None:
        logits = self.engine.model.forward(self.batch, self.engine.cache)
        self.logits = logits  # [rows, vocab]; after a replay, that step's logits (padding rows: anything)
        s = self.sampling
        ops.sample(logits, s.do_sample, s.temperature, s.top_k or 0, self.rng if s.do_sample else None, out=self.tokens)
        ops.advance_positions_(self.positions, self.seq_of_token)

    def capture(self) -> None:
        # Padding rows only (sequence -1): nothing is written to the cache while warming up and capturing.
        self.seq_of_token.fill_(-1)
        self.slots, self.next_tokens, self.stamps = (), None, []
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            self._run()  # warm-up: lazy initialisation and allocator growth happen outside the capture
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        # No garbage collection while the stream is capturing: a collector pass that finds an old engine's
        # graphs (they sit in reference cycles) would destroy them in the middle of the capture, which the
        # runtime refuses, and the refusal inside a destructor ends the process.  Collect before, not during.
        gc.collect()
        was_enabled = gc.isenabled()
        gc.disable()
        try:
            self.graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(self.graph):
                self._run()
        finally:
            if was_enabled:
                gc.enable()
        torch.cuda.synchronize()

    def load(self, slots: Sequence[int], tokens: Sequence[int], positions: Sequence[int], seeds, counters) -> None:
        """Describe a new batch composition in the static buffers (one small copy each)."""
        n = len(slots)
        cache = self.engine.cache
        pad = self.rows - n
        dev = self.engine.device
        self.tokens.copy_(torch.tensor(list(tokens) + [0] * pad, dtype=torch.int32), non_blocking=True)
        self.positions.copy_(torch.tensor(list(positions) + [0] * pad, dtype=torch.int32), non_blocking=True)
        self.seq_of_token.copy_(torch.tensor(list(range(n)) + [-1] * pad, dtype=torch.int32), non_blocking=True)
        self.slot_ids.copy_(torch.tensor(list(slots) + [0] * pad, dtype=torch.int32), non_blocking=True)
        # every sequence grows by one token a step: the order of the lengths holds as long as the batch does
        order = sorted(range(n), key=lambda b: -positions[b]) + list(range(n, self.rows))
        self.rows_by_length.copy_(torch.tensor(order, dtype=torch.int32), non_blocking=True)
        for g, table in self.tables.items():
            host = cache.block_table(g, slots, n_columns=self.table_width)
            table[:n].copy_(host, non_blocking=True)
        if self.sampling.do_sample:
            rng = [[int(s), int(c)] for s, c in zip(seeds, counters)] + [[0, 0]] * pad
            self.rng.copy_(torch.tensor(rng, dtype=torch.int64), non_blocking=True)
        self.slots = tuple(slots)
        self.n_pages = [(pages_for(cache.length(s)), cache.pages_held(s)) for s in slots]

    def refresh_pages(self) -> None:
        """Write the block-table rows of sequences that got a new page, or whose window gave one back, since the
        last step: a page that was given back may be another sequence's by now, and its entry must read -1 in
        the same step."""
        cache = self.engine.cache
        for row, slot in enumerate(self.slots):
            n = (pages_for(cache.length(slot)), cache.pages_held(slot))
            if n != self.n_pages[row]:
                for g, table in self.tables.items():
                    table[row].copy_(cache.block_table(g, [slot], n_columns=self.table_width)[0], non_blocking=True)
                self.n_pages[row] = n

    def replay(self, steps: int = 1) -> List[List[int]]:
        """`steps` replays back to back (every one reads the tokens and positions that the one before left on the
        device; the block tables already hold the pages of all of them) and one wait for the tokens of all."""
        n = len(self.slots)
        if steps == 1:
            self.graph.replay()
            out = [self.tokens[:n].tolist()]
        else:
            if self.chosen.shape[0] < steps:
                self.chosen = torch.empty(steps, self.rows, dtype=torch.int32, device=self.tokens.device)
            for i in range(steps):
                self.graph.replay()
                self.chosen[i].copy_(self.tokens)
            out = self.chosen[:steps, :n].tolist()
        self.next_tokens = out[-1]
        return out
