"""The step function: one batch of sequences, each bringing its next tokens,
run as one ragged batch from the cache; logits come back for the wanted places.

A step runs only the tokens it is given.  Sequences are named by their cache
slots; a sequence's position is its length in the cache, so the same call
serves whole prompts, single decoded tokens, and anything between.  There is
no padding: tokens of all sequences are laid end to end.
"""

from __future__ import annotations

import os
from typing import List, Optional, Sequence, Union

import torch

from ..cache import pages_for
from ..sampling import SamplingParams, choose
from .batch import StepBatch, build_batch
from .decode_graph import CONTEXT_HEADROOM, DecodeGraph, context_bucket, row_bucket
from .model import DecoderModel


class Engine:
    def __init__(self, model: DecoderModel, max_tokens: Optional[int] = None, max_slots: Optional[int] = None,
                 use_graphs: Optional[bool] = None):
        """max_tokens: the most tokens live sequences hold at a time, each rounded up to a page of 64
        (default: one sequence of the model's full length).  max_slots: the most live sequences.
        use_graphs: replay decode steps as captured HIP graphs (default: yes, if every part allows it
        and the environment variable FMS_AMD_NO_GRAPHS is not set)."""
        if model.device is None:
            raise RuntimeError("the model has no weights on a device yet (use get_model)")
        self.model = model
        self.device = model.device
        if max_tokens is None:
            max_tokens = model.spec.max_seq_len
        if max_slots is None:
            max_slots = max(1, pages_for(max_tokens))
        self.cache = model.make_cache(max_tokens, max_slots)
        self.vocab = model.spec.vocab
        if use_graphs is None:
            use_graphs = not os.environ.get("FMS_AMD_NO_GRAPHS")
        capturable = all(getattr(p, "graph_safe", True) for p in model.walk())
        self.use_graphs = bool(use_graphs) and capturable
        # Eager decode steps take the shape of the captured step of their row bucket (padding rows of sequence -1),
        # if every part knows such rows: eager steps and replays then run the same kernels with the same launches
        # and give the same bits.
        self.pads_decode_rows = capturable
        self._graphs = {}
        self.graph_captures = []  # (rows, context bound) of every capture, in order
        self.last_graph: Optional[DecodeGraph] = None  # the graph of the last replayed step (its .logits are that step's)

    # ---- sequences ---------------------------------------------------------
    def new_sequence(self) -> int:
        return self.cache.alloc_slot()

    def end_sequence(self, slot: int) -> None:
        self.cache.free_slot(slot)

    def length(self, slot: int) -> int:
        return self.cache.length(slot)

    # ---- the step ------------------------------------------------------------
    def step(
        self,
        slots: Sequence[int],
        tokens: Sequence[Sequence[int]],
        want: Union[str, Sequence[Sequence[int]]] = "last",
    ) -> torch.Tensor:
        """Append `tokens[b]` to sequence `slots[b]` and return float32 logits [n_wanted, vocab].

        want: "last" (the last token of every sequence), "all", or for each sequence the places
        among its new tokens.  Rows come in the order of the sequences and of `want`.
        """
        batch = self.prepare(slots, tokens, want)
        if batch.n_tokens == 0:
            return torch.empty(0, self.vocab, dtype=torch.float32, device=self.device)
        logits = self.model.forward(batch, self.cache)
        return logits if batch.n_wanted == batch.n_logit_rows else logits[: batch.n_wanted]

    def decode_and_choose(
        self,
        slots: Sequence[int],
        tokens: Sequence[int],
        sampling: SamplingParams,
        seeds: Optional[Sequence[int]] = None,
        counters: Optional[Sequence[int]] = None,
    ) -> List[int]:
        """One decode step and the choice of the next token for every sequence: `tokens[b]` is appended to
        `slots[b]`, the chosen tokens come back as host integers.  Replays a captured graph when it can."""
        return self.decode_and_choose_many(slots, tokens, sampling, seeds, counters, steps=1)[0]

    def decode_and_choose_many(
        self,
        slots: Sequence[int],
        tokens: Sequence[int],
        sampling: SamplingParams,
        seeds: Optional[Sequence[int]] = None,
        counters: Optional[Sequence[int]] = None,
        steps: int = 1,
    ) -> List[List[int]]:
        """`steps` decode steps of the same sequences, each fed what the step before chose: the chosen tokens of
        every step, `steps` lists of one token per sequence.  With graphs the steps are replayed back to back and
        the host waits once, for all their tokens; every step is the step that `decode_and_choose` runs, and
        chooses the same tokens.  All sequences go on for all steps: a caller that watches for stop tokens takes
        what it wants of the result and ends the sequence (whose cache then holds tokens past its end, which is
        harmless, as the slot is given back whole).  Room for all steps is made first, or for none of them."""
        slots = [int(s) for s in slots]
        tokens = [int(t) for t in tokens]
        steps = int(steps)
        if steps < 1:
            raise ValueError("at least one step")
        if not self.use_graphs:
            out = []
            for i in range(steps):
                logits = self.step(slots, [[t] for t in tokens], "last")
                step_counters = None if counters is None else [c + i for c in counters]
                tokens = choose(logits, sampling, seeds, step_counters).tolist()
                out.append(tokens)
            return out
        if len(set(slots)) != len(slots) or len(tokens) != len(slots):
            raise ValueError("one token per sequence, each sequence once")
        live = set(self.cache.live_slots())
        for s in slots:
            if s not in live:
                raise ValueError(f"slot {s} is not live")
        for t in tokens:
            if not 0 <= t < self.vocab:
                raise IndexError(f"token id {t} is outside the vocabulary of {self.vocab}")
        # what the sequences looked like before this step: a graph's buffers still describe them only if
        # nothing but the graph's own last replay has touched them since
        before = [self.cache.stamp(s) for s in slots]
        positions = self.cache.extend_many(slots, [steps] * len(slots))  # room for all, or for none
        rows = row_bucket(len(slots))
        longest = max(positions) + steps
        how = (sampling.do_sample, float(sampling.temperature), int(sampling.top_k or 0))
        fitting = [k for k in self._graphs if k[0] == rows and k[2:] == how and k[1] >= longest]
        if fitting:
            graph = self._graphs[min(fitting)]
        else:
            for old in [k for k in self._graphs if k[0] == rows and k[2:] == how]:
                del self._graphs[old]  # a longer context replaces the graph of the shorter one
            ctx = context_bucket(longest + CONTEXT_HEADROOM, self.cache.max_seq_len)
            graph = self._graphs[(rows, ctx) + how] = DecodeGraph(self, rows, ctx, sampling)
            graph.capture()
            self.graph_captures.append((rows, ctx))
        if graph.slots == tuple(slots) and graph.stamps == before and graph.next_tokens == tokens:
            graph.refresh_pages()  # the same sequences, one step on, fed what the graph chose: its buffers are current
        else:
            graph.load(slots, tokens, positions, seeds or [0] * len(slots), counters or [0] * len(slots))
        graph.stamps = [self.cache.stamp(s) for s in slots]
        self.last_graph = graph
        return graph.replay(steps)

    def prepare(self, slots, tokens, want) -> StepBatch:
        slots = [int(s) for s in slots]
        if len(slots) != len(tokens):
            raise ValueError("one token list per sequence is needed")
        if len(set(slots)) != len(slots):
            raise ValueError("a sequence appears twice in one step")
        for b, toks in enumerate(tokens):
            if len(toks) == 0:
                raise ValueError(f"sequence {b} of the step brings no token")
            lo, hi = min(toks), max(toks)
            if lo < 0 or hi >= self.vocab:
                raise IndexError(f"token id {lo if lo < 0 else hi} is outside the vocabulary of {self.vocab}")
        if want == "last":
            want = [[len(t) - 1] for t in tokens]
        elif want == "all":
            want = [list(range(len(t))) for t in tokens]
        elif len(want) != len(slots):
            raise ValueError("one list of wanted places per sequence is needed")
        for b, (w, t) in enumerate(zip(want, tokens)):
            for place in w:
                if not 0 <= int(place) < len(t):
                    raise IndexError(f"wanted place {place} is outside the {len(t)} tokens of sequence {b}")
        starts = self.cache.extend_many(slots, [len(t) for t in tokens])  # room for all, or for none
        n_tokens = sum(len(t) for t in tokens)
        sizes = set()
        if any(len(t) > 1 for t in tokens):
            for block in self.model.layers:
                size = block.mixer.prefill_qblock(n_tokens, self.model.dtype)
                if size:
                    sizes.add(size)
        pad_to = row_bucket(len(slots)) if self.pads_decode_rows and all(len(t) == 1 for t in tokens) else 0
        batch = build_batch(self.cache, slots, tokens, starts, want, self.device, sizes, pad_rows_to=pad_to)
        if batch.is_decode:
            # the bound a graph for this step would be captured for: eager steps and replays then launch the
            # same kernels in the same shape, and give the same bits
            batch.context_bound = context_bucket(batch.max_context + CONTEXT_HEADROOM, self.cache.max_seq_len)
        return batch
