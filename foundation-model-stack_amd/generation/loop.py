"""The generation loop above the step function.

``generate_requests`` takes any number of prompts of unequal lengths, runs them
in as many batches as the cache has room for, one batch after another; in a
batch the prompts go through in one step, then every sequence still alive gets
one token per step.  A sequence ends at a stop token, at max_new_tokens, or at
the model's last position; its slot goes back at once and the batch shrinks.

``generate`` has the reference's signature and meanings
(fms/utils/generation.py:182-369) on top of that.
"""

from __future__ import annotations

import time
from typing import Callable, Iterable, List, Optional, Sequence, Set

import torch

from ..cache import PAGE_TOKENS, pages_for
from ..sampling import SamplingParams, choose, request_seed

# Decode steps that the loop runs before it looks at their tokens, when nobody asked to see every step: the host
# then waits once for several steps (its share of a step is a per cent or two), and a request that meets a stop
# token runs at most this many steps less one for nothing.
STEPS_AHEAD = 4


def plan_batches(
    prompt_lens: Sequence[int],
    max_new_tokens: int,
    max_tokens: int,
    max_batch: int,
    max_seq_len: int,
) -> List[List[int]]:
    """Split requests (by index, in order) into batches that fit the cache.

    A request may grow to min(prompt + max_new_tokens, max_seq_len) tokens, rounded up to a
    page; a batch holds as many consecutive requests as fit into max_tokens and max_batch.
    """
    batches: List[List[int]] = []
    current: List[int] = []
    used = 0
    for i, n in enumerate(prompt_lens):
        if n <= 0:
            raise ValueError(f"request {i} has an empty prompt")
        if n > max_seq_len:
            raise IndexError(f"request {i} has {n} prompt tokens, the model has {max_seq_len} positions")
        need = pages_for(min(n + max_new_tokens, max_seq_len)) * PAGE_TOKENS
        if need > max_tokens:
            raise ValueError(f"request {i} may need {need} cached tokens, the cache holds {max_tokens}")
        if current and (used + need > max_tokens or len(current) >= max_batch):
            batches.append(current)
            current, used = [], 0
        current.append(i)
        used += need
    if current:
        batches.append(current)
    return batches


def generate_requests(
    engine,
    prompts: Sequence[Sequence[int]],
    max_new_tokens: int = 256,
    sampling: Optional[SamplingParams] = None,
    stop_token_ids: Optional[Iterable[int]] = None,
    seed: int = 0,
    max_batch: Optional[int] = None,
    chooser: Optional[Callable] = None,
    on_step: Optional[Callable[[int, List[int], List[int]], None]] = None,
    step_times: Optional[List[float]] = None,
    before_step: Optional[Callable[[int, List[int], List[List[int]]], Optional[List[List[int]]]]] = None,
    after_choice: Optional[Callable] = None,
) -> List[List[int]]:
    """New tokens of every request (a stop token is kept, nothing follows it).

    engine: anything with new_sequence(), end_sequence(slot), step(slots, tokens, want), and
    cache.max_tokens / cache.max_slots / cache.max_seq_len.  chooser(logits, request_indices,
    counters) -> token ids overrides the built-in sampler (tests use it).  before_step(step, requests, tokens)
    sees the tokens each live request is about to be fed and may return others in their place (as many lists).
    after_choice(step, requests, logits, tokens) sees the float32 logits [live requests, vocabulary] that the
    tokens were chosen from and may return other tokens in their place; with it every step is run eagerly, so
    that its logits are at hand.
    """
    sampling = sampling or SamplingParams(do_sample=False)
    stops: Set[int] = set(int(s) for s in (stop_token_ids or ()))
    prompts = [list(map(int, p)) for p in prompts]
    results: List[List[int]] = [[] for _ in prompts]
    if max_new_tokens <= 0 or not prompts:
        return results
    cache = engine.cache
    max_batch = min(max_batch or cache.max_slots, cache.max_slots)

    def pick(logits, request_ids, counters) -> List[int]:
        if chooser is not None:
            return [int(t) for t in chooser(logits, request_ids, counters)]
        seeds = [request_seed(seed, r) for r in request_ids]
        return choose(logits, sampling, seeds, counters).tolist()

    fused = chooser is None and after_choice is None and hasattr(engine, "decode_and_choose")
    watched = before_step is not None or on_step is not None or step_times is not None  # someone looks at every step
    for batch in plan_batches([len(p) for p in prompts], max_new_tokens, cache.max_tokens, max_batch, cache.max_seq_len):
        slots = {r: engine.new_sequence() for r in batch}
        alive = list(batch)
        feed = {r: prompts[r] for r in batch}
        step_no = 0
        try:
            while alive:
                if before_step is not None:
                    given = before_step(step_no, list(alive), [list(feed[r]) for r in alive])
                    if given is not None:
                        if len(given) != len(alive) or any(len(g) == 0 for g in given):
                            raise ValueError("before_step must return one non-empty token list per live request")
                        for r, g in zip(alive, given):
                            feed[r] = [int(x) for x in g]
                t0 = time.time()
                if fused and step_no > 0 and all(len(feed[r]) == 1 for r in alive):
                    # decode: the step and the choice in one call (a captured graph when the engine has one).  With
                    # nobody watching the single steps, several are run before the host looks at their tokens, never
                    # past a request's limit or the model's last position; a request that meets a stop token among
                    # them ends there, and what it chose after is dropped.
                    ahead = 1
                    if not watched and hasattr(engine, "decode_and_choose_many"):
                        ahead = min(STEPS_AHEAD, *(min(max_new_tokens - len(results[r]),
                                                       cache.max_seq_len + 1 - len(prompts[r]) - len(results[r])) for r in alive))
                    step_args = ([slots[r] for r in alive], [feed[r][0] for r in alive], sampling,
                                 [request_seed(seed, r) for r in alive], [len(results[r]) for r in alive])
                    if ahead > 1:
                        chosen = engine.decode_and_choose_many(*step_args, steps=ahead)
                    else:
                        chosen = [engine.decode_and_choose(*step_args)]
                else:
                    logits = engine.step([slots[r] for r in alive], [feed[r] for r in alive], "last")
                    tokens = pick(logits, alive, [len(results[r]) for r in alive])
                    if after_choice is not None:
                        given = after_choice(step_no, list(alive), logits, list(tokens))
                        if given is not None:
                            if len(given) != len(alive):
                                raise ValueError("after_choice must return one token per live request")
                            tokens = [int(t) for t in given]
                    chosen = [tokens]
                if step_times is not None:
                    step_times.append(time.time() - t0)
                if on_step is not None:
                    on_step(step_no, list(alive), list(chosen[0]))
                going = list(alive)
                for tokens in chosen:
                    for r, tok in zip(alive, tokens):
                        if r not in going:
                            continue
                        results[r].append(tok)
                        length = len(prompts[r]) + len(results[r])
                        # the token just chosen is not in the cache yet: it may be fed only if a position is left for it
                        if tok in stops or len(results[r]) >= max_new_tokens or length > cache.max_seq_len:
                            going.remove(r)
                        else:
                            feed[r] = [tok]
                    step_no += 1
                for r in alive:
                    if r not in going:
                        engine.end_sequence(slots.pop(r))
                alive = going
        finally:
            for slot in slots.values():
                engine.end_sequence(slot)
    return results


# --------------------------------------------------------------------------
# the reference's call
# --------------------------------------------------------------------------
def _real_tokens(input_ids: torch.Tensor, extra_kwargs) -> List[List[int]]:
    """Rows of a rectangular batch without their padding.

    pad_input_ids records the real lengths and the padding side; a mask from elsewhere is read
    as left padding, where the last row of a sequence's mask is open exactly at its real tokens.
    """
    rows = input_ids.tolist()
    extra = extra_kwargs or {}
    if "lengths" in extra:
        side = extra.get("padding_side", "left")
        return [row[len(row) - n :] if side == "left" else row[:n] for row, n in zip(rows, extra["lengths"])]
    mask = extra.get("mask")
    if mask is None:
        return rows
    return [[tok for tok, keep in zip(row, (mask[b][-1] == 0).tolist()) if keep] for b, row in enumerate(rows)]


def generate(
    model,
    input_ids: torch.Tensor,
    max_seq_len: int = 4096,
    max_new_tokens: int = 256,
    temperature: float = 1.0,
    top_k: int = 10,
    do_sample: bool = True,
    num_beams: int = 1,
    use_cache: bool = False,
    contiguous_cache: bool = False,
    eos_token_id: Optional[int] = None,
    pad_token_id: Optional[int] = None,
    timing: str = "",
    prepare_model_inputs_hook: Optional[Callable] = None,
    post_iteration_hook: Optional[Callable] = None,
    extra_kwargs: Optional[dict] = None,
    seed: int = 0,
):
    """The reference's generate (fms/utils/generation.py:182-369) on this engine.

    input_ids: a 1-D tensor (one prompt) or a 2-D tensor (a batch; rows padded by pad_input_ids
    carry their mask in extra_kwargs).  Returns prompt + generated tokens, [S + n] or [B, S + n];
    a row that ended early is filled up with eos_token_id (or pad_token_id, or 0).
    use_cache / contiguous_cache are accepted for compatibility: the engine always caches.
    With timing "per-token" or "e2e" returns (result, times) as the reference does.
    prepare_model_inputs_hook(i, input_ids, kwargs) -> (input_ids, kwargs) is called before step i, as in the
    reference (fms/utils/generation.py:295-296), with the tokens about to be fed as a tensor [rows alive, n]
    (left-padded with pad_token_id or 0 where the rows differ in length) and the extra_kwargs; the tokens it
    returns are fed instead (the same shape; padding places are ignored).
    post_iteration_hook(token_position, logits, next_val, kwargs) -> (next_val, kwargs) is called after every choice,
    as in the reference (fms/utils/generation.py:328-331): token_position counts from the padded prompt's width,
    logits [B, V] are what the choice was made from (divided by the temperature and cut to top_k when sampling),
    next_val [B, 1] the chosen tokens; the tokens it returns go on.  Rows that have ended show -inf logits and the
    fill token.  With this hook every step runs eagerly (its logits have to be at hand).
    """
    from ..engine import Engine  # late import: engine imports the kernels

    if num_beams != 1:
        raise NotImplementedError("generate() does yet not support beam search")
    if not isinstance(input_ids, torch.Tensor):
        raise TypeError("input_ids must be one of Tensor or List")
    is_batch = input_ids.dim() > 1
    ids2d = input_ids if is_batch else input_ids.unsqueeze(0)
    prompts = _real_tokens(ids2d.cpu(), extra_kwargs)
    prompts = [p[-max_seq_len:] for p in prompts]

    engine = model if isinstance(model, Engine) else default_engine(model, prompts, max_new_tokens)
    times: List[float] = []
    start = time.time()
    state = {"kwargs": dict(extra_kwargs or {})}  # the kwargs that the reference threads through both hooks
    pad = pad_token_id if pad_token_id is not None else 0
    before = None
    if prepare_model_inputs_hook is not None:

        def before(step, alive, tokens):
            width = max(len(t) for t in tokens)
            ids = torch.tensor([[pad] * (width - len(t)) + list(t) for t in tokens], dtype=ids2d.dtype)
            ids, state["kwargs"] = prepare_model_inputs_hook(step, ids, state["kwargs"])
            return [row[width - len(t):] for row, t in zip(ids.tolist(), tokens)]

    after = None
    if post_iteration_hook is not None:
        fill_token = eos_token_id if eos_token_id is not None else pad
        n_rows, prompt_length = ids2d.shape

        def after(step, alive, logits, tokens):
            # fms/utils/generation.py:328-331: (token position, the logits the choice was made from, next_val
            # [B, 1], kwargs) -> (next_val, kwargs).  With sampling the reference's logits are divided by the
            # temperature and, with top_k, set to -inf below the k-th largest (:317-323).  Rows that have ended
            # (the reference keeps feeding them) show -inf everywhere and the fill token.
            shown = logits.float()
            if do_sample:
                shown = shown / temperature
                if top_k:
                    kth = torch.topk(shown, min(int(top_k), shown.shape[-1])).values[:, [-1]]
                    shown = shown.masked_fill(shown < kth, float("-inf"))
            full = torch.full((n_rows, shown.shape[-1]), float("-inf"), dtype=shown.dtype, device=shown.device)
            rows = torch.tensor(alive, dtype=torch.long, device=shown.device)
            full[rows] = shown
            next_val = torch.full((n_rows, 1), fill_token, dtype=ids2d.dtype, device=shown.device)
            next_val[rows, 0] = torch.tensor(tokens, dtype=ids2d.dtype, device=shown.device)
            next_val, state["kwargs"] = post_iteration_hook(step + prompt_length, full, next_val, state["kwargs"])
            return [int(t) for t in next_val.reshape(n_rows, -1)[rows, 0].tolist()]

    new = generate_requests(
        engine,
        prompts,
        max_new_tokens=max_new_tokens,
        sampling=SamplingParams(do_sample=do_sample, temperature=temperature, top_k=top_k or 0),
        stop_token_ids=None if eos_token_id is None else [eos_token_id],
        seed=seed,
        step_times=times if timing == "per-token" else None,
        before_step=before,
        after_choice=after,
    )
    if timing == "e2e":
        if engine.device.type == "cuda":
            torch.cuda.synchronize()
        times = [time.time() - start]
    fill = eos_token_id if eos_token_id is not None else (pad_token_id if pad_token_id is not None else 0)
    width = max(len(n) for n in new) if new else 0
    rows = []
    for b in range(ids2d.shape[0]):
        tail = new[b] + [fill] * (width - len(new[b]))
        rows.append(torch.cat((ids2d[b].cpu(), torch.tensor(tail, dtype=ids2d.dtype))))
    result = torch.stack(rows).to(input_ids.device)
    if not is_batch:
        result = result[0]
    if timing != "":
        return result, times
    return result


def logits(model, input_ids: torch.Tensor, last_n_tokens: int = 0, extra_kwargs: Optional[dict] = None, **kwargs) -> torch.Tensor:
    """What the reference's model returns when it is called on token ids without a cache
    (fms/models/llama.py:425-450): float32 logits [B, S, V] of a rectangular batch ([S, V] for a 1-D input), or of
    the last `last_n_tokens` places only.  Rows padded by pad_input_ids come with its kwargs (as extra_kwargs or as
    keyword arguments, the way the reference's model takes `mask` and `position_ids`); a padding place holds zeros.
    """
    from ..engine import Engine  # late import: engine imports the kernels

    if not isinstance(input_ids, torch.Tensor) or input_ids.dim() not in (1, 2):
        raise TypeError("input_ids must be a Tensor [S] or [B, S]")
    if last_n_tokens < 0:
        raise ValueError("last_n_tokens counts places from the end: 0 (all) or more")
    extra = dict(extra_kwargs or {})
    extra.update(kwargs)
    if extra.get("use_cache") or extra.get("past_key_value_states") is not None:
        raise NotImplementedError("a call on token ids keeps no cache: sequences that go on are stepped through an Engine")
    is_batch = input_ids.dim() > 1
    ids2d = input_ids if is_batch else input_ids.unsqueeze(0)
    rows = _real_tokens(ids2d.cpu(), extra)
    side = extra.get("padding_side", "left")
    width = ids2d.shape[1]
    keep = width if last_n_tokens == 0 else min(last_n_tokens, width)
    # the wanted places of a row, as places among its real tokens (a place that is padding has no logits)
    wanted = []
    for tokens in rows:
        offset = width - len(tokens) if side == "left" else 0  # where the row's first real token sits
        wanted.append([p - offset for p in range(width - keep, width) if 0 <= p - offset < len(tokens)])
    engine = model if isinstance(model, Engine) else default_engine(model, rows, 0)
    slots = [engine.new_sequence() for _ in rows]
    try:
        flat = engine.step(slots, rows, wanted)
    finally:
        for slot in slots:
            engine.end_sequence(slot)
    out = torch.zeros(len(rows), keep, flat.shape[-1], dtype=flat.dtype, device=flat.device)
    at = 0
    for b, (tokens, places) in enumerate(zip(rows, wanted)):
        if places:
            offset = width - len(tokens) if side == "left" else 0
            first = places[0] + offset - (width - keep)
            out[b, first : first + len(places)] = flat[at : at + len(places)]
            at += len(places)
    return out if is_batch else out[0]


def default_engine(model, prompts, max_new_tokens):
    """An engine for `model` with room for these requests, kept on the model and reused while it is large enough."""
    from ..engine import Engine

    need = sum(pages_for(min(len(p) + max_new_tokens, model.spec.max_seq_len)) for p in prompts) * PAGE_TOKENS
    engine = getattr(model, "_default_engine", None)
    if engine is None or engine.cache.max_tokens < need or engine.cache.max_slots < len(prompts):
        engine = Engine(model, max_tokens=need, max_slots=max(len(prompts), 1))
        model._default_engine = engine
    return engine
