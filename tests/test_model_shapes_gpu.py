"""The engine at the layer sizes that are served and measured: two layers of the Llama-3-8B shape (grouped kv
heads) and of the Llama-2-7B shape (as many kv heads as heads), with a vocabulary cut to 4096 so that the plain
implementation on the CPU stays cheap.  These sizes take other kernels than the tiny configurations do: the
prefill attention with its head size known at compile time, the decode attention that stages pages in LDS, the
weight-streaming products with thousands of columns and their variants for 17 to 192 rows, vendor products above
192 rows.  float32 and bfloat16 against the plain implementation, and bfloat16 against the engine's own float32
path: whole prompts, the last 32 tokens one by one, ragged batches with reused slots, and decode batches of 5
to 140 sequences through captured graphs.  A third model has the depth of the served ones (32 layers) at a narrower
width.

The cache-consistency check of the reference's benchmark script (scripts/benchmark_inference.py:197-213: a cached
one-token step against the full recomputation) and its heterogeneous-batch test (tests/utils/test_generate.py:
77-136) are the nearest things it has."""

import gc

import pytest
import torch

pytestmark = pytest.mark.gpu

import plain_llama as P  # noqa: E402
from gpu_checks import MARGIN, check, expect  # noqa: E402

SHAPES = {
    "llama3_8b_layers": dict(src_vocab_size=4096, emb_dim=4096, nheads=32, kvheads=8, nlayers=2, hidden_dim=14336,
                             multiple_of=1, norm_eps=1e-5, rope_theta=500000.0, max_expected_seq_len=4096),
    "llama2_7b_layers": dict(src_vocab_size=4096, emb_dim=4096, nheads=32, kvheads=0, nlayers=2, hidden_dim=11008,
                             multiple_of=1, norm_eps=1e-5, rope_theta=10000.0, max_expected_seq_len=4096),
}
DTYPES = ["float32", "bfloat16"]


class Shape:
    def __init__(self, name, folder, lib):
        self.name, self.folder, self.lib = name, folder, lib
        self.cfg, self.weights = P.load_model_folder(folder)
        self.models = {}

    def model(self, dtype):
        if dtype not in self.models:
            self.models[dtype] = self.lib.get_model("hf_pretrained", model_path=self.folder, data_type=dtype)
        return self.models[dtype]

    def tokens(self, n, seed):
        g = torch.Generator().manual_seed(seed)
        return torch.randint(0, self.cfg.vocab, (n,), generator=g).tolist()


@pytest.fixture(scope="module", params=sorted(SHAPES))
def shape(request, tmp_path_factory):
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    import fms_amd
    from fms_amd.kernels import load

    load()
    folder = str(tmp_path_factory.mktemp(request.param))
    # the weights of the benchmark (N(0, 0.02)), and norm scales that are not all one, so that a norm in the wrong place shows
    fms_amd.write_model_folder(folder, fms_amd.LLaMAConfig(**SHAPES[request.param]), seed=17, std=0.02, norm_std=0.1)
    print(f"[{request.param}] model folder written", flush=True)
    s = Shape(request.param, folder, fms_amd)
    yield s
    s.models.clear()
    del s
    gc.collect()
    torch.cuda.empty_cache()


@pytest.mark.parametrize("dtype", DTYPES)
def test_whole_prompt_and_last_32_tokens_one_by_one(shape, dtype):
    from fms_amd.engine import Engine

    engine = Engine(shape.model(dtype), max_tokens=1024, max_slots=1)
    ids = shape.tokens(700, 1)
    want = expect(shape.weights, shape.cfg, ids, dtype)
    slot = engine.new_sequence()
    check(engine.step([slot], [ids], "all"), want, dtype)
    engine.end_sequence(slot)
    slot = engine.new_sequence()
    got = [engine.step([slot], [ids[:-32]], "all")]
    for tok in ids[-32:]:
        got.append(engine.step([slot], [[tok]], "last"))
    engine.end_sequence(slot)
    check(torch.cat(got), want, dtype)


@pytest.mark.parametrize("dtype", DTYPES)
def test_ragged_batches_with_early_ends_and_reused_slots(shape, dtype):
    from fms_amd.engine import Engine

    engine = Engine(shape.model(dtype), max_tokens=12 * 64, max_slots=5)  # the first round fills every page
    rounds = [
        [(70, 3), (5, 9), (200, 2), (129, 1), (64, 6)],  # (prompt length, decoded tokens)
        [(33, 8), (300, 4), (1, 5)],
    ]
    seed = 100
    for requests in rounds:
        seqs = []
        for prompt_len, n_decode in requests:
            seed += 1
            seqs.append(dict(ids=shape.tokens(prompt_len + n_decode, seed), prompt=prompt_len, slot=engine.new_sequence(),
                             got=[], at=prompt_len))
        logits = engine.step([s["slot"] for s in seqs], [s["ids"][: s["prompt"]] for s in seqs], "all")
        row = 0
        for s in seqs:
            s["got"].append(logits[row : row + s["prompt"]])
            row += s["prompt"]
        alive = list(seqs)
        while alive:
            for s in alive:
                if s["at"] == len(s["ids"]):
                    engine.end_sequence(s["slot"])  # ends earlier: its slot and pages go back while the others go on
            alive = [s for s in alive if s["at"] < len(s["ids"])]
            if not alive:
                break
            logits = engine.step([s["slot"] for s in alive], [[s["ids"][s["at"]]] for s in alive], "last")
            for i, s in enumerate(alive):
                s["got"].append(logits[i : i + 1])
                s["at"] += 1
        engine.cache.check()
        assert engine.cache.live_slots() == []
        for s in seqs:
            check(torch.cat(s["got"]), expect(shape.weights, shape.cfg, s["ids"], dtype), dtype)


@pytest.mark.parametrize("dtype", DTYPES)
def test_steps_of_any_mix(shape, dtype):
    """In one step some sequences bring a piece of their prompt, others one token, and new ones join while the rest go
    on (a seeded random schedule): at these sizes a step with any longer piece runs the prefill kernels for all of its
    rows, a step of single tokens the decode kernels."""
    import random

    from fms_amd.engine import Engine

    engine = Engine(shape.model(dtype), max_tokens=4 * 448, max_slots=4)
    rng = random.Random(23)
    waiting = [shape.tokens(rng.choice((3, 64, 65, 130, 300, 420)), 500 + i) for i in range(7)]
    running, finished, n_mixed = [], [], 0
    while waiting or running:
        while waiting and len(running) < 4 and (not running or rng.random() < 0.5):
            running.append(dict(ids=waiting.pop(), slot=engine.new_sequence(), at=0, got=[]))
        pieces = []
        for seq in running:
            n = min(len(seq["ids"]) - seq["at"], rng.choice((1, 1, 1, 2, 17, 64, 130)))
            pieces.append(seq["ids"][seq["at"] : seq["at"] + n])
        n_mixed += len({len(p) == 1 for p in pieces}) == 2
        logits = engine.step([seq["slot"] for seq in running], pieces, "all")
        row = 0
        for seq, piece in zip(running, pieces):
            seq["got"].append(logits[row : row + len(piece)])
            seq["at"] += len(piece)
            row += len(piece)
        for seq in [seq for seq in running if seq["at"] == len(seq["ids"])]:
            engine.end_sequence(seq["slot"])
            running.remove(seq)
            finished.append(seq)
        engine.cache.check()
    assert engine.cache.live_slots() == [] and len(finished) == 7 and n_mixed >= 4
    for seq in finished:
        check(torch.cat(seq["got"]), expect(shape.weights, shape.cfg, seq["ids"], dtype), dtype)


def prompt_lengths(n):
    special = [63, 64, 65, 1, 127, 128, 191, 320]
    return [(special[i] if i < len(special) else 2 + (53 * i * i + 17 * i) % 250) for i in range(n)]


@pytest.mark.parametrize("n_seqs", [5, 24, 64, 80, 128, 140, 180])
def test_decode_batches_through_graphs(shape, n_seqs):
    """bfloat16 decode steps of 5 to 180 sequences of unequal lengths (above 192 rows, which the tiny configurations run, the products are the vendor's
    and nothing is fused), as generation runs them
    (decode_and_choose: a captured graph, the token choice inside it), against the engine's float32 path fed
    the same tokens, and both against the plain implementation.  After three steps every third sequence ends."""
    from fms_amd.engine import Engine
    from fms_amd.sampling import SamplingParams

    greedy = SamplingParams(do_sample=False)
    lens = prompt_lengths(n_seqs)
    room = sum(-(-(n + 8) // 64) * 64 for n in lens)
    half = Engine(shape.model("bfloat16"), max_tokens=room, max_slots=n_seqs, use_graphs=True)
    full = Engine(shape.model("float32"), max_tokens=room, max_slots=n_seqs, use_graphs=False)
    assert half.use_graphs
    seqs = [dict(ids=shape.tokens(n, 700 + 3 * n_seqs + i), n=n, half=[], full=[]) for i, n in enumerate(lens)]
    for engine, key in ((half, "slot_h"), (full, "slot_f")):
        for s in seqs:
            s[key] = engine.new_sequence()
        for i in range(0, n_seqs, 16):
            group = seqs[i : i + 16]
            logits = engine.step([s[key] for s in group], [s["ids"] for s in group], "last")
            if engine is full:
                for s, tok in zip(group, logits.argmax(-1).tolist()):
                    s["next"] = tok
    alive = list(seqs)
    for step in range(6):
        if step == 3:
            for s in alive[::3]:
                half.end_sequence(s["slot_h"])
                full.end_sequence(s["slot_f"])
            alive = [s for i, s in enumerate(alive) if i % 3]
        fed = [s["next"] for s in alive]
        chosen = half.decode_and_choose([s["slot_h"] for s in alive], fed, greedy)
        from_graph = half.last_graph.logits[: len(alive)].float().cpu()
        assert chosen == from_graph.argmax(-1).tolist()
        exact = full.step([s["slot_f"] for s in alive], [[t] for t in fed], "last").cpu()
        for s, tok, row_h, row_f in zip(alive, chosen, from_graph, exact):
            s["ids"] = s["ids"] + [s["next"]]
            s["half"].append(row_h)
            s["full"].append(row_f)
            s["next"] = tok
    for s in alive:
        half.end_sequence(s["slot_h"])
        full.end_sequence(s["slot_f"])
    half.cache.check()
    assert half.cache.live_slots() == [] == full.cache.live_slots()
    assert len(half.graph_captures) >= 2  # the batch before and after the early ends
    # against the plain implementation: the sequences around the page borders and every eighth of the others
    largest = 0.0
    for i, s in enumerate(seqs):
        if i < 8 or i % 8 == 0:
            want = expect(shape.weights, shape.cfg, s["ids"], "bfloat16")[s["n"] :]
            check(torch.stack(s["half"]), want, "bfloat16")
            check(torch.stack(s["full"]), want.logits, "float32")
            largest = max(largest, float(want.ref_error.max()))
    # every sequence: the bfloat16 graph against the float32 path (which the check above ties to the plain
    # implementation), no further apart than the reference's own bfloat16 error on the sequences above
    for i, s in enumerate(seqs):
        error = float((torch.stack(s["half"]) - torch.stack(s["full"])).abs().max())
        assert error <= MARGIN * largest, f"sequence {i} ({s['n']} prompt tokens): bfloat16 is {error:.4g} from float32"


def test_replayed_and_eager_steps_choose_the_same_tokens(shape):
    """At these sizes too (the products for 17 to 192 rows cut K by the number of rows, the decode attention splits
    by it): an eager decode step is filled up to the rows of the captured step, so generation through graphs and
    through eager steps gives the same tokens bit for bit while the batch shrinks through the row buckets."""
    from fms_amd.engine import Engine
    from fms_amd.generation import generate_requests
    from fms_amd.sampling import SamplingParams

    model = shape.model("bfloat16")
    lens = prompt_lengths(45)
    prompts = [shape.tokens(n, 3000 + i) for i, n in enumerate(lens)]
    room = sum(-(-(n + 60) // 64) * 64 for n in lens)
    stops = list(range(5, shape.cfg.vocab, 19))
    got = {}
    for graphs in (True, False):
        engine = Engine(model, max_tokens=room, max_slots=len(lens), use_graphs=graphs)
        for sampling in (SamplingParams(do_sample=False), SamplingParams(do_sample=True, temperature=0.8, top_k=10)):
            got[(graphs, sampling.do_sample)] = generate_requests(engine, prompts, max_new_tokens=60, sampling=sampling, seed=9,
                                                                  stop_token_ids=stops)
        engine.cache.check()
        if graphs:
            assert len(set(engine.graph_captures)) >= 4
    assert got[(True, False)] == got[(False, False)] and got[(True, True)] == got[(False, True)]


# ---- depth ------------------------------------------------------------------------------------------------------
DEEP = dict(src_vocab_size=4096, emb_dim=1024, nheads=8, kvheads=2, nlayers=32, hidden_dim=3584, multiple_of=1,
            norm_eps=1e-5, rope_theta=500000.0, max_expected_seq_len=2048)


@pytest.fixture(scope="module")
def deep(tmp_path_factory):
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    import fms_amd
    from fms_amd.kernels import load

    load()
    folder = str(tmp_path_factory.mktemp("deep"))
    fms_amd.write_model_folder(folder, fms_amd.LLaMAConfig(**DEEP), seed=23, std=0.02, norm_std=0.1)
    s = Shape("deep", folder, fms_amd)
    yield s
    s.models.clear()
    del s
    gc.collect()
    torch.cuda.empty_cache()


@pytest.mark.parametrize("dtype", DTYPES)
def test_thirty_two_layers(deep, dtype):
    """As many layers as the served models have (head size 128, grouped kv heads, a narrower width so that the plain
    implementation stays cheap): what grows with depth - the rounding of the residual stream, of every layer's
    branch outputs, of the cache - shows here and not in two layers.  A prompt with its last 32 tokens decoded one by
    one, and a ragged batch, against the plain implementation; bfloat16 is held to the error that the reference's
    own bfloat16 arithmetic has at this depth (measured once on the full Llama-3-8B layer shape with 32 layers and
    200 tokens: float32 0.00014 off on average, bfloat16 0.255 where the reference's arithmetic is 0.339 off)."""
    from fms_amd.engine import Engine

    engine = Engine(deep.model(dtype), max_tokens=1024, max_slots=3)
    ids = deep.tokens(300, 4)
    want = expect(deep.weights, deep.cfg, ids, dtype)
    slot = engine.new_sequence()
    got = [engine.step([slot], [ids[:-32]], "all")]
    for tok in ids[-32:]:
        got.append(engine.step([slot], [[tok]], "last"))
    engine.end_sequence(slot)
    check(torch.cat(got), want, dtype)
    seqs = [deep.tokens(n, 40 + n) for n in (130, 65, 9)]
    slots = [engine.new_sequence() for _ in seqs]
    cut = [len(s) - 3 for s in seqs]
    logits = engine.step(slots, [s[:c] for s, c in zip(seqs, cut)], "all")
    per_seq, at = [], 0
    for c in cut:
        per_seq.append([logits[at : at + c]])
        at += c
    for k in range(3):
        logits = engine.step(slots, [[s[c + k]] for s, c in zip(seqs, cut)], "last")
        for i in range(len(seqs)):
            per_seq[i].append(logits[i : i + 1])
    for s, slot, parts in zip(seqs, slots, per_seq):
        engine.end_sequence(slot)
        check(torch.cat(parts), expect(deep.weights, deep.cfg, s, dtype), dtype)
    engine.cache.check()


# ---- the benchmark's context ---------------------------------------------------------------------------------------
LONG = dict(SHAPES["llama3_8b_layers"], nlayers=1, max_expected_seq_len=8192)


class LongShape(Shape):
    """One layer of the Llama-3-8B shape with positions up to 8192.  The plain implementation's answers for the
    two long sequences are worked out once and shared by the tests (a request that is the beginning of a longer one
    has the longer one's first rows: causality)."""

    def __init__(self, name, folder, lib):
        super().__init__(name, folder, lib)
        self.long_ids = self.tokens(8150, 1)
        self.other_ids = self.tokens(3000, 2)
        self._wanted = {}

    def want(self, which, dtype):
        if (which, dtype) not in self._wanted:
            print(f"[long] plain implementation: {which} in {dtype}", flush=True)
            self._wanted[(which, dtype)] = expect(self.weights, self.cfg, self.long_ids if which == "long" else self.other_ids, dtype)
        return self._wanted[(which, dtype)]


@pytest.fixture(scope="module")
def long_shape(tmp_path_factory):
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    import fms_amd
    from fms_amd.kernels import load

    load()
    folder = str(tmp_path_factory.mktemp("long"))
    fms_amd.write_model_folder(folder, fms_amd.LLaMAConfig(**LONG), seed=29, std=0.02, norm_std=0.1)
    s = LongShape("long", folder, fms_amd)
    yield s
    s.models.clear()
    s._wanted.clear()
    del s
    gc.collect()
    torch.cuda.empty_cache()


def _decode(engine, slots, fed, dtype):
    """The logits of one decode step: bfloat16 as generation runs it (a replayed graph, fed the given tokens whatever
    it chose before), float32 as an eager step."""
    if dtype == "bfloat16":
        from fms_amd.sampling import SamplingParams

        engine.decode_and_choose(slots, fed, SamplingParams(do_sample=False))
        return engine.last_graph.logits[: len(slots)].clone()
    return engine.step(slots, [[t] for t in fed], "last")


@pytest.mark.parametrize("dtype", DTYPES)
def test_context_of_8192_whole_and_last_32_one_by_one(long_shape, dtype):
    """A request that fills the benchmark's context (8150 of 8192 positions), whole and with its last 32 tokens one by
    one: 128 pages a sequence, the decode attention's split at that bound, the graph captured for a context of 8192."""
    from fms_amd.engine import Engine

    ids, want = long_shape.long_ids, long_shape.want("long", dtype)
    engine = Engine(long_shape.model(dtype), max_tokens=8192, max_slots=1, use_graphs=dtype == "bfloat16")
    slot = engine.new_sequence()
    check(engine.step([slot], [ids], "all"), want, dtype)
    engine.end_sequence(slot)
    slot = engine.new_sequence()
    rows = sorted(set(range(0, len(ids) - 32, 29)) | set(range(len(ids) - 96, len(ids) - 32)))
    got = [engine.step([slot], [ids[:-32]], [rows])]
    for tok in ids[-32:]:
        got.append(_decode(engine, [slot], [tok], dtype))
    engine.end_sequence(slot)
    check(torch.cat(got), want[rows + list(range(len(ids) - 32, len(ids)))], dtype)
    if dtype == "bfloat16":
        assert engine.graph_captures == [(1, 8192)]
    engine.cache.check()


@pytest.mark.parametrize("dtype", DTYPES)
def test_context_of_8192_in_a_ragged_batch_with_reused_slots(long_shape, dtype):
    """Requests of 8000, 130 and 3000 tokens start together; the short one ends first, then the middle one; a second
    batch takes their slots and pages."""
    from fms_amd.engine import Engine

    engine = Engine(long_shape.model(dtype), max_tokens=(125 + 3 + 47) * 64, max_slots=3, use_graphs=dtype == "bfloat16")
    first = [  # (ids, prompt length, expected)
        (long_shape.long_ids[:8000], 7990, long_shape.want("long", dtype)[:8000]),
        (long_shape.tokens(130, 3), 127, None),
        (long_shape.other_ids, 2993, long_shape.want("other", dtype)),
    ]
    second = [(long_shape.tokens(300, 4), 296, None), (long_shape.tokens(70, 5), 64, None), (long_shape.tokens(9, 6), 1, None)]
    for requests in (first, second):
        seqs = [dict(ids=ids, at=n, slot=engine.new_sequence(), want=w, got=[]) for ids, n, w in requests]
        # of the prompts: the last 64 rows and some hundred spread ones
        rows = [sorted(set(range(0, s["at"], 41)) | set(range(max(0, s["at"] - 64), s["at"]))) for s in seqs]
        logits = engine.step([s["slot"] for s in seqs], [s["ids"][: s["at"]] for s in seqs], rows)
        at = 0
        for s, r in zip(seqs, rows):
            s["rows"] = list(r)
            s["got"].append(logits[at : at + len(r)])
            at += len(r)
        alive = list(seqs)
        while True:
            for s in alive:
                if s["at"] == len(s["ids"]):
                    engine.end_sequence(s["slot"])
            alive = [s for s in alive if s["at"] < len(s["ids"])]
            if not alive:
                break
            logits = _decode(engine, [s["slot"] for s in alive], [s["ids"][s["at"]] for s in alive], dtype)
            for i, s in enumerate(alive):
                s["got"].append(logits[i : i + 1])
                s["rows"].append(s["at"])
                s["at"] += 1
        engine.cache.check()
        assert engine.cache.live_slots() == []
        for s in seqs:
            want = s["want"] if s["want"] is not None else expect(long_shape.weights, long_shape.cfg, s["ids"], dtype)
            check(torch.cat(s["got"]), want[s["rows"]], dtype)
    if dtype == "bfloat16":
        assert (4, 8192) in engine.graph_captures  # three sequences in a step of four rows, the bound of the long one
