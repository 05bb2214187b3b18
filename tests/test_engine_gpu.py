"""The engine against the plain implementation: whole sequences, token by token, ragged
batches with reused slots, long decoding, generation, and trace replay, in float32 and bfloat16."""

import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

import plain_llama as P  # noqa: E402

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

# Three tiny configurations that differ in every size and option.
CONFIGS = {
    # grouped kv heads, head size 16, untied, theta 1e4
    "A": dict(src_vocab_size=256, emb_dim=64, nheads=4, kvheads=2, nlayers=2, hidden_dim=176, multiple_of=1,
              norm_eps=1e-5, rope_theta=10000.0, max_expected_seq_len=512, tie_heads=False),
    # one kv head, head size 24 (no multiple of 16), tied head, theta 5e5, another eps
    "B": dict(src_vocab_size=384, emb_dim=96, nheads=4, kvheads=1, nlayers=3, hidden_dim=256, multiple_of=1,
              norm_eps=1e-6, rope_theta=500000.0, max_expected_seq_len=448, tie_heads=True),
    # as many kv heads as heads, head size 48, odd vocabulary, biases, scaled rotary frequencies
    "C": dict(src_vocab_size=301, emb_dim=144, nheads=3, kvheads=0, nlayers=1, hidden_dim=200, multiple_of=1,
              norm_eps=1e-4, rope_theta=50000.0, max_expected_seq_len=640, tie_heads=False, attn_bias=True,
              mlp_bias=True,
              rope_scaling={"rope_type": "llama3", "factor": 4.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0,
                            "original_max_position_embeddings": 64}),
}
DTYPES = ["float32", "bfloat16"]


@pytest.fixture(scope="module")
def lib():
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    import fms_amd
    from fms_amd.kernels import load

    load()
    return fms_amd


@pytest.fixture(scope="module")
def folders(tmp_path_factory, lib):
    out = {}
    for name, kw in CONFIGS.items():
        folder = str(tmp_path_factory.mktemp(f"model_{name}"))
        # std 0.08 and noisy norm scales: attention is not flat and a norm in the wrong place shows
        lib.write_model_folder(folder, lib.LLaMAConfig(**kw), seed=11 + len(out), std=0.08, norm_std=0.2)
        out[name] = folder
    return out


_models = {}


def get(lib, folders, name, dtype):
    key = (name, dtype)
    if key not in _models:
        _models[key] = lib.get_model("hf_pretrained", model_path=folders[name], data_type=dtype)
    return _models[key]


_plain = {}


def plain(folders, name):
    if name not in _plain:
        _plain[name] = P.load_model_folder(folders[name])
    return _plain[name]


def tokens_for(name, n, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, CONFIGS[name]["src_vocab_size"], (n,), generator=g).tolist()


def check(got, want, dtype):
    got = got.float().cpu()
    assert got.shape == want.shape
    if dtype == "float32":
        torch.testing.assert_close(got, want, atol=2e-4, rtol=1e-3)
    else:
        scale = float(want.abs().max())
        err = float((got - want).abs().max())
        assert err <= 0.03 * scale, f"bfloat16 logits differ by {err:.4g} at a scale of {scale:.4g}"


# --------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_whole_sequence(lib, folders, name, dtype):
    from fms_amd.engine import Engine

    cfg, weights = plain(folders, name)
    engine = Engine(get(lib, folders, name, dtype), max_tokens=512, max_slots=2)
    for n, seed in ((1, 1), (5, 2), (200, 3)):
        ids = tokens_for(name, n, seed)
        slot = engine.new_sequence()
        logits = engine.step([slot], [ids], "all")
        engine.end_sequence(slot)
        check(logits, P.forward(weights, cfg, ids), dtype)
    engine.cache.check()


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_last_32_tokens_one_by_one(lib, folders, name, dtype):
    from fms_amd.engine import Engine

    cfg, weights = plain(folders, name)
    engine = Engine(get(lib, folders, name, dtype), max_tokens=256, max_slots=1)
    ids = tokens_for(name, 150, 4)
    want = P.forward(weights, cfg, ids)
    slot = engine.new_sequence()
    got = [engine.step([slot], [ids[:-32]], "all")]
    for tok in ids[-32:]:
        got.append(engine.step([slot], [[tok]], "last"))
    engine.end_sequence(slot)
    check(torch.cat(got), want, dtype)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_first_tokens_and_chunks(lib, folders, name, dtype):
    """The first tokens of a sequence one by one, then chunks of unequal sizes across page borders."""
    from fms_amd.engine import Engine

    cfg, weights = plain(folders, name)
    engine = Engine(get(lib, folders, name, dtype), max_tokens=256, max_slots=1)
    ids = tokens_for(name, 140, 5)
    want = P.forward(weights, cfg, ids)
    slot = engine.new_sequence()
    got, at = [], 0
    for n in (1, 1, 1, 2, 59, 1, 63, 12):
        got.append(engine.step([slot], [ids[at : at + n]], "all"))
        at += n
    assert at == 140
    engine.end_sequence(slot)
    check(torch.cat(got), want, dtype)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_ragged_batches_with_reused_slots(lib, folders, name, dtype):
    """Batches of unequal prompts that go on token by token; shorter requests end earlier;
    one batch after another in a cache so small that slots and pages are used again."""
    from fms_amd.engine import Engine

    cfg, weights = plain(folders, name)
    engine = Engine(get(lib, folders, name, dtype), max_tokens=5 * 64 + 128, max_slots=4)
    rounds = [
        [(70, 3), (5, 20), (1, 9), (129, 1)],  # (prompt length, decoded tokens)
        [(33, 12), (64, 2), (100, 30)],
        [(7, 5), (190, 4), (2, 2), (20, 20)],
    ]
    seed = 100
    for requests in rounds:
        seqs = []
        for prompt_len, n_decode in requests:
            seed += 1
            ids = tokens_for(name, prompt_len + n_decode, seed)
            seqs.append(dict(ids=ids, prompt=prompt_len, slot=engine.new_sequence(), got=[], at=prompt_len))
        logits = engine.step([s["slot"] for s in seqs], [s["ids"][: s["prompt"]] for s in seqs], "all")
        row = 0
        for s in seqs:
            s["got"].append(logits[row : row + s["prompt"]])
            row += s["prompt"]
        alive = list(seqs)
        while alive:
            still = []
            for s in alive:
                if s["at"] < len(s["ids"]):
                    still.append(s)
                else:
                    engine.end_sequence(s["slot"])  # ends earlier: its slot goes back while the others go on
            alive = still
            if not alive:
                break
            logits = engine.step([s["slot"] for s in alive], [[s["ids"][s["at"]]] for s in alive], "last")
            for i, s in enumerate(alive):
                s["got"].append(logits[i : i + 1])
                s["at"] += 1
        engine.cache.check()
        assert engine.cache.live_slots() == []
        for s in seqs:
            check(torch.cat(s["got"]), P.forward(weights, cfg, s["ids"]), dtype)


@pytest.mark.parametrize("dtype", DTYPES)
def test_long_decoding(lib, folders, dtype):
    from fms_amd.engine import Engine

    name = "A"
    cfg, weights = plain(folders, name)
    engine = Engine(get(lib, folders, name, dtype), max_tokens=512 + 64, max_slots=2)
    ids = tokens_for(name, 400, 6)
    other = tokens_for(name, 30, 7)
    want = P.forward(weights, cfg, ids)
    slot, slot2 = engine.new_sequence(), engine.new_sequence()
    got = [engine.step([slot, slot2], [ids[:3], other[:10]], [[0, 1, 2], []])]
    for i in range(3, 400):
        if i < 23:  # a second sequence keeps the first company for a while, then ends
            got.append(engine.step([slot2, slot], [[other[7 + i]], [ids[i]]], [[], [0]]))
            if i == 22:
                engine.end_sequence(slot2)
        else:
            got.append(engine.step([slot], [[ids[i]]], "last"))
    engine.end_sequence(slot)
    check(torch.cat(got), want, dtype)


@pytest.mark.parametrize("dtype", DTYPES)
def test_far_key_decides(lib, folders, dtype, tmp_path):
    """Weights made so that attention is sharp: the logits depend on single far keys, so a key
    lost at a page border, a split or a slot shows as a large error instead of hiding in an average.

    Sharp attention also amplifies rounding.  For bfloat16 the bound is therefore taken from the
    plain implementation itself: the error that bfloat16 storage alone causes there."""
    from fms_amd.engine import Engine
    from fms_amd.weights import write_safetensors

    kw = dict(CONFIGS["A"], max_expected_seq_len=1024)
    folder = str(tmp_path / "sharp")
    lib.write_model_folder(folder, lib.LLaMAConfig(**kw), seed=5, std=0.08, norm_std=0.2)
    # scale the query and key projections up: scores spread over tens of units
    sharpness = 6 if dtype == "float32" else 3
    tensors = P.read_safetensors(os.path.join(folder, "model.safetensors"))
    for k in list(tensors):
        if "q_proj" in k or "k_proj" in k:
            tensors[k] = (tensors[k].float() * sharpness).to(torch.bfloat16)
    write_safetensors(os.path.join(folder, "model.safetensors"), [(k, tuple(v.shape), v.dtype) for k, v in tensors.items()],
                      lambda name: tensors[name])
    cfg, weights = P.load_model_folder(folder)
    model = lib.get_model("hf_pretrained", model_path=folder, data_type=dtype)
    engine = Engine(model, max_tokens=1024, max_slots=1)
    ids = tokens_for("A", 700, 8)
    want = P.forward(weights, cfg, ids)
    slot = engine.new_sequence()
    got = [engine.step([slot], [ids[:600]], "all")]
    for tok in ids[600:]:
        got.append(engine.step([slot], [[tok]], "last"))
    engine.end_sequence(slot)
    got = torch.cat(got).float().cpu()
    if dtype == "float32":
        check(got, want, dtype)
    else:
        storage_error = float((P.forward(weights, cfg, ids, storage=torch.bfloat16) - want).abs().max())
        scale = float(want.abs().max())
        assert 0.02 * scale < storage_error < 0.15 * scale  # sharp enough to matter, not so sharp that bfloat16 means nothing
        err = float((got - want).abs().max())
        assert err <= 1.5 * storage_error + 0.01 * scale, f"error {err:.3g}; bfloat16 storage alone gives {storage_error:.3g}"


# --------------------------------------------------------------------------
@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_greedy_generation_through_the_entry_point(lib, folders, name):
    from fms_amd.generation import generate

    cfg, weights = plain(folders, name)
    model = get(lib, folders, name, "float32")
    prompts = [tokens_for(name, n, 20 + n) for n in (5, 11, 17)]
    want = [P.greedy_generate(weights, cfg, p, 16) for p in prompts]
    for p, w in zip(prompts, want):
        out = generate(model, torch.tensor(p), max_new_tokens=16, do_sample=False)
        assert out.tolist() == p + w
    # the same prompts as a padded batch, the way the reference's script passes them
    from fms_amd.generation import pad_input_ids

    ids, extra = pad_input_ids([torch.tensor(p) for p in prompts], min_pad_length=20)
    out = generate(model, ids, max_new_tokens=16, do_sample=False, extra_kwargs=extra)
    for b, (p, w) in enumerate(zip(prompts, want)):
        assert out[b].tolist()[-16:] == w
        assert out[b].tolist()[20 - len(p) : 20] == p
    # the reference's hook before every step: it sees what is about to be fed (rows padded on the left) and may
    # change it; here it puts the second prompt in the first one's place at step 0 and leaves the rest alone
    calls = []

    def swap_first_prompt(i, input_ids, kwargs):
        calls.append((i, tuple(input_ids.shape), kwargs.get("note")))
        if i == 0:
            input_ids = input_ids.clone()
            input_ids[0, -len(prompts[0]) :] = torch.tensor(prompts[1][-len(prompts[0]) :])
        return input_ids, kwargs

    out = generate(model, torch.tensor(prompts[0]), max_new_tokens=4, do_sample=False, prepare_model_inputs_hook=swap_first_prompt,
                   extra_kwargs={"note": "kept"})
    assert out.tolist()[len(prompts[0]) :] == P.greedy_generate(weights, cfg, prompts[1][-len(prompts[0]) :], 4)
    assert calls[0] == (0, (1, len(prompts[0])), "kept") and calls[1] == (1, (1, 1), "kept") and len(calls) == 4
    # a stop token ends its own request only
    stop = want[1][3]
    out = generate(model, ids, max_new_tokens=16, do_sample=False, extra_kwargs=extra, eos_token_id=stop)
    for b, w in enumerate(want):
        row = out[b].tolist()[20:]
        cut = w.index(stop) + 1 if stop in w else len(w)
        assert row[:cut] == w[:cut]
        assert all(t == stop for t in row[cut:])


def test_bfloat16_generation_follows_the_plain_one(lib, folders):
    from fms_amd.generation import generate_requests
    from fms_amd.engine import Engine

    name = "A"
    cfg, weights = plain(folders, name)
    engine = Engine(get(lib, folders, name, "bfloat16"), max_tokens=1024, max_slots=8)
    prompts = [tokens_for(name, n, 40 + n) for n in (3, 30, 64, 65)]
    got = generate_requests(engine, prompts, max_new_tokens=12)
    for p, g in zip(prompts, got):
        ids = list(p)
        for tok in g:
            logits = P.forward(weights, cfg, ids)[-1]
            top = torch.topk(logits, 2).values
            # where the plain logits separate the best token clearly, bfloat16 must pick it
            if float(top[0] - top[1]) > 0.05 * float(logits.abs().max()):
                assert tok == int(logits.argmax())
            ids.append(tok)
    engine.cache.check()


def test_sampled_generation_is_batch_invariant(lib, folders):
    """Temperature sampling with a seed: a request draws the same tokens alone and in a batch,
    and every drawn token lies in the plain implementation's kept set."""
    from fms_amd.generation import generate_requests
    from fms_amd.engine import Engine
    from fms_amd.sampling import SamplingParams

    name = "B"
    cfg, weights = plain(folders, name)
    engine = Engine(get(lib, folders, name, "float32"), max_tokens=1024, max_slots=8)
    prompts = [tokens_for(name, n, 60 + n) for n in (1, 7, 30, 64)]
    params = SamplingParams(do_sample=True, temperature=0.8, top_k=10)
    together = generate_requests(engine, prompts, max_new_tokens=24, sampling=params, seed=3)
    again = generate_requests(engine, prompts, max_new_tokens=24, sampling=params, seed=3)
    assert together == again
    other_seed = generate_requests(engine, prompts, max_new_tokens=24, sampling=params, seed=4)
    assert together != other_seed
    for p, g in zip(prompts[:2], together[:2]):
        ids = list(p)
        for tok in g:
            dist = P.sampling_distribution(P.forward(weights, cfg, ids)[-1], 0.8, 10)
            assert dist[tok] > 0
            ids.append(tok)
    # one batch after another (batches of two) gives what one batch of four gives
    halves = generate_requests(engine, prompts, max_new_tokens=24, sampling=params, seed=3, max_batch=2)
    assert halves == together


@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_decode_products_that_fuse_the_norms_change_only_rounding(lib, folders, name, monkeypatch):
    """In bfloat16 decode steps the last product of a branch adds to the stream and prepares the next
    norm's input.  The same steps with every norm as a kernel of its own give the same logits up to
    rounding, and both follow the plain implementation."""
    from fms_amd.engine import Engine
    from fms_amd.kernels import ops
    from fms_amd.parts import ResidualStream

    calls = []
    real = ops.linear_into_stream
    monkeypatch.setattr(ops, "linear_into_stream", lambda *a, **k: (calls.append(1), real(*a, **k))[1])
    cfg, weights = plain(folders, name)
    model = get(lib, folders, name, "bfloat16")
    lens = [40, 3, 17]
    ids = [tokens_for(name, n + 6, 50 + n) for n in lens]
    results = []
    for fuse in (True, False):
        monkeypatch.setattr(ResidualStream, "fuse_products", fuse)
        engine = Engine(model, max_tokens=512, max_slots=3, use_graphs=False)
        slots = [engine.new_sequence() for _ in lens]
        engine.step(slots, [t[:n] for t, n in zip(ids, lens)], "last")
        before = len(calls)
        rows = [engine.step(slots, [[t[n + i]] for t, n in zip(ids, lens)], "last") for i in range(6)]
        assert (len(calls) > before) == fuse
        for s in slots:
            engine.end_sequence(s)
        results.append(torch.stack(rows).float().cpu())  # [6, 3, vocab]
    fused, plain_norms = results
    scale = float(plain_norms.abs().max())
    assert float((fused - plain_norms).abs().max()) <= 0.02 * scale
    for b, (t, n) in enumerate(zip(ids, lens)):
        want = P.forward(weights, cfg, t)[n:]
        check(fused[:, b], want, "bfloat16")


def graph_replay_case(lib, dtype, tmp_path, max_seq_len, prompt_lens, max_tokens):
    from fms_amd.engine import Engine
    from fms_amd.generation import generate_requests
    from fms_amd.sampling import SamplingParams

    kw = dict(CONFIGS["A"], max_expected_seq_len=max_seq_len)
    folder = str(tmp_path / "long")
    lib.write_model_folder(folder, lib.LLaMAConfig(**kw), seed=21, std=0.08, norm_std=0.2)
    model = lib.get_model("hf_pretrained", model_path=folder, data_type=dtype)
    prompts = [tokens_for("A", n, 300 + n) for n in prompt_lens]
    engines = []
    for params in (SamplingParams(do_sample=False), SamplingParams(do_sample=True, temperature=0.9, top_k=20)):
        eager = Engine(model, max_tokens=max_tokens, max_slots=3, use_graphs=False)
        graphs = Engine(model, max_tokens=max_tokens, max_slots=3, use_graphs=True)
        assert graphs.use_graphs
        want = generate_requests(eager, prompts, max_new_tokens=70, sampling=params, seed=9, stop_token_ids=[7])
        got = generate_requests(graphs, prompts, max_new_tokens=70, sampling=params, seed=9, stop_token_ids=[7])
        assert got == want  # float32 and bfloat16: equal kernels, equal order of operations: equal tokens
        captures = len(graphs.graph_captures)
        again = generate_requests(graphs, prompts, max_new_tokens=70, sampling=params, seed=9, stop_token_ids=[7])
        assert again == got
        assert len(graphs.graph_captures) == captures  # the graphs captured above are replayed, not captured anew
        graphs.cache.check()
        assert graphs.cache.live_slots() == []
        engines.append(graphs)
    return engines


@pytest.mark.parametrize("dtype", DTYPES)
def test_graph_replay_equals_eager_steps(lib, folders, dtype, tmp_path):
    """Decode through captured graphs gives the tokens of eager steps: across page borders, when the
    batch shrinks, and with the program's own eager work (prompts of later batches) between the replays."""
    graph_replay_case(lib, dtype, tmp_path, 1400, (60, 1000, 3, 64, 129), 2048)


@pytest.mark.parametrize("dtype", DTYPES)
def test_graph_for_a_longer_context_replaces_the_shorter_one(lib, folders, dtype, tmp_path):
    """The second batch of three holds a context beyond the bound (2048) of the graph captured for the first."""
    for graphs in graph_replay_case(lib, dtype, tmp_path, 4600, (60, 1000, 3, 64, 129, 2100), 4096):
        captured = graphs.graph_captures
        assert (4, 2048) in captured and (4, 4096) in captured and captured.index((4, 2048)) < captured.index((4, 4096))


# --------------------------------------------------------------------------
def run_trace(folder, dtype, steps, out_dir, max_tokens):
    proc = subprocess.Popen(
        [sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", folder, "--dtype", dtype, "--out", out_dir,
         "--max-tokens", str(max_tokens)],
        stdin=subprocess.PIPE, stdout=subprocess.PIPE, text=True, bufsize=1,
    )
    try:
        for step in steps:
            proc.stdin.write(json.dumps(step) + "\n")
            proc.stdin.flush()
            line = proc.stdout.readline().strip()
            assert line == f"done {step['step']}", f"trace_run answered {line!r}"
        proc.stdin.close()
        assert proc.wait(timeout=120) == 0
    finally:
        if proc.poll() is None:
            proc.kill()


def read_logits(out_dir, step, vocab):
    return torch.from_numpy(np.fromfile(os.path.join(out_dir, f"{step}.f32"), dtype="<f4").reshape(-1, vocab).copy())


@pytest.mark.parametrize("dtype", DTYPES)
def test_trace_replay(lib, folders, dtype, tmp_path):
    name = "A"
    cfg, weights = plain(folders, name)
    V = cfg.vocab
    reqs = {"a": tokens_for(name, 100, 71), "b": tokens_for(name, 37, 72), "c": tokens_for(name, 70, 73),
            "d": tokens_for(name, 50, 74)}
    want = {k: P.forward(weights, cfg, v) for k, v in reqs.items()}
    steps, expect = [], {}
    n = 0

    def add(entries, end=()):
        nonlocal n
        steps.append({"step": n, "entries": [{"id": i, "tokens": t, "want": w} for i, t, w in entries], "end": list(end)})
        n += 1
        return n - 1

    # 1. a whole, alone
    s = add([("a", reqs["a"], list(range(100)))], end=["a"])
    expect[s] = want["a"]
    # 2. a again: all but the last 32 whole, then one by one (no logits wanted in between for some)
    s = add([("a", reqs["a"][:68], [0, 67])])
    expect[s] = want["a"][[0, 67]]
    for i in range(68, 100):
        s = add([("a", [reqs["a"][i]], [0] if i % 2 else [])], end=["a"] if i == 99 else [])
        if i % 2:
            expect[s] = want["a"][i : i + 1]
    # 3. a batch of unequal lengths; b ends first, then d, c goes on alone; slots are used again
    prompt = {"b": 30, "c": 64, "d": 1}
    s = add([(k, reqs[k][: prompt[k]], [prompt[k] - 1]) for k in ("b", "c", "d")])
    expect[s] = torch.stack([want[k][prompt[k] - 1] for k in ("b", "c", "d")])
    at = dict(prompt)
    alive = ["b", "c", "d"]
    while alive:
        entries = [(k, [reqs[k][at[k]]], [0]) for k in alive]
        ending = [k for k in alive if at[k] + 1 == len(reqs[k])]
        s = add(entries, end=ending)
        expect[s] = torch.stack([want[k][at[k]] for k in alive])
        for k in alive:
            at[k] += 1
        alive = [k for k in alive if k not in ending]
        if len(steps) > 400:
            break
    out_dir = str(tmp_path / "out")
    run_trace(folders[name], dtype, steps, out_dir, max_tokens=64 * 5)
    for s, w in expect.items():
        check(read_logits(out_dir, s, V), w, dtype)
    written = {f for f in os.listdir(out_dir) if f.endswith(".f32")}
    assert written == {f"{s}.f32" for s in expect}
