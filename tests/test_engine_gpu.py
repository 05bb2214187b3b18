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
    # one kv head, head size 20, a width and a feed-forward width that are no multiples of 8 (60 and 50): rows that
    # are not 16-byte aligned, which the bfloat16 MFMA products cannot load
    "D": dict(src_vocab_size=260, emb_dim=60, nheads=3, kvheads=1, nlayers=2, hidden_dim=50, multiple_of=1,
              norm_eps=1e-5, rope_theta=10000.0, max_expected_seq_len=512, tie_heads=False),
    # head size 64 with grouped kv heads (the MFMA kernels' other compile-time head size), a larger vocabulary
    "E": dict(src_vocab_size=1000, emb_dim=256, nheads=4, kvheads=2, nlayers=2, hidden_dim=344, multiple_of=1,
              norm_eps=1e-5, rope_theta=500000.0, max_expected_seq_len=512, tie_heads=True),
    # head size 96 (a multiple of 16 that no kernel is specialised for), one kv head, another activation function
    "F": dict(src_vocab_size=333, emb_dim=192, nheads=2, kvheads=1, nlayers=1, hidden_dim=520, multiple_of=1,
              norm_eps=1e-6, rope_theta=10000.0, max_expected_seq_len=512, tie_heads=False, activation_fn="gelu-tanh"),
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


from gpu_checks import SHARP_MARGIN, Expected, check, expect  # noqa: E402


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
        check(logits, expect(weights, cfg, ids, dtype), dtype)
    engine.cache.check()


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_last_32_tokens_one_by_one(lib, folders, name, dtype):
    from fms_amd.engine import Engine

    cfg, weights = plain(folders, name)
    engine = Engine(get(lib, folders, name, dtype), max_tokens=256, max_slots=1)
    ids = tokens_for(name, 150, 4)
    want = expect(weights, cfg, ids, dtype)
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
    want = expect(weights, cfg, ids, dtype)
    slot = engine.new_sequence()
    got, at = [], 0
    for n in (1, 1, 1, 2, 59, 1, 63, 12):
        got.append(engine.step([slot], [ids[at : at + n]], "all"))
        at += n
    assert at == 140
    engine.end_sequence(slot)
    check(torch.cat(got), want, dtype)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["A", "B", "E"])
def test_steps_of_any_mix(lib, folders, name, dtype):
    """More than the loop above it asks of the step function: in one step some sequences bring a piece of their prompt,
    others one token, and new ones join while the rest go on; sequences end at different times and their slots are
    taken again.  A seeded random schedule; every logit is compared with the plain implementation's for the whole
    sequence."""
    import random

    from fms_amd.engine import Engine

    cfg, weights = plain(folders, name)
    engine = Engine(get(lib, folders, name, dtype), max_tokens=6 * 192, max_slots=4)
    rng = random.Random(17)
    waiting = [tokens_for(name, rng.choice((3, 40, 64, 65, 130, 180)), 300 + i) for i in range(9)]
    running = []  # [ids, slot, tokens fed so far, logits]
    finished = []
    n_mixed = 0
    while waiting or running:
        while waiting and len(running) < 4 and (not running or rng.random() < 0.5):
            running.append([waiting.pop(), engine.new_sequence(), 0, []])
        pieces = []
        for seq in running:
            left = len(seq[0]) - seq[2]
            n = min(left, rng.choice((1, 1, 1, 2, 17, 63, 64, 70)))
            pieces.append(seq[0][seq[2] : seq[2] + n])
        n_mixed += len({len(p) == 1 for p in pieces}) == 2
        logits = engine.step([seq[1] for seq in running], pieces, "all")
        row = 0
        for seq, piece in zip(running, pieces):
            seq[3].append(logits[row : row + len(piece)])
            seq[2] += len(piece)
            row += len(piece)
        assert row == logits.shape[0]
        for seq in [seq for seq in running if seq[2] == len(seq[0])]:
            engine.end_sequence(seq[1])
            running.remove(seq)
            finished.append(seq)
        engine.cache.check()
    assert engine.cache.live_slots() == [] and len(finished) == 9 and n_mixed >= 5
    for ids, _, _, got in finished:
        check(torch.cat(got), expect(weights, cfg, ids, dtype), dtype)


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
            check(torch.cat(s["got"]), expect(weights, cfg, s["ids"], dtype), dtype)


@pytest.mark.parametrize("dtype", DTYPES)
def test_long_decoding(lib, folders, dtype):
    from fms_amd.engine import Engine

    name = "A"
    cfg, weights = plain(folders, name)
    engine = Engine(get(lib, folders, name, dtype), max_tokens=512 + 64, max_slots=2)
    ids = tokens_for(name, 400, 6)
    other = tokens_for(name, 30, 7)
    want = expect(weights, cfg, ids, dtype)
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

    Sharp attention also amplifies rounding, for the reference's bfloat16 arithmetic as for the engine's: the
    bound at every position is what the reference's own roundings cost there (gpu_checks)."""
    from fms_amd.engine import Engine
    from fms_amd.weights import write_safetensors

    kw = dict(CONFIGS["A"], max_expected_seq_len=1024)
    folder = str(tmp_path / "sharp")
    lib.write_model_folder(folder, lib.LLaMAConfig(**kw), seed=5, std=0.08, norm_std=0.2)
    # scale the query and key projections up: scores spread over tens of units
    sharpness = 6
    tensors = P.read_safetensors(os.path.join(folder, "model.safetensors"))
    for k in list(tensors):
        if "q_proj" in k or "k_proj" in k:
            tensors[k] = (tensors[k].float() * sharpness).to(torch.bfloat16)
    write_safetensors(os.path.join(folder, "model.safetensors"), [(k, tuple(v.shape), v.dtype) for k, v in tensors.items()],
                      lambda name: tensors[name])
    cfg, weights = P.load_model_folder(folder)
    model = lib.get_model("hf_pretrained", model_path=folder, data_type=dtype)
    engine = Engine(model, max_tokens=1024, max_slots=1)
    engine_two = Engine(model, max_tokens=2048, max_slots=2)
    ids = tokens_for("A", 700, 8)
    want = expect(weights, cfg, ids, dtype)
    # sharp indeed: the heaviest key of a late query holds most of its weight, and it lies far back
    q, k = P.rotated_queries_and_keys(weights, cfg, ids, layer=0)
    probs = torch.softmax((q[650:, 0] @ k[:, 0].t() / 4.0).masked_fill(torch.arange(700)[None] > torch.arange(650, 700)[:, None], -1e30), -1)
    assert float(probs.max(-1).values.median()) > 0.5 and int((torch.arange(650, 700) - probs.argmax(-1)).max()) > 300
    slot = engine.new_sequence()
    got = [engine.step([slot], [ids[:600]], "all")]
    for tok in ids[600:]:
        got.append(engine.step([slot], [[tok]], "last"))
    engine.end_sequence(slot)
    check(torch.cat(got), want, dtype, margin=SHARP_MARGIN)

    # Negative controls: the same comparison has to fail when the cache loses one key, and when a step reads
    # another sequence's slot.  The key that the late queries of the first layer lean on most is taken out.
    heavy = int(torch.mode(probs.argmax(-1)).values)
    assert heavy < 600
    slot = engine.new_sequence()
    engine.step([slot], [ids[:600]], "all")
    for group in engine.cache.groups:
        page = group.pages[slot][heavy // 64]
        group.keys[:, page, :, heavy % 64, :] = 0
        group.values[:, page, :, :, heavy % 64] = 0
    lost = torch.cat([engine.step([slot], [[tok]], "last") for tok in ids[600:]])
    engine.end_sequence(slot)
    with pytest.raises(AssertionError):
        check(lost, want[600:], dtype, margin=SHARP_MARGIN)
    other = tokens_for("A", 600, 9)
    a, b = engine_two.new_sequence(), engine_two.new_sequence()
    engine_two.step([a, b], [ids[:600], other], "last")
    swapped = torch.cat([engine_two.step([b, a], [[tok], [1]], "last")[:1] for tok in ids[600:640]])
    with pytest.raises(AssertionError):
        check(swapped, want[600:640], dtype, margin=SHARP_MARGIN)
    engine.cache.check()


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
    # the reference's hook after every choice (fms/utils/generation.py:328-331): token position, the logits the
    # choice was made from [B, V], next_val [B, 1] and the kwargs; what it returns is what goes on.  Here it
    # checks what it is shown and forces the second request's third token.
    shown = []

    def force(position, logits, next_val, kwargs):
        shown.append((position, tuple(logits.shape), tuple(next_val.shape), next_val[:, 0].tolist(), kwargs.get("note")))
        assert logits.argmax(-1).tolist() == next_val[:, 0].tolist()
        if position == 20 + 2:
            next_val = next_val.clone()
            next_val[1, 0] = prompts[1][0]
        return next_val, kwargs

    hooked = generate(model, ids, max_new_tokens=5, do_sample=False, extra_kwargs=dict(extra, note="kept"), post_iteration_hook=force)
    assert [s[0] for s in shown] == [20, 21, 22, 23, 24]
    assert all(s[1] == (3, cfg.vocab) and s[2] == (3, 1) and s[4] == "kept" for s in shown)
    for b, (p, w) in enumerate(zip(prompts, want)):
        row = hooked[b].tolist()[20:]
        if b != 1:
            assert row == w[:5]
        else:
            forced = p + w[:2] + [p[0]]
            assert row[:2] == w[:2] and row[2] == p[0]
            assert row[3:] == P.greedy_generate(weights, cfg, forced, 2)
    # a stop token ends its own request only
    stop = want[1][3]
    out = generate(model, ids, max_new_tokens=16, do_sample=False, extra_kwargs=extra, eos_token_id=stop)
    for b, w in enumerate(want):
        row = out[b].tolist()[20:]
        cut = w.index(stop) + 1 if stop in w else len(w)
        assert row[:cut] == w[:cut]
        assert all(t == stop for t in row[cut:])


@pytest.mark.parametrize("name", ["A", "B"])
def test_a_call_on_token_ids_gives_the_logits_of_whole_sequences(lib, folders, name):
    """The model called the way the reference's is (fms/models/llama.py:425-450, no cache): one sequence, a padded
    batch with the kwargs of pad_input_ids, and the last n places only (headless.py:24-27)."""
    from fms_amd.generation import pad_input_ids

    cfg, weights = plain(folders, name)
    model = get(lib, folders, name, "float32")
    assert model.get_config() is model.config
    prompts = [tokens_for(name, n, 60 + n) for n in (9, 4, 13)]
    want = [P.forward(weights, cfg, p) for p in prompts]
    one = model(torch.tensor(prompts[0]))
    assert tuple(one.shape) == (9, cfg.vocab)
    torch.testing.assert_close(one.cpu(), want[0], atol=2e-4, rtol=1e-3)
    torch.testing.assert_close(model(torch.tensor(prompts[0]), last_n_tokens=2).cpu(), want[0][-2:], atol=2e-4, rtol=1e-3)
    for side in ("left", "right"):
        ids, extra = pad_input_ids([torch.tensor(p) for p in prompts], min_pad_length=15, padding_side=side)
        out = model(ids, **extra).cpu()
        assert tuple(out.shape) == (3, 15, cfg.vocab)
        for b, (p, w) in enumerate(zip(prompts, want)):
            first = 15 - len(p) if side == "left" else 0
            torch.testing.assert_close(out[b, first : first + len(p)], w, atol=2e-4, rtol=1e-3)
            rest = torch.cat((out[b, :first], out[b, first + len(p) :]))
            assert float(rest.abs().max()) == 0.0 if rest.numel() else True
        last = model(ids, last_n_tokens=3, **extra).cpu()
        assert tuple(last.shape) == (3, 3, cfg.vocab)
        for b, (p, w) in enumerate(zip(prompts, want)):
            if side == "left":
                torch.testing.assert_close(last[b], w[-3:], atol=2e-4, rtol=1e-3)
            else:  # the last three places of the padded row: real only where the row is long enough
                real = max(0, len(p) - 12)
                if real:
                    torch.testing.assert_close(last[b, :real], w[len(p) - real :], atol=2e-4, rtol=1e-3)
                assert float(last[b, real:].abs().max()) == 0.0 if real < 3 else True
    with pytest.raises(NotImplementedError):
        model(torch.tensor(prompts[0]), use_cache=True)
    assert getattr(model, "_default_engine").cache.live_slots() == []


def test_a_model_from_a_configuration_alone(lib):
    """The reference's `LLaMA(config, **kwargs)` (fms/models/llama.py:362-378): a model with random weights from a
    configuration; the same seed gives the weights that get_model gives the same variant."""
    from fms_amd.architectures import variant_config

    cfg = variant_config("llama", "micro", nlayers=2)
    ids = torch.tensor([5, 17, 3, 200, 9])
    a = lib.LLaMA(cfg, data_type="float32", random_seed=3)(ids)
    b = lib.get_model("llama", "micro", data_type="float32", random_seed=3, nlayers=2)(ids)
    c = lib.LLaMA(variant_config("llama", "micro"), nlayers=2, data_type="float32", random_seed=4)(ids)
    assert tuple(a.shape) == (5, 256) and torch.equal(a, b) and not torch.equal(a, c)
    assert lib.LLaMA(nlayers=1, emb_dim=64, nheads=2, src_vocab_size=50).get_config().nlayers == 1
    with pytest.raises(TypeError):
        lib.from_config(lib.ModelConfig())


def test_bfloat16_generation_follows_the_plain_one(lib, folders):
    from fms_amd.generation import generate_requests
    from fms_amd.engine import Engine

    name = "A"
    cfg, weights = plain(folders, name)
    engine = Engine(get(lib, folders, name, "bfloat16"), max_tokens=1024, max_slots=8)
    prompts = [tokens_for(name, n, 40 + n) for n in (3, 30, 64, 65)]
    got = generate_requests(engine, prompts, max_new_tokens=12)
    compared = total = 0
    for p, g in zip(prompts, got):
        ids = list(p)
        for tok in g:
            logits = P.forward(weights, cfg, ids)[-1]
            top = torch.topk(logits, 2).values
            total += 1
            # where the plain logits separate the best token clearly, bfloat16 must pick it
            if float(top[0] - top[1]) > 0.05 * float(logits.abs().max()):
                assert tok == int(logits.argmax())
                compared += 1
            ids.append(tok)
    assert total == 48 and compared >= total // 2, f"only {compared} of {total} tokens were compared"
    engine.cache.check()


def test_sampled_generation_is_batch_invariant(lib, folders):
    """Temperature sampling with a seed: a request draws the same tokens alone and in a batch, and they are the
    tokens that the plain implementation's sampler draws."""
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
    # every draw of every request is the plain sampler's: plain logits, plain distribution, the uniform number of
    # (request, number of tokens drawn so far), inverse CDF.  Float32 logits differ in the last digits, so a number
    # that falls within 1e-4 of an interval's edge may go either way: such draws (a handful at most) only have to
    # land on a token that was kept.
    near_edge = 0
    for r, (p, g) in enumerate(zip(prompts, together)):
        ids = list(p)
        for n, tok in enumerate(g):
            dist = P.sampling_distribution(P.forward(weights, cfg, ids)[-1], 0.8, 10)
            want, margin = P.inverse_cdf(dist, P.draw_uniform(P.seed_of_request(3, r), n))
            assert dist[tok] > 0
            if margin > 1e-4:
                assert tok == want, f"request {r}, draw {n}: {tok} drawn, the plain sampler draws {want}"
            else:
                near_edge += 1
            ids.append(tok)
    assert near_edge <= 3
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
        # rows of configuration D are not 16-byte aligned: its products never stream, so nothing is fused
        assert (len(calls) > before) == (fuse and name != "D")
        for s in slots:
            engine.end_sequence(s)
        results.append(torch.stack(rows).float().cpu())  # [6, 3, vocab]
    fused, plain_norms = results
    scale = float(plain_norms.abs().max())
    assert float((fused - plain_norms).abs().max()) <= 0.02 * scale
    for b, (t, n) in enumerate(zip(ids, lens)):
        check(fused[:, b], expect(weights, cfg, t, "bfloat16")[n:], "bfloat16")


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


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["B", "E"])
def test_logits_do_not_depend_on_the_place_in_the_cache(lib, folders, name, dtype):
    """The same sequence in a fresh cache (slot 0, pages 0, 1, 2, ...) and in one that other sequences have used
    and partly left (another slot, pages out of order that still hold the others' keys and values): the same
    kernels add the same numbers in the same order, so the logits are the same bits."""
    from fms_amd.engine import Engine

    model = get(lib, folders, name, dtype)
    ids = tokens_for(name, 300, 77)

    def run(others):
        engine = Engine(model, max_tokens=64 * 24, max_slots=8, use_graphs=False)
        held = []
        for i, n in enumerate(others):
            held.append(engine.new_sequence())
            engine.step([held[-1]], [tokens_for(name, n, 200 + i)], "last")
        for slot in held[::2]:
            engine.end_sequence(slot)
        slot = engine.new_sequence()
        out = [engine.step([slot], [ids[:200]], "all")]
        for tok in ids[200:]:
            out.append(engine.step([slot], [[tok]], "last"))
        return torch.cat(out), slot, list(engine.cache.groups[0].pages[slot])

    fresh, slot_a, pages_a = run([])
    used, slot_b, pages_b = run([100, 70, 129, 5, 64])
    assert slot_a != slot_b and pages_a != pages_b and pages_b != sorted(pages_b)
    assert torch.equal(fresh, used)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["A", "E"])
def test_replayed_and_eager_steps_choose_the_same_tokens(lib, folders, name, dtype):
    """An eager decode step has the shape of the captured step of its row bucket (padding rows, the same context
    bound), so both run the same kernels with the same launches: generation through graphs and through eager steps
    gives the same tokens, bit for bit, greedy and sampled, while sequences end at different times and the batch
    shrinks from one row bucket to the next.  Any index that a graph kept past its time would show here."""
    from fms_amd.engine import Engine
    from fms_amd.generation import generate_requests
    from fms_amd.sampling import SamplingParams

    model = get(lib, folders, name, dtype)
    lens = varied_lengths(37, 120)
    prompts = [tokens_for(name, n, 900 + i) for i, n in enumerate(lens)]
    room = sum(-(-(n + 90) // 64) * 64 for n in lens)
    stops = list(range(3, CONFIGS[name]["src_vocab_size"], 23))  # about one token in 23 ends its sequence
    got = {}
    for graphs in (True, False):
        engine = Engine(model, max_tokens=room, max_slots=len(lens), use_graphs=graphs)
        assert engine.use_graphs == graphs
        for sampling in (SamplingParams(do_sample=False), SamplingParams(do_sample=True, temperature=0.9, top_k=20)):
            got[(graphs, sampling.do_sample)] = generate_requests(engine, prompts, max_new_tokens=90, sampling=sampling, seed=5,
                                                                  stop_token_ids=stops)
            if graphs:
                # with someone watching every step the loop does not run steps ahead of the host: the same tokens
                got[("one by one", sampling.do_sample)] = generate_requests(
                    engine, prompts, max_new_tokens=90, sampling=sampling, seed=5, stop_token_ids=stops, on_step=lambda *a: None)
        engine.cache.check()
        if graphs:
            assert len(set(engine.graph_captures)) >= 3  # the batch went through several row buckets
    for sampled in (False, True):
        assert got[(True, sampled)] == got[(False, sampled)] == got[("one by one", sampled)]
        assert len(set(len(g) for g in got[(True, sampled)])) > 3  # they ended at different times


# --------------------------------------------------------------------------
def varied_lengths(n, longest):
    """n prompt lengths between 1 and `longest`, among them the neighbours of the page borders."""
    special = [63, 64, 65, 1, 127, 128, 2, 62]
    return [(special[i] if i < len(special) else 1 + (37 * i * i + 11 * i) % longest) for i in range(n)]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_decode_batches_of_many_sequences(lib, folders, name, dtype):
    """Decode steps of 20, 48, 70, 128, 140 and 200 sequences of unequal lengths (the products for 17 to 192 rows, their
    row buckets with padding rows, and the step above 192 rows), through captured graphs and as eager steps:
    both follow the plain implementation.  After three steps every third
    sequence ends and the batch goes on smaller."""
    from fms_amd.engine import Engine
    from fms_amd.sampling import SamplingParams

    cfg, weights = plain(folders, name)
    model = get(lib, folders, name, dtype)
    greedy = SamplingParams(do_sample=False)
    for n_seqs in (20, 48, 70, 128, 140, 200):
        lens = varied_lengths(n_seqs, 130)
        room = sum(-(-(n + 8) // 64) * 64 for n in lens)
        replayed = Engine(model, max_tokens=room, max_slots=n_seqs, use_graphs=True)
        eager = Engine(model, max_tokens=room, max_slots=n_seqs, use_graphs=False)
        assert replayed.use_graphs
        seqs = [dict(ids=tokens_for(name, n, 500 + 7 * n_seqs + i), n=n, got=[]) for i, n in enumerate(lens)]
        for engine, key in ((replayed, "slot_r"), (eager, "slot_e")):
            for s in seqs:
                s[key] = engine.new_sequence()
            for i in range(0, n_seqs, 16):
                group = seqs[i : i + 16]
                logits = engine.step([s[key] for s in group], [s["ids"] for s in group], "last")
                if engine is eager:
                    for s, tok in zip(group, logits.argmax(-1).tolist()):
                        s["next"] = tok
        alive = list(seqs)
        for step in range(6):
            if step == 3:
                for s in alive[::3]:
                    replayed.end_sequence(s["slot_r"])
                    eager.end_sequence(s["slot_e"])
                alive = [s for i, s in enumerate(alive) if i % 3]
            fed = [s["next"] for s in alive]
            chosen = replayed.decode_and_choose([s["slot_r"] for s in alive], fed, greedy)
            from_graph = replayed.last_graph.logits[: len(alive)].clone()
            from_steps = eager.step([s["slot_e"] for s in alive], [[t] for t in fed], "last")
            assert chosen == from_graph.argmax(-1).tolist()
            if dtype == "float32":  # the replayed step has padding rows and a rounder context bound, nothing else
                torch.testing.assert_close(from_graph, from_steps, atol=2e-4, rtol=1e-3)
            for s, tok, row_r, row_e in zip(alive, chosen, from_graph, from_steps):
                s["ids"] = s["ids"] + [s["next"]]
                s["got"].append(torch.stack((row_r, row_e)))
                s["next"] = tok
        for s in alive:
            replayed.end_sequence(s["slot_r"])
            eager.end_sequence(s["slot_e"])
        replayed.cache.check()
        eager.cache.check()
        assert replayed.cache.live_slots() == [] == eager.cache.live_slots()
        # every sequence of the two smaller batches, every fourth of the larger ones (the first eight hold the page borders)
        for i, s in enumerate(seqs):
            if n_seqs <= 48 or i < 8 or i % 4 == 0:
                want = expect(weights, cfg, s["ids"], dtype)[s["n"] :]
                got = torch.stack(s["got"])  # [steps, replayed or eager, vocab]
                check(got[:, 0], want, dtype)
                check(got[:, 1], want, dtype)


@pytest.mark.parametrize("dtype", DTYPES)
def test_a_graph_is_not_replayed_for_sequences_it_no_longer_describes(lib, folders, dtype):
    """One engine, one slot.  A request ends and the next one gets the same slot and happens to be fed the token
    that the graph chose last; or an eager step moves a sequence on between two replays and the same token is
    fed again.  Slots and tokens then look like the graph's own next step, but its positions and pages are the old
    ones: it has to be loaded anew."""
    from fms_amd.engine import Engine
    from fms_amd.sampling import SamplingParams

    name = "A"
    cfg, weights = plain(folders, name)
    model = get(lib, folders, name, dtype)
    greedy = SamplingParams(do_sample=False)
    engine = Engine(model, max_tokens=512, max_slots=1, use_graphs=True)
    first, second = tokens_for(name, 130, 901), tokens_for(name, 20, 902)
    slot = engine.new_sequence()
    engine.step([slot], [first], "last")
    a = engine.decode_and_choose([slot], [5], greedy)[0]
    b = engine.decode_and_choose([slot], [a], greedy)[0]  # the graph's own next step
    engine.end_sequence(slot)
    again = engine.new_sequence()
    assert again == slot
    engine.step([again], [second], "last")
    c = engine.decode_and_choose([again], [b], greedy)[0]  # fed what the graph chose last, but another sequence
    got = [engine.last_graph.logits[:1].clone()]
    ids = second + [b]
    # an eager step in between, then the graph's last choice once more
    got.append(engine.step([again], [[c]], "last"))
    ids.append(c)
    engine.decode_and_choose([again], [c], greedy)
    got.append(engine.last_graph.logits[:1].clone())
    ids.append(c)
    engine.end_sequence(again)
    check(torch.cat(got), expect(weights, cfg, ids, dtype)[len(second) :], dtype)


@pytest.mark.parametrize("dtype", DTYPES)
def test_a_step_that_is_refused_leaves_the_sequences_as_they_were(lib, folders, dtype):
    from fms_amd.cache import CacheFull
    from fms_amd.engine import Engine

    name = "B"
    cfg, weights = plain(folders, name)
    engine = Engine(get(lib, folders, name, dtype), max_tokens=64 * 3, max_slots=3)
    a, b = engine.new_sequence(), engine.new_sequence()
    ids_a, ids_b = tokens_for(name, 70, 911), tokens_for(name, 40, 912)
    got_a = [engine.step([a, b], [ids_a[:60], ids_b[:30]], "all")[:60]]
    free = engine.cache.groups[0].pool.n_free
    with pytest.raises(IndexError):  # a place that is not among the tokens
        engine.step([a, b], [ids_a[60:62], ids_b[30:31]], [[0], [1]])
    with pytest.raises(CacheFull):  # a needs a second page and b a second and a third one; one page is free
        engine.step([a, b], [ids_a[60:70], ids_b[30:40] + [1] * 60], "last")
    with pytest.raises(IndexError):  # beyond the model's positions
        engine.step([b, a], [[1], [2] * 500], "last")
    with pytest.raises(IndexError):  # a token the vocabulary does not have
        engine.step([a], [[cfg.vocab]], "last")
    assert (engine.length(a), engine.length(b), engine.cache.groups[0].pool.n_free) == (60, 30, free)
    got_a.append(engine.step([a, b], [ids_a[60:], ids_b[30:]], "all")[:10])
    check(torch.cat(got_a), expect(weights, cfg, ids_a, dtype), dtype)
    engine.end_sequence(a)
    engine.end_sequence(b)
    engine.cache.check()


def test_command_line(lib, folders):
    """bin/fms_inference, the reference's scripts/inference.py (:155-281): a model folder, the character tokenizer,
    prompts as token ids; one prompt, then two as a padded batch.  The printed text is the plain implementation's
    greedy continuation."""
    from fms_amd.tokenizers import CharTokenizer

    name = "A"  # its vocabulary is the character tokenizer's
    cfg, weights = plain(folders, name)
    tok = CharTokenizer()
    prompts = [[ord(c) for c in "Llama on one GPU"], [ord(c) for c in "ragged"]]
    want = [p + P.greedy_generate(weights, cfg, p, 16, stop=tok.eos_token_id) for p in prompts]

    def run(*prompt_args):
        cmd = [sys.executable, os.path.join(ROOT, "bin", "fms_inference"), "--architecture", "hf_pretrained", "--model_path",
               folders[name], "--tokenizer", "char_tokenizer", "--default_dtype", "fp32", "--max_new_tokens", "16", *prompt_args]
        env = dict(os.environ, PYTHONIOENCODING="utf-8")
        proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.PIPE, timeout=110, env=env)
        assert proc.returncode == 0, proc.stderr.decode(errors="replace")
        return proc.stdout.decode("utf-8")

    out = run("--prompt_ids", ",".join(map(str, prompts[0])))
    assert "loading complete" in out and tok.decode(want[0]) in out
    out = run("--prompt_ids", ",".join(map(str, prompts[0])), "--prompt_ids", ",".join(map(str, prompts[1])))
    first, second = tok.decode(want[0]), tok.decode(want[1])
    assert first in out and second in out and out.index(first) < out.index(second)
    # a text prompt gets the tokenizer's begin-of-text token in front, which is not printed
    text = "Hi there"
    ids = [tok.bos_token_id] + tok.encode(text)
    out = run("--prompt", text)
    assert tok.decode((ids + P.greedy_generate(weights, cfg, ids, 16, stop=tok.eos_token_id))[1:]) in out


def test_chat_command(lib, folders):
    """bin/fms_chat, the reference's scripts/chat.py (:196-243): two questions on piped input.  With --deterministic the
    answers are the plain implementation's greedy continuations of the conversation in the Llama layout, the second
    one with the first question and its answer in front."""
    from fms_amd.tokenizers import CharTokenizer

    name = "A"  # its vocabulary is the character tokenizer's
    cfg, weights = plain(folders, name)
    tok = CharTokenizer()
    bos, eos = tok.bos_token_id, tok.eos_token_id

    def plain_answer(ids):
        new = P.greedy_generate(weights, cfg, ids, 12, stop=eos)
        return new[:new.index(eos)] if eos in new else new

    ids = [bos] + tok.encode("<<SYS>>\nshort\n<</SYS>>\n\n") + tok.encode("[INST]one[/INST]")
    first = plain_answer(ids)
    ids += first + [eos] + tok.encode("[INST]two[/INST]")
    second = plain_answer(ids)

    cmd = [sys.executable, os.path.join(ROOT, "bin", "fms_chat"), "--architecture", "hf_pretrained", "--model_path", folders[name],
           "--tokenizer", "char_tokenizer", "--default_dtype", "fp32", "--max_new_tokens", "12", "--deterministic",
           "--system_message", "short"]
    env = dict(os.environ, PYTHONIOENCODING="utf-8")
    proc = subprocess.run(cmd, input="one\ntwo\n/buffer\n".encode(), stdout=subprocess.PIPE, stderr=subprocess.PIPE, timeout=110, env=env)
    assert proc.returncode == 0, proc.stderr.decode(errors="replace")
    out = proc.stdout.decode("utf-8")
    assert "loading complete" in out and out.rstrip().endswith("Exiting...")
    assert tok.decode(first) in out and tok.decode(second) in out
    assert f"The conversation has {len(ids) + len(second) + 1} tokens:" in out


def test_a_type_asked_for_casts_a_checkpoint_stored_in_32_bit(lib, tmp_path):
    """tests/models/test_getmodel_datatype.py:58-73: data_type wins over the checkpoint's type.  The bfloat16
    model made from a float32 folder runs the bfloat16 kernels and follows the plain implementation."""
    from fms_amd.engine import Engine

    name = "A"
    folder = str(tmp_path / "stored32")
    lib.write_model_folder(folder, lib.LLaMAConfig(**CONFIGS[name]), seed=31, std=0.08, norm_std=0.2, data_type="float32")
    cfg, weights = P.load_model_folder(folder)
    assert all(t.dtype == torch.float32 for t in P.read_safetensors(os.path.join(folder, "model.safetensors")).values())
    model = lib.get_model("hf_pretrained", model_path=folder, data_type="bf16")
    assert model.dtype == torch.bfloat16
    assert model.layers[0].mixer.qkv.w["weight"].dtype == torch.bfloat16 and model.head.w["weight"].dtype == torch.bfloat16
    assert model.layers[0].mixer.dense.streams(4, torch.bfloat16)
    assert model.final_norm.w["weight"].dtype == torch.float32  # a norm's scale stays as it is stored
    assert lib.get_model("hf_pretrained", model_path=folder).dtype == torch.float32  # no type asked for: the checkpoint's
    weights16 = {k: v.bfloat16().float() if v.dim() > 1 else v for k, v in weights.items()}
    engine = Engine(model, max_tokens=256, max_slots=1)
    ids = tokens_for(name, 90, 33)
    slot = engine.new_sequence()
    got = [engine.step([slot], [ids[:80]], "all")] + [engine.step([slot], [[t]], "last") for t in ids[80:]]
    check(torch.cat(got), expect(weights16, cfg, ids, "bfloat16"), "bfloat16")


@pytest.mark.parametrize("dtype", DTYPES)
def test_ntk_scaling(lib, dtype, tmp_path):
    """fms/modules/positions.py:135-168, 311-355: the rotation's base grows with the longest sequence of a call.  Up
    to max_expected_seq_len the model is the regular one (tests/modules/test_positions.py:216-241); a longer prompt
    in one step is rotated with the stretched base throughout, like the reference's call with that prompt; steps
    run eagerly, because a captured step would keep the table it was captured with."""
    from fms_amd.engine import Engine
    from fms_amd.sampling import SamplingParams

    kw = dict(CONFIGS["A"], max_expected_seq_len=64, rope_scaling={"rope_type": "ntk", "factor": 4.0})
    folder = str(tmp_path / "ntk")
    lib.write_model_folder(folder, lib.LLaMAConfig(**kw), seed=51, std=0.08, norm_std=0.2)
    cfg, weights = P.load_model_folder(folder)
    assert cfg.rope_scaling["rope_type"] == "ntk" and cfg.max_len == 64
    model = lib.get_model("hf_pretrained", model_path=folder, data_type=dtype)
    engine = Engine(model, max_tokens=512, max_slots=2)
    assert not engine.use_graphs and engine.cache.max_seq_len == 256
    regular = P.PlainConfig(**{**cfg.__dict__, "rope_scaling": {}})
    short, long_one = tokens_for("A", 64, 52), tokens_for("A", 150, 53)
    a, b = engine.new_sequence(), engine.new_sequence()
    got = engine.step([a], [short[:40]], "all")
    got = torch.cat([got] + [engine.step([a], [[t]], "last") for t in short[40:]])
    check(got, expect(weights, regular, short, dtype), dtype)  # alpha 1: the regular rotation
    check(engine.step([b], [long_one], "all"), expect(weights, cfg, long_one, dtype), dtype)  # alpha 4 throughout
    assert float((P.forward(weights, cfg, long_one) - P.forward(weights, P.PlainConfig(**{**cfg.__dict__, "max_len": 256, "rope_scaling": {}}), long_one)).abs().max()) > 0.05
    # decoding goes on across the borders where alpha changes (64, 128), eagerly, up to the last position
    tokens = engine.decode_and_choose([a, b], [1, 2], SamplingParams(do_sample=False))
    assert len(tokens) == 2 and engine.length(a) == 65
    engine.end_sequence(a)
    for _ in range(256 - 151):
        tokens = engine.decode_and_choose([b], tokens[-1:], SamplingParams(do_sample=False))
    assert engine.length(b) == 256
    with pytest.raises(IndexError):
        engine.step([b], [[1]], "last")
    engine.end_sequence(b)
    # a sequence that crosses both borders one token at a time: every step rotates its token with the alpha of its
    # own length, and the keys in the cache keep the rotation of the step that wrote them (positions.py:394-421)
    crossing = tokens_for("A", 140, 54)
    c = engine.new_sequence()
    got = [engine.step([c], [crossing[:60]], "all")] + [engine.step([c], [[t]], "last") for t in crossing[60:]]
    calls = [(60, 60)] + [(1, n) for n in range(61, 141)]
    check(torch.cat(got), expect(weights, cfg, crossing, dtype, calls=calls), dtype)
    # and the same fed whole is another function: the plain forward tells the two apart by far more than the tolerance
    assert float((P.forward(weights, cfg, crossing, calls=calls) - P.forward(weights, cfg, crossing))[60:].abs().max()) > 0.05


@pytest.mark.parametrize("name", ["A", "C"])
def test_a_meta_checkpoint_runs(lib, folders, name, tmp_path):
    """fms/models/llama.py:618-645: Meta's tensor names (w1 is the gate, w3 the up projection, adjacent rotary
    pairs as in the model, so no rows move), read with source="meta" and run, not only renamed."""
    from fms_amd.engine import Engine
    from fms_amd.weights import write_safetensors

    cfg, weights = plain(folders, name)
    H, K, D, F = cfg.nheads, cfg.kvheads, cfg.head_dim, cfg.hidden
    meta = {"tok_embeddings.weight": weights["base_model.embedding.weight"], "norm.weight": weights["base_model.dec_norm.weight"],
            "output.weight": weights["head.weight"]}
    for i in range(cfg.nlayers):
        p, m = f"base_model.layers.{i}.", f"layers.{i}."
        for kind in ("weight", "bias"):
            if p + "attn.in_proj.qkv_fused." + kind not in weights:
                continue
            q, k, v = torch.split(weights[p + "attn.in_proj.qkv_fused." + kind], [H * D, K * D, K * D])
            gate, up = torch.split(weights[p + "ff_sub_layer.wg1_fused." + kind], [F, F])
            meta.update({m + "attention.wq." + kind: q, m + "attention.wk." + kind: k, m + "attention.wv." + kind: v,
                         m + "attention.wo." + kind: weights[p + "attn.dense." + kind],
                         m + "feed_forward.w1." + kind: gate, m + "feed_forward.w3." + kind: up,
                         m + "feed_forward.w2." + kind: weights[p + "ff_sub_layer.w2." + kind]})
        meta[m + "attention_norm.weight"] = weights[p + "ln.weight"]
        meta[m + "ffn_norm.weight"] = weights[p + "ff_ln.weight"]
    meta = {k: v.contiguous() for k, v in meta.items()}
    folder = tmp_path / "meta"
    folder.mkdir()
    write_safetensors(str(folder / "consolidated.00.safetensors"), [(k, tuple(v.shape), v.dtype) for k, v in meta.items()],
                      lambda n: meta[n])
    model = lib.get_model("llama", "micro", model_path=str(folder), source="meta", data_type="fp32", **CONFIGS[name])
    engine = Engine(model, max_tokens=128, max_slots=1)
    ids = tokens_for(name, 70, 41)
    slot = engine.new_sequence()
    check(engine.step([slot], [ids], "all"), expect(weights, cfg, ids, "float32"), "float32")


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


@pytest.mark.parametrize("name", ["A", "B"])
@pytest.mark.parametrize("dtype", DTYPES)
def test_trace_replay(lib, folders, dtype, name, tmp_path):
    cfg, weights = plain(folders, name)
    V = cfg.vocab
    reqs = {"a": tokens_for(name, 100, 71), "b": tokens_for(name, 37, 72), "c": tokens_for(name, 70, 73),
            "d": tokens_for(name, 50, 74)}
    want = {k: expect(weights, cfg, v, dtype) for k, v in reqs.items()}
    steps, expected = [], {}
    n = 0

    def add(entries, end=()):
        nonlocal n
        steps.append({"step": n, "entries": [{"id": i, "tokens": t, "want": w} for i, t, w in entries], "end": list(end)})
        n += 1
        return n - 1

    # 1. a whole, alone
    s = add([("a", reqs["a"], list(range(100)))], end=["a"])
    expected[s] = want["a"]
    # 2. a again: all but the last 32 whole, then one by one (no logits wanted in between for some)
    s = add([("a", reqs["a"][:68], [0, 67])])
    expected[s] = want["a"][[0, 67]]
    for i in range(68, 100):
        s = add([("a", [reqs["a"][i]], [0] if i % 2 else [])], end=["a"] if i == 99 else [])
        if i % 2:
            expected[s] = want["a"][i : i + 1]
    # 3. a batch of unequal lengths; b ends first, then d, c goes on alone; slots are used again
    prompt = {"b": 30, "c": 64, "d": 1}
    s = add([(k, reqs[k][: prompt[k]], [prompt[k] - 1]) for k in ("b", "c", "d")])
    expected[s] = Expected.stack([want[k][prompt[k] - 1] for k in ("b", "c", "d")])
    at = dict(prompt)
    alive = ["b", "c", "d"]
    while alive:
        entries = [(k, [reqs[k][at[k]]], [0]) for k in alive]
        ending = [k for k in alive if at[k] + 1 == len(reqs[k])]
        s = add(entries, end=ending)
        expected[s] = Expected.stack([want[k][at[k]] for k in alive])
        for k in alive:
            at[k] += 1
        alive = [k for k in alive if k not in ending]
        if len(steps) > 400:
            break
    out_dir = str(tmp_path / "out")
    run_trace(folders[name], dtype, steps, out_dir, max_tokens=64 * 5)
    for s, w in expected.items():
        check(read_logits(out_dir, s, V), w, dtype)
    written = {f for f in os.listdir(out_dir) if f.endswith(".f32")}
    assert written == {f"{s}.f32" for s in expected}
