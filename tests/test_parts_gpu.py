"""Each part alone against its plain formula, and parts the library has never heard of:
a toy mixer with state of its own, defined here, registered, built into a model through the
ordinary registries and stepped by the ordinary engine, without touching the library's files."""

import dataclasses
import math

import pytest
import torch

pytestmark = pytest.mark.gpu

import plain_llama as P  # noqa: E402


@pytest.fixture(scope="module")
def lib():
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    import fms_amd
    from fms_amd.kernels import load

    load()
    return fms_amd


DEV = "cuda"


def bind_random(part, dtype, seed=0, std=0.2):
    """Random tensors for every declared parameter of a part; returns them as float32 CPU tensors by name."""
    g = torch.Generator().manual_seed(seed)
    values = {}
    for name, spec, owner, local in part.named_specs():
        t = torch.randn(spec.shape, generator=g) * std
        if spec.init == "ones":
            t = t + 1
        t = t.to(dtype)
        owner.bind(local, t.to(DEV))
        values[name] = t.float()
    for p in part.walk():
        p.finalize(torch.device(DEV), dtype)
    return values


def tol(dtype):
    return dict(atol=1e-4, rtol=1e-4) if dtype == torch.float32 else dict(atol=3e-2, rtol=3e-2)


def close(got, want, dtype):
    """float32: element by element; bfloat16: within 3 % of the largest value."""
    if dtype == torch.float32:
        torch.testing.assert_close(got, want, atol=1e-4, rtol=1e-4)
    else:
        err, scale = float((got - want).abs().max()), float(want.abs().max())
        assert err <= 0.03 * scale, f"differs by {err:.4g} at a scale of {scale:.4g}"


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_norm_part(lib, dtype):
    from fms_amd.parts import make_part

    norm = make_part("norm", "rmsnorm", width=72, eps=1e-3)
    w = bind_random(norm, dtype)
    x = torch.randn(6, 72)
    branch = torch.randn(6, 72).to(dtype)
    resid = x.clone().to(DEV)
    out = norm.add_norm(resid, branch.to(DEV), dtype)
    torch.testing.assert_close(resid.cpu(), x + branch.float())
    torch.testing.assert_close(out.cpu().float(), P.rms_norm(x + branch.float(), w["weight"], 1e-3), **tol(dtype))


def test_rotary_part(lib):
    from fms_amd.parts import make_part

    scaling = {"rope_type": "llama3", "factor": 8.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0,
               "original_max_position_embeddings": 64}
    rope = make_part("position", "rope", dim=48, theta=50000.0, max_seq_len=300, scaling=scaling)
    rope.finalize(torch.device(DEV), torch.float32)
    cos, sin, rot = rope.rotary_tables()
    assert rot == 48 and cos.shape == (300, 24)
    freqs = P.rope_frequencies(48, 50000.0, scaling)
    angles = torch.outer(torch.arange(300).float(), freqs)
    torch.testing.assert_close(cos.cpu(), torch.cos(angles), atol=2e-6, rtol=0)
    torch.testing.assert_close(sin.cpu(), torch.sin(angles), atol=2e-6, rtol=0)
    rope.check_positions(299)
    with pytest.raises(IndexError):  # tests/modules/test_positions.py:156-168
        rope.check_positions(300)
    half = make_part("position", "rope", dim=32, theta=1e4, max_seq_len=16, partial_rope=0.5)
    assert half.rot_dim == 16


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("rows,activation", [(3, "swish"), (100, "swish"), (3, "gelu"), (40, "gelu-tanh"), (100, "mish"), (9, "relu"),
                                             (20, "sigmoid"), (100, "tanh"), (3, "GELU_pytorch_tanh")])
def test_feed_forward_part(lib, dtype, rows, activation):
    """Every activation function the reference knows by name (fms/utils/activation.py:14-24), at row counts that
    take the products for few rows (gate and activation inside the product) and the separate activation kernel."""
    from fms_amd.parts import make_part

    ff = make_part("feed_forward", "glu", width=40, hidden_dim=72, activation=activation, use_bias=True)
    w = bind_random(ff, dtype, seed=1)
    x = torch.randn(rows, 40).to(dtype)
    out = ff.forward(x.to(DEV)).cpu().float()
    want = P.gated_feed_forward(x.float(), w["wg1_fused.weight"], w["w2.weight"], w["wg1_fused.bias"], w["w2.bias"],
                                act_name=activation)
    torch.testing.assert_close(out, want, **(dict(atol=1e-4, rtol=1e-4) if dtype == torch.float32 else dict(atol=0.1, rtol=5e-2)))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,K,D", [(4, 2, 16), (3, 1, 32)])
def test_attention_part_prefill_then_decode(lib, dtype, H, K, D):
    from fms_amd.cache import KVNeed, SequenceCache
    from fms_amd.engine.batch import build_batch
    from fms_amd.kernels import ops
    from fms_amd.parts import LayerCache, make_part

    width = H * D  # the plain block takes the head size as width / heads
    rope = make_part("position", "rope", dim=D, theta=1e4, max_seq_len=512)
    attn = make_part("mixer", "attention", width=width, nheads=H, kvheads=K, head_dim=D, use_bias=True, position_encoder=rope)
    w = bind_random(attn, dtype, seed=2, std=0.1)
    rope.finalize(torch.device(DEV), dtype)
    assert attn.kv_need() == KVNeed(K, D, 0) and attn.state_need() is None
    cache = SequenceCache([(0, attn.kv_need())], [], max_tokens=1024, max_slots=3, max_seq_len=512, dtype=dtype, device=DEV)
    lens = [70, 5]
    xs = [torch.randn(n + 3, width).to(dtype) for n in lens]
    slots = [cache.alloc_slot() for _ in lens]
    cfg = P.PlainConfig(vocab=1, width=width, nheads=H, kvheads=K, nlayers=1, hidden=1, eps=0, theta=1e4, max_len=512)
    freqs = P.rope_frequencies(D, 1e4)
    want = [P.attention_block(x.float(), torch.arange(x.shape[0]), cfg, w["in_proj.qkv_fused.weight"], w["dense.weight"],
                              freqs, w["in_proj.qkv_fused.bias"], w["dense.bias"]) for x in xs]
    group, keys, values = cache.kv_of_entry(0)
    view = LayerCache(group, keys, values, True, {})
    # prompts in one step
    starts = [cache.extend(s, n) for s, n in zip(slots, lens)]
    batch = build_batch(cache, slots, [[0] * n for n in lens], starts, [[] for _ in lens], DEV, [attn.prefill_qblock(sum(lens), dtype)])
    out = attn.forward(torch.cat([x[:n] for x, n in zip(xs, lens)]).to(DEV), batch, view).cpu().float()
    close(out, torch.cat([wt[:n] for wt, n in zip(want, lens)]), dtype)
    # three more tokens each, one at a time
    for i in range(3):
        starts = [cache.extend(s, 1) for s in slots]
        batch = build_batch(cache, slots, [[0], [0]], starts, [[], []], DEV)
        out = attn.forward(torch.stack([x[n + i] for x, n in zip(xs, lens)]).to(DEV), batch, view).cpu().float()
        close(out, torch.stack([wt[n + i] for wt, n in zip(want, lens)]), dtype)


# --------------------------------------------------------------------------
# parts the library does not have
# --------------------------------------------------------------------------
def test_a_toy_mixer_with_state_of_its_own(lib):
    """A mixer that keeps a running sum per sequence (state of fixed size, no keys or values):
    y_t = W * mean(x_0..x_t).  It is registered here, chosen by a configuration for some layers of a
    model whose other layers are attention, built by get_model, stepped by Engine in ragged batches
    with slots that are used again, and compared with a plain computation."""
    import fms_amd
    from fms_amd.architectures import Architecture, register_architecture, register_model
    from fms_amd.cache import StateNeed
    from fms_amd.config import ModelConfig
    from fms_amd.engine import Engine
    from fms_amd.parts import LayerSpec, Mixer, ModelSpec, PartSpec, ScheduleEntry, register_part, unregister_part

    class RunningMean(Mixer):
        graph_safe = False  # loops over sequences on the host

        def __init__(self, width, position_encoder=None):
            super().__init__()
            self.width = width
            self.declare("proj.weight", (width, width))

        def state_need(self):
            return StateNeed((("sum", (self.width,), "float32"), ("count", (1,), "float32")))

        def forward(self, x, batch, cache):
            total, count = cache.state["sum"], cache.state["count"]
            out = torch.empty_like(x)
            at = 0
            for slot, n in zip(batch.slots, batch.q_lens):
                xs = x[at : at + n].float()
                sums = torch.cumsum(xs, 0) + total[slot]
                counts = count[slot] + torch.arange(1, n + 1, device=x.device, dtype=torch.float32)
                out[at : at + n] = ((sums / counts[:, None]) @ self.w["proj.weight"].float().t()).to(x.dtype)
                total[slot] = sums[-1]
                count[slot] += n
                at += n
            return out

    @dataclasses.dataclass
    class ToyConfig(ModelConfig):
        vocab: int = 90
        width: int = 48
        hidden: int = 64
        max_len: int = 256

    def toy_spec(c: ToyConfig) -> ModelSpec:
        norm = PartSpec("rmsnorm", {"eps": 1e-5})
        ff = PartSpec("glu", {"hidden_dim": c.hidden, "activation": "swish"})
        mean_layer = LayerSpec(mixer=PartSpec("running_mean"), feed_forward=ff, norm=norm)
        attn_layer = LayerSpec(mixer=PartSpec("attention", {"nheads": 3, "kvheads": 1, "head_dim": 16}), feed_forward=ff,
                               norm=norm, position="rope")
        return ModelSpec(vocab=c.vocab, width=c.width, max_seq_len=c.max_len, layers=[mean_layer, attn_layer],
                         final_norm=norm, positions={"rope": PartSpec("rope", {"dim": 16, "theta": 1e4, "max_seq_len": c.max_len})},
                         # layer 0 runs twice (two states of its own), layer 1 in between
                         schedule=[ScheduleEntry(0), ScheduleEntry(1), ScheduleEntry(0)])

    register_part("mixer", "running_mean", RunningMean)
    try:
        try:
            register_architecture(Architecture("toy_running_mean", ToyConfig, toy_spec))
            register_model("toy_running_mean", "tiny", lambda **kw: ToyConfig().updated(**kw))
        except KeyError:
            pass  # a second run in one process
        model = fms_amd.get_model("toy_running_mean", "tiny", data_type="float32", random_seed=3)
        kv, state = model.cache_needs()
        assert [e for e, _ in kv] == [1] and [e for e, _ in state] == [0, 2]
        engine = Engine(model, max_tokens=512, max_slots=2)
        assert not engine.use_graphs  # the toy part cannot be captured, so steps run eagerly

        w = {name: owner.w[local].float().cpu() for name, _, owner, local in model.named_specs()}

        def plain(ids):
            x = w["base_model.embedding.weight"][torch.tensor(ids)]
            pos = torch.arange(len(ids))
            cfg = P.PlainConfig(vocab=90, width=48, nheads=3, kvheads=1, nlayers=2, hidden=64, eps=1e-5, theta=1e4, max_len=256)
            for layer in (0, 1, 0):
                p = f"base_model.layers.{layer}."
                h = P.rms_norm(x, w[p + "ln.weight"], 1e-5)
                if layer == 0:
                    mean = torch.cumsum(h, 0) / torch.arange(1, len(ids) + 1)[:, None]
                    h = mean @ w[p + "attn.proj.weight"].t()
                else:
                    h = P.attention_block(h, pos, cfg, w[p + "attn.in_proj.qkv_fused.weight"], w[p + "attn.dense.weight"],
                                          P.rope_frequencies(16, 1e4))
                x = x + h
                h = P.rms_norm(x, w[p + "ff_ln.weight"], 1e-5)
                x = x + P.gated_feed_forward(h, w[p + "ff_sub_layer.wg1_fused.weight"], w[p + "ff_sub_layer.w2.weight"])
            return P.rms_norm(x, w["base_model.dec_norm.weight"], 1e-5) @ w["head.weight"].t()

        g = torch.Generator().manual_seed(1)
        for round_ in range(2):  # the second round uses the slots again: their state must start at zero
            seqs = [torch.randint(0, 90, (n,), generator=g).tolist() for n in (30, 9)]
            slots = [engine.new_sequence() for _ in seqs]
            got = [[], []]
            logits = engine.step(slots, [s[:-4] for s in seqs], "all")
            got[0].append(logits[: len(seqs[0]) - 4])
            got[1].append(logits[len(seqs[0]) - 4 :])
            for i in range(4, 0, -1):
                logits = engine.step(slots, [[s[-i]] for s in seqs], "last")
                got[0].append(logits[0:1])
                got[1].append(logits[1:2])
            for s in slots:
                engine.end_sequence(s)
            for ids, rows in zip(seqs, got):
                torch.testing.assert_close(torch.cat(rows).cpu(), plain(ids), atol=2e-4, rtol=1e-3)
        engine.cache.check()
    finally:
        unregister_part("mixer", "running_mean")


def test_a_toy_mixer_whose_state_is_updated_on_the_device_under_capture(lib):
    """The same running mean, with its state updated by device code that a graph can hold: the decode step finds each
    row's state through the step's device-side index data (sequence of the row, slot of the sequence), padding rows add
    nothing, and nothing is decided on the host.  The engine then replays decode steps as captured graphs; they give
    what eager steps give and what the plain computation gives, over a batch that shrinks and slots that are reused."""
    from fms_amd.cache import StateNeed
    from fms_amd.engine import Engine
    from fms_amd.engine.model import DecoderModel
    from fms_amd.parts import LayerSpec, Mixer, ModelSpec, PartSpec, register_part, unregister_part
    from fms_amd.sampling import SamplingParams
    from fms_amd.weights import init_random

    class RunningMeanOnDevice(Mixer):
        def __init__(self, width, position_encoder=None):
            super().__init__()
            self.width = width
            self.declare("proj.weight", (width, width))

        def state_need(self):
            return StateNeed((("sum", (self.width,), "float32"), ("count", (1,), "float32")))

        def forward(self, x, batch, cache):
            total, count = cache.state["sum"], cache.state["count"]
            weight = self.w["proj.weight"].float()
            if batch.is_decode:  # one row a sequence: index operations only, all on the device
                live = batch.seq_of_token >= 0
                slots = batch.slot_ids.long()[batch.seq_of_token.clamp(min=0).long()]
                total.index_add_(0, slots, x.float() * live[:, None])
                count.index_add_(0, slots, live.float()[:, None])
                return ((total[slots] / count[slots].clamp(min=1.0)) @ weight.t()).to(x.dtype)
            out = torch.empty_like(x)
            at = 0
            for slot, n in zip(batch.slots, batch.q_lens):  # a prompt: its rows one after another
                sums = torch.cumsum(x[at : at + n].float(), 0) + total[slot]
                counts = count[slot] + torch.arange(1, n + 1, device=x.device, dtype=torch.float32)
                out[at : at + n] = ((sums / counts[:, None]) @ weight.t()).to(x.dtype)
                total[slot] = sums[-1]
                count[slot] += n
                at += n
            return out

    V, E = 90, 48

    def spec():
        norm = PartSpec("rmsnorm", {"eps": 1e-5})
        ff = PartSpec("glu", {"hidden_dim": 64, "activation": "swish"})
        mean_layer = LayerSpec(mixer=PartSpec("running_mean_on_device"), feed_forward=ff, norm=norm)
        attn_layer = LayerSpec(mixer=PartSpec("attention", {"nheads": 3, "kvheads": 1, "head_dim": 16}), feed_forward=ff,
                               norm=norm, position="rope")
        return ModelSpec(vocab=V, width=E, max_seq_len=256, layers=[mean_layer, attn_layer], final_norm=norm,
                         positions={"rope": PartSpec("rope", {"dim": 16, "theta": 1e4, "max_seq_len": 256})})

    register_part("mixer", "running_mean_on_device", RunningMeanOnDevice)
    try:
        model = DecoderModel(spec(), torch.float32)
        init_random(model, 8, torch.device(DEV), std=0.2, norm_std=0.1)
        model.finalize_all(DEV)
        w = {name: owner.w[local].float().cpu() for name, _, owner, local in model.named_specs()}

        def plain(ids):
            x = w["base_model.embedding.weight"][torch.tensor(ids)]
            cfg = P.PlainConfig(vocab=V, width=E, nheads=3, kvheads=1, nlayers=2, hidden=64, eps=1e-5, theta=1e4, max_len=256)
            for layer in (0, 1):
                p = f"base_model.layers.{layer}."
                h = P.rms_norm(x, w[p + "ln.weight"], 1e-5)
                if layer == 0:
                    h = (torch.cumsum(h, 0) / torch.arange(1, len(ids) + 1)[:, None]) @ w[p + "attn.proj.weight"].t()
                else:
                    h = P.attention_block(h, torch.arange(len(ids)), cfg, w[p + "attn.in_proj.qkv_fused.weight"],
                                          w[p + "attn.dense.weight"], P.rope_frequencies(16, 1e4))
                x = x + h
                h = P.rms_norm(x, w[p + "ff_ln.weight"], 1e-5)
                x = x + P.gated_feed_forward(h, w[p + "ff_sub_layer.wg1_fused.weight"], w[p + "ff_sub_layer.w2.weight"])
            return P.rms_norm(x, w["base_model.dec_norm.weight"], 1e-5) @ w["head.weight"].t()

        greedy = SamplingParams(do_sample=False)
        g = torch.Generator().manual_seed(5)
        chosen = {}
        for graphs in (True, False):
            engine = Engine(model, max_tokens=512, max_slots=3, use_graphs=graphs)
            assert engine.use_graphs == graphs  # nothing in the model refuses capture
            g.manual_seed(5)
            tokens_of_run = []
            for round_ in range(2):  # the second round takes the slots again: their state starts at zero
                prompts = [torch.randint(0, V, (n,), generator=g).tolist() for n in (20, 3, 9)]
                slots = [engine.new_sequence() for _ in prompts]
                first = engine.step(slots, prompts, "last").argmax(-1).tolist()
                seqs = [p + [t] for p, t in zip(prompts, first)]
                alive = [0, 1, 2]
                for step in range(7):
                    if step == 4:  # the middle sequence ends: the batch's rows change under the graph
                        engine.end_sequence(slots[1])
                        alive = [0, 2]
                    new = engine.decode_and_choose([slots[b] for b in alive], [seqs[b][-1] for b in alive], greedy)
                    logits = engine.last_graph.logits[: len(alive)].cpu() if graphs else None
                    for i, b in enumerate(alive):
                        if graphs:  # the logits of the fed token, against the plain computation of the sequence so far
                            torch.testing.assert_close(logits[i], plain(seqs[b])[-1], atol=2e-4, rtol=1e-3)
                        seqs[b].append(new[i])
                for b in alive:
                    engine.end_sequence(slots[b])
                tokens_of_run.append(seqs)
            if graphs:
                assert len(engine.graph_captures) >= 2
            engine.cache.check()
            chosen[graphs] = tokens_of_run
        assert chosen[True] == chosen[False]
    finally:
        unregister_part("mixer", "running_mean_on_device")


def test_a_layer_named_twice_and_a_layer_reading_another_cache(lib, tmp_path):
    """The order of layers is data: Llama's own layers in the order 0, 1, 0, with the last entry
    reading the keys and values that the first one cached (it computes queries only)."""
    import fms_amd
    from fms_amd.architectures.llama import llama_spec
    from fms_amd.engine import Engine
    from fms_amd.engine.model import DecoderModel
    from fms_amd.parts import ScheduleEntry
    from fms_amd.weights import init_random

    config = fms_amd.LLaMAConfig(src_vocab_size=70, emb_dim=64, nheads=4, kvheads=2, nlayers=2, hidden_dim=96, multiple_of=1,
                                 max_expected_seq_len=256)
    spec = llama_spec(config)
    spec.schedule = [ScheduleEntry(0), ScheduleEntry(1), ScheduleEntry(0, cache_of=0)]
    model = DecoderModel(spec, torch.float32, config=config)
    init_random(model, 5, torch.device(DEV), std=0.1, norm_std=0.1)
    model.finalize_all(DEV)
    engine = Engine(model, max_tokens=256, max_slots=1)
    w = {name: owner.w[local].float().cpu() for name, _, owner, local in model.named_specs()}
    cfg = P.PlainConfig(vocab=70, width=64, nheads=4, kvheads=2, nlayers=2, hidden=96, eps=1e-5, theta=1e4, max_len=256)
    ids = torch.randint(0, 70, (80,), generator=torch.Generator().manual_seed(2)).tolist()

    def plain(ids):
        S = len(ids)
        pos = torch.arange(S)
        freqs = P.rope_frequencies(16, 1e4)
        x = w["base_model.embedding.weight"][torch.tensor(ids)]
        kept = None
        for n, layer in enumerate((0, 1, 0)):
            p = f"base_model.layers.{layer}."
            h = P.rms_norm(x, w[p + "ln.weight"], 1e-5)
            qkv = h @ w[p + "attn.in_proj.qkv_fused.weight"].t()
            q, k, v = torch.split(qkv, [64, 32, 32], dim=-1)
            q = P.rope_rotate(q.reshape(S, 4, 16), pos, freqs)
            k = P.rope_rotate(k.reshape(S, 2, 16), pos, freqs)
            v = v.reshape(S, 2, 16)
            if n == 0:
                kept = (k, v)
            if n == 2:
                k, v = kept  # reads the first entry's cache
            a = P.causal_attention(q, k, v).reshape(S, 64) @ w[p + "attn.dense.weight"].t()
            x = x + a
            h = P.rms_norm(x, w[p + "ff_ln.weight"], 1e-5)
            x = x + P.gated_feed_forward(h, w[p + "ff_sub_layer.wg1_fused.weight"], w[p + "ff_sub_layer.w2.weight"])
        return P.rms_norm(x, w["base_model.dec_norm.weight"], 1e-5) @ w["head.weight"].t()

    slot = engine.new_sequence()
    got = [engine.step([slot], [ids[:70]], "all")] + [engine.step([slot], [[t]], "last") for t in ids[70:]]
    torch.testing.assert_close(torch.cat(got).cpu(), plain(ids), atol=2e-4, rtol=1e-3)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_a_layer_with_a_window_among_layers_without(lib, dtype):
    """Layers are configured one by one: Llama's parts with a window of 70 keys in the middle layer only.  That layer
    has a cache group of its own, which gives pages back while the sequences grow (the others keep theirs).  Two
    sequences of unequal lengths, a prompt step and 150 decode steps, as eager steps and through captured graphs,
    against the plain parts; the bfloat16 run against the float32 one."""
    import copy

    import fms_amd
    from fms_amd.architectures.llama import llama_spec
    from fms_amd.engine import Engine
    from fms_amd.engine.model import DecoderModel
    from fms_amd.sampling import SamplingParams
    from fms_amd.weights import init_random

    WINDOW = 70
    config = fms_amd.LLaMAConfig(src_vocab_size=120, emb_dim=64, nheads=4, kvheads=2, nlayers=3, hidden_dim=96, multiple_of=1,
                                 max_expected_seq_len=512)
    spec = llama_spec(config)
    spec.layers = [copy.deepcopy(layer) for layer in spec.layers]
    spec.layers[1].mixer.args["window"] = WINDOW
    model = DecoderModel(spec, dtype, config=config)
    init_random(model, 9, torch.device(DEV), std=0.1, norm_std=0.1)
    model.finalize_all(DEV)
    kv, _ = model.cache_needs()
    assert sorted(need.window for _, need in kv) == [0, 0, WINDOW]
    w = {name: owner.w[local].float().cpu() for name, _, owner, local in model.named_specs()}

    def plain(ids):
        S = len(ids)
        pos = torch.arange(S)
        freqs = P.rope_frequencies(16, 1e4)
        x = w["base_model.embedding.weight"][torch.tensor(ids)]
        for layer in range(3):
            p = f"base_model.layers.{layer}."
            h = P.rms_norm(x, w[p + "ln.weight"], 1e-5)
            qkv = h @ w[p + "attn.in_proj.qkv_fused.weight"].t()
            q, k, v = torch.split(qkv, [64, 32, 32], dim=-1)
            q = P.rope_rotate(q.reshape(S, 4, 16), pos, freqs)
            k = P.rope_rotate(k.reshape(S, 2, 16), pos, freqs)
            a = P.causal_attention(q, k, v.reshape(S, 2, 16), window=WINDOW if layer == 1 else 0)
            x = x + a.reshape(S, 64) @ w[p + "attn.dense.weight"].t()
            h = P.rms_norm(x, w[p + "ff_ln.weight"], 1e-5)
            x = x + P.gated_feed_forward(h, w[p + "ff_sub_layer.wg1_fused.weight"], w[p + "ff_sub_layer.w2.weight"])
        return P.rms_norm(x, w["base_model.dec_norm.weight"], 1e-5) @ w["head.weight"].t()

    g = torch.Generator().manual_seed(4)
    seqs = [torch.randint(0, 120, (n,), generator=g).tolist() for n in (290, 215)]
    prompt = (140, 65)
    want = [plain(ids) for ids in seqs]
    greedy = SamplingParams(do_sample=False)
    for graphs in (False, True):
        engine = Engine(model, max_tokens=64 * 12, max_slots=2, use_graphs=graphs)
        assert engine.use_graphs == graphs
        slots = [engine.new_sequence() for _ in seqs]
        logits = engine.step(slots, [ids[:n] for ids, n in zip(seqs, prompt)], "all")
        got = [[logits[: prompt[0]]], [logits[prompt[0] :]]]
        windowed = [i for i, group in enumerate(engine.cache.groups) if group.need.window][0]
        held_at_start = [len([p for p in engine.cache.groups[windowed].pages[s] if p >= 0]) for s in slots]
        for step in range(150):
            fed = [ids[n + step] for ids, n in zip(seqs, prompt)]
            if graphs:
                engine.decode_and_choose(slots, fed, greedy)
                rows = engine.last_graph.logits[:2].float()
            else:
                rows = engine.step(slots, [[t] for t in fed], "last")
            got[0].append(rows[0:1].clone())
            got[1].append(rows[1:2].clone())
        # the windowed group let pages go while the sequences grew by 150 tokens; the others hold every page
        full = [i for i, group in enumerate(engine.cache.groups) if not group.need.window][0]
        for b, s in enumerate(slots):
            live = [p for p in engine.cache.groups[windowed].pages[s] if p >= 0]
            assert len(live) <= 3 and len(live) <= held_at_start[b] + 1
            assert len([p for p in engine.cache.groups[full].pages[s] if p >= 0]) == -(-(prompt[b] + 150) // 64)
        engine.cache.check()
        for s in slots:
            engine.end_sequence(s)
        for rows, ref in zip(got, want):
            out = torch.cat(rows).cpu()
            if dtype == torch.float32:
                torch.testing.assert_close(out, ref, atol=2e-4, rtol=1e-3)
            else:
                assert float((out - ref).abs().max()) <= 0.06 * float(ref.abs().max())


def test_a_toy_feed_forward_with_routing_and_a_toy_position_encoding(lib):
    """Two more kinds of part that the library does not have, defined here and registered by name:
    a feed-forward that routes every token to one of three small experts (router logits and the chosen
    expert's probability in float32), and a position encoding that is no rotation (queries grow and keys
    shrink geometrically with the position, so a score is damped by the distance between them).
    One layer uses both, the other the library's own feed-forward; the model is built by get_model,
    stepped by Engine (prompts whole, then token by token, two sequences of unequal length) and
    compared with a plain computation that knows nothing of the parts."""
    import fms_amd
    from fms_amd.architectures import Architecture, register_architecture, register_model
    from fms_amd.config import ModelConfig
    from fms_amd.engine import Engine
    from fms_amd.engine.model import DecoderModel
    from fms_amd.weights import init_random
    from fms_amd.parts import FeedForward, LayerSpec, ModelSpec, PartSpec, register_part, unregister_part
    from fms_amd.parts.position import PositionEncoding

    class RoutedFeedForward(FeedForward):
        def __init__(self, width, hidden_dim, n_experts):
            super().__init__()
            self.width, self.hidden, self.n = width, hidden_dim, n_experts
            self.declare("router.weight", (n_experts, width))
            self.declare("experts.up", (n_experts, hidden_dim, width))
            self.declare("experts.down", (n_experts, width, hidden_dim))

        def forward(self, x):
            xf = x.float()
            logits = xf @ self.w["router.weight"].float().t()
            prob = torch.softmax(logits, -1)
            choice = logits.argmax(-1)
            out = torch.zeros_like(xf)
            for e in range(self.n):  # every expert on every token, the unchosen ones times zero: no host decision
                y = torch.relu(xf @ self.w["experts.up"][e].float().t()) @ self.w["experts.down"][e].float().t()
                out += y * (prob[:, e] * (choice == e))[:, None]
            return out.to(x.dtype)

    class DistanceDamping(PositionEncoding):
        def __init__(self, rate):
            super().__init__()
            self.rate = float(rate)

        def adjust_qk(self, qkv, batch, nheads, kvheads, head_dim):
            grow = torch.pow(torch.tensor(self.rate, device=qkv.device), -batch.positions.float())[:, None]
            q_cols, k_cols = nheads * head_dim, kvheads * head_dim
            qkv[:, :q_cols] = (qkv[:, :q_cols].float() / grow).to(qkv.dtype)  # q_i * rate^i
            qkv[:, q_cols : q_cols + k_cols] = (qkv[:, q_cols : q_cols + k_cols].float() * grow).to(qkv.dtype)  # k_j * rate^-j

    @dataclasses.dataclass
    class ToyConfig(ModelConfig):
        vocab: int = 77
        width: int = 40
        hidden: int = 56
        max_len: int = 128

    H, K, D, RATE = 5, 1, 8, 0.97

    def toy_spec(c: ToyConfig) -> ModelSpec:
        norm = PartSpec("rmsnorm", {"eps": 1e-6})
        attn = PartSpec("attention", {"nheads": H, "kvheads": K, "head_dim": D})
        routed = LayerSpec(mixer=attn, feed_forward=PartSpec("routed", {"hidden_dim": 24, "n_experts": 3}), norm=norm, position="damp")
        dense = LayerSpec(mixer=attn, feed_forward=PartSpec("glu", {"hidden_dim": c.hidden, "activation": "swish"}), norm=norm,
                          position="damp")
        return ModelSpec(vocab=c.vocab, width=c.width, max_seq_len=c.max_len, layers=[routed, dense], final_norm=norm,
                         positions={"damp": PartSpec("distance_damping", {"rate": RATE})})

    register_part("feed_forward", "routed", RoutedFeedForward)
    register_part("position", "distance_damping", DistanceDamping)
    try:
        try:
            register_architecture(Architecture("toy_routed", ToyConfig, toy_spec))
            register_model("toy_routed", "tiny", lambda **kw: ToyConfig().updated(**kw))
        except KeyError:
            pass  # a second run in one process
        built = fms_amd.get_model("toy_routed", "tiny", data_type="float32", random_seed=4)
        assert isinstance(built.layers[0].feed_forward, RoutedFeedForward) and isinstance(built.positions["damp"], DistanceDamping)
        # weights of std 0.02 would leave the router undecided and the damping invisible: the same model, wider weights
        model = DecoderModel(toy_spec(ToyConfig()), torch.float32, config=ToyConfig())
        init_random(model, 4, torch.device(DEV), std=0.2, norm_std=0.1)
        model.finalize_all(DEV)
        engine = Engine(model, max_tokens=256, max_slots=2)
        w = {name: owner.w[local].float().cpu() for name, _, owner, local in model.named_specs()}

        def plain(ids):
            S = len(ids)
            x = w["base_model.embedding.weight"][torch.tensor(ids)]
            dist = torch.arange(S)[:, None] - torch.arange(S)[None, :]
            damp = torch.where(dist >= 0, RATE ** dist.clamp(min=0).float(), torch.zeros(()))
            for layer in (0, 1):
                p = f"base_model.layers.{layer}."
                h = P.rms_norm(x, w[p + "ln.weight"], 1e-6)
                q, k, v = torch.split(h @ w[p + "attn.in_proj.qkv_fused.weight"].t(), [H * D, K * D, K * D], dim=-1)
                q, k, v = q.reshape(S, H, D), k.reshape(S, K, D), v.reshape(S, K, D)
                scores = torch.einsum("ihd,jd->hij", q, k[:, 0]) * damp / math.sqrt(D)
                scores = scores.masked_fill(dist < 0, float("-inf"))
                mixed = torch.einsum("hij,jd->ihd", torch.softmax(scores, -1), v[:, 0]).reshape(S, H * D)
                x = x + mixed @ w[p + "attn.dense.weight"].t()
                h = P.rms_norm(x, w[p + "ff_ln.weight"], 1e-6)
                if layer == 0:
                    logits = h @ w[p + "ff_sub_layer.router.weight"].t()
                    choice = logits.argmax(-1)
                    prob = torch.softmax(logits, -1)[torch.arange(S), choice]
                    up, down = w[p + "ff_sub_layer.experts.up"][choice], w[p + "ff_sub_layer.experts.down"][choice]
                    y = torch.einsum("sdh,sh->sd", down, torch.relu(torch.einsum("shd,sd->sh", up, h)))
                    x = x + y * prob[:, None]
                else:
                    x = x + P.gated_feed_forward(h, w[p + "ff_sub_layer.wg1_fused.weight"], w[p + "ff_sub_layer.w2.weight"])
            return P.rms_norm(x, w["base_model.dec_norm.weight"], 1e-6) @ w["head.weight"].t()

        g = torch.Generator().manual_seed(2)
        seqs = [torch.randint(0, 77, (n,), generator=g).tolist() for n in (41, 12)]
        slots = [engine.new_sequence() for _ in seqs]
        got = [[], []]
        logits = engine.step(slots, [s[:-3] for s in seqs], "all")
        got[0].append(logits[: len(seqs[0]) - 3])
        got[1].append(logits[len(seqs[0]) - 3 :])
        for i in range(3, 0, -1):
            logits = engine.step(slots, [[s[-i]] for s in seqs], "last")
            got[0].append(logits[0:1])
            got[1].append(logits[1:2])
        for ids, rows in zip(seqs, got):
            torch.testing.assert_close(torch.cat(rows).cpu(), plain(ids), atol=2e-4, rtol=1e-3)
        # and the damping did something: without it the logits differ visibly
        RATE_KEEP = RATE
        try:
            RATE = 1.0
            assert (plain(seqs[0]) - torch.cat(got[0]).cpu()).abs().max() > 1e-3
        finally:
            RATE = RATE_KEEP
    finally:
        unregister_part("feed_forward", "routed")
        unregister_part("position", "distance_damping")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_toy_parts_at_three_seams(lib, dtype):
    """Three more parts the library has never heard of, defined here and put together through the registries:
      * an embedding that adds a learned vector per position (it reads the step's positions: the model hands every
        embedding the batch);
      * a position encoding that acts on the scores and not on queries and keys (a slope per head times the
        distance, the reference's adjusted_mask seam, fms/modules/positions.py:9-36), with an attention whose
        scores are capped;
      * a block that wants four norms, before and after each branch, and says so.
    Stepped by the engine (prompts whole, then token by token, unequal lengths, a reused slot) against a plain
    computation; bfloat16 against float32 on the same rounded weights."""
    from fms_amd.engine import Engine
    from fms_amd.engine.model import DecoderModel
    from fms_amd.kernels import ops
    from fms_amd.parts import LayerSpec, ModelSpec, Part, PartSpec, register_part, unregister_part
    from fms_amd.parts.position import PositionEncoding
    from fms_amd.weights import init_random

    V, E, H, K, D, HID, MAXLEN, CAP = 61, 48, 4, 2, 16, 80, 96, 3.0

    class PositionedEmbedding(Part):
        def __init__(self, vocab, width, max_len):
            super().__init__()
            self.declare("weight", (vocab, width))
            self.declare("positions", (max_len, width))

        def forward(self, token_ids, batch=None):
            return ops.embed(token_ids, self.w["weight"]) + ops.embed(batch.positions, self.w["positions"])

    class DistanceSlopes(PositionEncoding):
        def __init__(self, steepest):
            super().__init__()
            self.steepest, self._slopes = float(steepest), {}

        def slope_values(self, nheads):
            return [self.steepest * 2.0 ** -h for h in range(nheads)]

        def score_slopes(self, nheads):
            if nheads not in self._slopes:
                self._slopes[nheads] = torch.tensor(self.slope_values(nheads), dtype=torch.float32, device=DEV)
            return self._slopes[nheads]

    class SandwichBlock(Part):
        norm_arguments = ("before_mixer", "after_mixer", "before_ff", "after_ff")

        def __init__(self, mixer, feed_forward, before_mixer, after_mixer, before_ff, after_ff):
            super().__init__()
            self.mixer = self.add_child("attn", mixer)
            self.feed_forward = self.add_child("ff_sub_layer", feed_forward)
            self.norms = [self.add_child(n, p) for n, p in zip(("ln", "post_attn_ln", "ff_ln", "post_ff_ln"),
                                                                (before_mixer, after_mixer, before_ff, after_ff))]

        def forward(self, stream, batch, cache, act_dtype, next_norm=None):
            h = stream.normed(self.norms[0], act_dtype)
            out = self.mixer.forward(h, batch, cache)
            zeros = torch.zeros(out.shape, dtype=torch.float32, device=out.device)
            stream.add_branch(self.norms[1].add_norm(zeros, out, act_dtype))  # the branch's output through a norm of its own
            h = stream.normed(self.norms[2], act_dtype)
            out = self.feed_forward.forward(h)
            zeros = torch.zeros(out.shape, dtype=torch.float32, device=out.device)
            stream.add_branch(self.norms[3].add_norm(zeros, out, act_dtype))

    def spec():
        norms = [PartSpec("rmsnorm", {"eps": e}) for e in (1e-5, 1e-6, 1e-5, 1e-4)]
        layer = LayerSpec(mixer=PartSpec("attention", {"nheads": H, "kvheads": K, "head_dim": D, "soft_cap": CAP}),
                          feed_forward=PartSpec("glu", {"hidden_dim": HID, "activation": "gelu"}), norms=norms,
                          block=PartSpec("sandwich"), position="slopes")
        return ModelSpec(vocab=V, width=E, max_seq_len=MAXLEN, layers=[layer, layer], final_norm=PartSpec("rmsnorm", {"eps": 1e-5}),
                         embedding=PartSpec("positioned", {"max_len": MAXLEN}),
                         positions={"slopes": PartSpec("distance_slopes", {"steepest": 0.5})})

    register_part("embedding", "positioned", PositionedEmbedding)
    register_part("position", "distance_slopes", DistanceSlopes)
    register_part("block", "sandwich", SandwichBlock)
    try:
        with pytest.raises(ValueError, match="takes 4 norms"):
            bad = spec()
            bad.layers[0].norms = bad.layers[0].norms[:2]
            DecoderModel(bad, torch.float32)
        model = DecoderModel(spec(), dtype)
        init_random(model, 6, torch.device(DEV), std=0.25, norm_std=0.2)
        model.finalize_all(DEV)
        assert len(model.layers[0].norms) == 4 and model.layers[1].norms[3].eps == 1e-4
        engine = Engine(model, max_tokens=256, max_slots=2)
        w = {name: owner.w[local].float().cpu() for name, _, owner, local in model.named_specs()}
        slopes = torch.tensor(DistanceSlopes(0.5).slope_values(H))

        def plain(ids):
            S = len(ids)
            x = w["base_model.embedding.weight"][torch.tensor(ids)] + w["base_model.embedding.positions"][:S]
            dist = (torch.arange(S)[:, None] - torch.arange(S)[None, :]).float()
            for layer in (0, 1):
                p = f"base_model.layers.{layer}."
                h = P.rms_norm(x, w[p + "ln.weight"], 1e-5)
                q, k, v = torch.split(h @ w[p + "attn.in_proj.qkv_fused.weight"].t(), [H * D, K * D, K * D], dim=-1)
                q, k, v = q.reshape(S, H, D), k.reshape(S, K, D), v.reshape(S, K, D)
                k, v = k.repeat_interleave(H // K, dim=1), v.repeat_interleave(H // K, dim=1)
                scores = CAP * torch.tanh(torch.einsum("ihd,jhd->hij", q, k) / math.sqrt(D) / CAP) - slopes[:, None, None] * dist.abs()
                probs = torch.softmax(scores.masked_fill(dist < 0, float("-inf")), -1)
                mixed = torch.einsum("hij,jhd->ihd", probs, v).reshape(S, H * D) @ w[p + "attn.dense.weight"].t()
                x = x + P.rms_norm(mixed, w[p + "post_attn_ln.weight"], 1e-6)
                h = P.rms_norm(x, w[p + "ff_ln.weight"], 1e-5)
                y = P.gated_feed_forward(h, w[p + "ff_sub_layer.wg1_fused.weight"], w[p + "ff_sub_layer.w2.weight"], act_name="gelu")
                x = x + P.rms_norm(y, w[p + "post_ff_ln.weight"], 1e-4)
            return P.rms_norm(x, w["base_model.dec_norm.weight"], 1e-5) @ w["head.weight"].t()

        g = torch.Generator().manual_seed(3)
        for lengths in ((70, 9), (33,)):  # the second round takes a slot of the first
            seqs = [torch.randint(0, V, (n,), generator=g).tolist() for n in lengths]
            slots = [engine.new_sequence() for _ in seqs]
            logits = engine.step(slots, [s[:-3] for s in seqs], "all")
            got, at = [], 0
            for s in seqs:
                got.append([logits[at : at + len(s) - 3]])
                at += len(s) - 3
            for i in range(3, 0, -1):
                logits = engine.step(slots, [[s[-i]] for s in seqs], "last")
                for b in range(len(seqs)):
                    got[b].append(logits[b : b + 1])
            for slot in slots:
                engine.end_sequence(slot)
            for ids, rows in zip(seqs, got):
                close(torch.cat(rows).cpu(), plain(ids), dtype)
        engine.cache.check()
        # each of the three did something: the plain computation without it is far from the engine's logits
        ids = torch.randint(0, V, (40,), generator=g).tolist()
        slot = engine.new_sequence()
        have = engine.step([slot], [ids], "all").cpu()
        engine.end_sequence(slot)
        full = plain(ids)
        close(have, full, dtype)
        w_keep = dict(w)
        w["base_model.embedding.positions"] = torch.zeros_like(w["base_model.embedding.positions"])
        assert float((plain(ids) - full).abs().max()) > 0.1 * float(full.abs().max())
        w.update(w_keep)
        slopes = slopes * 0
        assert float((plain(ids) - full).abs().max()) > 0.02 * float(full.abs().max())
    finally:
        unregister_part("embedding", "positioned")
        unregister_part("position", "distance_slopes")
        unregister_part("block", "sandwich")
