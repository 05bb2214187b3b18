"""Pins of the plain implementation: what fixes it beside the reference's text.

* the output signatures the reference's own tests store
  (tests/resources/expectations/models.test_llama.*.test_model_output),
* special cases that reduce to a library routine,
* invariants chosen so that a plausible mistake fails them.
"""

import math

import pytest
import torch
import torch.nn.functional as F

import plain_llama as P

# The four stored signatures (16 floats each), copied from the reference's
# tests/resources/expectations/models.test_llama.<Class>.test_model_output
SIGNATURES = {
    "TestLlama2": "0.052729345858097076,0.011515989899635315,0.007392197847366333,0.0,0.01378333568572998,0.012065891176462173,0.03835539519786835,0.02802693098783493,0.020719021558761597,0.027966909110546112,0.014432244002819061,0.03975895047187805,0.05111371725797653,0.04628599435091019,0.0315752848982811,0.01688060164451599",
    "TestLlama2GQA": "0.033434536308050156,0.03998075798153877,0.020981933921575546,0.0,0.040768157690763474,0.03792032226920128,0.026382219046354294,0.033903587609529495,0.012676555663347244,0.0020506493747234344,0.026054974645376205,0.003850828856229782,0.033241596072912216,0.006034858524799347,0.004931684583425522,0.022256117314100266",
    "TestLlama3": "0.03351592645049095,0.040137480944395065,0.021625619381666183,0.0,0.03257865831255913,0.036533039063215256,0.027063172310590744,0.037584420293569565,0.01366950199007988,0.002703893929719925,0.025658320635557175,0.0047348253428936005,0.03350717946887016,0.0010565221309661865,0.007586400955915451,0.02299729362130165",
    "TestLlama31": "0.03351592645049095,0.040137480944395065,0.021625619381666183,0.0,0.03257865831255913,0.036533039063215256,0.027063172310590744,0.03758440539240837,0.01366950199007988,0.002703893929719925,0.025658313184976578,0.0047348253428936005,0.03350717946887016,0.0010565221309661865,0.007586400955915451,0.02299729362130165",
}

# configurations of those tests: tests/models/test_llama.py:30-45, :108-122, :196-211 and :232-253
SIG_CONFIGS = {
    "TestLlama2": dict(seed=0, nheads=2, kvheads=2, grow=8 / 3, theta=10000.0, max_len=4096, scaling={}),
    "TestLlama2GQA": dict(seed=5, nheads=4, kvheads=2, grow=8 / 3, theta=10000.0, max_len=4096, scaling={}),
    "TestLlama3": dict(seed=5, nheads=4, kvheads=2, grow=3.5, theta=500000.0, max_len=8192, scaling={}),
    "TestLlama31": dict(
        seed=5,
        nheads=4,
        kvheads=2,
        grow=3.5,
        theta=500000.0,
        max_len=131072,
        scaling={
            "factor": 8.0,
            "low_freq_factor": 1.0,
            "high_freq_factor": 4.0,
            "original_max_position_embeddings": 8192,
            "rope_type": "llama3",
        },
    ),
}


def _fixture_weights(cfg: P.PlainConfig, seed: int):
    """fms/testing/_internal/model_test_suite.py:61-79: every tensor of the state dict,
    in sorted-name order, is (randn - 0.5) / 20 under one seed."""
    D = cfg.head_dim
    shapes = {
        "base_model.dec_norm.weight": (cfg.width,),
        "base_model.embedding.weight": (cfg.vocab, cfg.width),
        "head.weight": (cfg.vocab, cfg.width),
    }
    for i in range(cfg.nlayers):
        p = f"base_model.layers.{i}."
        shapes[p + "attn.dense.weight"] = (cfg.width, cfg.nheads * D)
        shapes[p + "attn.in_proj.qkv_fused.weight"] = ((cfg.nheads + 2 * cfg.kvheads) * D, cfg.width)
        shapes[p + "ff_ln.weight"] = (cfg.width,)
        shapes[p + "ff_sub_layer.w2.weight"] = (cfg.width, cfg.hidden)
        shapes[p + "ff_sub_layer.wg1_fused.weight"] = (2 * cfg.hidden, cfg.width)
        shapes[p + "ln.weight"] = (cfg.width,)
    torch.random.manual_seed(seed)
    weights = {}
    for name in sorted(shapes):
        values = torch.randn(shapes[name])
        values -= 0.5
        values /= 20.0
        weights[name] = values
    return weights


@pytest.mark.parametrize("name", sorted(SIGNATURES))
def test_reference_signature(name):
    c = SIG_CONFIGS[name]
    cfg = P.PlainConfig(
        vocab=381,
        width=16,
        nheads=c["nheads"],
        kvheads=c["kvheads"],
        nlayers=2,
        hidden=P.glu_hidden(16, c["grow"], 2),
        eps=1e-5,
        theta=c["theta"],
        max_len=c["max_len"],
        rope_scaling=c["scaling"],
    )
    weights = _fixture_weights(cfg, c["seed"])
    logits = P.forward(weights, cfg, list(range(16)))
    # fms/testing/comparison.py:104-105
    s = logits.max(-1).values - logits.min(-1).values
    signature = s - s.min()
    expected = torch.tensor([float(v) for v in SIGNATURES[name].split(",")])
    torch.testing.assert_close(signature, expected)


def test_glu_hidden_sizes():
    assert P.glu_hidden(16, 8 / 3, 2) == 42
    assert P.glu_hidden(4096, 8 / 3, 256) == 11008
    assert P.glu_hidden(4096, 3.5, 1024) == 14336
    assert P.glu_hidden(8192, 1.3 * 8 / 3, 4096) == 28672


def test_rms_norm_is_library_rms_norm():
    torch.manual_seed(1)
    x = torch.randn(5, 24) * 3
    w = torch.randn(24)
    torch.testing.assert_close(P.rms_norm(x, w, 1e-3), F.rms_norm(x, (24,), w, 1e-3))
    # eps inside the root: a zero row gives zeros, not NaN
    assert torch.equal(P.rms_norm(torch.zeros(1, 24), w, 1e-5), torch.zeros(1, 24))
    # a large eps visibly shrinks the output (eps outside the root or forgotten would not)
    y = P.rms_norm(torch.ones(1, 4), torch.ones(4), 3.0)
    torch.testing.assert_close(y, torch.full((1, 4), 0.5))


def test_rope_reference_vectors():
    """tests/modules/test_positions.py:47-72: D=2, theta=1 rotates by `pos` radians."""
    x = torch.tensor([[1.0, 0.0], [1.0, 0.0]]).reshape(2, 1, 2)
    out = P.rope_rotate(x, torch.arange(2), P.rope_frequencies(2, 1.0))
    torch.testing.assert_close(out[0, 0], torch.tensor([1.0, 0.0]))
    torch.testing.assert_close(out[1, 0], torch.tensor([math.cos(1.0), math.sin(1.0)]))


def test_rope_is_complex_multiplication():
    torch.manual_seed(2)
    D = 24
    x = torch.randn(7, 3, D)
    pos = torch.tensor([0, 1, 2, 5, 9, 100, 1000])
    freqs = P.rope_frequencies(D, 500000.0)
    out = P.rope_rotate(x, pos, freqs)
    z = torch.view_as_complex(x.reshape(7, 3, D // 2, 2).contiguous())
    rot = torch.polar(torch.ones(7, D // 2), torch.outer(pos.float(), freqs))[:, None, :]
    torch.testing.assert_close(out, torch.view_as_real(z * rot).reshape(7, 3, D))
    # position 0 is the identity; norms are kept
    torch.testing.assert_close(out[0], x[0])
    torch.testing.assert_close(out.norm(dim=-1), x.norm(dim=-1))


def test_rope_scores_depend_on_distance_only():
    """tests/modules/test_positions.py:191-214: a shift of all positions changes no score."""
    torch.manual_seed(3)
    D = 16
    q = torch.randn(6, 1, D)
    k = torch.randn(6, 1, D)
    freqs = P.rope_frequencies(D, 10000.0)
    pos = torch.arange(6)
    s0 = P.rope_rotate(q, pos, freqs)[:, 0] @ P.rope_rotate(k, pos, freqs)[:, 0].t()
    s1 = P.rope_rotate(q, pos + 37, freqs)[:, 0] @ P.rope_rotate(k, pos + 37, freqs)[:, 0].t()
    torch.testing.assert_close(s0, s1, atol=1e-4, rtol=1e-4)
    # ...and a wrong sign of the sine would still pass the above, so pin the direction:
    one = P.rope_rotate(torch.tensor([1.0, 0.0]).reshape(1, 1, 2), torch.tensor([1]), torch.tensor([0.5]))
    assert one[0, 0, 1] > 0


def test_rope_pairings_agree_after_row_permutation():
    """fms/models/llama.py:711-721: half-split rotation of HF-ordered rows equals
    adjacent-pair rotation of the permuted rows, up to the same permutation of the output."""
    torch.manual_seed(4)
    D, heads, E, S = 16, 3, 10, 5
    w_hf = torch.randn(heads * D, E)
    x = torch.randn(S, E)
    pos = torch.arange(S) + 3
    freqs = P.rope_frequencies(D, 10000.0)
    q_hf = P.rope_rotate_halves((x @ w_hf.t()).reshape(S, heads, D), pos, freqs)
    q_ref = P.rope_rotate((x @ P._halves_to_pairs(w_hf, D).t()).reshape(S, heads, D), pos, freqs)
    # scores are what matters: a dot product over the head is permutation invariant
    torch.testing.assert_close(
        torch.einsum("shd,thd->hst", q_hf, q_hf), torch.einsum("shd,thd->hst", q_ref, q_ref), atol=1e-4, rtol=1e-4
    )
    # and element-wise: reference element 2i+j is HF element j*D/2+i
    torch.testing.assert_close(q_ref.reshape(S, heads, D // 2, 2).transpose(2, 3).reshape(S, heads, D), q_hf)


def test_rope_ntk_scaling_reference_vector():
    """tests/modules/test_positions.py:216-241: up to the table's length ntk scaling changes nothing; for a
    sequence of twice that length it equals the regular rotation of a base that is 2^(D/(D-2)) times larger."""
    D, S = 50, 10
    x = torch.randn(S, 5, D)
    positions = torch.arange(S)
    regular = P.rope_rotate(x, positions, P.rope_frequencies(D, 10_000.0))
    same = P.rope_rotate(x, positions, P.rope_frequencies(D, 10_000.0, {"rope_type": "ntk"}, S, S))
    torch.testing.assert_close(same, regular)
    scaled_ratio = 10_000 / 2 ** (D / (D - 2))
    stretched = P.rope_rotate(x, positions, P.rope_frequencies(D, scaled_ratio, {"rope_type": "ntk"}, S, S // 2))
    torch.testing.assert_close(stretched, regular)
    assert [P.ntk_alpha(n, 5) for n in (1, 5, 6, 10, 11, 21)] == [1, 1, 2, 2, 4, 8]


def test_rope_llama3_scaling_limits():
    scaling = {
        "rope_type": "llama3",
        "factor": 8.0,
        "low_freq_factor": 1.0,
        "high_freq_factor": 4.0,
        "original_max_position_embeddings": 8192,
    }
    base = P.rope_frequencies(128, 500000.0)
    scaled = P.rope_frequencies(128, 500000.0, scaling)
    wavelen = 2 * math.pi / base
    assert torch.equal(scaled[wavelen < 8192 / 4], base[wavelen < 8192 / 4])
    torch.testing.assert_close(scaled[wavelen > 8192], base[wavelen > 8192] / 8)
    mid = (wavelen >= 8192 / 4) & (wavelen <= 8192)
    assert mid.any() and bool(((scaled[mid] < base[mid]) & (scaled[mid] > base[mid] / 8)).all())


def _llama3_checks(freq_fn):
    """What fixes the mid band of the llama3 scaling beside the reference's lines (fms/modules/positions.py:171-196).
    Returns the list of checks that `freq_fn(dim, theta, scaling)` fails."""
    failed = []
    # 1. two frequencies worked out by hand.  D=16, theta=1e4: f_i = 1e4^(-i/8) = 1, 0.3162.., 0.1, 0.03162.., ...;
    # original length 64, low 1, high 4, factor 8: wavelengths 6.28 (kept), 19.87 and 62.83 (between 64/4 and
    # 64/1: interpolated), 198.7 and longer (divided by 8).  For i=1: smooth = (64/19.869.. - 1)/3 = 0.74035..,
    # f = 0.25964..*0.31622../8 + 0.74035..*0.31622.. = 0.244384..; for i=2: smooth = 0.0061972.., f = 0.0130422..
    small = {"rope_type": "llama3", "factor": 8.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0,
             "original_max_position_embeddings": 64}
    got = freq_fn(16, 10000.0, small)
    by_hand = torch.tensor([1.0, 0.24438459943539834, 0.013042256043820465, 0.03162277660168379 / 8, 0.01 / 8])
    if not torch.allclose(got[:5], by_hand, rtol=2e-5, atol=0):
        failed.append("hand-computed vector")
    # 2. the band as a whole, on many frequencies (D=1024 puts some hundred of them into it): scaled / unscaled is a
    # straight line in 1/wavelength through (low edge, 1/factor) and (high edge, 1): continuous at both edges, and it
    # rises with the frequency.
    scaling = {"rope_type": "llama3", "factor": 8.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0,
               "original_max_position_embeddings": 8192}
    base = freq_fn(1024, 500000.0, None).double()
    ratio = freq_fn(1024, 500000.0, scaling).double() / base
    per_length = base * 8192 / (2 * math.pi)  # original length / wavelength: 1 at the low edge, 4 at the high edge
    mid = (per_length >= 1.0) & (per_length <= 4.0)
    assert int(mid.sum()) > 50
    line = 1 / 8 + (1 - 1 / 8) * (per_length - 1.0) / (4.0 - 1.0)
    if not torch.allclose(ratio[mid], line[mid], rtol=1e-4, atol=0):
        failed.append("line through the band's ends")
    lowest, highest = ratio[mid][-1], ratio[mid][0]  # frequencies fall with the index
    if not (abs(float(lowest) - 1 / 8) < 0.01 and abs(float(highest) - 1.0) < 0.02):
        failed.append("continuity at the edges")
    if not bool((ratio[mid][:-1] >= ratio[mid][1:]).all()):
        failed.append("monotone")
    if not (torch.equal(ratio[per_length > 4.0], torch.ones_like(ratio[per_length > 4.0]))
            and torch.allclose(ratio[per_length < 1.0], torch.full_like(ratio[per_length < 1.0], 1 / 8), rtol=1e-6)):
        failed.append("outside the band")
    return failed


def test_rope_llama3_mid_band():
    """The interpolation between the kept and the divided frequencies (a Llama-3.1 config.json takes it)."""
    assert _llama3_checks(lambda d, th, sc: P.rope_frequencies(d, th, sc)) == []


def test_rope_llama3_checks_reject_plausible_mistakes():
    """The checks above can fail: the interpolation weights swapped, the scaling left out, the band's ends swapped."""

    def variant(kind):
        def freqs(dim, theta, scaling):
            f = 1.0 / (theta ** (torch.arange(0, dim, 2)[: dim // 2].float() / dim))
            if not scaling or kind == "no scaling":
                return f
            factor, low, high = scaling["factor"], scaling["low_freq_factor"], scaling["high_freq_factor"]
            old = scaling["original_max_position_embeddings"]
            if kind == "ends swapped":
                low, high = high, low
            wavelen = 2 * math.pi / f
            smooth = (old / wavelen - low) / (high - low)
            if kind == "weights swapped":
                smooth = 1 - smooth
            out = torch.where(wavelen > old / min(low, high), f / factor, f)
            band = (wavelen >= old / max(low, high)) & (wavelen <= old / min(low, high))
            return torch.where(band, (1 - smooth) * f / factor + smooth * f, out)

        return freqs

    for kind in ("weights swapped", "no scaling", "ends swapped"):
        failed = _llama3_checks(variant(kind))
        assert "hand-computed vector" in failed and "line through the band's ends" in failed, (kind, failed)
    assert _llama3_checks(variant("right")) == []


def test_activations_are_the_library_functions():
    """fms/utils/activation.py:6-24: every name is a torch.nn module; the formulas written out in the plain
    implementation are those modules' functions."""
    x = torch.linspace(-9, 9, 721)
    x = torch.cat([x, torch.tensor([25.0, -25.0, 0.0])])  # mish's softplus is linear beyond 20
    table = {
        "gelu": F.gelu,
        "gelu-tanh": lambda t: F.gelu(t, approximate="tanh"),
        "gelu_pytorch_tanh": lambda t: F.gelu(t, approximate="tanh"),
        "mish": F.mish,
        "relu": F.relu,
        "sigmoid": torch.sigmoid,
        "silu": F.silu,
        "swish": F.silu,
        "tanh": torch.tanh,
    }
    for name, fn in table.items():
        torch.testing.assert_close(P.activation(name)(x), fn(x), atol=1e-6, rtol=1e-5, msg=lambda m, n=name: f"{n}: {m}")
        torch.testing.assert_close(P.activation(name.upper())(x), fn(x), atol=1e-6, rtol=1e-5)
    # the two gelus differ by more than the tolerance, so a swapped pair fails the above
    assert float((F.gelu(x) - F.gelu(x, approximate="tanh")).abs().max()) > 1e-4


def test_ntk_scaling_keeps_the_rotation_of_cached_keys():
    """fms/modules/positions.py:394-421 with a cache: every call rotates its new tokens with the frequencies of its
    own alpha.  P.forward(calls=...) states that; here it is pinned by its special cases: calls within one alpha are
    the whole-sequence forward, the last call's row depends on the alpha of earlier calls once a border was crossed,
    and scores between tokens of one call still depend on their distance only."""
    cfg = P.PlainConfig(vocab=50, width=24, nheads=3, kvheads=1, nlayers=2, hidden=40, eps=1e-5, theta=1e4, max_len=8,
                        rope_scaling={"rope_type": "ntk", "factor": 4.0})
    weights = {k: 8 * v for k, v in _fixture_weights(cfg, 12).items()}  # large enough for attention to choose
    ids = [3, 9, 4, 4, 17, 30, 2, 8, 11, 12, 40, 41]
    whole = P.forward(weights, cfg, ids)  # one call of 12 tokens: alpha 2 throughout
    torch.testing.assert_close(P.forward(weights, cfg, ids, calls=[(12, 12)]), whole)
    # fed in calls that all see alpha 2 (their batch's longest sequence has 9..16 tokens): the same logits
    torch.testing.assert_close(P.forward(weights, cfg, ids, calls=[(5, 16), (4, 9), (3, 12)]), whole, atol=1e-5, rtol=1e-5)
    # the first 8 tokens fed alone (alpha 1), the rest one by one (alpha 2): the first 8 rows are the regular model's,
    # and the later rows differ from the whole call's, because they read keys rotated with the other base
    stepped = P.forward(weights, cfg, ids, calls=[(8, 8), (1, 9), (1, 10), (1, 11), (1, 12)])
    regular = P.PlainConfig(**{**cfg.__dict__, "rope_scaling": {}})
    torch.testing.assert_close(stepped[:8], P.forward(weights, regular, ids[:8]), atol=1e-5, rtol=1e-5)
    assert float((stepped[8:] - whole[8:]).abs().max()) > 1e-3
    # the frequencies themselves: positions 0..7 those of alpha 1, 8..11 those of alpha 2 = theta * 2^(D/(D-2))
    D = cfg.head_dim
    f1 = P.rope_frequencies(D, cfg.theta)
    f2 = P.rope_frequencies(D, cfg.theta * 2 ** (D / (D - 2)))
    torch.testing.assert_close(P.rope_frequencies(D, cfg.theta, cfg.rope_scaling, 8, 8), f1)
    torch.testing.assert_close(P.rope_frequencies(D, cfg.theta, cfg.rope_scaling, 9, 8), f2)
    # a key of position 3 cached under alpha 1 against a query of position 9 under alpha 2: the score is the product
    # of the two rotations, not a function of the distance
    x = torch.randn(1, 1, D)
    k3 = P.rope_rotate(x, torch.tensor([3]), f1)
    q9 = P.rope_rotate(x, torch.tensor([9]), f2)
    k3_same = P.rope_rotate(x, torch.tensor([3]), f2)
    assert abs(float((q9 * k3).sum() - (q9 * k3_same).sum())) > 1e-3


@pytest.mark.parametrize("H,K", [(4, 4), (4, 2), (4, 1), (1, 1)])
def test_attention_is_library_attention(H, K):
    torch.manual_seed(5)
    S, D = 9, 8
    q, k, v = torch.randn(S, H, D), torch.randn(S, K, D), torch.randn(S, K, D)
    ours = P.causal_attention(q, k, v)
    ke = k.repeat_interleave(H // K, dim=1)
    ve = v.repeat_interleave(H // K, dim=1)
    lib = F.scaled_dot_product_attention(
        q.transpose(0, 1)[None], ke.transpose(0, 1)[None], ve.transpose(0, 1)[None], is_causal=True
    )[0].transpose(0, 1)
    torch.testing.assert_close(ours, lib, atol=1e-5, rtol=1e-5)


def test_attention_special_cases():
    torch.manual_seed(6)
    S, H, K, D = 6, 4, 2, 8
    q, k, v = torch.randn(S, H, D), torch.randn(S, K, D), torch.randn(S, K, D)
    out = P.causal_attention(q, k, v)
    # the first query sees one key: its output is that key's value, of its own kv head
    torch.testing.assert_close(out[0, 0], v[0, 0])
    torch.testing.assert_close(out[0, 3], v[0, 1])
    # zero queries average the visible values
    avg = P.causal_attention(torch.zeros_like(q), k, v)
    torch.testing.assert_close(avg[3, 2], v[:4, 1].mean(0))
    # a window of 1 sees only the token itself
    win = P.causal_attention(q, k, v, window=1)
    torch.testing.assert_close(win[:, 1], v[:, 0])


def test_feed_forward_gate_comes_first():
    """tests/utils/test_fusion.py:28-41, tests/utils/test_serialization.py:16-25: fused = [gate; up]."""
    torch.manual_seed(7)
    E, Fh = 6, 10
    wg, w1, w2 = torch.randn(Fh, E), torch.randn(Fh, E), torch.randn(E, Fh)
    x = torch.randn(4, E)
    fused = P.gated_feed_forward(x, torch.cat([wg, w1]), w2)
    torch.testing.assert_close(fused, (F.silu(x @ wg.t()) * (x @ w1.t())) @ w2.t())
    # a zero gate gives zero, a zero "up" too; swapping the halves would change this
    zero_gate = P.gated_feed_forward(x, torch.cat([torch.zeros(Fh, E), w1]), w2)
    assert torch.equal(zero_gate, torch.zeros(4, E))


def test_forward_prefix_property():
    """Causality: logits of a prefix do not change when tokens are appended."""
    cfg = P.PlainConfig(vocab=50, width=24, nheads=3, kvheads=1, nlayers=2, hidden=40, eps=1e-5, theta=1e4, max_len=64)
    weights = _fixture_weights(cfg, 11)
    ids = [3, 9, 4, 4, 17, 30, 2, 8]
    full = P.forward(weights, cfg, ids)
    part = P.forward(weights, cfg, ids[:5])
    torch.testing.assert_close(full[:5], part, atol=1e-5, rtol=1e-5)
    with pytest.raises(IndexError):
        P.forward(weights, cfg, list(range(40)), first_position=30)


def test_bfloat16_roundings_of_the_reference():
    """fms/modules/layernorm.py:60-66 in bfloat16 is the module's own sequence of casts; and a model run with
    the reference's roundings differs from the float32 one by bfloat16-sized errors, a little more than a run
    that rounds stored tensors only (it rounds in more places)."""
    torch.manual_seed(4)
    x = (torch.randn(7, 48) * 3).bfloat16()
    w = (1 + 0.3 * torch.randn(48)).bfloat16()
    xf = x.float()
    want = w * (xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + 1e-5)).type_as(x)  # bfloat16 * bfloat16
    assert want.dtype == torch.bfloat16
    got = P.rms_norm_as_stored(x.float(), w.float(), 1e-5, torch.bfloat16)
    assert torch.equal(got, want.float())
    assert not torch.equal(got, P.rms_norm(x.float(), w.float(), 1e-5).bfloat16().float())  # one rounding is not two

    cfg = P.PlainConfig(vocab=50, width=32, nheads=4, kvheads=2, nlayers=3, hidden=72, eps=1e-5, theta=1e4, max_len=64)
    weights = {k: (v * 3).bfloat16().float() for k, v in _fixture_weights(cfg, 12).items()}
    ids = list(range(5, 45))
    exact = P.forward(weights, cfg, ids)
    stored = P.forward(weights, cfg, ids, storage=torch.bfloat16)
    reference = P.forward(weights, cfg, ids, storage=torch.bfloat16, rounding="reference")
    assert torch.equal(reference, reference.bfloat16().float())  # the reference's logits are bfloat16 numbers
    scale = float(exact.abs().max())
    e_stored, e_ref = float((stored - exact).abs().max()), float((reference - exact).abs().max())
    assert 1e-4 * scale < e_stored < 0.05 * scale and 1e-4 * scale < e_ref < 0.05 * scale
    assert float((stored - exact).abs().mean()) < float((reference - exact).abs().mean())
    assert torch.equal(P.forward(weights, cfg, ids, storage=torch.float32, rounding="reference"), exact)


def test_seeded_draws():
    """The uniform numbers fill [0, 1) evenly and differ by request and by draw; the inverse CDF picks the token
    whose interval holds the number."""
    us = [P.draw_uniform(P.seed_of_request(3, r), n) for r in range(8) for n in range(250)]
    assert all(0 <= u < 1 for u in us) and len(set(us)) > 1990
    assert abs(sum(us) / len(us) - 0.5) < 0.03 and abs(sum(u < 0.1 for u in us) / len(us) - 0.1) < 0.03
    assert P.draw_uniform(5, 9) == P.draw_uniform(5, 9) != P.draw_uniform(5, 10)
    assert P.seed_of_request(3, 0) != P.seed_of_request(3, 1) != P.seed_of_request(4, 1)
    dist = torch.tensor([0.0, 0.25, 0.0, 0.5, 0.25, 0.0])
    assert [P.inverse_cdf(dist, u)[0] for u in (0.0, 0.2, 0.25, 0.7, 0.75, 0.999)] == [1, 1, 3, 3, 4, 4]
    assert abs(P.inverse_cdf(dist, 0.3)[1] - 0.05) < 1e-9


def test_sampling_distribution():
    logits = torch.tensor([1.0, 3.0, 2.0, 3.0, -1.0])
    p = P.sampling_distribution(logits, 0.5, 2)
    # ties at the threshold survive (fms/utils/generation.py:322-323)
    torch.testing.assert_close(p, torch.tensor([0.0, 0.5, 0.0, 0.5, 0.0]))
    p = P.sampling_distribution(logits, 2.0, 0)
    torch.testing.assert_close(p, torch.softmax(logits / 2.0, -1))
    assert P.greedy(torch.tensor([0.1, 0.7, 0.3])) == 1
