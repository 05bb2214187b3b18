"""A plain, slow Llama written from the reference's formulas.

Whole sequences, no cache, one function for each part, float32 torch tensor
ops on the CPU.  Nothing here imports the product package: this file is the
yardstick the engine is measured with, so it shares no code with it.  Every
function cites the lines of the reference (paths relative to the reference
checkout) that fix its arithmetic.

Weights are a dict from the reference's own tensor names
(``base_model.layers.0.attn.in_proj.qkv_fused.weight`` ...) to float32 tensors.
"""

from __future__ import annotations

import json
import math
import os
import struct
from dataclasses import dataclass, field
from typing import Dict, List, Optional

import torch


@dataclass
class PlainConfig:
    """The numbers of one Llama (fms/models/llama.py:42-62), already resolved."""

    vocab: int
    width: int
    nheads: int
    kvheads: int
    nlayers: int
    hidden: int
    eps: float
    theta: float
    max_len: int
    tie_heads: bool = False
    attn_bias: bool = False
    mlp_bias: bool = False
    rope_scaling: dict = field(default_factory=dict)
    activation: str = "swish"  # activation_fn (fms/models/llama.py:51)

    @property
    def head_dim(self) -> int:
        # fms/models/llama.py:69-70: head size is emb_dim // nheads
        return self.width // self.nheads


def glu_hidden(width: int, grow: float, multiple_of: Optional[int]) -> int:
    """fms/modules/feedforward.py:227-233: int(grow*width) rounded up to multiple_of."""
    hidden = int(grow * width)
    if multiple_of:
        hidden = multiple_of * ((hidden + multiple_of - 1) // multiple_of)
    return hidden


# ----------------------------------------------------------------------------
# parts
# ----------------------------------------------------------------------------


def embedding(table: torch.Tensor, ids: torch.Tensor) -> torch.Tensor:
    """fms/models/llama.py:332: a row of the table per token id, no scale."""
    return table[ids]


def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """fms/modules/layernorm.py:56-69 with use_mean=False, scale only.

    x * rsqrt(mean(x^2) + eps) (eps inside the root), then times the weight.
    """
    xf = x.float()
    xf = xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps)
    return weight.float() * xf


def linear(x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor] = None) -> torch.Tensor:
    """nn.Linear as the reference uses it (fms/modules/linear.py:254-255): x @ W^T + b."""
    y = x @ weight.t()
    if bias is not None:
        y = y + bias
    return y


def ntk_alpha(length: int, original_length: int) -> int:
    """fms/modules/positions.py:146-156: ceil(length / original), rounded up to a power of two."""
    alpha = math.ceil(length / original_length)
    return int(2 ** math.ceil(math.log(alpha) / math.log(2)))


def rope_frequencies(head_dim: int, theta: float, scaling: Optional[dict] = None, length: int = 0, max_len: int = 0) -> torch.Tensor:
    """fms/modules/positions.py:124-132 (no scaling), :171-196 (llama3 scaling) and :135-168 (ntk scaling: for a
    call whose longest sequence has `length` tokens, theta times alpha^(D / (D - 2)) with the power of two
    alpha that stretches the table's `max_len` positions over it; alpha 1 for shorter calls)."""
    scaling = scaling or {}
    kind = scaling.get("rope_type", "regular")
    if kind == "ntk":
        alpha = ntk_alpha(max(length, 1), max_len)
        theta = theta * alpha ** (head_dim / (head_dim - 2))
    freqs = 1.0 / (theta ** (torch.arange(0, head_dim, 2)[: head_dim // 2].float() / head_dim))
    if kind in ("regular", "ntk"):
        return freqs
    if kind != "llama3":
        raise ValueError(f"plain implementation has no rope_type {kind!r}")
    factor = scaling["factor"]
    low = scaling["low_freq_factor"]
    high = scaling["high_freq_factor"]
    old_len = scaling["original_max_position_embeddings"]
    low_wavelen = old_len / low
    high_wavelen = old_len / high
    wavelen = 2 * math.pi / freqs
    scaled = torch.where(wavelen > low_wavelen, freqs / factor, freqs)
    smooth = (old_len / wavelen - low) / (high - low)
    smoothed = (1 - smooth) * scaled / factor + smooth * scaled
    medium = ~(wavelen < high_wavelen) * ~(wavelen > low_wavelen)
    return torch.where(medium, smoothed, scaled)


def rope_rotate(x: torch.Tensor, positions: torch.Tensor, freqs: torch.Tensor) -> torch.Tensor:
    """fms/modules/positions.py:334-355, 439-456: rotate adjacent pairs.

    x is [S, heads, D]; pair i is (x[2i], x[2i+1]); angle = position * freqs[i];
    out[2i] = cos*x[2i] - sin*x[2i+1], out[2i+1] = sin*x[2i] + cos*x[2i+1].
    """
    # freqs [D/2], or [S, D/2] when the positions were rotated by different calls (ntk scaling with a cache)
    angles = (torch.outer(positions.float(), freqs) if freqs.dim() == 1 else positions.float()[:, None] * freqs).float()
    cos = torch.cos(angles)[:, None, :]
    sin = torch.sin(angles)[:, None, :]
    pairs = x.float().reshape(*x.shape[:-1], -1, 2)
    even, odd = pairs[..., 0], pairs[..., 1]
    out = torch.stack((cos * even - sin * odd, sin * even + cos * odd), dim=-1)
    return out.reshape(x.shape)


def causal_attention(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    scale: Optional[float] = None,
    window: int = 0,
) -> torch.Tensor:
    """fms/modules/attention.py:215-294 with the causal mask of a whole sequence.

    q is [S, H, D], k and v are [S, K, D].  Query head h reads kv head h // (H/K)
    (:241-250: unsqueeze(2).expand(G).flatten(1,2)); scores are scaled by
    1/sqrt(D) (:274-282 with scale=None); key j is visible to query i iff j <= i
    (and, with a window w > 0, i - j < w).  Returns [S, H, D].
    """
    S, H, D = q.shape
    K = k.shape[1]
    group = H // K
    if scale is None:
        scale = 1.0 / math.sqrt(D)
    out = torch.empty(S, H, v.shape[-1], dtype=torch.float32)
    idx = torch.arange(S)
    visible = idx[None, :] <= idx[:, None]
    if window:
        visible = visible & (idx[:, None] - idx[None, :] < window)
    for h in range(H):
        kh = h // group
        scores = (q[:, h, :].float() @ k[:, kh, :].float().t()) * scale
        scores = scores.masked_fill(~visible, float("-inf"))
        probs = torch.softmax(scores, dim=-1)
        out[:, h, :] = probs @ v[:, kh, :].float()
    return out


def silu(x: torch.Tensor) -> torch.Tensor:
    """fms/utils/activation.py: "swish" is nn.SiLU: x * sigmoid(x)."""
    return x * torch.sigmoid(x)


def activation(name: str):
    """fms/utils/activation.py:14-24, 47-50: the activation functions by name (case ignored); "gelu" is the one
    with the error function, the two "gelu...tanh" names its tanh approximation."""
    table = {
        "swish": silu,
        "silu": silu,
        "gelu": lambda x: 0.5 * x * (1.0 + torch.erf(x / math.sqrt(2.0))),
        "gelu-tanh": lambda x: 0.5 * x * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (x + 0.044715 * x**3))),
        "mish": lambda x: x * torch.tanh(torch.nn.functional.softplus(x)),
        "relu": lambda x: torch.clamp(x, min=0.0),
        "sigmoid": torch.sigmoid,
        "tanh": torch.tanh,
    }
    table["gelu_pytorch_tanh"] = table["gelu-tanh"]
    return table[name.lower()]


def gated_feed_forward(
    x: torch.Tensor,
    wg1_fused: torch.Tensor,
    w2: torch.Tensor,
    bias_fused: Optional[torch.Tensor] = None,
    bias2: Optional[torch.Tensor] = None,
    storage=None,
    rounding: str = "stored",
    act_name: str = "swish",
) -> torch.Tensor:
    """fms/modules/feedforward.py:288-297: first half of the fused rows is the gate.

    rounding "reference": the activation and the product are two operations of the model dtype there
    (self.a(out1) * out2), so each of them rounds."""
    st = _stored(storage)
    hidden = wg1_fused.shape[0] // 2
    both = st(linear(x, wg1_fused, bias_fused))
    gate, up = both[..., :hidden], both[..., hidden:]
    fn = activation(act_name)
    act = st(fn(gate)) if rounding == "reference" else fn(gate)
    return linear(st(act * up), w2, bias2)


def rms_norm_as_stored(x: torch.Tensor, weight: torch.Tensor, eps: float, storage) -> torch.Tensor:
    """fms/modules/layernorm.py:60-66 in a model dtype below float32: the statistics and the scaling are
    float32, the scaled row is cast to the model dtype (`.type_as(x)`), and only then multiplied by the
    weight, in the model dtype: two roundings."""
    st = _stored(storage)
    xf = x.float()
    xf = st(xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps))
    return st(st(weight.float()) * xf)


def _stored(storage):
    """Rounding to the type in which the reference would hold a tensor (identity for float32)."""
    if storage is None or storage == torch.float32:
        return lambda t: t
    return lambda t: t.to(storage).float()


def attention_block(
    x: torch.Tensor,
    positions: torch.Tensor,
    cfg: PlainConfig,
    qkv_w: torch.Tensor,
    dense_w: torch.Tensor,
    freqs: torch.Tensor,
    qkv_b: Optional[torch.Tensor] = None,
    dense_b: Optional[torch.Tensor] = None,
    storage=None,
) -> torch.Tensor:
    """fms/modules/attention.py:870-937: project, split [H*D, K*D, K*D], rotate q and k, attend, project."""
    st = _stored(storage)
    S = x.shape[0]
    H, K, D = cfg.nheads, cfg.kvheads, cfg.head_dim
    qkv = st(linear(x, qkv_w, qkv_b))
    q, k, v = torch.split(qkv, [H * D, K * D, K * D], dim=-1)
    q = st(rope_rotate(q.reshape(S, H, D), positions, freqs))
    k = st(rope_rotate(k.reshape(S, K, D), positions, freqs))
    v = v.reshape(S, K, D)
    mixed = st(causal_attention(q, k, v))
    return st(linear(mixed.reshape(S, H * D), dense_w, dense_b))


def rotated_queries_and_keys(weights: Dict[str, torch.Tensor], cfg: PlainConfig, ids: List[int], layer: int = 0):
    """Queries [S, H, D] and keys [S, K, D] of the first layer after the rotation (tests use them to see how
    sharp a model's attention is); only layer 0 can be had without running the layers before it."""
    if layer != 0:
        raise ValueError("only the first layer's queries and keys depend on nothing but the embedding")
    w = {name: t.float() for name, t in weights.items()}
    S, H, K, D = len(ids), cfg.nheads, cfg.kvheads, cfg.head_dim
    p = "base_model.layers.0."
    x = embedding(w["base_model.embedding.weight"], torch.as_tensor(ids, dtype=torch.long))
    h = rms_norm(x, w[p + "ln.weight"], cfg.eps)
    qkv = linear(h, w[p + "attn.in_proj.qkv_fused.weight"], w.get(p + "attn.in_proj.qkv_fused.bias"))
    q, k, _ = torch.split(qkv, [H * D, K * D, K * D], dim=-1)
    freqs = rope_frequencies(D, cfg.theta, cfg.rope_scaling)
    positions = torch.arange(S)
    return rope_rotate(q.reshape(S, H, D), positions, freqs), rope_rotate(k.reshape(S, K, D), positions, freqs)


def forward(
    weights: Dict[str, torch.Tensor],
    cfg: PlainConfig,
    ids: List[int],
    first_position: int = 0,
    storage=None,
    rounding: str = "stored",
    calls: Optional[List[tuple]] = None,
) -> torch.Tensor:
    """fms/models/llama.py:137-162, 332-353, 444-445: logits [S, V] of one whole sequence.

    calls (ntk scaling only): the sequence as a cache holds it after it was fed in several calls,
    [(tokens of the call, longest sequence of the call's batch after it), ...].  fms/modules/positions.py:394-421:
    a call rotates its queries and its new keys with the frequencies of alpha(max_start_pos + seq_len), and the
    keys that earlier calls cached keep the rotation they got (fms/modules/attention.py:877-898: rotated before they
    are stored).  Row p of the result is what the call that fed token p returned for it.

    storage=torch.bfloat16 sizes the error of running in bfloat16; `rounding` says where it rounds.
    "stored": every tensor that is stored between two operations (the outputs of norms, linears, rotation,
    attention and the gate product) is rounded once; the residual stream, the norm's multiplication by its
    weight and the logits stay float32.  "reference": the roundings of the reference run in that dtype:
    besides the above, the norm rounds before and after its weight (layernorm.py:60-66), the residual sums
    are sums of the model dtype (llama.py:153, 162), the embedding row and the activation round, and the
    logits leave the head in the model dtype (llama.py:445).  Norm statistics and the rotation are float32
    in both, as in the reference.
    """
    if rounding not in ("stored", "reference"):
        raise ValueError(rounding)
    st = _stored(storage)
    ref = rounding == "reference"
    rs = st if ref else (lambda t: t)  # roundings that only the reference's arithmetic has
    norm = (lambda x, w_: rms_norm_as_stored(x, w_, cfg.eps, storage)) if ref else (lambda x, w_: st(rms_norm(x, w_, cfg.eps)))
    w = {name: t.float() for name, t in weights.items()}
    tokens = torch.as_tensor(ids, dtype=torch.long)
    positions = torch.arange(len(ids)) + first_position
    stretches = (cfg.rope_scaling or {}).get("rope_type") == "ntk"
    if int(positions[-1]) >= cfg.max_len and not stretches:
        # tests/modules/test_positions.py:156-168: a position beyond the table raises
        raise IndexError("position beyond max_expected_seq_len")
    freqs = rope_frequencies(cfg.head_dim, cfg.theta, cfg.rope_scaling, int(positions[-1]) + 1, cfg.max_len)
    if calls is not None:
        if sum(n for n, _ in calls) != len(ids) or first_position:
            raise ValueError("the calls must cover the sequence from its first token")
        freqs = torch.cat([rope_frequencies(cfg.head_dim, cfg.theta, cfg.rope_scaling, longest, cfg.max_len)[None].expand(n, -1)
                           for n, longest in calls])
    x = rs(embedding(w["base_model.embedding.weight"], tokens))
    for i in range(cfg.nlayers):
        p = f"base_model.layers.{i}."
        residual = x
        h = norm(x, w[p + "ln.weight"])
        h = attention_block(
            h,
            positions,
            cfg,
            w[p + "attn.in_proj.qkv_fused.weight"],
            w[p + "attn.dense.weight"],
            freqs,
            w.get(p + "attn.in_proj.qkv_fused.bias"),
            w.get(p + "attn.dense.bias"),
            storage,
        )
        x = rs(h + residual)
        residual = x
        h = norm(x, w[p + "ff_ln.weight"])
        h = st(gated_feed_forward(
            h,
            w[p + "ff_sub_layer.wg1_fused.weight"],
            w[p + "ff_sub_layer.w2.weight"],
            w.get(p + "ff_sub_layer.wg1_fused.bias"),
            w.get(p + "ff_sub_layer.w2.bias"),
            storage,
            rounding,
            cfg.activation,
        ))
        x = rs(h + residual)
    x = norm(x, w["base_model.dec_norm.weight"])
    head = w["base_model.embedding.weight"] if cfg.tie_heads and "head.weight" not in w else w["head.weight"]
    return rs(linear(x, head))


# ----------------------------------------------------------------------------
# sampling (fms/utils/generation.py:316-328)
# ----------------------------------------------------------------------------


def greedy(logits: torch.Tensor) -> int:
    """fms/utils/generation.py:328: argmax."""
    return int(torch.argmax(logits.float()))


def sampling_distribution(logits: torch.Tensor, temperature: float, top_k: int) -> torch.Tensor:
    """fms/utils/generation.py:318-326: logits/T, keep those >= the k-th largest, softmax."""
    scaled = logits.float() / temperature
    if top_k:
        kth = torch.topk(scaled, min(top_k, scaled.numel())).values[-1]
        scaled = scaled.masked_fill(scaled < kth, float("-inf"))
    return torch.softmax(scaled, dim=-1)


# The seeded draw has no counterpart in the reference (its torch.multinomial takes the global generator,
# fms/utils/generation.py:326); what follows states this library's definition a second time, on its own: the
# uniform number of a request's n-th draw is splitmix64 of (request seed + (n + 1) * the golden-ratio constant),
# its top 24 bits; the request seed is two rounds of the same mixing over (call seed, request index); and the
# token is the first index at which the cumulative distribution passes the number.
_M64 = (1 << 64) - 1


def _splitmix_finish(z: int) -> int:
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & _M64
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & _M64
    return z ^ (z >> 31)


def draw_uniform(request_seed: int, n_drawn: int) -> float:
    return (_splitmix_finish((request_seed + (n_drawn + 1) * 0x9E3779B97F4A7C15) & _M64) >> 40) / float(1 << 24)


def seed_of_request(call_seed: int, request_index: int) -> int:
    return _splitmix_finish((_splitmix_finish(call_seed & _M64) + 0xD1342543DE82EF95 * (request_index + 1)) & _M64) >> 1


def inverse_cdf(dist: torch.Tensor, u: float):
    """(token, distance of u from the nearest edge of the token's interval): the first index whose cumulative
    probability exceeds u."""
    cdf = torch.cumsum(dist.double(), 0)
    tok = int(torch.searchsorted(cdf, torch.tensor(u, dtype=torch.float64), right=True).clamp(max=dist.numel() - 1))
    while dist[tok] == 0 and tok > 0:  # u at the very end, beyond rounding: the last token with mass
        tok -= 1
    lo = float(cdf[tok] - dist[tok].double())
    return tok, min(u - lo, float(cdf[tok]) - u)


def greedy_generate(weights, cfg: PlainConfig, prompt: List[int], n_new: int, stop: Optional[int] = None) -> List[int]:
    """fms/utils/generation.py:287-346 for one row, greedy, recomputing the whole sequence each step."""
    ids = list(prompt)
    new: List[int] = []
    for _ in range(n_new):
        tok = greedy(forward(weights, cfg, ids)[-1])
        ids.append(tok)
        new.append(tok)
        if stop is not None and tok == stop:
            break
    return new


# ----------------------------------------------------------------------------
# reading a model folder written in the Hugging Face layout
# ----------------------------------------------------------------------------

_ST_DTYPES = {"F32": torch.float32, "BF16": torch.bfloat16, "F16": torch.float16, "I32": torch.int32, "I64": torch.int64}


def read_safetensors(path: str) -> Dict[str, torch.Tensor]:
    """Own reader of the safetensors layout: u64 header length, JSON header, raw little-endian data."""
    with open(path, "rb") as f:
        (n,) = struct.unpack("<Q", f.read(8))
        header = json.loads(f.read(n))
        data = f.read()
    out = {}
    for name, meta in header.items():
        if name == "__metadata__":
            continue
        lo, hi = meta["data_offsets"]
        t = torch.frombuffer(bytearray(data[lo:hi]), dtype=_ST_DTYPES[meta["dtype"]])
        out[name] = t.reshape(meta["shape"]).clone()
    return out


def config_from_hf(cfg: dict) -> PlainConfig:
    """fms/models/hf/config_utils/param_builders.py:37-58, 512-546: the config.json keys that are read."""
    rope_theta = cfg.get("rope_theta")
    rope_scaling = cfg.get("rope_scaling")
    if cfg.get("rope_parameters") is not None:
        rope_theta = cfg["rope_parameters"]["rope_theta"]
        rope_scaling = cfg["rope_parameters"].get("rope_scaling")
    return PlainConfig(
        vocab=cfg["vocab_size"],
        width=cfg["hidden_size"],
        nheads=cfg["num_attention_heads"],
        kvheads=cfg["num_key_value_heads"] or cfg["num_attention_heads"],
        nlayers=cfg["num_hidden_layers"],
        hidden=cfg["intermediate_size"],
        eps=cfg["rms_norm_eps"],
        theta=10000.0 if rope_theta is None else rope_theta,
        max_len=cfg["max_position_embeddings"],
        tie_heads=bool(cfg.get("tie_word_embeddings", False)),
        attn_bias=bool(cfg.get("attention_bias", False)),
        mlp_bias=bool(cfg.get("mlp_bias", False)),
        rope_scaling=rope_scaling or {},
        # the reference's builder does not read hidden_act (its models keep activation_fn's default); a folder that
        # names another function is run with that one here
        activation=cfg.get("hidden_act", "silu"),
    )


def _halves_to_pairs(t: torch.Tensor, head_dim: int) -> torch.Tensor:
    """fms/models/llama.py:711-748: per head, row j*D/2+i of the HF layout becomes row 2i+j."""
    heads = t.shape[0] // head_dim
    if t.dim() == 2:
        return t.reshape(heads, 2, head_dim // 2, t.shape[1]).transpose(1, 2).reshape(t.shape)
    return t.reshape(heads, 2, head_dim // 2).transpose(1, 2).reshape(t.shape)


def hf_to_reference_names(hf: Dict[str, torch.Tensor], cfg: PlainConfig) -> Dict[str, torch.Tensor]:
    """fms/models/llama.py:648-673 (names), :685-748 (q/k rows), fms/utils/serialization.py:173-270 (fusion)."""
    out: Dict[str, torch.Tensor] = {}
    out["base_model.embedding.weight"] = hf["model.embed_tokens.weight"]
    out["base_model.dec_norm.weight"] = hf["model.norm.weight"]
    if "lm_head.weight" in hf:
        out["head.weight"] = hf["lm_head.weight"]
    D = cfg.head_dim
    for i in range(cfg.nlayers):
        src = f"model.layers.{i}."
        dst = f"base_model.layers.{i}."
        for kind in ("weight", "bias"):
            if f"{src}self_attn.q_proj.{kind}" not in hf:
                continue
            q = _halves_to_pairs(hf[f"{src}self_attn.q_proj.{kind}"], D)
            k = _halves_to_pairs(hf[f"{src}self_attn.k_proj.{kind}"], D)
            v = hf[f"{src}self_attn.v_proj.{kind}"]
            out[f"{dst}attn.in_proj.qkv_fused.{kind}"] = torch.cat([q, k, v], dim=0)
            out[f"{dst}attn.dense.{kind}"] = hf[f"{src}self_attn.o_proj.{kind}"]
            if f"{src}mlp.gate_proj.{kind}" in hf:
                out[f"{dst}ff_sub_layer.wg1_fused.{kind}"] = torch.cat(
                    [hf[f"{src}mlp.gate_proj.{kind}"], hf[f"{src}mlp.up_proj.{kind}"]], dim=0
                )
                out[f"{dst}ff_sub_layer.w2.{kind}"] = hf[f"{src}mlp.down_proj.{kind}"]
        out[f"{dst}ln.weight"] = hf[f"{src}input_layernorm.weight"]
        out[f"{dst}ff_ln.weight"] = hf[f"{src}post_attention_layernorm.weight"]
    return out


def load_model_folder(folder: str):
    """config.json + model.safetensors in the Hugging Face layout -> (PlainConfig, reference-named float32 weights)."""
    with open(os.path.join(folder, "config.json")) as f:
        cfg = config_from_hf(json.load(f))
    hf = read_safetensors(os.path.join(folder, "model.safetensors"))
    weights = {k: v.float() for k, v in hf_to_reference_names(hf, cfg).items()}
    return cfg, weights


def rope_rotate_halves(x: torch.Tensor, positions: torch.Tensor, freqs: torch.Tensor) -> torch.Tensor:
    """The other pairing (fms/modules/positions.py:255-258; fms/models/llama.py:711-721):
    pair i is (x[i], x[i + D/2]).  Used only to pin the row permutation above."""
    angles = torch.outer(positions.float(), freqs).float()
    cos = torch.cos(angles)[:, None, :]
    sin = torch.sin(angles)[:, None, :]
    x1, x2 = torch.chunk(x.float(), 2, dim=-1)
    return torch.cat((x1 * cos - x2 * sin, x2 * cos + x1 * sin), dim=-1)
