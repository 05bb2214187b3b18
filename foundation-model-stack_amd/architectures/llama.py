"""Llama: from its configuration to parts, and from checkpoint sources to its tensor names.

The model is the reference's (fms/models/llama.py): token embedding, `nlayers`
pre-norm blocks of grouped-query attention with rotary positions and a SwiGLU
feed-forward, a final RMSNorm and a linear head, optionally tied to the embedding.
Parameter names are the reference's, with fused qkv and fused gate/up
(tests/resources/expectations/models.test_llama.TestLlama2.test_model_weight_keys).
"""

from __future__ import annotations

import re
from typing import List, Tuple

from ..config import LLaMAConfig
from ..config.llama import HF_ARCHITECTURES
from ..parts import LayerSpec, ModelSpec, PartSpec
from ..weights.adapters import (
    fuse_attention_step,
    fuse_glu_step,
    register_adapter,
    register_adapter_step,
    rename_step,
)
from .registry import Architecture, register_architecture, register_model

NAME = "llama"


def llama_spec(config: LLaMAConfig) -> ModelSpec:
    """Which parts a Llama of this configuration is made of (fms/models/llama.py:65-116, 170-216)."""
    norm = PartSpec("rmsnorm", {"eps": config.norm_eps})
    layer = LayerSpec(
        mixer=PartSpec(
            "attention",
            {
                "nheads": config.nheads,
                "kvheads": config.kv_heads,
                "head_dim": config.head_dim,
                "use_bias": config.attn_bias,
            },
        ),
        feed_forward=PartSpec(
            "glu",
            {"hidden_dim": config.ffn_hidden_dim, "activation": config.activation_fn, "use_bias": config.mlp_bias},
        ),
        norm=norm,
        block=PartSpec("pre_norm"),
        position="rope",
    )
    return ModelSpec(
        vocab=config.src_vocab_size,
        width=config.emb_dim,
        max_seq_len=config.max_positions,
        layers=[layer for _ in range(config.nlayers)],
        final_norm=norm,
        positions={
            "rope": PartSpec(
                "rope",
                {
                    "dim": config.head_dim,
                    "theta": config.rope_theta,
                    "max_seq_len": config.max_expected_seq_len,
                    "max_positions": config.max_positions,
                    "scaling": dict(config.rope_scaling or {}),
                },
            )
        },
        tie_heads=config.tie_heads,
    )


# ---- checkpoint sources ---------------------------------------------------------
# fms/models/llama.py:618-645
_META_NAMES = [
    (r"^tok_embeddings", "base_model.embedding"),
    (r"^norm", "base_model.dec_norm"),
    (r"^output", "head"),
    (r"^layers", "base_model.layers"),
    (r"\.attention\.", ".attn."),
    (r"attn\.wq", "attn.in_proj.query"),
    (r"attn\.wk", "attn.in_proj.key"),
    (r"attn\.wv", "attn.in_proj.value"),
    (r"attn\.wo", "attn.dense"),
    (r"attention_norm", "ln"),
    (r"feed_forward\.w1", "ff_sub_layer.wg"),
    (r"feed_forward\.w2", "ff_sub_layer.w2"),
    (r"feed_forward\.w3", "ff_sub_layer.w1"),
    (r"ffn_norm", "ff_ln"),
]
# fms/models/llama.py:648-673
_HF_NAMES = [
    (r"^lm_head.weight", "head.weight"),
    (r"^model.embed_tokens.weight", "base_model.embedding.weight"),
    (r"^model.norm", "base_model.dec_norm"),
    (r"^model.layers", "base_model.layers"),
    (r"self_attn\.k_proj", "attn.in_proj.key"),
    (r"self_attn\.v_proj", "attn.in_proj.value"),
    (r"self_attn\.q_proj", "attn.in_proj.query"),
    (r"self_attn\.o_proj", "attn.dense"),
    (r"mlp\.gate_proj", "ff_sub_layer.wg"),
    (r"mlp\.up_proj", "ff_sub_layer.w1"),
    (r"mlp\.down_proj", "ff_sub_layer.w2"),
    (r"input_layernorm", "ln"),
    (r"post_attention_layernorm", "ff_ln"),
]

_ROPE_ROWS = re.compile(r"base_model\.layers\.[0-9]+\.attn\.in_proj\.(query|key)\.(weight|bias)$")


def _hf_rope_rows(sd, model_config=None, **kw):
    """Hugging Face keeps each head's query/key rows as [first halves; second halves] of the
    rotary pairs; the model rotates adjacent pairs, so row j*D/2+i of a head moves to row 2i+j
    (fms/models/llama.py:685-748)."""
    head = model_config.head_dim
    out = {}
    for name, t in sd.items():
        if _ROPE_ROWS.match(name) and t.shape[0] > 1:
            heads = t.shape[0] // head
            if t.dim() == 2:
                t = t.reshape(heads, 2, head // 2, t.shape[1]).transpose(1, 2).reshape(t.shape)
            else:
                t = t.reshape(heads, 2, head // 2).transpose(1, 2).reshape(t.shape)
        out[name] = t
    return out


def _fuse(sd, **kw):
    return fuse_glu_step(fuse_attention_step(sd))


register_adapter_step(NAME, "meta_to_fms_names", rename_step(_META_NAMES))
register_adapter_step(NAME, "hf_to_fms_names", rename_step(_HF_NAMES))
register_adapter_step(NAME, "hf_to_fms_rope", _hf_rope_rows)
register_adapter_step(NAME, "weight_fusion", _fuse)
# fms/models/llama.py:750-760
register_adapter(NAME, "meta", ["meta_to_fms_names", "weight_fusion"])
register_adapter(NAME, "hf", ["hf_to_fms_names", "hf_to_fms_rope", "weight_fusion"])
register_adapter(NAME, "fms_unfused", ["weight_fusion"])


def _pre006_attention_names(sd, **kw):
    """Checkpoints written before the reference's 0.0.6 name the projections attn.query/key/value, without
    "in_proj" (fms/utils/serialization.py:164-170, 182-227 with attn_prefix="attn")."""
    pattern = re.compile(r"\.attn\.(query|key|value)\.(weight|bias)$")
    return {pattern.sub(r".attn.in_proj.\1.\2", name): t for name, t in sd.items()}


register_adapter_step(NAME, "pre0.0.6_attn_unfused_to_fused", lambda sd, **kw: fuse_attention_step(_pre006_attention_names(sd)))
register_adapter_step(NAME, "swiglu_unfused_to_fused", fuse_glu_step)
# fms/models/llama.py:761-765
register_adapter(NAME, "fms.pre0.0.6", ["pre0.0.6_attn_unfused_to_fused", "swiglu_unfused_to_fused", "weight_fusion"])


def detect_source(names: List[str]) -> str:
    """Which source a checkpoint's tensor names come from."""
    if any(n.startswith("model.layers.") or n.startswith("model.embed_tokens") for n in names):
        return "hf"
    if any(n.startswith("tok_embeddings") or ".attention.wq" in n for n in names):
        return "meta"
    if any(re.search(r"\.attn\.(query|key|value)\.", n) for n in names):
        return "fms.pre0.0.6"
    if any(".in_proj.query." in n or ".ff_sub_layer.wg." in n for n in names):
        return "fms_unfused"
    return "fms"


def hf_tensor_layout(config: LLaMAConfig) -> List[Tuple[str, Tuple[int, ...], str]]:
    """(name, shape, init) of every tensor of a Hugging Face Llama checkpoint of this configuration."""
    E, H, K, D, F, V = (config.emb_dim, config.nheads, config.kv_heads, config.head_dim, config.ffn_hidden_dim,
                        config.src_vocab_size)
    out = [("model.embed_tokens.weight", (V, E), "normal")]
    for i in range(config.nlayers):
        p = f"model.layers.{i}."
        out += [
            (p + "input_layernorm.weight", (E,), "ones"),
            (p + "self_attn.q_proj.weight", (H * D, E), "normal"),
            (p + "self_attn.k_proj.weight", (K * D, E), "normal"),
            (p + "self_attn.v_proj.weight", (K * D, E), "normal"),
            (p + "self_attn.o_proj.weight", (E, H * D), "normal"),
            (p + "post_attention_layernorm.weight", (E,), "ones"),
            (p + "mlp.gate_proj.weight", (F, E), "normal"),
            (p + "mlp.up_proj.weight", (F, E), "normal"),
            (p + "mlp.down_proj.weight", (E, F), "normal"),
        ]
        if config.attn_bias:
            out += [
                (p + "self_attn.q_proj.bias", (H * D,), "normal"),
                (p + "self_attn.k_proj.bias", (K * D,), "normal"),
                (p + "self_attn.v_proj.bias", (K * D,), "normal"),
                (p + "self_attn.o_proj.bias", (E,), "normal"),
            ]
        if config.mlp_bias:
            out += [
                (p + "mlp.gate_proj.bias", (F,), "normal"),
                (p + "mlp.up_proj.bias", (F,), "normal"),
                (p + "mlp.down_proj.bias", (E,), "normal"),
            ]
    out.append(("model.norm.weight", (E,), "ones"))
    if not config.tie_heads:
        out.append(("lm_head.weight", (V, E), "normal"))
    return out


register_architecture(
    Architecture(
        name=NAME,
        config_class=LLaMAConfig,
        build_spec=llama_spec,
        hf_architectures=HF_ARCHITECTURES,
        from_hf_dict=LLaMAConfig.from_hf_dict,
        to_hf_dict=LLaMAConfig.to_hf_dict,
        hf_tensor_layout=hf_tensor_layout,
        detect_source=detect_source,
    )
)


# ---- variants (fms/models/llama.py:456-561) -------------------------------------------
def _variant(config: LLaMAConfig):
    def factory(**overrides) -> LLaMAConfig:
        return config.updated(**overrides)

    return factory


_7b = LLaMAConfig()
_13b = LLaMAConfig(emb_dim=5120, nheads=40, nlayers=40)
_70b = LLaMAConfig(emb_dim=8192, multiple_of=4096, nheads=64, kvheads=8, nlayers=80, hidden_grow_factor=(1.3 * 8 / 3))
_3_8b = LLaMAConfig(src_vocab_size=128256, emb_dim=4096, norm_eps=1e-5, nheads=32, kvheads=8, nlayers=32,
                    hidden_grow_factor=3.5, multiple_of=1024, max_expected_seq_len=8192, rope_theta=500_000.0)
_3_70b = LLaMAConfig(src_vocab_size=128256, emb_dim=8192, multiple_of=4096, nheads=64, kvheads=8, nlayers=80,
                     hidden_grow_factor=(1.3 * 8 / 3), max_expected_seq_len=8192, rope_theta=500_000.0)

register_model(NAME, "micro", _variant(LLaMAConfig(emb_dim=192, nheads=4, nlayers=5, max_expected_seq_len=1024, src_vocab_size=256)))
for _name, _cfg in (("7b", _7b), ("13b", _13b), ("70b", _70b), ("2-7b", _7b), ("2-13b", _13b), ("2-70b", _70b),
                    ("3-8b", _3_8b), ("3-70b", _3_70b)):
    register_model(NAME, _name, _variant(_cfg))
register_model(NAME, "granite-7b", _variant(LLaMAConfig(src_vocab_size=32008)))
register_model(NAME, "granite.code-3b", _variant(LLaMAConfig(
    src_vocab_size=49152, emb_dim=2560, pad_id=0, hidden_grow_factor=10240 / 2560, multiple_of=1,
    max_expected_seq_len=2048, attn_bias=True, mlp_bias=True, tie_heads=True)))
register_model(NAME, "granite.code-8b", _variant(LLaMAConfig(
    src_vocab_size=49152, emb_dim=4096, kvheads=8, nlayers=36, pad_id=0, hidden_grow_factor=14336 / 4096, multiple_of=1,
    max_expected_seq_len=4096, attn_bias=True, mlp_bias=True, tie_heads=True)))
