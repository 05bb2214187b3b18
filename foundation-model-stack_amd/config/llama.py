"""The Llama configuration: the reference's field names, defaults and derived sizes.

Fields and defaults are those of ``LLaMAConfig`` (fms/models/llama.py:42-62).
``from_hf_dict`` reads the keys of a Hugging Face ``config.json`` the way the
reference's parameter builder does (fms/models/hf/config_utils/param_builders.py:18-58,
512-546), except that the feed-forward width is carried as the integer that
config.json gives instead of being rebuilt from a float ratio, and that keys
the reference silently ignores are not: ``head_dim`` is checked and ``hidden_act``
becomes ``activation_fn``.
"""

from __future__ import annotations

import dataclasses
from typing import Optional

from .base import ModelConfig

HF_ARCHITECTURES = ("LlamaForCausalLM",)
# the activation functions the reference knows by name (fms/utils/activation.py:14-24)
ACTIVATION_NAMES = ("swish", "silu", "gelu", "gelu-tanh", "gelu_pytorch_tanh", "mish", "relu", "sigmoid", "tanh")


@dataclasses.dataclass
class LLaMAConfig(ModelConfig):
    src_vocab_size: int = 32_000
    emb_dim: int = 4096
    norm_eps: float = 1e-5
    nheads: int = 32
    kvheads: int = 0
    nlayers: int = 32
    pad_id: int = -1
    hidden_grow_factor: float = 8 / 3
    multiple_of: int = 256
    activation_fn: str = "swish"
    p_dropout: float = 0.0
    max_expected_seq_len: int = 4096
    attn_bias: bool = False
    mlp_bias: bool = False
    tie_heads: bool = False
    rope_theta: float = 10_000.0
    rope_scaling: dict = dataclasses.field(default_factory=dict)
    fused_weights: bool = True
    # The feed-forward width as an integer.  When set it wins over
    # hidden_grow_factor/multiple_of: int(ratio * emb_dim) can land one below
    # the intended width for ratios that came from a division.
    hidden_dim: Optional[int] = None

    def __post_init__(self):
        self.validate()

    # ---- derived sizes -------------------------------------------------
    @property
    def head_dim(self) -> int:
        """fms/models/llama.py:69-70: emb_dim // nheads."""
        return self.emb_dim // self.nheads

    @property
    def kv_heads(self) -> int:
        """fms/models/llama.py:89-93: 0 means as many as query heads."""
        return self.nheads if self.kvheads == 0 else self.kvheads

    @property
    def ffn_hidden_dim(self) -> int:
        """fms/modules/feedforward.py:227-233."""
        if self.hidden_dim is not None:
            return int(self.hidden_dim)
        hidden = int(self.hidden_grow_factor * self.emb_dim)
        if self.multiple_of:
            hidden = self.multiple_of * ((hidden + self.multiple_of - 1) // self.multiple_of)
        return hidden

    @property
    def max_positions(self) -> int:
        """The most tokens a sequence may hold.  max_expected_seq_len, except with "ntk" scaling, which stretches
        the rotation for longer sequences (fms/modules/positions.py:135-168): the reference sets no end to that,
        here a sequence may grow to rope_scaling["factor"] times max_expected_seq_len (factor 1 if not given)."""
        scaling = self.rope_scaling or {}
        if scaling.get("rope_type") == "ntk":
            return int(self.max_expected_seq_len * float(scaling.get("factor", 1.0)))
        return self.max_expected_seq_len

    def validate(self) -> None:
        problems = []
        if self.nheads <= 0 or self.emb_dim <= 0 or self.nlayers < 0 or self.src_vocab_size <= 0:
            problems.append("emb_dim, nheads and src_vocab_size must be positive")
        elif self.emb_dim % self.nheads:
            problems.append(f"emb_dim {self.emb_dim} is not a multiple of nheads {self.nheads}")
        elif (self.emb_dim // self.nheads) % 2:
            problems.append(f"head size {self.emb_dim // self.nheads} is odd: rotary pairs need an even size")
        if self.kvheads < 0 or (self.kvheads and self.nheads % self.kvheads):
            problems.append(f"nheads {self.nheads} is not a multiple of kvheads {self.kvheads}")
        if str(self.activation_fn).lower() not in ACTIVATION_NAMES:
            problems.append(f"activation_fn {self.activation_fn!r} is not one of {', '.join(ACTIVATION_NAMES)}")
        if self.p_dropout:
            problems.append("p_dropout must be 0: this library only generates")
        kind = (self.rope_scaling or {}).get("rope_type", "regular")
        if kind not in ("regular", "llama3", "ntk"):
            problems.append(f"rope_scaling rope_type {kind!r} is not one of regular, llama3, ntk")
        if kind == "ntk" and float((self.rope_scaling or {}).get("factor", 1.0)) < 1.0:
            problems.append("rope_scaling factor of ntk scaling must be at least 1")
        if problems:
            raise ValueError("invalid LLaMAConfig: " + "; ".join(problems))

    # ---- Hugging Face config.json ---------------------------------------
    @classmethod
    def from_hf_dict(cls, hf: dict) -> "LLaMAConfig":
        archs = hf.get("architectures") or []
        if archs and archs[0] not in HF_ARCHITECTURES:
            raise ValueError(f"config.json names architecture {archs[0]!r}, not one of {HF_ARCHITECTURES}")
        missing = [
            k
            for k in (
                "hidden_size",
                "num_attention_heads",
                "num_hidden_layers",
                "intermediate_size",
                "vocab_size",
                "rms_norm_eps",
                "max_position_embeddings",
            )
            if k not in hf
        ]
        if missing:
            raise ValueError(f"config.json lacks the keys {missing}")
        rope_theta = hf.get("rope_theta")
        rope_scaling = hf.get("rope_scaling")
        if hf.get("rope_parameters") is not None:
            rope_theta = hf["rope_parameters"]["rope_theta"]
            rope_scaling = hf["rope_parameters"].get("rope_scaling")
        if rope_scaling and "rope_type" not in rope_scaling and "type" in rope_scaling:
            rope_scaling = dict(rope_scaling, rope_type=rope_scaling["type"])
        if rope_scaling and rope_scaling.get("rope_type") == "default":
            rope_scaling = {}
        width, heads = hf["hidden_size"], hf["num_attention_heads"]
        if hf.get("head_dim") is not None and hf["head_dim"] * heads != width:
            raise ValueError(
                f"config.json head_dim {hf['head_dim']} differs from hidden_size/num_attention_heads "
                f"{width}/{heads}: the reference's Llama fixes the head size to that quotient"
            )
        act = str(hf.get("hidden_act", "silu")).lower()
        if act not in ACTIVATION_NAMES:
            raise ValueError(f"config.json hidden_act {act!r} is not one of {', '.join(ACTIVATION_NAMES)}")
        kv = hf.get("num_key_value_heads")
        kwargs = dict(
            src_vocab_size=hf["vocab_size"],
            emb_dim=width,
            nheads=heads,
            kvheads=heads if kv is None else kv,
            nlayers=hf["num_hidden_layers"],
            norm_eps=hf["rms_norm_eps"],
            max_expected_seq_len=hf["max_position_embeddings"],
            hidden_grow_factor=hf["intermediate_size"] / width,
            multiple_of=1,
            hidden_dim=hf["intermediate_size"],
            tie_heads=bool(hf.get("tie_word_embeddings", False)),
            attn_bias=bool(hf.get("attention_bias", False)),
            mlp_bias=bool(hf.get("mlp_bias", False)),
            activation_fn="swish" if act == "silu" else act,
        )
        if rope_theta is not None:
            kwargs["rope_theta"] = float(rope_theta)
        if rope_scaling:
            kwargs["rope_scaling"] = dict(rope_scaling)
        return cls(**kwargs)

    def to_hf_dict(self) -> dict:
        """The config.json that ``from_hf_dict`` reads back to an equal configuration."""
        out = {
            "architectures": [HF_ARCHITECTURES[0]],
            "model_type": "llama",
            "hidden_size": self.emb_dim,
            "num_attention_heads": self.nheads,
            "num_key_value_heads": self.kv_heads,
            "num_hidden_layers": self.nlayers,
            "intermediate_size": self.ffn_hidden_dim,
            "vocab_size": self.src_vocab_size,
            "rms_norm_eps": self.norm_eps,
            "max_position_embeddings": self.max_expected_seq_len,
            "rope_theta": self.rope_theta,
            "rope_scaling": dict(self.rope_scaling) if self.rope_scaling else None,
            "tie_word_embeddings": self.tie_heads,
            "attention_bias": self.attn_bias,
            "mlp_bias": self.mlp_bias,
            "hidden_act": "silu" if str(self.activation_fn).lower() in ("swish", "silu") else str(self.activation_fn).lower(),
            "head_dim": self.head_dim,
        }
        return out
