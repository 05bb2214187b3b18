"""A decoder model assembled from a ``ModelSpec``: embedding, layers run in the
order of the schedule, final norm, head.  It knows no architecture by name."""

from __future__ import annotations

from typing import List, Optional, Tuple

import torch

from ..cache import KVNeed, SequenceCache, StateNeed
from ..parts import LayerCache, ModelSpec, Part, ResidualStream, make_part, part_attribute


class DecoderModel(Part):
    def __init__(self, spec: ModelSpec, dtype: torch.dtype, config=None):
        super().__init__()
        if dtype not in (torch.float32, torch.bfloat16):
            raise TypeError(f"models run in float32 or bfloat16, not {dtype}")
        self.spec, self.dtype, self.config = spec, dtype, config
        self.device: Optional[torch.device] = None
        self.schedule = spec.resolved_schedule()

        self.positions = {name: make_part("position", p.kind, **p.args) for name, p in spec.positions.items()}
        self.embedding = self.add_child(spec.embedding_name, make_part("embedding", spec.embedding.kind, vocab=spec.vocab, width=spec.width, **spec.embedding.args))
        self.layers: List[Part] = []
        for i, layer in enumerate(spec.layers):
            pos = self.positions[layer.position] if layer.position is not None else None
            mixer = make_part("mixer", layer.mixer.kind, width=spec.width, position_encoder=pos, **layer.mixer.args)
            ff = make_part("feed_forward", layer.feed_forward.kind, width=spec.width, **layer.feed_forward.args)
            # a block names the norms it wants as constructor arguments (none, two, four ...); each is built from the
            # layer's list of norm specs, or from its one norm spec for all of them
            wanted = part_attribute("block", layer.block.kind, "norm_arguments", ("norm1", "norm2"))
            specs = layer.norms if layer.norms is not None else [layer.norm] * len(wanted)
            if len(specs) != len(wanted):
                raise ValueError(f"layer {i}: block {layer.block.kind!r} takes {len(wanted)} norms {tuple(wanted)}, {len(specs)} are given")
            norms = {name: make_part("norm", n.kind, width=spec.width, **n.args) for name, n in zip(wanted, specs)}
            block = make_part("block", layer.block.kind, mixer=mixer, feed_forward=ff, **norms, **layer.block.args)
            self.layers.append(self.add_child(spec.layer_name.format(i=i), block))
        self.final_norm = self.add_child(spec.final_norm_name, make_part("norm", spec.final_norm.kind, width=spec.width, **spec.final_norm.args))
        self.head = self.add_child(spec.head_name, make_part("head", spec.head.kind, width=spec.width, vocab=spec.vocab, **spec.head.args))
        # with tied heads the head's table is the embedding's (fms/models/llama.py:414-423)
        self.tied = {}
        if spec.tie_heads:
            self.tied[spec.head_name + ".weight"] = spec.embedding_name + ".weight"

    # ---- what the model asks of a cache ------------------------------------
    def cache_needs(self) -> Tuple[List[Tuple[int, KVNeed]], List[Tuple[int, StateNeed]]]:
        kv, state = [], []
        for n, entry in enumerate(self.schedule):
            mixer = self.layers[entry.layer].mixer
            need = mixer.kv_need()
            if need is not None and entry.cache_of is None:
                kv.append((n, need))
            if entry.cache_of is not None:
                other = self.layers[self.schedule[entry.cache_of].layer].mixer.kv_need()
                if need is None or other != need:
                    raise ValueError(f"schedule entry {n} cannot read the cache of entry {entry.cache_of}: their needs differ")
            sneed = mixer.state_need()
            if sneed is not None:
                state.append((n, sneed))
        return kv, state

    def make_cache(self, max_tokens: int, max_slots: int, device=None) -> SequenceCache:
        kv, state = self.cache_needs()
        return SequenceCache(kv, state, max_tokens, max_slots, self.spec.max_seq_len, self.dtype,
                             self.device if device is None else device)

    def finalize_all(self, device) -> None:
        self.device = torch.device(device)
        for part in self.walk():
            part.finalize(self.device, self.dtype)
        for part in self.positions.values():
            part.finalize(self.device, self.dtype)

    def state_dict(self, fused_weights: Optional[bool] = None) -> dict:
        """Parameter names -> tensors, as the reference's model.state_dict() names them.  fused_weights (default: the
        configuration's field): True gives the projections as the model holds them (qkv_fused, wg1_fused); False
        gives the parts that the reference's unfused modules hold (fms/utils/fusion.py:15-35,
        fms/modules/attention.py:666-687, fms/modules/feedforward.py:312-327): query/key/value and wg/w1, as views
        of the fused tensors.  The model itself always runs the fused products; the field changes names at this
        edge, and a checkpoint with either set of names loads (weights/adapters.py: weight_fusion)."""
        if fused_weights is None:
            fused_weights = bool(getattr(self.config, "fused_weights", True))
        out = {}
        for name, _, part, local in self.named_specs():
            tensor = part.w[local]
            if tensor is None:
                target = self.tied.get(name)
                tensor = out.get(target) if target else None
            out[name] = tensor
        if not fused_weights:
            for part_name, part in self.named_parts():
                for fused, pieces in getattr(part, "unfused_parameters", lambda: {})().items():
                    for kind in ("weight", "bias"):
                        whole = out.pop(f"{part_name}{fused}.{kind}", None)
                        if whole is None:
                            continue
                        at = 0
                        for piece, rows in pieces:
                            out[f"{part_name}{piece}.{kind}"] = whole[at : at + rows]
                            at += rows
        return out

    def named_parts(self, prefix: str = ""):
        """(dotted name with a trailing dot, part) of every part below the model."""
        stack = [(prefix, self)]
        while stack:
            name, part = stack.pop()
            yield name, part
            stack.extend((name + child_name + ".", child) for child_name, child in part.children().items())

    def get_config(self):
        """The configuration the model was built from (the reference's LLaMA.get_config, fms/models/llama.py:380-381)."""
        return self.config

    def __call__(self, input_ids: torch.Tensor, last_n_tokens: int = 0, **kwargs) -> torch.Tensor:
        """Called on token ids as the reference's model is: float32 logits [B, S, V] without a cache kept
        (generation.logits has the details).  Generation does not come through here: it steps an Engine."""
        from ..generation import logits

        return logits(self, input_ids, last_n_tokens=last_n_tokens, **kwargs)

    # ---- one pass over the tokens of a step --------------------------------
    def forward(self, batch, cache: SequenceCache) -> torch.Tensor:
        """float32 logits [n wanted rows, vocab] of the tokens in `batch`; the cache is extended in place."""
        max_position = batch.max_context - 1
        stream = ResidualStream(self.embedding.forward(batch.token_ids, batch))
        for n, entry in enumerate(self.schedule):
            block = self.layers[entry.layer]
            block.mixer.check_step(max_position)
            owner = n if entry.cache_of is None else entry.cache_of
            if owner in cache.group_of_entry:
                group, keys, values = cache.kv_of_entry(owner)
            else:
                group, keys, values = -1, None, None
            view = LayerCache(group, keys, values, entry.cache_of is None, cache.state_of_entry(n))
            if getattr(block, "fuses_next_norm", False) and n + 1 < len(self.schedule):
                # the norm that reads the stream next, so that this block's last product can prepare its input
                first_norm = getattr(self.layers[self.schedule[n + 1].layer], "first_norm", None)
                block.forward(stream, batch, view, self.dtype, next_norm=first_norm() if first_norm else None)
            else:
                block.forward(stream, batch, view, self.dtype)
        normed = stream.normed(self.final_norm, self.dtype, rows=batch.logit_rows)
        return self.head.forward(normed)
