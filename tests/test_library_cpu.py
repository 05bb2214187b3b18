"""Configuration, registry, weight reading and its errors, the cache's bookkeeping and the
generation loop's decisions.  None of this needs a GPU."""

import json
import os
import random

import pytest
import torch

import fms_amd
from fms_amd.architectures import list_models, list_variants, register_model, variant_config
from fms_amd.cache import CacheFull, KVNeed, PagePool, SequenceCache, StateNeed
from fms_amd.config import LLaMAConfig
from fms_amd.engine.model import DecoderModel
from fms_amd.architectures.llama import detect_source, llama_spec
from fms_amd.generation import generate_requests, pad_input_ids, plan_batches, trim_prefix, truncate_after_eos
from fms_amd.parts import ScheduleEntry
from fms_amd.weights import Checkpoint, WeightsError, get_adapter, kept_dtype, load_checkpoint, write_safetensors

import plain_llama as P


# --------------------------------------------------------------------------
# configuration
# --------------------------------------------------------------------------
def test_config_defaults_and_derived_sizes():
    c = LLaMAConfig()
    assert (c.head_dim, c.kv_heads, c.ffn_hidden_dim) == (128, 32, 11008)
    c = variant_config("llama", "3-8b")
    assert (c.head_dim, c.kv_heads, c.ffn_hidden_dim, c.src_vocab_size) == (128, 8, 14336, 128256)
    assert variant_config("llama", "3-70b").ffn_hidden_dim == 28672
    assert LLaMAConfig(emb_dim=16, nheads=2, hidden_grow_factor=8 / 3, multiple_of=2).ffn_hidden_dim == 42


def test_config_round_trip_and_updated(tmp_path):
    c = LLaMAConfig(emb_dim=64, nheads=4, kvheads=2, rope_scaling={"rope_type": "llama3", "factor": 2.0})
    path = tmp_path / "c.json"
    c.save(path)
    assert LLaMAConfig.load(path).as_dict() == c.as_dict()
    # unknown keys in a file are dropped; updated() copies, does not touch the original, logs unknown names
    data = c.as_dict()
    data["never_heard_of"] = 1
    path.write_text(json.dumps(data))
    assert LLaMAConfig.load(path).as_dict() == c.as_dict()
    d = c.updated(pad_id=5, bogus=1)
    assert d.pad_id == 5 and c.pad_id == -1 and d is not c
    d.rope_scaling["factor"] = 9.0
    assert c.rope_scaling["factor"] == 2.0


@pytest.mark.parametrize("bad", [dict(emb_dim=100, nheads=3), dict(nheads=4, kvheads=3), dict(emb_dim=12, nheads=4),
                                 dict(activation_fn="gelu_new"), dict(rope_scaling={"rope_type": "yarn"})])
def test_config_refuses_impossible_numbers(bad):
    with pytest.raises(ValueError):
        LLaMAConfig(**bad)


def test_config_from_hugging_face_keys():
    """The keys and the expected result of the reference's own mapping test
    (tests/resources/fms_model_kwargs/tiny-LlamaForCausalLM-3.2.json)."""
    hf = {"architectures": ["LlamaForCausalLM"], "hidden_size": 8, "intermediate_size": 32, "num_attention_heads": 4,
          "num_key_value_heads": 2, "num_hidden_layers": 2, "rms_norm_eps": 1e-6, "rope_theta": 10000.0,
          "vocab_size": 128256, "max_position_embeddings": 2048, "tie_word_embeddings": False,
          "attention_bias": False, "mlp_bias": False, "hidden_act": "silu", "bos_token_id": 1, "torch_dtype": "float32"}
    c = LLaMAConfig.from_hf_dict(hf)
    expected = {"attn_bias": False, "emb_dim": 8, "hidden_grow_factor": 4.0, "kvheads": 2, "max_expected_seq_len": 2048,
                "mlp_bias": False, "multiple_of": 1, "nheads": 4, "nlayers": 2, "norm_eps": 1e-06, "rope_theta": 10000.0,
                "src_vocab_size": 128256, "tie_heads": False}
    for k, v in expected.items():
        assert getattr(c, k) == v, k
    assert c.ffn_hidden_dim == 32
    # the integer width survives ratios that int(ratio * width) would truncate
    c = LLaMAConfig.from_hf_dict(dict(hf, hidden_size=440, num_attention_heads=4, intermediate_size=14336))
    assert c.ffn_hidden_dim == 14336
    assert LLaMAConfig.from_hf_dict(LLaMAConfig(emb_dim=64, nheads=4, kvheads=0).to_hf_dict()).kv_heads == 4
    # rope parameters in the newer nesting; what the reference ignores silently is checked here
    c = LLaMAConfig.from_hf_dict({**hf, "rope_parameters": {"rope_theta": 5e5, "rope_scaling": {"rope_type": "llama3", "factor": 8.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0, "original_max_position_embeddings": 8192}}})
    assert c.rope_theta == 5e5 and c.rope_scaling["rope_type"] == "llama3"
    with pytest.raises(ValueError):
        LLaMAConfig.from_hf_dict(dict(hf, head_dim=16))
    # hidden_act, which the reference's builder does not read, becomes activation_fn: one of the names that the
    # reference's activation table has (fms/utils/activation.py:14-24)
    assert c.activation_fn == "swish" and LLaMAConfig.from_hf_dict(dict(hf, hidden_act="gelu")).activation_fn == "gelu"
    assert LLaMAConfig.from_hf_dict(LLaMAConfig(emb_dim=64, nheads=4, activation_fn="Mish").to_hf_dict()).activation_fn == "mish"
    with pytest.raises(ValueError):
        LLaMAConfig.from_hf_dict(dict(hf, hidden_act="gelu_new"))
    with pytest.raises(ValueError):
        LLaMAConfig.from_hf_dict({k: v for k, v in hf.items() if k != "vocab_size"})


def test_registry():
    assert "llama" in list_models()
    assert {"micro", "7b", "2-7b", "3-8b", "3-70b", "granite.code-8b"} <= set(list_variants("llama"))
    with pytest.raises(KeyError):
        register_model("llama", "micro", lambda **kw: LLaMAConfig())
    with pytest.raises(KeyError):
        list_variants("no_such_architecture")
    with pytest.raises(KeyError):
        variant_config("llama", "no_such_variant")
    with pytest.raises(KeyError):
        fms_amd.get_model("no_such_architecture", "x")
    with pytest.raises(ValueError):
        fms_amd.get_model("llama", "micro", data_type="int7")
    # the reference's parameters for several GPUs are known by name and refused, not taken for configuration fields
    with pytest.raises(NotImplementedError):
        fms_amd.get_model("llama", "micro", distributed_strategy="tp")
    assert variant_config("llama", "micro", nlayers=2).nlayers == 2
    # a model folder's architecture comes from its config.json
    from fms_amd.architectures import architecture_for_hf

    assert architecture_for_hf("LlamaForCausalLM").name == "llama"
    with pytest.raises(KeyError):
        architecture_for_hf("GPTBigCodeForCausalLM")


# --------------------------------------------------------------------------
# weights
# --------------------------------------------------------------------------
TINY = dict(src_vocab_size=50, emb_dim=32, nheads=2, kvheads=1, nlayers=2, hidden_dim=40, multiple_of=1,
            max_expected_seq_len=64)


def test_model_declares_the_reference_tensor_names():
    """tests/resources/expectations/models.test_llama.TestLlama2.test_model_weight_keys"""
    model = DecoderModel(llama_spec(LLaMAConfig(**TINY)), torch.float32)
    names = sorted(n for n, *_ in model.named_specs())
    want = ["base_model.dec_norm.weight", "base_model.embedding.weight"]
    for i in range(2):
        p = f"base_model.layers.{i}."
        want += [p + "attn.dense.weight", p + "attn.in_proj.qkv_fused.weight", p + "ff_ln.weight",
                 p + "ff_sub_layer.w2.weight", p + "ff_sub_layer.wg1_fused.weight", p + "ln.weight"]
    want.append("head.weight")
    assert names == sorted(want)
    biased = DecoderModel(llama_spec(LLaMAConfig(**TINY, attn_bias=True, mlp_bias=True)), torch.float32)
    names = {n for n, *_ in biased.named_specs()}
    assert "base_model.layers.0.attn.in_proj.qkv_fused.bias" in names and "base_model.layers.1.ff_sub_layer.w2.bias" in names


def test_written_folder_is_read_back_the_same_by_both_readers(tmp_path):
    config = LLaMAConfig(**TINY, tie_heads=True, attn_bias=True)
    folder = fms_amd.write_model_folder(str(tmp_path / "m"), config, seed=3, norm_std=0.1)
    again = fms_amd.write_model_folder(str(tmp_path / "m2"), config, seed=3, norm_std=0.1)
    a = P.read_safetensors(os.path.join(folder, "model.safetensors"))
    b = P.read_safetensors(os.path.join(again, "model.safetensors"))
    assert a.keys() == b.keys() and all(torch.equal(a[k], b[k]) for k in a)  # a function of the seed
    c = P.read_safetensors(os.path.join(fms_amd.write_model_folder(str(tmp_path / "m3"), config, seed=4), "model.safetensors"))
    assert not torch.equal(a["model.embed_tokens.weight"], c["model.embed_tokens.weight"])
    assert "lm_head.weight" not in a  # tied
    assert a["model.layers.0.self_attn.q_proj.weight"].dtype == torch.bfloat16
    # the product's reader and the installed safetensors package read the same values
    ckpt = Checkpoint(folder, "hf")
    from safetensors import safe_open

    with safe_open(os.path.join(folder, "model.safetensors"), "pt") as f:
        assert sorted(f.keys()) == sorted(ckpt.keys())
        for k in f.keys():
            assert torch.equal(f.get_tensor(k), ckpt.read(k))
            assert torch.equal(a[k], ckpt.read(k))
    ckpt.close()
    from fms_amd.models import read_model_folder_config

    arch, cfg = read_model_folder_config(folder)
    assert arch.name == "llama" and cfg.ffn_hidden_dim == 40 and cfg.tie_heads and cfg.attn_bias


def test_hf_adapter_matches_the_plain_conversion(tmp_path):
    """Names, the row permutation of q/k (weights and biases) and the fusion order."""
    config = LLaMAConfig(**TINY, attn_bias=True, mlp_bias=True)
    folder = fms_amd.write_model_folder(str(tmp_path / "m"), config, seed=5)
    cfg, want = P.load_model_folder(folder)
    ckpt = Checkpoint(folder, "hf")
    assert detect_source(ckpt.keys()) == "hf"
    adapter = get_adapter("llama", "hf")
    got = {}
    from fms_amd.weights.loader import _layer_groups

    for group in _layer_groups(ckpt.keys()):
        got.update(adapter({n: ckpt.read(n) for n in group}, model_config=config))
    ckpt.close()
    assert sorted(got) == sorted(want)
    for k in want:
        assert torch.equal(got[k].float(), want[k]), k


def test_meta_adapter_names_and_fusion():
    """tests/utils/test_serialization.py:16-30: w1 is the gate, w3 the up projection, fused [w1; w3]."""
    sd = {"layers.0.feed_forward.w1.weight": torch.ones(3, 2), "layers.0.feed_forward.w3.weight": torch.zeros(3, 2),
          "layers.0.feed_forward.w2.weight": torch.ones(2, 3), "layers.0.attention.wq.weight": torch.full((4, 2), 1.0),
          "layers.0.attention.wk.weight": torch.full((2, 2), 2.0), "layers.0.attention.wv.weight": torch.full((2, 2), 3.0),
          "layers.0.attention.wo.weight": torch.ones(2, 4), "layers.0.attention_norm.weight": torch.ones(2),
          "layers.0.ffn_norm.weight": torch.ones(2), "tok_embeddings.weight": torch.ones(5, 2),
          "norm.weight": torch.ones(2), "output.weight": torch.ones(5, 2)}
    assert detect_source(list(sd)) == "meta"
    out = get_adapter("llama", "meta")(sd, model_config=None)
    fused = out["base_model.layers.0.ff_sub_layer.wg1_fused.weight"]
    assert torch.equal(fused, torch.cat([torch.ones(3, 2), torch.zeros(3, 2)]))
    qkv = out["base_model.layers.0.attn.in_proj.qkv_fused.weight"]
    assert qkv[:, 0].tolist() == [1, 1, 1, 1, 2, 2, 3, 3]
    assert {"base_model.embedding.weight", "base_model.dec_norm.weight", "head.weight", "base_model.layers.0.ln.weight",
            "base_model.layers.0.ff_ln.weight", "base_model.layers.0.attn.dense.weight",
            "base_model.layers.0.ff_sub_layer.w2.weight"} <= set(out)
    with pytest.raises(KeyError):
        get_adapter("llama", "no_such_source")


def test_adapters_are_registered_extended_and_applied_by_name():
    """fms/utils/serialization.py:27-148, 292-317: steps and sources are registered once; an existing source can be
    given further steps; get_adapted applies a source's steps to a state dict and hands an empty one back."""
    from fms_amd.weights import extend_adapter, get_adapted, list_sources, register_adapter, register_adapter_step

    arch = "toy_adapters"
    register_adapter_step(arch, "prefix", lambda sd, **kw: {"m." + k: v for k, v in sd.items()})
    register_adapter_step(arch, "double", lambda sd, factor=2, **kw: {k: v * factor for k, v in sd.items()})
    with pytest.raises(KeyError):
        register_adapter_step(arch, "prefix", lambda sd, **kw: sd)
    register_adapter(arch, "theirs", ["prefix"])
    with pytest.raises(KeyError):
        register_adapter(arch, "theirs", ["prefix"])
    with pytest.raises(KeyError):
        register_adapter(arch, "other", ["no_such_step"])
    assert list_sources(arch) == ["theirs"] and list_sources("no_such_architecture") == []
    sd = {"w": torch.ones(2)}
    assert list(get_adapted(arch, "theirs", sd, {})) == ["m.w"]
    extend_adapter(arch, "theirs", ["double"])
    out = get_adapted(arch, "theirs", sd, {"factor": 3})
    assert list(out) == ["m.w"] and out["m.w"].tolist() == [3.0, 3.0]
    with pytest.raises(KeyError):
        extend_adapter(arch, "no_such_source", ["double"])
    with pytest.raises(KeyError):
        extend_adapter(arch, "theirs", ["no_such_step"])
    empty = {}
    assert get_adapted(arch, "theirs", empty, {}) is empty
    assert get_adapted(arch, None, sd, {}) is sd and get_adapted(arch, "fms", sd, None) is sd


def test_kept_dtypes():
    assert kept_dtype(torch.bfloat16, "float", torch.bfloat16) == torch.bfloat16
    assert kept_dtype(torch.float16, "float", torch.bfloat16) == torch.bfloat16
    assert kept_dtype(torch.float32, "float", torch.bfloat16) == torch.float32  # stored in 32-bit: stays so
    assert kept_dtype(torch.bfloat16, "float", torch.float32) == torch.float32
    assert kept_dtype(torch.int64, "int", torch.bfloat16) == torch.int32
    # a type that the caller asked for is what floating tensors get (tests/models/test_getmodel_datatype.py:58-90) ...
    assert kept_dtype(torch.float32, "float", torch.bfloat16, forced=True) == torch.bfloat16
    assert kept_dtype(torch.bfloat16, "float", torch.float32, forced=True) == torch.float32
    # ... except a norm's scale, which the kernels read in either type
    assert kept_dtype(torch.float32, "scale", torch.bfloat16, forced=True) == torch.float32
    assert kept_dtype(torch.bfloat16, "scale", torch.bfloat16, forced=True) == torch.bfloat16


def test_one_error_lists_missing_unexpected_and_wrong_shapes(tmp_path):
    config = LLaMAConfig(**TINY)
    folder = fms_amd.write_model_folder(str(tmp_path / "m"), config, seed=1)
    tensors = P.read_safetensors(os.path.join(folder, "model.safetensors"))
    del tensors["model.layers.1.mlp.down_proj.weight"]
    del tensors["model.norm.weight"]
    tensors["model.layers.0.rotary_emb.inv_freq"] = torch.zeros(8)
    tensors["model.layers.0.self_attn.o_proj.weight"] = torch.zeros(32, 48, dtype=torch.bfloat16)
    write_safetensors(os.path.join(folder, "model.safetensors"), [(k, tuple(v.shape), v.dtype) for k, v in tensors.items()],
                      lambda name: tensors[name])
    model = DecoderModel(llama_spec(config), torch.float32, config=config)
    with pytest.raises(WeightsError) as err:
        load_checkpoint(model, folder, "llama", "hf", "cpu")
    e = err.value
    assert e.missing == ["base_model.dec_norm.weight", "base_model.layers.1.ff_sub_layer.w2.weight"]
    assert e.unexpected == ["base_model.layers.0.rotary_emb.inv_freq"]
    assert e.wrong_shapes == [("base_model.layers.0.attn.dense.weight", (32, 48), (32, 32))]
    text = str(e)
    for word in ("missing", "unexpected", "wrong shapes", "base_model.dec_norm.weight", "rotary_emb.inv_freq", "(32, 48)"):
        assert word in text
    with pytest.raises(FileNotFoundError, match="Can't find the requested checkpoint data at"):
        Checkpoint(str(tmp_path / "nowhere"))


def test_loading_keeps_types_and_ties_the_head(tmp_path):
    config = LLaMAConfig(**TINY, tie_heads=True)
    folder = fms_amd.write_model_folder(str(tmp_path / "m"), config, seed=2)
    tensors = P.read_safetensors(os.path.join(folder, "model.safetensors"))
    tensors["model.norm.weight"] = tensors["model.norm.weight"].float()  # one tensor stored in 32-bit
    write_safetensors(os.path.join(folder, "model.safetensors"), [(k, tuple(v.shape), v.dtype) for k, v in tensors.items()],
                      lambda name: tensors[name])
    model = DecoderModel(llama_spec(config), torch.bfloat16, config=config)
    load_checkpoint(model, folder, "llama", "hf", "cpu")
    assert model.final_norm.w["weight"].dtype == torch.float32
    assert model.layers[0].mixer.qkv.w["weight"].dtype == torch.bfloat16
    assert model.head.w["weight"] is model.embedding.w["weight"]
    model32 = DecoderModel(llama_spec(config), torch.float32, config=config)
    load_checkpoint(model32, folder, "llama", "hf", "cpu")
    assert model32.layers[1].feed_forward.w2.w["weight"].dtype == torch.float32


def test_a_forced_type_casts_what_the_file_stores_in_32_bit(tmp_path):
    """tests/models/test_getmodel_datatype.py: a checkpoint in 32-bit loaded with data_type bf16 gives a bfloat16
    model (every linear takes the bfloat16 kernels); with no type given the stored type is kept."""
    config = LLaMAConfig(**TINY)
    folder = fms_amd.write_model_folder(str(tmp_path / "m"), config, seed=2, data_type="float32")
    forced = DecoderModel(llama_spec(config), torch.bfloat16, config=config)
    load_checkpoint(forced, folder, "llama", "hf", "cpu", forced_dtype=True)
    for name, spec, part, local in forced.named_specs():
        want = torch.float32 if spec.kind == "scale" else torch.bfloat16
        assert part.w[local].dtype == want, name
    assert forced.layers[0].mixer.dense.streams(4, torch.bfloat16)
    kept = DecoderModel(llama_spec(config), torch.bfloat16, config=config)
    load_checkpoint(kept, folder, "llama", "hf", "cpu")
    assert all(part.w[local].dtype == torch.float32 for _, _, part, local in kept.named_specs())
    assert not kept.layers[0].mixer.dense.streams(4, torch.bfloat16)


def test_state_dict_names_follow_fused_weights_and_load_back(tmp_path):
    """tests/models/test_getmodel_fusedweights.py:30-33: a fused model's state dict has .qkv_fused. and .wg1_fused.,
    an unfused one's .query./.key./.value. and .wg./.w1.; either loads into the model (fms/utils/fusion.py:15-35),
    and so does a checkpoint with the names of before 0.0.6 (fms/models/llama.py:761-765)."""
    config = LLaMAConfig(**TINY)
    folder = fms_amd.write_model_folder(str(tmp_path / "m"), config, seed=4, data_type="float32")
    model = DecoderModel(llama_spec(config), torch.float32, config=config)
    load_checkpoint(model, folder, "llama", "hf", "cpu")
    fused = model.state_dict()
    assert any(".qkv_fused." in n for n in fused) and any(".wg1_fused." in n for n in fused)
    assert not any(part in n for n in fused for part in (".query.", ".key.", ".value.", ".w1.", ".wg."))
    model.config = config.updated(fused_weights=False)
    unfused = model.state_dict()
    assert not any(".qkv_fused." in n or ".wg1_fused." in n for n in unfused)
    H, K, D, F = config.nheads, config.kv_heads, config.head_dim, config.ffn_hidden_dim
    p = "base_model.layers.1."
    q, k, v = (unfused[p + f"attn.in_proj.{w}.weight"] for w in ("query", "key", "value"))
    assert q.shape[0] == H * D and k.shape[0] == K * D == v.shape[0]
    assert torch.equal(torch.cat([q, k, v]), fused[p + "attn.in_proj.qkv_fused.weight"])
    assert torch.equal(torch.cat([unfused[p + "ff_sub_layer.wg.weight"], unfused[p + "ff_sub_layer.w1.weight"]]),
                       fused[p + "ff_sub_layer.wg1_fused.weight"])
    assert unfused[p + "ff_sub_layer.wg.weight"].shape[0] == F
    assert model.state_dict(fused_weights=True).keys() == fused.keys()

    def reload(sd, name):
        path = tmp_path / name
        path.mkdir()
        sd = {n: t.contiguous() for n, t in sd.items()}
        write_safetensors(str(path / "model.safetensors"), [(n, tuple(t.shape), t.dtype) for n, t in sd.items()], lambda n: sd[n])
        again = DecoderModel(llama_spec(config), torch.float32, config=config)
        load_checkpoint(again, str(path), "llama", detect_source(list(sd)), "cpu")  # as get_model finds the source
        for n, t in fused.items():
            assert torch.equal(again.state_dict(fused_weights=True)[n], t), n

    reload(fused, "fused")
    reload(unfused, "unfused")
    old_names = {n.replace(".attn.in_proj.", ".attn."): t for n, t in unfused.items()}
    assert detect_source(list(old_names)) == "fms.pre0.0.6" and detect_source(list(unfused)) == "fms_unfused"
    reload(old_names, "pre006")


def test_the_architecture_tells_a_checkpoints_source():
    from fms_amd.architectures import get_architecture

    arch = get_architecture("llama")
    assert arch.detect_source(["model.layers.0.self_attn.q_proj.weight"]) == "hf"
    assert arch.detect_source(["tok_embeddings.weight", "layers.0.attention.wq.weight"]) == "meta"
    assert arch.detect_source(["base_model.layers.0.attn.in_proj.query.weight"]) == "fms_unfused"
    assert arch.detect_source(["base_model.layers.0.attn.in_proj.qkv_fused.weight"]) == "fms"
    import fms_amd.models as models

    assert not hasattr(models, "detect_source")  # the generic loader asks the architecture


def test_ntk_scaling_stretches_the_positions():
    """fms/modules/positions.py:135-168: alpha is the power of two that covers the call's longest sequence; up to
    the table's length it is 1.  The configuration lets sequences grow to factor times max_expected_seq_len."""
    from fms_amd.parts.position import RotaryEncoding, ntk_alpha, rope_frequencies

    for n, want in ((1, 1), (64, 1), (65, 2), (128, 2), (129, 4), (256, 4), (257, 8), (1000, 16)):
        assert ntk_alpha(n, 64) == want == P.ntk_alpha(n, 64)
    config = LLaMAConfig(**TINY, rope_scaling={"rope_type": "ntk", "factor": 4.0})
    assert config.max_positions == 4 * config.max_expected_seq_len
    assert LLaMAConfig(**TINY, rope_scaling={"rope_type": "ntk"}).max_positions == config.max_expected_seq_len
    assert LLaMAConfig(**TINY).max_positions == config.max_expected_seq_len
    back = LLaMAConfig.from_hf_dict(config.to_hf_dict())
    assert back.rope_scaling == config.rope_scaling and back.max_positions == config.max_positions
    spec = llama_spec(config)
    assert spec.max_seq_len == config.max_positions
    assert spec.positions["rope"].args["max_seq_len"] == config.max_expected_seq_len
    with pytest.raises(ValueError, match="factor"):
        LLaMAConfig(**TINY, rope_scaling={"rope_type": "ntk", "factor": 0.5})
    scaling = {"rope_type": "ntk"}
    for alpha in (1, 2, 8):
        torch.testing.assert_close(rope_frequencies(16, 1e4, scaling, alpha), P.rope_frequencies(16, 1e4, scaling, 64 * alpha, 64))
    torch.testing.assert_close(rope_frequencies(16, 1e4, scaling, 1), rope_frequencies(16, 1e4))
    rope = RotaryEncoding(16, 1e4, 64, scaling, max_positions=256)
    assert not rope.graph_safe and RotaryEncoding(16, 1e4, 64, scaling).graph_safe and RotaryEncoding(16, 1e4, 64).graph_safe
    rope.check_positions(255)
    with pytest.raises(IndexError):
        rope.check_positions(256)
    with pytest.raises(IndexError):
        RotaryEncoding(16, 1e4, 64, {}, max_positions=256).check_positions(64)  # only ntk stretches


def test_schedule_is_data():
    config = LLaMAConfig(**TINY)
    spec = llama_spec(config)
    spec.schedule = [ScheduleEntry(0), ScheduleEntry(1), ScheduleEntry(0), ScheduleEntry(1, cache_of=1)]
    model = DecoderModel(spec, torch.float32)
    kv, state = model.cache_needs()
    assert [e for e, _ in kv] == [0, 1, 2] and state == []  # entry 3 reads entry 1's cache
    cache = model.make_cache(256, 2, device=None)
    assert len(cache.groups) == 1 and cache.groups[0].entries == [0, 1, 2]
    for bad in ([ScheduleEntry(5)], [ScheduleEntry(0, cache_of=0)], [ScheduleEntry(0), ScheduleEntry(1, cache_of=1)]):
        spec.schedule = bad
        with pytest.raises(ValueError):
            DecoderModel(spec, torch.float32)


# --------------------------------------------------------------------------
# cache
# --------------------------------------------------------------------------
def test_page_pool_accounting():
    pool = PagePool(3)
    pages = [pool.alloc() for _ in range(3)]
    assert sorted(pages) == [0, 1, 2] and pool.n_free == 0
    with pytest.raises(CacheFull):
        pool.alloc()
    pool.free(pages[1])
    with pytest.raises(ValueError):
        pool.free(pages[1])  # freed twice
    with pytest.raises(ValueError):
        pool.free(7)
    assert pool.alloc() == pages[1]
    pool.check()


def make_cache(max_tokens=64 * 6, max_slots=3, window=0):
    needs = [(0, KVNeed(2, 16)), (1, KVNeed(2, 16)), (2, KVNeed(2, 16, window))] if window else [(0, KVNeed(2, 16)), (1, KVNeed(2, 16))]
    return SequenceCache(needs, [(1, StateNeed((("sum", (4,), "float32"),)))], max_tokens, max_slots, 1000)


def test_cache_slots_and_pages_never_leak():
    cache = make_cache()
    rng = random.Random(0)
    live = {}
    for _ in range(2000):
        action = rng.random()
        if action < 0.3 and cache.n_free_slots:
            s = cache.alloc_slot()
            assert s not in live
            live[s] = 0
        elif action < 0.8 and live:
            s = rng.choice(list(live))
            n = rng.choice([1, 1, 1, 5, 64, 70])
            try:
                start = cache.extend(s, n)
                assert start == live[s]
                live[s] += n
            except CacheFull:
                assert cache.length(s) == live[s]  # nothing changed
        elif live:
            s = rng.choice(list(live))
            cache.free_slot(s)
            del live[s]
            with pytest.raises(ValueError):
                cache.free_slot(s)  # freed twice
        cache.check()
        held = sum(-(-n // 64) for n in live.values())
        assert cache.groups[0].pool.n_held == held
    for s in list(live):
        cache.free_slot(s)
    cache.check()
    assert cache.groups[0].pool.n_free == 6 and cache.n_free_slots == 3
    with pytest.raises(CacheFull):
        [cache.alloc_slot() for _ in range(4)]


def test_cache_groups_and_window_pages():
    cache = make_cache(max_tokens=64 * 8, window=100)
    assert len(cache.groups) == 2 and cache.groups[0].entries == [0, 1] and cache.groups[1].entries == [2]
    s = cache.alloc_slot()
    cache.extend(s, 300)
    assert len(cache.groups[0].pages[s]) == 5 and cache.groups[1].pool.n_held == 5
    for _ in range(100):
        cache.extend(s, 1)  # decoding: the windowed group gives back pages no later query can see
    cache.check()
    assert cache.groups[0].pool.n_held == 7
    # position 399 sees keys >= 300: logical pages 0..3 are gone
    table = cache.block_table(1, [s])
    assert (table[0, :4] == -1).all() and (table[0, 4:7] >= 0).all()
    assert cache.groups[1].pool.n_held == 3
    with pytest.raises(IndexError):
        cache.extend(s, 1000)  # beyond the model's positions
    cache.free_slot(s)
    cache.check()
    assert cache.groups[1].pool.n_free == 8


def test_a_step_that_cannot_be_made_changes_nothing():
    """Room for all or for none, across groups (one of them windowed) and across the sequences of a step."""
    kv = [(0, KVNeed(2, 16, 0)), (1, KVNeed(2, 16, 128))]
    cache = SequenceCache(kv, [], 64 * 8, 4, 2000, device=None)
    a, b, c = cache.alloc_slot(), cache.alloc_slot(), cache.alloc_slot()
    assert cache.extend_many([a, b, c], [200, 100, 64]) == [0, 0, 0]  # 4 + 2 + 1 pages in both groups
    assert cache.extend_many([a], [1]) == [200]  # the window lets go of a's first page: 7 of 8 held there, 7 in full
    cache.check()

    def snapshot():
        return ({s: cache.length(s) for s in cache.live_slots()}, [g.pool.n_free for g in cache.groups],
                [{s: list(p) for s, p in g.pages.items()} for g in cache.groups], [cache.stamp(s) for s in (a, b, c)])

    before = snapshot()
    with pytest.raises(CacheFull):  # b and c want a page each, the full group has one
        cache.extend_many([a, b, c], [1, 30, 1])
    assert snapshot() == before
    with pytest.raises(IndexError):  # c would pass the model's positions; a and b come first and must not grow
        cache.extend_many([a, b, c], [1, 1, 3000])
    assert snapshot() == before
    with pytest.raises(ValueError):
        cache.extend_many([a, a], [1, 1])
    assert snapshot() == before
    assert cache.pages_needed(b, 30) == 1 and cache.pages_needed(a, 1) == 0
    assert cache.extend_many([b, a], [30, 1]) == [100, 201]
    cache.check()
    # a stamp changes with every growth and with every hand-out, and never repeats
    stamps = {cache.stamp(a)}
    cache.extend(a, 1)
    stamps.add(cache.stamp(a))
    cache.free_slot(a)
    again = cache.alloc_slot()
    assert again == a
    stamps.add(cache.stamp(again))
    assert len(stamps) == 3


def test_a_graph_rewrites_its_table_when_a_window_gives_a_page_back():
    """A windowed group gives a page back at a step that brings no new page.  The captured step's block table must
    show -1 there in the same step: the page may be another sequence's by the next one."""
    from types import SimpleNamespace

    from fms_amd.engine.decode_graph import DecodeGraph
    from fms_amd.sampling import SamplingParams

    cache = make_cache(max_tokens=64 * 8, window=100)
    engine = SimpleNamespace(device=torch.device("cpu"), cache=cache)
    graph = DecodeGraph(engine, rows=2, max_context=2048, sampling=SamplingParams(do_sample=False))
    a, b = cache.alloc_slot(), cache.alloc_slot()
    cache.extend_many([a, b], [160, 10])
    positions = cache.extend_many([a, b], [1, 1])
    graph.load([a, b], [1, 2], positions, [0, 0], [0, 0])
    windowed = 1
    released_at = None
    for step in range(40):
        before = [len(g.pages[a]) for g in cache.groups]
        cache.extend_many([a, b], [1, 1])
        graph.refresh_pages()
        for g in range(len(cache.groups)):
            assert torch.equal(graph.tables[g][:2], cache.block_table(g, [a, b], n_columns=graph.table_width)), (step, g)
        if released_at is None and cache.groups[windowed].pages[a][0] == -1:
            released_at = step
            assert [len(g.pages[a]) for g in cache.groups] == before  # no new page came with the release
            assert int(graph.tables[windowed][0, 0]) == -1 and int(graph.tables[0][0, 0]) >= 0
    assert released_at is not None
    cache.check()


def test_a_decode_step_on_an_ended_slot_is_refused_like_any_step():
    from fms_amd.engine import Engine
    from fms_amd.sampling import SamplingParams

    cache = make_cache()
    engine = object.__new__(Engine)
    engine.cache, engine.vocab, engine.use_graphs = cache, 100, True
    a, b = cache.alloc_slot(), cache.alloc_slot()
    cache.extend_many([a, b], [3, 3])
    cache.free_slot(b)
    greedy = SamplingParams(do_sample=False)
    with pytest.raises(ValueError, match="not live"):
        engine.decode_and_choose([a, b], [1, 2], greedy)
    with pytest.raises(ValueError, match="not live"):
        engine.decode_and_choose([7], [1], greedy)
    with pytest.raises(ValueError):
        engine.decode_and_choose([a, a], [1, 2], greedy)
    with pytest.raises(ValueError, match="not live"):
        cache.stamp(b)
    assert cache.length(a) == 3  # nothing grew
    cache.check()


def test_a_windows_releases_are_found_without_walking_the_sequence():
    """The pages a window gives back are looked for from the first page still held: the plan of a step touches as
    many list entries as it releases, however long the sequence is."""
    cache = SequenceCache([(0, KVNeed(2, 16, 128))], [], 64 * 40, 2, 100_000, device=None)
    s = cache.alloc_slot()
    cache.extend(s, 64 * 30)
    group = cache.groups[0]
    assert group.first_held[s] == 0 and cache.pages_held(s) == 30
    cache.extend(s, 1)  # the first query of this step is position 1920: keys before 1793 are out of sight
    assert group.first_held[s] == 28 and group.pages[s][:28] == [-1] * 28 and cache.pages_held(s) == 3
    for _ in range(200):
        (_, release, _), = cache._plan(s, 1)
        assert len(release) <= 1 and all(i >= group.first_held[s] for i in release)
        cache.extend(s, 1)
        cache.check()
    cache.free_slot(s)
    assert group.pool.n_free == 40 and s not in group.first_held


def test_block_table_rows_follow_the_step_order():
    cache = make_cache()
    a, b = cache.alloc_slot(), cache.alloc_slot()
    cache.extend(a, 65)
    cache.extend(b, 3)
    table = cache.block_table(0, [b, a])
    assert table.shape == (2, 2) and table[0, 1] == -1 and table[1, 1] >= 0
    assert set(table.flatten().tolist()) - {-1} == set(cache.groups[0].pages[a] + cache.groups[0].pages[b])


def test_a_decode_batch_lists_its_rows_longest_context_first():
    from fms_amd.engine.batch import build_batch

    cache = make_cache(max_tokens=64 * 12, max_slots=5)
    slots = [cache.alloc_slot() for _ in range(4)]
    for slot, n in zip(slots, (5, 130, 64, 70)):
        cache.extend(slot, n)
    starts = [cache.extend(slot, 1) for slot in slots]
    batch = build_batch(cache, slots, [[1], [2], [3], [4]], starts, [[0]] * 4, "cpu")
    assert batch.is_decode and batch.rows_by_length.tolist() == [1, 3, 2, 0]
    assert batch.n_tokens == 4 and batch.n_wanted == 4 == batch.n_logit_rows
    # filled up to the rows of a captured step: padding rows of sequence -1 at the end, which are computed and not wanted
    more = [cache.extend(slot, 1) for slot in slots]
    padded = build_batch(cache, slots, [[1], [2], [3], [4]], more, [[0]] * 4, "cpu", pad_rows_to=8)
    assert padded.n_tokens == 8 and padded.n_seqs == 4 and padded.n_wanted == 4 and padded.n_logit_rows == 8
    assert padded.seq_of_token.tolist() == [0, 1, 2, 3, -1, -1, -1, -1] and padded.token_ids.tolist() == [1, 2, 3, 4, 0, 0, 0, 0]
    assert padded.positions.tolist()[:4] == more and padded.rows_by_length.tolist() == [1, 3, 2, 0, 4, 5, 6, 7]
    assert padded.logit_rows.tolist() == list(range(8)) and padded.max_context == max(more) + 1
    # where only some rows are wanted, nothing is computed for padding rows
    few = build_batch(cache, slots, [[1], [2], [3], [4]], [cache.extend(slot, 1) for slot in slots], [[0], [], [0], []], "cpu", pad_rows_to=8)
    assert few.n_tokens == 8 and few.logit_rows.tolist() == [0, 2] and few.n_wanted == 2 == few.n_logit_rows
    # a step that brings a prompt has no such order
    other = cache.alloc_slot()
    batch = build_batch(cache, [other], [[1, 2, 3]], [cache.extend(other, 3)], [[2]], "cpu")
    assert not batch.is_decode and batch.rows_by_length is None
    batch = build_batch(cache, [other], [[1, 2]], [cache.extend(other, 2)], [[1]], "cpu", pad_rows_to=8)
    assert batch.n_tokens == 2  # only decode steps are filled up


# --------------------------------------------------------------------------
# generation loop
# --------------------------------------------------------------------------
class FakeEngine:
    """Next token = last token + 1 (the mock of tests/utils/test_generate.py:15-30), with a real cache's bookkeeping."""

    class _Cache:
        pass

    def __init__(self, max_tokens=64 * 8, max_slots=4, max_seq_len=100, vocab=256):
        self.cache = SequenceCache([(0, KVNeed(1, 2))], [], max_tokens, max_slots, max_seq_len)
        self.vocab = vocab
        self.device = torch.device("cpu")
        self.steps = []
        self.last = {}

    def new_sequence(self):
        return self.cache.alloc_slot()

    def end_sequence(self, slot):
        self.cache.free_slot(slot)
        self.cache.check()

    def step(self, slots, tokens, want):
        assert want == "last"
        self.steps.append([len(t) for t in tokens])
        logits = torch.zeros(len(slots), self.vocab)
        for i, (s, t) in enumerate(zip(slots, tokens)):
            self.cache.extend(s, len(t))
            logits[i, (t[-1] + 1) % self.vocab] = 1.0
        return logits


def argmax_chooser(logits, request_ids, counters):
    return logits.argmax(-1).tolist()


def test_loop_counts_up_like_the_reference_mock():
    """tests/utils/test_generate.py:33-50: "ABCDE" -> "ABCDEFGHIJ"."""
    engine = FakeEngine()
    out = generate_requests(engine, [[ord(c) for c in "ABCDE"]], max_new_tokens=5, chooser=argmax_chooser)
    assert "".join(chr(t) for t in out[0]) == "FGHIJ"
    assert engine.steps == [[5], [1], [1], [1], [1]]  # the prompt in one step, then one token each
    assert engine.cache.live_slots() == []


def test_loop_unequal_prompts_stops_and_limits():
    engine = FakeEngine()
    prompts = [[10, 11, 12], [50], [20, 21], [97, 98]]
    out = generate_requests(engine, prompts, max_new_tokens=6, stop_token_ids=[23, 52], chooser=argmax_chooser)
    assert out == [[13, 14, 15, 16, 17, 18], [51, 52], [22, 23], [99, 100, 101, 102, 103, 104]]
    # the batch shrinks as sequences end: 4 prompts, 4 alive, then 2
    assert engine.steps == [[3, 1, 2, 2], [1, 1, 1, 1], [1, 1], [1, 1], [1, 1], [1, 1]]
    # a sequence stops at the model's last position: prompt 2 + 98 new = 100 tokens, the last one is not fed
    engine = FakeEngine(max_seq_len=100, max_tokens=64 * 4)
    out = generate_requests(engine, [[1, 2]], max_new_tokens=500, chooser=argmax_chooser)
    assert len(out[0]) == 99 and engine.cache.live_slots() == []
    assert generate_requests(engine, [[1]], max_new_tokens=0, chooser=argmax_chooser) == [[]]


def test_loop_lets_a_hook_change_what_is_fed():
    """before_step sees the tokens about to be fed and may replace them (the reference's
    prepare_model_inputs_hook, fms/utils/generation.py:295-296, reaches the loop through it)."""
    engine = FakeEngine()
    seen = []

    def hook(step, requests, tokens):
        seen.append((step, list(requests), [list(t) for t in tokens]))
        if step == 2:
            return [[40] for _ in tokens]  # from here the mock counts on from 40
        return None

    out = generate_requests(engine, [[10, 11], [20]], max_new_tokens=4, chooser=argmax_chooser, before_step=hook)
    assert out == [[12, 13, 41, 42], [21, 22, 41, 42]]
    assert seen[0] == (0, [0, 1], [[10, 11], [20]]) and seen[1] == (1, [0, 1], [[12], [21]]) and seen[2][2] == [[13], [22]]
    with pytest.raises(ValueError):
        generate_requests(FakeEngine(), [[1]], max_new_tokens=2, chooser=argmax_chooser, before_step=lambda s, r, t: [])


def test_loop_lets_a_hook_see_the_logits_and_change_the_choice():
    """after_choice sees the logits of the live requests and the tokens chosen from them, and may put others in
    their place (the reference's post_iteration_hook, fms/utils/generation.py:328-331, reaches the loop through it)."""
    engine = FakeEngine()
    seen = []

    def hook(step, requests, logits, tokens):
        seen.append((step, list(requests), tuple(logits.shape), list(tokens)))
        assert logits.argmax(-1).tolist() == tokens
        if step == 1:
            return [70 for _ in tokens]  # the mock counts on from 70
        return None

    out = generate_requests(engine, [[10, 11], [20], [30]], max_new_tokens=3, chooser=argmax_chooser, stop_token_ids=[31],
                            after_choice=hook)
    assert out == [[12, 70, 71], [21, 70, 71], [31]]
    assert seen == [(0, [0, 1, 2], (3, 256), [12, 21, 31]), (1, [0, 1], (2, 256), [13, 22]), (2, [0, 1], (2, 256), [71, 71])]
    with pytest.raises(ValueError):
        generate_requests(FakeEngine(), [[1]], max_new_tokens=2, chooser=argmax_chooser, after_choice=lambda s, r, l, t: [])


def test_loop_runs_as_many_batches_as_the_requests_need():
    engine = FakeEngine(max_tokens=64 * 2, max_slots=2)
    prompts = [[i] for i in range(7)]
    out = generate_requests(engine, prompts, max_new_tokens=3, chooser=argmax_chooser)
    assert out == [[i + 1, i + 2, i + 3] for i in range(7)]
    assert engine.steps[0] == [1, 1] and len([s for s in engine.steps if s == [1]]) == 3  # 3 full batches and a last one of 1
    assert plan_batches([5, 70, 10, 200], 60, 64 * 6, 3, 1000) == [[0, 1], [2], [3]]
    assert plan_batches([5, 70, 10, 100], 60, 64 * 6, 3, 1000) == [[0, 1], [2, 3]]
    assert plan_batches([1, 1, 1], 1, 64 * 8, 2, 1000) == [[0, 1], [2]]
    with pytest.raises(ValueError):
        plan_batches([500], 10, 64 * 4, 2, 1000)
    with pytest.raises(IndexError):
        plan_batches([50], 10, 64 * 4, 2, 40)
    with pytest.raises(ValueError):
        plan_batches([0], 10, 64 * 4, 2, 40)
    # a failing step gives its slots back
    class Broken(FakeEngine):
        def step(self, *a):
            raise RuntimeError("boom")

    engine = Broken()
    with pytest.raises(RuntimeError):
        generate_requests(engine, [[1], [2]], max_new_tokens=3, chooser=argmax_chooser)
    assert engine.cache.live_slots() == []


def test_loop_runs_steps_ahead_when_nobody_watches_them(monkeypatch):
    """With an engine that runs several decode steps in one call (decode_and_choose_many), and no hook, chooser or timer
    that looks at single steps, the loop asks for up to STEPS_AHEAD steps at a time: never past max_new_tokens or the
    model's last position, and a request that meets a stop token among them ends there.  The results are those of the
    loop that goes step by step."""
    from fms_amd.generation import loop
    from fms_amd.generation.loop import STEPS_AHEAD
    from fms_amd.sampling import SamplingParams

    # the prompts' step chooses with the sampling kernel, which needs the GPU: here the largest logit stands in for it
    monkeypatch.setattr(loop, "choose", lambda logits, sampling, seeds, counters: logits.argmax(-1))

    class Ahead(FakeEngine):
        def __init__(self, **kw):
            super().__init__(**kw)
            self.asked = []

        def decode_and_choose(self, slots, tokens, sampling, seeds=None, counters=None):
            return self.decode_and_choose_many(slots, tokens, sampling, seeds, counters, steps=1)[0]

        def decode_and_choose_many(self, slots, tokens, sampling, seeds=None, counters=None, steps=1):
            self.asked.append((len(slots), steps))
            self.cache.extend_many(slots, [steps] * len(slots))
            out, tokens = [], list(tokens)
            for _ in range(steps):
                tokens = [(t + 1) % self.vocab for t in tokens]
                out.append(tokens)
            return out

    greedy = SamplingParams(do_sample=False)
    prompts = [[10, 11, 12], [50], [20, 21], [97, 98]]
    step_by_step = generate_requests(FakeEngine(), prompts, max_new_tokens=11, stop_token_ids=[23, 57], chooser=argmax_chooser)
    engine = Ahead()
    out = generate_requests(engine, prompts, max_new_tokens=11, stop_token_ids=[23, 57], sampling=greedy)
    assert out == step_by_step == [list(range(13, 24)), list(range(51, 58)), [22, 23], list(range(99, 110))]
    # the prompts' step chooses the first token; 10 are left: 4 and 4 ahead, then the 2 that remain.  Request 2 met its
    # stop token in the first call and request 1 in the second: each ended there, and what it chose after was dropped
    assert STEPS_AHEAD == 4 and engine.asked == [(4, 4), (3, 4), (2, 2)]
    assert engine.cache.live_slots() == []
    # the model's last position bounds the steps ahead: a prompt of 2 in a model of 12 positions takes 11 new tokens,
    # the last of which is never fed
    engine = Ahead(max_seq_len=12)
    assert generate_requests(engine, [[1, 2]], max_new_tokens=500, sampling=greedy) == [list(range(3, 14))]
    assert engine.asked == [(1, 4), (1, 4), (1, 2)] and engine.cache.live_slots() == []
    # someone who watches every step gets single steps
    engine = Ahead()
    seen = []
    generate_requests(engine, [[1]], max_new_tokens=6, sampling=greedy, on_step=lambda step, alive, tokens: seen.append(step))
    assert engine.asked == [(1, 1)] * 5 and seen == list(range(6))


def test_padding_helpers_follow_the_reference():
    """tests/utils/test_generate.py:148-198: exact tensors of pad_input_ids."""
    ids, extra = pad_input_ids([torch.arange(1, 5), torch.arange(1, 8)])
    assert ids.tolist() == [[0, 0, 0, 1, 2, 3, 4], [1, 2, 3, 4, 5, 6, 7]]
    assert extra["position_ids"].tolist() == [[0, 0, 0, 0, 1, 2, 3], [0, 1, 2, 3, 4, 5, 6]]
    m = extra["mask"][0]
    assert m[3, 3] == 0 and m[3, 2] == -torch.inf and m[6, 3] == 0 and m[6, 0] == -torch.inf and m[1, 0] == 0 and m[0, 1] == -torch.inf
    assert extra["lengths"] == [4, 7]
    # tests/utils/test_generate.py:139-145 and :281-286
    assert truncate_after_eos(torch.tensor([5, 6, 3, 9, 3]), 3).tolist() == [5, 6, 3]
    assert truncate_after_eos(torch.tensor([5, 6]), None).tolist() == [5, 6]
    assert trim_prefix(torch.tensor([0, 0, 0, 0, 1, 2, 3, 4])).tolist() == [1, 2, 3, 4]
    assert trim_prefix(torch.tensor([0, 0, 0, 0, 1, 2, 3, 4]), 5).tolist() == [0, 0, 0, 0, 1, 2, 3, 4]
    assert trim_prefix(torch.tensor([1, 2, 3, 4, 0, 1])).tolist() == [1, 2, 3, 4, 0, 1]


def test_padding_helpers_reference_vectors():
    """tests/utils/test_generate.py:148-198 (the mask as the reference's test builds it) and :289-323
    (a pad token that is not zero)."""
    prompts = [torch.arange(1, 5), torch.arange(1, 10)]
    for min_pad, pads in ((0, (5, 0)), (64, (60, 55))):
        ids, extra = pad_input_ids(prompts, min_pad_length=min_pad)
        assert ids.dtype == torch.long and extra["position_ids"].dtype == torch.long
        assert ids.tolist() == [[0] * pads[0] + list(range(1, 5)), [0] * pads[1] + list(range(1, 10))]
        assert extra["position_ids"].tolist() == [[0] * pads[0] + list(range(4)), [0] * pads[1] + list(range(9))]
        is_pad = torch.tensor([[1] * pads[0] + [0] * 4, [1] * pads[1] + [0] * 9], dtype=torch.bool)
        expected = (is_pad.unsqueeze(-1) == is_pad.unsqueeze(-2)).tril()
        expected = torch.where(expected.logical_not(), -torch.inf, 0.0)
        torch.testing.assert_close(extra["mask"], expected)
    _, extra = pad_input_ids(prompts, min_pad_length=12, pad_token_id=100256)
    for b, n in enumerate((4, 9)):
        first = 12 - n
        for q in range(first, 12):
            assert (extra["mask"][b, q] == 0).nonzero().flatten().tolist() == list(range(first, q + 1))
        for q in range(first):
            assert extra["mask"][b, q, q] == 0
    ids, extra = pad_input_ids(prompts, padding_side="right", position_ids_offset=3, is_causal_mask=False)
    assert ids[0].tolist() == [1, 2, 3, 4, 0, 0, 0, 0, 0] and extra["position_ids"][0].tolist() == [3, 4, 5, 6, 3, 3, 3, 3, 3]
    assert (extra["mask"][0, 0] == 0).nonzero().flatten().tolist() == [0, 1, 2, 3]
    with pytest.raises(NotImplementedError):
        pad_input_ids(prompts, padding_side="middle")
    # tests/utils/test_generate.py:139-145, :281-286
    result = torch.ones(20)
    result[10] = 5
    assert truncate_after_eos(result, 5).tolist() == [1.0] * 10 + [5.0]
    sentence = torch.cat((torch.zeros(10), torch.ones(20)))
    assert trim_prefix(sentence).tolist() == [1.0] * 20 and trim_prefix(sentence, pad_token_id=2).tolist() == sentence.tolist()
    assert trim_prefix(torch.zeros(4)).tolist() == [0.0] * 4


def test_char_tokenizer():
    """fms/utils/tokenizers.py:97-143 and tests/utils/test_generate.py:33-50: a character is its code point."""
    from fms_amd.tokenizers import CharTokenizer, get_tokenizer

    tok = get_tokenizer("char_tokenizer")
    assert isinstance(tok, CharTokenizer) and tok.vocab_size() == 256 and (tok.bos_token_id, tok.eos_token_id) == (2, 3)
    assert tok.encode("AB é\u4e2d") == [65, 66, 32, 233, 0]
    assert tok.decode([65, 66, 67]) == "ABC"
    ids = tok.convert_tokens_to_ids(tok.tokenize("ABCDE"))
    assert ids == [65, 66, 67, 68, 69] and tok.convert_tokens_to_ids("A") == 65
    assert tok.convert_tokens_to_string(tok.convert_ids_to_tokens(torch.tensor(ids))) == "ABCDE"
    with pytest.raises(RuntimeError):
        tok.convert_tokens_to_ids("AB")
    with pytest.raises(RuntimeError):
        get_tokenizer("/no/such/tokenizer")
    # the Hugging Face arguments of the reference's interface (fms/utils/tokenizers.py:37-64)
    assert tok.encode("AB", add_special_tokens=True) == [2, 65, 66]
    assert tok.decode([2, 65, 66, 3]) == "AB" and tok.decode([2, 65, 3], skip_special_tokens=False) == "\x02A\x03"
    assert isinstance(get_tokenizer("char_tokenizer", style="fms"), CharTokenizer)
    with pytest.raises(RuntimeError):
        get_tokenizer("char_tokenizer", style="sentencepiece")  # no such file
    with pytest.raises(RuntimeError):
        get_tokenizer("char_tokenizer", style="no_such_style")


def test_file_tokenizers_have_the_reference_interface(tmp_path):
    """A sentencepiece model and a tokenizer.json, both made here from a few words: encode/decode with the
    reference's arguments and the four calls its script makes (scripts/inference.py:179-181, 232-234)."""
    from fms_amd.tokenizers import get_tokenizer

    text = "the cat sat on the mat and the dog sat on the log"
    spm = pytest.importorskip("sentencepiece")
    corpus = tmp_path / "corpus.txt"
    corpus.write_text("\n".join([text, "a cat and a dog", "the log and the mat"] * 20))
    spm.SentencePieceTrainer.train(input=str(corpus), model_prefix=str(tmp_path / "tiny"), vocab_size=40, model_type="bpe",
                                   bos_id=1, eos_id=2, unk_id=0, minloglevel=2)
    for style in (None, "sentencepiece"):
        tok = get_tokenizer(str(tmp_path / "tiny.model"), style=style)
        assert (tok.bos_token_id, tok.eos_token_id) == (1, 2) and tok.vocab_size() == 40
        pieces = tok.tokenize("the cat sat")
        ids = tok.convert_tokens_to_ids(pieces)
        assert ids == tok.encode("the cat sat") and tok.encode("the cat sat", add_special_tokens=True) == [1] + ids
        assert tok.convert_ids_to_tokens(torch.tensor(ids)) == pieces and isinstance(tok.convert_tokens_to_ids(pieces[0]), int)
        assert tok.convert_tokens_to_string(pieces) == "the cat sat" == tok.decode([1] + ids + [2])

    tokenizers = pytest.importorskip("tokenizers")
    words = sorted(set(text.split()))
    vocab = {"<s>": 0, "</s>": 1, "<unk>": 2, **{w: i + 3 for i, w in enumerate(words)}}
    tk = tokenizers.Tokenizer(tokenizers.models.WordLevel(vocab, unk_token="<unk>"))
    tk.pre_tokenizer = tokenizers.pre_tokenizers.Whitespace()
    tk.add_special_tokens(["<s>", "</s>"])
    folder = tmp_path / "hf"
    folder.mkdir()
    tk.save(str(folder / "tokenizer.json"))
    for name, style in ((str(folder), None), (str(folder), "hf"), (str(folder / "tokenizer.json"), None)):
        tok = get_tokenizer(name, style=style)
        assert (tok.bos_token_id, tok.eos_token_id) == (0, 1) and tok.vocab_size() == len(vocab)
        pieces = tok.tokenize("the dog sat")
        assert pieces == ["the", "dog", "sat"]
        ids = tok.convert_tokens_to_ids(pieces)
        assert ids == [vocab[w] for w in pieces] == tok.encode("the dog sat") and tok.convert_tokens_to_ids("dog") == vocab["dog"]
        assert tok.encode("the dog sat", add_special_tokens=True) == [0] + ids
        assert tok.convert_ids_to_tokens(ids) == pieces and tok.convert_tokens_to_string(pieces) == "the dog sat"
        assert tok.decode([0] + ids + [1]) == "the dog sat"


def test_command_line_refusals(capsys):
    """scripts/inference.py:23-113: the reference's option names; what this library cannot do is refused with 2
    before anything is loaded, and a machine without a GPU gets this library's own words."""
    from fms_amd.cli.inference import build_parser, main

    options = {a.dest for a in build_parser()._actions}
    assert {"device_type", "architecture", "variant", "model_path", "model_source", "tokenizer", "no_use_cache",
            "unfuse_weights", "default_dtype", "compile", "compile_mode", "deterministic", "distributed", "batch_input",
            "min_pad_length", "attn_name", "context_file"} <= options
    base = ["--tokenizer", "char_tokenizer"]
    assert main(base + ["--variant", "micro", "--distributed"]) == 2
    assert "one process on one GPU" in capsys.readouterr().err
    assert main(base + ["--variant", "micro", "--default_dtype", "fp16"]) == 2
    assert "bf16 or fp32" in capsys.readouterr().err
    assert main(base + ["--variant", "micro", "--attn_name", "sdpa_bidirectional"]) == 2
    capsys.readouterr()
    assert main(base) == 2  # --architecture llama without a variant
    assert "--variant is needed" in capsys.readouterr().err
    with pytest.raises(SystemExit):  # --tokenizer is required, as in the reference
        main(["--variant", "micro"])
    capsys.readouterr()
    if not torch.cuda.is_available():
        assert main(base + ["--variant", "micro"]) == 1
        assert "shows none to PyTorch" in capsys.readouterr().err
        assert main(base + ["--variant", "no-such-variant"]) == 1
        assert "not a registered variant" in capsys.readouterr().err


def test_chat_keeps_the_conversation_in_the_llama_layout(capsys):
    """scripts/chat.py:162-173 (the layout), :217-243 (a turn), :245-281 (the commands): the conversation is one list of
    token ids, bos, the system message between its marks, then [INST] question [/INST] answer eos for every turn; the
    model sees all of it at every question; nothing after an answer's end is kept."""
    import io

    from fms_amd.cli.chat import Conversation, build_parser, main, run_line
    from fms_amd.tokenizers import CharTokenizer

    tok = CharTokenizer()
    seen = []

    def answer(ids, max_new_tokens):
        seen.append((list(ids), max_new_tokens))
        reply = tok.encode(f"answer {len(seen)}") + [tok.eos_token_id] + tok.encode("never kept")
        return reply[:max_new_tokens]

    talk = Conversation(tok, answer, system_message="be brief", max_new_tokens=50)
    out = io.StringIO()
    assert run_line(talk, "hello\n", out) and run_line(talk, "   \n", out)  # an empty line asks nothing
    assert run_line(talk, "/set max_new_tokens=6\n", out) and talk.max_new_tokens == 6
    assert run_line(talk, "and again\n", out)
    assert run_line(talk, "/set max_new_tokens\n", out) and run_line(talk, "/nonsense\n", out) and run_line(talk, "/help\n", out)
    assert run_line(talk, "/buffer\n", out)
    assert not run_line(talk, "/quit\n", out)
    bos, eos = [tok.bos_token_id], [tok.eos_token_id]
    first = bos + tok.encode("<<SYS>>\nbe brief\n<</SYS>>\n\n") + tok.encode("[INST]hello[/INST]")
    second = first + tok.encode("answer 1") + eos + tok.encode("[INST]and again[/INST]")
    assert seen == [(first, 50), (second, 6)]
    assert talk.ids == second + tok.encode("answer") + eos  # six tokens of "answer 2", then the end mark
    printed = out.getvalue().splitlines()
    assert printed[0] == "answer 1" and printed[1] == "answer"
    assert "usage: /set max_new_tokens=100" in printed and "Unknown command: /nonsense" in printed
    assert f"The conversation has {len(talk.ids)} tokens:" in printed and "Exiting..." == printed[-1]
    assert Conversation(tok, answer).ids == bos  # no system message, no marks

    options = {a.dest for a in build_parser()._actions}
    assert {"device_type", "architecture", "variant", "model_path", "model_source", "tokenizer", "no_use_cache", "compile",
            "compile_mode", "deterministic", "distributed", "max_new_tokens", "system_message"} <= options
    assert main(["--tokenizer", "char_tokenizer", "--variant", "micro", "--distributed"]) == 2
    assert main(["--tokenizer", "char_tokenizer"]) == 2
    capsys.readouterr()


def test_sampling_uniforms_are_a_function_of_seed_and_counter():
    from fms_amd.sampling import SamplingParams, request_seed, uniform

    us = [uniform(request_seed(3, r), c) for r in range(4) for c in range(50)]
    assert all(0 <= u < 1 for u in us) and len(set(us)) > 190
    assert 0.35 < sum(us) / len(us) < 0.65
    assert uniform(5, 9) == uniform(5, 9) and uniform(5, 9) != uniform(5, 10) != uniform(6, 9)
    with pytest.raises(ValueError):
        SamplingParams(do_sample=True, temperature=0.0)


def test_bench_refuses_more_than_one_gpu():
    """The benchmark's contract: for N > 1 one line that says so, and exit code 2 (this library runs on one GPU)."""
    import subprocess
    import sys

    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    for args, env in ((["--gpus", "2"], {}), ([], {"WORLD_SIZE": "4"})):
        run = subprocess.run([sys.executable, os.path.join(root, "bench.py"), *args], capture_output=True, text=True,
                             env={**os.environ, **env}, timeout=120)
        assert run.returncode == 2
        assert len(run.stdout.strip().splitlines()) == 1 and "one GPU" in run.stdout


def test_no_gpu_means_a_loud_failure():
    if torch.cuda.is_available():
        pytest.skip("this machine has a GPU")
    with pytest.raises(RuntimeError, match="no CPU path"):
        fms_amd.get_model("llama", "micro", device_type="cpu")
    with pytest.raises(RuntimeError, match="shows none to PyTorch"):  # this library's words, before any allocation
        fms_amd.get_model("llama", "micro", device_type="cuda")
    from fms_amd.kernels import ops

    with pytest.raises(RuntimeError, match="no CPU fallback"):
        ops.embed(torch.zeros(2, dtype=torch.int32), torch.zeros(4, 4))


# --------------------------------------------------------------------------
# the compiled kernels
# --------------------------------------------------------------------------
def test_a_library_older_than_the_sources_is_never_used(tmp_path, monkeypatch):
    import importlib

    build = importlib.import_module("fms_amd.kernels.build")
    folder = tmp_path / "built"
    folder.mkdir()
    lib = folder / build.LIB_NAME
    lib.write_bytes(b"not a library; only its digest is looked at")
    monkeypatch.setattr(build, "build_dirs", lambda: [str(folder)])
    calls = []

    def fake_build(verbose=True):
        calls.append("build")
        return "rebuilt"

    monkeypatch.setattr(build, "build", fake_build)
    (folder / build.DIGEST_NAME).write_text(build.source_digest())
    assert build.ensure_built(verbose=False) == str(lib) and calls == []
    (folder / build.DIGEST_NAME).write_text("0" * 64)  # built from other sources
    assert build.ensure_built(verbose=False) == "rebuilt" and calls == ["build"]
    (folder / build.DIGEST_NAME).unlink()  # no record of what it was built from
    assert build.ensure_built(verbose=False) == "rebuilt"

    def no_compiler(verbose=True):
        raise RuntimeError("hipcc was not found")

    monkeypatch.setattr(build, "build", no_compiler)
    with pytest.raises(RuntimeError, match="does not match the present sources"):
        build.ensure_built(verbose=False)


def test_kernels_compile_without_relative_register_indexing(tmp_path):
    """A private array indexed by a run-time value is addressed through relative register
    indexing (s_set_gpr_idx / v_movrel); the compiler may then write the indexed register
    unconditionally and select afterwards, and an index past the array lands in a live
    register of the same wave.  No kernel here may need that, nor spill registers."""
    import re
    import subprocess

    import importlib

    build = importlib.import_module("fms_amd.kernels.build")
    try:
        hipcc = build.hipcc_path()
    except RuntimeError:
        pytest.skip("no hipcc")
    for src in build.sources():
        out = tmp_path / (os.path.basename(src) + ".s")
        subprocess.run([hipcc, *build.HIPCC_FLAGS, "-I", build.CSRC, "-S", "--cuda-device-only", src, "-o", str(out)],
                       check=True, stdout=subprocess.DEVNULL, stderr=subprocess.DEVNULL)
        text = out.read_text()
        assert not re.search(r"s_set_gpr_idx|v_movrel", text), f"{os.path.basename(src)} uses relative register indexing"
        spills = [int(m) for m in re.findall(r"\.vgpr_spill_count:\s+(\d+)", text)]
        assert spills and max(spills) == 0, f"{os.path.basename(src)} spills registers: {spills}"
