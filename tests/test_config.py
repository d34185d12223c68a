"""Configuration: keys of config.json, defaults the reference applies to its own
keys, typed errors, the registry."""
import json

import pytest

import transformer_amd as ta
from transformer_amd.config.llama import LlamaConfig
from transformer_amd.config.registry import (UnknownArchitecture, get_architecture,
                                             read_model_folder_config)
from transformer_amd.config.spec import ConfigError, ModelSpec, RunSpec
import plain_llama as P


def test_reads_every_size_from_config_json():
    c = LlamaConfig.from_dict(P.TINY_A)
    assert (c.num_layers, c.hidden, c.num_heads, c.num_kv_heads, c.head_dim) == (2, 64, 4, 2, 16)
    assert (c.intermediate, c.vocab, c.max_position) == (176, 256, 128)
    assert c.rope_theta == 10000.0 and c.rms_eps == 1e-5 and c.tie_embeddings is False
    b = LlamaConfig.from_dict(P.TINY_B)
    assert b.head_dim == 32 and b.num_kv_heads == 3 and b.rope_style == "interleaved"
    assert b.rms_eps == 1e-6 and b.rope_theta == 500000.0 and b.tie_embeddings is True


def test_defaults_mirror_the_reference():
    # models/llama/common/src/storage.rs:54-59
    d = {"num_hidden_layers": 1, "hidden_size": 64, "num_attention_heads": 4,
         "intermediate_size": 32, "vocab_size": 10, "max_position_embeddings": 16}
    c = LlamaConfig.from_dict(d)
    assert c.num_kv_heads == 4 and c.head_dim == 16
    assert c.rms_eps == 1e-5 and c.rope_theta == 1e4 and c.tie_embeddings is None


@pytest.mark.parametrize("key", ["num_hidden_layers", "hidden_size", "num_attention_heads",
                                 "intermediate_size", "vocab_size", "max_position_embeddings"])
def test_missing_required_key_names_the_key(key):
    d = dict(P.TINY_A)
    del d[key]
    with pytest.raises(ConfigError, match=key):
        LlamaConfig.from_dict(d)


def test_refuses_what_it_cannot_run():
    with pytest.raises(ConfigError, match="rope_scaling"):
        LlamaConfig.from_dict({**P.TINY_A, "rope_scaling": {"type": "linear", "factor": 2.0}})
    with pytest.raises(ConfigError, match="hidden_act"):
        LlamaConfig.from_dict({**P.TINY_A, "hidden_act": "gelu"})
    with pytest.raises(ConfigError, match="multiple"):
        LlamaConfig.from_dict({**P.TINY_A, "num_key_value_heads": 3})
    with pytest.raises(ConfigError, match="integer"):
        LlamaConfig.from_dict({**P.TINY_A, "hidden_size": "64"})
    with pytest.raises(ConfigError, match="rope_style"):
        LlamaConfig.from_dict({**P.TINY_A, "rope_style": "spiral"})


def test_round_trip_through_config_json():
    for cfg in (P.TINY_A, P.TINY_B):
        c = LlamaConfig.from_dict(cfg)
        assert LlamaConfig.from_dict(json.loads(json.dumps(c.to_dict()))) == c


def test_stop_ids_from_eos_token_id():
    assert LlamaConfig.from_dict({**P.TINY_A, "eos_token_id": 7}).stop_ids == (7,)
    assert LlamaConfig.from_dict({**P.TINY_A, "eos_token_id": [7, 9]}).stop_ids == (7, 9)


def test_model_spec_spells_out_every_block():
    c = LlamaConfig.from_dict(P.TINY_B)
    s = c.model_spec()
    assert len(s.blocks) == 3 and [r.block for r in s.schedule] == [0, 1, 2]
    m = s.blocks[0].mixer
    assert (m.num_heads, m.num_kv_heads, m.head_dim) == (3, 3, 32)
    assert abs(m.scale - 32 ** -0.5) < 1e-12 and m.qkv_bias and m.position.theta == 500000.0
    assert s.blocks[0].norm1.eps == 1e-6 and s.blocks[0].ffn.intermediate == 256


def test_schedule_validation():
    s = LlamaConfig.from_dict(P.TINY_A).model_spec()
    import dataclasses
    bad = dataclasses.replace(s, schedule=(RunSpec(0), RunSpec(5)))
    with pytest.raises(ConfigError, match="block 5"):
        bad.validate()
    bad = dataclasses.replace(s, schedule=(RunSpec(0, cache_of=0),))
    with pytest.raises(ConfigError, match="earlier"):
        bad.validate()
    ok = dataclasses.replace(s, schedule=(RunSpec(0), RunSpec(1), RunSpec(0), RunSpec(1, cache_of=1)))
    ok.validate()


def test_registry():
    assert get_architecture("LlamaForCausalLM") is get_architecture("llama")
    with pytest.raises(UnknownArchitecture, match="LlamaForCausalLM"):
        get_architecture("GPT2LMHeadModel")
    assert "llama" in ta.known_architectures()


def test_model_class_is_chosen_by_config_json(tmp_path):
    (tmp_path / "config.json").write_text(json.dumps(P.TINY_A))
    arch, cfg = read_model_folder_config(tmp_path)
    assert arch.name == "LlamaForCausalLM" and cfg.hidden == 64
    (tmp_path / "config.json").write_text(json.dumps({**P.TINY_A, "architectures": ["Mamba"]}))
    with pytest.raises(UnknownArchitecture):
        read_model_folder_config(tmp_path)
    (tmp_path / "config.json").write_text("{not json")
    with pytest.raises(ConfigError, match="JSON"):
        read_model_folder_config(tmp_path)


def test_gguf_metadata_defaults():
    meta = {"general.architecture": "llama", "llama.embedding_length": 64, "llama.block_count": 2,
            "llama.attention.head_count": 4, "llama.feed_forward_length": 100,
            "llama.context_length": 32}
    c = LlamaConfig.from_gguf_metadata(meta, vocab_rows=50)
    assert c.num_kv_heads == 4 and c.head_dim == 16 and c.vocab == 50
    assert c.rope_style == "interleaved" and c.rms_eps == 1e-5 and c.rope_theta == 1e4
    with pytest.raises(ConfigError, match="context_length"):
        LlamaConfig.from_gguf_metadata({k: v for k, v in meta.items() if "context" not in k}, 50)


def test_torch_dtype_is_read_and_chooses_the_engines_type_where_none_is_named():
    import plain_llama as P
    import transformer_amd as ta
    base = dict(P.TINY_A)
    assert ta.LlamaConfig.from_dict(base).torch_dtype is None
    assert ta.LlamaConfig.from_dict(base).default_engine_dtype() == "bfloat16"
    for said, engine in (("float32", "float32"), ("bfloat16", "bfloat16"), ("float16", "bfloat16"),
                         ("torch.float32", "float32")):
        cfg = ta.LlamaConfig.from_dict({**base, "torch_dtype": said})
        assert cfg.default_engine_dtype() == engine
        assert ta.LlamaConfig.from_dict(cfg.to_dict()) == cfg           # it survives the round trip
    from transformer_amd.config.spec import ConfigError
    with pytest.raises(ConfigError, match="torch_dtype"):
        ta.LlamaConfig.from_dict({**base, "torch_dtype": 32})
    assert ta.LlamaConfig.from_dict(base).with_layers(1).num_layers == 1
