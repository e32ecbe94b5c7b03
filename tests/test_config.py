"""Configuration and registry (CPU)."""
import json

import pytest

from sonicboom_amd.config import (ConfigError, Qwen2Config, architecture_of, load_config,
                                  registered_architectures)
from sonicboom_amd.architectures.qwen2 import build_spec


def test_reads_every_size_from_its_own_keys(tiny_configs):
    a = Qwen2Config.from_dict(tiny_configs["A"])
    b = Qwen2Config.from_dict(tiny_configs["B"])
    assert (a.num_hidden_layers, a.hidden_size, a.num_attention_heads, a.num_key_value_heads) == (2, 64, 4, 2)
    assert (a.head_dim, a.intermediate_size, a.vocab_size) == (16, 128, 256)
    assert (a.rope_theta, a.rms_norm_eps, a.max_position_embeddings, a.tie_word_embeddings) == (1e4, 1e-6, 128, True)
    assert (b.num_hidden_layers, b.hidden_size, b.num_attention_heads, b.num_key_value_heads) == (3, 96, 3, 1)
    assert (b.head_dim, b.intermediate_size, b.vocab_size) == (32, 224, 384)
    assert (b.rope_theta, b.rms_norm_eps, b.tie_word_embeddings, b.eos_token_ids) == (1e6, 1e-5, False, (7,))


def test_benchmark_shape():
    """The 7B sizes of the reference's frozen facts
    (/root/reference/tests/core/test_qwen2_config.cpp:62-75)."""
    c = Qwen2Config.from_dict({
        "architectures": ["Qwen2ForCausalLM"], "num_hidden_layers": 28, "hidden_size": 3584,
        "num_attention_heads": 28, "num_key_value_heads": 4, "intermediate_size": 18944,
        "vocab_size": 152064, "rope_theta": 1e6, "rms_norm_eps": 1e-6, "max_position_embeddings": 32768})
    assert (c.head_dim, c.q_width, c.kv_width) == (128, 3584, 512)
    spec = build_spec(c)
    assert len(spec.blocks) == 28 and len(spec.order) == 28
    n_params = sum(int(__import__("numpy").prod(t.shape)) for t in spec.all_tensors())
    assert 7.5e9 < n_params < 7.7e9


@pytest.mark.parametrize("key", ["vocab_size", "hidden_size", "intermediate_size", "num_hidden_layers",
                                 "num_attention_heads", "num_key_value_heads", "rms_norm_eps", "rope_theta"])
def test_required_keys_are_named(tiny_configs, key):
    d = dict(tiny_configs["A"])
    del d[key]
    with pytest.raises(ConfigError, match=key):
        Qwen2Config.from_dict(d)


@pytest.mark.parametrize("patch, word", [
    ({"num_key_value_heads": 3}, "num_key_value_heads"),
    ({"hidden_size": 66}, "hidden_size"),
    ({"rope_theta": 0.0}, "rope_theta"),
    ({"rms_norm_eps": -1.0}, "rms_norm_eps"),
    ({"hidden_act": "gelu"}, "hidden_act"),
    ({"use_sliding_window": True}, "use_sliding_window"),
    ({"rope_scaling": {"type": "longrope", "factor": 2.0}}, "rope scaling"),
    ({"vocab_size": 12.5}, "vocab_size"),
    ({"tie_word_embeddings": 1}, "tie_word_embeddings"),
    ({"head_dim": 32}, "head_dim"),
    ({"eos_token_id": 999}, "eos_token_id"),
    ({"hidden_size": 60, "num_attention_heads": 4}, "odd"),
])
def test_rejections(tiny_configs, patch, word):
    d = dict(tiny_configs["A"])
    d.update(patch)
    with pytest.raises(ConfigError, match=word):
        Qwen2Config.from_dict(d)


def test_round_trip(tiny_configs):
    for d in tiny_configs.values():
        c = Qwen2Config.from_dict(d)
        assert Qwen2Config.from_dict(json.loads(json.dumps(c.to_dict()))) == c


def test_registry(tiny_configs, tmp_path):
    assert "Qwen2ForCausalLM" in registered_architectures()
    assert architecture_of(tiny_configs["A"]).name == "Qwen2ForCausalLM"
    with pytest.raises(ConfigError, match="unknown architecture: LlamaForCausalLM.*Qwen2ForCausalLM"):
        architecture_of({"architectures": ["LlamaForCausalLM"]})
    with pytest.raises(ConfigError, match="architectures"):
        architecture_of({})
    (tmp_path / "config.json").write_text(json.dumps(tiny_configs["B"]))
    arch, cfg = load_config(str(tmp_path))
    assert arch.name == "Qwen2ForCausalLM" and cfg.hidden_size == 96
    with pytest.raises(ConfigError, match="no config.json"):
        load_config(str(tmp_path / "nowhere"))


def test_stop_ids_of_generation_config_are_added(tiny_configs, tmp_path):
    """B's config.json names eos 7; the folder's generation_config.json adds 9 and repeats 7."""
    (tmp_path / "config.json").write_text(json.dumps(tiny_configs["B"]))
    (tmp_path / "generation_config.json").write_text(json.dumps({"eos_token_id": [9, 7], "temperature": 0.7}))
    _, cfg = load_config(str(tmp_path))
    assert cfg.eos_token_ids == (7, 9) and build_spec(cfg).stop_tokens == (7, 9)
    (tmp_path / "generation_config.json").write_text(json.dumps({"eos_token_id": 7}))
    assert load_config(str(tmp_path))[1].eos_token_ids == (7,)
    (tmp_path / "generation_config.json").write_text(json.dumps({"eos_token_id": 100000}))
    with pytest.raises(ConfigError, match="eos_token_id"):
        load_config(str(tmp_path))                       # outside the vocabulary
    (tmp_path / "generation_config.json").write_text("{not json")
    with pytest.raises(ConfigError, match="generation_config.json"):
        load_config(str(tmp_path))


def test_spec_carries_the_configuration(tiny_configs):
    a = build_spec(Qwen2Config.from_dict(tiny_configs["A"]))
    b = build_spec(Qwen2Config.from_dict(tiny_configs["B"]))
    c = build_spec(Qwen2Config.from_dict(tiny_configs["C"]))
    ma, mb = a.blocks[0].parts["mixer"], b.blocks[0].parts["mixer"]
    assert (ma.params["heads_q"], ma.params["heads_kv"], ma.params["head_dim"]) == (4, 2, 16)
    assert (mb.params["heads_q"], mb.params["heads_kv"], mb.params["head_dim"]) == (3, 1, 32)
    assert ma.parts["position"].params["base"] == 1e4 and mb.parts["position"].params["base"] == 1e6
    assert a.blocks[0].parts["mixer_norm"].params["eps"] == 1e-6
    assert b.blocks[0].parts["ffn_norm"].params["eps"] == 1e-5
    # tied head: the head names the embedding table, and a stray lm_head is tolerated
    assert a.head.tensors["weight"].name == "model.embed_tokens.weight"
    assert a.ignorable_tensors == ("lm_head.weight",)
    assert b.head.tensors["weight"].name == "lm_head.weight"
    assert b.stop_tokens == (7,) and c.stop_tokens == (5, 9)
    pos = c.blocks[0].parts["mixer"].parts["position"].params
    assert len(pos["freq_factors"]) == 24 and pos["score_scale"] > 1.0
    # the yarn table leaves fast pairs alone and slows the slow ones by the factor
    assert pos["freq_factors"][0] == 1.0 and abs(pos["freq_factors"][-1] - 4.0) < 1e-6
