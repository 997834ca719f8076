"""Configuration and registry (CPU)."""
import json

import pytest

from spyinfer_amd.config import ConfigError, EngineConfig, Qwen3Config, get_architecture, load_model_config, registered_architectures
from tests.configs import TINY_A, TINY_B


def test_defaults_follow_the_reference():
    # src/models/model_config.hpp:34-46
    cfg = Qwen3Config.from_dict(dict(model_type="qwen3", hidden_act="silu", hidden_size=64, intermediate_size=8, num_key_value_heads=2,
                                     num_hidden_layers=1, num_attention_heads=4, vocab_size=10))
    assert cfg.head_dim == 16 and cfg.rope_theta == 1000000.0 and cfg.rms_norm_eps == 1e-6
    assert cfg.max_position_embeddings == 16384 and cfg.tie_word_embeddings is False
    assert cfg.bos_token_id == -1 and cfg.eos_token_id == -1


def test_head_dim_is_its_own_key():
    assert Qwen3Config.from_dict(TINY_B).head_dim == 32 and TINY_B["hidden_size"] // TINY_B["num_attention_heads"] == 12


@pytest.mark.parametrize("change,word", [
    (dict(hidden_act="gelu"), "hidden_act"), (dict(num_key_value_heads=3), "multiple"), (dict(head_dim=15), "even"),
    (dict(vocab_size=0), "vocab_size"), (dict(attention_bias=True), "attention_bias"), (dict(rope_scaling={"type": "yarn"}), "rope_scaling"),
    (dict(use_sliding_window=True), "sliding"), (dict(hidden_size="big"), "hidden_size"), (dict(rms_norm_eps=0.0), "rms_norm_eps"),
    (dict(eos_token_id=[1, 2]), "eos_token_id")])
def test_bad_values_are_refused(change, word):
    raw = dict(TINY_A)
    raw.update(change)
    with pytest.raises(ConfigError, match=word):
        Qwen3Config.from_dict(raw)


def test_required_keys():
    raw = dict(TINY_A)
    del raw["hidden_act"]
    with pytest.raises(ConfigError, match="hidden_act"):
        Qwen3Config.from_dict(raw)


def test_registry(tmp_path):
    assert "Qwen3ForCausalLM" in registered_architectures()
    assert get_architecture("Qwen3ForCausalLM").config_cls is Qwen3Config
    with pytest.raises(ConfigError, match="Qwen3ForCausalLM"):
        get_architecture("LlamaForCausalLM")       # the error lists what is registered
    (tmp_path / "config.json").write_text(json.dumps(TINY_A))
    arch, cfg = load_model_config(str(tmp_path))
    assert arch.name == "Qwen3ForCausalLM" and cfg.hidden_size == 64
    raw = dict(TINY_A)
    del raw["architectures"]
    (tmp_path / "config.json").write_text(json.dumps(raw))
    with pytest.raises(ConfigError, match="architectures"):
        load_model_config(str(tmp_path))


def test_model_is_built_from_configuration_only():
    arch = get_architecture("Qwen3ForCausalLM")
    for raw in (TINY_A, TINY_B):
        m = arch.build(arch.config_cls.from_dict(raw))
        assert len(m.layers) == raw["num_hidden_layers"]
        a = m.layers[0].mixer
        assert (a.num_heads, a.num_kv_heads, a.head_dim) == (raw["num_attention_heads"], raw["num_key_value_heads"], raw["head_dim"])
        assert m.layers[0].norm1.eps == raw["rms_norm_eps"] and a.qk_norm_eps == raw["rms_norm_eps"]
        assert a.position.theta == raw["rope_theta"]
        assert (m.lm_head.tied_to is not None) == raw["tie_word_embeddings"]
        names = [s.name for s in m.weight_specs() if not s.optional]
        assert ("lm_head.weight" in names) == (not raw["tie_word_embeddings"])
        assert len(names) == 2 + 11 * raw["num_hidden_layers"] + (0 if raw["tie_word_embeddings"] else 1)


def test_engine_config():
    c = EngineConfig()
    # names and defaults of src/config.hpp:17-30 (the page size default differs: 16, not 4)
    assert (c.max_num_batched_tokens, c.max_num_seqs, c.max_model_len, c.gpu_memory_utilization) == (16384, 512, 4096, 0.9)
    with pytest.raises(ValueError):
        EngineConfig(dtype="float16").validate()
    with pytest.raises(ValueError):
        EngineConfig(kvcache_block_size=0).validate()
    assert c.weight_copies == "both"
    EngineConfig(weight_copies="tiled").validate()
    with pytest.raises(ValueError):
        EngineConfig(weight_copies="rows").validate()
