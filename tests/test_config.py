"""Configuration: typed reading of config.json, defaults of the reference, registry, engine TOML."""
import json

import pytest

from atoma_infer_amd.config import (ConfigError, EngineConfig, LlamaConfig, known_architectures, load_model_config,
                                    register_architecture, resolve_architecture, unregister_architecture)
from util import TINY_A, TINY_B


def test_llama_defaults_follow_the_reference():
    """models/src/llama.rs:54-82: kv heads default to the heads, rope_theta to 10000, tied to false."""
    cfg = LlamaConfig.from_dict({"hidden_size": 64, "intermediate_size": 100, "vocab_size": 50, "num_hidden_layers": 1,
                                 "num_attention_heads": 4, "rms_norm_eps": 1e-5, "max_position_embeddings": 32})
    assert cfg.num_key_value_heads == 4 and cfg.rope_theta == 10000.0 and cfg.tie_word_embeddings is False
    assert cfg.rope_scaling is None and cfg.eos_token_id == () and cfg.head_size == 16


def test_llama_reads_every_key():
    cfg = LlamaConfig.from_dict(TINY_B)
    assert (cfg.hidden_size, cfg.intermediate_size, cfg.vocab_size, cfg.num_hidden_layers) == (96, 256, 1000, 3)
    assert (cfg.num_attention_heads, cfg.num_key_value_heads, cfg.head_size) == (3, 3, 32)
    assert cfg.rms_norm_eps == 1e-6 and cfg.rope_theta == 500000.0 and cfg.max_position_embeddings == 256
    assert cfg.eos_token_id == (1, 7)          # a list; TINY_A has a single integer (models/src/llama.rs:29-34)
    assert LlamaConfig.from_dict(TINY_A).eos_token_id == (2,)
    rs = cfg.rope_scaling
    assert (rs.factor, rs.low_freq_factor, rs.high_freq_factor, rs.original_max_position_embeddings, rs.rope_type) \
        == (8.0, 1.0, 4.0, 64, "llama3")
    again = LlamaConfig.from_dict(cfg.to_dict())
    assert again == cfg
    # an optional window of keys: none unless given, kept through to_dict, and its layers' cache plan has it
    assert cfg.sliding_window is None and "sliding_window" not in cfg.to_dict()
    windowed = LlamaConfig.from_dict(dict(TINY_B, sliding_window=48))
    assert windowed.sliding_window == 48 and LlamaConfig.from_dict(windowed.to_dict()) == windowed
    from atoma_infer_amd.cache import plan_cache
    arch = resolve_architecture(windowed.to_dict())
    assert [g.spec.window for g in plan_cache(arch.build(windowed)).groups] == [48]
    with pytest.raises(ConfigError):
        LlamaConfig.from_dict(dict(TINY_B, sliding_window=0))


def test_one_error_lists_every_fault():
    with pytest.raises(ConfigError) as e:
        LlamaConfig.from_dict({"hidden_size": "64", "vocab_size": 0, "num_hidden_layers": 1,
                               "num_attention_heads": 4, "max_position_embeddings": 32})
    msg = str(e.value)
    for part in ("hidden_size", "vocab_size", "intermediate_size", "rms_norm_eps"):
        assert part in msg


@pytest.mark.parametrize("patch,needle", [
    ({"num_attention_heads": 5}, "multiple"),
    ({"num_key_value_heads": 3}, "num_key_value_heads"),
    ({"head_dim": 32}, "head_dim"),
    ({"hidden_act": "gelu"}, "hidden_act"),
    ({"attention_bias": True}, "bias"),
    ({"rms_norm_eps": 0.0}, "rms_norm_eps"),
    ({"eos_token_id": 99999}, "eos_token_id"),
    ({"rope_scaling": {"factor": 8.0}}, "rope_scaling"),
    ({"rope_scaling": {"factor": 8.0, "low_freq_factor": 1.0, "high_freq_factor": 1.0,
                       "original_max_position_embeddings": 64, "rope_type": "llama3"}}, "division"),
    ({"rope_scaling": {"factor": 8.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0,
                       "original_max_position_embeddings": 64, "rope_type": "yarn"}}, "yarn"),
])
def test_what_the_architecture_cannot_run_is_refused(patch, needle):
    with pytest.raises(ConfigError) as e:
        LlamaConfig.from_dict(dict(TINY_A, **patch))
    assert needle in str(e.value)


def test_head_dim_key_is_accepted_when_it_agrees():
    assert LlamaConfig.from_dict(dict(TINY_A, head_dim=16)).head_size == 16


def test_registry_resolves_by_architectures_then_model_type(tmp_path):
    assert "LlamaForCausalLM" in known_architectures()
    assert resolve_architecture({"architectures": ["LlamaForCausalLM"]}).config_cls is LlamaConfig
    assert resolve_architecture({"model_type": "llama"}).config_cls is LlamaConfig
    with pytest.raises(ConfigError) as e:
        resolve_architecture({"architectures": ["MambaForCausalLM"]})
    assert "LlamaForCausalLM" in str(e.value)
    with pytest.raises(ConfigError):
        resolve_architecture({})
    (tmp_path / "config.json").write_text(json.dumps(TINY_A))
    arch, cfg = load_model_config(str(tmp_path))
    assert arch.name in ("LlamaForCausalLM", "llama") and cfg.hidden_size == 64
    spec = arch.build(cfg)
    assert len(spec.layers) == 2 and len(spec.run_order) == 2
    with pytest.raises(ConfigError):
        load_model_config(str(tmp_path / "nowhere"))


def test_registering_another_architecture():
    marker = object()
    register_architecture("ToyTestArch", LlamaConfig, lambda cfg: marker)
    try:
        assert resolve_architecture({"architectures": ["ToyTestArch"]}).build(None) is marker
        with pytest.raises(ValueError):
            register_architecture("ToyTestArch", LlamaConfig, lambda cfg: None)
    finally:
        unregister_architecture("ToyTestArch")


def test_engine_toml_has_the_references_sections(tmp_path):
    """The reference's own example file parses (backends/vllm/src/tests/test_config.toml)."""
    p = tmp_path / "cfg.toml"
    p.write_text('''
[inference]
api_key = ""
cache_dir = "./cache/"
flush_storage = true
model_name = "/models/tiny"
device_ids = [0]
dtype = "bf16"
num_tokenizer_workers = 4
revision = "main"
[cache]
block_size = 16
cache_dtype = "bf16"
gpu_memory_utilization = 0.5
swap_space_fraction = 0.1
[scheduler]
max_num_batched_tokens = 1024
max_num_sequences = 32
max_model_len = 1024
delay_factor = 0.8
enable_chunked_prefill = false
block_size = 16
[validation]
best_of = 1
max_stop_sequences = 1
max_top_n_tokens = 1
max_input_length = 4096
max_total_tokens = 8192
''')
    cfg = EngineConfig.from_toml(str(p))
    assert cfg.inference.model_name == "/models/tiny" and cfg.inference.dtype == "bfloat16"
    assert cfg.cache.block_size == 16 and cfg.cache.gpu_memory_utilization == 0.5
    assert cfg.scheduler.max_num_sequences == 32 and cfg.scheduler.enable_chunked_prefill is False
    assert cfg.validation.max_total_tokens == 8192


def test_scheduler_config_checks():
    """backends/vllm/src/config.rs:388-406."""
    with pytest.raises(ConfigError):
        EngineConfig.from_dict({"scheduler": {"max_num_batched_tokens": 512, "max_model_len": 1024,
                                              "enable_chunked_prefill": False}})
    with pytest.raises(ConfigError):
        EngineConfig.from_dict({"scheduler": {"max_num_batched_tokens": 16, "max_num_sequences": 32,
                                              "max_model_len": 8}})
    EngineConfig.from_dict({"scheduler": {"max_num_batched_tokens": 512, "max_model_len": 1024,
                                          "enable_chunked_prefill": True}})
    with pytest.raises(ConfigError):
        EngineConfig.from_dict({"inference": {"dtype": "int4"}})
