"""Typed configuration, registry and launch file (no GPU)."""
import json

import pytest

from rustinfer_amd.config import (ConfigError, EngineConfig, LlamaConfig, load_engine_config,
                                  load_model_config, parse_toml, register_architecture,
                                  registered_architectures, resolve_architecture,
                                  unregister_architecture)

BASE = dict(architectures=["LlamaForCausalLM"], hidden_size=64, intermediate_size=176,
            num_hidden_layers=2, num_attention_heads=4, num_key_value_heads=2, vocab_size=256)


def test_defaults_follow_the_reference():
    # crates/infer-worker/src/bin/worker_main.rs:173-181, :390-392
    c = LlamaConfig.from_dict(BASE)
    assert c.max_position_embeddings == 4096 and c.rms_norm_eps == 1e-5 and c.rope_theta == 10000.0
    assert c.head_dim == 16 and c.rope_scaling is None and c.tie_word_embeddings is False
    assert (c.q_dim, c.kv_dim, c.qkv_dim) == (64, 32, 128)
    assert c.eos_token_ids == (128001, 128008, 128009)


def test_every_key_is_read():
    d = dict(BASE, head_dim=24, max_position_embeddings=77, rms_norm_eps=1e-6, rope_theta=5e5,
             tie_word_embeddings=True, eos_token_id=[3, 4],
             rope_scaling=dict(rope_type="llama3", factor=8.0, low_freq_factor=1.0,
                               high_freq_factor=4.0, original_max_position_embeddings=32))
    c = LlamaConfig.from_dict(d)
    assert c.head_dim == 24 and c.q_dim == 96 and c.max_position_embeddings == 77
    assert c.rms_norm_eps == 1e-6 and c.rope_theta == 5e5 and c.tie_word_embeddings
    assert c.eos_token_ids == (3, 4) and c.rope_scaling.factor == 8.0
    assert c.rope_scaling.original_max_position_embeddings == 32
    assert LlamaConfig.from_dict(c.to_dict()) == c            # what random-weights mode writes reads back


@pytest.mark.parametrize("change,match", [
    (dict(hidden_size=None), "hidden_size"),
    (dict(num_key_value_heads=3), "multiple"),
    (dict(head_dim=15), "even"),
    (dict(head_dim=272), "largest head"),
    (dict(vocab_size=0), "vocab_size"),
    (dict(hidden_act="gelu"), "hidden_act"),
    (dict(attention_bias=True), "attention_bias"),
    (dict(rope_scaling=dict(rope_type="yarn", factor=2.0)), "rope_type"),
    (dict(rope_scaling=dict(rope_type="llama3", factor=8.0)), "low_freq_factor"),
    (dict(rms_norm_eps="x"), "rms_norm_eps"),
    (dict(num_hidden_layers=2.5), "integer"),
])
def test_bad_configs_are_refused(change, match):
    d = dict(BASE, **change)
    d = {k: v for k, v in d.items() if v is not None}
    with pytest.raises(ConfigError, match=match):
        LlamaConfig.from_dict(d)


def test_rope_type_default_means_no_scaling():
    assert LlamaConfig.from_dict(dict(BASE, rope_scaling=dict(rope_type="default"))).rope_scaling is None


def test_registry_resolves_by_architecture_then_model_type():
    # crates/infer-protocol/src/config.rs:498-527
    assert resolve_architecture({"architectures": ["LlamaForCausalLM"]}).name == "LlamaForCausalLM"
    assert resolve_architecture({"model_type": "llama"}).name == "LlamaForCausalLM"
    with pytest.raises(ConfigError, match="unsupported architecture mistral.*LlamaForCausalLM"):
        resolve_architecture({"model_type": "mistral"})
    with pytest.raises(ConfigError, match="missing"):
        resolve_architecture({})
    with pytest.raises(ConfigError, match="Qwen3ForCausalLM"):
        resolve_architecture({"architectures": ["Qwen3ForCausalLM"]})


def test_registry_takes_new_architectures():
    register_architecture("XForCausalLM", LlamaConfig, lambda cfg: ("built", cfg))
    try:
        assert "XForCausalLM" in registered_architectures()
        e = resolve_architecture({"architectures": ["XForCausalLM"]})
        assert e.builder(1) == ("built", 1)
        with pytest.raises(ValueError):
            register_architecture("XForCausalLM", LlamaConfig, lambda cfg: None)
    finally:
        unregister_architecture("XForCausalLM")


def test_load_model_config_and_generation_config(tmp_path):
    (tmp_path / "config.json").write_text(json.dumps(dict(BASE, eos_token_id=5)))
    (tmp_path / "generation_config.json").write_text(json.dumps({"eos_token_id": [7, 8]}))
    entry, cfg = load_model_config(str(tmp_path))
    assert entry.name == "LlamaForCausalLM" and cfg.eos_token_ids == (7, 8)
    with pytest.raises(ConfigError, match="no such file"):
        load_model_config(str(tmp_path / "missing"))


def test_toml_of_the_reference_loads(tmp_path):
    # the reference's own launch file for this architecture (run_llama1b.toml), with our page size
    text = '''
# comment
model = "./models/Llama-3.2-1B-Instruct"
model_name = "Llama-3.2-1B-Instruct"
cluster_id = "rustinfer-llama1b"
device = "cuda:0"
host = "127.0.0.1"
port = 8102
request_timeout_secs = 600
max_batch_tokens = 8192
max_batch_seqs = 32
max_model_len = 4096
batch_wait_ms = 0
paged_block_size = 16
chunked_prefill_size = 0
enable_prefix_caching = false
mem_fraction_static = 0.9
num_blocks = 0
ignore_eos = false
mode = "llm"
worker_id = "worker-0"
log_level = "info"
capture_sizes = [1, 2, 4, 8,
                 16, 24, 32]   # over two lines

[cuda_memory]
kernel_workspace_mib = 256
'''
    p = tmp_path / "run.toml"
    p.write_text(text)
    cfg = load_engine_config(str(p))
    assert cfg.model.endswith("1B-Instruct") and cfg.capture_sizes == (1, 2, 4, 8, 16, 24, 32)
    assert cfg.max_batch_tokens == 8192 and cfg.mem_fraction_static == 0.9 and cfg.dtype == "bfloat16"


def test_engine_config_defaults_and_checks():
    c = EngineConfig(model="m")
    # crates/infer-protocol/src/config.rs:197-262
    assert (c.max_batch_tokens, c.max_batch_seqs, c.max_model_len) == (8192, 32, 4096)
    assert c.capture_sizes == (1, 2, 4, 8, 16, 24, 32, 40, 48, 56, 64) and c.mem_fraction_static == 0.9
    for bad, match in ((dict(model=""), "model"), (dict(mem_fraction_static=0.0), "mem_fraction"),
                       (dict(max_model_len=0), "max_model_len"), (dict(mode="diffusion"), "mode"),
                       (dict(tensor_parallel_size=2), "one GPU"), (dict(dtype="fp8"), "dtype"),
                       (dict(enable_prefix_caching=True), "prefix"), (dict(paged_block_size=0), "paged_block_size")):
        with pytest.raises(ConfigError, match=match):
            EngineConfig.from_dict(dict(dict(model="m"), **bad))
    with pytest.raises(ConfigError, match="unknown keys: bogus"):
        EngineConfig.from_dict(dict(model="m", bogus=1))
    with pytest.raises(ConfigError, match="wrong type"):
        EngineConfig.from_dict(dict(model="m", max_batch_seqs="many"))


def test_toml_parser_values_and_errors():
    d = parse_toml('a = 1\nb = -2.5\nc = "x # y"\nd = true\ne = [1, 2]\nf = 1_000\n[t]\ng = \'lit\'\n[t.u]\nh = 0x10')
    assert d == {"a": 1, "b": -2.5, "c": "x # y", "d": True, "e": [1, 2], "f": 1000,
                 "t": {"g": "lit", "u": {"h": 16}}}
    for bad in ("a", "a = ", "a = [1, 2", "a = 1\na = 2", "[[x]]", 'a = "x'):
        with pytest.raises(ConfigError):
            parse_toml(bad)


def test_random_weights_seed_option():
    assert EngineConfig(model="m").random_weights_seed == -1
    assert EngineConfig.from_dict(dict(model="m", random_weights_seed=7)).random_weights_seed == 7
    with pytest.raises(ConfigError, match="random_weights_seed"):
        EngineConfig.from_dict(dict(model="m", random_weights_seed=-5))


def test_profiler_ranges_cost_nothing_when_off():
    # RUSTINFER_PROFILE_GPU off: one shared null context, no library loaded
    from rustinfer_amd.engine import markers
    markers.set_enabled(False)
    a, b = markers.profile_range("x"), markers.profile_range("y")
    assert a is b
    with a:
        pass
