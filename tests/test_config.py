"""CPU: typed configuration, registry, engine options."""

import json

import pytest

from conftest import TINY_A, TINY_B
from cie_amd.config import (
    ARCHITECTURES, ConfigError, LayerCall, ModelSpec, PartSpec, Qwen2Config, build_engine_config,
    config_from_dict, load_config, register_architecture,
)


def test_reads_every_size_from_config_json():
    a, b = Qwen2Config.from_hf_config(TINY_A), Qwen2Config.from_hf_config(TINY_B)
    assert (a.hidden_size, a.num_hidden_layers, a.num_attention_heads, a.num_key_value_heads) == (64, 2, 4, 2)
    assert (a.head_dim, a.intermediate_size, a.vocab_size, a.rope_theta, a.rms_norm_eps) == (16, 128, 256, 1e4, 1e-6)
    assert a.tie_word_embeddings and not b.tie_word_embeddings
    assert (b.head_dim, b.num_key_value_heads, b.max_position_embeddings, b.eos_token_id) == (32, 1, 320, 7)


def test_defaults_follow_the_reference():
    raw = {k: v for k, v in TINY_A.items() if k not in ("rope_theta", "attention_bias", "hidden_act", "architectures")}
    config = config_from_dict(raw)  # model_type alone selects the architecture
    assert config.rope_theta == 10000.0 and config.attention_bias is True
    assert Qwen2Config.from_hf_config(dict(TINY_A, head_dim=24)).head_dim == 24


@pytest.mark.parametrize("drop", ["hidden_size", "num_hidden_layers", "num_attention_heads", "num_key_value_heads",
                                  "intermediate_size", "vocab_size", "rms_norm_eps"])
def test_missing_key_is_named(drop):
    raw = {k: v for k, v in TINY_A.items() if k != drop}
    with pytest.raises(ConfigError, match=drop):
        Qwen2Config.from_hf_config(raw)


@pytest.mark.parametrize("change,match", [
    ({"model_type": "llama"}, "unsupported"),
    ({"hidden_act": "gelu"}, "SwiGLU"),
    ({"rope_scaling": {"type": "yarn", "factor": 4}}, "unscaled RoPE"),
    ({"hidden_size": 66}, "not divisible"),
    ({"num_key_value_heads": 3}, "multiple"),
    ({"use_sliding_window": True, "sliding_window": 32}, "sliding_window"),
    ({"rms_norm_eps": 0.0}, "eps"),
    ({"vocab_size": 0}, "vocab_size"),
])
def test_refused_configurations(change, match):
    with pytest.raises(ConfigError, match=match):
        Qwen2Config.from_hf_config(dict(TINY_A, **change))


def test_registry_names_known_architectures(tmp_path):
    assert "Qwen2ForCausalLM" in ARCHITECTURES
    with pytest.raises(ConfigError, match="Qwen2ForCausalLM"):
        config_from_dict(dict(TINY_A, architectures=["MixtralForCausalLM"]))
    (tmp_path / "config.json").write_text(json.dumps(TINY_B))
    assert load_config(tmp_path) == Qwen2Config.from_hf_config(TINY_B)
    with pytest.raises(FileNotFoundError):
        load_config(tmp_path / "nowhere")


def test_round_trip_through_config_json():
    config = Qwen2Config.from_hf_config(TINY_B)
    assert config_from_dict(config.to_hf_config()) == config


def test_model_spec_lists_layers_and_order():
    spec = Qwen2Config.from_hf_config(TINY_B).model_spec()
    assert len(spec.layers) == 3 and [c.layer for c in spec.order] == [0, 1, 2]
    assert [c.cache for c in spec.order] == [0, 1, 2] and spec.cache_units == 3
    mixer = spec.layers[0].mixer.as_dict()
    assert mixer["num_heads"] == 3 and mixer["num_kv_heads"] == 1 and mixer["head_dim"] == 32
    assert mixer["position"].as_dict() == {"head_dim": 32, "theta": 1e6, "max_position": 320}
    assert spec.layers[0].norm1.as_dict() == {"size": 96, "eps": 1e-5}
    assert spec.layers[0].name_of("mixer") == "self_attn" and spec.layers[0].name_of("feed_forward") == "mlp"


def test_run_order_is_data():
    base = Qwen2Config.from_hf_config(TINY_A).model_spec()
    fields = dict(architecture="x", vocab_size=8, hidden_size=64, layers=base.layers, final_norm=base.final_norm,
                  tie_word_embeddings=True, max_position=16)
    twice = ModelSpec(order=(LayerCall(0, 0), LayerCall(1, 1), LayerCall(0, 2)), **fields)
    assert twice.cache_units == 3
    shared = ModelSpec(order=(LayerCall(0, 0), LayerCall(1, 0, writes=False)), **fields)
    assert shared.cache_units == 1
    with pytest.raises(ValueError, match="never written"):
        ModelSpec(order=(LayerCall(0, 0), LayerCall(1, 1, writes=False)), **fields)
    with pytest.raises(ValueError, match="names layer 5"):
        ModelSpec(order=(LayerCall(5, 0),), **fields)


def test_engine_options():
    config = build_engine_config(dtype="bf16", page_size=8, token_budget=48)
    assert config.dtype == "bfloat16" and config.page_size == 8 and config.token_budget == 48
    assert build_engine_config(dtype="fp32").dtype == "float32"
    with pytest.raises(ValueError, match="unknown config overrides.*block_sizes"):
        build_engine_config(block_sizes=16)
    with pytest.raises(ValueError, match="power of two"):
        build_engine_config(page_size=12)
    with pytest.raises(ValueError, match="dtype"):
        build_engine_config(dtype="float16")
    with pytest.raises(ValueError, match="token_budget"):
        build_engine_config(token_budget=0)
    with pytest.raises(ValueError, match="kv_cache_fraction"):
        build_engine_config(kv_cache_fraction=0.0)
    with pytest.raises(ValueError, match="kv_cache_bytes"):
        build_engine_config(kv_cache_bytes=0)
    assert build_engine_config().kv_cache_bytes is None and build_engine_config().kv_cache_fraction == 0.9


def test_engine_options_under_the_references_names():
    """src/cloud_engine/config.py:25-48 names six of the options otherwise; both names mean the same."""
    theirs = build_engine_config(max_active_sequences=5, max_batched_tokens=96, prefill_chunk_size=24, block_size=8,
                                 prefix_cache_max_blocks=7, cuda_graph_decode=False, kv_cache_bytes=1 << 20)
    ours = build_engine_config(max_running=5, token_budget=96, prefill_chunk=24, page_size=8, prefix_cache_pages=7,
                               graph_decode=False, kv_cache_bytes=1 << 20)
    assert theirs == ours
    with pytest.raises(ValueError, match="block_size and page_size name the same option"):
        build_engine_config(block_size=8, page_size=16)
    with pytest.raises(ValueError, match="max_batched_tokens|token_budget"):
        build_engine_config(max_batched_tokens=0)


def test_another_architecture_registers_without_touching_the_package():
    class ToyConfig(Qwen2Config):
        architecture = "ToyForCausalLM"

    register_architecture("ToyForCausalLM", ToyConfig)
    try:
        config = config_from_dict(dict(TINY_A, architectures=["ToyForCausalLM"]))
        assert type(config) is ToyConfig and config.model_spec().architecture == "ToyForCausalLM"
    finally:
        ARCHITECTURES.pop("ToyForCausalLM")


def test_part_spec_is_hashable_and_sorted():
    a = PartSpec.of("rms_norm", size=8, eps=1e-6)
    assert a == PartSpec.of("rms_norm", eps=1e-6, size=8) and hash(a) == hash(PartSpec.of("rms_norm", eps=1e-6, size=8))


def test_command_line_without_a_gpu(tmp_path):
    """What of ``cie`` needs no GPU: the registry's names, a model folder with random weights, the benchmark's refusal
    of more than one GPU handed through."""
    import json
    import subprocess
    import sys

    from conftest import ROOT, TINY_B

    cie = [sys.executable, str(ROOT / "bin" / "cie")]
    done = subprocess.run(cie + ["models"], capture_output=True, text=True, timeout=120)
    assert done.returncode == 0 and "Qwen2ForCausalLM" in json.loads(done.stdout)["architectures"]
    (tmp_path / "config.json").write_text(json.dumps(TINY_B))
    done = subprocess.run(cie + ["init-model", "--config", str(tmp_path / "config.json"), "--out", str(tmp_path / "model"),
                                 "--seed", "3"], capture_output=True, text=True, timeout=120)
    assert done.returncode == 0, done.stderr[-2000:]
    assert (tmp_path / "model" / "model.safetensors").is_file()
    assert json.loads((tmp_path / "model" / "config.json").read_text())["hidden_size"] == TINY_B["hidden_size"]
    done = subprocess.run(cie + ["bench", "--gpus", "4"], capture_output=True, text=True, timeout=120)
    assert done.returncode == 2 and "one GPU" in done.stdout
