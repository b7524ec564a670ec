"""Configuration: config.json keys, checks (after src/minillm/qwen3_model.cpp:9-40) and the
architecture registry."""
import copy
import json

import pytest

from conftest import TINY
from mini_llm_runtime_amd.config import (ConfigError, Qwen3Config, config_from_dict, known_architectures,
                                         load_config, register_architecture)


def test_reads_every_size_from_its_key():
    for name, raw in TINY.items():
        cfg = config_from_dict(raw)
        assert isinstance(cfg, Qwen3Config)
        for key in ("hidden_size", "num_hidden_layers", "num_attention_heads", "num_key_value_heads", "head_dim",
                    "intermediate_size", "vocab_size", "max_position_embeddings", "rms_norm_eps", "rope_theta",
                    "tie_word_embeddings"):
            assert getattr(cfg, key) == raw[key], (name, key)
    assert config_from_dict(TINY["C"]).eos_token_ids == (5,)
    assert config_from_dict(TINY["A"]).eos_token_ids == ()


def test_model_spec_describes_the_layers():
    cfg = config_from_dict(TINY["B"])
    spec = cfg.model_spec()
    assert len(spec.layers) == 3 and [r.layer for r in spec.schedule] == [0, 1, 2]
    assert [r.cache for r in spec.schedule] == [0, 1, 2]
    mixer = spec.layers[0].mixer
    assert (mixer.q_heads, mixer.kv_heads, mixer.head_dim, mixer.window) == (4, 1, 32, None)
    assert mixer.scale == pytest.approx(32 ** -0.5)
    assert mixer.qk_norm.size == 32 and mixer.qk_norm.eps == 1e-5
    assert mixer.position.base == 1e6 and mixer.position.dim == 32
    assert spec.layers[0].ffn.intermediate == 208 and spec.final_norm.eps == 1e-5
    assert not spec.tie_embeddings and config_from_dict(TINY["A"]).model_spec().tie_embeddings


def test_round_trip_through_to_dict():
    for raw in TINY.values():
        cfg = config_from_dict(raw)
        assert config_from_dict(cfg.to_dict()) == cfg


def test_head_dim_is_its_own_key():
    raw = dict(TINY["B"])
    assert config_from_dict(raw).head_dim == 32          # not hidden / heads = 20
    del raw["head_dim"]
    assert config_from_dict(raw).head_dim == 20
    raw["hidden_size"] = 81
    with pytest.raises(ConfigError):
        config_from_dict(raw)


@pytest.mark.parametrize("change", [
    {"hidden_size": 0}, {"hidden_size": 2_000_000}, {"num_hidden_layers": -1}, {"num_attention_heads": 3},
    {"head_dim": 15}, {"rms_norm_eps": 0.0}, {"rms_norm_eps": float("inf")}, {"rope_theta": -1.0},
    {"rope_theta": float("nan")}, {"rope_scaling": {"rope_type": "yarn", "factor": 4.0}},
    {"use_sliding_window": True}, {"attention_bias": True}, {"hidden_act": "gelu"},
    {"vocab_size": "many"}, {"tie_word_embeddings": "yes"}, {"intermediate_size": 1.5},
    {"eos_token_id": 10_000}, {"eos_token_id": "x"}, {"num_hidden_layers": True},
    {"use_sliding_window": "no"}, {"attention_bias": 0}, {"model_type": "qwen2"}, {"model_type": 3},
    {"layer_types": ["sliding_attention", "full_attention"]}, {"layer_types": ["full_attention"]},
    {"layer_types": "full_attention"}, {"layer_types": [1, 2]},
])
def test_rejects(change):
    raw = copy.deepcopy(TINY["A"])
    raw.update(change)
    with pytest.raises(ConfigError):
        config_from_dict(raw)


@pytest.mark.parametrize("key", ["hidden_size", "num_hidden_layers", "num_attention_heads", "intermediate_size",
                                 "vocab_size", "max_position_embeddings", "rms_norm_eps", "rope_theta"])
def test_missing_key(key):
    raw = dict(TINY["A"])
    del raw[key]
    with pytest.raises(ConfigError, match=key):
        config_from_dict(raw)


def test_registry():
    assert "Qwen3ForCausalLM" in known_architectures()
    with pytest.raises(ConfigError, match="Qwen3ForCausalLM"):
        config_from_dict(dict(TINY["A"], architectures=["LlamaForCausalLM"]))
    with pytest.raises(ConfigError):
        config_from_dict(dict(TINY["A"], architectures=[]))
    with pytest.raises(ConfigError):
        config_from_dict({k: v for k, v in TINY["A"].items() if k != "architectures"})

    @register_architecture("ToyForTests")
    class Toy:
        @classmethod
        def from_dict(cls, data):
            return cls()
    assert isinstance(config_from_dict({"architectures": ["ToyForTests"]}), Toy)


def test_load_config_from_folder(tmp_path):
    with pytest.raises(ConfigError):
        load_config(str(tmp_path))
    (tmp_path / "config.json").write_text("{not json")
    with pytest.raises(ConfigError):
        load_config(str(tmp_path))
    (tmp_path / "config.json").write_text(json.dumps(TINY["C"]))
    assert load_config(str(tmp_path)).hidden_size == 76
    # keys that other tools write are ignored
    (tmp_path / "config.json").write_text(json.dumps(dict(TINY["C"], torch_dtype="bfloat16", model_type="qwen3",
                                                          sliding_window=None, max_window_layers=2,
                                                          use_sliding_window=False, attention_bias=False,
                                                          layer_types=["full_attention"] * 2,
                                                          use_cache=True, bos_token_id=1)))
    assert load_config(str(tmp_path)).vocab_size == 517


def test_the_benchmark_refuses_more_than_one_gpu():
    """One line and exit code 2, before anything touches a GPU."""
    import os
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    done = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--gpus", "2"], capture_output=True, text=True,
                          timeout=120)
    assert done.returncode == 2 and len(done.stdout.strip().splitlines()) == 1 and "--gpus 2" in done.stdout


def test_the_package_exports_its_entry_points():
    """What a user imports first is at the top level, and importing it touches no GPU."""
    import mini_llm_runtime_amd as package
    from mini_llm_runtime_amd.api import LLM, generate
    assert package.LLM is LLM and package.generate is generate
    for name in package.__all__:
        assert hasattr(package, name), name


def test_profiler_rates_keep_their_leading_digits():
    """A small model's rates (a first product's time holds the library's set-up) must not round to zero."""
    from mini_llm_runtime_amd.kernels.profile import _significant
    assert _significant(0.00012345678) == 0.0001235
    assert _significant(1234.5678) == 1235.0
    assert _significant(0.0) == 0.0
