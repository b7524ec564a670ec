"""Weights: the safetensors reader and writer, loading by tensor name, one error for everything
that is wrong, the random-weights mode.  The reference's counterparts: tests/gguf_tests.cpp:65-82
(truncated file, bad header, unsupported type) and tests/host_model_tests.cpp:169-184 (every
tensor x {missing, bad shape})."""
import json
import os
import struct

import pytest
import torch

from conftest import TINY
from mini_llm_runtime_amd.config import config_from_dict
from mini_llm_runtime_amd.parts import expected_tensors
from mini_llm_runtime_amd.weights import (SafetensorsError, SafetensorsFile, WeightError, WeightSpec, load_weights,
                                          random_tensors, write_random_model, write_safetensors)


def test_writer_agrees_with_the_safetensors_package(tmp_path):
    from safetensors.torch import load_file, save_file
    g = torch.Generator().manual_seed(0)
    tensors = {"a.weight": torch.randn((5, 7), generator=g).to(torch.bfloat16), "b": torch.randn(9, generator=g),
               "c.table": torch.arange(12, dtype=torch.int64).view(3, 4), "d": torch.randn((2, 3), generator=g).half()}
    ours, theirs = str(tmp_path / "ours.safetensors"), str(tmp_path / "theirs.safetensors")
    write_safetensors(ours, tensors)
    save_file(tensors, theirs)
    back = load_file(ours)
    f = SafetensorsFile(theirs)
    for name, t in tensors.items():
        assert torch.equal(back[name], t)
        assert f.entries[name] == (t.dtype, tuple(t.shape))
        assert torch.equal(f.tensor(name).clone(), t)
    f.close()


def test_reader_refuses_broken_files(tmp_path):
    path = str(tmp_path / "x.safetensors")
    with pytest.raises(SafetensorsError):
        SafetensorsFile(path)
    open(path, "wb").write(b"\x01\x02")
    with pytest.raises(SafetensorsError, match="truncated"):
        SafetensorsFile(path)
    open(path, "wb").write(struct.pack("<Q", 1000) + b"{}")
    with pytest.raises(SafetensorsError, match="header length"):
        SafetensorsFile(path)
    open(path, "wb").write(struct.pack("<Q", 4) + b"nope")
    with pytest.raises(SafetensorsError, match="JSON"):
        SafetensorsFile(path)

    def with_header(header, data=b""):
        text = json.dumps(header).encode()
        open(path, "wb").write(struct.pack("<Q", len(text)) + text + data)
    with_header({"w": {"dtype": "F32", "shape": [2, 2], "data_offsets": [0, 16]}}, b"\0" * 12)
    with pytest.raises(SafetensorsError, match="byte range"):
        SafetensorsFile(path)
    with_header({"w": {"dtype": "F32", "shape": [2, 2], "data_offsets": [0, 8]}}, b"\0" * 16)
    with pytest.raises(SafetensorsError, match="byte range"):
        SafetensorsFile(path)
    with_header({"w": {"dtype": "F8_E4M3", "shape": [4], "data_offsets": [0, 4]}}, b"\0" * 4)
    with pytest.raises(SafetensorsError, match="unsupported dtype"):
        SafetensorsFile(path)
    with_header({"w": {"dtype": "F32", "shape": [1]}}, b"\0" * 4)
    with pytest.raises(SafetensorsError, match="malformed"):
        SafetensorsFile(path)


def folder_with(tmp_path, cfg_name, mutate=None, dtype=torch.bfloat16):
    cfg = config_from_dict(TINY[cfg_name])
    folder = str(tmp_path / f"m{len(os.listdir(tmp_path))}")
    os.makedirs(folder)
    tensors = random_tensors(expected_tensors(cfg), seed=3, dtype=dtype)
    if mutate:
        mutate(tensors)
    json.dump(cfg.to_dict(), open(os.path.join(folder, "config.json"), "w"))
    write_safetensors(os.path.join(folder, "model.safetensors"), tensors)
    return cfg, folder


def test_names_and_shapes_of_the_architecture():
    cfg = config_from_dict(TINY["B"])
    exp = expected_tensors(cfg)
    assert exp["model.embed_tokens.weight"].shape == (311, 80)
    assert exp["model.layers.2.self_attn.q_proj.weight"].shape == (128, 80)
    assert exp["model.layers.0.self_attn.k_proj.weight"].shape == (32, 80)
    assert exp["model.layers.0.self_attn.o_proj.weight"].shape == (80, 128)
    assert exp["model.layers.1.self_attn.q_norm.weight"].shape == (32,)
    assert exp["model.layers.1.mlp.down_proj.weight"].shape == (80, 208)
    assert exp["model.norm.weight"].shape == (80,) and exp["model.norm.weight"].keep_float32
    assert not exp["lm_head.weight"].optional
    assert expected_tensors(config_from_dict(TINY["A"]))["lm_head.weight"].optional
    assert len(exp) == 3 + 11 * 3


def test_load_keeps_types(tmp_path):
    cfg, folder = folder_with(tmp_path, "A")
    exp = expected_tensors(cfg)
    w = load_weights(folder, exp, torch.bfloat16, "cpu")
    assert "lm_head.weight" not in w                               # tied: absent from the file
    assert w["model.embed_tokens.weight"].dtype == torch.bfloat16
    assert w["model.layers.0.mlp.up_proj.weight"].dtype == torch.bfloat16
    assert w["model.norm.weight"].dtype == torch.float32           # norms are computed in 32-bit
    w32 = load_weights(folder, exp, torch.float32, "cpu")
    assert all(t.dtype == torch.float32 for t in w32.values())
    assert torch.equal(w32["model.embed_tokens.weight"], w["model.embed_tokens.weight"].float())
    # a file stored in 32-bit: the float engine keeps every bit, the bfloat16 engine rounds matrices once
    cfg, folder = folder_with(tmp_path, "A", dtype=torch.float32)
    raw = SafetensorsFile(os.path.join(folder, "model.safetensors"))
    stored = raw.tensor("model.layers.1.self_attn.v_proj.weight").clone()
    stored_norm = raw.tensor("model.layers.1.input_layernorm.weight").clone()
    raw.close()
    w32 = load_weights(folder, exp, torch.float32, "cpu")
    assert torch.equal(w32["model.layers.1.self_attn.v_proj.weight"], stored)
    wb = load_weights(folder, exp, torch.bfloat16, "cpu")
    assert torch.equal(wb["model.layers.1.self_attn.v_proj.weight"], stored.to(torch.bfloat16))
    assert torch.equal(wb["model.layers.1.input_layernorm.weight"], stored_norm)     # stays 32-bit


def test_integer_tables_become_int32(tmp_path):
    path = str(tmp_path / "model.safetensors")
    write_safetensors(path, {"table": torch.arange(6, dtype=torch.int64).view(2, 3)})
    w = load_weights(str(tmp_path), {"table": WeightSpec((2, 3))}, torch.bfloat16, "cpu")
    assert w["table"].dtype == torch.int32 and w["table"].tolist() == [[0, 1, 2], [3, 4, 5]]


def test_one_error_lists_everything(tmp_path):
    def mutate(t):
        del t["model.layers.0.self_attn.q_norm.weight"]
        del t["model.norm.weight"]
        t["model.layers.0.extra.weight"] = torch.zeros(3)
        t["model.layers.1.mlp.gate_proj.weight"] = torch.zeros((128, 65), dtype=torch.bfloat16)
        t["model.embed_tokens.weight"] = torch.zeros((255, 64), dtype=torch.bfloat16)
    cfg, folder = folder_with(tmp_path, "A", mutate)
    with pytest.raises(WeightError) as info:
        load_weights(folder, expected_tensors(cfg), torch.bfloat16, "cpu")
    text = str(info.value)
    for piece in ("missing tensors (2)", "model.layers.0.self_attn.q_norm.weight", "model.norm.weight",
                  "unexpected tensors (1)", "model.layers.0.extra.weight", "wrong shapes (2)",
                  "model.layers.1.mlp.gate_proj.weight: expected [128, 64], found [128, 65]",
                  "model.embed_tokens.weight: expected [256, 64], found [255, 64]"):
        assert piece in text, piece


def test_every_tensor_missing_or_misshapen_is_refused(tmp_path):
    cfg = config_from_dict(TINY["B"])
    for name, spec in expected_tensors(cfg).items():
        def drop(t, name=name):
            del t[name]

        def reshape(t, name=name, spec=spec):
            shape = list(spec.shape)
            shape[-1] += 1
            t[name] = torch.zeros(shape, dtype=torch.bfloat16)
        for mutate in (drop, reshape):
            _, folder = folder_with(tmp_path, "B", mutate)
            with pytest.raises(WeightError, match=name.replace(".", r"\.")):
                load_weights(folder, expected_tensors(cfg), torch.bfloat16, "cpu")


def test_untied_needs_lm_head_and_tied_may_carry_one(tmp_path):
    cfg, folder = folder_with(tmp_path, "A", lambda t: t.update({"lm_head.weight": torch.ones((256, 64))}))
    w = load_weights(folder, expected_tensors(cfg), torch.float32, "cpu")
    assert "lm_head.weight" in w


def test_nonfinite_weight_is_refused(tmp_path):
    def mutate(t):
        t["model.layers.1.mlp.down_proj.weight"][0, 0] = float("inf")
    cfg, folder = folder_with(tmp_path, "A", mutate)
    with pytest.raises(WeightError, match="not finite"):
        load_weights(folder, expected_tensors(cfg), torch.bfloat16, "cpu")


def test_missing_file_and_shards(tmp_path):
    with pytest.raises(WeightError, match="no model.safetensors"):
        load_weights(str(tmp_path), {}, torch.float32, "cpu")
    cfg = config_from_dict(TINY["A"])
    tensors = random_tensors(expected_tensors(cfg), seed=1)
    names = sorted(tensors)
    half = len(names) // 2
    write_safetensors(str(tmp_path / "s1.safetensors"), {n: tensors[n] for n in names[:half]})
    write_safetensors(str(tmp_path / "s2.safetensors"), {n: tensors[n] for n in names[half:]})
    index = {"weight_map": {n: ("s1.safetensors" if i < half else "s2.safetensors") for i, n in enumerate(names)}}
    json.dump(index, open(tmp_path / "model.safetensors.index.json", "w"))
    w = load_weights(str(tmp_path), expected_tensors(cfg), torch.bfloat16, "cpu")
    assert torch.equal(w[names[0]].float(), tensors[names[0]].float())
    assert torch.equal(w[names[-1]].float(), tensors[names[-1]].float())


def test_random_mode_is_seeded(tmp_path):
    cfg = config_from_dict(TINY["C"])
    a = write_random_model(str(tmp_path / "a"), cfg, seed=5)
    b = write_random_model(str(tmp_path / "b"), cfg, seed=5)
    c = write_random_model(str(tmp_path / "c"), cfg, seed=6)
    fa, fb, fc = (SafetensorsFile(os.path.join(d, "model.safetensors")) for d in (a, b, c))
    assert set(fa.entries) == set(expected_tensors(cfg))
    name = "model.layers.1.self_attn.k_proj.weight"
    assert torch.equal(fa.tensor(name).clone(), fb.tensor(name).clone())
    assert not torch.equal(fa.tensor(name).clone(), fc.tensor(name).clone())
    t = fa.tensor(name).float()
    assert t.dtype == torch.float32 and abs(t.std().item() - 0.02) < 0.004
    n = fa.tensor("model.layers.0.input_layernorm.weight").float()
    assert abs(n.mean().item() - 1.0) < 0.1
    assert json.load(open(os.path.join(a, "config.json")))["head_dim"] == 48
    # a tensor's values do not depend on which other tensors exist
    other = config_from_dict(dict(TINY["C"], num_hidden_layers=1))
    d = write_random_model(str(tmp_path / "d"), other, seed=5)
    fd = SafetensorsFile(os.path.join(d, "model.safetensors"))
    assert torch.equal(fd.tensor("model.embed_tokens.weight").clone(), fa.tensor("model.embed_tokens.weight").clone())
    for f in (fa, fb, fc, fd):
        f.close()


def test_the_command_line_inspects_a_folder_without_a_gpu(tmp_path):
    """`mini-llm --model DIR --inspect` (the reference's --inspect, apps/mini_main.cpp:54-69): architecture,
    configuration, files, tensor count, and whether the tensors are the expected ones."""
    import json
    import os
    import subprocess
    import sys
    from safetensors.torch import load_file, save_file
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    folder = str(tmp_path / "m")
    config = config_from_dict(dict(architectures=["Qwen3ForCausalLM"], hidden_size=32, num_hidden_layers=2,
                                   num_attention_heads=2, num_key_value_heads=1, head_dim=16, intermediate_size=48,
                                   vocab_size=50, max_position_embeddings=128, rms_norm_eps=1e-6, rope_theta=10000.0,
                                   tie_word_embeddings=True))
    write_random_model(folder, config, seed=1)

    def inspect():
        done = subprocess.run([sys.executable, os.path.join(root, "bin", "mini-llm"), "--model", folder, "--inspect"],
                              capture_output=True, text=True, timeout=120)
        assert done.returncode == 0, done.stderr
        return json.loads(done.stdout)
    report = inspect()
    assert report["architecture"] == "Qwen3ForCausalLM" and report["dimensions"]["head_dim"] == 16
    assert report["tensors"] == 2 + 2 * 11 and report["complete"] and report["files"] == ["model.safetensors"]
    path = os.path.join(folder, "model.safetensors")
    tensors = load_file(path)
    del tensors["model.layers.1.mlp.up_proj.weight"]
    save_file(tensors, path)
    report = inspect()
    assert not report["complete"] and "model.layers.1.mlp.up_proj.weight" in report["problems"]
