"""The framework takes parts it has never seen: a toy mixer with fixed-size state of its own and a toy
architecture, both defined here, are registered, built, loaded from a safetensors folder and stepped --
whole and in portions, beside each other in one batch -- without a change to the framework's files.
A second toy architecture shows that the run order is data: a layer named twice, and a run that reads
another run's cache."""
import json
import math
import os

import numpy as np
import pytest
import torch

from plain import qwen3_plain as P

pytestmark = pytest.mark.gpu


def register_toys():
    from dataclasses import dataclass
    from mini_llm_runtime_amd.cache import StateSpec
    from mini_llm_runtime_amd.config import (AttentionSpec, LayerRun, LayerSpec, MlpSpec, ModelSpec, NormSpec,
                                             PositionSpec, register_architecture)
    from mini_llm_runtime_amd.parts import register_part
    from mini_llm_runtime_amd.weights import WeightSpec

    @dataclass(frozen=True)
    class RunningMeanSpec:
        kind: str
        hidden: int

    @register_part("mixer", "toy_running_mean")
    class RunningMean:
        """out_t = gain * mean(x_0 .. x_t): the state of a request is the running sum and the count."""

        def __init__(self, spec):
            self.hidden = spec.hidden
            self.gain = None

        def weight_specs(self):
            return {"gain": WeightSpec((self.hidden,), keep_float32=True)}

        def bind(self, weights):
            self.gain = weights["gain"]

        def cache_spec(self):
            return StateSpec((self.hidden + 1,), torch.float32)

        def libraries(self):
            return []

        def forward(self, ctx, x, cache_id, write_cache=True):
            state = ctx.cache.state_view(cache_id)
            out = torch.empty_like(x)
            for slot, first, n, _ in ctx.segments:
                seg = x[first:first + n].float()
                sums = state[slot, :self.hidden] + torch.cumsum(seg, dim=0)
                count = state[slot, self.hidden] + torch.arange(1, n + 1, device=x.device, dtype=torch.float32)
                out[first:first + n] = (self.gain * sums / count[:, None]).to(x.dtype)
                if write_cache:
                    state[slot, :self.hidden] = sums[-1]
                    state[slot, self.hidden] = count[-1]
            return out

    def attention(hidden, heads, kv_heads, head_dim, eps):
        return AttentionSpec("gqa_attention", hidden, heads, kv_heads, head_dim, 1 / math.sqrt(head_dim),
                             NormSpec("rmsnorm", head_dim, eps), PositionSpec("rope_split_half", head_dim, 10000.0))

    class ToyBase:
        def __init__(self, data):
            self.data = data
            self.hidden, self.vocab, self.inter = data["width"], data["vocab"], data["inner"]

        @classmethod
        def from_dict(cls, data):
            return cls(data)

        def to_dict(self):
            return dict(self.data)

        @staticmethod
        def global_tensor_name(local):
            return {"embed": "tok.weight", "final_norm.weight": "out_norm.weight", "lm_head": "out.weight"}[local]

        @staticmethod
        def layer_tensor_name(layer, part, local):
            return f"layer{layer}.{part}.{local}"

    @register_architecture("ToyStateForTests")
    class ToyState(ToyBase):
        """Layer 0: attention; layer 1: the running-mean mixer; layer 2: attention again."""

        def model_spec(self):
            norm = NormSpec("rmsnorm", self.hidden, 1e-5)
            ffn = MlpSpec("swiglu", self.hidden, self.inter)
            attn = LayerSpec("prenorm", norm, attention(self.hidden, 2, 1, 16, 1e-5), norm, ffn)
            mean = LayerSpec("prenorm", norm, RunningMeanSpec("toy_running_mean", self.hidden), norm, ffn)
            return ModelSpec("ToyStateForTests", self.vocab, self.hidden, (attn, mean, attn),
                             (LayerRun(0, 0), LayerRun(1, 1), LayerRun(2, 2)), norm, False, 512)

    @register_architecture("ToyOrderForTests")
    class ToyOrder(ToyBase):
        """Two layers run as 0, 1, 0, 1: layer 0's second run has a cache entry of its own, layer 1's
        second run reads the keys and values its first run wrote."""

        def model_spec(self):
            norm = NormSpec("rmsnorm", self.hidden, 1e-5)
            ffn = MlpSpec("swiglu", self.hidden, self.inter)
            layer = LayerSpec("prenorm", norm, attention(self.hidden, 2, 2, 16, 1e-5), norm, ffn)
            return ModelSpec("ToyOrderForTests", self.vocab, self.hidden, (layer, layer),
                             (LayerRun(0, 0), LayerRun(1, 1), LayerRun(0, 2), LayerRun(1, 1, write_cache=False)),
                             norm, False, 512)

    return ToyState, ToyOrder


_registered = []


def toys():
    if not _registered:
        _registered.extend(register_toys())
    return _registered


def write_folder(tmp_path, arch, seed):
    from mini_llm_runtime_amd.config import config_from_dict
    from mini_llm_runtime_amd.weights import write_random_model
    toys()
    cfg = config_from_dict({"architectures": [arch], "width": 40, "vocab": 97, "inner": 56})
    folder = str(tmp_path / arch)
    write_random_model(folder, cfg, seed, matrix_std=0.15, norm_std=0.2)
    return folder


def plain_weights(folder):
    from safetensors.torch import load_file
    return {k: v.double().numpy() for k, v in load_file(os.path.join(folder, "model.safetensors")).items()}


ATTN_CFG = dict(num_attention_heads=2, head_dim=16, rms_norm_eps=1e-5, rope_theta=10000.0)


def plain_layer_weights(w, i):
    return {"q_proj": w[f"layer{i}.mixer.q_proj"], "k_proj": w[f"layer{i}.mixer.k_proj"],
            "v_proj": w[f"layer{i}.mixer.v_proj"], "o_proj": w[f"layer{i}.mixer.o_proj"],
            "q_norm": w[f"layer{i}.mixer.q_norm.weight"], "k_norm": w[f"layer{i}.mixer.k_norm.weight"],
            "gate_proj": w[f"layer{i}.ffn.gate_proj"], "up_proj": w[f"layer{i}.ffn.up_proj"],
            "down_proj": w[f"layer{i}.ffn.down_proj"]}


def plain_toy_state(w, tokens):
    pos = np.arange(len(tokens))
    h = P.embed(tokens, w["tok.weight"])
    for i in range(3):
        x = P.rms_norm(h, w[f"layer{i}.norm1.weight"], 1e-5)
        if i == 1:
            mixed = w["layer1.mixer.gain"] * np.cumsum(x, axis=0) / (pos + 1)[:, None]
        else:
            mixed = P.attention_block(x, plain_layer_weights(w, i), dict(ATTN_CFG, num_key_value_heads=1), pos)
        h = h + mixed
        ffn = {k: w[f"layer{i}.ffn.{k}"] for k in ("gate_proj", "up_proj", "down_proj")}
        h = h + P.swiglu_mlp(P.rms_norm(h, w[f"layer{i}.norm2.weight"], 1e-5), ffn)
    return P.output_logits(h, w["out_norm.weight"], w["out.weight"], 1e-5)


def plain_toy_order(w, tokens):
    pos = np.arange(len(tokens))
    cfg = dict(ATTN_CFG, num_key_value_heads=2)
    h = P.embed(tokens, w["tok.weight"])
    kept = None
    for run, i in enumerate([0, 1, 0, 1]):
        lw = plain_layer_weights(w, i)
        x = P.rms_norm(h, w[f"layer{i}.norm1.weight"], 1e-5)
        q, k, v = P.project_qkv(x, lw, cfg, pos)
        if run == 1:
            kept = (k, v)
        if run == 3:
            k, v = kept                              # reads what run 1 wrote
        mixed = P.causal_attention(q, k, v, pos, 0.25).reshape(len(tokens), -1) @ lw["o_proj"].T
        h = h + mixed
        h = h + P.swiglu_mlp(P.rms_norm(h, w[f"layer{i}.norm2.weight"], 1e-5), lw)
    return P.output_logits(h, w["out_norm.weight"], w["out.weight"], 1e-5)


@pytest.mark.parametrize("arch,plain", [("ToyStateForTests", plain_toy_state), ("ToyOrderForTests", plain_toy_order)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_toy_architectures_step_like_their_plain_twins(tmp_path, arch, plain, dtype):
    from helpers import compare, make_requests, mixed, portions, run_steps, whole
    from mini_llm_runtime_amd.cache import KvSpec, StateSpec
    from mini_llm_runtime_amd.engine import Runner
    from mini_llm_runtime_amd.parts import DecoderModel
    folder = write_folder(tmp_path, arch, seed=4)
    assert json.load(open(os.path.join(folder, "config.json")))["architectures"] == [arch]
    model = DecoderModel.load(folder, dtype)
    if arch == "ToyStateForTests":
        assert [type(s) for s in model.cache_entry_specs] == [KvSpec, StateSpec, KvSpec]
    else:
        assert len(model.cache_entry_specs) == 3 and len(model.blocks) == 2
    w = plain_weights(folder)
    reqs = make_requests(97, [50, 23, 70, 9, 31], seed=8)
    want = {(rid, p): row for rid, toks in reqs.items() for p, row in enumerate(plain(w, toks))}
    name = "float32" if dtype == torch.float32 else "bfloat16"
    r = Runner(model, max_tokens=128, max_slots=4, page_size=8)
    compare(run_steps(r, whole(reqs)), want, name)
    compare(run_steps(r, portions(reqs)), want, name)          # slots and their state are used again
    steps, peak = mixed(reqs, seed=2)
    r = Runner(model, max_tokens=peak, max_slots=4, page_size=8)
    compare(run_steps(r, steps), want, name)
    r.cache.check()
