"""The Python entry point: load (or randomly initialise) a model and generate.

    llm = LLM("path/to/folder", dtype="bfloat16")
    tokens = llm.generate([1, 2, 3], max_tokens=16)                     # one prompt -> one list
    many = llm.generate([[1, 2, 3], [4, 5]], max_tokens=8, temperature=0.8, seed=7)

Generation goes through the scheduler (continuous batching over the step function); `runner`
gives direct access to the step function for tests and tools.
"""
from __future__ import annotations

import torch

from .engine import Engine, EngineOptions
from .parts import DecoderModel

DTYPES = {"bfloat16": torch.bfloat16, "bf16": torch.bfloat16, "float32": torch.float32, "fp32": torch.float32,
          "f32": torch.float32}


def parse_dtype(name):
    if isinstance(name, torch.dtype):
        if name in (torch.bfloat16, torch.float32):
            return name
    elif name in DTYPES:
        return DTYPES[name]
    raise ValueError(f"dtype must be bfloat16 or float32, got {name!r}")


class LLM:
    def __init__(self, model, dtype="bfloat16", device="cuda:0", options: EngineOptions = None, **overrides):
        """`model`: a folder with config.json and model.safetensors.  `overrides` set single
        fields of EngineOptions (context_tokens, max_model_len, max_active, batch_tokens,
        prefill_chunk, block_size, policy, ...)."""
        self.dtype = parse_dtype(dtype)
        self.model = DecoderModel.load(model, self.dtype, device)
        opts = options or EngineOptions()
        for key, value in overrides.items():
            if not hasattr(opts, key):
                raise ValueError(f"unknown engine option {key!r}")
            setattr(opts, key, value)
        opts.max_model_len = min(opts.max_model_len, self.model.spec.max_positions)
        self.engine = Engine(self.model, opts)

    @property
    def runner(self):
        return self.engine.runner

    def generate(self, prompts, max_tokens=32, temperature=0.0, seed=None, ignore_eos=False, timeout_ms=None):
        """`prompts`: one list of token ids or a list of such lists.  Returns the generated ids
        (without the prompt), in the same shape.  A request that runs out of `timeout_ms` returns what it
        has generated until then."""
        single = len(prompts) > 0 and not isinstance(prompts[0], (list, tuple))
        batch = [prompts] if single else list(prompts)
        ids = []
        for i, prompt in enumerate(batch):
            ids.append(self.engine.submit(prompt, max_tokens=max_tokens, temperature=temperature,
                                          seed=None if seed is None else seed + i, ignore_eos=ignore_eos,
                                          timeout_ms=timeout_ms))
        done = self.engine.run_until_done()
        out = [done[i] for i in ids]
        for i in ids:
            self.engine.finished.pop(i, None)      # handed over: a long-lived engine keeps no record of them
        return out[0] if single else out


def generate(model, prompts, max_tokens=32, temperature=0.0, seed=None, dtype="bfloat16", **engine_options):
    """One call: load the model folder, generate, return the token ids."""
    return LLM(model, dtype=dtype, **engine_options).generate(prompts, max_tokens, temperature, seed)
