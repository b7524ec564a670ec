"""The Python entry point: load (or randomly initialise) a model and generate.

    llm = LLM("path/to/folder", dtype="bfloat16")
    tokens = llm.generate([1, 2, 3], max_tokens=16)                     # one prompt -> one list
    many = llm.generate([[1, 2, 3], [4, 5]], max_tokens=8, temperature=0.8, seed=7)
    text = llm.generate("The capital of France is", max_tokens=16)      # needs tokenizer.json in the folder

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
        prefill_chunk, block_size, policy, kv_dtype, device_budget_bytes, ...).  Left alone, the options
        come from the model and the device: requests as long as the model's positions allow, a page pool
        as large as the device's budget leaves room for, prompts in portions of 2048 tokens."""
        from dataclasses import replace
        self.dtype = parse_dtype(dtype)
        self.folder = model
        self._tokenizer = None
        opts = replace(options) if options is not None else EngineOptions()
        for key, value in overrides.items():
            if not hasattr(opts, key):
                raise ValueError(f"unknown engine option {key!r}")
            setattr(opts, key, value)
        # the same budget gates the weights and, in the engine, the cache and the scratch buffers
        self.model = DecoderModel.load(model, self.dtype, device, device_budget_bytes=opts.device_budget_bytes)
        self.engine = Engine(self.model, opts)

    @property
    def runner(self):
        return self.engine.runner

    @property
    def tokenizer(self):
        """The vocabulary of the model folder's tokenizer.json (read when text is first asked for)."""
        if self._tokenizer is None:
            from .tokenizer import Tokenizer
            self._tokenizer = Tokenizer(self.folder, self.model.spec.vocab_size, self.model.spec.eos_token_ids)
        return self._tokenizer

    def generate(self, prompts, max_tokens=32, temperature=0.0, seed=None, ignore_eos=False, timeout_ms=None):
        """`prompts`: one list of token ids or a list of such lists; or one text or a list of texts (the
        model folder must hold a tokenizer.json then).  Returns the generated ids (without the prompt), in
        the same shape; for text, the generated text (the token that ended it left out).  A request that
        runs out of `timeout_ms` returns what it has generated until then."""
        as_text = isinstance(prompts, str) or (len(prompts) > 0 and all(isinstance(p, str) for p in prompts))
        if as_text:
            one = isinstance(prompts, str)
            ids = self.generate([self.tokenizer.tokenize(p) for p in ([prompts] if one else prompts)], max_tokens,
                                temperature, seed, ignore_eos, timeout_ms)
            eos = set() if ignore_eos else set(self.model.spec.eos_token_ids)
            texts = [self.tokenizer.text([t for t in row if t not in eos]) for row in ids]
            return texts[0] if one else texts
        single = len(prompts) > 0 and not isinstance(prompts[0], (list, tuple))
        ids = self._submit_all([prompts] if single else list(prompts), max_tokens, temperature, seed, ignore_eos,
                               timeout_ms)
        done = self.engine.run_until_done()
        out = [done[i] for i in ids]
        for i in ids:
            self.engine.finished.pop(i, None)      # handed over: a long-lived engine keeps no record of them
        return out[0] if single else out

    def stream(self, prompts, max_tokens=32, temperature=0.0, seed=None, ignore_eos=False, timeout_ms=None):
        """As `generate` for token ids, but a generator: yields (index of the prompt, token id or None, finish
        reason or None) as soon as a step of the scheduler has produced it; a request's last event carries its
        reason ("stop", "length", "timeout", "cancelled").  A caller that stops reading early (closes the
        generator) cancels what still runs: nothing of it is left in the engine."""
        single = len(prompts) > 0 and not isinstance(prompts[0], (list, tuple))
        ids = self._submit_all([prompts] if single else list(prompts), max_tokens, temperature, seed, ignore_eos,
                               timeout_ms)
        index = {rid: i for i, rid in enumerate(ids)}
        live = set(ids)
        try:
            while live:
                for rid, token, reason in self.engine.step():
                    if rid in index:
                        if reason is not None:
                            live.discard(rid)
                        yield index[rid], token, reason
        finally:
            self._withdraw(live)
            for rid in ids:
                self.engine.finished.pop(rid, None)

    def _submit_all(self, batch, max_tokens, temperature, seed, ignore_eos, timeout_ms):
        """Queues every prompt or none: when one is refused, those queued before it are taken back."""
        ids = []
        try:
            for i, prompt in enumerate(batch):
                ids.append(self.engine.submit(prompt, max_tokens=max_tokens, temperature=temperature,
                                              seed=None if seed is None else seed + i, ignore_eos=ignore_eos,
                                              timeout_ms=timeout_ms))
        except Exception:
            self._withdraw(ids)
            for rid in ids:
                self.engine.finished.pop(rid, None)
            raise
        return ids

    def _withdraw(self, ids):
        if ids and not self.engine.failed:
            for rid in ids:
                self.engine.cancel(rid)
            self.engine.expire()


def generate(model, prompts, max_tokens=32, temperature=0.0, seed=None, dtype="bfloat16", **engine_options):
    """One call: load the model folder, generate, return the token ids."""
    return LLM(model, dtype=dtype, **engine_options).generate(prompts, max_tokens, temperature, seed)
