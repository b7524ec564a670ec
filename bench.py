"""Decode and prefill throughput of Qwen3-sized models (random weights, synthetic token ids) on one MI355X.

    python bench.py [--gpus 1] [--steps 64] [--warmup 8] [--size 0.6b] [--layers 0] [--batch 8] [--context 4096]

A "step" is one decode step of the whole batch: one token per request through the engine's step function
and the greedy sampler.  Requests are first filled by real prefill (portions of 2048 tokens) so that the
timed steps end at the context length.  The model of the default size is a random-weights model folder that is
written and loaded like any other (the larger ones are drawn on the GPU: the same tensors without a file of
many gigabytes).  Every runner is built with the product's own defaults.  One JSON line is printed:

  * value / ms_per_step / roofline: decode at --batch (8) of the --size (0.6b) model, with the step's share of
    the HBM roofline (bytes it has to read: every weight once and the live requests' cache; 8 TB/s);
  * points: the same at batch 1 and 64, and at batch 8 behind contexts of 1024, 8192 and 32768 tokens;
    prefill: 2048 tokens in one step (the median of several; the fastest beside it), with its share of the
    MFMA peak, and `generate_ms`: the same prompt through the scheduler with its options left alone, from
    submission to the first generated token;
  * with the default size, a block "8b" and a block "32b": decode at batch 64, 8 and 1, the prefill and a mixed
    step (64 decoding requests beside a 2048-token prompt portion in ONE step) at those sizes, each with its
    share of its roofline; the 64 requests of a block are filled once and serve all of its measurements.
    `--size 32b --only mixed` measures the mixed step alone.
  * --profile: time per kernel class (event pairs around every launch, steps run eagerly) beside the line.
"""
import argparse
import json
import os
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK = 8.0e12              # bytes/s, MI355X
MFMA_PEAK = {"bf16": 2.5e15, "fp32": 157.3e12}
# layer sizes of the Qwen3 dense family; the default is the 0.6B one
SIZES = {
    "0.6b": (28, dict(hidden_size=1024, num_attention_heads=16, num_key_value_heads=8, head_dim=128,
                      intermediate_size=3072, vocab_size=151936, max_position_embeddings=40960,
                      rms_norm_eps=1e-6, rope_theta=1000000.0, tie_word_embeddings=True)),
    "8b": (36, dict(hidden_size=4096, num_attention_heads=32, num_key_value_heads=8, head_dim=128,
                    intermediate_size=12288, vocab_size=151936, max_position_embeddings=40960,
                    rms_norm_eps=1e-6, rope_theta=1000000.0, tie_word_embeddings=False)),
    "32b": (64, dict(hidden_size=5120, num_attention_heads=64, num_key_value_heads=8, head_dim=128,
                     intermediate_size=25600, vocab_size=151936, max_position_embeddings=40960,
                     rms_norm_eps=1e-6, rope_theta=1000000.0, tie_word_embeddings=False)),
}
PREFILL_TOKENS = 2048


class Bench:
    """One model of the given sizes on the GPU and the measurements on it."""

    def __init__(self, size, layers, args):
        import torch
        from mini_llm_runtime_amd.api import parse_dtype
        from mini_llm_runtime_amd.config import config_from_dict
        from mini_llm_runtime_amd.parts import DecoderModel, expected_tensors
        self.torch, self.args, self.size = torch, args, size
        self.dtype = parse_dtype(args.dtype)
        self.tag = "bf16" if self.dtype == torch.bfloat16 else "fp32"
        self.full_layers, sizes = SIZES[size]
        self.layers = layers if layers > 0 else self.full_layers
        self.cfg = c = config_from_dict(dict(sizes, architectures=["Qwen3ForCausalLM"], num_hidden_layers=self.layers))
        if args.weights == "folder" or (args.weights == "auto" and size == "0.6b"):
            # the product's way: a random-weights model folder (N(0, 0.02), norm weights 1 + N(0, 0.1)), written
            # and loaded like any model folder, through the planned arena and its budget gate
            import shutil
            import tempfile
            from mini_llm_runtime_amd.weights import write_random_model
            base = "/dev/shm" if os.path.isdir("/dev/shm") and shutil.disk_usage("/dev/shm").free > (8 << 30) else None
            with tempfile.TemporaryDirectory(prefix="mlr-bench-", dir=base) as folder:
                write_random_model(folder, c, seed=0)
                self.model = DecoderModel.load(folder, self.dtype, "cuda:0", device_budget_bytes=0)
            self.weights_from = "model folder"
        else:
            # the same tensors drawn on the GPU, without the trip through a file of many gigabytes
            torch.manual_seed(0)
            weights = {}
            for name, spec in expected_tensors(c).items():
                if spec.optional:
                    continue
                if spec.keep_float32:
                    weights[name] = 1.0 + 0.1 * torch.randn(spec.shape, device="cuda", dtype=torch.float32)
                else:
                    weights[name] = torch.randn(spec.shape, device="cuda", dtype=self.dtype).mul_(0.02)
            self.model = DecoderModel(c, weights, self.dtype, "cuda:0")
            del weights
            self.weights_from = "drawn on the GPU"
        self.layer_params = c.hidden_size * (c.num_attention_heads + 2 * c.num_key_value_heads) * c.head_dim \
            + c.num_attention_heads * c.head_dim * c.hidden_size + 3 * c.hidden_size * c.intermediate_size
        self.elem = 2 if self.dtype == torch.bfloat16 else 4
        self.weight_bytes = (self.layers * self.layer_params + c.vocab_size * c.hidden_size) * self.elem
        self.kv_bytes_per_token = self.layers * 2 * c.num_key_value_heads * c.head_dim * self.elem
        self.g = torch.Generator().manual_seed(0)

    def close(self):
        self.model = None
        self.torch.cuda.empty_cache()

    def runner(self, slots, max_tokens, max_length, max_batch_tokens, **kwargs):
        from mini_llm_runtime_amd.engine import Runner
        a = self.args
        return Runner(self.model, max_tokens=max_tokens, max_slots=slots, max_length=max_length,
                      max_batch_tokens=max_batch_tokens, page_size=a.page_size, target_workgroups=a.attn_workgroups,
                      library_gemm=bool(a.library), split_keys=a.split_keys, max_logits_rows=slots,
                      profile=bool(a.profile), **kwargs)

    def fill(self, runner, slots, tokens):
        """`tokens` tokens into every slot's cache: by real prefill (default) or, as a profiling aid, at random."""
        from mini_llm_runtime_amd.engine import Entry
        torch, c = self.torch, self.cfg
        if self.args.fill == "random":
            runner.cache.commit(slots, [tokens] * len(slots))
            for slab in runner.cache.paged_tensors():
                slab.normal_()
            return
        for s in slots:
            ids = torch.randint(0, c.vocab_size, (tokens,), generator=self.g).tolist()
            for at in range(0, tokens, PREFILL_TOKENS):
                runner.step([Entry(s, ids[at:at + PREFILL_TOKENS], [])])

    def decode(self, batch, steps, warmup, context=None):
        """Fill `batch` requests so that warmup + steps decode steps end at the context length; time `steps`.
        Returns (seconds, mean context, profile report or None)."""
        from mini_llm_runtime_amd.engine import Entry
        from mini_llm_runtime_amd.sampling import Sampler
        torch, a, c = self.torch, self.args, self.cfg
        context = context or a.context
        runner = self.runner(batch, batch * (-(-context // 64) * 64), context, max(PREFILL_TOKENS, batch))
        sampler = Sampler(runner.kernels, runner.device, max_rows=batch)
        fill = context - steps - warmup
        assert fill >= 1
        # (part of the set-up, like compiling: the decoding step of this batch and context is captured before the
        # requests exist, so that the timed steps are replays whatever --warmup is)
        runner.warm_up(batch_sizes=[batch], contexts=[context])
        slots = [runner.open_request() for _ in range(batch)]
        self.fill(runner, slots, fill)
        tokens = torch.randint(0, c.vocab_size, (batch,), generator=self.g).tolist()
        zeros = [0.0] * batch

        def one(tokens):
            logits = runner.step([Entry(s, [t], [0]) for s, t in zip(slots, tokens)])
            return sampler.sample(logits, zeros, zeros)
        for _ in range(warmup):
            tokens = one(tokens)
        runner.profile_report(reset=True)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            tokens = one(tokens)
        torch.cuda.synchronize()
        seconds = time.perf_counter() - t0
        report = runner.profile_report()
        for s in slots:
            runner.close_request(s)
        del runner, sampler
        torch.cuda.empty_cache()
        return seconds, context - steps / 2.0, report

    def decode_point(self, batch, steps, warmup, context=None):
        """{tok_s, ms, frac}: decoded tokens a second, milliseconds a step, share of the HBM roofline."""
        seconds, mean_context, report = self.decode(batch, steps, warmup, context)
        step_bytes = self.weight_bytes + batch * mean_context * self.kv_bytes_per_token
        out = dict(tok_s=round(batch * steps / seconds, 1), ms=round(seconds / steps * 1e3, 4),
                   frac=round(step_bytes / (seconds / steps) / HBM_PEAK, 5))
        return out, step_bytes, report

    def prefill(self):
        from mini_llm_runtime_amd.engine import Entry
        torch, a, c = self.torch, self.args, self.cfg
        # (the product's defaults: a step of this many tokens is not captured as a graph unless --prefill-graph 1)
        extra = dict(graph_max_tokens=PREFILL_TOKENS) if a.prefill_graph and not a.profile else {}
        runner = self.runner(1, PREFILL_TOKENS, PREFILL_TOKENS, PREFILL_TOKENS, **extra)
        ids = torch.randint(0, c.vocab_size, (PREFILL_TOKENS,), generator=self.g).tolist()
        times = []
        for i in range(a.prefill_reps):
            s = runner.open_request()
            if i == 1:
                runner.profile_report(reset=True)
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            runner.step([Entry(s, ids, [PREFILL_TOKENS - 1])])
            torch.cuda.synchronize()
            times.append(time.perf_counter() - t0)
            runner.close_request(s)
        seconds = statistics.median(times[1:])         # what a request meets; the fastest run beside it
        t = PREFILL_TOKENS
        flops = 2.0 * t * self.layers * self.layer_params \
            + 2.0 * t * t * c.num_attention_heads * c.head_dim * self.layers \
            + 2.0 * c.vocab_size * c.hidden_size
        out = dict(value=round(t / seconds, 1), tokens=t, ms=round(seconds * 1e3, 3),
                   ms_best=round(min(times[1:]) * 1e3, 3),
                   frac=round(flops / seconds / MFMA_PEAK[self.tag], 5))
        report = runner.profile_report()
        if report is not None:
            out["profile"] = report
        del runner
        torch.cuda.empty_cache()
        return out

    def generate_prompt(self, reps=6):
        """A 2048-token prompt through the scheduler with its options left alone but for the slots (`Engine`, as
        `LLM.generate` drives it): milliseconds from submission to the first generated token (the median), to be
        held against the one-step prefill."""
        from mini_llm_runtime_amd.engine import Engine, EngineOptions
        torch, c = self.torch, self.cfg
        engine = Engine(self.model, EngineOptions(max_active=4))
        times = []
        for _ in range(reps + 1):
            ids = torch.randint(0, c.vocab_size, (PREFILL_TOKENS,), generator=self.g).tolist()
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            engine.submit(ids, max_tokens=1, ignore_eos=True)
            engine.run_until_done()
            torch.cuda.synchronize()
            times.append(time.perf_counter() - t0)
        steps = engine.stats["batches"] / (reps + 1)
        del engine
        torch.cuda.empty_cache()
        return dict(ms=round(statistics.median(times[1:]) * 1e3, 3), steps=steps)

    def prompt(self, portion=PREFILL_TOKENS):
        """One prompt of --context tokens, run in portions of `portion` tokens (the last one wants its logits):
        tokens a second over the whole prompt and the time of every portion, whose attention reads all the keys
        before it.  The fastest of several runs counts; a short prompt is run often enough for its step to be
        captured and replayed, as on a server that has met the shape before."""
        from mini_llm_runtime_amd.engine import Entry
        torch, a, c = self.torch, self.args, self.cfg
        total = a.context
        reps = 10 if total <= 2 * portion else 2
        runner = self.runner(1, total, total, portion, **(dict(graph_max_tokens=portion) if a.prefill_graph else {}))
        ids = torch.randint(0, c.vocab_size, (total,), generator=self.g).tolist()
        best = None
        for _ in range(reps):
            s = runner.open_request()
            times = []
            for at in range(0, total, portion):
                part = ids[at:at + portion]
                torch.cuda.synchronize()
                t0 = time.perf_counter()
                runner.step([Entry(s, part, [len(part) - 1] if at + portion >= total else [])])
                torch.cuda.synchronize()
                times.append(time.perf_counter() - t0)
            runner.close_request(s)
            best = times if best is None or sum(times) < sum(best) else best
        seconds = sum(best)
        flops = 2.0 * total * self.layers * self.layer_params \
            + 2.0 * total * total * c.num_attention_heads * c.head_dim * self.layers \
            + 2.0 * c.vocab_size * c.hidden_size
        del runner
        torch.cuda.empty_cache()
        return dict(value=round(total / seconds, 1), tokens=total, portion=portion, ms=round(seconds * 1e3, 2),
                    frac=round(flops / seconds / MFMA_PEAK[self.tag], 5),
                    first_portion_ms=round(best[0] * 1e3, 2), last_portion_ms=round(best[-1] * 1e3, 2))

    def mixed(self, decoding=64, reps=6):
        """ONE step that holds `decoding` single tokens of requests at the context length beside a portion of
        2048 tokens of another request's prompt (the reference's mixed workload,
        benchmarks/runtime-inputs/qwen3-cuda-v0.json:96-97).  Milliseconds a step (median, and the fastest)
        against max(bytes / 8 TB/s, flops / MFMA peak)."""
        from mini_llm_runtime_amd.engine import Entry
        from mini_llm_runtime_amd.sampling import Sampler
        torch, a, c = self.torch, self.args, self.cfg
        ctx_tokens = -(-a.context // 64) * 64
        runner = self.runner(decoding + 1, decoding * ctx_tokens + PREFILL_TOKENS, a.context, PREFILL_TOKENS + decoding)
        sampler = Sampler(runner.kernels, runner.device, max_rows=decoding)
        slots = [runner.open_request() for _ in range(decoding)]
        start = a.context - reps - 1
        self.fill(runner, slots, start)
        ids = torch.randint(0, c.vocab_size, (PREFILL_TOKENS,), generator=self.g).tolist()
        tokens = torch.randint(0, c.vocab_size, (decoding,), generator=self.g).tolist()
        zeros = [0.0] * decoding
        times = []
        for i in range(reps + 1):
            prompt = runner.open_request()
            if i == 1:
                runner.profile_report(reset=True)
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            logits = runner.step([Entry(s, [t], [0]) for s, t in zip(slots, tokens)] + [Entry(prompt, ids, [])])
            tokens = sampler.sample(logits, zeros, zeros)
            torch.cuda.synchronize()
            times.append(time.perf_counter() - t0)
            runner.close_request(prompt)
        times = times[1:]
        t, hq, d = PREFILL_TOKENS, c.num_attention_heads, c.head_dim
        context = start + (reps + 1) / 2.0
        step_bytes = self.weight_bytes + (decoding * context + t) * self.kv_bytes_per_token
        flops = 2.0 * (t + decoding) * self.layers * self.layer_params \
            + (2.0 * t * t + 4.0 * decoding * context) * hq * d * self.layers + 2.0 * decoding * c.vocab_size * c.hidden_size
        floor = max(step_bytes / HBM_PEAK, flops / MFMA_PEAK[self.tag])
        seconds = statistics.median(times)
        out = dict(ms=round(seconds * 1e3, 3), ms_best=round(min(times) * 1e3, 3), decode_rows=decoding, prefill_tokens=t,
                   context=a.context, floor_ms=round(floor * 1e3, 3),
                   bound="mfma" if flops / MFMA_PEAK[self.tag] > step_bytes / HBM_PEAK else "hbm",
                   frac=round(floor / seconds, 5), tok_s=round((t + decoding) / seconds, 1))
        report = runner.profile_report()
        if report is not None:
            out["profile"] = report
        for s in slots:
            runner.close_request(s)
        del runner, sampler
        torch.cuda.empty_cache()
        return out

    def block(self, steps, warmup, reps=6):
        """Decode at batch 64, 8 and 1 and the mixed step on ONE runner whose 64 requests are filled once, by real
        prefill, and serve every measurement (a large model's prompts are its longest set-up).  Each decode
        point: tokens a second, milliseconds a step and the share of the HBM roofline at the contexts its
        requests had meanwhile."""
        from mini_llm_runtime_amd.engine import Entry
        from mini_llm_runtime_amd.sampling import Sampler
        torch, a, c = self.torch, self.args, self.cfg
        decoding = 64
        ctx_tokens = -(-a.context // 64) * 64
        runner = self.runner(decoding + 1, decoding * ctx_tokens + PREFILL_TOKENS, a.context, PREFILL_TOKENS + decoding)
        sampler = Sampler(runner.kernels, runner.device, max_rows=decoding)
        runner.warm_up(batch_sizes=[1, 8, decoding], contexts=[a.context])
        slots = [runner.open_request() for _ in range(decoding)]
        fill = a.context - 3 * (steps + warmup) - (reps + 1)     # the first request decodes in every measurement
        assert fill >= 1
        self.fill(runner, slots, fill)
        out = {"layers": self.layers}
        for batch in (decoding, 8, 1):
            live = slots[:batch]
            tokens = torch.randint(0, c.vocab_size, (batch,), generator=self.g).tolist()
            zeros = [0.0] * batch

            def one(tokens):
                logits = runner.step([Entry(s, [t], [0]) for s, t in zip(live, tokens)])
                return sampler.sample(logits, zeros, zeros)
            for _ in range(warmup):
                tokens = one(tokens)
            before = sum(runner.length(s) for s in live) / batch
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(steps):
                tokens = one(tokens)
            torch.cuda.synchronize()
            seconds = time.perf_counter() - t0
            step_bytes = self.weight_bytes + batch * (before + steps / 2.0) * self.kv_bytes_per_token
            out[f"decode_b{batch}"] = round(batch * steps / seconds, 1)
            out[f"ms_b{batch}"] = round(seconds / steps * 1e3, 4)
            out[f"frac_b{batch}"] = round(step_bytes / (seconds / steps) / HBM_PEAK, 5)
        # the mixed step: every request brings one token, beside them a portion of 2048 tokens of a new prompt
        ids = torch.randint(0, c.vocab_size, (PREFILL_TOKENS,), generator=self.g).tolist()
        tokens = torch.randint(0, c.vocab_size, (decoding,), generator=self.g).tolist()
        zeros = [0.0] * decoding
        times = []
        context = sum(runner.length(s) for s in slots) / decoding
        for i in range(reps + 1):
            prompt = runner.open_request()
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            logits = runner.step([Entry(s, [t], [0]) for s, t in zip(slots, tokens)] + [Entry(prompt, ids, [])])
            tokens = sampler.sample(logits, zeros, zeros)
            torch.cuda.synchronize()
            times.append(time.perf_counter() - t0)
            runner.close_request(prompt)
        times = times[1:]
        t, hq, d = PREFILL_TOKENS, c.num_attention_heads, c.head_dim
        context += (reps + 1) / 2.0
        step_bytes = self.weight_bytes + (decoding * context + t) * self.kv_bytes_per_token
        flops = 2.0 * (t + decoding) * self.layers * self.layer_params \
            + (2.0 * t * t + 4.0 * decoding * context) * hq * d * self.layers + 2.0 * decoding * c.vocab_size * c.hidden_size
        floor = max(step_bytes / HBM_PEAK, flops / MFMA_PEAK[self.tag])
        seconds = statistics.median(times)
        out.update(mixed_ms=round(seconds * 1e3, 3), mixed_floor_ms=round(floor * 1e3, 3), mixed_frac=round(floor / seconds, 5),
                   mixed_bound="mfma" if flops / MFMA_PEAK[self.tag] > step_bytes / HBM_PEAK else "hbm",
                   mixed_tok_s=round((t + decoding) / seconds, 1))
        for s in slots:
            runner.close_request(s)
        del runner, sampler
        torch.cuda.empty_cache()
        return out

    def engine_burst(self):
        from mini_llm_runtime_amd.engine import Engine, EngineOptions
        torch, a, c = self.torch, self.args, self.cfg
        slots, prompt, output = a.batch, 512, 128
        engine = Engine(self.model, EngineOptions(context_tokens=slots * 1024, max_model_len=1024, max_active=slots,
                                                  batch_tokens=max(256, 16 * slots), prefill_chunk=max(128, 8 * slots),
                                                  block_size=a.page_size))
        requests = 3 * slots

        def burst(n):
            for _ in range(n):
                engine.submit(torch.randint(0, c.vocab_size, (prompt,), generator=self.g).tolist(), max_tokens=output,
                              ignore_eos=True)
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            engine.run_until_done()
            torch.cuda.synchronize()
            return time.perf_counter() - t0
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        warmed = engine.warm_up() if a.warm_up else 0      # the decoding steps captured before the first request
        torch.cuda.synchronize()
        warm = time.perf_counter() - t0
        first = burst(requests)                 # a server's first minute: step shapes are met and captured
        before = dict(engine.stats)
        seconds = burst(requests)               # the same burst again: what a server that has run a while does
        return {"requests": requests, "slots": slots, "prompt_tokens": prompt, "output_tokens": output,
                "seconds": round(seconds, 3), "generated_tok_s": round(requests * output / seconds, 1),
                "total_tok_s": round(requests * (prompt + output) / seconds, 1), "first_burst_seconds": round(first, 3),
                "warm_up_seconds": round(warm, 3), "warm_up_graphs": warmed,
                "batches": engine.stats["batches"] - before["batches"],
                "mixed_batches": engine.stats["mixed_batches"] - before["mixed_batches"]}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=64)
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--size", default="0.6b", choices=sorted(SIZES), help="layer sizes of which Qwen3 dense model")
    ap.add_argument("--layers", type=int, default=0, help="fewer layers than the model has (0: all of them)")
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--context", type=int, default=4096)
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--page-size", type=int, default=16, help="tokens in a page of the cache")
    ap.add_argument("--attn-workgroups", type=int, default=512,
                    help="tuning aid: workgroups that the split of a token's keys aims for")
    ap.add_argument("--no-points", action="store_true", help="skip the batch 1 and 64 points, the prefill and the 8B block")
    ap.add_argument("--no-8b", action="store_true", help="skip the block of 8B measurements in the default run")
    ap.add_argument("--no-32b", action="store_true", help="skip the block of 32B measurements in the default run")
    ap.add_argument("--weights", default="auto", choices=["auto", "folder", "gpu"],
                    help="folder: a random-weights model folder, written and loaded like any other; gpu: the same "
                         "tensors drawn on the GPU; auto: folder for the 0.6B sizes, gpu for the larger ones")
    ap.add_argument("--warm-up", type=int, default=0,
                    help="--only engine: 1 captures the decoding steps (Engine.warm_up) before the first burst")
    ap.add_argument("--only", default="all", choices=["all", "decode", "prefill", "prompt", "engine", "mixed"],
                    help="profiling aid: run just the decode steps, just the prefill or just the mixed step; prompt: one "
                         "prompt of --context tokens in portions of 2048; engine: the "
                         "scheduler over a burst of requests (3 x batch requests of 512 prompt and 128 output tokens, "
                         "batch slots), printed as one line of its own")
    ap.add_argument("--library", type=int, default=1,
                    help="0: every matrix product on the hand-written kernels, none in the vendor library")
    ap.add_argument("--split-keys", type=int, default=256, help="the smallest range of keys of one attention workgroup")
    ap.add_argument("--tune", type=int, default=1,
                    help="0: the vendor library's first candidate for every shape, none timed (the engine's default is 1)")
    ap.add_argument("--prefill-graph", type=int, default=0,
                    help="1: the prefill step may be captured as a graph once its shape has come often enough (the "
                         "product's default keeps steps of more than 512 tokens eager)")
    ap.add_argument("--prefill-reps", type=int, default=10, help="prefill steps; the median of all but the first counts")
    ap.add_argument("--fill", default="prefill", choices=["prefill", "random"],
                    help="how the requests' caches are filled before the timed steps: by real prefill "
                         "(default) or, as a profiling aid, with random keys and values")
    ap.add_argument("--profile", action="store_true",
                    help="time per kernel class (event pairs around every launch; steps then run eagerly, so the "
                         "step times themselves are those of the eager engine)")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py measures one GPU; --gpus {args.gpus} is not built (single-GPU engine)")
        return 2

    if not args.tune:
        from mini_llm_runtime_amd.kernels import build
        build.load("library_gemm").mlr_library_gemm_tuning(0)
    bench = Bench(args.size, args.layers, args)
    c = bench.cfg
    if args.only == "prefill":
        print(json.dumps({"prefill": bench.prefill()}))
        return 0
    if args.only == "prompt":
        print(json.dumps({"prompt": dict(bench.prompt(), model=f"Qwen3-{args.size.upper()} sizes", layers=bench.layers)}))
        return 0
    if args.only == "engine":
        print(json.dumps({"engine": bench.engine_burst()}))
        return 0
    if args.only == "mixed":
        print(json.dumps({"mixed": dict(bench.mixed(), model=f"Qwen3-{args.size.upper()} sizes", layers=bench.layers,
                                        layers_full=bench.full_layers, fill=args.fill)}))
        return 0
    point, step_bytes, report = bench.decode_point(args.batch, args.steps, args.warmup)
    achieved = step_bytes / (point["ms"] / 1e3) / 1e9
    line = {
        "metric": f"decode tok/s, Qwen3-{args.size.upper()} sizes, batch {args.batch}, context {args.context}",
        "value": point["tok_s"],
        "unit": "tok/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": point["ms"], "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": bench.tag, "data": "synthetic token ids, random weights N(0, 0.02)",
        "config": {"model": f"Qwen3-{args.size.upper()} sizes", "layers": bench.layers, "layers_full": bench.full_layers,
                   "hidden_size": c.hidden_size, "q_heads": c.num_attention_heads,
                   "kv_heads": c.num_key_value_heads, "head_dim": c.head_dim,
                   "intermediate_size": c.intermediate_size, "vocab_size": c.vocab_size,
                   "tied_embeddings": c.tie_word_embeddings, "rope_theta": c.rope_theta, "rms_norm_eps": c.rms_norm_eps,
                   "global_batch": args.batch, "seq_len": args.context, "page_size": args.page_size,
                   "sampling": "greedy", "parallelism": "single GPU"},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK / 1e9, "unit": "GB/s",
                     "frac": round(achieved * 1e9 / HBM_PEAK, 5)},
        "library_tuning": bool(args.tune), "weights": bench.weights_from,
    }
    if report is not None:
        line["profile"] = report
    if not args.no_points and args.only == "all":
        line["prefill"] = bench.prefill()
        through = bench.generate_prompt()
        line["prefill"].update(generate_ms=through["ms"], generate_steps=through["steps"])
        points = {}
        few = (max(8, args.steps // 2), max(2, args.warmup // 2))
        for batch in (1, 64):
            p, _, _ = bench.decode_point(batch, *few)
            points[f"decode_b{batch}"] = p["tok_s"]
            points[f"frac_b{batch}"] = p["frac"]
        for context in (1024, 8192, 32768):              # the same batch behind shorter and longer contexts
            if context <= c.max_position_embeddings:
                p, _, _ = bench.decode_point(args.batch, *few, context=context)
                points[f"decode_b{args.batch}_ctx{context}"] = p["tok_s"]
                points[f"frac_b{args.batch}_ctx{context}"] = p["frac"]
        line["points"] = points
        if args.size == "0.6b" and args.layers <= 0:
            # the other sizes the metric names: the same measurements at the Qwen3-8B and the Qwen3-32B sizes
            # (all 36 and all 64 layers)
            bench.close()
            for size, skip in (("8b", args.no_8b), ("32b", args.no_32b)):
                if skip:
                    continue
                big = Bench(size, 0, args)
                block = big.block(*few)
                pre = big.prefill()
                block.update(prefill_tok_s=pre["value"], prefill_ms=pre["ms"], prefill_frac=pre["frac"])
                line[size] = block
                big.close()
                del big
    print(json.dumps(line))
    return 0


if __name__ == "__main__":
    sys.exit(main())
