"""Decode throughput of the Qwen3-0.6B-sized model (random weights, synthetic token ids) on one MI355X.

    python bench.py [--gpus 1] [--steps 64] [--warmup 8] [--layers 28] [--batch 8] [--context 4096]

A "step" is one decode step of the whole batch: one token per request through the engine's step
function and the greedy sampler.  Requests are first filled by real prefill (portions of 2048 tokens)
so that the timed steps end at the context length.  One JSON line is printed with decoded tokens a
second, the same at batch 1 and 64, the prefill of 2048 tokens and the decode step's share of the
HBM roofline.
"""
import argparse
import json
import os
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
    ap.add_argument("--no-points", action="store_true", help="skip the batch 1 and 64 points and the prefill")
    ap.add_argument("--only", default="all", choices=["all", "decode", "prefill", "engine"],
                    help="profiling aid: run just the decode steps or just the prefill; engine: the scheduler "
                         "over a burst of requests (3 x batch requests of 512 prompt and 128 output tokens, "
                         "batch slots), printed as one line of its own")
    ap.add_argument("--library", type=int, default=1,
                    help="0: every matrix product on the hand-written kernels, none in the vendor library")
    ap.add_argument("--split-keys", type=int, default=256, help="the smallest range of keys of one attention workgroup")
    ap.add_argument("--tune", type=int, default=1,
                    help="0: the vendor library's first candidate for every shape, none timed")
    ap.add_argument("--prefill-graph", type=int, default=1,
                    help="1: the prefill step may be captured as a graph once its shape has come often enough")
    ap.add_argument("--prefill-reps", type=int, default=10, help="prefill steps; the fastest but the first counts")
    ap.add_argument("--fill", default="prefill", choices=["prefill", "random"],
                    help="how the requests' caches are filled before the timed steps: by real prefill "
                         "(default) or, as a profiling aid, with random keys and values")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py measures one GPU; --gpus {args.gpus} is not built (single-GPU engine)")
        return 2

    import torch
    from mini_llm_runtime_amd.api import parse_dtype
    from mini_llm_runtime_amd.config import config_from_dict
    from mini_llm_runtime_amd.engine import Entry, Runner
    from mini_llm_runtime_amd.parts import DecoderModel, expected_tensors
    from mini_llm_runtime_amd.sampling import Sampler

    dtype = parse_dtype(args.dtype)
    if not args.tune:
        from mini_llm_runtime_amd.kernels import build
        build.load("library_gemm").mlr_library_gemm_tuning(0)
    tag = "bf16" if dtype == torch.bfloat16 else "fp32"
    FULL_LAYERS, sizes = SIZES[args.size]
    if args.layers <= 0:
        args.layers = FULL_LAYERS
    cfg = config_from_dict(dict(sizes, architectures=["Qwen3ForCausalLM"], num_hidden_layers=args.layers))
    # Random weights N(0, 0.02) (norm weights 1 + N(0, 0.1)) drawn on the GPU: the same tensors that the
    # random-weights mode would write to a model folder, without the trip through a file of many gigabytes.
    torch.manual_seed(0)
    weights = {}
    for name, spec in expected_tensors(cfg).items():
        if spec.optional:
            continue
        if spec.keep_float32:
            weights[name] = 1.0 + 0.1 * torch.randn(spec.shape, device="cuda", dtype=torch.float32)
        else:
            weights[name] = (0.02 * torch.randn(spec.shape, device="cuda", dtype=torch.float32)).to(dtype)
    model = DecoderModel(cfg, weights, dtype, "cuda:0")
    del weights
    c = cfg
    layer_params = c.hidden_size * (c.num_attention_heads + 2 * c.num_key_value_heads) * c.head_dim \
        + c.num_attention_heads * c.head_dim * c.hidden_size + 3 * c.hidden_size * c.intermediate_size
    elem = 2 if dtype == torch.bfloat16 else 4
    weight_bytes = (args.layers * layer_params + c.vocab_size * c.hidden_size) * elem     # layers + output projection
    kv_bytes_per_token = args.layers * 2 * c.num_key_value_heads * c.head_dim * elem
    g = torch.Generator().manual_seed(0)

    def decode_run(batch, steps, warmup):
        """Fill `batch` requests so that warmup + steps decode steps end at the context length; time `steps`."""
        runner = Runner(model, max_tokens=batch * (-(-args.context // 64) * 64), max_slots=batch,
                        max_length=args.context, max_batch_tokens=max(PREFILL_TOKENS, batch), page_size=args.page_size,
                        target_workgroups=args.attn_workgroups, library_gemm=bool(args.library),
                        split_keys=args.split_keys)
        sampler = Sampler(runner.kernels, runner.device, max_rows=batch)
        fill = args.context - steps - warmup
        assert fill >= 1
        slots = [runner.open_request() for _ in range(batch)]
        if args.fill == "random":
            runner.cache.commit(slots, [fill] * batch)
            for slab in runner.cache._k + runner.cache._v:
                slab.normal_()
        else:
            for s in slots:
                ids = torch.randint(0, c.vocab_size, (fill,), generator=g).tolist()
                for at in range(0, fill, PREFILL_TOKENS):
                    runner.step([Entry(s, ids[at:at + PREFILL_TOKENS], [])])
        tokens = torch.randint(0, c.vocab_size, (batch,), generator=g).tolist()
        zeros = [0.0] * batch

        def one(tokens):
            logits = runner.step([Entry(s, [t], [0]) for s, t in zip(slots, tokens)])
            return sampler.sample(logits, zeros, zeros)
        for _ in range(warmup):
            tokens = one(tokens)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            tokens = one(tokens)
        torch.cuda.synchronize()
        seconds = time.perf_counter() - t0
        mean_context = args.context - steps / 2.0
        for s in slots:
            runner.close_request(s)
        del runner
        torch.cuda.empty_cache()
        return seconds, mean_context

    def prefill_run():
        runner = Runner(model, max_tokens=PREFILL_TOKENS, max_slots=1, max_length=PREFILL_TOKENS,
                        max_batch_tokens=PREFILL_TOKENS, page_size=args.page_size,
                        graph_max_tokens=PREFILL_TOKENS if args.prefill_graph else 512,
                        library_gemm=bool(args.library))
        ids = torch.randint(0, c.vocab_size, (PREFILL_TOKENS,), generator=g).tolist()
        times = []
        for i in range(args.prefill_reps):
            s = runner.open_request()
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            runner.step([Entry(s, ids, [PREFILL_TOKENS - 1])])
            torch.cuda.synchronize()
            times.append(time.perf_counter() - t0)
            runner.close_request(s)
        seconds = min(times[1:])
        t = PREFILL_TOKENS
        flops = 2.0 * t * args.layers * layer_params \
            + 2.0 * t * t * c.num_attention_heads * c.head_dim * args.layers \
            + 2.0 * c.vocab_size * c.hidden_size
        return dict(value=round(t / seconds, 1), tokens=t, ms=round(seconds * 1e3, 3),
                    frac=round(flops / seconds / MFMA_PEAK[tag], 5))

    if args.only == "prefill":
        print(json.dumps({"prefill": prefill_run()}))
        return 0
    if args.only == "engine":
        from mini_llm_runtime_amd.engine import Engine, EngineOptions
        slots, prompt, output = args.batch, 512, 128
        engine = Engine(model, EngineOptions(context_tokens=slots * 1024, max_model_len=1024, max_active=slots,
                                             batch_tokens=max(256, 16 * slots), prefill_chunk=max(128, 8 * slots),
                                             block_size=args.page_size))
        requests = 3 * slots

        def burst(n):
            for _ in range(n):
                engine.submit(torch.randint(0, c.vocab_size, (prompt,), generator=g).tolist(), max_tokens=output,
                              ignore_eos=True)
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            engine.run_until_done()
            torch.cuda.synchronize()
            return time.perf_counter() - t0
        first = burst(requests)                 # a server's first minute: step shapes are met and captured
        before = dict(engine.stats)
        seconds = burst(requests)               # the same burst again: what a server that has run a while does
        print(json.dumps({"engine": {"requests": requests, "slots": slots, "prompt_tokens": prompt,
                                     "output_tokens": output, "seconds": round(seconds, 3),
                                     "generated_tok_s": round(requests * output / seconds, 1),
                                     "total_tok_s": round(requests * (prompt + output) / seconds, 1),
                                     "first_burst_seconds": round(first, 3),
                                     "batches": engine.stats["batches"] - before["batches"],
                                     "mixed_batches": engine.stats["mixed_batches"] - before["mixed_batches"]}}))
        return 0
    seconds, mean_context = decode_run(args.batch, args.steps, args.warmup)
    ms_per_step = seconds / args.steps * 1e3
    value = args.batch * args.steps / seconds
    step_bytes = weight_bytes + args.batch * mean_context * kv_bytes_per_token
    achieved = step_bytes / (seconds / args.steps) / 1e9
    line = {
        "metric": f"decode tok/s, Qwen3-{args.size.upper()} sizes, batch {args.batch}, context {args.context}",
        "value": round(value, 1),
        "unit": "tok/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": tag, "data": "synthetic token ids, random weights N(0, 0.02)",
        "config": {"model": f"Qwen3-{args.size.upper()} sizes", "layers": args.layers, "layers_full": FULL_LAYERS,
                   "hidden_size": c.hidden_size, "q_heads": c.num_attention_heads,
                   "kv_heads": c.num_key_value_heads, "head_dim": c.head_dim,
                   "intermediate_size": c.intermediate_size, "vocab_size": c.vocab_size,
                   "tied_embeddings": c.tie_word_embeddings, "rope_theta": c.rope_theta, "rms_norm_eps": c.rms_norm_eps,
                   "global_batch": args.batch, "seq_len": args.context, "page_size": args.page_size,
                   "sampling": "greedy", "parallelism": "single GPU"},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK / 1e9, "unit": "GB/s",
                     "frac": round(achieved * 1e9 / HBM_PEAK, 5)},
    }
    if not args.no_points and args.only == "all":
        line["prefill"] = prefill_run()
        points = {}
        for batch in (1, 64):
            s, _ = decode_run(batch, max(8, args.steps // 2), max(2, args.warmup // 2))
            points[f"decode_b{batch}"] = round(batch * max(8, args.steps // 2) / s, 1)
        line["points"] = points
    print(json.dumps(line))
    return 0


if __name__ == "__main__":
    sys.exit(main())
