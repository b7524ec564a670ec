"""`mini-llm`: generate from token ids on one MI355X.  Options keep the names and meanings of the
reference's CLIs (apps/mini_main.cpp:19-83, apps/cuda_main.cpp:18-54) where it has them.  Prompts are
token ids, or text when the model folder (or --tokenizer) holds a tokenizer.json.

Two ways to run:

  * `--prompt-ids 1,2,3` or `--prompt TEXT`: one sequence straight on the step function, as the reference's
    CLIs run theirs: the prompt in portions of --chunk tokens with logits asked for at its last token only,
    then one token per step; the last generated token is never fed back, so the cache must hold prompt +
    tokens - 1 positions.  With a tokenizer the report holds the generated `text` as well, and without any
    prompt option the reference's default prompt is taken ("The capital of France is").
  * `--prompts-file FILE` (one comma-separated prompt a line): every prompt becomes a request of the
    scheduler (`Engine`): admission, portions under the token budget, continuous batching over
    --sequences slots, --policy mixed or prefill_first.
"""
from __future__ import annotations

import json
import os
import sys
import tempfile
import time

from .options import Option, OptionError, parse

USAGE = """mini-llm (--model DIR | --random-weights CONFIG.json [--seed 0])
         (--prompt-ids 1,2,3 | --prompt TEXT | --prompts-file FILE) [--tokenizer tokenizer.json|DIR]
         [--tokens 32] [--context MODEL'S] [--batch 2048] [--chunk BATCH] [--sequences 4]
         [--dtype bfloat16|float32] [--kv-dtype auto] [--temperature 0] [--sample-seed 0] [--page-size 16]
         [--policy mixed|prefill_first] [--device 0] [--device-budget-bytes 0] [--ignore-eos]
         [--device-time] [--profile] [--check-finite] [--output NEW_REPORT.json]
         [--cuda-precision f32-pedantic] [--kv-layout paged]
mini-llm --model DIR --inspect
"""

TABLE = [
    Option("--help", "switch"), Option("--inspect", "switch"), Option("--ignore-eos", "switch"),
    Option("--device-time", "switch"), Option("--profile", "switch"), Option("--check-finite", "switch"),
    Option("--model"), Option("--random-weights"), Option("--output"), Option("--prompts-file"),
    Option("--prompt"), Option("--tokenizer"),
    Option("--dtype", default="bfloat16"), Option("--policy", default="mixed"), Option("--kv-dtype", default="auto"),
    Option("--cuda-precision"), Option("--kv-layout", default="paged"),
    Option("--prompt-ids", "ints", default=[]),
    Option("--seed", "int", 0, 0, 2 ** 63 - 1), Option("--sample-seed", "int", 0, 0, 2 ** 63 - 1),
    Option("--tokens", "int", 32, 1, 4096), Option("--context", "int", None, 1, 2 ** 31 - 1),
    Option("--batch", "int", 2048, 1, 2 ** 20), Option("--chunk", "int", None, 1, 2 ** 20),
    Option("--sequences", "int", 4, 1, 4096), Option("--page-size", "int", 16, 1, 1024),
    Option("--device", "int", 0, 0, 2 ** 31 - 1), Option("--device-budget-bytes", "int", 0, 0, 2 ** 63 - 1),
    Option("--temperature", "float", 0.0, 0.0, 1e6),
]


def inspect(opts):
    """What the model folder holds, without a GPU: architecture, configuration, files, tensors, and whether
    the tensors are the ones the architecture expects (apps/mini_main.cpp:54-69 prints the same of its file)."""
    from .config import load_config
    from .parts.model import expected_tensors
    from .weights.loader import WeightError, check_names, open_model_folder
    if not opts.given("--model"):
        raise OptionError("--inspect needs --model")
    folder = opts["--model"]
    config = load_config(folder)
    names, files = open_model_folder(folder)
    found = {name: f.entries[name] for name, f in names.items()}
    try:
        check_names(expected_tensors(config), found)
        problems = None
    except WeightError as error:
        problems = str(error)
    dimensions = config.to_dict()
    report = {"architecture": (dimensions.get("architectures") or [type(config).__name__])[0], "dimensions": dimensions,
              "files": [os.path.basename(f.path) for f in files],
              "bytes": sum(os.path.getsize(f.path) for f in files), "tensors": len(found),
              "tensor_types": sorted({str(dtype).replace("torch.", "") for dtype, _ in found.values()}),
              "complete": problems is None, "problems": problems}
    for f in files:
        f.close()
    print(json.dumps(report, indent=2))
    return 0


def read_prompts(path, vocab):
    prompts = []
    with open(path) as f:
        for number, line in enumerate(f, 1):
            line = line.strip()
            if not line or line.startswith("#"):
                continue
            try:
                ids = [int(piece) for piece in line.split(",")]
            except ValueError:
                raise OptionError(f"--prompts-file line {number}: not a comma-separated list of integers") from None
            if any(t < 0 or t >= vocab for t in ids):
                raise OptionError(f"--prompts-file line {number}: a token id lies outside the vocabulary")
            prompts.append(ids)
    if not prompts:
        raise OptionError("--prompts-file names no prompt")
    return prompts


DEFAULT_PROMPT = "The capital of France is"        # apps/cuda_main.cpp:53, apps/mini_main.cpp:85


def one_sequence(opts, model, runner, sampler, prompt, count, chunk, tokenizer=None):
    """The reference CLI's loop (apps/cuda_main.cpp:91-119): portions, then one token per step."""
    import torch
    from .engine import Entry
    from .sampling import RequestRng
    temperature = opts["--temperature"]
    rng = RequestRng(opts["--sample-seed"])
    timing = opts["--device-time"]
    forwards = []

    def run(entry, phase):
        t0 = time.perf_counter()
        if timing:
            start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            start.record()
        logits = runner.step([entry])
        token = None
        if logits is not None:
            token = sampler.sample(logits, [temperature], [rng.uniform() if temperature > 0 else 0.0])[0]
        else:
            torch.cuda.synchronize()
        if timing:
            end.record()
            end.synchronize()
        forwards.append({"phase": phase, "input_tokens": len(entry.tokens),
                         "logits_rows": 0 if logits is None else 1,
                         "host_forward_to_token_ns": int((time.perf_counter() - t0) * 1e9),
                         "device_elapsed_ms": start.elapsed_time(end) if timing else None})
        return token

    slot = runner.open_request()
    started = time.perf_counter()
    token = None
    for begin in range(0, len(prompt), chunk):
        part = prompt[begin:begin + chunk]
        last = begin + len(part) == len(prompt)
        token = run(Entry(slot, part, [len(part) - 1] if last else []), "prefill")
    prefill_s = time.perf_counter() - started
    generated = []
    eos = set(model.spec.eos_token_ids)
    for i in range(count):
        generated.append(token)
        stop = token in eos and not opts["--ignore-eos"]
        if stop or i + 1 == count:
            break
        token = run(Entry(slot, [token], [0]), "decode")
    elapsed = time.perf_counter() - started
    pages_before = runner.cache.num_pages - runner.cache.free_pages()
    runner.close_request(slot)
    text = {} if tokenizer is None else \
        {"text": tokenizer.text([t for t in generated if opts["--ignore-eos"] or t not in eos])}
    return {"input_token_ids": prompt, "token_ids": generated, **text, "prompt_tokens": len(prompt),
            "completion_tokens": len(generated), "ttft_ms": prefill_s * 1e3, "elapsed_s": elapsed,
            "output_tokens_per_second": len(generated) / elapsed if elapsed > 0 else None,
            "used_kv_pages_before_release": pages_before,
            "used_kv_pages_after_release": runner.cache.num_pages - runner.cache.free_pages(),
            "forwards": forwards}


def many_requests(opts, engine, prompts, count, tokenizer=None):
    """Every prompt a request of the scheduler; the report lists them in the order of the file."""
    started = time.perf_counter()
    ids = [engine.submit(p, max_tokens=count, temperature=opts["--temperature"], seed=opts["--sample-seed"] + i,
                         ignore_eos=opts["--ignore-eos"]) for i, p in enumerate(prompts)]
    first = {}
    while engine.has_work():
        for rid, token, _ in engine.step():
            if token is not None and rid not in first:
                first[rid] = time.perf_counter() - started
    elapsed = time.perf_counter() - started
    requests = [{"input_token_ids": p, "token_ids": list(engine.finished[rid].generated),
                 "finish_reason": engine.finished[rid].finish_reason, "ttft_ms": first.get(rid, 0.0) * 1e3}
                for rid, p in zip(ids, prompts)]
    if tokenizer is not None:
        for r in requests:
            r["text"] = tokenizer.text(r["token_ids"])
    generated = sum(len(r["token_ids"]) for r in requests)
    return {"requests": requests, "prompt_tokens": sum(len(p) for p in prompts), "completion_tokens": generated,
            "elapsed_s": elapsed, "output_tokens_per_second": generated / elapsed if elapsed > 0 else None,
            "policy": engine.options.policy, "scheduler": dict(engine.stats),
            "used_kv_pages_after_release": engine.runner.cache.num_pages - engine.runner.cache.free_pages()}


def main(argv=None):
    argv = sys.argv[1:] if argv is None else argv
    try:
        opts = parse(argv, TABLE)
        if opts["--help"] or not (opts.given("--model") or opts.given("--random-weights")):
            sys.stdout.write(USAGE)
            return 0 if opts["--help"] else 1
        if opts.given("--model") and opts.given("--random-weights"):
            raise OptionError("give --model or --random-weights, not both")
        if opts["--inspect"]:
            return inspect(opts)
        output = opts["--output"]
        if opts.given("--output") and (not output or os.path.exists(output)):
            raise OptionError("--output must be a new file")
        ways = [name for name in ("--prompt-ids", "--prompt", "--prompts-file") if opts.given(name)]
        if len(ways) > 1:
            raise OptionError(f"give --prompt-ids, --prompt or --prompts-file (one of them), not {' and '.join(ways)}")
        if not ways or ways == ["--prompt"] or opts.given("--tokenizer"):
            # text needs a vocabulary: looked for now, before the weights are read
            from .tokenizer import tokenizer_file
            where = opts["--tokenizer"] if opts.given("--tokenizer") else opts["--model"]
            if not where or tokenizer_file(where) is None:
                raise OptionError("no tokenizer.json in the model folder or under --tokenizer: give --prompt-ids "
                                  "or --prompts-file" if not opts.given("--tokenizer") else
                                  f"--tokenizer {where}: no tokenizer.json there")
        context, batch, sequences = opts["--context"], opts["--batch"], opts["--sequences"]
        chunk = opts["--chunk"] if opts.given("--chunk") else batch
        if chunk > batch:
            raise OptionError(f"--chunk {chunk}: not an integer in 1..{batch} (--batch)")
        count, page, budget = opts["--tokens"], opts["--page-size"], opts["--device-budget-bytes"]
        # the reference's names for what is a choice of one here (apps/cuda_main.cpp:18-47): its 32-bit mode
        # is --dtype float32; its FP16-matrix mode and its contiguous cache layout are not built
        if opts["--kv-layout"] != "paged":
            raise OptionError("--kv-layout: only the paged cache is built")
        if opts.given("--cuda-precision"):
            if opts["--cuda-precision"] != "f32-pedantic":
                raise OptionError("--cuda-precision: only f32-pedantic (= --dtype float32) is built; "
                                  "the reduced-precision engine is --dtype bfloat16")
            if opts.given("--dtype") and opts["--dtype"] not in ("float32", "fp32"):
                raise OptionError("--cuda-precision f32-pedantic contradicts --dtype")
        if opts["--policy"] not in ("mixed", "prefill_first"):
            raise OptionError("--policy: mixed or prefill_first")
        if opts["--kv-dtype"] not in ("auto", "bfloat16", "float32"):
            raise OptionError("--kv-dtype: auto, bfloat16 or float32 (the engine's own element type)")

        import torch
        from .api import parse_dtype
        from .config import config_from_dict
        from .engine import Engine, EngineOptions, MemoryBudgetError, Runner
        from .parts import DecoderModel
        from .sampling import Sampler
        from .weights import write_random_model
        dtype = parse_dtype("float32" if opts.given("--cuda-precision") else opts["--dtype"])
        scratch = None
        if opts.given("--random-weights"):
            with open(opts["--random-weights"]) as f:
                config = config_from_dict(json.load(f))
            scratch = tempfile.TemporaryDirectory(prefix="mini-llm-random-")
            folder = write_random_model(scratch.name, config, opts["--seed"])
        else:
            folder = opts["--model"]
        try:
            model = DecoderModel.load(folder, dtype, f"cuda:{opts['--device']}", device_budget_bytes=budget)
        except MemoryBudgetError as error:
            raise OptionError(str(error)) from None
        vocab = model.spec.vocab_size
        tokenizer = None
        if opts.given("--tokenizer") or not (opts.given("--prompt-ids") or opts.given("--prompts-file")):
            from .tokenizer import Tokenizer, TokenizerError
            try:
                tokenizer = Tokenizer(opts["--tokenizer"] if opts.given("--tokenizer") else folder, vocab,
                                      model.spec.eos_token_ids)
            except TokenizerError as error:
                raise OptionError(str(error)) from None
        # --context left out: requests as long as the model's positions allow, and a pool as large as the
        # device's budget leaves room for (at most that of --sequences such requests); given: the reference's
        # pool of --sequences x --context tokens (apps/cuda_main.cpp:60-69 sizes its cache so)
        limit = min(context, model.spec.max_positions) if context is not None else model.spec.max_positions
        pool = sequences * ((limit + page - 1) // page) * page if context is not None else None
        batch = min(batch, limit)
        chunk = min(chunk, batch)
        common = {"backend": "mini-llm-runtime_amd", "dtype": str(dtype).replace("torch.", "")}
        try:
            if opts.given("--prompts-file"):
                prompts = read_prompts(opts["--prompts-file"], vocab)
                for p in prompts:
                    if len(p) + count > limit:
                        raise OptionError("a prompt and its output tokens exceed the context")
                engine = Engine(model, EngineOptions(
                    context_tokens=pool, max_model_len=limit, max_active=sequences, batch_tokens=max(batch, sequences),
                    prefill_chunk=min(chunk, max(batch, sequences)), block_size=page, policy=opts["--policy"],
                    kv_dtype=opts["--kv-dtype"]),
                    device_budget_bytes=budget, check_finite=opts["--check-finite"], profile=opts["--profile"])
                runner = engine.runner
                report = many_requests(opts, engine, prompts, count, tokenizer)
            else:
                if opts.given("--prompt-ids"):
                    prompt = opts["--prompt-ids"]
                    if not prompt or any(t < 0 or t >= vocab for t in prompt):
                        raise OptionError("--prompt-ids must name at least one token id inside the vocabulary")
                else:
                    prompt = tokenizer.tokenize(opts["--prompt"] if opts.given("--prompt") else DEFAULT_PROMPT)
                    if not prompt:
                        raise OptionError("--prompt: the text gives no token")
                if len(prompt) > limit or count - 1 > limit - len(prompt):
                    raise OptionError("prompt and the output tokens written to the cache exceed the context")
                runner = Runner(model, max_tokens=pool, max_slots=sequences, max_length=limit, max_batch_tokens=batch,
                                page_size=page, device_budget_bytes=budget, check_finite=opts["--check-finite"],
                                profile=opts["--profile"], kv_dtype=opts["--kv-dtype"])
                sampler = Sampler(runner.kernels, runner.device, max_rows=1)
                report = one_sequence(opts, model, runner, sampler, prompt, count, chunk, tokenizer)
        except MemoryBudgetError as error:
            raise OptionError(str(error)) from None
        report = {**common, **report,
                  "limits": {"max_sequences": sequences, "max_model_len": limit, "batch_tokens": batch, "page_size": page},
                  "device_bytes": {"weights": model.weight_bytes(), "cache": runner.cache.kv_bytes(), "budget": budget,
                                   "plan": runner.memory_plan.as_dict()}}
        if opts["--profile"]:
            report["profile"] = runner.profile_report()
        text = json.dumps(report, indent=2)
        if output:
            with open(output, "x") as f:
                f.write(text + "\n")
        print(text)
        if scratch is not None:
            scratch.cleanup()
        return 0
    except Exception as error:   # one line, like the reference's CLIs
        sys.stderr.write(f"mini-llm: {error}\n")
        return 1


if __name__ == "__main__":
    sys.exit(main())
