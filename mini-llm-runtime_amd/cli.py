"""`mini-llm`: generate from token ids on one MI355X.  Options keep the names and meanings of the
reference's CLIs (apps/mini_main.cpp:19-83, apps/cuda_main.cpp:18-54) where it has them: the
prompt runs in portions of --chunk tokens with logits asked for at its last token only, then one
token per step; the last generated token is never fed back, so the cache must hold
prompt + tokens - 1 positions.  There is no tokenizer here: the prompt is given as ids.
"""
from __future__ import annotations

import json
import os
import sys
import tempfile
import time

USAGE = """mini-llm (--model DIR | --random-weights CONFIG.json [--seed 0]) --prompt-ids 1,2,3
         [--tokens 32] [--context 2048] [--batch 128] [--chunk 128] [--sequences 4]
         [--dtype bfloat16|float32] [--temperature 0] [--sample-seed 0] [--page-size 16]
         [--device 0] [--device-budget-bytes 0] [--ignore-eos] [--device-time] [--output NEW_REPORT.json]
         [--cuda-precision f32-pedantic] [--kv-layout paged]
mini-llm --model DIR --inspect
"""


def inspect(opts):
    """What the model folder holds, without a GPU: architecture, configuration, files, tensors, and whether
    the tensors are the ones the architecture expects (apps/mini_main.cpp:54-69 prints the same of its file)."""
    from .config import load_config
    from .options import OptionError
    from .parts.model import expected_tensors
    from .weights.loader import WeightError, check_names, open_model_folder
    if not opts.has("--model"):
        raise OptionError("--inspect needs --model")
    folder = opts.get("--model")
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


def main(argv=None):
    from .options import OptionError, Options
    argv = sys.argv[1:] if argv is None else argv
    try:
        opts = Options(argv, {"--model", "--random-weights", "--seed", "--prompt-ids", "--tokens", "--context",
                              "--batch", "--chunk", "--sequences", "--dtype", "--temperature", "--sample-seed",
                              "--page-size", "--device", "--output", "--device-budget-bytes", "--cuda-precision",
                              "--kv-layout"},
                       {"--help", "--ignore-eos", "--device-time", "--inspect"})
        if opts.has("--help") or not (opts.has("--model") or opts.has("--random-weights")):
            sys.stdout.write(USAGE)
            return 0 if opts.has("--help") else 1
        if opts.has("--model") and opts.has("--random-weights"):
            raise OptionError("give --model or --random-weights, not both")
        if opts.has("--inspect"):
            return inspect(opts)
        output = opts.get("--output")
        if opts.has("--output") and (not output or os.path.exists(output)):
            raise OptionError("--output must be a new file")
        context = opts.integer("--context", 2048, 1, 2 ** 31 - 1)
        batch = opts.integer("--batch", 128, 1, 2 ** 20)
        chunk = opts.integer("--chunk", batch, 1, batch)
        sequences = opts.integer("--sequences", 4, 1, 4096)
        count = opts.integer("--tokens", 32, 1, 4096)
        page = opts.integer("--page-size", 16, 1, 1024)
        device = opts.integer("--device", 0, 0, 2 ** 31 - 1)
        temperature = opts.number("--temperature", 0.0, 0.0, 1e6)
        sample_seed = opts.integer("--sample-seed", 0, 0, 2 ** 63 - 1)
        prompt = opts.integers("--prompt-ids")
        budget = opts.integer("--device-budget-bytes", 0, 0, 2 ** 63 - 1)
        # the reference's names for what is a choice of one here (apps/cuda_main.cpp:18-47): its 32-bit mode
        # is --dtype float32; its FP16-matrix mode and its contiguous cache layout are not built
        if opts.get("--kv-layout", "paged") != "paged":
            raise OptionError("--kv-layout: only the paged cache is built")
        if opts.has("--cuda-precision"):
            if opts.get("--cuda-precision") != "f32-pedantic":
                raise OptionError("--cuda-precision: only f32-pedantic (= --dtype float32) is built; "
                                  "the reduced-precision engine is --dtype bfloat16")
            if opts.has("--dtype") and opts.get("--dtype") not in ("float32", "fp32"):
                raise OptionError("--cuda-precision f32-pedantic contradicts --dtype")

        import torch
        from .api import parse_dtype
        from .config import config_from_dict
        from .engine import Entry, Runner
        from .parts import DecoderModel
        from .sampling import RequestRng, Sampler
        from .weights import write_random_model
        dtype = parse_dtype("float32" if opts.has("--cuda-precision") else opts.get("--dtype", "bfloat16"))
        scratch = None
        if opts.has("--random-weights"):
            with open(opts.get("--random-weights")) as f:
                config = config_from_dict(json.load(f))
            scratch = tempfile.TemporaryDirectory(prefix="mini-llm-random-")
            folder = write_random_model(scratch.name, config, opts.integer("--seed", 0, 0, 2 ** 63 - 1))
        else:
            folder = opts.get("--model")
        model = DecoderModel.load(folder, dtype, f"cuda:{device}")
        vocab = model.spec.vocab_size
        if not prompt or any(t < 0 or t >= vocab for t in prompt):
            raise OptionError("--prompt-ids must name at least one token id inside the vocabulary")
        limit = min(context, model.spec.max_positions)
        if len(prompt) > limit or count - 1 > limit - len(prompt):
            raise OptionError("prompt and the output tokens written to the cache exceed the context")
        pages = sequences * ((limit + page - 1) // page)
        # the budget gate, before the cache is allocated (src/minillm/cuda/storage.cpp:168-175)
        element = 4 if dtype == torch.float32 else 2
        cache_bytes = sum(2 * spec.kv_heads * spec.head_dim * element for spec in model.cache_entry_specs
                          if hasattr(spec, "kv_heads")) * (pages + 1) * page
        weight_bytes = model.weight_bytes()
        if budget and weight_bytes + cache_bytes > budget:
            raise OptionError(f"weights ({weight_bytes} bytes) and cache ({cache_bytes} bytes) exceed "
                              f"--device-budget-bytes {budget}")
        runner = Runner(model, max_tokens=pages * page, max_slots=sequences, max_length=limit,
                        max_batch_tokens=batch, page_size=page)
        sampler = Sampler(runner.kernels, runner.device, max_rows=1)
        rng = RequestRng(sample_seed)
        timing = opts.has("--device-time")
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
            stop = token in eos and not opts.has("--ignore-eos")
            if stop or i + 1 == count:
                break
            token = run(Entry(slot, [token], [0]), "decode")
        elapsed = time.perf_counter() - started
        pages_before = runner.cache.num_pages - runner.cache.free_pages()
        runner.close_request(slot)
        report = {
            "backend": "mini-llm-runtime_amd", "dtype": str(dtype).replace("torch.", ""),
            "input_token_ids": prompt, "token_ids": generated, "prompt_tokens": len(prompt),
            "completion_tokens": len(generated), "ttft_ms": prefill_s * 1e3, "elapsed_s": elapsed,
            "output_tokens_per_second": len(generated) / elapsed if elapsed > 0 else None,
            "limits": {"max_sequences": sequences, "max_model_len": limit, "batch_tokens": batch,
                       "page_size": page},
            "device_bytes": {"weights": weight_bytes, "cache": runner.cache.kv_bytes(), "budget": budget},
            "used_kv_pages_before_release": pages_before,
            "used_kv_pages_after_release": runner.cache.num_pages - runner.cache.free_pages(),
            "forwards": forwards,
        }
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
