"""Generation through the entry points: the Python API over the scheduler, and the command line.
Greedy generation must give the plain implementation's tokens; temperature sampling must give, for a
request, the same tokens whatever else runs beside it."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest

from conftest import PAGE_SIZE, ROOT, TINY
from helpers import make_requests

pytestmark = pytest.mark.gpu


def prompts_for(name, lengths=(7, 13, 5, 1, 30)):
    return list(make_requests(TINY[name]["vocab_size"], lengths, seed=31).values())


def check_greedy(plain, prompt, got, dtype):
    """Token by token; in bfloat16 a step may differ only where the plain top two are nearly tied, and the
    comparison stops there (the continuations differ legitimately)."""
    tokens = list(prompt)
    for i, t in enumerate(got):
        row = plain.logits(tokens, [len(tokens) - 1])[0]
        best = int(np.argmax(row))
        if t != best:
            top = np.sort(row)[-2:]
            assert dtype == "bfloat16" and top[1] - top[0] < 0.05 * np.abs(row).max(), (i, t, best)
            return
        tokens.append(t)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B"])
def test_greedy_generation_through_the_python_entry_point(model_folders, plain_models, name, dtype):
    from mini_llm_runtime_amd.api import LLM
    llm = LLM(model_folders[name], dtype=dtype, context_tokens=256, max_model_len=128, max_active=4,
              batch_tokens=16, prefill_chunk=8, block_size=PAGE_SIZE[name])
    prompts = prompts_for(name)
    outs = llm.generate(prompts, max_tokens=8)
    assert [len(o) for o in outs] == [8] * len(prompts)
    for prompt, out in zip(prompts, outs):
        check_greedy(plain_models[name], prompt, out, dtype)
    assert llm.engine.stats["mixed_batches"] > 0                   # prompts ran in portions beside decoding requests
    assert llm.engine.runner.cache.free_pages() == llm.engine.total_pages
    one = llm.generate(prompts[0], max_tokens=8)                    # one prompt in, one list out
    if dtype == "float32":
        assert one == outs[0] == plain_models[name].greedy(prompts[0], 8)


def test_options_left_alone_through_the_python_entry_point(model_folders, plain_models):
    """`LLM(folder)` and nothing else: requests as long as the model's positions, 64 slots, a step that holds a
    2048-token portion beside a token of every slot, and a page pool sized by the runner (here: what the slots
    can hold at all, far below the device's budget).  Every prompt, a 300-token one among them, runs whole in the
    first step; then the requests decode together."""
    from mini_llm_runtime_amd.api import LLM
    llm = LLM(model_folders["A"])
    o = llm.engine.options
    assert (o.max_model_len, o.max_active, o.prefill_chunk, o.batch_tokens) == (1024, 64, 2048, 2112)
    assert o.context_tokens == 64 * 1024 == llm.runner.max_tokens and o.device_budget_bytes == 0
    prompts = prompts_for("A") + [make_requests(TINY["A"]["vocab_size"], [300], seed=77)["r0"]]
    outs = llm.generate(prompts, max_tokens=6, ignore_eos=True)
    for prompt, out in zip(prompts, outs):
        assert len(out) == 6
        check_greedy(plain_models["A"], prompt, out, "bfloat16")
    assert llm.engine.stats["batches"] == 6 and llm.engine.stats["mixed_batches"] == 0
    assert llm.runner.cache.free_pages() == llm.runner.cache.num_pages
    assert llm.runner.memory_report()["actual"]["workspace_beyond_plan"] == 0


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_prefill_first_through_the_engine(model_folders, plain_models, dtype):
    """Policy prefill_first on the GPU, requests arriving while others decode: decoding requests are left out
    of the steps that run prompts and resume from an untouched cache; every request gets the plain greedy
    tokens; pages and slots come back."""
    import torch
    from mini_llm_runtime_amd.engine import Engine, EngineOptions
    from mini_llm_runtime_amd.parts import DecoderModel
    name = "B"
    model = DecoderModel.load(model_folders[name], torch.float32 if dtype == "float32" else torch.bfloat16)
    eng = Engine(model, EngineOptions(context_tokens=512, max_model_len=128, max_active=4, batch_tokens=16,
                                      prefill_chunk=8, block_size=PAGE_SIZE[name], policy="prefill_first"))
    prompts = prompts_for(name, (9, 30, 17, 5, 22))
    ids = [eng.submit(prompts[0], max_tokens=10)]
    for _ in range(4):
        eng.step()                                           # the first request decodes already
    ids += [eng.submit(p, max_tokens=7) for p in prompts[1:3]]
    for _ in range(3):
        eng.step()
    ids += [eng.submit(p, max_tokens=7) for p in prompts[3:]]
    done = eng.run_until_done()
    for rid, prompt in zip(ids, prompts):
        check_greedy(plain_models[name], prompt, done[rid], dtype)
    assert eng.stats["mixed_batches"] == 0 and eng.stats["batches"] > 10
    assert eng.runner.cache.free_pages() == eng.total_pages and eng.runner.free_slots() == 4
    eng.runner.cache.check()


def test_many_requests_on_a_pool_that_holds_three(model_folders, plain_models):
    """Thirty requests of every length on a cache of 192 tokens: most of them wait for pages, pages and slots
    are used again and again, portions of prompts run beside decoding requests; every request still gets
    the plain implementation's greedy tokens, and everything is given back at the end."""
    from mini_llm_runtime_amd.api import LLM
    rng = np.random.default_rng(41)
    llm = LLM(model_folders["A"], dtype="float32", context_tokens=192, max_model_len=64, max_active=8,
              batch_tokens=24, prefill_chunk=16, block_size=PAGE_SIZE["A"])
    lengths = [int(x) for x in rng.integers(1, 50, 30)]
    prompts = prompts_for("A", lengths)
    outs = llm.generate(prompts, max_tokens=9)
    for prompt, out in zip(prompts, outs):
        assert out == plain_models["A"].greedy(prompt, 9)
    stats = llm.engine.stats
    assert stats["mixed_batches"] > 0
    assert llm.engine.runner.cache.free_pages() == llm.engine.total_pages
    llm.engine.runner.cache.check()


def test_a_cancelled_request_leaves_the_others_alone(model_folders, plain_models):
    from mini_llm_runtime_amd.engine import Engine, EngineOptions
    from mini_llm_runtime_amd.parts import DecoderModel
    import torch
    model = DecoderModel.load(model_folders["A"], torch.float32)
    eng = Engine(model, EngineOptions(context_tokens=256, max_model_len=64, max_active=3, batch_tokens=16,
                                      prefill_chunk=8, block_size=PAGE_SIZE["A"]))
    prompts = prompts_for("A", (20, 9, 14))
    ids = [eng.submit(p, max_tokens=12) for p in prompts]
    for _ in range(4):
        eng.step()
    assert eng.cancel(ids[0])
    done = eng.run_until_done()
    assert eng.finished[ids[0]].finish_reason == "cancelled" and len(done[ids[0]]) < 12
    for i in (1, 2):
        assert done[ids[i]] == plain_models["A"].greedy(prompts[i], 12)
    assert eng.runner.cache.free_pages() == eng.total_pages and eng.runner.free_slots() == 3
    eng.runner.cache.check()


def test_temperature_sampling_is_per_request(model_folders, plain_models):
    """Same seed, same tokens, alone or beside others; each token is the inverse-CDF draw of the plain
    distribution at the request's own uniform number."""
    from mini_llm_runtime_amd.api import LLM
    from mini_llm_runtime_amd.sampling import RequestRng
    from plain.qwen3_plain import temperature_cdf
    llm = LLM(model_folders["B"], dtype="float32", context_tokens=512, max_model_len=128, max_active=4,
              batch_tokens=32, prefill_chunk=16, block_size=8)
    prompts = prompts_for("B", (1, 9, 17, 30))
    together = llm.generate(prompts, max_tokens=6, temperature=0.8, seed=100)
    for i, prompt in enumerate(prompts):
        alone = llm.generate(prompt, max_tokens=6, temperature=0.8, seed=100 + i)
        assert alone == together[i]
        rng = RequestRng(100 + i)
        tokens = list(prompt)
        for t in together[i]:
            u = rng.uniform()
            cdf = temperature_cdf(plain_models["B"].logits(tokens, [len(tokens) - 1])[0], 0.8)
            lo = cdf[t - 1] if t > 0 else 0.0
            assert lo - 1e-4 <= u <= cdf[t] + 1e-4
            tokens.append(t)
    assert llm.generate(prompts[1], max_tokens=6, temperature=0.8, seed=5) != \
        llm.generate(prompts[1], max_tokens=6, temperature=0.8, seed=6)


def test_end_of_sequence_stops_generation(model_folders, plain_models):
    """Configuration C names token 5 as end of sequence: generation stops there unless told to go on."""
    from mini_llm_runtime_amd.api import LLM
    plain = plain_models["C"]
    llm = LLM(model_folders["C"], dtype="float32", context_tokens=512, max_model_len=256, max_active=2,
              batch_tokens=64, prefill_chunk=64, block_size=32)
    # find a prompt whose greedy continuation reaches token 5 early
    vocab = TINY["C"]["vocab_size"]
    found = None
    for first in range(vocab):
        out = plain.greedy([first], 4)
        if 5 in out[:3]:
            found = ([first], out)
            break
    if found is None:
        pytest.skip("no short greedy path to the end-of-sequence id with these weights")
    prompt, out = found
    stop = out.index(5)
    assert llm.generate(prompt, max_tokens=4) == out[:stop + 1]
    assert llm.generate(prompt, max_tokens=4, ignore_eos=True) == out


def run_cli(args):
    return subprocess.run([sys.executable, os.path.join(ROOT, "bin", "mini-llm")] + args, capture_output=True,
                          text=True, timeout=300)


def test_command_line(model_folders, plain_models, tmp_path):
    prompt = prompts_for("A")[1]
    ids = ",".join(str(t) for t in prompt)
    report_path = str(tmp_path / "report.json")
    done = run_cli(["--model", model_folders["A"], "--prompt-ids", ids, "--tokens", "6", "--dtype", "float32",
                    "--chunk", "4", "--context", "64", "--sequences", "1", "--output", report_path, "--device-time"])
    assert done.returncode == 0, done.stderr
    report = json.loads(done.stdout)
    assert report == json.load(open(report_path))
    assert report["token_ids"] == plain_models["A"].greedy(prompt, 6)
    assert report["prompt_tokens"] == 13 and report["completion_tokens"] == 6
    phases = [f["phase"] for f in report["forwards"]]
    assert phases == ["prefill"] * 4 + ["decode"] * 5               # 13 tokens in portions of 4; the last token is not fed back
    assert [f["input_tokens"] for f in report["forwards"][:4]] == [4, 4, 4, 1]
    assert report["used_kv_pages_before_release"] == 2 and report["used_kv_pages_after_release"] == 0
    assert report["forwards"][0]["device_elapsed_ms"] > 0
    # random-weights mode from a configuration file, seeded
    cfg_path = str(tmp_path / "cfg.json")
    json.dump(TINY["B"], open(cfg_path, "w"))
    a = run_cli(["--random-weights", cfg_path, "--seed", "3", "--prompt-ids", "1,2,3", "--tokens", "5"])
    b = run_cli(["--random-weights", cfg_path, "--seed", "3", "--prompt-ids", "1,2,3", "--tokens", "5"])
    assert a.returncode == 0 and json.loads(a.stdout)["token_ids"] == json.loads(b.stdout)["token_ids"]
    # the reference's names for what is one choice here, and its budget gate
    c = run_cli(["--model", model_folders["A"], "--prompt-ids", ids, "--tokens", "6", "--cuda-precision", "f32-pedantic",
                 "--kv-layout", "paged", "--context", "64", "--sequences", "1", "--device-budget-bytes", "100000000"])
    assert c.returncode == 0, c.stderr
    rc = json.loads(c.stdout)
    assert rc["token_ids"] == report["token_ids"] and rc["dtype"] == "float32"
    assert rc["device_bytes"]["cache"] == 2 * 2 * 2 * 16 * 4 * (4 + 1) * 16      # 2 layers x (k, v) x 2 heads x 16 x float x 5 pages x 16
    # errors: one line on stderr, exit code 1
    for args, text in [(["--model", model_folders["A"], "--prompt-ids", ids, "--output", report_path], "new file"),
                       (["--model", model_folders["A"], "--prompt-ids", "1,2", "--tokens", "0"], "not an integer in 1..4096"),
                       (["--model", model_folders["A"], "--prompt-ids", "999"], "vocabulary"),
                       (["--model", model_folders["A"], "--prompt-ids", ids, "--context", "15", "--tokens", "4"], "exceed"),
                       (["--model", model_folders["A"], "--bogus"], "not an option"),
                       (["--model", model_folders["A"], "--prompt-ids", ids, "--kv-layout", "contiguous"], "paged"),
                       (["--model", model_folders["A"], "--prompt-ids", ids, "--cuda-precision", "f16-matrix-f32acc"],
                        "f32-pedantic"),
                       (["--model", model_folders["A"], "--prompt-ids", ids, "--device-budget-bytes", "1000"], "exceed"),
                       (["--model", model_folders["A"], "--prompt-ids", ids, "--kv-dtype", "int8"], "--kv-dtype"),
                       (["--model", model_folders["A"], "--prompt-ids", ids, "--kv-dtype", "float32"], "element type"),
                       (["--model", str(tmp_path), "--prompt-ids", "1"], "config.json")]:
        bad = run_cli(args)
        assert bad.returncode == 1 and text in bad.stderr, (args, bad.stderr)
    ok = run_cli(["--model", model_folders["A"], "--prompt-ids", ids, "--tokens", "6", "--kv-dtype", "bfloat16", "--context", "64"])
    assert ok.returncode == 0, ok.stderr                             # (the bfloat16 engine's own element type)
    assert run_cli(["--help"]).returncode == 0 and run_cli([]).returncode == 1


def test_command_line_through_the_scheduler(model_folders, plain_models, tmp_path):
    """--prompts-file: every line a request of the scheduler (continuous batching over --sequences slots)."""
    prompts = prompts_for("A", (7, 13, 5, 1, 30, 9))
    path = str(tmp_path / "prompts.txt")
    with open(path, "w") as f:
        f.write("# one prompt a line\n" + "\n".join(",".join(str(t) for t in p) for p in prompts) + "\n")
    for policy in ("mixed", "prefill_first"):
        done = run_cli(["--model", model_folders["A"], "--prompts-file", path, "--tokens", "6", "--dtype", "float32",
                        "--context", "64", "--sequences", "3", "--batch", "16", "--chunk", "8", "--policy", policy,
                        "--check-finite"])
        assert done.returncode == 0, done.stderr
        report = json.loads(done.stdout)
        assert [r["input_token_ids"] for r in report["requests"]] == prompts
        for r, p in zip(report["requests"], prompts):
            assert r["token_ids"] == plain_models["A"].greedy(p, 6) and r["finish_reason"] == "length"
        assert report["policy"] == policy and report["completion_tokens"] == 36
        assert (report["scheduler"]["mixed_batches"] > 0) == (policy == "mixed")
        assert report["scheduler"]["max_batch_sequences"] <= 3 and report["used_kv_pages_after_release"] == 0
        plan = report["device_bytes"]["plan"]
        assert plan["kv_pages"] == report["device_bytes"]["cache"] and plan["total"] > plan["weights"] > 0
    for args, text in [(["--model", model_folders["A"], "--prompts-file", path, "--prompt-ids", "1"], "one of them"),
                       (["--model", model_folders["A"], "--prompts-file", path, "--policy", "fastest"], "--policy"),
                       (["--model", model_folders["A"], "--prompts-file", str(tmp_path / "none.txt")], "none.txt"),
                       (["--model", model_folders["A"], "--prompts-file", path, "--context", "32", "--tokens", "8"],
                        "exceed"),
                       (["--model", model_folders["A"], "--prompts-file", path, "--device-budget-bytes", "1000"],
                        "exceed")]:
        bad = run_cli(args)
        assert bad.returncode == 1 and text in bad.stderr, (args, bad.stderr)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_warm_up_stops_at_the_number_of_graphs_the_runner_keeps(model_folders, dtype):
    """A runner that keeps three captured shapes: the warm-up captures three (the shortest contexts' first)
    and stops, instead of pushing out what it has just captured."""
    from mini_llm_runtime_amd.api import parse_dtype
    from mini_llm_runtime_amd.engine import Runner
    from mini_llm_runtime_amd.parts import DecoderModel
    model = DecoderModel.load(model_folders["A"], parse_dtype(dtype), "cuda:0")
    r = Runner(model, max_tokens=4096, max_slots=4, max_length=1024, page_size=PAGE_SIZE["A"], max_graphs=3)
    assert r.warm_up() == 3 and len(r._graphs) == 3
    assert all(st["graph"] is not None and key[1] == 512 for key, st in r._graphs.items())
    assert r.warm_up() == 0 and r.graph_failures == 0
    assert r.free_slots() == 4 and r.cache.free_pages() == r.cache.num_pages


def test_warm_up_reaches_a_top_bucket_that_is_no_power_of_two(model_folders):
    """A limit of 768 tokens: the buckets are 512 and 768 (the capped top one is not twice the one below), and
    the warm-up captures the decoding step in both.  And a batch is never filled up beyond the rows of logits
    that were planned: nine slots decode as nine rows, not as ten."""
    import torch
    from mini_llm_runtime_amd.engine import Entry, Runner
    from mini_llm_runtime_amd.parts import DecoderModel
    model = DecoderModel.load(model_folders["A"], torch.bfloat16, "cuda:0")
    r = Runner(model, max_tokens=2048, max_slots=2, max_length=768, page_size=PAGE_SIZE["A"])
    assert r.warm_up() == 4
    one = (1, (0,))
    assert all(r._graphs[((one,) * n, b)]["graph"] is not None for n in (1, 2) for b in (512, 768))
    r = Runner(model, max_tokens=1024, max_slots=9, max_length=64, page_size=PAGE_SIZE["A"], max_logits_rows=9)
    slots = [r.open_request() for _ in range(9)]
    for _ in range(3):
        assert r.step([Entry(s, [5], [0]) for s in slots]).shape[0] == 9
    assert r.memory_report()["actual"]["workspace_beyond_plan"] == 0
    assert r._graphs[((one,) * 9, 64)]["graph"] is not None and ((one,) * 10, 64) not in r._graphs


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_warm_up_captures_the_decoding_steps_ahead_of_the_requests(model_folders, plain_models, dtype):
    """`Engine.warm_up`: the decoding steps of every batch size (and of the context buckets that fit) are
    captured while the engine is idle; the requests that follow find their graphs, meet no capture, read no
    leftover of the warm-up (the pages are NaN again) and get the plain greedy tokens."""
    import torch
    from mini_llm_runtime_amd.api import parse_dtype
    from mini_llm_runtime_amd.engine import Engine, EngineOptions
    from mini_llm_runtime_amd.parts import DecoderModel
    model = DecoderModel.load(model_folders["A"], parse_dtype(dtype), "cuda:0")
    eng = Engine(model, EngineOptions(context_tokens=4096, max_model_len=1024, max_active=6, batch_tokens=64,
                                      prefill_chunk=32, block_size=PAGE_SIZE["A"]))
    captured = eng.warm_up()
    runner = eng.runner
    one = (1, (0,))
    assert captured == 12 and all(runner._graphs[((one,) * n, b)]["graph"] is not None
                                  for n in range(1, 7) for b in (512, 1024))
    assert runner.graph_failures == 0 and runner.free_slots() == 6 and runner.cache.free_pages() == runner.cache.num_pages
    assert all(bool(torch.isnan(t).all()) for t in runner.cache.paged_tensors())
    assert eng.warm_up() == 0                                       # nothing left to capture
    prompts = prompts_for("A", (7, 13, 5, 1, 30, 9))
    ids = [eng.submit(p, max_tokens=12, ignore_eos=True) for p in prompts]
    eng.run_until_done()
    for rid, prompt in zip(ids, prompts):
        check_greedy(plain_models["A"], prompt, eng.finished[rid].generated, dtype)
    decode_graphs = [key for key, st in runner._graphs.items() if all(e == one for e in key[0]) and st["graph"] is not None]
    assert len(decode_graphs) == 12 and runner.graph_failures == 0
    assert runner.cache.free_pages() == runner.cache.num_pages


def test_text_prompts_through_the_command_line_and_the_entry_point(model_folders, plain_models, tmp_path):
    """A model folder that holds a tokenizer.json: --prompt TEXT (and no prompt option at all: the reference's
    default prompt, apps/cuda_main.cpp:53) runs the same tokens as --prompt-ids, the report holds the generated
    text, and `LLM.generate` takes and returns text."""
    import shutil
    pytest.importorskip("tokenizers")
    from test_tokenizer import WORDS, write_tokenizer
    from mini_llm_runtime_amd.api import LLM
    folder = str(tmp_path / "model")
    shutil.copytree(model_folders["A"], folder)
    write_tokenizer(os.path.join(folder, "tokenizer.json"))
    prompt = [2, 3, 4, 5, 6]                                           # "The capital of France is"
    expect = plain_models["A"].greedy(prompt, 6)
    common = ["--tokens", "6", "--dtype", "float32", "--context", "64", "--sequences", "1", "--ignore-eos"]
    by_ids = run_cli(["--model", folder, "--prompt-ids", "2,3,4,5,6"] + common)
    by_text = run_cli(["--model", folder, "--prompt", "The capital of France is"] + common)
    by_default = run_cli(["--model", folder] + common)
    elsewhere = run_cli(["--model", model_folders["A"], "--tokenizer", os.path.join(folder, "tokenizer.json"),
                         "--prompt", "the capital of france is"] + common)
    for done in (by_ids, by_text, by_default, elsewhere):
        assert done.returncode == 0, done.stderr
    reports = [json.loads(done.stdout) for done in (by_ids, by_text, by_default, elsewhere)]
    assert all(r["input_token_ids"] == prompt and r["token_ids"] == expect for r in reports)
    assert "text" not in reports[0]
    words = lambda ids: " ".join(WORDS[t] for t in ids if t < len(WORDS) and WORDS[t] != "<eos>")
    assert all(r["text"] == words(expect) for r in reports[1:])
    llm = LLM(folder, dtype="float32", context_tokens=256, max_model_len=64, max_active=2, block_size=PAGE_SIZE["A"])
    assert llm.generate("The capital of France is", max_tokens=6, ignore_eos=True) == words(expect)
    both = llm.generate(["the capital", "paris is a city"], max_tokens=4, ignore_eos=True)
    assert both == [words(plain_models["A"].greedy([2, 3], 4)), words(plain_models["A"].greedy([7, 6, 8, 9], 4))]
    bad = run_cli(["--model", folder, "--prompt", ""] + common)
    assert bad.returncode == 1 and "no token" in bad.stderr


def test_tokens_as_they_come(model_folders, plain_models):
    """`LLM.stream`: the same tokens as `generate`, handed out step by step, each request's last event with its reason."""
    from mini_llm_runtime_amd.api import LLM
    llm = LLM(model_folders["A"], dtype="float32", context_tokens=256, max_model_len=64, max_active=2,
              block_size=PAGE_SIZE["A"], batch_tokens=16, prefill_chunk=8)
    prompts = prompts_for("A", (7, 13, 5))
    got, reasons, order = {i: [] for i in range(3)}, {}, []
    for i, token, reason in llm.stream(prompts, max_tokens=5, ignore_eos=True):
        assert i not in reasons                                         # nothing after a request's last event
        if token is not None:
            got[i].append(token)
            order.append(i)
        if reason is not None:
            reasons[i] = reason
    assert reasons == {0: "length", 1: "length", 2: "length"}
    for i, prompt in enumerate(prompts):
        assert got[i] == plain_models["A"].greedy(prompt, 5)
    assert order != sorted(order)                                       # two slots: the requests' tokens come interleaved
    assert not llm.engine.finished and llm.runner.cache.free_pages() == llm.runner.cache.num_pages
    assert llm.generate(prompts[0], max_tokens=5, ignore_eos=True) == got[0]      # the engine goes on as before


def test_nothing_is_left_behind(model_folders, plain_models):
    """A batch with a prompt that is refused queues none of its prompts, and a stream that its reader closes
    early cancels what still runs: afterwards the engine is idle, every page and slot is free, and the next
    call answers as a fresh engine would."""
    from mini_llm_runtime_amd.api import LLM
    llm = LLM(model_folders["A"], dtype="float32", context_tokens=256, max_model_len=64, max_active=2,
              block_size=PAGE_SIZE["A"], batch_tokens=16, prefill_chunk=8)
    prompts = prompts_for("A", (7, 13, 5))

    def idle():
        return (not llm.engine.has_work() and not llm.engine.finished
                and llm.runner.cache.free_pages() == llm.runner.cache.num_pages
                and llm.runner.free_slots() == 2 and llm.engine.free_credits == llm.engine.total_pages)

    vocab = llm.model.spec.vocab_size
    with pytest.raises(ValueError, match="outside the vocabulary"):
        llm.generate([prompts[0], prompts[1], [1, vocab]], max_tokens=5)
    assert idle()
    with pytest.raises(ValueError, match="exceed max_model_len"):
        next(llm.stream([prompts[0], list(range(70))], max_tokens=5))
    assert idle()

    withdrawn = llm.engine.stats["cancelled"]               # (the prompts queued before the refused ones)
    assert withdrawn == 3
    events = llm.stream(prompts, max_tokens=20, ignore_eos=True)
    seen = [next(events) for _ in range(4)]                 # the first two requests run, the third still waits
    assert all(reason is None for _, _, reason in seen)
    events.close()
    assert idle() and llm.engine.stats["cancelled"] == withdrawn + 3
    assert llm.generate(prompts[2], max_tokens=6, ignore_eos=True) == plain_models["A"].greedy(prompts[2], 6)
    assert idle()
