"""The engine against the plain implementation, in 32-bit and in bfloat16, for every way of cutting
the same requests into steps: whole; most in one step and the last 32 tokens one by one; portions
of changing size down to two tokens; mixed, up to four live requests with so few pages that freed
pages are used again; long decoding; the first tokens of a sequence.  (The reference's counterpart:
240 teacher-forcing cases over chunk sizes and sequence counts, tests/cuda_validation_support.h:53-70.)
"""
import numpy as np
import pytest
import torch

from conftest import PAGE_SIZE, TINY
from helpers import (compare, last_one_by_one, make_requests, max_difference, mixed, plain_logits, portions,
                     run_steps, whole)

pytestmark = pytest.mark.gpu

DTYPES = {"float32": torch.float32, "bfloat16": torch.bfloat16}
LENGTHS = [70, 33, 100, 17, 64, 129, 2, 45]
_models = {}


def load(model_folders, name, dtype_name):
    from mini_llm_runtime_amd.parts import DecoderModel
    key = (name, dtype_name)
    if key not in _models:
        _models[key] = DecoderModel.load(model_folders[name], DTYPES[dtype_name])
    return _models[key]


def runner_for(model, name, max_tokens, **kwargs):
    from mini_llm_runtime_amd.engine import Runner
    return Runner(model, max_tokens=max_tokens, max_slots=4, page_size=PAGE_SIZE[name], **kwargs)


@pytest.fixture(scope="module")
def expected(plain_models):
    out = {}
    for name in TINY:
        reqs = make_requests(TINY[name]["vocab_size"], LENGTHS, seed=11)
        out[name] = (reqs, plain_logits(plain_models[name], reqs))
    return out


@pytest.mark.parametrize("dtype_name", DTYPES)
@pytest.mark.parametrize("name", TINY)
def test_every_way_of_cutting_gives_the_plain_logits(model_folders, expected, name, dtype_name):
    reqs, want = expected[name]
    model = load(model_folders, name, dtype_name)
    results = {}
    r = runner_for(model, name, max_tokens=192)          # one request at a time: 129 tokens -> 192
    for mode, steps in [("whole", whole(reqs)), ("last32", last_one_by_one(reqs)), ("portions", portions(reqs))]:
        results[mode] = run_steps(r, steps)
        compare(results[mode], want, dtype_name)
        r.cache.check()
        assert r.cache.free_pages() == r.cache.num_pages
    steps, peak = mixed(reqs, seed=5)
    assert max(len(s["entries"]) for s in steps) == 4
    # some step holds a portion of a prompt beside a single (decoded) token of another request
    assert any(min(len(e["tokens"]) for e in s["entries"]) == 1 and max(len(e["tokens"]) for e in s["entries"]) > 1
               for s in steps)
    total = sum(-(-n // 64) * 64 for n in LENGTHS)
    assert peak < total                                   # the pool is smaller than all requests together
    r = runner_for(model, name, max_tokens=peak)
    results["mixed"] = run_steps(r, steps)
    compare(results["mixed"], want, dtype_name)
    r.cache.check()
    assert r.cache.free_pages() == r.cache.num_pages
    # the same position, however it was cut and batched: the float engine has one order of additions per row and
    # key ranges of a fixed width, so its logits are the same to the bit (the reference's chunked and whole runs:
    # max_abs 0.0, tests/data/qwen3_greedy_reference.json:43-70); the bfloat16 engine runs few rows and many rows
    # through different kernels (streamed or tiled projections, fused or separate activation), so there the modes
    # differ by bfloat16 rounding, bounded here by 3 % of the largest logit
    scale = max(float(np.abs(v).max()) for v in want.values())
    limit = 0.0 if dtype_name == "float32" else 0.03 * scale
    for mode in ("last32", "portions", "mixed"):
        assert max_difference(results["whole"], results[mode]) <= limit, mode


@pytest.mark.parametrize("name", TINY)
def test_the_engine_without_the_vendor_library_gives_the_plain_logits(model_folders, expected, name):
    """`Runner(library_gemm=False)`: every matrix product of the bfloat16 engine on the hand-written kernels
    (the kernel for inner sizes that are no multiple of 64, the wide kernel's plain form, weight streaming up
    to 64 rows), whole, in portions, one by one and mixed, against the plain logits."""
    reqs, want = expected[name]
    model = load(model_folders, name, "bfloat16")
    r = runner_for(model, name, max_tokens=192, library_gemm=False)
    assert not r.kernels.library_gemm and r.memory_plan.library_scratch == 0
    for steps in (whole(reqs), last_one_by_one(reqs), portions(reqs)):
        compare(run_steps(r, steps), want, "bfloat16")
    steps, peak = mixed(reqs, seed=5)
    r = runner_for(model, name, max_tokens=peak, library_gemm=False)
    compare(run_steps(r, steps), want, "bfloat16")
    r.cache.check()
    assert r.cache.free_pages() == r.cache.num_pages
    assert r.kernels.library_workspace_bytes() == 0          # the library was never asked


@pytest.mark.parametrize("dtype_name", DTYPES)
@pytest.mark.parametrize("name", TINY)
@pytest.mark.parametrize("split_keys,split_max_tokens", [(64, 10 ** 6), (0, 0)])
def test_key_splits_do_not_change_the_result(model_folders, expected, name, dtype_name, split_keys, split_max_tokens):
    """Attention over key ranges split across workgroups (forced on for every batch, and off): single
    tokens, and prompt portions of changing size (the kernels for portions have splits of their own)."""
    reqs, want = expected[name]
    model = load(model_folders, name, dtype_name)
    for trace in (last_one_by_one(reqs), portions(reqs, sizes=(40, 3, 64, 17, 2, 33))):
        r = runner_for(model, name, max_tokens=192, split_keys=split_keys, split_max_tokens=split_max_tokens)
        compare(run_steps(r, trace), want, dtype_name)


@pytest.mark.parametrize("dtype_name", DTYPES)
@pytest.mark.parametrize("name", TINY)
def test_a_step_shape_that_comes_again_is_captured_and_stays_right(model_folders, plain_models, name, dtype_name):
    """A portion of 20 tokens of one request beside single tokens of two others, ten times over: the last
    times the step is a replayed graph.  Every step's logits against the plain ones."""
    vocab = TINY[name]["vocab_size"]
    reqs = make_requests(vocab, [215, 40, 33], seed=31)
    want = plain_logits(plain_models[name], reqs)
    model = load(model_folders, name, dtype_name)
    r = runner_for(model, name, max_tokens=384)
    a, b, c = reqs["r0"], reqs["r1"], reqs["r2"]
    steps = [dict(step=0, entries=[dict(id="r0", tokens=a[:15], want=[14]), dict(id="r1", tokens=b[:30], want=[29]),
                                   dict(id="r2", tokens=c[:23], want=[22])], end=[])]
    for i in range(10):
        steps.append(dict(step=1 + i, end=[], entries=[
            dict(id="r0", tokens=a[15 + 20 * i:35 + 20 * i], want=[0, 19]),
            dict(id="r1", tokens=[b[30 + i]], want=[0]), dict(id="r2", tokens=[c[23 + i]], want=[0])]))
    steps[-1]["end"] = ["r0", "r1", "r2"]
    got = run_steps(r, steps)
    compare(got, {k: v for k, v in want.items() if k in got}, dtype_name)
    assert len(got) == 3 + 10 * 4
    shape = ((20, (0, 19)), (1, (0,)), (1, (0,)))
    assert r.graph_failures == 0 and r._graphs[(shape, 512)]["graph"] is not None
    r.cache.check()
    assert r.cache.free_pages() == r.cache.num_pages


@pytest.mark.parametrize("dtype_name", DTYPES)
@pytest.mark.parametrize("name", ["A", "C"])
def test_decode_batches_are_filled_up_to_a_size_that_comes_again(model_folders, plain_models, name, dtype_name):
    """Eleven requests decode together, then ten, then nine: the steps run as graphs of twelve and of ten
    rows, the rows beyond the live requests being tokens of a scratch request that owns a page outside the
    pool.  Every step's logits against the plain ones, and against the same steps without graphs."""
    from mini_llm_runtime_amd.engine import Entry
    vocab = TINY[name]["vocab_size"]
    n = 11
    reqs = make_requests(vocab, [5 + (7 * i) % 19 + 12 for i in range(n)], seed=37)
    want = plain_logits(plain_models[name], reqs)
    model = load(model_folders, name, dtype_name)
    outs = []
    for use_graphs in (True, False):
        from mini_llm_runtime_amd.engine import Runner
        r = Runner(model, max_tokens=n * 64, max_slots=n, page_size=PAGE_SIZE[name], use_graphs=use_graphs)
        slots, at, got = {}, {}, {}
        for rid, toks in reqs.items():
            slots[rid] = r.open_request()
            at[rid] = len(toks) - 12
            r.step([Entry(slots[rid], toks[:at[rid]], [])])
        live = list(reqs)
        for step in range(12):
            if step in (4, 8):                              # one request ends: eleven -> ten -> nine
                r.close_request(slots.pop(live.pop()))
            logits = r.step([Entry(slots[rid], [reqs[rid][at[rid]]], [0]) for rid in live])
            assert logits.shape[0] == len(live)
            rows = logits.double().cpu().numpy()
            for rid, row in zip(live, rows):
                got[(rid, at[rid])] = row
                at[rid] += 1
        compare(got, {k: want[k] for k in got}, dtype_name)
        if use_graphs:
            sizes = sorted(len(sig[0]) for sig, st in r._graphs.items() if st["graph"] is not None)
            assert sizes == [10, 12] and r.graph_failures == 0
        for rid in live:
            r.close_request(slots[rid])
        r.cache.check()
        assert r.cache.free_pages() == r.cache.num_pages
        outs.append(got)
    limit = 2e-5 if dtype_name == "float32" else 0.03 * max(float(np.abs(v).max()) for v in outs[0].values())
    assert max_difference(outs[0], outs[1]) <= limit


@pytest.mark.parametrize("dtype_name", DTYPES)
@pytest.mark.parametrize("name", ["A", "C"])
def test_mixed_batches_fill_their_single_tokens_too(model_folders, plain_models, name, dtype_name):
    """Eleven, then ten, then nine requests decode beside a portion of 16 tokens of a long prompt, as the
    scheduler orders a mixed batch (single tokens first): the single tokens are filled up to twelve and to
    ten with rows of the scratch request, in front, so two shapes are captured where three came.  Every
    step's logits against the plain ones and against the same steps without graphs."""
    from mini_llm_runtime_amd.engine import Entry, Runner
    vocab = TINY[name]["vocab_size"]
    n = 11
    reqs = make_requests(vocab, [5 + (7 * i) % 19 + 12 for i in range(n)] + [16 * 13], seed=41)
    want = plain_logits(plain_models[name], reqs)
    model = load(model_folders, name, dtype_name)
    long_id = f"r{n}"
    outs = []
    for use_graphs in (True, False):
        r = Runner(model, max_tokens=n * 64 + 256, max_slots=n + 1, page_size=PAGE_SIZE[name], use_graphs=use_graphs,
                   graph_after=1)
        slots, at, got = {}, {}, {}
        for rid, toks in reqs.items():
            slots[rid] = r.open_request()
            if rid == long_id:
                at[rid] = 0
                continue
            at[rid] = len(toks) - 12
            r.step([Entry(slots[rid], toks[:at[rid]], [])])
        live = [rid for rid in reqs if rid != long_id]
        for step in range(12):
            if step in (4, 8):
                r.close_request(slots.pop(live.pop()))
            entries = [Entry(slots[rid], [reqs[rid][at[rid]]], [0]) for rid in live]
            entries.append(Entry(slots[long_id], reqs[long_id][16 * step:16 * step + 16], [3, 15]))
            logits = r.step(entries)
            assert logits.shape[0] == len(live) + 2
            rows = logits.double().cpu().numpy()
            for rid, row in zip(live, rows):
                got[(rid, at[rid])] = row
                at[rid] += 1
            got[(long_id, 16 * step + 3)], got[(long_id, 16 * step + 15)] = rows[len(live)], rows[len(live) + 1]
        compare(got, {k: want[k] for k in got}, dtype_name)
        if use_graphs:
            shapes = sorted(len(sig[0]) for sig, st in r._graphs.items() if st["graph"] is not None)
            assert shapes == [11, 13] and r.graph_failures == 0        # ten and twelve single tokens + the portion
        for rid in list(slots):
            r.close_request(slots[rid])
        r.cache.check()
        assert r.cache.free_pages() == r.cache.num_pages
        outs.append(got)
    limit = 2e-5 if dtype_name == "float32" else 0.03 * max(float(np.abs(v).max()) for v in outs[0].values())
    assert max_difference(outs[0], outs[1]) <= limit


@pytest.mark.parametrize("mode", ["evict", "mismatch"])
def test_graphs_that_are_dropped_or_do_not_hold(model_folders, plain_models, mode, monkeypatch):
    """With room for one captured shape, two alternating shapes push each other out again and again; and a
    shape whose replays do not match its eager run stays eager.  The logits are the plain ones either way."""
    from mini_llm_runtime_amd.engine import Runner
    name, dtype_name = "A", "bfloat16"
    reqs = make_requests(TINY[name]["vocab_size"], [120, 60], seed=37)
    want = plain_logits(plain_models[name], reqs)
    model = load(model_folders, name, dtype_name)
    if mode == "mismatch":
        monkeypatch.setattr(Runner, "_replays_match", staticmethod(lambda graph, result, expect, rewind=None: False))
    r = runner_for(model, name, max_tokens=256, max_graphs=1 if mode == "evict" else 48, graph_after=0)
    a, b = reqs["r0"], reqs["r1"]
    steps = [dict(step=0, entries=[dict(id="r0", tokens=a[:20], want=[19]), dict(id="r1", tokens=b[:30], want=[29])], end=[])]
    for i in range(12):                                  # a portion of 8 beside a single token; then two single tokens
        steps.append(dict(step=1 + 2 * i, end=[], entries=[dict(id="r0", tokens=a[20 + 8 * i:28 + 8 * i], want=[7]),
                                                           dict(id="r1", tokens=[b[30 + 2 * i]], want=[0])]))
        steps.append(dict(step=2 + 2 * i, end=[], entries=[dict(id="r1", tokens=[b[31 + 2 * i]], want=[0])]))
    steps[-1]["end"] = ["r0", "r1"]
    got = run_steps(r, steps)
    compare(got, {k: v for k, v in want.items() if k in got}, dtype_name)
    if mode == "evict":
        assert len(r._graphs) == 1 and r.graph_failures == 0
    else:
        tried = [st for st in r._graphs.values() if st["runs"] > 1]
        assert r.graph_failures == 2 == len(tried) and all(st["eager"] and st["graph"] is None for st in tried)


@pytest.mark.parametrize("dtype_name", DTYPES)
@pytest.mark.parametrize("name", ["A", "C"])
def test_long_decoding(model_folders, plain_models, name, dtype_name):
    """A five-token prompt, then 600 tokens one by one (teacher-forced): crosses many pages and key tiles."""
    toks = make_requests(TINY[name]["vocab_size"], [605], seed=3)["r0"]
    want = plain_logits(plain_models[name], {"r0": toks})
    model = load(model_folders, name, dtype_name)
    r = runner_for(model, name, max_tokens=640)
    steps = [dict(step=0, entries=[dict(id="r0", tokens=toks[:5], want=[0, 1, 2, 3, 4])], end=[])]
    steps += [dict(step=i, entries=[dict(id="r0", tokens=[toks[i]], want=[0])], end=[]) for i in range(5, 605)]
    steps[-1]["end"] = ["r0"]
    compare(run_steps(r, steps), want, dtype_name)
    # the single-token step was captured once for contexts up to 512 and once for the longer ones: a graph is
    # laid out (key splits) for its context bucket, not for the longest request the runner allows
    one = ((1, (0,)),)
    assert r._graphs[(one, 512)]["graph"] is not None and r._graphs[(one, 1024)]["graph"] is not None
    assert r.graph_failures == 0


@pytest.mark.parametrize("dtype_name", DTYPES)
@pytest.mark.parametrize("name", TINY)
def test_first_tokens_of_a_sequence(model_folders, plain_models, name, dtype_name):
    """Positions 0 and 1: a key set of one; four single-token prompts in one batch, then their second tokens."""
    vocab = TINY[name]["vocab_size"]
    reqs = {f"r{i}": [(17 * i + 3) % vocab, (5 * i + 1) % vocab] for i in range(4)}
    want = plain_logits(plain_models[name], reqs)
    model = load(model_folders, name, dtype_name)
    r = runner_for(model, name, max_tokens=256)
    steps = [dict(step=0, entries=[dict(id=rid, tokens=t[:1], want=[0]) for rid, t in reqs.items()], end=[]),
             dict(step=1, entries=[dict(id=rid, tokens=t[1:], want=[0]) for rid, t in reqs.items()], end=list(reqs))]
    compare(run_steps(r, steps), want, dtype_name)


def test_refused_batches_change_nothing(model_folders, plain_models):
    """The reference's list of invalid batches (tests/cuda_layer_tests.cpp:88-95) and an overcommitted pool:
    each is refused before anything is written, and the request goes on as if nothing had happened."""
    from mini_llm_runtime_amd.cache import CacheError, CacheFull
    from mini_llm_runtime_amd.engine import Entry, Runner, StepError
    model = load(model_folders, "A", "float32")
    r = Runner(model, max_tokens=64, max_slots=2, max_length=48, max_batch_tokens=40, page_size=16)
    toks = make_requests(256, [40], seed=9)["r0"]
    want = plain_models["A"].logits(toks)
    s = r.open_request()
    r.step([Entry(s, toks[:20], [])])                    # nothing wanted: the cache is written all the same
    other = r.open_request()
    bad = [[], [Entry(s, [], [])], [Entry(s, [256], [0])], [Entry(s, [-1], [0])], [Entry(s, [1, 2], [2])],
           [Entry(s, [1], [-1])], [Entry(7, [1], [0])], [Entry(s, [1], [0]), Entry(s, [2], [0])],
           [Entry(s, [1] * 41, [])], [Entry(s, [1] * 29, [])],            # beyond the step's limit; beyond max_length
           [Entry(s, [1, 2], [0, 0])], [Entry(s, [1] * 28, [3] * 60)],    # a place named twice; more rows than tokens
           [Entry(s, [1] * 10, []), Entry(other, [1] * 40, [])]]          # `other` needs 3 pages, 2 are free
    for batch in bad:
        with pytest.raises((StepError, CacheError, CacheFull)):
            r.step(batch)
        assert r.length(s) == 20 and r.length(other) == 0 and not r.poisoned
        r.cache.check()
    got = r.step([Entry(s, toks[20:], list(range(20)))]).double().cpu().numpy()
    np.testing.assert_allclose(got, want[20:], atol=2e-4, rtol=2e-4)
    # a slot used again after its request ended behaves like a fresh one
    r.close_request(s)
    s2 = r.open_request()
    again = r.step([Entry(s2, toks, list(range(40)))]).double().cpu().numpy()
    np.testing.assert_allclose(again, want, atol=2e-4, rtol=2e-4)


def test_steady_steps_allocate_nothing(model_folders):
    """After the first steps have sized the scratch memory, a step allocates no device memory (the
    reference asserts the same of its hot path, tests/cuda_runtime_tests.cpp:81-84)."""
    from mini_llm_runtime_amd.engine import Entry
    model = load(model_folders, "B", "bfloat16")
    r = runner_for(model, "B", max_tokens=256)
    s = r.open_request()
    r.step([Entry(s, list(range(40)), [39])])
    for t in range(3):                                   # eager, then captured as a graph, then replayed
        r.step([Entry(s, [t], [0])])
    for t in range(8):                                   # a shape that comes again and again is captured too
        r.step([Entry(s, [5, 6], [1])])
    torch.cuda.synchronize()
    before = torch.cuda.memory_stats()["allocation.all.allocated"]
    for t in range(30):
        r.step([Entry(s, [t], [0])])
        if t % 7 == 0:
            r.step([Entry(s, [t, t + 1], [1])])          # a portion between decoded tokens
    torch.cuda.synchronize()
    assert torch.cuda.memory_stats()["allocation.all.allocated"] == before


@pytest.mark.parametrize("seed", range(16))
def test_configurations_drawn_at_random(seed, tmp_path):
    """Sizes nobody chose: head sizes in steps of 16 up to 256 (and a few even ones between, which the scalar
    kernels serve), any number of heads and groups, widths and vocabularies that are multiples of nothing in
    particular, pages of 4 to 64 tokens (powers of two or not), tied or not.  Whole, last tokens one by one,
    portions and mixed, in both engines, against the plain implementation."""
    from mini_llm_runtime_amd.config import config_from_dict
    from mini_llm_runtime_amd.engine import Runner
    from mini_llm_runtime_amd.parts import DecoderModel
    from mini_llm_runtime_amd.weights import write_random_model
    from plain.qwen3_plain import PlainQwen3
    rng = np.random.default_rng(1000 + seed)
    kv_heads = int(rng.integers(1, 5))
    cfg = dict(architectures=["Qwen3ForCausalLM"],
               hidden_size=int(rng.integers(16, 150)) * 2 if seed % 2 else int(rng.integers(4, 40)) * 8,
               num_hidden_layers=int(rng.integers(1, 4)),
               num_attention_heads=kv_heads * int(rng.choice([1, 2, 3, 4, 5, 8])), num_key_value_heads=kv_heads,
               head_dim=int(rng.choice([16, 32, 48, 64, 80, 96, 112, 128, 144, 256] + ([24, 40, 72] if seed >= 8 else []))),
               intermediate_size=int(rng.integers(8, 200)) * 2, vocab_size=int(rng.integers(20, 700)),
               max_position_embeddings=2048, rms_norm_eps=float(rng.choice([1e-6, 1e-5, 3e-6])),
               rope_theta=float(rng.choice([1e4, 1e6, 5e5])), tie_word_embeddings=bool(rng.random() < 0.5))
    page = int(rng.choice([8, 16, 32, 64] + ([4, 12, 24] if seed >= 8 else [])))
    folder = str(tmp_path)
    write_random_model(folder, config_from_dict(cfg), seed=seed, matrix_std=0.12, norm_std=0.2)
    reqs = make_requests(cfg["vocab_size"], [int(x) for x in rng.integers(2, 160, 5)] + [int(rng.integers(260, 400))],
                         seed=seed)
    want = plain_logits(PlainQwen3(folder), reqs)
    for dtype_name, dtype in DTYPES.items():
        model = DecoderModel.load(folder, dtype)
        r = Runner(model, max_tokens=448, max_slots=4, page_size=page)
        for steps in (whole(reqs), last_one_by_one(reqs), portions(reqs)):
            compare(run_steps(r, steps), want, dtype_name)
        steps, peak = mixed(reqs, seed=seed)
        # (`peak` counts every request rounded up to 64 tokens; with pages that do not divide 64 a request of 64
        # tokens holds a little more: whole pages)
        r = Runner(model, max_tokens=peak // 64 * (-(-64 // page) * page), max_slots=4, page_size=page)
        compare(run_steps(r, steps), want, dtype_name)
        r.cache.check()
        assert r.cache.free_pages() == r.cache.num_pages
