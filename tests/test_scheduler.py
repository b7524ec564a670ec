"""The scheduler's decisions without a GPU.  The batch-forming vectors are the reference's own
(tests/core_tests.cpp:123-146).  The engine runs against a fake step function whose "logits" are
a hash of the request's token history, so any wrong position, order or mixing of requests changes
the output (the reference's FakeRunner idea, tests/core_tests.cpp:518-594)."""
import pytest

from mini_llm_runtime_amd.cache import CacheFull, PageBook
from mini_llm_runtime_amd.engine import Engine, EngineOptions, effective_priority, schedule_batch
from mini_llm_runtime_amd.options import Option, OptionError, parse


def test_mixed_budget_and_decode_protection():
    plan = schedule_batch([(0, 0, 0, 0, 0), (1, 10, 3, 0, 1), (2, 10, 0, 0, 2)], batch_tokens=8, prefill_chunk=4)
    assert plan == [(0, 1, False), (1, 4, True), (2, 3, True)]


def test_prefill_first_and_aging():
    plan = schedule_batch([(0, 0, 0, 0, 0), (1, 20, 3, 0, 1), (2, 20, 0, 2000, 2)], 8, 8, "prefill_first", 250)
    assert plan == [(2, 8, True)]                       # priority 0 + 2000/250 beats 3; no decode beside a prefill
    assert effective_priority(0, 2000, 250) == 8 and effective_priority(3, -5, 250) == 3


def test_decodes_first_then_prompts_in_order():
    items = [(0, 5, 0, 0, 3), (1, 0, 0, 0, 2), (2, 0, 0, 0, 1), (3, 100, 0, 0, 0)]
    assert schedule_batch(items, 16, 8) == [(2, 1, False), (1, 1, False), (3, 8, True), (0, 5, True)]
    assert schedule_batch(items, 2, 8) == [(2, 1, False), (1, 1, False)]           # budget spent on decodes
    assert schedule_batch(items, 3, 8) == [(2, 1, False), (1, 1, False), (3, 1, True)]
    assert schedule_batch([(7, 3, 0, 0, 0)], 100, 2) == [(7, 2, True)]
    assert schedule_batch([], 4, 4) == []
    with pytest.raises(ValueError):
        schedule_batch(items, 0, 8)
    with pytest.raises(ValueError):
        schedule_batch(items, 8, 8, "fastest")


def test_options_validation():
    """src/config.cpp:8-36; tests/core_tests.cpp:148-158."""
    EngineOptions().resolved(4096).validate()
    for change in [dict(max_active=0), dict(batch_tokens=4), dict(context_tokens=65), dict(max_model_len=1),
                   dict(prefill_chunk=0), dict(prefill_chunk=1000, batch_tokens=256), dict(aging_ms=0), dict(policy="x"),
                   dict(max_model_len=10000, context_tokens=8192), dict(kv_dtype="int8"), dict(device_budget_bytes=-1)]:
        with pytest.raises(ValueError):
            EngineOptions(**change).resolved(40960).validate()
    with pytest.raises(ValueError):
        EngineOptions().validate()                               # not resolved: the model's positions are not known yet


def test_options_left_alone_come_from_the_model_and_the_slots():
    """What is None is filled in: requests as long as the model allows, a step that holds one portion of 2048
    tokens beside a token of every slot; the pool stays None for the runner to size from the device's budget."""
    o = EngineOptions().resolved(40960)
    assert (o.max_model_len, o.prefill_chunk, o.batch_tokens, o.context_tokens) == (40960, 2048, 2048 + o.max_active, None)
    assert EngineOptions(max_model_len=1 << 20).resolved(40960).max_model_len == 40960
    o = EngineOptions(context_tokens=256, max_active=4).resolved(1024)            # a small pool bounds the step
    assert (o.batch_tokens, o.prefill_chunk) == (256, 256)
    o.validate()
    assert EngineOptions(batch_tokens=16, prefill_chunk=8).resolved(64).batch_tokens == 16


# ------------------------------------------------------------------------------- fake step function
class FakeSpec:
    vocab_size = 1000
    max_positions = 4096
    eos_token_ids = (999,)


class FakeModel:
    spec = FakeSpec()


def next_token(history):
    h = 1469598103934665603
    for i, t in enumerate(history):
        h = ((h ^ (t + 31 * i)) * 1099511628211) % (1 << 64)
    return h % 998                                          # never the end-of-sequence id


class FakeRunner:
    """Keeps the page bookkeeping real (native PageBook) and the model fake."""

    def __init__(self, options, eos_after=None):
        self.book = PageBook(options.max_active, options.max_model_len)
        self.book.add_group(options.block_size, options.context_tokens // options.block_size)
        self.history = {}
        self.batches = []
        self.max_batch_tokens = options.batch_tokens
        self.eos_after = eos_after or {}
        self.kernels = self.device = None

    def free_slots(self):
        return self.book.free_slots()

    def reserve_unit(self):
        return self.book.groups[0][0]

    def open_request(self):
        s = self.book.acquire_slot()
        self.history[s] = []
        return s

    def close_request(self, slot):
        self.book.release_slot(slot)
        del self.history[slot]

    def step(self, entries):
        assert sum(len(e.tokens) for e in entries) <= self.max_batch_tokens
        self.book.commit([e.slot for e in entries], [len(e.tokens) for e in entries])
        self.book.check()
        self.batches.append([(e.slot, len(e.tokens), list(e.want)) for e in entries])
        out = []
        for e in entries:
            for i, t in enumerate(e.tokens):
                self.history[e.slot].append(t)
                if i in e.want:
                    hist = self.history[e.slot]
                    out.append(999 if self.eos_after.get(tuple(hist[:2])) == len(hist) else next_token(hist))
        return out


class FakeSampler:
    def sample(self, logits, temperatures, uniforms):
        return list(logits)


def serial(prompt, n):
    hist, out = list(prompt), []
    for _ in range(n):
        out.append(next_token(hist))
        hist.append(out[-1])
    return out


def engine(clock=None, eos_after=None, **changes):
    opts = EngineOptions(**{**dict(context_tokens=256, max_model_len=128, max_active=4, batch_tokens=16,
                                   prefill_chunk=8, block_size=16), **changes})
    now = [0.0]
    eng = Engine(FakeModel(), opts, clock=clock or (lambda: now[0]), runner=FakeRunner(opts, eos_after),
                 sampler=FakeSampler())
    return eng, now


def test_batched_equals_serial():
    eng, _ = engine()
    prompts = [[1, 2, 3], list(range(10, 33)), [7], list(range(50, 59)), [4, 4, 4, 4], list(range(100, 140))]
    ids = [eng.submit(p, max_tokens=5 + i) for i, p in enumerate(prompts)]
    out = eng.run_until_done()
    for i, (rid, p) in enumerate(zip(ids, prompts)):
        assert out[rid] == serial(p, 5 + i)
        assert eng.finished[rid].finish_reason == "length"
    assert eng.stats["mixed_batches"] > 0 and eng.stats["max_batch_sequences"] > 1
    assert eng.stats["max_batch_tokens"] <= 16
    assert eng.free_credits == eng.total_pages and eng.runner.book.free_pages() == eng.total_pages
    assert eng.runner.book.free_slots() == 4


def test_prefill_first_leaves_decoding_requests_out_while_prompts_run():
    """Policy prefill_first through the engine: a request that is decoding gets no token in a step that runs
    a prompt, goes on later with an untouched history, and serial == batched; everything comes back."""
    eng, _ = engine(policy="prefill_first", batch_tokens=8, prefill_chunk=8)
    a = eng.submit([1, 2, 3], max_tokens=7)
    eng.step()
    eng.step()                                       # a has its first two tokens
    b = eng.submit(list(range(40, 60)), max_tokens=3)
    eng.step()
    assert eng.runner.batches[-1] == [(1, 8, [])]    # the prompt alone: a sits out
    c = eng.submit(list(range(70, 79)), max_tokens=2)
    out = eng.run_until_done()
    prompts = {a: [1, 2, 3], b: list(range(40, 60)), c: list(range(70, 79))}
    for rid, n in ((a, 7), (b, 3), (c, 2)):
        assert out[rid] == serial(prompts[rid], n)
    for batch in eng.runner.batches:                 # never a decoded token beside a prompt portion
        kinds = {"decode" if (n == 1 and want == [0]) else "prompt" for _, n, want in batch}
        assert kinds != {"decode", "prompt"} or all(n == 1 for _, n, _ in batch)
    assert eng.stats["mixed_batches"] == 0
    assert eng.free_credits == eng.total_pages and eng.runner.book.free_pages() == eng.total_pages
    assert eng.runner.book.free_slots() == 4


def test_prompt_portions_and_wanted_places():
    eng, _ = engine(batch_tokens=8, prefill_chunk=5)
    eng.submit(list(range(12)), max_tokens=3)
    eng.run_until_done()
    # 12 prompt tokens in portions of 5, 5, 2; logits only at the prompt's last token, then decode steps
    assert eng.runner.batches == [[(0, 5, [])], [(0, 5, [])], [(0, 2, [1])], [(0, 1, [0])], [(0, 1, [0])]]


def test_decode_runs_beside_a_long_prompt():
    eng, _ = engine(batch_tokens=8, prefill_chunk=8)
    a = eng.submit([1, 2], max_tokens=6)
    eng.step()                                       # a: whole prompt, first token sampled
    b = eng.submit(list(range(30)), max_tokens=2)
    eng.step()
    assert eng.runner.batches[-1] == [(0, 1, [0]), (1, 7, [])]      # the decode first, the rest of the budget to b
    out = eng.run_until_done()
    assert out[a] == serial([1, 2], 6) and out[b] == serial(list(range(30)), 2)


def test_stops_on_end_of_sequence_unless_ignored():
    eng, _ = engine(eos_after={(1, 2): 5})
    a = eng.submit([1, 2, 3], max_tokens=10)
    b = eng.submit([1, 2, 3], max_tokens=4, ignore_eos=True)
    out = eng.run_until_done()
    assert out[a][-1] == 999 and len(out[a]) == 3 and eng.finished[a].finish_reason == "stop"
    assert len(out[b]) == 4 and out[b][2] == 999 and eng.finished[b].finish_reason == "length"


def test_submit_refuses_what_can_never_run():
    eng, _ = engine()
    for kwargs in [dict(prompt=[]), dict(prompt=[1000]), dict(prompt=[-1]), dict(prompt=[1], max_tokens=0),
                   dict(prompt=[1] * 100, max_tokens=29), dict(prompt=[1], priority=4), dict(prompt=[1], temperature=-1.0)]:
        with pytest.raises(ValueError):
            eng.submit(**kwargs)
    small, _ = engine(context_tokens=64, max_model_len=64, batch_tokens=16)
    small.submit([1] * 30, max_tokens=34)            # exactly the whole pool
    big, _ = engine(context_tokens=64, max_model_len=64, batch_tokens=16)
    with pytest.raises(ValueError):
        big.submit([1] * 40, max_tokens=30)


def test_when_pages_run_out_requests_wait():
    """Every request sets aside the pages of its whole life at admission, so a running request can
    never be short of pages; one that does not fit waits for others to finish."""
    eng, _ = engine(context_tokens=64, max_model_len=64, max_active=4, batch_tokens=16)   # 4 pages
    a = eng.submit([1] * 20, max_tokens=12)          # 2 pages
    b = eng.submit([2] * 10, max_tokens=20)          # 2 pages
    c = eng.submit([3] * 5, max_tokens=5)            # 1 page: has to wait
    eng.step()
    assert [r.id for r in eng.active] == [a, b] and [r.id for r in eng.waiting] == [c]
    assert eng.free_credits == 0
    live_when_c_started = None
    while eng.has_work():
        eng.step()
        if live_when_c_started is None and any(r.id == c for r in eng.active):
            live_when_c_started = {r.id for r in eng.active}
        assert eng.runner.book.free_pages() >= eng.free_credits >= 0     # held pages never exceed what was set aside
    assert live_when_c_started is not None and len(live_when_c_started) <= 2
    out = {rid: r.generated for rid, r in eng.finished.items()}
    assert out[a] == serial([1] * 20, 12) and out[b] == serial([2] * 10, 20) and out[c] == serial([3] * 5, 5)
    assert eng.stats["admission_waits"] > 0 and eng.free_credits == 4


def test_the_step_function_refuses_an_overcommitted_batch_untouched():
    """Below the scheduler (as the trace tool drives it) a batch that needs more pages than are free
    is refused before anything changes."""
    opts = EngineOptions(context_tokens=32, max_model_len=32, max_active=2, batch_tokens=32, prefill_chunk=32)
    r = FakeRunner(opts)
    s0, s1 = r.open_request(), r.open_request()
    from mini_llm_runtime_amd.engine import Entry
    r.step([Entry(s0, [1] * 17, [])])
    with pytest.raises(CacheFull):
        r.step([Entry(s1, [1] * 5, [])])
    assert r.book.length(s1) == 0 and r.book.free_pages() == 0
    r.close_request(s0)
    r.step([Entry(s1, [1] * 5, [])])


def test_small_later_requests_overtake_until_the_reserve_time():
    eng, now = engine(context_tokens=64, max_model_len=64, max_active=4, batch_tokens=16, admission_reserve_ms=2000)
    a = eng.submit([1] * 30, max_tokens=18)          # 3 of 4 pages
    eng.step()
    big = eng.submit([2] * 20, max_tokens=20)        # 3 pages: waits
    small = eng.submit([3] * 4, max_tokens=4)        # 1 page: may overtake
    eng.step()
    assert {r.id for r in eng.active} == {a, small}
    eng.run_until_done()
    # the same, but the big request has already waited the reserve time: nothing overtakes it
    eng, now = engine(context_tokens=64, max_model_len=64, max_active=4, batch_tokens=16, admission_reserve_ms=2000)
    a = eng.submit([1] * 30, max_tokens=18)
    eng.step()
    big = eng.submit([2] * 20, max_tokens=20)
    now[0] = 2.5
    small = eng.submit([3] * 4, max_tokens=4)
    eng.step()
    assert {r.id for r in eng.active} == {a}
    out = eng.run_until_done()
    assert out[big] == serial([2] * 20, 20) and out[small] == serial([3] * 4, 4)


def test_priority_decides_who_is_admitted_first():
    eng, _ = engine(max_active=1, batch_tokens=16)
    low = eng.submit([1], max_tokens=2, priority=0)
    high = eng.submit([2], max_tokens=2, priority=3)
    eng.step()
    assert [r.id for r in eng.active] == [high]
    out = eng.run_until_done()
    assert out[low] == serial([1], 2) and out[high] == serial([2], 2)


def test_a_failed_step_stops_the_engine():
    eng, _ = engine()
    eng.submit([1, 2, 3], max_tokens=4)
    eng.sampler.sample = lambda *a: [5000]           # outside the vocabulary
    with pytest.raises(RuntimeError, match="invalid sample"):
        eng.step()
    with pytest.raises(RuntimeError, match="stopped"):
        eng.step()
    with pytest.raises(RuntimeError, match="stopped"):
        eng.submit([1], max_tokens=1)


# ------------------------------------------------------------------------------- command-line options
def test_option_parser():
    """The reference's rules (apps/options.h:12-62): exact names, a switch or one value, an option named twice
    or unknown is an error, numbers lie in their declared range."""
    table = [Option("--help", "switch"), Option("--ignore-eos", "switch"), Option("--model"),
             Option("--tokens", "int", 32, 1, 4096), Option("--chunk", "int", 7, 1, 10),
             Option("--temperature", "float", 0.0, 0.0, 10.0), Option("--prompt-ids", "ints", [])]
    o = parse(["--model", "m", "--tokens", "8", "--ignore-eos", "--temperature", "0.5", "--prompt-ids", "1,2,3"], table)
    assert o["--model"] == "m" and o["--ignore-eos"] is True and o["--help"] is False
    assert o.given("--tokens") and not o.given("--chunk") and not o.given("--help")
    assert o["--tokens"] == 8 and o["--chunk"] == 7 and o["--temperature"] == 0.5 and o["--prompt-ids"] == [1, 2, 3]
    assert parse([], table)["--tokens"] == 32 and parse(["--prompt-ids", ""], table)["--prompt-ids"] == []
    assert parse(["--model", "--help"], table)["--model"] == "--help"        # a value is whatever follows
    for argv in [["--model", "a", "--model", "b"], ["--bogus"], ["--model"], ["--tokens", "8", "extra"],
                 ["--help", "--help"], ["--tok", "8"], ["-model", "a"]]:
        with pytest.raises(OptionError):
            parse(argv, table)
    for text in ["0", "5000", "8x", "", " 8", "+8", "1e3", "8.0", "0x10"]:
        with pytest.raises(OptionError):
            parse(["--tokens", text], table)
    for text in ["nan", "inf", "-1", "x", "10.5", ""]:
        with pytest.raises(OptionError):
            parse(["--temperature", text], table)
    for text in ["1,a", "1,,2", "1, 2", ","]:
        with pytest.raises(OptionError):
            parse(["--prompt-ids", text], table)


def test_cancelled_requests_end_at_the_next_step_and_give_everything_back():
    """The reference's engine_bounded_queue_and_cancellation (tests/core_tests.cpp:969-981): a cancelled request
    ends with the reason "cancelled", the engine is idle afterwards, and an unknown id is not cancelled."""
    eng, now = engine(context_tokens=128, max_active=2)
    a = eng.submit(list(range(1, 30)), max_tokens=20)
    b = eng.submit(list(range(40, 50)), max_tokens=20)
    c = eng.submit(list(range(60, 70)), max_tokens=20)       # waits: two slots
    for _ in range(3):
        eng.step()
    assert eng.cancel(a) and eng.cancel(c) and not eng.cancel(12345)
    events = eng.step()
    assert (a, None, "cancelled") in events and (c, None, "cancelled") in events
    assert eng.finished[a].finish_reason == "cancelled" and eng.finished[c].generated == []
    done = eng.run_until_done()
    assert done[b] == serial(list(range(40, 50)), 20)          # the neighbour is not disturbed
    assert len(done[a]) < 20
    assert eng.free_credits == eng.total_pages and eng.runner.book.free_pages() == 128 // 16
    assert eng.runner.free_slots() == 2 and not eng.has_work()
    assert not eng.cancel(b)                                    # finished: nothing to cancel


def test_a_request_out_of_time_ends_waiting_or_running():
    """tests/core_tests.cpp:983-997: the reason is "timeout" and the resources come back."""
    eng, now = engine(context_tokens=128, max_active=1)
    a = eng.submit(list(range(1, 20)), max_tokens=40, timeout_ms=50)
    b = eng.submit(list(range(30, 40)), max_tokens=5, timeout_ms=20)     # waits behind a; runs out of time there
    c = eng.submit(list(range(50, 60)), max_tokens=5)
    eng.step()
    now[0] += 0.03
    events = eng.step()
    assert (b, None, "timeout") in events and eng.finished[b].generated == []
    now[0] += 0.03
    events = eng.step()
    assert (a, None, "timeout") in events and eng.finished[a].finish_reason == "timeout"
    assert eng.stats["timeouts"] == 2 and eng.stats["cancelled"] == 0
    done = eng.run_until_done()
    assert done[c] == serial(list(range(50, 60)), 5)
    assert eng.free_credits == eng.total_pages and eng.runner.free_slots() == 1
    for bad in (0, 300001):
        with pytest.raises(ValueError):
            eng.submit([1, 2], max_tokens=2, timeout_ms=bad)


def test_shutdown_ends_queued_and_running_requests():
    """tests/core_tests.cpp:1054: everything ends as cancelled, everything comes back, nothing new is taken."""
    eng, now = engine(context_tokens=128, max_active=2)
    ids = [eng.submit(list(range(1 + 10 * i, 9 + 10 * i)), max_tokens=30) for i in range(4)]
    for _ in range(3):
        eng.step()
    events = eng.shutdown()
    assert sorted(e[0] for e in events) == ids and all(e[2] == "cancelled" for e in events)
    assert not eng.has_work() and eng.free_credits == eng.total_pages and eng.runner.free_slots() == 2
    with pytest.raises(RuntimeError):
        eng.submit([1, 2, 3])


def test_portions_that_do_not_end_a_prompt_are_multiples_of_the_step():
    """Ours, not the reference's: with portion_step the shapes of steps come again.  The last portion of a
    prompt and portions shorter than the step stay as they are, so nothing starves."""
    items = [(0, 0, 0, 0, 0), (1, 0, 0, 0, 1), (2, 500, 0, 0, 2), (3, 500, 0, 0, 3)]
    assert schedule_batch(items, 256, 128, portion_step=0) == [(0, 1, False), (1, 1, False), (2, 128, True), (3, 126, True)]
    assert schedule_batch(items, 256, 128, portion_step=32) == [(0, 1, False), (1, 1, False), (2, 128, True), (3, 96, True)]
    # the prompt's end is not cut
    items = [(0, 0, 0, 0, 0), (2, 70, 0, 0, 2), (3, 45, 0, 0, 3)]
    assert schedule_batch(items, 256, 128, portion_step=32) == [(0, 1, False), (2, 70, True), (3, 45, True)]
    # less than a step left of the budget: the portion runs all the same
    items = [(0, 0, 0, 0, 0), (2, 500, 0, 0, 2)]
    assert schedule_batch(items, 8, 8, portion_step=32) == [(0, 1, False), (2, 7, True)]
    with pytest.raises(ValueError):
        schedule_batch(items, 8, 8, portion_step=-1)


def test_admission_is_a_pure_function_of_the_queue():
    """`admit` (native): the walk by aged priority, what fits starts, what does not is passed over until it has
    waited the reserve time, and then holds everything behind it back (src/engine.cpp:295-355)."""
    from mini_llm_runtime_amd.engine import admit
    # (pages of the whole life, priority, waited ms, order)
    queue = [(4, 0, 0, 0), (10, 0, 0, 1), (2, 0, 0, 2)]
    assert admit(queue, free_pages=6, free_slots=3) == ([0, 1, 2], [0, 2], 1)          # the second is passed over
    assert admit(queue, free_pages=16, free_slots=3) == ([0, 1, 2], [0, 1, 2], 0)
    assert admit(queue, free_pages=16, free_slots=1) == ([0, 1, 2], [0], 0)            # no slot: no wait counted
    assert admit(queue, free_pages=1, free_slots=3) == ([0, 1, 2], [], 3)
    assert admit([], free_pages=5, free_slots=2) == ([], [], 0)
    # one that has waited the reserve time walks first (eight aging intervals) and, not fitting, holds the rest back
    held = [(4, 0, 0, 0), (10, 0, 2000, 1), (2, 0, 0, 2)]
    assert admit(held, free_pages=6, free_slots=3) == ([1, 0, 2], [], 1)
    assert admit(held, free_pages=6, free_slots=3, reserve_ms=2001) == ([1, 0, 2], [0, 2], 1)
    assert admit(held, free_pages=12, free_slots=3) == ([1, 0, 2], [1, 2], 1)          # it starts; the first no longer fits
    # priority first, then waiting (an aging interval is worth one level), then arrival
    ranked = [(1, 0, 0, 0), (1, 3, 0, 1), (1, 1, 600, 2), (1, 3, 0, 3), (1, 2, 250, 4)]
    assert admit(ranked, free_pages=2, free_slots=5)[:2] == ([1, 2, 3, 4, 0], [1, 2])
    assert admit(ranked, free_pages=2, free_slots=5, aging_ms=1000)[0] == [1, 3, 4, 2, 0]
    for bad in (dict(aging_ms=0), dict(reserve_ms=-1), dict(free_pages=-1)):
        with pytest.raises(ValueError):
            admit(queue, **{"free_pages": 6, "free_slots": 3, **bad})
