"""Shared by the GPU tests: builders of step traces (the trace tool's input format) in the ways
of cutting that must all give the same logits, a driver that feeds a trace to a Runner, and the
comparison with the plain implementation."""
import numpy as np

TOLERANCE = {
    # float engine against float64: rounding only (the reference's unit tolerance, 2e-4 + 2e-4 |e|,
    # tests/cuda_ops_tests.cu:38-41)
    "float32": dict(atol=2e-4, rtol=2e-4),
}


def make_requests(vocab, lengths, seed):
    rng = np.random.default_rng(seed)
    return {f"r{i}": rng.integers(0, vocab, n).tolist() for i, n in enumerate(lengths)}


def whole(requests):
    """Each request alone, whole, every position wanted."""
    return [dict(step=i, entries=[dict(id=rid, tokens=toks, want=list(range(len(toks))))], end=[rid])
            for i, (rid, toks) in enumerate(requests.items())]


def last_one_by_one(requests, tail=32):
    """Most of a request in one step, its last `tail` tokens one by one."""
    steps = []
    for rid, toks in requests.items():
        head = max(1, len(toks) - tail)
        steps.append(dict(entries=[dict(id=rid, tokens=toks[:head], want=list(range(head)))], end=[]))
        for i in range(head, len(toks)):
            steps.append(dict(entries=[dict(id=rid, tokens=[toks[i]], want=[0])], end=[]))
        steps[-1]["end"] = [rid]
    for i, s in enumerate(steps):
        s["step"] = i
    return steps


def portions(requests, sizes=(7, 2, 16, 3, 2, 33, 5, 2, 64, 9)):
    """Portions of changing size, down to two tokens."""
    steps = []
    for rid, toks in requests.items():
        at, k = 0, 0
        while at < len(toks):
            n = min(sizes[k % len(sizes)], len(toks) - at)
            k += 1
            steps.append(dict(entries=[dict(id=rid, tokens=toks[at:at + n], want=list(range(n)))], end=[]))
            at += n
        steps[-1]["end"] = [rid]
    for i, s in enumerate(steps):
        s["step"] = i
    return steps


def mixed(requests, seed, max_live=4, prefill_fraction=0.6):
    """Up to `max_live` requests at a time: portions of some prompts beside single (decoded) tokens of
    others; a request is sometimes left out of a step; a new one starts as soon as one has ended.
    Returns (steps, most tokens held at any time with every request rounded up to 64)."""
    rng = np.random.default_rng(seed)
    waiting = list(requests.items())
    live = {}                          # rid -> (tokens, tokens already run, prompt length)
    steps, peak = [], 0
    while waiting or live:
        while waiting and len(live) < max_live:
            rid, toks = waiting.pop(0)
            live[rid] = [toks, 0, max(1, int(len(toks) * prefill_fraction))]
        entries, ended = [], []
        for rid in list(live):
            toks, done, prompt = live[rid]
            if len(live) > 1 and rng.random() < 0.2:
                continue                                   # sits this step out
            if done < prompt:
                n = min(prompt - done, int(rng.choice([2, 2, 3, 5, 8, 13, 21])))
            else:
                n = 1
            entries.append(dict(id=rid, tokens=toks[done:done + n], want=list(range(n))))
            live[rid][1] = done + n
        held = sum(-(-state[1] // 64) * 64 for state in live.values())
        peak = max(peak, held)
        for rid in list(live):
            if live[rid][1] == len(live[rid][0]):
                ended.append(rid)
                del live[rid]
        if entries:
            steps.append(dict(step=len(steps), entries=entries, end=ended))
        elif ended:
            steps[-1]["end"] += ended
    return steps, peak


def run_steps(runner, steps):
    """Feed a trace to the engine's step function the way the trace tool does.
    Returns {(request id, position): float64 logits row}."""
    from mini_llm_runtime_amd.engine import Entry
    slots, position, out = {}, {}, {}
    for s in steps:
        entries, keys = [], []
        for e in s["entries"]:
            rid = e["id"]
            if rid not in slots:
                slots[rid] = runner.open_request()
                position[rid] = 0
            entries.append(Entry(slots[rid], e["tokens"], e["want"]))
            keys += [(rid, position[rid] + w) for w in e["want"]]
            position[rid] += len(e["tokens"])
        logits = runner.step(entries)
        if keys:
            rows = logits.double().cpu().numpy()
            assert rows.shape[0] == len(keys)
            for key, row in zip(keys, rows):
                assert key not in out
                out[key] = row
        for rid in s["end"]:
            runner.close_request(slots.pop(rid))
    return out


def plain_logits(plain, requests):
    out = {}
    for rid, toks in requests.items():
        rows = plain.logits(toks)
        for p in range(len(toks)):
            out[(rid, p)] = rows[p]
    return out


def bf16_close(got, want):
    """Bfloat16 engine against float64.  Thresholds in the manner of the reference's model-level
    contract (tests/data/qwen3_validation_cases.json:41-54: rmse, max abs, cosine, argmax unless a
    near tie), scaled to bfloat16's 8-bit mantissa: per row, max abs error <= 4 % of the row's
    largest logit, rmse <= 1.5 % of it, cosine >= 0.999, and the argmax agrees unless the plain top
    two are closer than twice the observed error."""
    scale = np.abs(want).max()
    err = np.abs(got - want)
    assert np.isfinite(got).all()
    assert err.max() <= 0.04 * scale, (err.max(), scale)
    assert np.sqrt((err ** 2).mean()) <= 0.015 * scale, (np.sqrt((err ** 2).mean()), scale)
    cos = float(got @ want / (np.linalg.norm(got) * np.linalg.norm(want)))
    assert cos >= 0.999, cos
    top = np.sort(want)[-2:]
    if top[1] - top[0] > 2 * err.max():
        assert int(np.argmax(got)) == int(np.argmax(want))


def compare(got, want, dtype_name):
    assert set(got) == set(want), (len(got), len(want))
    for key in sorted(want):
        if dtype_name == "float32":
            np.testing.assert_allclose(got[key], want[key], err_msg=str(key), **TOLERANCE["float32"])
        else:
            try:
                bf16_close(got[key], want[key])
            except AssertionError as err:
                raise AssertionError(f"{key}: {err}") from None


def max_difference(a, b):
    assert set(a) == set(b)
    return max(float(np.abs(a[k] - b[k]).max()) for k in a)
