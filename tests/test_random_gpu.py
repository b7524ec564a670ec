"""Runs drawn at random, each checked against the plain implementation: the scheduler with requests that
come, go, are cancelled and time out (greedy and temperature sampling, end-of-sequence ids that do occur), and
the step function fed valid and invalid batches side by side.  A few seeds each here; the same generators
have run for thousands."""
import numpy as np
import pytest

from conftest import PAGE_SIZE, TINY

pytestmark = pytest.mark.gpu


class SteppedClock:
    """The engine's clock, moved by the test: time-outs fall where the draw puts them, not where the machine does."""

    def __init__(self):
        self.t = 0.0

    def __call__(self):
        return self.t


@pytest.mark.parametrize("dtype_name", ["float32", "bfloat16"])
@pytest.mark.parametrize("seed", range(8))
def test_scheduler_runs_drawn_at_random(seed, dtype_name, tmp_path):
    """In bfloat16 (captured steps, batches filled up with scratch rows, norms handed between projections) the
    bounds follow from the engine's own tolerance against the plain logits, an error of at most d = 4 % of a
    row's largest logit: the greedy token's plain logit lies within 2 d of the best, and the plain cumulative
    distribution at temperature T differs from the engine's by at most (exp(2 d / T) - 1) / 2."""
    import math
    import torch
    from mini_llm_runtime_amd.config import config_from_dict
    from mini_llm_runtime_amd.engine import Engine, EngineOptions
    from mini_llm_runtime_amd.parts import DecoderModel
    from mini_llm_runtime_amd.sampling import RequestRng
    from mini_llm_runtime_amd.weights import write_random_model
    from plain.qwen3_plain import PlainQwen3, temperature_cdf
    rng = np.random.default_rng(210000 + seed)
    kv_heads = int(rng.integers(1, 4))
    vocab = int(rng.integers(12, 120))                     # small: the end-of-sequence id is drawn now and then
    cfg = dict(architectures=["Qwen3ForCausalLM"], hidden_size=int(rng.integers(4, 24)) * 8,
               num_hidden_layers=int(rng.integers(1, 3)), num_attention_heads=kv_heads * int(rng.choice([1, 2, 4])),
               num_key_value_heads=kv_heads, head_dim=int(rng.choice([16, 32, 64, 24])),
               intermediate_size=int(rng.integers(4, 40)) * 8, vocab_size=vocab, max_position_embeddings=512,
               rms_norm_eps=1e-6, rope_theta=10000.0, tie_word_embeddings=bool(rng.random() < 0.5),
               eos_token_id=int(rng.integers(0, vocab)))
    page = int(rng.choice([4, 8, 16, 32]))
    folder = str(tmp_path)
    write_random_model(folder, config_from_dict(cfg), seed=seed, matrix_std=0.12, norm_std=0.2)
    plain = PlainQwen3(folder)
    model = DecoderModel.load(folder, torch.float32 if dtype_name == "float32" else torch.bfloat16)
    pool = int(np.lcm(page, 16)) * int(rng.integers(8, 30))
    budget = int(rng.integers(8, 64))
    clock = SteppedClock()
    opts = EngineOptions(context_tokens=pool, max_model_len=min(160, pool), max_active=min(budget, int(rng.integers(1, 7))),
                         batch_tokens=budget, prefill_chunk=min(budget, int(rng.integers(2, 40))), block_size=page,
                         policy=str(rng.choice(["mixed", "prefill_first"])), aging_ms=int(rng.choice([1, 50, 250])),
                         portion_step=int(rng.choice([0, 8, 32])))
    eng = Engine(model, opts, clock=clock)
    sent, to_send, iterations = {}, int(rng.integers(5, 40)), 0
    while to_send or eng.has_work():
        for _ in range(int(rng.integers(0, 4))):
            n, out = int(rng.integers(1, 70)), int(rng.integers(1, 26))
            if not to_send or n + out > opts.max_model_len:
                continue
            kw = dict(max_tokens=out, temperature=float(rng.choice([0.0, 0.0, 0.7, 1.3])), seed=int(rng.integers(0, 1 << 40)),
                      ignore_eos=bool(rng.random() < 0.5), priority=int(rng.integers(0, 4)),
                      timeout_ms=None if rng.random() < 0.8 else int(rng.integers(1, 400)))
            prompt = rng.integers(0, vocab, n).tolist()
            if eng._pages_for(n + out) > eng.total_pages:
                continue                                    # (would be refused at submission: does not fit an idle pool)
            sent[eng.submit(prompt, **kw)] = (prompt, kw)
            to_send -= 1
        if sent and rng.random() < 0.1:
            eng.cancel(int(rng.choice(list(sent))))
        if eng.has_work():
            eng.step()
        clock.t += float(rng.choice([0.001, 0.01, 0.05]))
        iterations += 1
        assert iterations < 20000, "the engine makes no progress"
    assert set(eng.finished) == set(sent)
    eos = cfg["eos_token_id"]
    for rid, (prompt, kw) in sent.items():
        req = eng.finished[rid]
        got, reason = list(req.generated), req.finish_reason
        assert reason in ("length", "stop", "cancelled", "timeout") and len(got) <= kw["max_tokens"]
        assert (reason != "length" or len(got) == kw["max_tokens"]) and (reason != "stop" or got[-1] == eos)
        assert kw["ignore_eos"] or eos not in got[:-1]
        draws, context = RequestRng(kw["seed"]), list(prompt)
        for i, token in enumerate(got):
            row = plain.logits(context, [len(context) - 1])[0]
            d = 0.04 * float(np.abs(row).max())           # the bfloat16 engine's bound on a logit's error
            if kw["temperature"] > 0:                     # the token's stretch of the plain CDF holds the request's i-th number
                u, cdf = draws.uniform(), temperature_cdf(row, kw["temperature"])
                slack = 1e-4 if dtype_name == "float32" else (math.exp(2 * d / kw["temperature"]) - 1) / 2
                assert (cdf[token - 1] if token > 0 else 0.0) - slack <= u <= cdf[token] + slack, (rid, i)
            else:                                         # the largest logit (or within rounding of it)
                best = int(np.argmax(row))
                slack = 1e-4 * max(1.0, abs(row[best])) if dtype_name == "float32" else 2 * d
                assert token == best or row[best] - row[token] < slack, (rid, i)
            context.append(token)
    eng.runner.cache.check()
    assert eng.runner.cache.free_pages() == eng.runner.cache.num_pages and eng.free_credits == eng.total_pages
    assert eng.runner.graph_failures == 0


@pytest.mark.parametrize("seed", range(12))
def test_valid_and_invalid_batches_drawn_at_random(seed, model_folders, plain_models):
    """Whatever is wrong with a batch (a token id outside the vocabulary, a wanted place outside its entry or named
    twice, a slot twice or one that is not open, an empty entry, more tokens than the step, the request or the free
    pages take), it is refused with nothing changed; the valid batches between them go on giving the plain logits."""
    import torch
    from mini_llm_runtime_amd.cache import CacheError, CacheFull
    from mini_llm_runtime_amd.engine import Entry, Runner, StepError
    from mini_llm_runtime_amd.parts import DecoderModel
    rng = np.random.default_rng(250000 + seed)
    name = "ABC"[seed % 3]
    dtype_name = ("float32", "bfloat16")[(seed // 3) % 2]
    vocab, page = TINY[name]["vocab_size"], PAGE_SIZE[name]
    n_slots, max_length = int(rng.integers(1, 5)), int(rng.integers(8, 120))
    step_limit = int(rng.integers(4, 80))
    model = DecoderModel.load(model_folders[name], torch.float32 if dtype_name == "float32" else torch.bfloat16)
    r = Runner(model, max_tokens=page * int(rng.integers(2, 24)), max_slots=n_slots, max_length=max_length,
               max_batch_tokens=step_limit, page_size=page)
    live, refused, ran = {}, 0, 0                          # slot -> its tokens so far
    for _ in range(60):
        if len(live) < n_slots and rng.random() < 0.4:
            live[r.open_request()] = []
        if live and rng.random() < 0.1:
            s = int(rng.choice(list(live)))
            r.close_request(s)
            del live[s]
        if not live:
            continue
        chosen = [int(s) for s in rng.permutation(list(live))[:int(rng.integers(1, len(live) + 1))]]
        entries = []
        for s in chosen:
            n = int(rng.choice([1, 1, 2, 3, 5, 9, 17, 30]))
            want = sorted(set(int(w) for w in rng.integers(0, n, int(rng.integers(0, n + 1)))))
            entries.append(Entry(s, rng.integers(0, vocab, n).tolist(), want))
        pages = sum(-(-(len(live[e.slot]) + len(e.tokens)) // page) - -(-len(live[e.slot]) // page) for e in entries)
        ok = (sum(len(e.tokens) for e in entries) <= step_limit and pages <= r.cache.free_pages()
              and all(len(live[e.slot]) + len(e.tokens) <= max_length for e in entries))
        if rng.random() < 0.35:                            # something wrong on purpose
            kind, e = int(rng.integers(0, 7)), entries[int(rng.integers(0, len(entries)))]
            if kind == 0:
                e.tokens[int(rng.integers(0, len(e.tokens)))] = int(rng.choice([-1, vocab, vocab + 7]))
            elif kind == 1:
                e.want = list(e.want) + [len(e.tokens) + int(rng.integers(0, 3))]
            elif kind == 2:
                e.want = list(e.want) + [-1]
            elif kind == 3:
                entries.append(Entry(e.slot, [0], [0]))
            elif kind == 4:
                e.slot = int(rng.choice([s for s in range(-2, n_slots + 3) if s not in live]))
            elif kind == 5:
                e.tokens, e.want = [], []
            elif e.want:
                e.want = list(e.want) + [e.want[0]]
            ok = ok and kind == 6 and len(set(e.want)) == len(e.want)
        if not ok:
            before = ({s: r.length(s) for s in live}, r.cache.free_pages(), r.free_slots())
            with pytest.raises((StepError, CacheError, CacheFull)):
                r.step(entries)
            assert not r.poisoned and before == ({s: r.length(s) for s in live}, r.cache.free_pages(), r.free_slots())
            r.cache.check()
            refused += 1
            continue
        logits = r.step(entries)
        ran += 1
        rows = [] if logits is None else list(logits.double().cpu().numpy())
        for e in entries:
            seq = live[e.slot] + list(e.tokens)
            if e.want:
                for w, ref in zip(e.want, plain_models[name].logits(seq, [len(live[e.slot]) + w for w in e.want])):
                    scale = np.abs(ref).max()
                    bound = 2e-4 * (1 + scale) if dtype_name == "float32" else 0.04 * scale
                    assert np.abs(rows.pop(0) - ref).max() <= bound, (e.slot, w)
            live[e.slot] = seq
        assert not rows
    for s in list(live):
        r.close_request(s)
    r.cache.check()
    assert r.cache.free_pages() == r.cache.num_pages and ran > 0
