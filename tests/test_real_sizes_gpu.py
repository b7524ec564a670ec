"""The engine at the widths of the benchmark models, with few layers so that the plain implementation stays
quick: hidden 1024, 16 q / 8 kv heads of 128, feed-forward 3072, vocabulary 151936, tied (two layers); and
hidden 4096, 32 q / 8 kv heads of 128, feed-forward 12288, untied, with a small vocabulary (one layer).  A
256-token prompt whole, in portions and with its last tokens decoded one by one, in 32-bit and in bfloat16,
against the plain logits.  Tiny models cannot show a fault that needs a head of 128 channels, four query
heads per kv head on the matrix cores, rows of 4096 or a vocabulary that fills many workgroups."""
import numpy as np
import pytest
import torch

from helpers import compare, make_requests

pytestmark = pytest.mark.gpu

CFG = dict(architectures=["Qwen3ForCausalLM"], hidden_size=1024, num_hidden_layers=2, num_attention_heads=16,
           num_key_value_heads=8, head_dim=128, intermediate_size=3072, vocab_size=151936,
           max_position_embeddings=4096, rms_norm_eps=1e-6, rope_theta=1000000.0, tie_word_embeddings=True)
WIDE = dict(architectures=["Qwen3ForCausalLM"], hidden_size=4096, num_hidden_layers=1, num_attention_heads=32,
            num_key_value_heads=8, head_dim=128, intermediate_size=12288, vocab_size=8192,
            max_position_embeddings=4096, rms_norm_eps=1e-6, rope_theta=1000000.0, tie_word_embeddings=False)
CONFIGS = {"narrow": CFG, "wide": WIDE}
WANT = [0, 1, 15, 16, 17, 32, 127, 128, 255]          # the reference's probe positions (tests/data/qwen3_validation_cases.json)


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    from mini_llm_runtime_amd.config import config_from_dict
    from mini_llm_runtime_amd.weights import write_random_model
    out = {}
    for name, cfg in CONFIGS.items():
        out[name] = str(tmp_path_factory.mktemp(f"real-sizes-{name}"))
        # N(0, 0.02) as in the benchmark; norm weights 1 + N(0, 0.1)
        write_random_model(out[name], config_from_dict(cfg), seed=7)
    return out


@pytest.fixture(scope="module")
def expectations(folders):
    from plain.qwen3_plain import PlainQwen3
    out = {}
    for name, cfg in CONFIGS.items():
        toks = make_requests(cfg["vocab_size"], [256], seed=17)["r0"]
        rows = PlainQwen3(folders[name]).logits(toks, WANT)
        out[name] = (toks, {("r0", p): rows[i] for i, p in enumerate(WANT)})
    return out


@pytest.mark.parametrize("dtype_name", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", list(CONFIGS))
def test_prompt_of_256_tokens_every_way(folders, expectations, name, dtype_name):
    from helpers import run_steps
    from mini_llm_runtime_amd.engine import Runner
    from mini_llm_runtime_amd.parts import DecoderModel
    toks, want = expectations[name]
    model = DecoderModel.load(folders[name], torch.float32 if dtype_name == "float32" else torch.bfloat16)
    r = Runner(model, max_tokens=512, max_slots=2, page_size=16)

    def wanted(lo, hi):
        return [p - lo for p in WANT if lo <= p < hi]
    whole = [dict(step=0, entries=[dict(id="r0", tokens=toks, want=WANT)], end=["r0"])]
    cuts = [0, 7, 16, 18, 100, 128, 224]
    portions = [dict(step=i, entries=[dict(id="r0", tokens=toks[lo:hi], want=wanted(lo, hi))], end=[])
                for i, (lo, hi) in enumerate(zip(cuts, cuts[1:]))]
    portions += [dict(step=100 + p, entries=[dict(id="r0", tokens=[toks[p]], want=wanted(p, p + 1))], end=[])
                 for p in range(224, 256)]
    portions[-1]["end"] = ["r0"]
    results = []
    for steps in (whole, portions):
        got = run_steps(r, steps)
        compare(got, want, dtype_name)
        results.append(got)
    scale = max(float(np.abs(v).max()) for v in want.values())
    limit = 2e-5 if dtype_name == "float32" else 0.03 * scale
    assert max(float(np.abs(results[0][k] - results[1][k]).max()) for k in want) <= limit
    # greedy continuation through the sampler: the plain argmax of the last position
    from mini_llm_runtime_amd.sampling import Sampler
    from mini_llm_runtime_amd.engine import Entry
    s = r.open_request()
    logits = r.step([Entry(s, toks, [255])])
    token = Sampler(r.kernels, r.device, 1).sample(logits, [0.0], [0.0])[0]
    row = want[("r0", 255)]
    top = np.sort(row)[-2:]
    if dtype_name == "float32" or top[1] - top[0] > 0.05 * np.abs(row).max():
        assert token == int(np.argmax(row))


@pytest.mark.parametrize("name", list(CONFIGS))
def test_prompt_of_256_tokens_without_the_vendor_library(folders, expectations, name):
    """The same prompt with every product on the hand-written kernels (`library_gemm=False`): whole (256 rows:
    the wide kernel, plain and gated), in portions of 7 to 96 tokens (17 to 64 rows: weight streaming, the
    16x16-tile kernel where the inner size allows) and one by one."""
    from helpers import run_steps
    from mini_llm_runtime_amd.engine import Runner
    from mini_llm_runtime_amd.parts import DecoderModel
    toks, want = expectations[name]
    model = DecoderModel.load(folders[name], torch.bfloat16)
    r = Runner(model, max_tokens=512, max_slots=2, max_batch_tokens=256, page_size=16, library_gemm=False)
    cuts = [0, 7, 16, 34, 98, 128, 224]
    steps = [dict(step=0, entries=[dict(id="w", tokens=toks, want=WANT)], end=["w"])]
    steps += [dict(step=1 + i, entries=[dict(id="r0", tokens=toks[lo:hi], want=[p - lo for p in WANT if lo <= p < hi])],
                   end=[]) for i, (lo, hi) in enumerate(zip(cuts, cuts[1:]))]
    steps += [dict(step=100 + p, entries=[dict(id="r0", tokens=[toks[p]], want=[0] if p in WANT else [])], end=[])
              for p in range(224, 256)]
    steps[-1]["end"] = ["r0"]
    got = run_steps(r, steps)
    compare({k: v for k, v in got.items() if k[0] == "w"}, {("w", p): v for (_, p), v in want.items()}, "bfloat16")
    compare({k: v for k, v in got.items() if k[0] == "r0"}, want, "bfloat16")
    assert r.kernels.library_workspace_bytes() == 0


@pytest.mark.parametrize("name", list(CONFIGS))
def test_graph_replays_with_library_products_match_eager(folders, name):
    """24 requests decode together: their projections have more than 16 rows and go to the vendor library,
    inside the captured graph.  Every replay (with eager work and synchronisations between the replays) must
    give what the same steps give without a graph: a library call that records a clearing node would show
    here as a difference on a later replay."""
    from mini_llm_runtime_amd.engine import Entry, Runner
    from mini_llm_runtime_amd.parts import DecoderModel
    model = DecoderModel.load(folders[name], torch.bfloat16)
    n = 24
    vocab = CONFIGS[name]["vocab_size"]
    prompts = make_requests(vocab, [9 + (5 * i) % 23 for i in range(n)], seed=23)
    feeds = make_requests(vocab, [8] * n, seed=29)
    outs = []
    for use_graphs in (True, False):
        r = Runner(model, max_tokens=n * 64, max_slots=n, page_size=16, use_graphs=use_graphs)
        slots = [r.open_request() for _ in range(n)]
        for s, toks in zip(slots, prompts.values()):
            r.step([Entry(s, toks, [])])
        steps = []
        for j in range(8):
            logits = r.step([Entry(s, [feeds[f"r{i}"][j]], [0]) for i, s in enumerate(slots)])
            steps.append(logits.float().cpu().numpy().copy())
            torch.cuda.synchronize()
            _ = (torch.ones(1000, device="cuda") * 2).sum().item()        # eager work between the replays
        outs.append(steps)
        assert r.use_graphs == use_graphs
    for j, (a, b) in enumerate(zip(*outs)):
        assert np.isfinite(a).all(), j
        np.testing.assert_array_equal(a, b, err_msg=f"decode step {j}")


LONG = {
    # heads as in the 0.6B sizes (two query heads a kv head, 128 channels), narrow otherwise
    "pairs": dict(architectures=["Qwen3ForCausalLM"], hidden_size=256, num_hidden_layers=2, num_attention_heads=4,
                  num_key_value_heads=2, head_dim=128, intermediate_size=512, vocab_size=1000,
                  max_position_embeddings=8192, rms_norm_eps=1e-6, rope_theta=1000000.0, tie_word_embeddings=True),
    # four query heads a kv head, as in the 8B sizes
    "fours": dict(architectures=["Qwen3ForCausalLM"], hidden_size=192, num_hidden_layers=1, num_attention_heads=8,
                  num_key_value_heads=2, head_dim=128, intermediate_size=384, vocab_size=777,
                  max_position_embeddings=8192, rms_norm_eps=1e-6, rope_theta=1000000.0, tie_word_embeddings=False),
}
LONG_TOKENS = 4700
LONG_WANT = [0, 100, 2047, 2048, 4095, 4096, 4600] + list(range(LONG_TOKENS - 33, LONG_TOKENS))


@pytest.mark.parametrize("name", list(LONG))
def test_a_context_of_4700_tokens(tmp_path, name):
    """A context beyond 4096 with heads of 128 channels: the prompt in portions of 1500, 1700 and the rest
    (the later portions attend to thousands of cached keys, in key splits where the engine chooses them),
    the last 32 tokens one by one (decoding over 4700 keys in key splits).  Both engines against the plain
    logits at the first, some middle and the last positions."""
    from helpers import run_steps
    from mini_llm_runtime_amd.config import config_from_dict
    from mini_llm_runtime_amd.engine import Runner
    from mini_llm_runtime_amd.parts import DecoderModel
    from mini_llm_runtime_amd.weights import write_random_model
    from plain.qwen3_plain import PlainQwen3
    cfg = LONG[name]
    folder = str(tmp_path)
    write_random_model(folder, config_from_dict(cfg), seed=3, matrix_std=0.06, norm_std=0.1)
    toks = make_requests(cfg["vocab_size"], [LONG_TOKENS], seed=31)["r0"]
    rows = PlainQwen3(folder).logits(toks, LONG_WANT)
    want = {("r0", p): rows[i] for i, p in enumerate(LONG_WANT)}
    cuts = [0, 1500, 3200, LONG_TOKENS - 32]
    steps = [dict(step=i, entries=[dict(id="r0", tokens=toks[lo:hi], want=[p - lo for p in LONG_WANT if lo <= p < hi])],
                  end=[]) for i, (lo, hi) in enumerate(zip(cuts, cuts[1:]))]
    steps += [dict(step=10 + p, entries=[dict(id="r0", tokens=[toks[p]], want=[0] if p in LONG_WANT else [])], end=[])
              for p in range(LONG_TOKENS - 32, LONG_TOKENS)]
    steps[-1]["end"] = ["r0"]
    for dtype_name, dtype in (("float32", torch.float32), ("bfloat16", torch.bfloat16)):
        model = DecoderModel.load(folder, dtype)
        r = Runner(model, max_tokens=4800, max_slots=2, max_length=4800, max_batch_tokens=2048, page_size=16)
        compare(run_steps(r, steps), want, dtype_name)
        r.cache.check()
        assert r.cache.free_pages() == r.cache.num_pages


@pytest.mark.parametrize("dtype_name", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", list(CONFIGS))
def test_six_requests_decode_together(folders, name, dtype_name):
    """Six requests of different lengths decode side by side at the benchmark models' widths: projections of
    six rows (with an inner size of 4096 and 12288 in the wide model, where the rows are staged through LDS),
    decoding attention over contexts of different lengths in one launch.  Against the plain logits."""
    from helpers import plain_logits, run_steps
    from mini_llm_runtime_amd.engine import Runner
    from mini_llm_runtime_amd.parts import DecoderModel
    from plain.qwen3_plain import PlainQwen3
    cfg = CONFIGS[name]
    reqs = make_requests(cfg["vocab_size"], [21, 40, 33, 17, 52, 28], seed=43)
    plain = PlainQwen3(folders[name])
    want = {}
    for rid, toks in reqs.items():
        rows = plain.logits(toks, list(range(len(toks) - 5, len(toks))))
        for i, p in enumerate(range(len(toks) - 5, len(toks))):
            want[(rid, p)] = rows[i]
    model = DecoderModel.load(folders[name], torch.float32 if dtype_name == "float32" else torch.bfloat16)
    r = Runner(model, max_tokens=6 * 64, max_slots=6, page_size=16)
    steps = [dict(step=i, entries=[dict(id=rid, tokens=toks[:len(toks) - 5], want=[])], end=[])
             for i, (rid, toks) in enumerate(reqs.items())]
    for j in range(5):
        steps.append(dict(step=10 + j, end=[], entries=[
            dict(id=rid, tokens=[toks[len(toks) - 5 + j]], want=[0]) for rid, toks in reqs.items()]))
    steps[-1]["end"] = list(reqs)
    compare(run_steps(r, steps), want, dtype_name)
    r.cache.check()


def test_a_request_of_70000_tokens_on_one_layer(tmp_path):
    """`max_length` 70 000 with pages of 16: more pages than one workgroup of either attention kernel keeps ids
    of, so the runner forces key ranges on prompt portions (from 32 736 keys on) and on single tokens (from
    65 504 on).  One layer of two heads of 64 channels; the prompt in portions of 8192, the last tokens one by
    one (captured and replayed in the bucket of 70 000), against the plain logits of the last positions, which
    are computed from the plain parts for those rows alone."""
    from helpers import run_steps
    from plain import qwen3_plain as P
    from mini_llm_runtime_amd.config import config_from_dict
    from mini_llm_runtime_amd.engine import Runner
    from mini_llm_runtime_amd.kernels import Kernels
    from mini_llm_runtime_amd.parts import DecoderModel
    from mini_llm_runtime_amd.weights import write_random_model
    cfg = dict(architectures=["Qwen3ForCausalLM"], hidden_size=64, num_hidden_layers=1, num_attention_heads=2,
               num_key_value_heads=1, head_dim=64, intermediate_size=96, vocab_size=301, max_position_embeddings=70000,
               rms_norm_eps=1e-6, rope_theta=1000000.0, tie_word_embeddings=True)
    total, tail = 69990, 6
    assert total > Kernels.mfma_longest_context(16) > Kernels.tiles_longest_context(16)
    folder = str(tmp_path)
    write_random_model(folder, config_from_dict(cfg), seed=9, matrix_std=0.2, norm_std=0.1)
    toks = make_requests(cfg["vocab_size"], [total], seed=12)["r0"]
    plain = P.PlainQwen3(folder)
    w, eps = plain.layers[0], cfg["rms_norm_eps"]
    positions = np.arange(total)
    h = P.embed(toks, plain.embed)
    q, k, v = P.project_qkv(P.rms_norm(h, w["input_layernorm"], eps), w, cfg, positions)
    wanted = [total - tail - 1] + list(range(total - tail, total))     # the prompt's last token, then every decoded one
    rows = []
    for t in wanted:
        heads = []
        for head in range(2):
            s = (k[:t + 1, 0] @ q[t, head]) / np.sqrt(64)
            a = np.exp(s - s.max())
            heads.append((a / a.sum()) @ v[:t + 1, 0])
        x = h[t] + np.concatenate(heads) @ w["o_proj"].T
        x = x + P.swiglu_mlp(P.rms_norm(x, w["post_attention_layernorm"], eps)[None], w)[0]
        rows.append(P.output_logits(x[None], plain.final_norm, plain.lm_head, eps)[0])
    want = {("r0", t): row for t, row in zip(wanted, rows)}
    cuts = list(range(0, total - tail, 8192)) + [total - tail]
    steps = [dict(step=i, entries=[dict(id="r0", tokens=toks[lo:hi], want=[hi - lo - 1] if hi == total - tail else [])],
                  end=[]) for i, (lo, hi) in enumerate(zip(cuts, cuts[1:]))]
    steps += [dict(step=100 + p, entries=[dict(id="r0", tokens=[toks[p]], want=[0])], end=[]) for p in range(total - tail, total)]
    steps[-1]["end"] = ["r0"]
    model = DecoderModel.load(folder, torch.bfloat16)
    r = Runner(model, max_tokens=70016, max_slots=1, max_length=70000, max_batch_tokens=8192, page_size=16)
    compare(run_steps(r, steps), want, "bfloat16")
    assert r.graph_failures == 0 and r._graphs[(((1, (0,)),), 70000)]["graph"] is not None
    report = r.memory_report()
    assert report["actual"]["workspace_beyond_plan"] == 0
    r.cache.check()
    assert r.cache.free_pages() == r.cache.num_pages
