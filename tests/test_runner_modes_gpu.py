"""What a runner can be asked for beside logits: its memory plan and budget gate, the check of the hidden
state after every layer, and time per kernel class."""
import numpy as np
import pytest
import torch

from conftest import PAGE_SIZE, TINY
from helpers import compare, make_requests, mixed, plain_logits, portions, run_steps, whole

pytestmark = pytest.mark.gpu

DTYPES = {"float32": torch.float32, "bfloat16": torch.bfloat16}


def load(model_folders, name, dtype_name, **kwargs):
    from mini_llm_runtime_amd.parts import DecoderModel
    return DecoderModel.load(model_folders[name], DTYPES[dtype_name], **kwargs)


# ------------------------------------------------------------------------------------------- memory
@pytest.mark.parametrize("dtype_name", DTYPES)
@pytest.mark.parametrize("name", ["A", "C"])
def test_what_is_held_is_what_was_planned(model_folders, name, dtype_name):
    """The reference asserts actual == planned for its arenas (src/minillm/cuda/runtime.cpp:134).  Here: the
    weights' arena, the cache and the scratch buffers hold exactly the planned bytes, and after steps of every
    kind (the largest allowed among them) nothing was allocated beyond the plan."""
    from mini_llm_runtime_amd.engine import Runner
    model = load(model_folders, name, dtype_name)
    assert model.arena.used == model.arena.planned >= model.weight_bytes()
    assert model.arena.planned - model.weight_bytes() < 256 * 64          # only the padding between tensors
    r = Runner(model, max_tokens=640, max_slots=4, max_length=160, max_batch_tokens=160, page_size=PAGE_SIZE[name])
    reqs = make_requests(TINY[name]["vocab_size"], [160, 33, 70, 2, 129], seed=3)
    for steps in (whole(reqs), portions(reqs), mixed(reqs, seed=2)[0]):
        run_steps(r, steps)
    report = r.memory_report()
    planned, actual = report["planned"], report["actual"]
    for key in ("weights", "kv_pages", "block_tables", "state", "workspace", "library_scratch"):
        assert actual[key] == planned[key], key
    assert actual["workspace_beyond_plan"] == 0
    assert planned["total"] == sum(v for k, v in planned.items() if k != "total")
    spec = model.cache_entry_specs[0]
    element = 4 if dtype_name == "float32" else 2
    pages = 640 // PAGE_SIZE[name] + 1
    assert planned["kv_pages"] == len(model.cache_entry_specs) * 2 * pages * PAGE_SIZE[name] * spec.kv_heads * \
        spec.head_dim * element


def test_stacked_projections_share_the_arena_without_a_copy(model_folders):
    model = load(model_folders, "B", "bfloat16")
    lo, hi = model.arena.memory.data_ptr(), model.arena.memory.data_ptr() + model.arena.memory.numel()
    for block in model.blocks:
        for t in (block.mixer.qkv, block.mixer.o, block.ffn.gate_up, block.ffn.down, block.norm1.weight):
            assert lo <= t.data_ptr() < hi and t.is_contiguous()
        assert block.mixer.qkv.shape == (4 * 32 + 2 * 32, 80) and block.ffn.gate_up.shape == (2 * 208, 80)
    assert lo <= model.embed.weight.data_ptr() < hi and lo <= model.head.weight.data_ptr() < hi


def test_the_budget_gate_refuses_before_anything_is_allocated(model_folders):
    from mini_llm_runtime_amd.engine import MemoryBudgetError, Runner
    torch.cuda.synchronize()
    before = torch.cuda.memory_allocated()
    with pytest.raises(MemoryBudgetError, match="weights need"):
        load(model_folders, "A", "float32", device_budget_bytes=1000)
    assert torch.cuda.memory_allocated() == before
    model = load(model_folders, "A", "float32", device_budget_bytes=0)        # no cap of the user's: the rule's share
    held = torch.cuda.memory_allocated()
    with pytest.raises(MemoryBudgetError, match="kv_pages"):
        Runner(model, max_tokens=1 << 20, max_slots=4, max_length=256, page_size=16, device_budget_bytes=50 << 20)
    assert torch.cuda.memory_allocated() == held
    r = Runner(model, max_tokens=256, max_slots=4, max_length=256, page_size=16, device_budget_bytes=50 << 20)
    assert r.memory_plan.to_allocate() <= 50 << 20
    # more wanted places than the runner was planned for are refused untouched
    from mini_llm_runtime_amd.engine import Entry, StepError
    r = Runner(model, max_tokens=256, max_slots=4, max_length=256, page_size=16, max_logits_rows=2)
    s = r.open_request()
    with pytest.raises(StepError, match="wanted places"):
        r.step([Entry(s, [1, 2, 3], [0, 1, 2])])
    assert r.length(s) == 0 and not r.poisoned
    assert r.step([Entry(s, [1, 2, 3], [0, 2])]).shape == (2, 256)


def test_a_pool_sized_from_the_budget_is_the_largest_that_fits_the_plan(model_folders):
    """`max_tokens=None`: the page pool takes what the budget leaves beside everything else that is planned
    (the reference has the cache's capacity and the budget side by side in its configuration,
    include/minillm/cuda/runtime.h:18-30, src/minillm/cuda/storage.cpp:168-181).  With a cap of the user's:
    what is held is what was planned, the plan fits the cap and one page more in every layer would not; without
    one and with few slots: the pool is what the slots can hold at all."""
    from mini_llm_runtime_amd.cache import CacheManager
    from mini_llm_runtime_amd.engine import Engine, EngineOptions, MemoryBudgetError, Runner
    model = load(model_folders, "A", "float32")
    cap = 24 << 20
    r = Runner(model, max_tokens=None, max_slots=64, max_length=1024, max_batch_tokens=64, page_size=16,
               device_budget_bytes=cap)
    plan, actual = r.memory_plan, r.memory_report()["actual"]
    assert r.max_tokens % 16 == 0 and 0 < r.max_tokens < 64 * 1024
    assert plan.to_allocate() <= cap and actual["kv_pages"] == plan.kv_pages == r.cache.kv_bytes()
    cache_bytes = plan.kv_pages + plan.block_tables + plan.state
    more = sum(CacheManager.plan(model.cache_entry_specs, torch.float32, 16, r.max_tokens + 16, 64, 1024))
    assert more > cache_bytes and plan.to_allocate() - cache_bytes + more > cap
    small = Runner(model, max_tokens=None, max_slots=3, max_length=100, max_batch_tokens=64, page_size=16)
    assert small.max_tokens == 3 * 112                       # three requests of 100 tokens, in whole pages
    with pytest.raises(MemoryBudgetError, match="leaves"):
        Runner(model, max_tokens=None, max_slots=4, max_length=1024, max_batch_tokens=64, page_size=16, device_budget_bytes=1 << 16)
    # the cache's element type is the engine's own
    with pytest.raises(ValueError, match="kv_dtype"):
        Runner(model, max_tokens=256, max_slots=4, max_length=256, page_size=16, kv_dtype="bfloat16")
    with pytest.raises(ValueError, match="kv_dtype"):
        Runner(model, max_tokens=256, max_slots=4, max_length=256, page_size=16, kv_dtype="int8")
    Runner(model, max_tokens=256, max_slots=4, max_length=256, page_size=16, kv_dtype="float32")
    # through the engine's options: what is left alone comes from the model and the device
    cap = 64 << 20
    eng = Engine(model, EngineOptions(max_active=4, device_budget_bytes=cap))
    o = eng.options
    assert (o.max_model_len, o.prefill_chunk, o.batch_tokens) == (1024, 2048, 2052)
    assert o.context_tokens == eng.runner.max_tokens == eng.total_pages * 16 == 4 * 1024
    assert eng.runner.memory_plan.to_allocate() <= cap
    out = eng.submit(list(range(1, 200)), max_tokens=4, ignore_eos=True)
    assert len(eng.run_until_done()[out]) == 4 and eng.stats["batches"] == 4      # the whole prompt in one step


# ------------------------------------------------------------------------------------- finite check
def overflowing_copy(folder, out, scale_tensor, factor):
    """A copy of a model folder with one tensor scaled (the reference's idiom for a hidden state that
    overflows, tests/cuda_runtime_tests.cpp:222-238)."""
    import json
    import os
    import shutil
    from mini_llm_runtime_amd.weights import SafetensorsFile, write_safetensors
    os.makedirs(out, exist_ok=True)
    shutil.copy(os.path.join(folder, "config.json"), os.path.join(out, "config.json"))
    f = SafetensorsFile(os.path.join(folder, "model.safetensors"))
    tensors = {name: f.tensor(name).clone() for name in f.entries}
    f.close()
    tensors[scale_tensor] = (tensors[scale_tensor].float() * factor).to(torch.float32)
    write_safetensors(os.path.join(out, "model.safetensors"), tensors, {"format": "pt"})
    return out


@pytest.mark.parametrize("dtype_name", DTYPES)
def test_a_hidden_state_that_overflows_is_reported_with_layer_and_row(model_folders, tmp_path, dtype_name):
    from mini_llm_runtime_amd.engine import Entry, NonFiniteHidden, Runner, StepError
    from mini_llm_runtime_amd.parts import DecoderModel
    folder = overflowing_copy(model_folders["A"], str(tmp_path / "big"), "model.layers.1.mlp.down_proj.weight", 3e38)
    model = DecoderModel.load(folder, DTYPES[dtype_name])
    toks = make_requests(256, [12], seed=5)["r0"]
    # without the check the step hands out what it has (the sampler would notice, a replay would not)
    quiet = Runner(model, max_tokens=64, max_slots=2, page_size=16)
    logits = quiet.step([Entry(quiet.open_request(), toks, [11])])
    assert not torch.isfinite(logits).all()
    r = Runner(model, max_tokens=64, max_slots=2, page_size=16, check_finite=True)
    s = r.open_request()
    with pytest.raises(NonFiniteHidden, match="layer run 1, batch row 0"):
        r.step([Entry(s, toks, [])])                                    # nothing wanted: noticed all the same
    assert r.poisoned
    with pytest.raises(StepError, match="earlier step failed"):
        r.step([Entry(s, [1], [0])])


@pytest.mark.parametrize("dtype_name", DTYPES)
@pytest.mark.parametrize("name", ["A", "C"])
def test_a_page_that_was_never_written_is_reported(model_folders, plain_models, name, dtype_name):
    """The cache is filled with NaN when it is made, so that a block table that points at a page nobody wrote
    shows: with the check on, the step that reads it raises.  A healthy run with the check on, also as
    replayed graphs, gives the plain logits and reports nothing."""
    from mini_llm_runtime_amd.engine import Entry, NonFiniteHidden, Runner
    model = load(model_folders, name, dtype_name)
    page = PAGE_SIZE[name]
    reqs = make_requests(TINY[name]["vocab_size"], [3 * page + 12], seed=7)
    want = plain_logits(plain_models[name], reqs)
    toks = reqs["r0"]
    r = Runner(model, max_tokens=8 * page, max_slots=2, page_size=page, check_finite=True)
    steps = [dict(step=0, entries=[dict(id="r0", tokens=toks[:3 * page], want=[0, 3 * page - 1])], end=[])]
    steps += [dict(step=1 + i, entries=[dict(id="r0", tokens=[toks[3 * page + i]], want=[0])], end=[]) for i in range(12)]
    got = run_steps(r, steps)                                           # the single tokens end as graph replays
    compare(got, {k: want[k] for k in got}, dtype_name)
    assert not r.poisoned and any(st["graph"] is not None for st in r._graphs.values())
    # now a request whose second block points at a page that was never written
    r = Runner(model, max_tokens=8 * page, max_slots=2, page_size=page, check_finite=True)
    s = r.open_request()
    r.step([Entry(s, toks[:2 * page + 1], [])])
    table = r.cache.kv_view(0).block_table
    used = set(table[s, :3].tolist())
    fresh = next(p for p in range(r.cache.num_pages) if p not in used)
    table[s, 1] = fresh
    with pytest.raises(NonFiniteHidden, match="layer run 0"):
        r.step([Entry(s, [toks[2 * page + 1]], [0])])
    assert r.poisoned


# ------------------------------------------------------------------------------------------ profile
def test_time_per_kernel_class(model_folders, plain_models):
    """profile=True: events around every launch, summed by class; steps run eagerly and still give the plain
    logits; the products' flops are the ones the shapes give."""
    from mini_llm_runtime_amd.engine import Runner
    name = "B"
    model = load(model_folders, name, "bfloat16")
    reqs = make_requests(TINY[name]["vocab_size"], [40], seed=9)
    want = plain_logits(plain_models[name], reqs)
    r = Runner(model, max_tokens=128, max_slots=2, page_size=PAGE_SIZE[name], profile=True, check_finite=True)
    assert not r.use_graphs
    steps = [dict(step=0, entries=[dict(id="r0", tokens=reqs["r0"][:32], want=list(range(32)))], end=[])]
    steps += [dict(step=1 + i, entries=[dict(id="r0", tokens=[reqs["r0"][32 + i]], want=[0])], end=[]) for i in range(8)]
    compare(run_steps(r, steps), want, "bfloat16")
    report = r.profile_report()
    assert set(report) >= {"embed", "gemm", "attention", "check", "total_ms"}
    layers, steps_run = 3, 9
    assert report["embed"]["calls"] == steps_run and report["check"]["calls"] == steps_run * (layers + 1)
    assert report["attention"]["calls"] >= steps_run * layers
    assert all(v["ms"] > 0 for k, v in report.items() if k != "total_ms")
    assert abs(report["total_ms"] - sum(v["ms"] for k, v in report.items() if k != "total_ms")) < 1e-2
    assert report["gemm"]["tflop_s"] > 0 and report["attention"]["gb_s"] > 0
    assert r.profile_report(reset=True) is not None and r.profile_report() == {"total_ms": 0}
    assert Runner(model, max_tokens=128, max_slots=2, page_size=8).profile_report() is None
