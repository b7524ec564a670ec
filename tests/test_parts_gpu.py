"""Each part of a layer alone, built from its spec through the registry, against the plain
implementation's function for that part; sizes differ from the tiny models'."""
import math

import numpy as np
import pytest
import torch

from plain import qwen3_plain as P

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.bfloat16]


def tol(dtype, want=None):
    """32-bit: the reference's unit tolerance.  Bfloat16 (8-bit mantissa, several roundings on the way):
    2 % of the output's scale, so that an element near zero is judged by the size of the sums behind it."""
    if dtype == torch.float32:
        return dict(atol=2e-4, rtol=2e-4)
    scale = 1.0 if want is None else float(np.abs(want).max())
    return dict(atol=2e-2 * max(scale, 1.0), rtol=2e-2)


def make_ctx(dtype, cache_specs, page_size=16, max_tokens=512, max_slots=4, max_length=512, split_keys=256,
             split_max_tokens=256):
    from mini_llm_runtime_amd.cache import CacheManager
    from mini_llm_runtime_amd.engine import StepContext, Workspace
    from mini_llm_runtime_amd.kernels import Kernels
    cache = CacheManager(cache_specs, dtype, "cuda", page_size, max_tokens, max_slots, max_length)
    return StepContext(Kernels(dtype), cache, Workspace("cuda"), dtype, max_length, split_keys, split_max_tokens)


def feed(ctx, segments):
    """segments: [(slot, number of tokens)]; reserves the pages and fills the step's vectors."""
    slots = [s for s, _ in segments]
    counts = [n for _, n in segments]
    first = [ctx.cache.length(s) for s in slots]
    ctx.cache.commit(slots, counts)
    pos, slot_of, segs, base = [], [], [], 0
    for s, n, p0 in zip(slots, counts, first):
        segs.append((s, base, n, p0))
        pos += list(range(p0, p0 + n))
        slot_of += [s] * n
        base += n
    ctx.n_tokens = base
    ctx.positions = torch.tensor(pos, dtype=torch.int32, device="cuda")
    ctx.slots = torch.tensor(slot_of, dtype=torch.int32, device="cuda")
    ctx.segments = segs
    ctx.max_context = max(p0 + n for (_, _, n, p0) in segs)


def rnd(shape, seed, scale=1.0):
    return scale * torch.randn(shape, generator=torch.Generator().manual_seed(seed))


def bind(part, tensors, dtype):
    specs = part.weight_specs()
    assert set(specs) == set(tensors)
    part.bind({k: v.to("cuda", torch.float32 if specs[k].keep_float32 else dtype).contiguous()
               for k, v in tensors.items()})


@pytest.mark.parametrize("dtype", DTYPES)
def test_norm_part(dtype):
    from mini_llm_runtime_amd.config import NormSpec
    from mini_llm_runtime_amd.parts import build_part
    norm = build_part("norm", NormSpec("rmsnorm", 96, 1e-4))
    w = 1 + rnd(96, 1, 0.3)
    bind(norm, {"weight": w}, dtype)
    ctx = make_ctx(dtype, [])
    h0 = rnd((6, 96), 2, 2.0).cuda()
    delta = rnd((6, 96), 3).to(dtype).cuda()
    h = h0.clone()
    out = torch.empty((6, 96), dtype=dtype, device="cuda")
    norm.forward(ctx, h, delta, out)
    x = h0.double().cpu().numpy() + delta.double().cpu().numpy()
    np.testing.assert_allclose(h.cpu().numpy(), x, atol=1e-6)
    np.testing.assert_allclose(out.double().cpu().numpy(), P.rms_norm(x, w.numpy(), 1e-4), **tol(dtype))


def test_position_part_table():
    from mini_llm_runtime_amd.config import PositionSpec
    from mini_llm_runtime_amd.parts import build_part
    rope = build_part("position", PositionSpec("rope_split_half", 48, 500000.0))
    table = rope.rotation_table(300, "cuda").cpu().numpy()
    cos, sin = P.rope_cos_sin(np.arange(300), 48, 500000.0)
    assert table.shape == (300, 48) and table.dtype == np.float32
    np.testing.assert_allclose(table[:, :24], cos, atol=1e-7)
    np.testing.assert_allclose(table[:, 24:], sin, atol=1e-7)


def attention_weights(hidden, hq, hkv, d, seed):
    return {"q_proj": rnd((hq * d, hidden), seed, 0.3), "k_proj": rnd((hkv * d, hidden), seed + 1, 0.3),
            "v_proj": rnd((hkv * d, hidden), seed + 2, 0.3), "o_proj": rnd((hidden, hq * d), seed + 3, 0.3),
            "q_norm.weight": 1 + rnd(d, seed + 4, 0.2), "k_norm.weight": 1 + rnd(d, seed + 5, 0.2)}


def plain_attention_block(x, w, hq, hkv, d, eps, base, positions, window):
    cfg = dict(num_attention_heads=hq, num_key_value_heads=hkv, head_dim=d, rms_norm_eps=eps, rope_theta=base)
    pw = {k.replace(".weight", ""): v.double().numpy() for k, v in w.items()}
    return P.attention_block(x, pw, cfg, positions, window)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("shape", [(40, 2, 2, 16, None), (72, 6, 2, 48, None), (64, 8, 1, 64, None),
                                   (40, 4, 2, 32, 21), (40, 4, 2, 32, 5)])
def test_attention_part_in_portions(dtype, shape):
    """The mixer on two requests side by side, cut into portions (and single tokens), against the plain
    mixer on each whole sequence.  With a window the cache gives pages back behind it."""
    from mini_llm_runtime_amd.config import AttentionSpec, NormSpec, PositionSpec
    from mini_llm_runtime_amd.parts import build_part
    hidden, hq, hkv, d, window = shape
    eps, base = 1e-5, 20000.0
    spec = AttentionSpec("gqa_attention", hidden, hq, hkv, d, 1 / math.sqrt(d), NormSpec("rmsnorm", d, eps),
                         PositionSpec("rope_split_half", d, base), window)
    mixer = build_part("mixer", spec)
    w = attention_weights(hidden, hq, hkv, d, 10)
    if dtype == torch.bfloat16:
        w = {k: v.to(torch.bfloat16).float() for k, v in w.items()}
    bind(mixer, w, dtype)
    ctx = make_ctx(dtype, [mixer.cache_spec()], page_size=8, max_tokens=160 if window else 256, max_length=256)
    lengths = [90, 61]
    xs = [rnd((n, hidden), 20 + i).to(dtype) for i, n in enumerate(lengths)]
    want = [plain_attention_block(x.double().numpy(), w, hq, hkv, d, eps, base, np.arange(n), window)
            for x, n in zip(xs, lengths)]
    slots = [ctx.cache.acquire_slot(), ctx.cache.acquire_slot()]
    done = [0, 0]
    got = [[], []]
    cuts = [(13, 1), (2, 1), (30, 1), (1, 7), (5, 1), (1, 1), (38, 50)]
    for cut in cuts:
        segs = [(slots[i], min(c, lengths[i] - done[i])) for i, c in enumerate(cut) if done[i] < lengths[i]]
        idx = [i for i in range(2) if done[i] < lengths[i]]
        feed(ctx, segs)
        x = torch.cat([xs[i][done[i]:done[i] + n] for i, (_, n) in zip(idx, segs)]).cuda().contiguous()
        out = mixer.forward(ctx, x, 0).double().cpu().numpy()
        at = 0
        for i, (_, n) in zip(idx, segs):
            got[i].append(out[at:at + n])
            at += n
            done[i] += n
        ctx.cache.retire([s for s, _ in segs])
        ctx.cache.check()
    assert done == lengths
    for i in range(2):
        np.testing.assert_allclose(np.concatenate(got[i]), want[i], **tol(dtype, want[i]))
    if window:
        live = sum(1 for p in ctx.cache.book.table(0).ravel() if p >= 0)
        assert live <= 2 * (-(-window // 8) + 1)           # only the pages a window still reaches are held


@pytest.mark.parametrize("dtype", DTYPES)
def test_attention_part_reads_another_entrys_cache(dtype):
    """write_cache=False: the mixer reads keys and values that an earlier run wrote into the entry."""
    from mini_llm_runtime_amd.config import AttentionSpec, NormSpec, PositionSpec
    from mini_llm_runtime_amd.parts import build_part
    hidden, hq, hkv, d = 32, 4, 2, 16
    spec = AttentionSpec("gqa_attention", hidden, hq, hkv, d, 0.25, NormSpec("rmsnorm", d, 1e-6),
                         PositionSpec("rope_split_half", d, 10000.0), None)
    mixer = build_part("mixer", spec)
    w = {k: v.to(torch.bfloat16).float() for k, v in attention_weights(hidden, hq, hkv, d, 30).items()}
    bind(mixer, w, dtype)
    ctx = make_ctx(dtype, [mixer.cache_spec()])
    slot = ctx.cache.acquire_slot()
    feed(ctx, [(slot, 20)])
    xa, xb = rnd((20, hidden), 31).to(dtype), rnd((20, hidden), 32).to(dtype)
    mixer.forward(ctx, xa.cuda(), 0, write_cache=True)
    out = mixer.forward(ctx, xb.cuda(), 0, write_cache=False).double().cpu().numpy()
    cfg = dict(num_attention_heads=hq, num_key_value_heads=hkv, head_dim=d, rms_norm_eps=1e-6, rope_theta=10000.0)
    pw = {k.replace(".weight", ""): v.double().numpy() for k, v in w.items()}
    pos = np.arange(20)
    _, k, v = P.project_qkv(xa.double().numpy(), pw, cfg, pos)
    q, _, _ = P.project_qkv(xb.double().numpy(), pw, cfg, pos)
    want = P.causal_attention(q, k, v, pos, 0.25).reshape(20, -1) @ pw["o_proj"].T
    np.testing.assert_allclose(out, want, **tol(dtype, want))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("sizes", [(40, 100), (76, 136), (128, 384)])
def test_feed_forward_part(dtype, sizes):
    from mini_llm_runtime_amd.config import MlpSpec
    from mini_llm_runtime_amd.parts import build_part
    hidden, inter = sizes
    ffn = build_part("ffn", MlpSpec("swiglu", hidden, inter))
    w = {"gate_proj": rnd((inter, hidden), 40, 0.3), "up_proj": rnd((inter, hidden), 41, 0.3),
         "down_proj": rnd((hidden, inter), 42, 0.3)}
    if dtype == torch.bfloat16:
        w = {k: v.to(torch.bfloat16).float() for k, v in w.items()}
    bind(ffn, w, dtype)
    ctx = make_ctx(dtype, [])
    x = rnd((9, hidden), 43).to(dtype)
    out = ffn.forward(ctx, x.cuda()).double().cpu().numpy()
    want = P.swiglu_mlp(x.double().numpy(), {k: v.double().numpy() for k, v in w.items()})
    np.testing.assert_allclose(out, want, **tol(dtype, want))


@pytest.mark.parametrize("dtype", DTYPES)
def test_block_part(dtype):
    """The arrangement: two pre-norm residuals; the block's last output is handed on as `pending`."""
    from mini_llm_runtime_amd.config import AttentionSpec, LayerSpec, MlpSpec, NormSpec, PositionSpec
    from mini_llm_runtime_amd.parts import build_part
    hidden, hq, hkv, d, inter, eps = 48, 3, 3, 16, 72, 1e-5
    norm = NormSpec("rmsnorm", hidden, eps)
    spec = LayerSpec("prenorm", norm, AttentionSpec("gqa_attention", hidden, hq, hkv, d, 0.25,
                                                     NormSpec("rmsnorm", d, eps),
                                                     PositionSpec("rope_split_half", d, 10000.0), None),
                     norm, MlpSpec("swiglu", hidden, inter))
    block = build_part("block", spec)
    aw = attention_weights(hidden, hq, hkv, d, 50)
    fw = {"gate_proj": rnd((inter, hidden), 56, 0.3), "up_proj": rnd((inter, hidden), 57, 0.3),
          "down_proj": rnd((hidden, inter), 58, 0.3)}
    n1, n2 = 1 + rnd(hidden, 59, 0.2), 1 + rnd(hidden, 60, 0.2)
    if dtype == torch.bfloat16:
        aw = {k: v.to(torch.bfloat16).float() for k, v in aw.items()}
        fw = {k: v.to(torch.bfloat16).float() for k, v in fw.items()}
    bind(block.norm1, {"weight": n1}, dtype)
    bind(block.norm2, {"weight": n2}, dtype)
    bind(block.mixer, aw, dtype)
    bind(block.ffn, fw, dtype)
    ctx = make_ctx(dtype, [block.mixer.cache_spec()])
    slot = ctx.cache.acquire_slot()
    feed(ctx, [(slot, 25)])
    h0 = rnd((25, hidden), 61)
    pending0 = rnd((25, hidden), 62).to(dtype)
    h = h0.cuda().clone()
    pending = block.forward(ctx, h, pending0.cuda(), 0).double().cpu().numpy()
    pw = {k.replace(".weight", ""): v.double().numpy() for k, v in {**aw, **fw}.items()}
    pw["input_layernorm"], pw["post_attention_layernorm"] = n1.double().numpy(), n2.double().numpy()
    cfg = dict(num_attention_heads=hq, num_key_value_heads=hkv, head_dim=d, rms_norm_eps=eps, rope_theta=10000.0)
    start = h0.double().numpy() + pending0.double().numpy()
    want = P.decoder_layer(start, pw, cfg, np.arange(25))
    np.testing.assert_allclose(h.double().cpu().numpy() + pending, want, **tol(dtype, want))


def test_block_part_with_few_rows_shares_its_norms_between_the_projections():
    """Up to 16 rows in the bfloat16 engine: every norm is split between the projection before it (which adds
    into h and leaves h * weight and partial sums of squares) and the projection after it (which applies the
    scale).  Two blocks in a row: the first hands the second's first norm over; the second, with nothing to
    follow, leaves a complete h.  Against the plain layers."""
    from mini_llm_runtime_amd.config import AttentionSpec, LayerSpec, MlpSpec, NormSpec, PositionSpec
    from mini_llm_runtime_amd.parts import build_part
    from mini_llm_runtime_amd.parts.registry import Handoff
    dtype = torch.bfloat16
    hidden, hq, hkv, d, inter, eps = 80, 4, 2, 32, 112, 1e-5
    norm = NormSpec("rmsnorm", hidden, eps)
    spec = LayerSpec("prenorm", norm, AttentionSpec("gqa_attention", hidden, hq, hkv, d, d ** -0.5,
                                                     NormSpec("rmsnorm", d, eps),
                                                     PositionSpec("rope_split_half", d, 10000.0), None),
                     norm, MlpSpec("swiglu", hidden, inter))
    blocks, plain_weights = [], []
    for i in range(2):
        block = build_part("block", spec)
        aw = {k: v.to(dtype).float() for k, v in attention_weights(hidden, hq, hkv, d, 150 + 10 * i).items()}
        fw = {k: v.to(dtype).float() for k, v in
              {"gate_proj": rnd((inter, hidden), 156 + i, 0.3), "up_proj": rnd((inter, hidden), 166 + i, 0.3),
               "down_proj": rnd((hidden, inter), 176 + i, 0.3)}.items()}
        n1, n2 = 1 + rnd(hidden, 186 + i, 0.2), 1 + rnd(hidden, 196 + i, 0.2)
        bind(block.norm1, {"weight": n1}, dtype)
        bind(block.norm2, {"weight": n2}, dtype)
        bind(block.mixer, aw, dtype)
        bind(block.ffn, fw, dtype)
        pw = {k.replace(".weight", ""): v.double().numpy() for k, v in {**aw, **fw}.items()}
        pw["input_layernorm"], pw["post_attention_layernorm"] = n1.double().numpy(), n2.double().numpy()
        blocks.append(block)
        plain_weights.append(pw)
    rows = 11
    ctx = make_ctx(dtype, [blocks[0].mixer.cache_spec(), blocks[1].mixer.cache_spec()])
    slot = ctx.cache.acquire_slot()
    feed(ctx, [(slot, rows)])
    assert ctx.kernels.handoff_supported(rows)
    h0 = rnd((rows, hidden), 161)
    pending0 = rnd((rows, hidden), 162).to(dtype)
    h = h0.cuda().clone()
    hand = blocks[0].forward(ctx, h, pending0.cuda(), 0, next_norm=blocks[1].norm1)
    assert isinstance(hand, Handoff) and hand.norm is blocks[1].norm1
    cfg = dict(num_attention_heads=hq, num_key_value_heads=hkv, head_dim=d, rms_norm_eps=eps, rope_theta=10000.0)
    want1 = P.decoder_layer(h0.double().numpy() + pending0.double().numpy(), plain_weights[0], cfg, np.arange(rows))
    np.testing.assert_allclose(h.double().cpu().numpy(), want1, **tol(dtype, want1))
    got_h = h.double().cpu().numpy()
    np.testing.assert_allclose(hand.ss.double().sum(-1).cpu().numpy(), (got_h ** 2).sum(-1), rtol=1e-5)
    np.testing.assert_allclose(hand.x.double().cpu().numpy(), got_h * plain_weights[1]["input_layernorm"], rtol=2 ** -7)
    last = blocks[1].forward(ctx, h, hand, 1, next_norm=None)
    assert last is None
    want2 = P.decoder_layer(want1, plain_weights[1], cfg, np.arange(rows))
    np.testing.assert_allclose(h.double().cpu().numpy(), want2, **tol(dtype, want2))
