"""Each HIP kernel alone against a plain formula in float64, at sizes other than the tiny
models' (the reference tests each op against a host formula in the same way,
tests/cuda_ops_tests.cu:38-72)."""
import math

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.bfloat16]


def tol(dtype):
    return dict(atol=2e-4, rtol=2e-4) if dtype == torch.float32 else dict(atol=2e-2, rtol=2e-2)


def kernels(dtype):
    from mini_llm_runtime_amd.kernels import Kernels
    return Kernels(dtype)


def sample(k, logits, temp, u, tokens, status):
    need_f, need_i = k.sample_scratch(logits.shape[0])
    k.sample(logits, temp, u, tokens, status, torch.empty(need_f, device="cuda"),
             torch.empty(need_i, dtype=torch.int32, device="cuda"))


def rnd(shape, dtype, seed, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (scale * torch.randn(shape, generator=g)).to(dtype).cuda()


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("width", [1, 17, 76, 128, 1000, 3072])
def test_embed_gather(dtype, width):
    k = kernels(dtype)
    table = rnd((37, width), dtype, 1)
    ids = torch.tensor([0, 36, 5, 5, 17], dtype=torch.int32).cuda()
    h = torch.full((5, width), 7.0, device="cuda")
    k.embed_gather(ids, table, h)
    assert torch.equal(h, table.float()[ids.long()])


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("width", [1, 17, 31, 32, 33, 128, 1024, 3072])
def test_add_rmsnorm(dtype, width):
    k = kernels(dtype)
    rows = 5
    h0 = rnd((rows, width), torch.float32, 2, 3.0)
    delta = rnd((rows, width), dtype, 3)
    w = rnd((width,), torch.float32, 4)
    eps = 1e-5
    x = h0.double() + delta.double()
    want = x * torch.rsqrt((x * x).mean(-1, keepdim=True) + eps) * w.double()
    # fused add: h is updated
    h = h0.clone()
    out = torch.empty((rows, width), dtype=dtype, device="cuda")
    k.add_rmsnorm(h, delta, w, out, eps)
    torch.testing.assert_close(h.double(), x, atol=1e-6, rtol=1e-6)
    torch.testing.assert_close(out.double(), want, **tol(dtype))
    # gathered rows, h untouched
    h = h0.clone()
    idx = torch.tensor([4, 0, 4], dtype=torch.int32).cuda()
    out = torch.empty((3, width), dtype=dtype, device="cuda")
    k.add_rmsnorm(h, delta, w, out, eps, rows=idx, write_h=False)
    assert torch.equal(h, h0)
    torch.testing.assert_close(out.double(), want[idx.long()], **tol(dtype))
    # no delta
    out = torch.empty((rows, width), dtype=dtype, device="cuda")
    k.add_rmsnorm(h, None, w, out, eps)
    x = h0.double()
    torch.testing.assert_close(out.double(), x * torch.rsqrt((x * x).mean(-1, keepdim=True) + eps) * w.double(),
                               **tol(dtype))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("width,repeat", [(257, 1), (256, 1), (256, 10)])
def test_rmsnorm_extremes(dtype, width, repeat):
    """Amplitudes from 0 to the largest float and an eps from the smallest to the largest
    (tests/cuda_ops_tests.cu:274-301): a row whose squares do not fit 32 bits is scaled by its largest element
    first, as the reference's kernel does for every row (src/minillm/cuda/ops.cu:87-126).  The widths and row
    counts reach each variant of the kernel (one workgroup a row, scalar or 16 bytes a thread; one wavefront a
    row from 64 rows on), with and without a delta that is still to be added."""
    k = kernels(dtype)
    top = float(np.finfo(np.float32).max)
    amps = [0.0, 1e-30, 1e-15, 1.0, 1e15, 1e30, top] * repeat
    h = torch.zeros((len(amps), width))
    for r, a in enumerate(amps):
        h[r, 0::3] = -a
        h[r, 1::3] = 0.5 * a
        h[r, 2::3] = 0.5 * a
    h = h.cuda()
    w = torch.ones(width, device="cuda")
    zero = torch.zeros((len(amps), width), dtype=dtype, device="cuda")
    for eps in (float(np.finfo(np.float32).smallest_subnormal), 1e-6, top):
        x = h.double()
        want = x * torch.rsqrt((x * x).mean(-1, keepdim=True) + eps)
        for delta, write_h in ((None, True), (zero, True), (zero, False)):
            out = torch.full((len(amps), width), 7.0, dtype=dtype, device="cuda")
            k.add_rmsnorm(h.clone(), delta, w, out, eps, write_h=write_h)
            assert torch.isfinite(out.float()).all(), (eps, write_h)
            torch.testing.assert_close(out.double(), want, **tol(dtype))
    # an infinity or a NaN in a row gives a row of NaN, and only that row
    bad = h.clone()
    bad[3, 5], bad[4, 7] = float("inf"), float("nan")
    out = torch.empty((len(amps), width), dtype=dtype, device="cuda")
    k.add_rmsnorm(bad, None, w, out, 1e-6)
    assert torch.isnan(out[3].float()).all() and torch.isnan(out[4].float()).all()
    assert torch.isfinite(out[[0, 1, 2, 5, 6]].float()).all()


@pytest.mark.parametrize("dtype", DTYPES)
def test_silu_mul_and_residual(dtype):
    k = kernels(dtype)
    inter = 100
    gate_up = rnd((7, 2 * inter), dtype, 5, 3.0)
    gate_up[0, :9] = torch.tensor([0, 1, -1, 80, -80, 1e4, -1e4, 30, -30], dtype=dtype)
    act = torch.empty((7, inter), dtype=dtype, device="cuda")
    k.silu_mul(gate_up, act)
    g, u = gate_up.double()[:, :inter], gate_up.double()[:, inter:]
    want = g / (1 + torch.exp(-g)) * u
    assert torch.isfinite(act.float()).all()
    torch.testing.assert_close(act.double(), want, **tol(dtype))
    h0 = rnd((7, inter), torch.float32, 6)
    h = h0.clone()
    k.residual_add(h, act)
    torch.testing.assert_close(h, h0 + act.float())


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("mnk", [(7, 19, 33), (5, 37, 131), (1, 311, 80), (16, 64, 64), (17, 130, 100),
                                 (64, 200, 76), (65, 257, 256), (200, 300, 1024), (2, 2048, 1024),
                                 (33, 48, 520), (48, 1000, 264), (8, 6144, 1024), (129, 100, 40),
                                 (5, 40, 192), (11, 72, 4160), (16, 33, 1024), (9, 130, 3072), (2, 24, 8192), (16, 40, 4096), (40, 96, 4096), (24, 56, 2048),
                                 (130, 70, 128), (300, 520, 192), (257, 1030, 64), (1000, 90, 320), (66, 4100, 1024)])
def test_gemm(dtype, mnk):
    """Odd shapes as in the reference's GEMM test (tests/cuda_unit_tests.cu:207-209)."""
    from mini_llm_runtime_amd.kernels import Kernels
    m, n, kk = mnk
    a = rnd((m, kk), dtype, 7)
    w = rnd((n, kk), dtype, 8)
    want = a.double() @ w.double().T
    # the engine's choice (many rows of the bfloat16 engine go to the library) and the hand-written kernels alone
    for k in (kernels(dtype), Kernels(dtype, library_gemm=False)):
        for out_dtype in {dtype, torch.float32}:
            out = torch.full((m, n), float("nan"), dtype=out_dtype, device="cuda")
            k.gemm(a, w, out)
            t = dict(atol=1e-4 * math.sqrt(kk), rtol=1e-5) if out_dtype == torch.float32 else \
                dict(atol=2e-2 * math.sqrt(kk) / 4, rtol=2e-2)
            torch.testing.assert_close(out.double(), want, **t)


@pytest.mark.parametrize("mnk", [(8, 6144, 2048), (3, 6100, 2048), (16, 5120, 2112), (1, 10240, 2048), (5, 4100, 4096),
                                 (8, 6144, 4096), (2, 5120, 8192)])
def test_gemm_two_strips_a_workgroup(mnk):
    """Few rows and numbers of columns that would deal strips of 16 unevenly to the compute units: a workgroup
    then owns two strips side by side (24, 20, ... columns), the last workgroup fewer.  Plain and with the rows'
    scale of a norm that was handed over; rows stay independent of the batch."""
    m, n, kk = mnk
    k = kernels(torch.bfloat16)
    a = rnd((m, kk), torch.bfloat16, 17)
    w = rnd((n, kk), torch.bfloat16, 18)
    want = a.double() @ w.double().T
    for out_dtype in (torch.bfloat16, torch.float32):
        out = torch.full((m, n), float("nan"), dtype=out_dtype, device="cuda")
        k.gemm(a, w, out)
        t = dict(atol=1e-4 * math.sqrt(kk), rtol=1e-5) if out_dtype == torch.float32 else \
            dict(atol=2e-2 * math.sqrt(kk) / 4, rtol=2e-2)
        torch.testing.assert_close(out.double(), want, **t)
    one = torch.empty((1, n), dtype=torch.bfloat16, device="cuda")
    k.gemm(a[m - 1:].contiguous(), w, one)
    assert torch.equal(one[0], out.to(torch.bfloat16)[m - 1]) or out_dtype != torch.bfloat16
    full = torch.empty((m, n), dtype=torch.bfloat16, device="cuda")
    k.gemm(a, w, full)
    assert torch.equal(one[0], full[m - 1])
    ss = (torch.rand((m, k.handoff_parts(kk)), device="cuda") + 0.5).float()
    scaled = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device="cuda")
    k.gemm_prenormed(a, ss, 1e-6, w, scaled)
    scale = 1.0 / torch.sqrt(ss.double().sum(dim=1) / kk + 1e-6)
    torch.testing.assert_close(scaled.double(), want * scale[:, None], atol=2e-2 * math.sqrt(kk) / 4, rtol=2e-2)


@pytest.mark.parametrize("dtype", DTYPES)
def test_gemm_rows_do_not_depend_on_the_batch(dtype):
    """A row's result is the same bits whatever rows stand beside it.  The float kernel has one order of
    additions for every M; the bfloat16 engine has two kernels (up to 64 rows the weight is streamed with k
    split over four wavefronts, above that it is tiled), each with a fixed order, so bits agree within a
    kernel and differ by rounding across the two."""
    from mini_llm_runtime_amd.kernels import Kernels
    k = Kernels(dtype, library_gemm=False)
    a = rnd((200, 264), dtype, 9)
    w = rnd((150, 264), dtype, 10)

    def run(lo, hi):
        out = torch.empty((hi - lo, 150), dtype=dtype, device="cuda")
        k.gemm(a[lo:hi].contiguous(), w, out)
        return out
    full = run(0, 200)
    small = run(0, 64)
    for lo, hi in [(0, 1), (3, 20), (30, 64), (0, 33)]:
        assert torch.equal(run(lo, hi), small[lo:hi])
    for lo, hi in [(0, 130), (100, 200), (65, 135)]:
        assert torch.equal(run(lo, hi), full[lo:hi])
    if dtype == torch.float32:
        assert torch.equal(small, full[:64])
    else:
        torch.testing.assert_close(small.float(), full[:64].float(), atol=0.13, rtol=1e-2)   # one bfloat16 step at |x| ~ 16


@pytest.mark.parametrize("shape", [0, 1, 2, 3])
@pytest.mark.parametrize("gated", [False, True])
@pytest.mark.parametrize("mnk", [(65, 70, 64), (300, 257, 192), (513, 1000, 128), (128, 256, 1024), (1, 5, 320)])
def test_gemm_wide_every_shape(shape, gated, mnk):
    """The many-row kernel in each of its workgroup shapes, plain and with the feed-forward's activation
    in its epilogue, at sizes that fill no tile; and the same bits from every shape (an output element is
    one chain of matrix-core sums over k, whatever tile it lies in)."""
    from mini_llm_runtime_amd.kernels.ops import _c_int, _p, _stream
    m, n, kk = mnk
    lib = kernels(torch.bfloat16)._lib("gemm")
    a = rnd((m, kk), torch.bfloat16, 60)
    w = rnd((2 * n if gated else n, kk), torch.bfloat16, 61, 0.3)

    def run(which, out_dtype):
        out = torch.full((m, n), float("nan"), dtype=out_dtype, device="cuda")
        rc = lib.mlr_gemm_wide(_p(a), _p(w), _p(out), _c_int(m), _c_int(n), _c_int(kk),
                               _c_int(1 if out_dtype == torch.float32 else 0), _c_int(which), _c_int(1 if gated else 0),
                               _stream())
        assert rc == 0, rc
        return out
    out = run(shape, torch.bfloat16)
    if gated:
        g = a.double() @ w.double()[:n].T
        u = a.double() @ w.double()[n:].T
        want = g / (1 + torch.exp(-g)) * u
    else:
        want = a.double() @ w.double().T
        torch.testing.assert_close(run(shape, torch.float32).double(), want, atol=1e-4 * math.sqrt(kk), rtol=1e-5)
    torch.testing.assert_close(out.double(), want, atol=2e-2 * float(want.abs().max()), rtol=2e-2)
    assert torch.equal(out, run(0, torch.bfloat16))
    assert torch.equal(out, run(-1, torch.bfloat16))


def test_gemm_wide_rows_do_not_depend_on_the_batch():
    """More than 64 rows with an inner size that is a multiple of 64: the tile shape follows the number of
    rows, a row's bits do not."""
    from mini_llm_runtime_amd.kernels import Kernels
    k = Kernels(torch.bfloat16, library_gemm=False)
    a = rnd((700, 256), torch.bfloat16, 62)
    w = rnd((1100, 256), torch.bfloat16, 63)

    def run(lo, hi):
        out = torch.empty((hi - lo, 1100), dtype=torch.bfloat16, device="cuda")
        k.gemm(a[lo:hi].contiguous(), w, out)
        return out
    full = run(0, 700)
    for lo, hi in [(0, 65), (100, 400), (630, 700), (1, 699)]:
        assert torch.equal(run(lo, hi), full[lo:hi])


def test_gemm_gated_silu_many_rows():
    """Without the library the feed-forward's first projection keeps its fused activation at any number
    of rows (inner size a multiple of 64)."""
    from mini_llm_runtime_amd.kernels import Kernels
    k = Kernels(torch.bfloat16, library_gemm=False)
    assert k.gated_silu_fused(2048, 1024) and not k.gated_silu_fused(2048, 1000)
    # beside the library it stays the way while the inner size is short
    assert kernels(torch.bfloat16).gated_silu_fused(2048, 1024) and kernels(torch.bfloat16).gated_silu_fused(256, 2048)
    assert not kernels(torch.bfloat16).gated_silu_fused(2048, 4096) and not kernels(torch.bfloat16).gated_silu_fused(512, 2048)
    m, n, kk = 333, 424, 384
    a = rnd((m, kk), torch.bfloat16, 64)
    w = rnd((2 * n, kk), torch.bfloat16, 65, 0.3)
    out = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device="cuda")
    k.gemm_gated_silu(a, w, out)
    g = a.double() @ w.double()[:n].T
    u = a.double() @ w.double()[n:].T
    want = g / (1 + torch.exp(-g)) * u
    torch.testing.assert_close(out.double(), want, atol=2e-2 * float(want.abs().max()), rtol=2e-2)


def plain_rope(x, pos, base):
    """x [T, H, D] float64 by the plain implementation's rotation (angles held in 32-bit, as the
    reference computes them)."""
    from plain.qwen3_plain import rope_cos_sin, rope_rotate
    cos, sin = rope_cos_sin(pos.numpy(), x.shape[-1], base)
    return torch.from_numpy(rope_rotate(x.numpy(), cos, sin))


def rope_table(max_pos, dim, base):
    from mini_llm_runtime_amd.config import PositionSpec
    from mini_llm_runtime_amd.parts.rope import RopeSplitHalf
    return RopeSplitHalf(PositionSpec("rope_split_half", dim, base)).rotation_table(max_pos, "cuda")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("shape", [(1, 1, 16, 4), (8, 2, 128, 16), (6, 3, 48, 8), (16, 16, 256, 32), (5, 1, 32, 1)])
def test_qk_norm_rope_kv(dtype, shape):
    """Positions around page edges and far ones (tests/cuda_ops_tests.cu:326); shuffled pages."""
    hq, hkv, d, page = shape
    k = kernels(dtype)
    positions = [0, 1, page - 1, page, page + 1, 2 * page + 3, 1535, 2047]
    positions = sorted(set(p for p in positions))
    m = len(positions)
    max_blocks = 2048 // page + 1
    # two slots: even rows in slot 1, odd rows in slot 0; pages handed out in a shuffled order
    slots = torch.tensor([1 - (i % 2) for i in range(m)], dtype=torch.int32)
    n_pages = 2 * m + 3
    perm = torch.randperm(n_pages, generator=torch.Generator().manual_seed(11)).tolist()
    table = torch.full((2, max_blocks), -1, dtype=torch.int32)
    for i, p in enumerate(positions):
        table[slots[i], p // page] = perm.pop()
    qkv = rnd((m, (hq + 2 * hkv) * d), dtype, 12)
    qw, kw = rnd((d,), torch.float32, 13) + 1, rnd((d,), torch.float32, 14) + 1
    eps, base = 1e-5, 1e6
    rope = rope_table(2048, d, base)
    k_pages = torch.full((n_pages, hkv, page, d), float("nan"), dtype=dtype, device="cuda")
    v_pages = torch.full((n_pages, hkv, d, page), float("nan"), dtype=dtype, device="cuda")
    q_out = torch.empty((m, hq * d), dtype=dtype, device="cuda")
    pos_t = torch.tensor(positions, dtype=torch.int32)
    k.qk_norm_rope_kv(qkv, q_out, k_pages, v_pages, table.cuda(), slots.cuda(), pos_t.cuda(), qw, kw, eps,
                      rope, hq, hkv, d, page)
    x = qkv.double().cpu()
    q = x[:, :hq * d].view(m, hq, d)
    kk = x[:, hq * d:(hq + hkv) * d].view(m, hkv, d)
    v = x[:, (hq + hkv) * d:].view(m, hkv, d)

    def norm(t, w):
        return t * torch.rsqrt((t * t).mean(-1, keepdim=True) + eps) * w.double().cpu()
    q_want = plain_rope(norm(q, qw), pos_t, base)
    k_want = plain_rope(norm(kk, kw), pos_t, base)
    torch.testing.assert_close(q_out.double().cpu().view(m, hq, d), q_want, **tol(dtype))
    written = torch.zeros((n_pages, page), dtype=torch.bool)
    for i, p in enumerate(positions):
        pg = table[slots[i], p // page].item()
        written[pg, p % page] = True
        torch.testing.assert_close(k_pages[pg, :, p % page].double().cpu(), k_want[i], **tol(dtype))
        assert torch.equal(v_pages[pg, :, :, p % page].cpu(), qkv[i, (hq + hkv) * d:].view(hkv, d).cpu())
    # nothing else was touched
    untouched = ~written[:, None, :, None].expand(n_pages, hkv, page, d)
    assert torch.isnan(k_pages.float().cpu()[untouched]).all()
    assert torch.isnan(v_pages.float().cpu().transpose(2, 3)[untouched]).all()
    # no norm, no rotation, no cache write
    k2 = torch.full_like(k_pages, float("nan"))
    k.qk_norm_rope_kv(qkv, q_out, k2, v_pages, table.cuda(), slots.cuda(), pos_t.cuda(), None, None, 0.0,
                      None, hq, hkv, d, page, write_cache=False)
    assert torch.equal(q_out.cpu(), qkv[:, :hq * d].cpu())
    assert torch.isnan(k2.float()).all()


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("case", [
    # (q heads, kv heads, head_dim, channels turned, interleaved, rows)
    (4, 2, 16, 8, True, 5), (4, 2, 16, 16, True, 70), (2, 1, 64, 32, False, 9), (2, 1, 64, 32, False, 130),
    (3, 3, 48, 2, True, 4), (2, 2, 128, 64, True, 66), (1, 1, 20, 10, False, 3), (2, 1, 256, 128, False, 2)])
def test_rotation_of_part_of_a_head_in_either_pairing(dtype, case):
    """The rotation kernel takes the extent and the pairing from its caller: the first `turned` channels of a
    head in pairs (j, j + turned / 2) or (2 j, 2 j + 1), the rest unrotated; the per-head norm spans the whole
    head either way.  (70 and 130 rows: the vector kernel for many rows must not be taken for these.)"""
    hq, hkv, d, turned, interleaved, rows = case
    k = kernels(dtype)
    page, eps = 16, 1e-5
    width = (hq + 2 * hkv) * d
    qkv = rnd((rows, width), dtype, 300)
    qw, kw = rnd((d,), torch.float32, 301) + 1, rnd((d,), torch.float32, 302) + 1
    n_pages = (rows + page - 1) // page + 1
    table = torch.arange(n_pages, dtype=torch.int32).flip(0).view(1, -1).contiguous().cuda()
    slots = torch.zeros(rows, dtype=torch.int32, device="cuda")
    pos = torch.arange(rows, dtype=torch.int32, device="cuda")
    angle = torch.arange(rows, dtype=torch.float64)[:, None] * (100.0 ** (-2.0 * torch.arange(turned // 2, dtype=torch.float64) / turned))[None, :]
    rope = torch.cat([torch.cos(angle), torch.sin(angle)], dim=1).float().cuda()
    k_pages = torch.full((n_pages, hkv, page, d), float("nan"), dtype=dtype, device="cuda")
    v_pages = torch.full((n_pages, hkv, d, page), float("nan"), dtype=dtype, device="cuda")
    q_out = torch.full((rows, hq * d), float("nan"), dtype=dtype, device="cuda")
    k.qk_norm_rope_kv(qkv, q_out, k_pages, v_pages, table, slots, pos, qw, kw, eps, rope, hq, hkv, d, page,
                      interleaved=interleaved)

    def want(x, w):                                      # x [rows, heads, d] float64
        x = x * torch.rsqrt((x * x).mean(-1, keepdim=True) + eps) * w.double().cpu()
        c, s = torch.cos(angle)[:, None, :], torch.sin(angle)[:, None, :]
        out = x.clone()
        if interleaved:
            a, b = x[..., 0:turned:2], x[..., 1:turned:2]
            out[..., 0:turned:2], out[..., 1:turned:2] = a * c - b * s, a * s + b * c
        else:
            a, b = x[..., :turned // 2], x[..., turned // 2:turned]
            out[..., :turned // 2], out[..., turned // 2:turned] = a * c - b * s, a * s + b * c
        return out
    x = qkv.double().cpu()
    torch.testing.assert_close(q_out.double().cpu().view(rows, hq, d), want(x[:, :hq * d].view(rows, hq, d), qw), **tol(dtype))
    k_want = want(x[:, hq * d:(hq + hkv) * d].view(rows, hkv, d), kw)
    for r in range(rows):
        pg = int(table[0, r // page])
        torch.testing.assert_close(k_pages[pg, :, r % page].double().cpu(), k_want[r], **tol(dtype))
        assert torch.equal(v_pages[pg, :, :, r % page].cpu(), qkv[r, (hq + hkv) * d:].view(hkv, d).cpu())


def plain_attention(q, keys, values, scale, window):
    """One query row over its visible keys, float64.  q [Hq, D]; keys, values [L, Hkv, D]."""
    hq, hkv = q.shape[0], keys.shape[1]
    g = hq // hkv
    L = keys.shape[0]
    lo = 0 if window is None else max(0, L - window)
    out = torch.zeros_like(q)
    for h in range(hq):
        s = (keys[lo:, h // g] @ q[h]) * scale
        a = torch.softmax(s, dim=0)
        out[h] = a @ values[lo:, h // g]
    return out


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("case", [
    # (q heads, kv heads, head_dim, page, lengths of the requests, window, split_keys)
    (4, 1, 16, 16, [1, 17, 33], None, 0),
    (4, 2, 128, 16, [15, 16, 17, 127, 128, 129], None, 0),
    (16, 8, 128, 16, [300, 1], None, 64),
    (6, 3, 48, 8, [70, 131], None, 64),
    (20, 1, 32, 32, [100], None, 0),
    (4, 4, 256, 16, [65], None, 0),
    (4, 2, 64, 16, [200, 40], 33, 0),
    (4, 2, 64, 16, [200, 40], 64, 128),
    (2, 1, 16, 4, [1000], None, 256),
    (6, 3, 48, 32, [100, 70], None, 0),
    (32, 2, 64, 16, [130, 5], None, 64),
    (8, 8, 80, 16, [77], 40, 0),
    (16, 8, 128, 16, [530, 3], None, 0),
    (4, 1, 96, 32, [150], 50, 0),
    (14, 2, 192, 16, [40], None, 0),
    (2, 1, 224, 16, [40], None, 0),
    (4, 2, 32, 16, [300], 70, 0),
    (8, 2, 64, 64, [333, 20], None, 128),
    (4, 2, 128, 128, [400, 130], None, 0),
    (6, 2, 96, 256, [300], 100, 64),
    (3, 1, 112, 32, [200], None, 0),
    (10, 2, 16, 16, [150, 64], 64, 0),
])
def test_paged_attention(dtype, case):
    """Every length is one request whose LAST token is the query (a decoded token) plus, for the
    first request, a query at every position (a whole prompt); pages shuffled.  Shapes after
    tests/cuda_layer_tests.cpp:528-536."""
    hq, hkv, d, page, lengths, window, split_keys = case
    k = kernels(dtype)
    g = torch.Generator().manual_seed(20)
    max_len = max(lengths)
    max_blocks = (max_len + page - 1) // page
    n_pages = sum((L + page - 1) // page for L in lengths) + 2
    perm = torch.randperm(n_pages, generator=g).tolist()
    table = torch.full((len(lengths), max_blocks), -1, dtype=torch.int32)
    k_pages = torch.full((n_pages, hkv, page, d), float("nan"), dtype=dtype)
    v_pages = torch.full((n_pages, hkv, d, page), float("nan"), dtype=dtype)
    keys, values = [], []
    for s, L in enumerate(lengths):
        kk = torch.randn((L, hkv, d), generator=g).to(dtype)
        vv = torch.randn((L, hkv, d), generator=g).to(dtype)
        keys.append(kk)
        values.append(vv)
        for b in range((L + page - 1) // page):
            pg = perm.pop()
            table[s, b] = pg
            n = min(page, L - b * page)
            k_pages[pg, :, :n] = kk[b * page:b * page + n].transpose(0, 1)
            v_pages[pg, :, :, :n] = vv[b * page:b * page + n].permute(1, 2, 0)
    rows = [(0, p) for p in range(lengths[0])] + [(s, L - 1) for s, L in enumerate(lengths) if s > 0]
    m = len(rows)
    q = (torch.randn((m, hq, d), generator=g) * 2).to(dtype)
    scale = 1 / math.sqrt(d)
    out = torch.full((m, hq * d), float("nan"), dtype=dtype, device="cuda")
    slots = torch.tensor([r[0] for r in rows], dtype=torch.int32).cuda()
    pos = torch.tensor([r[1] for r in rows], dtype=torch.int32).cuda()
    max_splits, partial = 1, None
    if split_keys:
        max_splits = (max_len + split_keys - 1) // split_keys
        partial = torch.full((k.attention_partial_numel(m, hq, d, max_splits),), float("nan"), device="cuda")
    k.paged_attention(q.view(m, hq * d).cuda(), k_pages.cuda(), v_pages.cuda(), table.cuda(), slots, pos, out,
                      hq, hkv, d, page, scale, window=window, split_keys=split_keys, max_splits=max_splits,
                      partial=partial)
    got = out.double().cpu().view(m, hq, d)
    wants = [plain_attention(q[i].double(), keys[s][:p + 1].double(), values[s][:p + 1].double(), scale, window)
             for i, (s, p) in enumerate(rows)]
    for i in range(m):
        torch.testing.assert_close(got[i], wants[i], **tol(dtype))
    if not k.mfma_attention_supported(hq, hkv, d, page):
        return
    # the matrix-core kernel: the first request's rows in groups of consecutive tokens, the others alone
    tq = max(1, 16 // (hq // hkv))
    first = list(range(0, lengths[0], tq)) + list(range(lengths[0], m))
    count = [min(tq, lengths[0] - r) for r in range(0, lengths[0], tq)] + [1] * (m - lengths[0])
    out2 = torch.full((m, hq * d), float("nan"), dtype=dtype, device="cuda")
    if partial is not None:
        partial.fill_(float("nan"))
    k.attention_mfma(q.view(m, hq * d).cuda(), k_pages.cuda(), v_pages.cuda(), table.cuda(), slots, pos, out2,
                     torch.tensor(first, dtype=torch.int32).cuda(), torch.tensor(count, dtype=torch.int32).cuda(),
                     len(first), hq, hkv, d, page, scale, window=window, split_keys=split_keys,
                     max_splits=max_splits, partial=partial)
    got = out2.double().cpu().view(m, hq, d)
    for i in range(m):
        torch.testing.assert_close(got[i], wants[i], **tol(dtype))
    if not k.prefill_attention_supported(hq, hkv, d, page):
        return
    # the kernel for prompt portions: the first request's rows in groups of up to 4 tq tokens; other rows untouched
    big = 4 * tq
    first = list(range(0, lengths[0], big))
    count = [min(big, lengths[0] - r) for r in first]
    out3 = torch.full((m, hq * d), float("nan"), dtype=dtype, device="cuda")
    k.attention_prefill(q.view(m, hq * d).cuda(), k_pages.cuda(), v_pages.cuda(), table.cuda(), slots, pos, out3,
                        torch.tensor(first, dtype=torch.int32).cuda(), torch.tensor(count, dtype=torch.int32).cuda(),
                        len(first), hq, hkv, d, page, scale, window=window)
    got = out3.double().cpu().view(m, hq, d)
    for i in range(lengths[0]):
        torch.testing.assert_close(got[i], wants[i], **tol(dtype))
    assert torch.isnan(out3[lengths[0]:].float()).all()
    if not k.tiles_attention_supported(hq, hkv, d, page):
        return
    # the 32x32-tile kernel for prompt portions, with both sizes of workgroup: groups of as many tokens as a
    # workgroup takes, and of fewer
    # (workgroups of 128 columns that take two groups each, and one: small batches would only meet the latter)
    for columns, big, split, pairing in ((128, k.tiles_group_tokens(hq, hkv, 128), 0, "pairs"), (128, 8 * tq, 0, "pairs"),
                                         (128, 8 * tq, 0, "single"),
                                         (64, k.tiles_group_tokens(hq, hkv, 64), 0, "auto"), (64, 3 * tq, 0, "auto"),
                                         (128, k.tiles_group_tokens(hq, hkv, 128), 64, "auto"), (64, 3 * tq, 128, "auto")):
        first = list(range(0, lengths[0], big))
        count = [min(big, lengths[0] - r) for r in first]
        out4 = torch.full((m, hq * d), float("nan"), dtype=dtype, device="cuda")
        splits, part = 1, None
        if split:
            splits = (max_len + split - 1) // split
            part = torch.full((k.attention_partial_numel(m, hq, d, splits),), float("nan"), device="cuda")
        k.attention_tiles(q.view(m, hq * d).cuda(), k_pages.cuda(), v_pages.cuda(), table.cuda(), slots, pos, out4,
                          torch.tensor(first, dtype=torch.int32).cuda(), torch.tensor(count, dtype=torch.int32).cuda(),
                          len(first), hq, hkv, d, page, scale, window=window, columns=columns,
                          split_keys=split, max_splits=splits, partial=part, pairing=pairing)
        got = out4.double().cpu().view(m, hq, d)
        for i in range(lengths[0]):
            torch.testing.assert_close(got[i], wants[i], **tol(dtype))
        assert torch.isnan(out4[lengths[0]:].float()).all()


@pytest.mark.parametrize("dtype", DTYPES)
def test_attention_finds_one_far_key(dtype):
    """One key among a thousand matches the query (scaled so that its score stands out): the
    output must be that key's value, wherever in the pages it lies."""
    k = kernels(dtype)
    hq = hkv = 1
    d, page, L = 64, 16, 1000
    g = torch.Generator().manual_seed(21)
    for far in [0, 15, 16, 63, 64, 511, 512, 998, 999]:
        kk = 0.05 * torch.randn((L, 1, d), generator=g)
        vv = torch.randn((L, 1, d), generator=g)
        q = torch.randn((1, d), generator=g)
        kk[far, 0] = 40 * q[0] / q[0].norm()
        n_blocks = (L + page - 1) // page
        table = torch.arange(n_blocks - 1, -1, -1, dtype=torch.int32)[None, :].contiguous()
        k_pages = torch.zeros((n_blocks, 1, page, d))
        v_pages = torch.zeros((n_blocks, 1, d, page))
        for b in range(n_blocks):
            n = min(page, L - b * page)
            k_pages[table[0, b], 0, :n] = kk[b * page:b * page + n, 0]
            v_pages[table[0, b], 0, :, :n] = vv[b * page:b * page + n, 0].T
        out = torch.empty((1, d), dtype=dtype, device="cuda")
        for split_keys in (0, 128):
            max_splits = (L + split_keys - 1) // split_keys if split_keys else 1
            partial = torch.empty(k.attention_partial_numel(1, 1, d, max_splits), device="cuda") if split_keys else None
            k.paged_attention(q.to(dtype).cuda(), k_pages.to(dtype).cuda(), v_pages.to(dtype).cuda(), table.cuda(),
                              torch.zeros(1, dtype=torch.int32).cuda(), torch.tensor([L - 1], dtype=torch.int32).cuda(),
                              out, 1, 1, d, page, 1.0, split_keys=split_keys, max_splits=max_splits, partial=partial)
            torch.testing.assert_close(out.float().cpu()[0], vv[far, 0].to(dtype).float(), atol=3e-2, rtol=3e-2)
            if k.mfma_attention_supported(1, 1, d, page):
                out.fill_(float("nan"))
                one = torch.ones(1, dtype=torch.int32).cuda()
                k.attention_mfma(q.to(dtype).cuda(), k_pages.to(dtype).cuda(), v_pages.to(dtype).cuda(), table.cuda(),
                                 torch.zeros(1, dtype=torch.int32).cuda(), torch.tensor([L - 1], dtype=torch.int32).cuda(),
                                 out, torch.zeros(1, dtype=torch.int32).cuda(), one, 1, 1, 1, d, page, 1.0,
                                 split_keys=split_keys, max_splits=max_splits, partial=partial)
                torch.testing.assert_close(out.float().cpu()[0], vv[far, 0].to(dtype).float(), atol=3e-2, rtol=3e-2)


@pytest.mark.parametrize("vocab", [1, 31, 32, 33, 257, 1024, 1025, 151936])
def test_sample_greedy(vocab):
    """Ties -> lowest id; a NaN or infinity -> -1 and the status names the row
    (tests/cuda_ops_tests.cu:408-435)."""
    k = kernels(torch.float32)
    g = torch.Generator().manual_seed(vocab)
    logits = torch.randn((4, vocab), generator=g)
    if vocab > 2:
        logits[1, vocab - 1] = 50.0
        logits[1, vocab // 2] = 50.0
        logits[2, 0] = 60.0
    if vocab > 40:
        logits[3, 37] = float("nan")
    temp = torch.zeros(4).cuda()
    u = torch.zeros(4).cuda()
    tokens = torch.full((4,), -7, dtype=torch.int32).cuda()
    status = torch.zeros(2, dtype=torch.int32).cuda()
    sample(k, logits.cuda(), temp, u, tokens, status)
    got = tokens.cpu().tolist()
    for r in range(4):
        row = logits[r]
        if not torch.isfinite(row).all():
            assert got[r] == -1
        else:
            assert got[r] == int(np.argmax(row.numpy()))
    if vocab > 40:
        assert status.cpu().tolist() == [1, 3]
    else:
        assert status.cpu().tolist() == [0, 2 ** 31 - 1]
    if vocab > 2:
        assert got[1] == vocab // 2 and got[2] == 0


@pytest.mark.parametrize("vocab", [5, 311, 4099, 151936, 1859, 2680, 2769, 146254, 236821])
def test_sample_temperature(vocab):
    """The drawn token's slice of the CDF of softmax(logits / T) (float64) holds u.  Row 1 draws u = 1 - 2^-23:
    in 32-bit its target is the total itself or a rounding below it, and the token must still come from the
    CDF's end (the last five sizes are ones at which the running sums, added in another order, end below it)."""
    from plain.qwen3_plain import temperature_cdf
    k = kernels(torch.float32)
    g = torch.Generator().manual_seed(vocab + 1)
    rows = 64
    logits = 3 * torch.randn((rows, vocab), generator=g)
    temp = torch.rand(rows, generator=g) * 1.5 + 0.2
    u = torch.rand(rows, generator=g)
    u[0], u[1] = 0.0, 0.9999999
    tokens = torch.empty(rows, dtype=torch.int32).cuda()
    status = torch.zeros(2, dtype=torch.int32).cuda()
    sample(k, logits.cuda(), temp.cuda(), u.cuda(), tokens, status)
    got = tokens.cpu().tolist()
    for r in range(rows):
        cdf = temperature_cdf(logits[r].numpy(), float(temp[r]))
        t = got[r]
        lo = cdf[t - 1] if t > 0 else 0.0
        assert lo - 1e-4 <= float(u[r]) <= cdf[t] + 1e-4, (r, t, lo, float(u[r]), cdf[t])


def test_sample_frequencies():
    """Empirical frequencies over many draws follow softmax(logits / T)."""
    k = kernels(torch.float32)
    logits = torch.tensor([0.0, 1.0, 2.0, -1.0, 0.5, 3.0, -2.0])
    temp_value = 0.8
    rows = 20000
    g = torch.Generator().manual_seed(5)
    u = torch.rand(rows, generator=g).cuda()
    tokens = torch.empty(rows, dtype=torch.int32).cuda()
    sample(k, logits[None, :].repeat(rows, 1).cuda().contiguous(), torch.full((rows,), temp_value).cuda(), u, tokens,
           torch.zeros(2, dtype=torch.int32).cuda())
    freq = torch.bincount(tokens.cpu().long(), minlength=7).double() / rows
    want = torch.softmax(logits.double() / temp_value, 0)
    assert (freq - want).abs().max() < 0.015


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("window", [1, 16, 17, 64, 100])
def test_attention_window_edge(dtype, window):
    """The key just outside the window matches the query strongly and must not be seen; then the key
    just inside does and must be seen."""
    k = kernels(dtype)
    d, page, L = 32, 16, 300
    g = torch.Generator().manual_seed(31)
    q = torch.randn((1, d), generator=g)
    for inside in (False, True):
        kk = 0.05 * torch.randn((L, d), generator=g)
        vv = torch.randn((L, d), generator=g)
        hot = L - window + (0 if inside else -1)
        kk[hot] = 40 * q[0] / q[0].norm()
        n_blocks = (L + page - 1) // page
        table = torch.arange(n_blocks, dtype=torch.int32)[None, :].contiguous()
        k_pages = torch.zeros((n_blocks, 1, page, d))
        k_pages.view(-1, d)[:L] = kk
        rows = torch.zeros((n_blocks * page, d))
        rows[:L] = vv
        v_pages = rows.view(n_blocks, 1, page, d).transpose(2, 3).contiguous()
        out = torch.empty((1, d), dtype=dtype, device="cuda")
        k.paged_attention(q.to(dtype).cuda(), k_pages.to(dtype).cuda(), v_pages.to(dtype).cuda(), table.cuda(),
                          torch.zeros(1, dtype=torch.int32).cuda(), torch.tensor([L - 1], dtype=torch.int32).cuda(),
                          out, 1, 1, d, page, 1.0, window=window)
        lo = L - window
        want = plain_attention(q.to(dtype).double(), kk[:, None, :].to(dtype).double(), vv[:, None, :].to(dtype).double(),
                               1.0, window)
        torch.testing.assert_close(out.double().cpu(), want, **tol(dtype))
        close_to_hot = (out.float().cpu()[0] - vv[hot].to(dtype).float()).abs().max() < 0.05
        assert bool(close_to_hot) == inside, (window, inside, lo)
        if k.mfma_attention_supported(1, 1, d, page):
            out.fill_(float("nan"))
            k.attention_mfma(q.to(dtype).cuda(), k_pages.to(dtype).cuda(), v_pages.to(dtype).cuda(), table.cuda(),
                             torch.zeros(1, dtype=torch.int32).cuda(), torch.tensor([L - 1], dtype=torch.int32).cuda(),
                             out, torch.zeros(1, dtype=torch.int32).cuda(), torch.ones(1, dtype=torch.int32).cuda(),
                             1, 1, 1, d, page, 1.0, window=window)
            torch.testing.assert_close(out.double().cpu(), want, **tol(dtype))
            assert bool((out.float().cpu()[0] - vv[hot].to(dtype).float()).abs().max() < 0.05) == inside


@pytest.mark.parametrize("mnk", [(1, 48, 64), (8, 3072, 1024), (17, 100, 76), (40, 208, 80), (64, 136, 264),
                                 (3, 56, 192), (16, 40, 4160), (13, 72, 2048)])
def test_gemm_gated_silu(mnk):
    """The feed-forward's activation fused into its first projection (few rows, bfloat16):
    silu(a Wgate^T) * (a Wup^T) with the sums kept in 32-bit until the product."""
    from mini_llm_runtime_amd.kernels import Kernels
    m, n, kk = mnk
    k = Kernels(torch.bfloat16, library_gemm=False)
    assert k.gated_silu_fused(m) and not k.gated_silu_fused(65)
    assert kernels(torch.bfloat16).gated_silu_fused(16) and not kernels(torch.bfloat16).gated_silu_fused(17)
    # with the library at hand, more rows stay here only while the inner size is small
    assert kernels(torch.bfloat16).gated_silu_fused(64, 1024) and not kernels(torch.bfloat16).gated_silu_fused(33, 2048)
    a = rnd((m, kk), torch.bfloat16, 50)
    w = rnd((2 * n, kk), torch.bfloat16, 51, 0.3)
    out = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device="cuda")
    k.gemm_gated_silu(a, w, out)
    g = a.double() @ w.double()[:n].T
    u = a.double() @ w.double()[n:].T
    want = g / (1 + torch.exp(-g)) * u
    torch.testing.assert_close(out.double(), want, atol=2e-2 * float(want.abs().max()), rtol=2e-2)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("shape", [(4, 2, 128, 16), (6, 3, 48, 32), (16, 8, 64, 16), (3, 1, 16, 16), (2, 2, 256, 64)])
@pytest.mark.parametrize("layout", [([90, 10], [37, 0]), ([96, 16], [32, 8]), ([64, 3, 40], [0, 5, 16])])
def test_qk_norm_rope_kv_many_rows(dtype, shape, layout):
    """Whole prompt portions (the many-row variants of the kernels): consecutive positions of a few requests,
    starting inside a page, at a page's edge and at multiples of eight."""
    hq, hkv, d, page = shape
    k = kernels(dtype)
    counts, starts = layout
    m = sum(counts)
    n_req = len(counts)
    positions = torch.tensor([starts[s] + i for s in range(n_req) for i in range(counts[s])], dtype=torch.int32)
    slots = torch.tensor([s for s in range(n_req) for _ in range(counts[s])], dtype=torch.int32)
    max_blocks = 16
    n_pages = n_req * max_blocks
    perm = torch.randperm(n_pages, generator=torch.Generator().manual_seed(3)).to(torch.int32)
    table = perm.view(n_req, max_blocks).contiguous()
    qkv = rnd((m, (hq + 2 * hkv) * d), dtype, 60)
    qw, kw = rnd((d,), torch.float32, 61) + 1, rnd((d,), torch.float32, 62) + 1
    eps, base = 1e-6, 10000.0
    rope = rope_table(256, d, base)
    k_pages = torch.full((n_pages, hkv, page, d), float("nan"), dtype=dtype, device="cuda")
    v_pages = torch.full((n_pages, hkv, d, page), float("nan"), dtype=dtype, device="cuda")
    q_out = torch.empty((m, hq * d), dtype=dtype, device="cuda")
    k.qk_norm_rope_kv(qkv, q_out, k_pages, v_pages, table.cuda(), slots.cuda(), positions.cuda(), qw, kw, eps, rope,
                      hq, hkv, d, page)
    x = qkv.double().cpu()
    q = x[:, :hq * d].view(m, hq, d)
    kk = x[:, hq * d:(hq + hkv) * d].view(m, hkv, d)

    def norm(t, w):
        return t * torch.rsqrt((t * t).mean(-1, keepdim=True) + eps) * w.double().cpu()
    q_want = plain_rope(norm(q, qw), positions, base)
    k_want = plain_rope(norm(kk, kw), positions, base)
    torch.testing.assert_close(q_out.double().cpu().view(m, hq, d), q_want, **tol(dtype))
    kp, vp = k_pages.cpu(), v_pages.cpu()
    for i in range(m):
        p, s = int(positions[i]), int(slots[i])
        pg = int(table[s, p // page])
        torch.testing.assert_close(kp[pg, :, p % page].double(), k_want[i], **tol(dtype))
        assert torch.equal(vp[pg, :, :, p % page], qkv[i, (hq + hkv) * d:].view(hkv, d).cpu())
    written = sum(counts) * hkv * d
    assert int((~torch.isnan(kp.float())).sum()) == written and int((~torch.isnan(vp.float())).sum()) == written


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("width", [8, 72, 1024, 2048, 2056, 76])
def test_add_rmsnorm_many_rows(dtype, width):
    k = kernels(dtype)
    rows = 130
    h0 = rnd((rows, width), torch.float32, 70, 2.0)
    delta = rnd((rows, width), dtype, 71)
    w = rnd((width,), torch.float32, 72)
    x = h0.double() + delta.double()
    want = x * torch.rsqrt((x * x).mean(-1, keepdim=True) + 1e-6) * w.double()
    h = h0.clone()
    out = torch.empty((rows, width), dtype=dtype, device="cuda")
    k.add_rmsnorm(h, delta, w, out, 1e-6)
    torch.testing.assert_close(h.double(), x, atol=1e-6, rtol=1e-6)
    torch.testing.assert_close(out.double(), want, **tol(dtype))
    idx = torch.arange(rows - 1, -1, -1, dtype=torch.int32).cuda()[:100].contiguous()
    h = h0.clone()
    out = torch.empty((100, width), dtype=dtype, device="cuda")
    k.add_rmsnorm(h, delta, w, out, 1e-6, rows=idx, write_h=False)
    assert torch.equal(h, h0)
    torch.testing.assert_close(out.double(), want[idx.long()], **tol(dtype))
    out = torch.empty((rows, width), dtype=dtype, device="cuda")
    k.add_rmsnorm(h, None, w, out, 1e-6)
    x = h0.double()
    torch.testing.assert_close(out.double(), x * torch.rsqrt((x * x).mean(-1, keepdim=True) + 1e-6) * w.double(), **tol(dtype))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("inter", [8, 104, 3072])
def test_silu_mul_wide(dtype, inter):
    k = kernels(dtype)
    gate_up = rnd((70, 2 * inter), dtype, 80, 3.0)
    act = torch.empty((70, inter), dtype=dtype, device="cuda")
    k.silu_mul(gate_up, act)
    g, u = gate_up.double()[:, :inter], gate_up.double()[:, inter:]
    torch.testing.assert_close(act.double(), g / (1 + torch.exp(-g)) * u, **tol(dtype))


@pytest.mark.parametrize("rows,width", [(1, 64), (8, 1024), (16, 100), (5, 97), (3, 4096)])
def test_rows_prenorm(rows, width):
    """The first half of a norm that is handed to the projection after it: h += delta, out = bf16(h * w) without
    the scale, and the rows' sums of squares."""
    k = kernels(torch.bfloat16)
    h0 = rnd((rows, width), torch.float32, 94, 2.0)
    delta = rnd((rows, width), torch.bfloat16, 95)
    nw = rnd((width,), torch.float32, 96) + 1
    for d in (delta, None):
        h = h0.clone()
        out = torch.full((rows, width), float("nan"), dtype=torch.bfloat16, device="cuda")
        ss = torch.full((rows, 1), float("nan"), device="cuda")
        k.rows_prenorm(h, d, nw, out, ss)
        x = h0.double() + (d.double() if d is not None else 0)
        torch.testing.assert_close(h.double(), x, atol=1e-6, rtol=1e-6)
        torch.testing.assert_close(out.double(), (x * nw.double()).to(torch.bfloat16).double(), atol=0, rtol=2 ** -7)
        torch.testing.assert_close(ss[:, 0].double(), (x * x).sum(-1), rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("gated", [False, True])
@pytest.mark.parametrize("mnk,parts", [((1, 48, 64), 1), ((8, 4096, 1024), 64), ((16, 100, 1024), 3), ((5, 208, 96), 6),
                                       ((3, 40, 4096), 256), ((7, 24, 32), 2), ((2, 50, 100), 7), ((16, 333, 2048), 128),
                                       ((4, 48, 8320), 520), ((6, 32, 2096), 131), ((9, 64, 5120), 320)])
def test_projection_after_a_handed_over_norm(mnk, parts, gated):
    """`gemm_prenormed`: the rows' scale rsqrt(sum of the partial sums / K + eps), applied to the finished sums
    of x . w^T (or inside the gated activation), equals the projection of the normed rows.  The partial sums are
    read four a load where their number is a multiple of four and they start at a multiple of 16 bytes, else
    one a load, in rounds of four loads (520 and 131 parts: more than one round)."""
    m, n, kk = mnk
    k = kernels(torch.bfloat16)
    assert k.handoff_supported(m) and not k.handoff_supported(17) and not kernels(torch.float32).handoff_supported(m)
    xf = rnd((m, kk), torch.float32, 90, 2.0)
    nw = rnd((kk,), torch.float32, 92) + 1
    x = (xf * nw).to(torch.bfloat16)
    # the rows' sums of squares, cut into parts of any sizes (some of them zero)
    cuts = torch.linspace(0, kk, parts + 1).long().tolist()
    ss = torch.stack([(xf[:, a:b].double() ** 2).sum(-1) for a, b in zip(cuts, cuts[1:])], dim=1).float().contiguous()
    w = rnd(((2 if gated else 1) * n, kk), torch.bfloat16, 93, 0.2)
    eps = 1e-5
    out = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device="cuda")
    k.gemm_prenormed(x, ss, eps, w, out, gated=gated)
    scale = torch.rsqrt((xf.double() ** 2).mean(-1, keepdim=True) + eps)
    if gated:
        g, u = scale * (x.double() @ w.double()[:n].T), scale * (x.double() @ w.double()[n:].T)
        want = g / (1 + torch.exp(-g)) * u
    else:
        want = scale * (x.double() @ w.double().T)
    torch.testing.assert_close(out.double(), want, atol=1e-2 * float(want.abs().max()), rtol=1e-2)
    # a row's result does not depend on the rows beside it
    if m > 1:
        one = torch.full((1, n), float("nan"), dtype=torch.bfloat16, device="cuda")
        k.gemm_prenormed(x[m - 1:].contiguous(), ss[m - 1:].contiguous(), eps, w, one, gated=gated)
        assert torch.equal(one[0], out[m - 1])
    # the same sums at an address that is no multiple of 16 bytes (read one a load)
    shifted = torch.empty(m * parts + 1, dtype=torch.float32, device="cuda")[1:].view(m, parts)
    shifted.copy_(ss)
    assert shifted.data_ptr() % 16 == 4
    again = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device="cuda")
    k.gemm_prenormed(x, shifted, eps, w, again, gated=gated)
    torch.testing.assert_close(again.double(), want, atol=1e-2 * float(want.abs().max()), rtol=1e-2)


@pytest.mark.parametrize("mnk", [(1, 64, 48), (8, 1024, 2048), (16, 1024, 3072), (5, 96, 208), (3, 4096, 4096), (7, 50, 96),
                                 (2, 97, 100), (16, 40, 64), (9, 4096, 12288), (8, 5120, 2048), (3, 4100, 2048),
                                 (16, 5120, 8192)])
def test_projection_that_adds_into_the_residual_stream(mnk):
    """`gemm_residual`: h += a . w^T in 32-bit; with a norm to follow also bf16(h * next_w) and partial sums of
    squares of the new h: per row and strip of 16 columns or, where a workgroup owns two strips side by side
    (the last three shapes), per row and workgroup, the parts beyond the workgroups zero."""
    m, n, kk = mnk
    k = kernels(torch.bfloat16)
    a = rnd((m, kk), torch.bfloat16, 97)
    w = rnd((n, kk), torch.bfloat16, 98, 0.2)
    h0 = rnd((m, n), torch.float32, 99, 2.0)
    nw = rnd((n,), torch.float32, 100) + 1
    want_h = h0.double() + a.double() @ w.double().T
    tol_h = dict(atol=2e-5 * float(want_h.abs().max()) * max(1, kk // 512), rtol=1e-5)
    h = h0.clone()
    k.gemm_residual(a, w, h)
    torch.testing.assert_close(h.double(), want_h, **tol_h)
    h2 = h0.clone()
    parts = k.handoff_parts(n)
    x = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device="cuda")
    ss = torch.full((m, parts), float("nan"), device="cuda")
    k.gemm_residual(a, w, h2, nw, x, ss)
    assert torch.equal(h2, h)
    torch.testing.assert_close(x.double(), (h.double() * nw.double()).to(torch.bfloat16).double(), atol=0, rtol=2 ** -7)
    padded = torch.zeros((m, parts * 16), dtype=torch.float64, device="cuda")
    padded[:, :n] = h.double() ** 2
    if n in (5120, 4100):
        used = int((ss != 0).any(dim=0).sum())              # a part a workgroup: fewer than strips of 16, a prefix
        assert bool(torch.isfinite(ss).all()) and parts // 2 <= used < parts and bool((ss[:, used:] == 0).all())
        torch.testing.assert_close(ss.double().sum(-1), padded.sum(-1), rtol=1e-5, atol=1e-6)
    else:
        torch.testing.assert_close(ss.double(), padded.view(m, parts, 16).sum(-1), rtol=1e-5, atol=1e-6)
    # the two halves together are the norm: the next projection on (x, ss) gives rmsnorm(h) . w2^T
    w2 = rnd((64, n), torch.bfloat16, 101, 0.2)
    out = torch.full((m, 64), float("nan"), dtype=torch.bfloat16, device="cuda")
    k.gemm_prenormed(x, ss, 1e-6, w2, out)
    hn = h.double() * torch.rsqrt((h.double() ** 2).mean(-1, keepdim=True) + 1e-6) * nw.double()
    want = hn @ w2.double().T
    torch.testing.assert_close(out.double(), want, atol=2e-2 * float(want.abs().max()), rtol=2e-2)


def test_prompt_portion_beyond_the_page_cache_of_a_workgroup():
    """A portion of 70 tokens at the end of a context of 33 000 keys: more pages than a workgroup of the
    32x32-tile kernel keeps, so the keys must be split; unsplit the call is refused."""
    from mini_llm_runtime_amd.kernels.ops import KernelError
    dtype = torch.bfloat16
    k = kernels(dtype)
    hq, hkv, d, page, L, n = 2, 1, 64, 16, 33000, 70
    g = torch.Generator().manual_seed(77)
    kk = torch.randn((L, hkv, d), generator=g).to(dtype)
    vv = torch.randn((L, hkv, d), generator=g).to(dtype)
    blocks = (L + page - 1) // page
    perm = torch.randperm(blocks, generator=g)
    table = perm.to(torch.int32)[None, :].contiguous()
    k_pages = torch.zeros((blocks, hkv, page, d), dtype=dtype)
    v_pages = torch.zeros((blocks, hkv, d, page), dtype=dtype)
    pad = blocks * page - L
    kp = torch.cat([kk, torch.zeros((pad, hkv, d), dtype=dtype)]).view(blocks, page, hkv, d)
    vp = torch.cat([vv, torch.zeros((pad, hkv, d), dtype=dtype)]).view(blocks, page, hkv, d)
    k_pages[perm] = kp.permute(0, 2, 1, 3)
    v_pages[perm] = vp.permute(0, 2, 3, 1)
    q = (torch.randn((n, hq, d), generator=g) * 2).to(dtype)
    pos = torch.arange(L - n, L, dtype=torch.int32).cuda()
    slots = torch.zeros(n, dtype=torch.int32).cuda()
    first = torch.tensor([0, 64], dtype=torch.int32).cuda()
    count = torch.tensor([64, 6], dtype=torch.int32).cuda()
    out = torch.full((n, hq * d), float("nan"), dtype=dtype, device="cuda")
    args = (q.view(n, hq * d).cuda(), k_pages.cuda(), v_pages.cuda(), table.cuda(), slots, pos, out, first, count, 2,
            hq, hkv, d, page, 1 / math.sqrt(d))
    with pytest.raises(KernelError):
        k.attention_tiles(*args, max_context=L)
    split = 16384
    splits = (L + split - 1) // split
    part = torch.full((k.attention_partial_numel(n, hq, d, splits),), float("nan"), device="cuda")
    k.attention_tiles(*args, max_context=L, split_keys=split, max_splits=splits, partial=part)
    got = out.double().cpu().view(n, hq, d)
    for i in (0, 1, 31, 63, 64, 69):
        want = plain_attention(q[i].double(), kk[:L - n + i + 1].double(), vv[:L - n + i + 1].double(), 1 / math.sqrt(d), None)
        torch.testing.assert_close(got[i], want, **tol(dtype))


@pytest.mark.parametrize("case", [
    # (q heads, kv heads, head_dim, page, context lengths of the requests, window, split_keys, norm, rotation)
    (16, 8, 128, 16, [1, 2, 17, 300, 4096], None, 512, True, True),
    (4, 4, 64, 16, [1, 33, 64, 65, 130], None, 0, True, True),
    (8, 2, 64, 32, [5, 100, 257], 40, 64, True, True),
    (6, 1, 192, 16, [1, 70], None, 0, False, True),
    (2, 1, 256, 16, [129, 1], 1, 64, True, False),
    (32, 8, 128, 64, [513, 512, 511], 512, 256, True, True),
    # (heads above 128 channels, where a lane holds two rotation pairs: cases in which the two ways once differed
    # in a key's last bit, the compiler having fused the products and sums of the two kernels differently)
    (10, 5, 256, 32, [2078, 867, 853, 202], 441, 0, True, True),
    (15, 3, 192, 128, [1, 246, 75, 83, 345, 236, 609], None, 64, True, True),
    (64, 8, 256, 16, [2270, 123, 1915, 575, 687], None, 0, False, True),
])
def test_decode_attention_that_norms_rotates_and_caches_itself(case):
    """Every request brings one new token.  The fused pair of launches against the separate ones (per-head
    norm + rotation + cache write, then attention): the same output within bfloat16 rounding, the same key and
    value in the cache bit for bit, nothing else in the cache touched; and against the plain attention."""
    hq, hkv, d, page, lengths, window, split_keys, with_norm, with_rope = case
    dtype = torch.bfloat16
    k = kernels(dtype)
    gen = torch.Generator().manual_seed(41)
    n = len(lengths)
    max_len = max(lengths)
    max_blocks = (max_len + page - 1) // page
    n_pages = sum((L + page - 1) // page for L in lengths) + 3
    perm = torch.randperm(n_pages, generator=gen).tolist()
    table = torch.full((n, max_blocks), -1, dtype=torch.int32)
    k_pages = torch.full((n_pages, hkv, page, d), float("nan"), dtype=dtype)
    v_pages = torch.full((n_pages, hkv, d, page), float("nan"), dtype=dtype)
    keys, values = [], []
    for s, L in enumerate(lengths):
        kk = torch.randn((L - 1, hkv, d), generator=gen).to(dtype)
        vv = torch.randn((L - 1, hkv, d), generator=gen).to(dtype)
        keys.append(kk)
        values.append(vv)
        for b in range((L + page - 1) // page):
            pg = perm.pop()
            table[s, b] = pg
            cnt = max(0, min(page, L - 1 - b * page))
            if cnt:
                k_pages[pg, :, :cnt] = kk[b * page:b * page + cnt].transpose(0, 1)
                v_pages[pg, :, :, :cnt] = vv[b * page:b * page + cnt].permute(1, 2, 0)
    qkv = (torch.randn((n, (hq + 2 * hkv) * d), generator=gen) * 1.5).to(dtype).cuda()
    qw = (1 + 0.2 * torch.randn(d, generator=gen)).cuda() if with_norm else None
    kw = (1 + 0.2 * torch.randn(d, generator=gen)).cuda() if with_norm else None
    eps, base, scale = 1e-5, 10000.0, 1 / math.sqrt(d)
    rope = rope_table(max_len, d, base).cuda() if with_rope else None
    slots = torch.arange(n, dtype=torch.int32).cuda()
    pos = torch.tensor([L - 1 for L in lengths], dtype=torch.int32).cuda()
    first = torch.arange(n, dtype=torch.int32).cuda()
    ones = torch.ones(n, dtype=torch.int32).cuda()
    max_splits = (max_len + split_keys - 1) // split_keys if split_keys else 1
    partial = torch.full((k.attention_partial_numel(n, hq, d, max_splits),), float("nan"), device="cuda")
    # the separate launches
    k1, v1 = k_pages.clone().cuda(), v_pages.clone().cuda()
    q1 = torch.empty((n, hq * d), dtype=dtype, device="cuda")
    k.qk_norm_rope_kv(qkv, q1, k1, v1, table.cuda(), slots, pos, qw, kw, eps, rope, hq, hkv, d, page)
    out1 = torch.full((n, hq * d), float("nan"), dtype=dtype, device="cuda")
    k.attention_mfma(q1, k1, v1, table.cuda(), slots, pos, out1, first, ones, n, hq, hkv, d, page, scale, window=window,
                     split_keys=split_keys, max_splits=max_splits, partial=partial if max_splits > 1 else None)
    # the fused ones
    k2, v2 = k_pages.clone().cuda(), v_pages.clone().cuda()
    out2 = torch.full((n, hq * d), float("nan"), dtype=dtype, device="cuda")
    partial.fill_(float("nan"))
    k.attention_decode_fused(qkv, k2, v2, table.cuda(), slots, pos, out2, first, ones, n, hq, hkv, d, page, scale,
                             qw, kw, eps, rope, partial, window=window, split_keys=split_keys, max_splits=max_splits)
    same = lambda x, y: torch.equal(x.view(torch.int16), y.view(torch.int16))     # NaN-filled entries compare too
    assert same(k1, k2) and same(v1, v2)
    torch.testing.assert_close(out2.float(), out1.float(), atol=2e-2, rtol=2e-2)
    # and the plain attention over the cached keys plus the new one, as the separate launches cached it
    for s, L in enumerate(lengths):
        pg, at = table[s, (L - 1) // page].item(), (L - 1) % page
        kk = torch.cat([keys[s], k1[pg, :, at].cpu()[None]]).double()
        vv = torch.cat([values[s], v1[pg, :, :, at].cpu()[None]]).double()
        want = plain_attention(q1[s].double().cpu().view(hq, d), kk, vv, scale, window)
        torch.testing.assert_close(out2[s].double().cpu().view(hq, d), want, **tol(dtype))


@pytest.mark.parametrize("d", [64, 128])
def test_decoding_beyond_the_page_cache_of_a_workgroup(d):
    """One new token behind 66 000 keys in pages of 16 (4125 pages: more than the 4096 ids that a workgroup of
    the single-token kernels keeps), beside a short request: unsplit the calls are refused; with the key ranges
    that the engine forces on such a context both kernels (queries prepared, and the one that norms, rotates and
    caches inside itself) give the plain attention and the same cache.  Random keys would hide a range that is
    skipped among thousands: a key near the start, the last key of the first range, the first of the last range
    and the last cached key are made to stand out, each with a value of its own."""
    from mini_llm_runtime_amd.kernels.ops import KernelError, Kernels
    dtype = torch.bfloat16
    k = kernels(dtype)
    hq, hkv, page = 2, 1, 16
    lengths = [66000, 40]
    assert lengths[0] > Kernels.mfma_longest_context(page)
    gen = torch.Generator().manual_seed(5)
    n, max_len = len(lengths), max(lengths)
    max_blocks = (max_len + page - 1) // page
    n_pages = sum((L + page - 1) // page for L in lengths) + 3
    perm = torch.randperm(n_pages, generator=gen).tolist()
    table = torch.full((n, max_blocks), -1, dtype=torch.int32)
    k_pages = torch.full((n_pages, hkv, page, d), float("nan"), dtype=dtype)
    v_pages = torch.full((n_pages, hkv, d, page), float("nan"), dtype=dtype)
    qkv = (torch.randn((n, (hq + 2 * hkv) * d), generator=gen) * 1.5).to(dtype)
    split_keys = 32768
    marked = [5, split_keys - 1, 2 * split_keys, lengths[0] - 2]
    keys, values = [], []
    for s, L in enumerate(lengths):
        kk = torch.randn((L - 1, hkv, d), generator=gen).to(dtype)
        vv = torch.randn((L - 1, hkv, d), generator=gen).to(dtype)
        if s == 0:
            for j, at in enumerate(marked):            # along the first head's query: a score far above the others'
                kk[at, 0] = (qkv[0, :d].float() * (1.2 + 0.01 * j)).to(dtype)
                vv[at, 0] = 0
                vv[at, 0, j] = 8.0
        keys.append(kk)
        values.append(vv)
        flat_k = torch.cat([kk, torch.full((1, hkv, d), float("nan"), dtype=dtype)])       # (the new token's place)
        flat_v = torch.cat([vv, torch.full((1, hkv, d), float("nan"), dtype=dtype)])
        for b in range((L + page - 1) // page):
            pg = perm.pop()
            table[s, b] = pg
            cnt = min(page, L - b * page)
            k_pages[pg, :, :cnt] = flat_k[b * page:b * page + cnt].transpose(0, 1)
            v_pages[pg, :, :, :cnt] = flat_v[b * page:b * page + cnt].permute(1, 2, 0)
    qkv = qkv.cuda()
    scale = 1 / math.sqrt(d)
    slots = torch.arange(n, dtype=torch.int32).cuda()
    pos = torch.tensor([L - 1 for L in lengths], dtype=torch.int32).cuda()
    first = torch.arange(n, dtype=torch.int32).cuda()
    ones = torch.ones(n, dtype=torch.int32).cuda()
    max_splits = (max_len + split_keys - 1) // split_keys
    partial = torch.full((k.attention_partial_numel(n, hq, d, max_splits),), float("nan"), device="cuda")
    # no norm and no rotation: what is cached is the raw key, so the plain result below needs no second path
    k1, v1 = k_pages.clone().cuda(), v_pages.clone().cuda()
    q1 = torch.empty((n, hq * d), dtype=dtype, device="cuda")
    k.qk_norm_rope_kv(qkv, q1, k1, v1, table.cuda(), slots, pos, None, None, 0.0, None, hq, hkv, d, page)
    out1 = torch.full((n, hq * d), float("nan"), dtype=dtype, device="cuda")
    with pytest.raises(KernelError, match="4096 pages"):
        k.attention_mfma(q1, k1, v1, table.cuda(), slots, pos, out1, first, ones, n, hq, hkv, d, page, scale)
    k.attention_mfma(q1, k1, v1, table.cuda(), slots, pos, out1, first, ones, n, hq, hkv, d, page, scale,
                     split_keys=split_keys, max_splits=max_splits, partial=partial)
    k2, v2 = k_pages.clone().cuda(), v_pages.clone().cuda()
    out2 = torch.full((n, hq * d), float("nan"), dtype=dtype, device="cuda")
    with pytest.raises(KernelError, match="4096 pages"):
        k.attention_decode_fused(qkv, k2, v2, table.cuda(), slots, pos, out2, first, ones, n, hq, hkv, d, page, scale,
                                 None, None, 0.0, None, partial)
    partial.fill_(float("nan"))
    k.attention_decode_fused(qkv, k2, v2, table.cuda(), slots, pos, out2, first, ones, n, hq, hkv, d, page, scale,
                             None, None, 0.0, None, partial, split_keys=split_keys, max_splits=max_splits)
    same = lambda x, y: torch.equal(x.view(torch.int16), y.view(torch.int16))
    assert same(k1, k2) and same(v1, v2)
    own_k = qkv[:, hq * d:(hq + hkv) * d].cpu().view(n, 1, hkv, d)
    own_v = qkv[:, (hq + hkv) * d:].cpu().view(n, 1, hkv, d)
    for s, L in enumerate(lengths):
        kk = torch.cat([keys[s], own_k[s]]).double()
        vv = torch.cat([values[s], own_v[s]]).double()
        want = plain_attention(qkv[s, :hq * d].double().cpu().view(hq, d), kk, vv, scale, None)
        if s == 0:                                   # each marked key carries a visible share of the first head's result
            assert all(float(want[0, j]) > 0.5 for j in range(len(marked))), want[0, :len(marked)]
        for out in (out1, out2):
            torch.testing.assert_close(out[s].double().cpu().view(hq, d), want, **tol(dtype))


def test_bfloat16_widening_and_rounding():
    """Every one of the 65536 bfloat16 patterns widens to the float of the same value (the embedding gather
    is the kernel that does nothing else), and a 32-bit sum that lies exactly between two bfloat16 values
    is rounded to the even one (the projections' epilogue), below and above one, in both signs -- the
    reference checks its 16-bit conversions the same way (tests/core_tests.cpp:244-254,
    tests/cuda_ops_tests.cu:75-101)."""
    from mini_llm_runtime_amd.kernels import Kernels
    k = kernels(torch.bfloat16)
    patterns = torch.arange(65536, dtype=torch.int32).to(torch.int16).view(torch.bfloat16).view(512, 128).cuda()
    ids = torch.arange(512, dtype=torch.int32, device="cuda")
    h = torch.empty((512, 128), dtype=torch.float32, device="cuda")
    k.embed_gather(ids, patterns, h)
    want = patterns.float()
    assert torch.equal(h.view(torch.int32), want.view(torch.int32))          # bit for bit, NaN payloads too
    # sums a0 * 1 + a1 * 1 with a0 a bfloat16 value and a1 half a unit in its last place
    cases = []
    for exponent in (-20, -1, 0, 1, 7, 30):
        for mantissa in (0, 1, 2, 126, 127):
            base = (1.0 + mantissa / 128.0) * 2.0 ** exponent
            half_ulp = 2.0 ** (exponent - 8)
            even = base if mantissa % 2 == 0 else base + 2 * half_ulp
            for sign in (1.0, -1.0):
                cases.append((sign * base, sign * half_ulp, sign * even))
    a = torch.tensor([[c[0], c[1]] for c in cases], dtype=torch.float32)
    assert torch.equal(a.to(torch.bfloat16).float(), a)                      # the summands are exact in bfloat16
    w = torch.ones((8, 2), dtype=torch.bfloat16, device="cuda")
    want = torch.tensor([c[2] for c in cases], dtype=torch.float32)
    for engine in (k, Kernels(torch.bfloat16, library_gemm=False)):
        for rows in (len(cases), 16, 5):                                     # many rows (the library, or tiles) and few
            out = torch.empty((rows, 8), dtype=torch.bfloat16, device="cuda")
            engine.gemm(a[:rows].to(torch.bfloat16).cuda(), w, out)
            assert torch.equal(out.float().cpu(), want[:rows, None].expand(rows, 8)), rows


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("rows", [3, 96])
def test_a_position_beyond_the_block_table_has_no_page(dtype, rows):
    """The engine never asks for it (the cache manager bounds a request's length by its row of the table); a
    caller of the kernels that does gets what a missing page gives: the query is normed and rotated, nothing
    is cached, and no kernel reads past the table's row.  Few rows (the general kernel) and many (the vector
    kernel and its transposing value writer)."""
    hq, hkv, d, page, max_blocks = 4, 2, 64, 16, 2
    k = kernels(dtype)
    inside = max_blocks * page                                         # 32 positions have a page
    positions = torch.tensor([30 + 3 * (i // 2) for i in range(rows)], dtype=torch.int32)      # 30, 30, 33, 33, ...
    slots = torch.tensor([i % 2 for i in range(rows)], dtype=torch.int32)
    seen = {(int(slots[i]), int(positions[i])): i for i in range(rows)}         # (every position of a slot once)
    assert len(seen) == rows
    table = torch.tensor([[3, 0], [1, 2]], dtype=torch.int32)
    qkv = rnd((rows, (hq + 2 * hkv) * d), dtype, 70)
    qw, kw = rnd((d,), torch.float32, 71) + 1, rnd((d,), torch.float32, 72) + 1
    rope = rope_table(256, d, 10000.0)
    k_pages = torch.full((4, hkv, page, d), float("nan"), dtype=dtype, device="cuda")
    v_pages = torch.full((4, hkv, d, page), float("nan"), dtype=dtype, device="cuda")
    q_out = torch.full((rows, hq * d), float("nan"), dtype=dtype, device="cuda")
    k.qk_norm_rope_kv(qkv, q_out, k_pages, v_pages, table.cuda(), slots.cuda(), positions.cuda(), qw, kw, 1e-6, rope,
                      hq, hkv, d, page)
    assert bool(torch.isfinite(q_out.float()).all())
    cached = sum(1 for (s, p) in seen if p < inside)
    kp, vp = k_pages.cpu().float(), v_pages.cpu().float()
    assert int((~torch.isnan(kp)).sum()) == cached * hkv * d and int((~torch.isnan(vp)).sum()) == cached * hkv * d
    for (s, p), i in seen.items():
        if p < inside:
            assert torch.equal(v_pages[int(table[s, p // page]), :, :, p % page].cpu(),
                               qkv[i, (hq + hkv) * d:].view(hkv, d).cpu())
