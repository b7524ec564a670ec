"""Python side of the HIP kernels: one `Kernels` object per element type.

Every method checks on the host that its operands lie on the GPU, are contiguous, have the
element type and the shapes that the kernel and its grid assume, and only then launches on
torch's current stream.  A kernel that cannot take a size refuses it here with a clear error.
There is no other implementation behind these methods: without the compiled extension, or
without a GPU, they raise.
"""
from __future__ import annotations

import ctypes

import torch

from . import build
from .profile import timed

_c_int = ctypes.c_int
_c_float = ctypes.c_float
_c_size_t = ctypes.c_size_t
_ptr = ctypes.c_void_p

MAX_HEAD_DIM = 256          # the attention and rotation kernels keep head_dim / 64 values per lane
ATTENTION_TILE_KEYS = 64
LIBRARY_GEMM_MIN_ROWS = 16    # above this many rows the bfloat16 engine's projections go to the library
LIBRARY_GEMM_WORKSPACE = 128 << 20   # bytes of scratch memory that the library may use
PREFILL_MAX_PAGES = 2048      # page ids of one group that the prompt-portion attention kernel keeps in LDS
TILES_MAX_HEAD_DIM = 128      # the 32x32-tile kernel for prompt portions keeps two sets of accumulators per lane
TILES_COLUMNS = (128, 64)     # (token, head) columns of one of its workgroups: the usual and the small one
TILES_PAIRING = {"auto": 0, "single": 1, "pairs": 2}
MFMA_MAX_PAGES = 4096         # page ids of one key range that the single-token attention kernel keeps in LDS
MAX_KEY_SPLITS = 1024         # the merge of key splits keeps one weight per split in LDS


class KernelError(RuntimeError):
    pass


def _p(t):
    return _ptr(t.data_ptr()) if t is not None else _ptr(0)


try:
    _raw_stream = torch._C._cuda_getCurrentRawStream          # the current stream's handle without a Stream object
except AttributeError:                                         # pragma: no cover
    _raw_stream = None


_device_index = getattr(torch._C, "_cuda_getDevice", None)    # (the current device's index without torch.cuda's wrapper)


def _stream():
    """Handle of torch's current stream on the current device."""
    if _raw_stream is not None:
        return _ptr(_raw_stream(_device_index() if _device_index is not None else torch.cuda.current_device()))
    return _ptr(torch.cuda.current_stream().cuda_stream)


def _need(cond, message):
    """`message` is a string or, where building it costs time, a function that returns one."""
    if not cond:
        raise KernelError(message() if callable(message) else message)


def _tensor(t, name, dtype, shape=None, ndim=None):
    # one cheap test on the way that every launch takes; the message is only put together on failure
    try:
        if (t.is_cuda and t.dtype is dtype and t.is_contiguous() and (ndim is None or t.dim() == ndim)
                and (shape is None or t.shape == shape or t.shape == tuple(shape))):
            return t
    except AttributeError:                                # (no tensor: said below)
        pass
    _need(isinstance(t, torch.Tensor), f"{name}: expected a tensor")
    _need(t.is_cuda, f"{name}: must lie on the GPU (there is no CPU path)")
    _need(t.dtype == dtype, f"{name}: expected {dtype}, got {t.dtype}")
    _need(t.is_contiguous(), f"{name}: must be contiguous")
    _need(ndim is None or t.dim() == ndim, f"{name}: expected {ndim} dimensions, got {tuple(t.shape)}")
    raise KernelError(f"{name}: expected shape {tuple(shape)}, got {tuple(t.shape)}")


def _ok(code, what):
    if code != 0:
        raise KernelError(f"{what}: launch failed with code {code}")


def _size(t):
    return 0 if t is None else t.numel() * t.element_size()


def _gemm_work(self, a, w, out, *rest, **kw):
    return _size(a) + _size(w) + _size(out), 2 * a.shape[0] * w.shape[0] * w.shape[1]


def _rows_prenorm_work(self, h, delta, weight, out, ss):
    return 2 * _size(h) + _size(delta) + _size(out), 0


def _prenormed_work(self, x, ss, eps, w, out, *rest, **kw):
    return _size(x) + _size(ss) + _size(w) + _size(out), 2 * x.shape[0] * w.shape[0] * w.shape[1]


def _residual_work(self, a, w, h, *rest, **kw):
    return _size(a) + _size(w) + 2 * _size(h), 2 * a.shape[0] * w.shape[0] * w.shape[1]


def _norm_work(self, h, delta, weight, out, eps, rows=None, write_h=True):
    n, width = out.shape[0], h.shape[1]
    moved = n * width * 4 + _size(out)
    if delta is not None:
        moved += n * width * (delta.element_size() + (4 if write_h else 0))
    return moved, 0


def _embed_work(self, ids, table, h):
    return _size(h) + h.numel() * table.element_size(), 0


def _rope_work(self, qkv, *rest, **kw):
    return 2 * _size(qkv), 0


def _tensors_work(*names):
    def work(self, *args, **kw):
        return sum(_size(a) for a in args if isinstance(a, torch.Tensor)), 0
    return work


class Kernels:
    def __init__(self, dtype, library_gemm=True):
        _need(dtype in (torch.float32, torch.bfloat16), f"no kernels for element type {dtype}")
        if not torch.cuda.is_available():
            raise KernelError("no GPU is visible: the engine's kernels are HIP only")
        self.dtype = dtype
        self.library_gemm = library_gemm
        self._library_workspace = None      # scratch memory of the vendor library's products, allocated once
        self._libs = {}
        self.profiler = None                # a `Profiler`: every launch is then bracketed by events

    # -- libraries ---------------------------------------------------------------------------
    def prepare(self, names):
        """Build (if need be) and load several libraries at once."""
        typed = [n for n in names if build.HIP_LIBRARIES[n][2]]
        untyped = [n for n in names if not build.HIP_LIBRARIES[n][2]]
        if typed:
            build.ensure_built(typed, self.dtype)
        if untyped:
            build.ensure_built(untyped)
        for n in names:
            self._lib(n)

    def _lib(self, name):
        lib = self._libs.get(name)
        if lib is None:
            lib = build.load(name, self.dtype)
            self._libs[name] = lib
        return lib

    # -- row-wise ----------------------------------------------------------------------------
    @timed("embed", _embed_work)
    def embed_gather(self, ids, table, h):
        """h[m] = float(table[ids[m]])."""
        rows = ids.numel()
        _tensor(ids, "ids", torch.int32, ndim=1)
        _tensor(table, "table", self.dtype, ndim=2)
        vocab, width = table.shape
        _tensor(h, "h", torch.float32, (rows, width))
        fn = self._lib("elementwise").mlr_embed_gather
        _ok(fn(_p(ids), _p(table), _p(h), _c_int(rows), _c_int(width), _c_int(vocab), _stream()),
            "embed_gather")

    @timed("norm", _norm_work)
    def add_rmsnorm(self, h, delta, weight, out, eps, rows=None, write_h=True):
        """x = h[src] + delta[src] (delta may be None); h[src] = x when write_h; out[r] =
        rmsnorm(x) * weight, src = rows[r] or r."""
        _tensor(h, "h", torch.float32, ndim=2)
        m, width = h.shape
        if delta is not None:
            _tensor(delta, "delta", self.dtype, (m, width))
        _tensor(weight, "weight", torch.float32, (width,))
        if rows is not None:
            _tensor(rows, "rows", torch.int32, ndim=1)
            n_out = rows.numel()
        else:
            n_out = m
        _tensor(out, "out", self.dtype, (n_out, width))
        fn = self._lib("elementwise").mlr_add_rmsnorm
        _ok(fn(_p(h), _p(delta), _p(weight), _p(out), _p(rows), _c_int(n_out), _c_int(width),
               _c_float(eps), _c_int(1 if (write_h and delta is not None) else 0), _stream()),
            "add_rmsnorm")

    @timed("check")
    def status_reset(self, status):
        """status = (0, INT_MAX): nothing seen yet.  A kernel, so that a captured step can hold it."""
        _tensor(status, "status", torch.int32, (2,))
        _ok(self._lib("elementwise").mlr_status_reset(_p(status), _stream()), "status_reset")

    @timed("check")
    def finite_check(self, h, delta, layer, status):
        """ORs into status[0] which kinds of non-finite values h + delta holds (1: NaN, 2: infinity) and keeps
        in status[1] the smallest (layer << 20 | row) that held one."""
        _tensor(h, "h", torch.float32, ndim=2)
        m, width = h.shape
        if delta is not None:
            _tensor(delta, "delta", self.dtype, (m, width))
        _tensor(status, "status", torch.int32, (2,))
        _need(0 <= layer < 2047, "finite_check: layer index out of range")
        _ok(self._lib("elementwise").mlr_finite_check(_p(h), _p(delta), _c_int(m), _c_int(width), _c_int(layer),
                                                      _p(status), _stream()), "finite_check")

    @timed("norm", _tensors_work())
    def residual_add(self, h, delta):
        _tensor(h, "h", torch.float32, ndim=2)
        _tensor(delta, "delta", self.dtype, tuple(h.shape))
        fn = self._lib("elementwise").mlr_residual_add
        _ok(fn(_p(h), _p(delta), _c_size_t(h.numel()), _stream()), "residual_add")

    @timed("activation", _tensors_work())
    def silu_mul(self, gate_up, act):
        """act[m, f] = silu(gate_up[m, f]) * gate_up[m, F + f]."""
        _tensor(gate_up, "gate_up", self.dtype, ndim=2)
        m, two_f = gate_up.shape
        _need(two_f % 2 == 0, "gate_up: the width must be even")
        _tensor(act, "act", self.dtype, (m, two_f // 2))
        fn = self._lib("elementwise").mlr_silu_mul
        _ok(fn(_p(gate_up), _p(act), _c_int(m), _c_int(two_f // 2), _stream()), "silu_mul")

    # -- projections -------------------------------------------------------------------------
    @timed("gemm", _gemm_work)
    def gemm(self, a, w, out):
        """out[M, N] = a[M, K] . w[N, K]^T; out has the element type or is float32."""
        _tensor(a, "a", self.dtype, ndim=2)
        _tensor(w, "w", self.dtype, ndim=2)
        m, k = a.shape
        n, k2 = w.shape
        _need(k == k2, lambda: f"gemm: inner sizes differ ({k} and {k2})")
        _need(out.dtype in (self.dtype, torch.float32), lambda: f"gemm: output type {out.dtype} not supported")
        _tensor(out, "out", out.dtype, (m, n))
        if self.library_gemm and self.dtype == torch.bfloat16 and m > LIBRARY_GEMM_MIN_ROWS and \
                (out.dtype == torch.float32 or not self.streams_weight(m, k)):
            # many rows: a plain matrix product, handed to the vendor library (hipBLASLt), as the reference
            # hands its projections to cuBLAS (src/minillm/cuda/matrix.cpp:11-37).  (Float outputs are
            # logits, a vocabulary wide: there the library wins from 17 rows on at any inner size.)
            ws = self.reserve_library_workspace(a.device)
            _ok(self._lib("library_gemm").mlr_library_gemm(_p(a), _p(w), _p(out), _c_int(m), _c_int(n), _c_int(k),
                                                           _c_int(1 if out.dtype == torch.float32 else 0),
                                                           _p(ws), _c_size_t(ws.numel()), _stream()), "library_gemm")
            return
        fn = self._lib("gemm").mlr_gemm
        _ok(fn(_p(a), _p(w), _p(out), _c_int(m), _c_int(n), _c_int(k),
               _c_int(1 if out.dtype == torch.float32 else 0), _stream()), "gemm")

    def reserve_library_workspace(self, device):
        """The vendor library's scratch memory, allocated once."""
        if self._library_workspace is None:
            self._library_workspace = torch.empty(LIBRARY_GEMM_WORKSPACE, dtype=torch.uint8, device=device)
        return self._library_workspace

    def library_workspace_bytes(self):
        return 0 if self._library_workspace is None else self._library_workspace.numel()

    def streams_weight(self, rows, k):
        """Whether a projection of this many rows and inner size goes to the kernels that stream the weight
        once into the matrix cores, and not to the vendor library: up to 16 rows always; up to 64 rows while
        the rows, which every workgroup reads again, stay small beside its strip of the weight (measured on
        weights that do not sit in a cache: k = 1024 up to 64 rows, k = 2048 up to 32)."""
        if self.dtype != torch.bfloat16:
            return False
        if not self.library_gemm:
            return rows <= 64
        return rows <= LIBRARY_GEMM_MIN_ROWS or (rows <= 64 and k * ((rows + 15) // 16) <= 4096)

    def gated_silu_fused(self, rows, k=None):
        """Whether `gemm_gated_silu` is the path for this many rows and inner size: the bfloat16 engine, where
        `streams_weight` says so (elsewhere the library's product and a separate activation are faster), and
        without the library any number of rows when the inner size is a multiple of 64."""
        if self.dtype == torch.bfloat16 and rows > 64 and k is not None and k % 64 == 0 and rows * k < 2 ** 31:
            # many rows: the wide kernel's gated form.  Beside the library it is the faster way while the inner
            # size is short (measured against the library's product followed by the activation kernel, at 128
            # to 2048 rows: 0.58-0.95 of their time at k = 1024, 0.84-1.07 at k = 2048, 1.01-1.40 beyond)
            return not self.library_gemm or k <= 1024 or (k <= 2048 and rows <= 256)
        return self.streams_weight(rows, k if k is not None else 1 << 30)

    @timed("gemm", _gemm_work)
    def gemm_gated_silu(self, a, w, out):
        """out[M, N] = silu(a . w[:N]^T) * (a . w[N:]^T), w = [gate; up] stacked: up to 64 rows, or any number
        when the inner size is a multiple of 64 (the wide kernel's gated form)."""
        _need(self.dtype == torch.bfloat16, "gemm_gated_silu: bfloat16 only")
        _need(a.shape[0] <= 64 or (a.shape[1] % 64 == 0 and a.numel() < 2 ** 31 and w.numel() < 2 ** 31),
              "gemm_gated_silu: more than 64 rows need an inner size that is a multiple of 64 (and matrices "
              "below 2^31 elements)")
        _tensor(a, "a", self.dtype, ndim=2)
        _tensor(w, "w", self.dtype, ndim=2)
        m, k = a.shape
        two_n, k2 = w.shape
        _need(k == k2 and two_n % 2 == 0, "gemm_gated_silu: sizes do not fit")
        _tensor(out, "out", self.dtype, (m, two_n // 2))
        fn = self._lib("gemm").mlr_gemm_gated_silu
        _ok(fn(_p(a), _p(w), _p(out), _c_int(m), _c_int(two_n // 2), _c_int(k), _stream()), "gemm_gated_silu")

    # -- an RMSNorm handed from one projection to the next (few rows) ------------------------------
    HANDOFF_MAX_ROWS = 16

    def handoff_supported(self, rows):
        """Whether the projections before and after a norm can share it between them: the bfloat16 engine, up to
        16 rows.  The projection before the norm adds its sums to the residual stream h and leaves
        x = bf16(h * norm_w) and partial sums of squares of h's rows (`gemm_residual`); the projection after it
        multiplies its finished sums by the rows' scale rsqrt(mean(h^2) + eps) (`gemm_prenormed`): the scale is
        a factor per row, so the product with it commutes with the projection."""
        return self.dtype == torch.bfloat16 and 1 <= rows <= self.HANDOFF_MAX_ROWS

    @staticmethod
    def handoff_parts(width):
        """Partial sums of squares a row that `gemm_residual` leaves for an output `width` wide."""
        return (width + 15) // 16

    @timed("norm", _rows_prenorm_work)
    def rows_prenorm(self, h, delta, weight, out, ss):
        """h += delta (delta may be None); out = T(h * weight), without the norm's scale; ss[r, 0] = sum(h[r]^2)."""
        _tensor(h, "h", torch.float32, ndim=2)
        m, width = h.shape
        if delta is not None:
            _tensor(delta, "delta", self.dtype, (m, width))
        _tensor(weight, "weight", torch.float32, (width,))
        _tensor(out, "out", self.dtype, (m, width))
        _tensor(ss, "ss", torch.float32, (m, 1))
        fn = self._lib("elementwise").mlr_rows_prenorm
        _ok(fn(_p(h), _p(delta), _p(weight), _p(out), _p(ss), _c_int(m), _c_int(width), _stream()), "rows_prenorm")

    @timed("gemm", _prenormed_work)
    def gemm_prenormed(self, x, ss, eps, w, out, gated=False):
        """out = rsqrt(sum(ss[m]) / K + eps) * (x . w^T), x being T(h * norm_w) [M, K] and ss [M, parts] partial
        sums of squares of h's rows; gated=True (w = [gate; up] stacked): silu(scale * gate) * (scale * up)."""
        _tensor(x, "x", self.dtype, ndim=2)
        m, k = x.shape
        _need(self.handoff_supported(m), "gemm_prenormed: bfloat16, at most 16 rows")
        _tensor(ss, "ss", torch.float32, ndim=2)
        _need(ss.shape[0] == m and ss.shape[1] >= 1, "gemm_prenormed: one row of partial sums per row of x")
        _tensor(w, "w", self.dtype, ndim=2)
        n = w.shape[0] // 2 if gated else w.shape[0]
        _need(w.shape[1] == k and (not gated or w.shape[0] % 2 == 0), "gemm_prenormed: weight does not fit")
        _tensor(out, "out", self.dtype, (m, n))
        fn = self._lib("gemm").mlr_gemm_prenormed
        _ok(fn(_p(x), _p(ss), _c_int(ss.shape[1]), _c_float(eps), _c_int(k), _p(w), _p(out), _c_int(m), _c_int(n),
               _c_int(k), _c_int(1 if gated else 0), _stream()), "gemm_prenormed")

    @timed("gemm", _residual_work)
    def gemm_residual(self, a, w, h, next_w=None, x_out=None, ss_out=None):
        """h += a . w^T (32-bit, in place).  With next_w (the weights of the norm that follows) also
        x_out = T(h * next_w) and ss_out[m, p] = the sum of squares of h[m, 16 p : 16 p + 16]."""
        _tensor(a, "a", self.dtype, ndim=2)
        m, k = a.shape
        _need(self.handoff_supported(m), "gemm_residual: bfloat16, at most 16 rows")
        _tensor(w, "w", self.dtype, ndim=2)
        n = w.shape[0]
        _need(w.shape[1] == k, "gemm_residual: inner sizes differ")
        _tensor(h, "h", torch.float32, (m, n))
        if next_w is not None:
            _tensor(next_w, "next_w", torch.float32, (n,))
            _tensor(x_out, "x_out", self.dtype, (m, n))
            _tensor(ss_out, "ss_out", torch.float32, (m, self.handoff_parts(n)))
        fn = self._lib("gemm").mlr_gemm_residual
        _ok(fn(_p(a), _p(w), _p(h), _p(next_w), _p(x_out if next_w is not None else None),
               _p(ss_out if next_w is not None else None), _c_int(m), _c_int(n), _c_int(k), _stream()), "gemm_residual")

    # -- attention ---------------------------------------------------------------------------
    def _check_cache(self, k_pages, v_pages, kv_heads, head_dim, page_size):
        _tensor(k_pages, "k_pages", self.dtype, ndim=4)
        _need(k_pages.shape[1:] == (kv_heads, page_size, head_dim),
              lambda: f"k_pages: expected [pages, {kv_heads}, {page_size}, {head_dim}], got {tuple(k_pages.shape)}")
        _tensor(v_pages, "v_pages", self.dtype, (k_pages.shape[0], kv_heads, head_dim, page_size))

    @timed("rope_kv", _rope_work)
    def qk_norm_rope_kv(self, qkv, q_out, k_pages, v_pages, block_table, slots, positions, q_norm_w,
                        k_norm_w, eps, rope, q_heads, kv_heads, head_dim, page_size, write_cache=True,
                        interleaved=False):
        """Per head: RMSNorm of q and k (weights may be None), rotation by `rope` [max_positions, rot_dim]
        (cosines | sines; may be None) of the head's first rot_dim channels in pairs (j, j + rot_dim / 2), or
        (2 j, 2 j + 1) when `interleaved`; q into q_out, k and v into their pages."""
        _need(head_dim % 2 == 0 and 2 <= head_dim <= MAX_HEAD_DIM,
              lambda: f"head_dim {head_dim}: the rotation kernel takes even sizes up to {MAX_HEAD_DIM}")
        width = (q_heads + 2 * kv_heads) * head_dim
        _tensor(qkv, "qkv", self.dtype, ndim=2)
        m = qkv.shape[0]
        _need(qkv.shape[1] == width, lambda: f"qkv: expected width {width}, got {qkv.shape[1]}")
        _tensor(q_out, "q_out", self.dtype, (m, q_heads * head_dim))
        self._check_cache(k_pages, v_pages, kv_heads, head_dim, page_size)
        _tensor(block_table, "block_table", torch.int32, ndim=2)
        _tensor(slots, "slots", torch.int32, (m,))
        _tensor(positions, "positions", torch.int32, (m,))
        if q_norm_w is not None:
            _tensor(q_norm_w, "q_norm_w", torch.float32, (head_dim,))
            _tensor(k_norm_w, "k_norm_w", torch.float32, (head_dim,))
        rot_dim = head_dim
        if rope is not None:
            _tensor(rope, "rope", torch.float32, ndim=2)
            rot_dim = rope.shape[1]
            _need(2 <= rot_dim <= head_dim and rot_dim % 2 == 0,
                  lambda: f"rope: the table's width {rot_dim} must be even and at most head_dim {head_dim}")
        fn = self._lib("rope_kv").mlr_qk_norm_rope_kv
        _ok(fn(_p(qkv), _c_int(width), _p(q_out), _p(k_pages), _p(v_pages), _p(block_table),
               _c_int(block_table.shape[1]), _p(slots), _p(positions), _p(q_norm_w), _p(k_norm_w),
               _c_float(eps), _p(rope), _c_int(m), _c_int(q_heads), _c_int(kv_heads), _c_int(head_dim),
               _c_int(page_size), _c_int(1 if write_cache else 0), _c_int(rot_dim), _c_int(1 if interleaved else 0),
               _stream()), "qk_norm_rope_kv")

    @staticmethod
    def attention_partial_numel(rows, q_heads, head_dim, max_splits):
        """Floats of scratch memory for the partial results of split attention: per (row, head, split) the
        unnormalised output, its maximum and its sum (the prompt-portion kernel keeps them 16 bytes apart)."""
        return rows * q_heads * max_splits * (head_dim + 4)

    @timed("attention")
    def paged_attention(self, q, k_pages, v_pages, block_table, slots, positions, out, q_heads,
                        kv_heads, head_dim, page_size, scale, window=None, split_keys=0, max_splits=1,
                        partial=None):
        """out[m, h] = softmax over the keys seen by token m (positions <= its own, within the
        window) of q.k * scale, times v; keys and values from the pages of slots[m]."""
        _need(1 <= head_dim <= MAX_HEAD_DIM,
              lambda: f"head_dim {head_dim}: the attention kernel takes up to {MAX_HEAD_DIM}")
        _need(q_heads % kv_heads == 0, "q_heads must be a multiple of kv_heads")
        _tensor(q, "q", self.dtype, ndim=2)
        m = q.shape[0]
        _need(q.shape[1] == q_heads * head_dim, "q: wrong width")
        _tensor(out, "out", self.dtype, (m, q_heads * head_dim))
        self._check_cache(k_pages, v_pages, kv_heads, head_dim, page_size)
        _tensor(block_table, "block_table", torch.int32, ndim=2)
        _tensor(slots, "slots", torch.int32, (m,))
        _tensor(positions, "positions", torch.int32, (m,))
        _need(kv_heads <= 65535, "too many kv heads for the grid")
        if max_splits > 1:
            _need(split_keys > 0 and split_keys % ATTENTION_TILE_KEYS == 0,
                  lambda: f"split_keys must be a multiple of {ATTENTION_TILE_KEYS}")
            _need(partial is not None, "partial buffer needed for split attention")
            _tensor(partial, "partial", torch.float32, ndim=1)
            _need(partial.numel() >= self.attention_partial_numel(m, q_heads, head_dim, max_splits),
                  "partial buffer too small")
            group = q_heads // kv_heads
            _need(((group + 7) // 8) * max_splits <= 65535 and max_splits <= MAX_KEY_SPLITS,
                  "too many key splits for the grid")
        fn = self._lib("attention").mlr_paged_attention
        _ok(fn(_p(q), _p(k_pages), _p(v_pages), _p(block_table), _c_int(block_table.shape[1]), _p(slots),
               _p(positions), _p(out), _p(partial), _c_int(m), _c_int(q_heads), _c_int(kv_heads),
               _c_int(head_dim), _c_int(page_size), _c_int(window or 0), _c_float(scale),
               _c_int(split_keys), _c_int(max_splits), _stream()), "paged_attention")

    def mfma_attention_supported(self, q_heads, kv_heads, head_dim, page_size):
        """The matrix-core attention kernel serves the bfloat16 engine for pages that are a multiple of
        16 tokens, head sizes that are a multiple of 16 and up to 16 query heads per kv head."""
        return (self.dtype == torch.bfloat16 and page_size % 16 == 0 and head_dim % 16 == 0
                and head_dim <= MAX_HEAD_DIM and q_heads % kv_heads == 0 and q_heads // kv_heads <= 16)

    @timed("attention")
    def attention_mfma(self, q, k_pages, v_pages, block_table, slots, positions, out, group_row0, group_ntok,
                       groups, q_heads, kv_heads, head_dim, page_size, scale, window=None, split_keys=0,
                       max_splits=1, partial=None, partial_rows=None):
        """As `paged_attention`, on the matrix cores.  The batch rows are covered by `groups` groups of
        consecutive rows of one request each (group_row0[i], group_ntok[i]), at most 16 // (q_heads //
        kv_heads) tokens a group.  `partial_rows`: the caller vouches that every group's rows lie below this
        batch row (the partial results are indexed by batch row and need not reach further); default: all rows."""
        _need(self.mfma_attention_supported(q_heads, kv_heads, head_dim, page_size),
              "attention_mfma: sizes not supported (bfloat16, page_size % 16 == 0, head_dim % 16 == 0, "
              "at most 16 query heads per kv head)")
        _tensor(q, "q", self.dtype, ndim=2)
        m = q.shape[0]
        _need(q.shape[1] == q_heads * head_dim, "q: wrong width")
        _tensor(out, "out", self.dtype, (m, q_heads * head_dim))
        self._check_cache(k_pages, v_pages, kv_heads, head_dim, page_size)
        _tensor(block_table, "block_table", torch.int32, ndim=2)
        _tensor(slots, "slots", torch.int32, (m,))
        _tensor(positions, "positions", torch.int32, (m,))
        _tensor(group_row0, "group_row0", torch.int32, (groups,))
        _tensor(group_ntok, "group_ntok", torch.int32, (groups,))
        _need(kv_heads <= 65535 and max_splits <= MAX_KEY_SPLITS, "too many kv heads or key splits for the grid")
        if max_splits > 1:
            _need(split_keys > 0 and split_keys % ATTENTION_TILE_KEYS == 0,
                  lambda: f"split_keys must be a multiple of {ATTENTION_TILE_KEYS}")
            _need(partial is not None, "partial buffer needed for split attention")
            _tensor(partial, "partial", torch.float32, ndim=1)
            reach = m if partial_rows is None else partial_rows
            _need(0 < reach <= m and partial.numel() >= self.attention_partial_numel(reach, q_heads, head_dim, max_splits),
                  "partial buffer too small")
        _need((split_keys // page_size + 2 if max_splits > 1 else block_table.shape[1]) <= MFMA_MAX_PAGES,
              "attention_mfma: a workgroup's key range spans more than 4096 pages; split the keys")
        fn = self._lib("attention").mlr_attention_mfma
        _ok(fn(_p(q), _p(k_pages), _p(v_pages), _p(block_table), _c_int(block_table.shape[1]), _p(slots),
               _p(positions), _p(out), _p(partial), _p(group_row0), _p(group_ntok), _c_int(groups), _c_int(m),
               _c_int(q_heads), _c_int(kv_heads), _c_int(head_dim), _c_int(page_size), _c_int(window or 0),
               _c_float(scale), _c_int(split_keys), _c_int(max_splits), _stream()), "attention_mfma")

    @staticmethod
    def max_key_splits():
        return MAX_KEY_SPLITS

    @staticmethod
    def mfma_longest_context(page_size):
        """The most keys that one workgroup of `attention_mfma` / `attention_decode_fused` can walk (it keeps
        their page ids in LDS; a key split that does not start at a page's edge touches one page more)."""
        return (MFMA_MAX_PAGES - 2) * page_size

    def decode_fusion_supported(self, q_heads, kv_heads, head_dim, page_size):
        """Attention for single new tokens that norms, rotates and caches inside itself: the matrix-core
        kernel's sizes and head sizes that are multiples of 64."""
        return self.mfma_attention_supported(q_heads, kv_heads, head_dim, page_size) and head_dim % 64 == 0

    @timed("attention")
    def attention_decode_fused(self, qkv, k_pages, v_pages, block_table, slots, positions, out, group_row0, group_ntok,
                               groups, q_heads, kv_heads, head_dim, page_size, scale, q_norm_w, k_norm_w, eps, rope,
                               partial, window=None, split_keys=0, max_splits=1):
        """For a batch in which every group is ONE new token of a request (the caller vouches for that):
        per-head RMSNorm of q and k (weights may both be None), rotation by `rope` (may be None), attention
        over the cached keys and the token's own, and the write of the token's key and value into their
        pages, in two launches.  `qkv` holds the raw projections; `partial` is needed also without splits."""
        _need(self.decode_fusion_supported(q_heads, kv_heads, head_dim, page_size),
              "attention_decode_fused: sizes not supported")
        width = (q_heads + 2 * kv_heads) * head_dim
        _tensor(qkv, "qkv", self.dtype, ndim=2)
        m = qkv.shape[0]
        _need(qkv.shape[1] == width, lambda: f"qkv: expected width {width}, got {qkv.shape[1]}")
        _need(groups == m, "attention_decode_fused: one group per row")
        _tensor(out, "out", self.dtype, (m, q_heads * head_dim))
        self._check_cache(k_pages, v_pages, kv_heads, head_dim, page_size)
        _tensor(block_table, "block_table", torch.int32, ndim=2)
        _tensor(slots, "slots", torch.int32, (m,))
        _tensor(positions, "positions", torch.int32, (m,))
        _tensor(group_row0, "group_row0", torch.int32, (groups,))
        _tensor(group_ntok, "group_ntok", torch.int32, (groups,))
        _need((q_norm_w is None) == (k_norm_w is None), "q and k norm weights come together")
        if q_norm_w is not None:
            _tensor(q_norm_w, "q_norm_w", torch.float32, (head_dim,))
            _tensor(k_norm_w, "k_norm_w", torch.float32, (head_dim,))
        if rope is not None:
            _tensor(rope, "rope", torch.float32, ndim=2)
            _need(rope.shape[1] == head_dim, "rope: table width must equal head_dim")
        max_splits = max(1, max_splits)
        _need(kv_heads <= 65535 and max_splits <= MAX_KEY_SPLITS, "too many kv heads or key splits for the grid")
        if max_splits > 1:
            _need(split_keys > 0 and split_keys % ATTENTION_TILE_KEYS == 0,
                  lambda: f"split_keys must be a multiple of {ATTENTION_TILE_KEYS}")
        _tensor(partial, "partial", torch.float32, ndim=1)
        _need(partial.numel() >= self.attention_partial_numel(m, q_heads, head_dim, max_splits), "partial buffer too small")
        _need((split_keys // page_size + 2 if max_splits > 1 else block_table.shape[1]) <= MFMA_MAX_PAGES,
              "attention_decode_fused: a workgroup's key range spans more than 4096 pages; split the keys")
        fn = self._lib("attention").mlr_attention_decode_fused
        _ok(fn(_p(qkv), _c_int(width), _p(k_pages), _p(v_pages), _p(block_table), _c_int(block_table.shape[1]),
               _p(slots), _p(positions), _p(out), _p(partial), _p(group_row0), _p(group_ntok), _c_int(groups),
               _c_int(q_heads), _c_int(kv_heads), _c_int(head_dim), _c_int(page_size), _c_int(window or 0),
               _c_float(scale), _c_int(split_keys), _c_int(max_splits), _p(q_norm_w), _p(k_norm_w), _c_float(eps),
               _p(rope), _stream()), "attention_decode_fused")

    def prefill_attention_supported(self, q_heads, kv_heads, head_dim, page_size, max_context=0):
        """The LDS-staged kernel for prompt portions: as the matrix-core kernel, head sizes up to 192 and
        contexts of at most 2048 pages (it keeps a group's page ids in LDS)."""
        return (self.mfma_attention_supported(q_heads, kv_heads, head_dim, page_size) and head_dim <= 192
                and max_context <= PREFILL_MAX_PAGES * page_size)

    @timed("attention")
    def attention_prefill(self, q, k_pages, v_pages, block_table, slots, positions, out, group_row0, group_ntok,
                          groups, q_heads, kv_heads, head_dim, page_size, scale, window=None, max_context=None):
        """Attention for prompt portions: groups of up to 4 * (16 // (q_heads // kv_heads)) consecutive rows
        of one request each; keys and values of a group are staged once through LDS."""
        _need(self.prefill_attention_supported(q_heads, kv_heads, head_dim, page_size),
              "attention_prefill: sizes not supported")
        _need(block_table.shape[1] <= PREFILL_MAX_PAGES or max_context is not None,
              "attention_prefill: give max_context when the block table is wider than the kernel's page cache")
        _need((max_context or 0) <= PREFILL_MAX_PAGES * page_size, "attention_prefill: context too long")
        _tensor(q, "q", self.dtype, ndim=2)
        m = q.shape[0]
        _need(q.shape[1] == q_heads * head_dim, "q: wrong width")
        _tensor(out, "out", self.dtype, (m, q_heads * head_dim))
        self._check_cache(k_pages, v_pages, kv_heads, head_dim, page_size)
        _tensor(block_table, "block_table", torch.int32, ndim=2)
        _tensor(slots, "slots", torch.int32, (m,))
        _tensor(positions, "positions", torch.int32, (m,))
        _tensor(group_row0, "group_row0", torch.int32, (groups,))
        _tensor(group_ntok, "group_ntok", torch.int32, (groups,))
        _need(kv_heads <= 65535, "too many kv heads for the grid")
        fn = self._lib("attention").mlr_attention_prefill
        _ok(fn(_p(q), _p(k_pages), _p(v_pages), _p(block_table), _c_int(block_table.shape[1]), _p(slots),
               _p(positions), _p(out), _p(group_row0), _p(group_ntok), _c_int(groups), _c_int(q_heads),
               _c_int(kv_heads), _c_int(head_dim), _c_int(page_size), _c_int(window or 0), _c_float(scale),
               _stream()), "attention_prefill")

    def tiles_attention_supported(self, q_heads, kv_heads, head_dim, page_size, max_context=0, num_pages=0,
                                  split_keys=0):
        """The 32x32-tile kernel for prompt portions: bfloat16, head sizes up to 128 in steps of 16, pages
        of a power of two of keys, at most 16 query heads per kv head, contexts of at most 2048 pages (it
        keeps a group's page ids in LDS), a cache of fewer than 2^32 elements per layer (32-bit offsets)."""
        stride = kv_heads * page_size * head_dim
        return (self.mfma_attention_supported(q_heads, kv_heads, head_dim, page_size) and head_dim <= TILES_MAX_HEAD_DIM
                and page_size & (page_size - 1) == 0
                and (split_keys > 0 or max_context <= PREFILL_MAX_PAGES * page_size)
                and stride < 2 ** 24 and num_pages < 2 ** 24 and stride * num_pages < 2 ** 32)

    @staticmethod
    def tiles_sizes_supported(q_heads, kv_heads, head_dim, page_size):
        """The part of `tiles_attention_supported` that the model's sizes and the page size decide (bfloat16 engine)."""
        return (page_size % 16 == 0 and page_size & (page_size - 1) == 0 and head_dim % 16 == 0
                and head_dim <= TILES_MAX_HEAD_DIM and q_heads % kv_heads == 0 and q_heads // kv_heads <= 16)

    @staticmethod
    def tiles_longest_context(page_size):
        """The most keys that one workgroup of `attention_tiles` can walk (it keeps their page ids in LDS;
        a key split that does not start at a page's edge touches one page more)."""
        return (PREFILL_MAX_PAGES - 2) * page_size

    @staticmethod
    def tiles_group_tokens(q_heads, kv_heads, columns=TILES_COLUMNS[0]):
        """The most tokens of a group of `attention_tiles` with workgroups of `columns` columns."""
        return columns // (q_heads // kv_heads)

    @timed("attention")
    def attention_tiles(self, q, k_pages, v_pages, block_table, slots, positions, out, group_row0, group_ntok,
                        groups, q_heads, kv_heads, head_dim, page_size, scale, window=None, max_context=None,
                        columns=TILES_COLUMNS[0], split_keys=0, max_splits=1, partial=None, pairing="auto"):
        """Attention for prompt portions: groups of up to columns // (q_heads // kv_heads) consecutive rows
        of one request each (columns = 128, or 64 for batches that would not fill the GPU with the larger
        workgroups); keys and values of a group are staged once through LDS in blocks of 64.  With
        max_splits > 1 a group's keys are split over workgroups in ranges of split_keys (a multiple of 64)
        and merged through `partial`.  `pairing`: whether a workgroup of 128 columns (without splits) takes two
        groups, an early and a late one of a prompt, which evens out their key ranges: "auto" unless that would
        leave compute units idle, "single" never, "pairs" always.  The caller vouches for the groups (consecutive rows of one request,
        no more tokens than `tiles_group_tokens`)."""
        _need(columns in TILES_COLUMNS, lambda: f"attention_tiles: columns must be one of {TILES_COLUMNS}")
        _need(pairing in TILES_PAIRING, lambda: f"attention_tiles: pairing must be one of {sorted(TILES_PAIRING)}")
        _need(self.tiles_attention_supported(q_heads, kv_heads, head_dim, page_size, num_pages=k_pages.shape[0]),
              "attention_tiles: sizes not supported")
        _tensor(q, "q", self.dtype, ndim=2)
        m = q.shape[0]
        if max_splits > 1:
            _need(split_keys > 0 and split_keys % ATTENTION_TILE_KEYS == 0,
                  lambda: f"split_keys must be a multiple of {ATTENTION_TILE_KEYS}")
            _need(max_splits <= MAX_KEY_SPLITS and groups <= 65535, "too many key splits or groups for the grid")
            _need(split_keys // page_size + 2 <= PREFILL_MAX_PAGES, "attention_tiles: a split spans too many pages")
            _need(partial is not None, "partial buffer needed for split attention")
            _tensor(partial, "partial", torch.float32, ndim=1)
            _need(partial.numel() >= self.attention_partial_numel(m, q_heads, head_dim, max_splits),
                  "partial buffer too small")
        else:
            _need(block_table.shape[1] <= PREFILL_MAX_PAGES or max_context is not None,
                  "attention_tiles: give max_context when the block table is wider than the kernel's page cache")
            _need((max_context or 0) <= PREFILL_MAX_PAGES * page_size, "attention_tiles: context too long")
        _need(q.shape[1] == q_heads * head_dim, "q: wrong width")
        _tensor(out, "out", self.dtype, (m, q_heads * head_dim))
        self._check_cache(k_pages, v_pages, kv_heads, head_dim, page_size)
        _tensor(block_table, "block_table", torch.int32, ndim=2)
        _tensor(slots, "slots", torch.int32, (m,))
        _tensor(positions, "positions", torch.int32, (m,))
        _tensor(group_row0, "group_row0", torch.int32, (groups,))
        _tensor(group_ntok, "group_ntok", torch.int32, (groups,))
        _need(kv_heads <= 65535, "too many kv heads for the grid")
        fn = self._lib("attention_tiles").mlr_attention_tiles
        _ok(fn(_p(q), _p(k_pages), _p(v_pages), _p(block_table), _c_int(block_table.shape[1]), _p(slots),
               _p(positions), _p(out), _p(group_row0), _p(group_ntok), _c_int(groups), _c_int(columns),
               _c_int(q_heads), _c_int(kv_heads), _c_int(head_dim), _c_int(page_size), _c_int(k_pages.shape[0]),
               _c_int(window or 0), _c_float(scale), _c_int(split_keys), _c_int(max_splits), _p(partial),
               _c_int(TILES_PAIRING[pairing]), _stream()), "attention_tiles")

    # -- sampling ----------------------------------------------------------------------------
    def sample_scratch(self, rows):
        """(floats, ints) of scratch memory that `sample` needs for this many rows."""
        lib = self._lib("sampling")
        return lib.mlr_sample_scratch_floats(_c_int(rows)), lib.mlr_sample_scratch_ints(_c_int(rows))

    @timed("sampler")
    def sample(self, logits, temperature, uniform, tokens, status, scratch_f, scratch_i, any_sampling=True):
        """tokens[r] = argmax (temperature <= 0) or the inverse-CDF draw at uniform[r]."""
        _tensor(logits, "logits", torch.float32, ndim=2)
        rows, vocab = logits.shape
        _tensor(temperature, "temperature", torch.float32, (rows,))
        _tensor(uniform, "uniform", torch.float32, (rows,))
        _tensor(tokens, "tokens", torch.int32, (rows,))
        _tensor(status, "status", torch.int32, (2,))
        need_f, need_i = self.sample_scratch(rows)
        _tensor(scratch_f, "scratch_f", torch.float32, ndim=1)
        _tensor(scratch_i, "scratch_i", torch.int32, ndim=1)
        _need(scratch_f.numel() >= need_f and scratch_i.numel() >= need_i, "sample: scratch buffers too small")
        _need(rows <= 65535, "sample: too many rows for the grid")
        fn = self._lib("sampling").mlr_sample
        _ok(fn(_p(logits), _c_int(rows), _c_int(vocab), _p(temperature), _p(uniform), _p(tokens),
               _p(status), _p(scratch_f), _p(scratch_i), _c_int(1 if any_sampling else 0), _stream()), "sample")
