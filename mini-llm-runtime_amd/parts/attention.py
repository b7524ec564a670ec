"""Grouped-query attention over the paged cache: fused q/k/v projection, per-head RMSNorm of q
and k before the rotation, rotation, write of k and v into their pages, attention of every
token of the step over the keys at positions <= its own (optionally only a window of them),
output projection.  Order of operations as in the reference (src/minillm/runtime.cpp:250-319,
src/minillm/cuda/layer.cpp:42-63).  Consecutive query heads share a kv head."""
from __future__ import annotations

import torch

from ..cache.manager import KvSpec
from ..weights.loader import WeightSpec, stacked
from .registry import Handoff, PartError, build_part, register_part


@register_part("mixer", "gqa_attention")
class GqaAttention:
    graph_safe = True        # forward launches kernels over the step's device vectors only
    def __init__(self, spec):
        self.spec = spec
        s = spec
        if s.q_heads % s.kv_heads != 0:
            raise PartError(f"q_heads {s.q_heads} is no multiple of kv_heads {s.kv_heads}")
        if s.head_dim % 2 != 0 or not 2 <= s.head_dim <= 256:
            # (multiples of 16 run on the matrix cores in the bfloat16 engine, other even sizes on the
            # scalar kernels that serve the float engine)
            raise PartError(f"head_dim {s.head_dim}: the attention kernels take even sizes up to 256")
        if s.window is not None and s.window < 1:
            raise PartError("window must be positive")
        self.q_norm = build_part("norm", s.qk_norm) if s.qk_norm is not None else None
        self.k_norm = build_part("norm", s.qk_norm) if s.qk_norm is not None else None
        if s.qk_norm is not None and s.qk_norm.size != s.head_dim:
            raise PartError("the q/k norm must span one head")
        # (how much of a head a position part turns, and in which pairs, is the part's own business: it says
        # so in the `Rotation` it hands over at run time)
        self.position = build_part("position", s.position) if s.position is not None else None
        self.qkv = None
        self.o = None

    def weight_specs(self):
        s = self.spec
        specs = {
            "q_proj": WeightSpec((s.q_heads * s.head_dim, s.hidden), stack="qkv"),
            "k_proj": WeightSpec((s.kv_heads * s.head_dim, s.hidden), stack="qkv"),
            "v_proj": WeightSpec((s.kv_heads * s.head_dim, s.hidden), stack="qkv"),
            "o_proj": WeightSpec((s.hidden, s.q_heads * s.head_dim)),
        }
        if self.q_norm is not None:
            specs["q_norm.weight"] = self.q_norm.weight_specs()["weight"]
            specs["k_norm.weight"] = self.k_norm.weight_specs()["weight"]
        return specs

    def bind(self, weights):
        # rows of a projection are independent sums, so stacking q, k, v changes no result (the loader has
        # laid them out one after the other already: no copy then)
        self.qkv = stacked([weights["q_proj"], weights["k_proj"], weights["v_proj"]])
        self.o = weights["o_proj"]
        if self.q_norm is not None:
            self.q_norm.bind({"weight": weights["q_norm.weight"]})
            self.k_norm.bind({"weight": weights["k_norm.weight"]})

    def cache_spec(self):
        return KvSpec(self.spec.kv_heads, self.spec.head_dim, self.spec.window)

    def check_limits(self, kernels, max_length, page_size, split_keys):
        """Called once when a runner is built: whether every context up to `max_length` can be served
        with these pages and this smallest key range of a workgroup.  What cannot is refused here and
        not in the middle of a step."""
        s = self.spec
        if not kernels.mfma_attention_supported(s.q_heads, s.kv_heads, s.head_dim, page_size):
            return                        # the scalar kernel walks the block table itself: no limit
        # the kernel for single tokens and short portions, and the one for prompt portions where it takes the
        # sizes: each keeps the page ids of a workgroup's key range in LDS
        reaches = [("single tokens", kernels.mfma_longest_context(page_size))]
        if kernels.dtype == torch.bfloat16 and kernels.tiles_sizes_supported(s.q_heads, s.kv_heads, s.head_dim, page_size):
            reaches.append(("prompt portions", kernels.tiles_longest_context(page_size)))
        for what, longest in reaches:
            if split_keys > longest:
                # (a portion's key ranges are never narrower than split_keys: refused also where max_length
                # would fit, since a short portion of a long context may be split to fill the GPU)
                raise PartError(f"split_keys {split_keys} exceeds the {longest} keys one workgroup can walk "
                                f"for {what} with pages of {page_size} tokens")
            if max_length <= longest:
                continue
            if split_keys <= 0:
                if what == "prompt portions":
                    continue              # (without splits such contexts go to the kernel for single tokens)
                raise PartError(f"max_length {max_length} with pages of {page_size} tokens needs key splits "
                                f"(split_keys > 0): one workgroup walks at most {longest} keys")
            keys = split_keys
            while keys * 2 <= longest:
                keys *= 2
            if max_length > keys * kernels.max_key_splits():
                raise PartError(f"max_length {max_length} needs more than {kernels.max_key_splits()} key splits "
                                f"of {keys} keys")

    def workspace_plan(self, rows, dtype, limits):
        """{(buffer name, dtype): elements} that `forward` asks the workspace for in a step of `rows` tokens
        at most.  The partial results of split attention (indexed by batch row) are bounded twice: where a
        split only serves to fill the GPU it is made while (workgroups without it) x (splits) stays below
        twice `target_workgroups`, each workgroup serving at most 128 (token, head) columns; a context beyond
        one workgroup's reach is split for every row, into as few ranges as that reach allows.  `StepContext`
        keeps every choice of splits within this number (`partial_budget`)."""
        from ..engine.context import StepContext
        from ..kernels.ops import Kernels
        s = self.spec
        width = s.q_heads * s.head_dim
        page, base, longest_context = limits["page_size"], limits["split_keys"], limits["max_length"]
        forced = StepContext.forced_splits(longest_context, base, Kernels.mfma_longest_context(page))
        if dtype == torch.bfloat16 and Kernels.tiles_sizes_supported(s.q_heads, s.kv_heads, s.head_dim, page):
            forced = max(forced, StepContext.forced_splits(longest_context, base, Kernels.tiles_longest_context(page)))
        per_split = Kernels.attention_partial_numel(1, s.q_heads, s.head_dim, 1)
        partial = max(2 * limits["target_workgroups"] * 128 * (s.head_dim + 4), rows * forced * per_split)
        tq = max(1, 16 // (s.q_heads // s.kv_heads))
        plan = {("qkv", dtype): rows * (width + 2 * s.kv_heads * s.head_dim), ("q", dtype): rows * width,
                ("attn", dtype): rows * width, ("mixer_out", dtype): rows * s.hidden,
                ("attn_partial", torch.float32): partial}
        for big_factor in (0, 4, 8):
            plan[(f"token_groups_{tq}_{big_factor}", torch.int32)] = 2 * rows + 2
        return plan

    def libraries(self):
        tiles = ["attention_tiles"] if self.qkv is not None and self.qkv.dtype == torch.bfloat16 else []
        return ["gemm", "rope_kv", "attention"] + tiles

    def forward_handoff(self, ctx, hand, h, norm_after, cache_id, write_cache=True):
        """As `forward` on the norm that `hand` describes, its scale applied inside the q/k/v projection; the
        output projection adds into h and prepares `norm_after` (None: nothing follows)."""
        s = self.spec
        m = h.shape[0]
        k = ctx.kernels
        qkv = ctx.workspace.get("qkv", (m, (s.q_heads + 2 * s.kv_heads) * s.head_dim), ctx.dtype)
        k.gemm_prenormed(hand.x, hand.ss, hand.norm.eps, self.qkv, qkv)
        attn = self._attend(ctx, qkv, cache_id, write_cache)
        if norm_after is None:
            k.gemm_residual(attn, self.o, h)
            return None
        x = ctx.workspace.get("handoff_x", (m, s.hidden), ctx.dtype)
        ss = ctx.workspace.get("handoff_ss", (m, k.handoff_parts(s.hidden)), torch.float32)
        k.gemm_residual(attn, self.o, h, norm_after.weight, x, ss)
        return Handoff(norm_after, x, ss)

    def forward(self, ctx, x, cache_id, write_cache=True):
        s = self.spec
        m = x.shape[0]
        qkv = ctx.workspace.get("qkv", (m, (s.q_heads + 2 * s.kv_heads) * s.head_dim), x.dtype)
        ctx.kernels.gemm(x, self.qkv, qkv)
        attn = self._attend(ctx, qkv, cache_id, write_cache)
        out = ctx.workspace.get("mixer_out", (m, s.hidden), x.dtype)
        ctx.kernels.gemm(attn, self.o, out)
        return out

    def _attention_work(self, ctx, element_size):
        """For the profile: (bytes, flops) of this step's attention, from the host's view of the contexts."""
        s = self.spec
        keys_read = pairs = 0
        for _, _, n, p0 in ctx.segments:
            last = p0 + n
            keys_read += min(last, s.window + n - 1) if s.window else last
            for p in (range(p0, last) if s.window else ()):
                pairs += min(p + 1, s.window)
            if not s.window:
                pairs += n * p0 + n * (n + 1) // 2
        moved = keys_read * 2 * s.kv_heads * s.head_dim * element_size \
            + 2 * ctx.n_tokens * s.q_heads * s.head_dim * element_size
        return moved, 4 * pairs * s.q_heads * s.head_dim

    def _hint(self, kernels):
        if self._work is not None:                        # the step's attention work goes to its first launch
            kernels.profiler.next_work(*self._work)
            self._work = None

    def _attend(self, ctx, qkv, cache_id, write_cache):
        """Norm of q and k, rotation, cache write and attention on the fused projection's output; the heads'
        outputs [B, q_heads * head_dim] (before the output projection)."""
        s = self.spec
        k = ctx.kernels
        if k.profiler is not None and not ctx.fixed_groups:
            self._work = self._attention_work(ctx, qkv.element_size())
        else:
            self._work = None
        x = qkv
        m = qkv.shape[0]
        view = ctx.cache.kv_view(cache_id)
        rotation = self.position.rotation(ctx.max_positions, x.device) if self.position is not None else None
        if rotation is not None and not (2 <= rotation.dim <= s.head_dim and rotation.dim % 2 == 0
                                         and rotation.table.shape[1] == rotation.dim):
            raise PartError(f"the position part turns {rotation.dim} channels of a head of {s.head_dim}: must be "
                            "even, at most the head, and as wide as its table")
        rope = rotation.table if rotation is not None else None
        interleaved = rotation is not None and rotation.interleaved
        whole_split_half = rotation is None or (rotation.dim == s.head_dim and not rotation.interleaved)
        if (ctx.single_tokens and write_cache and x.dtype == torch.bfloat16 and whole_split_half
                and k.decode_fusion_supported(s.q_heads, s.kv_heads, s.head_dim, view.page_size)):
            # decoding: norm, rotation and cache write ride in the attention's two launches
            attn = ctx.workspace.get("attn", (m, s.q_heads * s.head_dim), x.dtype)
            groups, _, _ = ctx.token_groups(max(1, 16 // (s.q_heads // s.kv_heads)), 0)
            split_keys, max_splits, partial = ctx.attention_split(m, m, s.kv_heads, s.q_heads, s.head_dim,
                                                                  longest=k.mfma_longest_context(view.page_size))
            if partial is None:
                partial = ctx.workspace.get("attn_partial", (k.attention_partial_numel(m, s.q_heads, s.head_dim, 1),),
                                            torch.float32)
            self._hint(k)
            k.attention_decode_fused(
                qkv, view.k_pages, view.v_pages, view.block_table, ctx.slots, ctx.positions, attn, groups[0], groups[1],
                groups[2], s.q_heads, s.kv_heads, s.head_dim, view.page_size, float(s.scale),
                self.q_norm.weight if self.q_norm is not None else None,
                self.k_norm.weight if self.k_norm is not None else None,
                self.q_norm.eps if self.q_norm is not None else 0.0, rope, partial,
                window=s.window, split_keys=split_keys, max_splits=max_splits)
            return attn
        q = ctx.workspace.get("q", (m, s.q_heads * s.head_dim), x.dtype)
        k.qk_norm_rope_kv(
            qkv, q, view.k_pages, view.v_pages, view.block_table, ctx.slots, ctx.positions,
            self.q_norm.weight if self.q_norm is not None else None,
            self.k_norm.weight if self.k_norm is not None else None,
            self.q_norm.eps if self.q_norm is not None else 0.0, rope,
            s.q_heads, s.kv_heads, s.head_dim, view.page_size, write_cache, interleaved=interleaved)
        attn = ctx.workspace.get("attn", (m, s.q_heads * s.head_dim), x.dtype)
        if k.mfma_attention_supported(s.q_heads, s.kv_heads, s.head_dim, view.page_size):
            # prompt portions go to one of the LDS-staged kernels (the 32x32-tile one where it takes the
            # sizes), single tokens and short portions to the one that can split a token's keys over
            # workgroups
            sizes = (s.q_heads, s.kv_heads, s.head_dim, view.page_size)
            g = s.q_heads // s.kv_heads
            tq = max(1, 16 // g)
            # (with key splits the 32x32-tile kernel takes any context length)
            tiles = k.tiles_attention_supported(*sizes, max_context=ctx.max_context, num_pages=view.k_pages.shape[0],
                                                split_keys=ctx.split_keys)
            # workgroups of 128 columns (half the loads and LDS writes a column of those of 64) when the batch
            # brings at least one of them for every compute unit: else of 64
            columns = 128 if m * s.q_heads >= 128 * ctx.compute_units else 64
            big_factor = (columns // 16 if tiles
                          else 4 if k.prefill_attention_supported(*sizes, ctx.max_context) else 0)
            small, big, (small_rows, small_end) = ctx.token_groups(tq, big_factor)
            if big[2] and tiles:
                split_keys, max_splits, partial = ctx.group_split(
                    big[2], m, s.kv_heads, s.q_heads, s.head_dim, longest=k.tiles_longest_context(view.page_size))
                self._hint(k)
                k.attention_tiles(q, view.k_pages, view.v_pages, view.block_table, ctx.slots, ctx.positions, attn,
                                  big[0], big[1], big[2], s.q_heads, s.kv_heads, s.head_dim, view.page_size,
                                  float(s.scale), window=s.window, max_context=ctx.max_context, columns=columns,
                                  split_keys=split_keys, max_splits=max_splits, partial=partial)
            elif big[2]:
                self._hint(k)
                k.attention_prefill(q, view.k_pages, view.v_pages, view.block_table, ctx.slots, ctx.positions, attn,
                                    big[0], big[1], big[2], s.q_heads, s.kv_heads, s.head_dim, view.page_size,
                                    float(s.scale), window=s.window, max_context=ctx.max_context)
            if small[2]:
                # (partial results are indexed by batch row: they reach as far as the last row of a small group,
                # which in the scheduler's batches -- single tokens first -- is the number of single tokens)
                split_keys, max_splits, partial = ctx.attention_split(
                    small_rows, small_end, s.kv_heads, s.q_heads, s.head_dim, longest=k.mfma_longest_context(view.page_size))
                self._hint(k)
                k.attention_mfma(q, view.k_pages, view.v_pages, view.block_table, ctx.slots, ctx.positions, attn,
                                 small[0], small[1], small[2], s.q_heads, s.kv_heads, s.head_dim, view.page_size,
                                 float(s.scale), window=s.window, split_keys=split_keys, max_splits=max_splits,
                                 partial=partial, partial_rows=small_end)
        else:
            # the float engine (and sizes that the matrix-core kernels do not take): key ranges of a fixed width,
            # so that a token's result is the same to the bit however the step was cut or batched
            split_keys, max_splits, chunk, partial = ctx.fixed_split(m, s.q_heads, s.head_dim)
            self._hint(k)
            for r0 in range(0, m, chunk):
                r1 = min(m, r0 + chunk)
                k.paged_attention(q[r0:r1], view.k_pages, view.v_pages, view.block_table, ctx.slots[r0:r1],
                                  ctx.positions[r0:r1], attn[r0:r1], s.q_heads, s.kv_heads, s.head_dim, view.page_size,
                                  float(s.scale), window=s.window, split_keys=split_keys, max_splits=max_splits,
                                  partial=partial)
        return attn
