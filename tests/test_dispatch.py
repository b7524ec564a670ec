"""The host-side decisions about attention's key splits, without a GPU: a context whose pages do not fit
one workgroup's page cache is split whatever the batch, and a runner that could not serve its own
max_length is refused when it is built, not in the middle of a step."""
import pytest
import torch

from mini_llm_runtime_amd.config.specs import AttentionSpec, NormSpec, PositionSpec
from mini_llm_runtime_amd.engine.context import StepContext, Workspace
from mini_llm_runtime_amd.kernels.ops import MAX_KEY_SPLITS, MFMA_MAX_PAGES, Kernels
from mini_llm_runtime_amd.parts.registry import PartError, build_part


def kernels_without_gpu(dtype=torch.bfloat16):
    k = Kernels.__new__(Kernels)              # the size questions need no device
    k.dtype, k.library_gemm = dtype, True
    return k


def context(max_context, split_keys=256, split_max_tokens=256):
    ctx = StepContext(kernels_without_gpu(), None, Workspace("cpu"), torch.bfloat16, max_context, split_keys,
                      split_max_tokens)
    ctx.max_context = max_context
    return ctx


@pytest.mark.parametrize("page", [16, 32, 64])
@pytest.mark.parametrize("rows", [1, 64, 300, 4096])
def test_a_context_beyond_the_page_cache_is_split_whatever_the_batch(page, rows):
    longest = Kernels.mfma_longest_context(page)
    assert longest == (MFMA_MAX_PAGES - 2) * page
    ctx = context(longest + 5000)
    keys, splits, partial = ctx.attention_split(rows, rows, 8, 16, 128, longest=longest)
    assert splits > 1 and keys % 64 == 0 and keys <= longest and keys // page + 2 <= MFMA_MAX_PAGES
    assert splits == -(-ctx.max_context // keys) <= MAX_KEY_SPLITS
    assert partial.numel() >= rows * 16 * splits * (128 + 4)
    # at or below the limit a large batch is left alone (it fills the GPU without splits)
    ctx = context(longest)
    assert ctx.attention_split(4096, 4096, 8, 16, 128, longest=longest)[1] == 1


def test_small_batches_over_long_contexts_are_split_and_short_ones_not():
    ctx = context(4096)
    keys, splits, _ = ctx.attention_split(1, 1, 8, 16, 128, longest=65504)
    assert splits > 1 and keys * splits >= 4096
    assert context(200).attention_split(1, 1, 8, 16, 128, longest=65504)[1] == 1
    assert context(4096, split_keys=0).attention_split(1, 1, 8, 16, 128, longest=65504)[1] == 1


def attention_part(head_dim=128):
    norm = NormSpec("rmsnorm", head_dim, 1e-6)
    return build_part("mixer", AttentionSpec("gqa_attention", 1024, 16, 8, head_dim, head_dim ** -0.5, norm,
                                             PositionSpec("rope_split_half", head_dim, 1e6)))


def test_limits_are_checked_when_the_runner_is_built():
    part, k = attention_part(), kernels_without_gpu()
    part.check_limits(k, 40960, 16, 256)                         # the benchmark's sizes
    part.check_limits(k, 65504, 16, 0)                           # fits without splits
    with pytest.raises(PartError, match="needs key splits"):
        part.check_limits(k, 65505, 16, 0)
    with pytest.raises(PartError, match="exceeds"):
        part.check_limits(k, 1 << 20, 16, 1 << 17)
    part.check_limits(k, 1 << 20, 16, 256)
    with pytest.raises(PartError, match="more than"):
        part.check_limits(k, (1 << 15) * MAX_KEY_SPLITS + 1, 16, 256)
    # the float engine's kernel walks the block table itself
    part.check_limits(kernels_without_gpu(torch.float32), 1 << 22, 16, 0)


def test_even_head_sizes_are_taken_and_odd_ones_refused():
    for d in (2, 6, 20, 34, 256):
        attention_part(d)
    for d in (15, 258):
        with pytest.raises(PartError, match="head_dim"):
            attention_part(d)


def test_the_planned_partial_results_hold_every_choice_of_splits():
    """The 8B sizes with requests of up to 40960 tokens: whatever the step (single tokens, a 2048-token portion
    behind 34816 tokens of context, one single token beside such a portion), the partial results of split
    attention stay within what the part planned for them, and a forced split still covers the context."""
    spec = AttentionSpec("gqa_attention", 4096, 32, 8, 128, 128 ** -0.5, NormSpec("rmsnorm", 128, 1e-6),
                         PositionSpec("rope_split_half", 128, 1e6))
    part = build_part("mixer", spec)
    rows, page = 2048 + 64, 16
    limits = dict(max_length=40960, page_size=page, split_keys=256, split_max_tokens=256, target_workgroups=512)
    planned = part.workspace_plan(rows, torch.bfloat16, limits)[("attn_partial", torch.float32)]
    tiles_longest, mfma_longest = Kernels.tiles_longest_context(page), Kernels.mfma_longest_context(page)
    assert limits["max_length"] > tiles_longest          # prompt portions are split for every row at this length
    seen = 0
    for context in (300, 4096, 20000, tiles_longest, tiles_longest + 1, 34816 + 2048, 40960):
        ctx = context_with_budget(context, planned)
        for units_rows, batch_rows in ((1, 1), (8, 8), (64, 64), (1, rows), (8, rows), (200, rows)):
            keys, splits, partial = ctx.attention_split(units_rows, batch_rows, 8, 32, 128, longest=mfma_longest)
            assert partial is None or partial.numel() <= planned
            assert splits == 1 or keys * splits >= context
            seen = max(seen, 0 if partial is None else partial.numel())
        for groups in (1, 16, 128):                        # groups of a prompt portion (16 tokens x 4 heads a kv head)
            keys, splits, partial = ctx.group_split(groups, rows, 8, 32, 128, longest=tiles_longest)
            assert partial is None or partial.numel() <= planned
            if context > tiles_longest:
                assert splits > 1 and keys <= tiles_longest and keys * splits >= context
            seen = max(seen, 0 if partial is None else partial.numel())
    assert seen == planned                                 # the plan is met by some step, not merely an upper bound
    assert ctx.workspace.unplanned_bytes() <= 4 * planned  # (this workspace has no plan: one buffer, never beyond it)


def context_with_budget(max_context, budget):
    ctx = context(max_context)
    ctx.partial_budget = budget
    return ctx


def test_a_smallest_key_range_beyond_the_portion_kernels_reach_is_refused_when_the_runner_is_built():
    part, k = attention_part(), kernels_without_gpu()
    longest = Kernels.tiles_longest_context(16)
    part.check_limits(k, 40960, 16, longest - longest % 64)
    with pytest.raises(PartError, match="prompt portions"):
        part.check_limits(k, 40960, 16, 49152)             # fits the single-token kernel, not the portions'
    with pytest.raises(PartError, match="prompt portions"):
        part.check_limits(k, 4096, 16, 49152)              # refused whatever max_length: splits also fill the GPU
    # pages that the portion kernel does not take (no power of two) leave only the other kernel's limit
    part.check_limits(k, 40960, 48, 49152)


def test_key_ranges_of_one_width_whatever_the_batch():
    """The float engine's attention (`StepContext.fixed_split`): the width of a key range is the runner's setting
    for every number of rows and every context (so a token's sums do not depend on the batch), the ranges cover
    the context, and rows whose partial results would not fit what was planned are served by several launches."""
    per = lambda splits: Kernels.attention_partial_numel(1, 16, 128, splits)
    for max_context in (100, 256, 257, 4096, 40960):
        for rows in (1, 7, 300, 2048):
            ctx = context_with_budget(max_context, 2 * 512 * 128 * 132)
            keys, splits, chunk, partial = ctx.fixed_split(rows, 16, 128)
            if max_context <= 256:
                assert (keys, splits, chunk, partial) == (0, 1, rows, None)
                continue
            assert keys == 256 and splits == -(-max_context // 256)
            assert 1 <= chunk <= rows and partial.numel() == chunk * per(splits) <= ctx.partial_budget
            assert chunk == rows or (chunk + 1) * per(splits) > ctx.partial_budget
    # beyond 1024 ranges the width doubles (the merge kernel keeps one weight a range in LDS)
    ctx = context_with_budget(300000, None)
    keys, splits, chunk, _ = ctx.fixed_split(3, 16, 128)
    assert keys == 512 and splits == -(-300000 // 512) <= MAX_KEY_SPLITS and chunk == 3
