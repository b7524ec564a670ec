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
