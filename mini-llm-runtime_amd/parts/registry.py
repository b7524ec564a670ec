"""Registries of the parts a layer is put together from.  A spec's `kind` picks the class; a
class is registered with a decorator and may live anywhere (a test can register a toy part
without touching this package).

Interfaces (B = the tokens of a step, E = the model width, T = the engine's element type):

  norm            weight_specs() -> {local name: WeightSpec};  bind({local name: tensor});
                  forward(ctx, h, delta, out, rows=None, write_h=True): h is the float residual
                  stream [B, E]; x = h + delta (delta may be None) is written back to h when
                  write_h; out[r] = norm(x[rows[r] or r]) as T.
  position        rotation(max_positions, device) -> Rotation (the table of cosines and sines, how
                  many channels of a head it turns and how they pair up), or None for "no rotation".
  mixer           weight_specs(), bind();  cache_spec() -> KvSpec | PagedSpec | StateSpec | None;
                  libraries() -> names of the kernel libraries it launches;
                  forward(ctx, x, cache_id, write_cache) -> T [B, E], x being the normed input.
  feed-forward    weight_specs(), bind(), libraries();  forward(ctx, x) -> T [B, E].
  block           built from (norm1, mixer, norm2, ffn);  forward(ctx, h, pending, cache_id,
                  write_cache, next_norm=None) -> the next pending delta: a block adds `pending`
                  (the previous block's last output) into h itself, fused with its first norm.
                  `pending` may also be a `Handoff` (h is complete and the first half of a norm is
                  done); a block may return one for `next_norm`, the norm the next block starts with.
  embed           weight_specs(), bind(), libraries();  forward(ctx) -> the float residual stream [B, E] of
                  the step's tokens (ctx.token_ids);  optional table() -> the [vocab, E] matrix that a tied head
                  may share;  workspace_plan(rows, logits_rows, dtype, limits).
  head            weight_specs(), bind(weights, embed=the embedding part), libraries();
                  forward(ctx, final) -> float logits [R, V] of the normed rows final [R, E];
                  workspace_plan(rows, logits_rows, dtype, limits).
  Optional, for steps of few rows (each falls back to forward when a part lacks it):
  norm            handoff-capable norms set `fusable_rmsnorm = True` and offer
                  prenorm(ctx, h, delta) -> Handoff.
  mixer           forward_handoff(ctx, hand, h, norm_after, cache_id, write_cache) -> Handoff | None:
                  the first projection takes `hand`, the last adds into h and prepares `norm_after`.
  feed-forward    forward_handoff(ctx, hand, h, norm_after) -> Handoff | None, likewise.

A mixer that keeps something else than keys and values per token names it in a PagedSpec: tensors by their
shape within a page, optionally a page size and an element type of its own; it finds them, with the group's
block table, in ctx.cache.paged_view(cache_id).

A mixer with state of fixed size (cache_spec() -> StateSpec) reads a request's live state from
ctx.cache.state_view(cache_id)[slot] and leaves the state its step leads to in
ctx.cache.state_stage(cache_id)[slot], for every slot of the step (when write_cache).  The staged rows become
live when every layer of the step has run, so a step that fails on the way leaves the live state as it was.
ctx.segment_slots holds the step's slots as a device vector (one a segment).

A part may set the class attribute `graph_safe = True` when what it launches depends only on the step's
SHAPE -- how many tokens each entry brings (ctx.n_tokens, the lengths in ctx.segments, ctx.single_tokens,
ctx.token_groups) and ctx.max_context, which in a step that is to be captured is its context bucket (512, 1024,
2048, ... up to the runner's max_length: the smallest that holds the step's longest context) --
and everything else reaches its kernels through device memory (ctx.token_ids, positions, slots, the cache
views).  Steps of a shape that comes again are then captured once as a HIP graph and replayed.  A part
that reads the slots or positions of ctx.segments on the host, or keeps host-side state per request, must
leave it unset; a model with such a part runs every step eagerly.  The capture of a shape runs the step three
times (an eager reference and two replays of the fresh graph, which are compared): writes of keys and values
are the same each time, and the live state of fixed size is put back before every further run, so a part needs
no care of its own for that.

No part is told which model it is in; sizes and constants arrive through its spec.
"""
from __future__ import annotations

from dataclasses import dataclass

_REGISTRIES = {"norm": {}, "position": {}, "mixer": {}, "ffn": {}, "block": {}, "embed": {}, "head": {}}


@dataclass
class Rotation:
    """What a position part hands a mixer: `table` float [max_positions, dim] on the device, the cosines of
    the pairs' angles in its first half and their sines in the second; the first `dim` channels of a head
    (even, at most the head size) are rotated, the rest pass through; pair j is the channels
    (j, j + dim / 2), or (2 j, 2 j + 1) when `interleaved`.  The extent and the pairing are the position
    part's to decide; the attention part and its kernels take what they are given."""
    table: object
    dim: int
    interleaved: bool = False


@dataclass
class Handoff:
    """A norm shared between the projection before it and the projection after it (few rows, see
    `Kernels.handoff_supported`): the residual stream h is complete (nothing is pending), `x` holds
    T(h * norm.weight) without the rows' scale and `ss` [rows, parts] partial sums of squares of h's rows.
    Whoever runs the first projection after `norm` applies rsqrt(sum(ss) / width + norm.eps) to its sums
    (`Kernels.gemm_prenormed`).  A block may hand one to the next block instead of a pending delta."""
    norm: object
    x: object
    ss: object


class PartError(ValueError):
    pass


def register_part(family, kind):
    if family not in _REGISTRIES:
        raise PartError(f"unknown part family {family!r}")

    def add(cls):
        _REGISTRIES[family][kind] = cls
        return cls
    return add


def part_class(family, kind):
    try:
        return _REGISTRIES[family][kind]
    except KeyError:
        known = ", ".join(sorted(_REGISTRIES.get(family, {}))) or "none"
        raise PartError(f"no {family} part of kind {kind!r}; known: {known}") from None


def build_part(family, spec, **kwargs):
    return part_class(family, spec.kind)(spec, **kwargs)
