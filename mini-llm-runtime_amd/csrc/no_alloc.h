// An entry point that allocates nothing.
//
// It has no counterpart in the reference (lilong555/mini-llm-runtime samples on the host or with an argmax
// kernel over buffers of its runtime's arena).  It is for callers that cannot allocate device memory: code
// under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.
//
// mlr_sample_static is mlr_sample (sampling.hip: greedy and temperature token choice from float logits) with
// the scratch memory of its four passes -- per (row, chunk of the vocabulary) a maximum, its index, a
// non-finite flag and a sum of exponentials, per row its maximum -- taken from an array that is part of the
// library's code object instead of from two workspace arguments.  The caller passes inputs and outputs only.
//
//   * At most MLR_SAMPLE_STATIC_MAX_ROWS rows a call; more is refused with MLR_SAMPLE_STATIC_TOO_MANY_ROWS
//     (a line on standard error says so) and nothing is launched.
//   * The array takes MLR_SAMPLE_STATIC_BYTES (257 KiB) of device memory on every GPU the library is used
//     on, from the library's load on that GPU until the process ends.
//   * Nothing in the array has to start at zero: every word that a pass reads was written by an earlier pass
//     of the same call.  The array keeps the last call's contents.
//   * Every call on a GPU uses that GPU's one array: calls that overlap on one GPU (different streams, or
//     several host threads) race.  Calls on one stream are ordered by the stream.
//   * The address of the array on the current device is looked up once per device, on the first call there
//     (hipGetSymbolAddress; a call with rows == 0 does just that and launches nothing: make it before a
//     stream capture begins).  No hipMalloc, hipFree or allocating library routine is called, ever.
//
// Returns 0, a HIP error code of the launches (positive), or one of the negative codes below.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#define MLR_SAMPLE_STATIC_MAX_ROWS 256
#define MLR_SAMPLE_STATIC_BYTES (MLR_SAMPLE_STATIC_MAX_ROWS * (2 * 64 + 1) * 4 + MLR_SAMPLE_STATIC_MAX_ROWS * 2 * 64 * 4)

#define MLR_SAMPLE_STATIC_BAD_VOCAB (-1)
#define MLR_SAMPLE_STATIC_TOO_MANY_ROWS (-3)
#define MLR_SAMPLE_STATIC_NO_DEVICE (-10)        // hipGetDevice failed, or a device index beyond 63
#define MLR_SAMPLE_STATIC_NO_SYMBOL (-12)        // hipGetSymbolAddress failed on this device

extern "C" int mlr_sample_static(const float* logits, int rows, int vocab, const float* temperature,
                                 const float* uniform, int32_t* tokens, int32_t* status, int any_sampling,
                                 hipStream_t stream);
