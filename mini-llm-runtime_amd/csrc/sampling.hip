// Token choice from float logits:
//   temperature <= 0: the largest logit, ties -> lowest id;
//   temperature  > 0: inverse-CDF draw from softmax(logits / T) with the uniform number u[r]
//                     that the host derived from the request's own generator state.
// A row that holds a NaN or an infinity gives token -1 and sets status[0] |= 1,
// status[1] = min(status[1], row).  Max, exponentials and sums are 32-bit.
//
// A row is cut into CHUNKS equal ranges of the vocabulary, one workgroup each, so that a few rows
// still fill the GPU; inside a workgroup every thread owns a contiguous sub-range.  All sums run in
// ascending order of the vocabulary and the cut depends on the vocabulary size only, so a row's token
// depends on that row only.
//   pass 1 (rows x CHUNKS): max, first argmax and a non-finite flag per chunk;
//   pass 2 (rows): row max and argmax; greedy rows are done here;
//   pass 3 (rows x CHUNKS, only if some row samples): sum of exp((x - max) / T) per chunk;
//   pass 4 (rows): scan of the chunk sums, the chunk that holds u * total, then the token inside it.
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>

#include <mutex>

#include "no_alloc.h"

#define CHUNKS 64
#define THREADS 256

__device__ __forceinline__ void chunk_range(int vocab, int chunk, int* begin, int* end) {
    const int per = (vocab + CHUNKS - 1) / CHUNKS;
    *begin = min(vocab, chunk * per);
    *end = min(vocab, *begin + per);
}

// (Also clears the status words, which the next pass sets: one launch less than a kernel of its own.)
__global__ __launch_bounds__(THREADS) void chunk_max_kernel(const float* __restrict__ logits, int vocab,
                                                            float* __restrict__ cmax, int32_t* __restrict__ cidx,
                                                            int32_t* __restrict__ cbad, int32_t* __restrict__ status) {
    __shared__ float vals[THREADS];
    __shared__ int idxs[THREADS];
    __shared__ int bad;
    const int r = blockIdx.x, chunk = blockIdx.y, t = threadIdx.x;
    const float* row = logits + (size_t)r * vocab;
    int cb, ce;
    chunk_range(vocab, chunk, &cb, &ce);
    if (t == 0) bad = 0;
    if (t == 0 && r == 0 && chunk == 0) {
        status[0] = 0;
        status[1] = 0x7fffffff;
    }
    __syncthreads();
    // neighbouring threads read neighbouring elements; a thread meets its elements in ascending order, so
    // the first of equal maxima it keeps is the lowest, and the merge below prefers the lower index
    float best = -INFINITY;
    int best_i = 0x7fffffff;
    bool nonfinite = false;
    // (four loads are asked for before the first is used, each at an index inside the chunk: one load a turn
    // would cost a trip to memory each, one after the other)
    for (int i0 = cb + t; i0 < ce; i0 += 4 * THREADS) {
        float x[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) x[j] = row[min(i0 + j * THREADS, ce - 1)];
        asm volatile("" : "+v"(x[0]), "+v"(x[1]), "+v"(x[2]), "+v"(x[3]));      // (all four loaded here, none moved behind a branch)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int i = i0 + j * THREADS;
            if (i < ce) {
                if (!(fabsf(x[j]) <= 3.402823466e38f)) nonfinite = true;
                if (x[j] > best) { best = x[j]; best_i = i; }
            }
        }
    }
    if (nonfinite) bad = 1;
    vals[t] = best;
    idxs[t] = best_i;
    __syncthreads();
    for (int s = THREADS / 2; s > 0; s >>= 1) {
        if (t < s) {
            const float ov = vals[t + s];
            const int oi = idxs[t + s];
            if (ov > vals[t] || (ov == vals[t] && oi < idxs[t])) { vals[t] = ov; idxs[t] = oi; }
        }
        __syncthreads();
    }
    if (t == 0) {
        cmax[r * CHUNKS + chunk] = vals[0];
        cidx[r * CHUNKS + chunk] = idxs[0];
        cbad[r * CHUNKS + chunk] = bad;
    }
}

// One wavefront per row: CHUNKS == 64 lanes.
__global__ __launch_bounds__(64) void row_max_kernel(const float* __restrict__ cmax, const int32_t* __restrict__ cidx,
                                                     const int32_t* __restrict__ cbad,
                                                     const float* __restrict__ temperature,
                                                     float* __restrict__ rmax, int32_t* __restrict__ tokens,
                                                     int32_t* __restrict__ status) {
    const int r = blockIdx.x, lane = threadIdx.x;
    float v = cmax[r * CHUNKS + lane];
    int i = cidx[r * CHUNKS + lane];
    int bad = cbad[r * CHUNKS + lane];
    for (int off = 32; off > 0; off >>= 1) {
        const float ov = __shfl_xor(v, off, 64);
        const int oi = __shfl_xor(i, off, 64);
        bad |= __shfl_xor(bad, off, 64);
        if (ov > v || (ov == v && oi < i)) { v = ov; i = oi; }
    }
    if (lane != 0) return;
    rmax[r] = v;
    if (bad) {
        tokens[r] = -1;
        atomicOr(&status[0], 1);
        atomicMin(&status[1], r);
    } else {
        tokens[r] = i;                              // sampling rows overwrite this in pass 4
    }
}

__global__ __launch_bounds__(THREADS) void chunk_sum_kernel(const float* __restrict__ logits, int vocab,
                                                            const float* __restrict__ temperature,
                                                            const float* __restrict__ rmax,
                                                            float* __restrict__ csum) {
    __shared__ float vals[THREADS];
    const int r = blockIdx.x, chunk = blockIdx.y, t = threadIdx.x;
    const float temp = temperature[r];
    if (!(temp > 0.f)) return;
    const float* row = logits + (size_t)r * vocab;
    int cb, ce;
    chunk_range(vocab, chunk, &cb, &ce);
    const int per = (ce - cb + THREADS - 1) / THREADS;
    const int begin = min(ce, cb + t * per), end = min(ce, begin + per);
    const float inv_t = 1.0f / temp, row_max = rmax[r];
    float sum = 0.f;
    for (int i0 = begin; i0 < end; i0 += 4) {          // (four loads asked for at once; added in ascending order)
        float x[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) x[j] = row[min(i0 + j, end - 1)];
        asm volatile("" : "+v"(x[0]), "+v"(x[1]), "+v"(x[2]), "+v"(x[3]));
#pragma unroll
        for (int j = 0; j < 4; ++j)
            if (i0 + j < end) sum += expf((x[j] - row_max) * inv_t);
    }
    vals[t] = sum;
    __syncthreads();
    if (t == 0) {                                   // ascending order
        float c = 0.f;
        for (int i = 0; i < THREADS; ++i) c += vals[i];
        csum[r * CHUNKS + chunk] = c;
    }
}

__global__ __launch_bounds__(THREADS) void pick_kernel(const float* __restrict__ logits, int vocab,
                                                       const float* __restrict__ temperature,
                                                       const float* __restrict__ uniform,
                                                       const float* __restrict__ rmax, const float* __restrict__ csum,
                                                       int32_t* __restrict__ tokens) {
    __shared__ float scan[CHUNKS];
    __shared__ float vals[THREADS];
    __shared__ int chosen_chunk, chosen, last_thread;
    __shared__ float chunk_lo;
    const int r = blockIdx.x, t = threadIdx.x;
    const float temp = temperature[r];
    if (!(temp > 0.f) || tokens[r] < 0) return;     // greedy, or a row that is not finite
    if (t == 0) {
        float c = 0.f;
        for (int i = 0; i < CHUNKS; ++i) { c += csum[r * CHUNKS + i]; scan[i] = c; }
        const float target = uniform[r] * c;
        // the first chunk whose running sum passes the target; when rounding has pushed the target to the
        // total itself (u within 2^-23 of 1), the last chunk that holds any probability
        int pick = -1, last = -1;
        for (int i = 0; i < CHUNKS; ++i) {
            if (!(csum[r * CHUNKS + i] > 0.f)) continue;
            last = i;
            if (target < scan[i]) { pick = i; break; }
        }
        if (pick < 0) pick = last;
        chosen_chunk = pick;
        chunk_lo = pick > 0 ? scan[pick - 1] : 0.f;
        chosen = -1;
    }
    __syncthreads();
    if (chosen_chunk < 0) return;                   // (no chunk holds any probability: cannot happen; the argmax stays)
    const float target = uniform[r] * scan[CHUNKS - 1];
    const float* row = logits + (size_t)r * vocab;
    int cb, ce;
    chunk_range(vocab, chosen_chunk, &cb, &ce);
    const int per = (ce - cb + THREADS - 1) / THREADS;
    const int begin = min(ce, cb + t * per), end = min(ce, begin + per);
    const float inv_t = 1.0f / temp, row_max = rmax[r];
    float sum = 0.f;
    for (int i0 = begin; i0 < end; i0 += 4) {          // (four loads asked for at once; added in ascending order)
        float x[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) x[j] = row[min(i0 + j, end - 1)];
        asm volatile("" : "+v"(x[0]), "+v"(x[1]), "+v"(x[2]), "+v"(x[3]));
#pragma unroll
        for (int j = 0; j < 4; ++j)
            if (i0 + j < end) sum += expf((x[j] - row_max) * inv_t);
    }
    vals[t] = sum;
    __syncthreads();
    if (t == 0) {
        float c = chunk_lo;
        int last = -1;                              // the last thread whose tokens hold any probability
        for (int i = 0; i < THREADS; ++i) {
            if (vals[i] > 0.f) last = i;
            c += vals[i];
            vals[i] = c;
        }
        last_thread = last;
    }
    __syncthreads();
    const float lo = t ? vals[t - 1] : chunk_lo, hi = vals[t];
    // The thread whose stretch of the running sum holds the target.  The sums within the chunk are added in
    // another order than the chunk's own sum was, so the target may come to lie at or past their end by a
    // rounding: then the last thread that holds any probability takes it, and gives its last such token.
    const bool mine = target >= lo && target < hi && end > begin;
    const bool past_the_end = t == last_thread && target >= vals[THREADS - 1];
    if (mine || past_the_end) {
        float c = lo;
        int pick = -1, last = end - 1;
        for (int i = begin; i < end; ++i) {
            const float e = expf((row[i] - row_max) * inv_t);
            if (e > 0.f) last = i;
            c += e;
            if (c > target) { pick = i; break; }
        }
        chosen = pick >= 0 ? pick : last;
    }
    __syncthreads();
    if (t == 0 && chosen >= 0) tokens[r] = chosen;
}

extern "C" int mlr_sample_scratch_floats(int rows) { return rows * (2 * CHUNKS + 1); }
extern "C" int mlr_sample_scratch_ints(int rows) { return rows * 2 * CHUNKS; }

// The four passes over scratch memory scratch_f (rows * (2 CHUNKS + 1) floats) and scratch_i (rows * 2 CHUNKS
// ints), wherever it comes from.
static int launch_sample(const float* logits, int rows, int vocab, const float* temperature, const float* uniform,
                         int32_t* tokens, int32_t* status, float* scratch_f, int32_t* scratch_i, int any_sampling,
                         hipStream_t stream) {
    float* cmax = scratch_f;
    float* csum = scratch_f + (size_t)rows * CHUNKS;
    float* rmax = scratch_f + (size_t)rows * 2 * CHUNKS;
    int32_t* cidx = scratch_i;
    int32_t* cbad = scratch_i + (size_t)rows * CHUNKS;
    chunk_max_kernel<<<dim3(rows, CHUNKS), THREADS, 0, stream>>>(logits, vocab, cmax, cidx, cbad, status);
    row_max_kernel<<<rows, 64, 0, stream>>>(cmax, cidx, cbad, temperature, rmax, tokens, status);
    if (any_sampling) {
        chunk_sum_kernel<<<dim3(rows, CHUNKS), THREADS, 0, stream>>>(logits, vocab, temperature, rmax, csum);
        pick_kernel<<<rows, THREADS, 0, stream>>>(logits, vocab, temperature, uniform, rmax, csum, tokens);
    }
    return (int)hipGetLastError();
}

// scratch_f: rows * (2 CHUNKS + 1) floats; scratch_i: rows * 2 CHUNKS ints.  `any_sampling` = 0 skips
// passes 3 and 4 (every temperature <= 0).
extern "C" int mlr_sample(const float* logits, int rows, int vocab, const float* temperature,
                          const float* uniform, int32_t* tokens, int32_t* status, float* scratch_f,
                          int32_t* scratch_i, int any_sampling, hipStream_t stream) {
    if (rows <= 0) return 0;
    if (vocab <= 0) return -1;
    return launch_sample(logits, rows, vocab, temperature, uniform, tokens, status, scratch_f, scratch_i, any_sampling,
                         stream);
}

// ------------------------------------------------------------------------------------------------
// The same without workspace arguments (no_alloc.h).  `scratch` is part of this library's code object; every
// GPU that loads it holds a copy at an address of its own.  In host code the array's NAME is only a stand-in
// for the symbol, not a device address: the address on the current device is asked for once per device and
// kept, and only that pointer is ever handed to a kernel.
static_assert(CHUNKS == 64, "no_alloc.h states the scratch size for 64 chunks");
static __device__ __align__(256) unsigned char scratch[MLR_SAMPLE_STATIC_BYTES];

#define MLR_MAX_DEVICES 64
static void* g_scratch_on_device[MLR_MAX_DEVICES];        // [device index] -> address of `scratch` there, or null
static std::mutex g_scratch_lock;

static int scratch_on_current_device(unsigned char** out) {
    int device = -1;
    if (hipGetDevice(&device) != hipSuccess || device < 0 || device >= MLR_MAX_DEVICES) return MLR_SAMPLE_STATIC_NO_DEVICE;
    std::lock_guard<std::mutex> guard(g_scratch_lock);
    if (g_scratch_on_device[device] == nullptr) {
        void* address = nullptr;
        const hipError_t err = hipGetSymbolAddress(&address, HIP_SYMBOL(scratch));     // (with `device` current)
        if (err != hipSuccess || address == nullptr) {
            fprintf(stderr, "mlr_sample_static: hipGetSymbolAddress failed on device %d: %s\n", device,
                    hipGetErrorString(err));
            return MLR_SAMPLE_STATIC_NO_SYMBOL;
        }
        g_scratch_on_device[device] = address;
    }
    *out = static_cast<unsigned char*>(g_scratch_on_device[device]);
    return 0;
}

extern "C" int mlr_sample_static(const float* logits, int rows, int vocab, const float* temperature,
                                 const float* uniform, int32_t* tokens, int32_t* status, int any_sampling,
                                 hipStream_t stream) {
    if (rows > MLR_SAMPLE_STATIC_MAX_ROWS) {
        fprintf(stderr, "mlr_sample_static: %d rows exceed the %d that the static scratch memory holds\n", rows,
                MLR_SAMPLE_STATIC_MAX_ROWS);
        return MLR_SAMPLE_STATIC_TOO_MANY_ROWS;
    }
    unsigned char* base = nullptr;
    const int rc = scratch_on_current_device(&base);
    if (rc != 0) return rc;
    if (rows <= 0) return 0;                               // the set-up call: the address is known now
    if (vocab <= 0) return MLR_SAMPLE_STATIC_BAD_VOCAB;
    float* scratch_f = reinterpret_cast<float*>(base);
    int32_t* scratch_i = reinterpret_cast<int32_t*>(base + (size_t)MLR_SAMPLE_STATIC_MAX_ROWS * (2 * CHUNKS + 1) * sizeof(float));
    return launch_sample(logits, rows, vocab, temperature, uniform, tokens, status, scratch_f, scratch_i, any_sampling,
                         stream);
}
