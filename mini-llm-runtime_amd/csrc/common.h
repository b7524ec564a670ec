// Shared device helpers for the gfx950 kernels: element type of the engine (bfloat16 or
// float, chosen at compile time with -DMLR_BF16=1/0), wavefront (64 lanes) and workgroup
// reductions, 16-byte vector access.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#ifndef MLR_BF16
#error "compile with -DMLR_BF16=0 (float engine) or -DMLR_BF16=1 (bfloat16 engine)"
#endif

#if MLR_BF16
typedef __bf16 elem_t;
#define MLR_VEC 8            // elements in a 16-byte access
#else
typedef float elem_t;
#define MLR_VEC 4
#endif

#define MLR_WAVE 64

__device__ __forceinline__ float to_float(float x) { return x; }
__device__ __forceinline__ float to_float(__bf16 x) { return (float)x; }
template <class T> __device__ __forceinline__ T from_float(float x);
template <> __device__ __forceinline__ float from_float<float>(float x) { return x; }
template <> __device__ __forceinline__ __bf16 from_float<__bf16>(float x) { return (__bf16)x; }

struct alignas(16) vec16 { uint32_t w[4]; };

// Load MLR_VEC consecutive elements (16 bytes, 16-byte aligned) as floats.
__device__ __forceinline__ void load_vec(const elem_t* p, float* out) {
    vec16 v = *reinterpret_cast<const vec16*>(p);
#if MLR_BF16
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        out[2 * i] = __uint_as_float(v.w[i] << 16);
        out[2 * i + 1] = __uint_as_float(v.w[i] & 0xffff0000u);
    }
#else
#pragma unroll
    for (int i = 0; i < 4; ++i) out[i] = __uint_as_float(v.w[i]);
#endif
}

__device__ __forceinline__ void store_vec(elem_t* p, const float* in) {
    alignas(16) elem_t tmp[MLR_VEC];
#pragma unroll
    for (int i = 0; i < MLR_VEC; ++i) tmp[i] = from_float<elem_t>(in[i]);
    *reinterpret_cast<vec16*>(p) = *reinterpret_cast<const vec16*>(tmp);
}

// The same bits whatever fused operations the compiler would choose: a token's key is written by one of three
// kernels (the general and the vector kernel of rope_kv.hip, the decode merge of attention.hip) and should not
// depend on which.  An empty asm makes an intermediate opaque, so that a product cannot be drawn into the
// sum that follows it; the fused multiply-adds that are meant are written out.
__device__ __forceinline__ float opaque(float v) {
    asm("" : "+v"(v));
    return v;
}
// (x, y) = (a, b) turned by the angle with cosine c and sine s
__device__ __forceinline__ float turn_x(float a, float b, float c, float s) { return __builtin_fmaf(a, c, -opaque(b * s)); }
__device__ __forceinline__ float turn_y(float a, float b, float c, float s) { return __builtin_fmaf(a, s, opaque(b * c)); }
// a^2 + b^2, to be added to a running sum
__device__ __forceinline__ float squares(float a, float b) { return opaque(__builtin_fmaf(a, a, opaque(b * b))); }

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, MLR_WAVE);
    return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, MLR_WAVE));
    return v;
}

// Sum over a workgroup of up to 1024 threads (a multiple of 64); every thread gets the
// result.  `scratch` holds at least 16 floats of LDS.  The order of the additions depends on
// the workgroup size only.
__device__ __forceinline__ float block_sum(float v, float* scratch) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, waves = (blockDim.x + 63) >> 6;
    v = wave_sum(v);
    __syncthreads();
    if (lane == 0) scratch[wave] = v;
    __syncthreads();
    float total = 0.f;
    for (int i = 0; i < waves; ++i) total += scratch[i];
    return total;
}
