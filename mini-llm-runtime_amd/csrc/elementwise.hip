// Row-wise kernels of the decoder: embedding gather, residual add + RMSNorm (fused),
// SiLU(gate) * up.  The residual stream is float in both engines; norm sums, the
// activation and the residual sum are computed in 32-bit.
#include "common.h"

// h[m, :] = float(table[ids[m], :]).  An id outside [0, vocab) gives a row of NaN
// (the host refuses such a batch before anything runs).
__global__ void embed_gather_kernel(const int32_t* __restrict__ ids, const elem_t* __restrict__ table,
                                    float* __restrict__ h, int width, int vocab) {
    const int m = blockIdx.x;
    const int id = ids[m];
    float* out = h + (size_t)m * width;
    if (id < 0 || id >= vocab) {
        for (int i = threadIdx.x; i < width; i += blockDim.x) out[i] = __int_as_float(0x7fc00000);
        return;
    }
    const elem_t* row = table + (size_t)id * width;
    for (int i = threadIdx.x; i < width; i += blockDim.x) out[i] = to_float(row[i]);
}

__device__ __forceinline__ float block_max(float v, float* scratch) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, waves = (blockDim.x + 63) >> 6;
    v = wave_max(v);
    __syncthreads();
    if (lane == 0) scratch[wave] = v;
    __syncthreads();
    float total = scratch[0];
    for (int i = 1; i < waves; ++i) total = fmaxf(total, scratch[i]);
    return total;
}

// A row whose sum of squares does not fit 32 bits (elements beyond about 1e19) or is no number: the
// reference's way of norming (src/minillm/cuda/ops.cu:87-126), the row divided by its largest element before
// it is squared, and eps scaled alike: largest = max(max |x|, sqrt(eps)), den = sqrt(mean((x / largest)^2) +
// eps / largest^2), y = ((x / largest) / den) * w; a row with an infinity or a NaN comes out as NaN.  The usual
// row never gets here, so it keeps its one pass and its bits.  x = hrow + drow (drow: what is still to be
// added, or null).  WAVE: one wavefront serves the row, else the whole workgroup (every thread of it must
// call, `scratch` holds 16 floats of LDS).
template <bool WAVE>
__device__ void norm_row_rescaled(const float* hrow, const elem_t* drow, const float* __restrict__ weight,
                                  elem_t* __restrict__ orow, int width, float eps, float* scratch) {
    __threadfence_block();                     // (the row may have been written back by other lanes just now)
    const int t = WAVE ? (int)(threadIdx.x & 63) : (int)threadIdx.x, step = WAVE ? 64 : (int)blockDim.x;
    float largest = 0.f;
    for (int i = t; i < width; i += step) {
        const float x = hrow[i] + (drow ? to_float(drow[i]) : 0.f);
        largest = fmaxf(largest, isfinite(x) ? fabsf(x) : INFINITY);
    }
    largest = WAVE ? wave_max(largest) : block_max(largest, scratch);
    largest = fmaxf(largest, sqrtf(eps));
    if (!isfinite(largest)) {
        for (int i = t; i < width; i += step) orow[i] = from_float<elem_t>(__int_as_float(0x7fc00000));
        return;
    }
    float sum = 0.f;
    for (int i = t; i < width; i += step) {
        const float scaled = (hrow[i] + (drow ? to_float(drow[i]) : 0.f)) / largest;
        sum += scaled * scaled;
    }
    sum = WAVE ? wave_sum(sum) : block_sum(sum, scratch);
    const float den = sqrtf(sum / (float)width + (eps / largest) / largest);
    for (int i = t; i < width; i += step) {
        const float x = hrow[i] + (drow ? to_float(drow[i]) : 0.f);
        orow[i] = from_float<elem_t>(((x / largest) / den) * weight[i]);
    }
}

// For output row r: src = rows ? rows[r] : r;  x = h[src] + (delta ? delta[src] : 0);
// if write_h: h[src] = x;  out[r] = (x * rsqrt(mean(x^2) + eps)) * weight.
// One workgroup per row; the sum of squares is taken over the row in a fixed order.
__global__ void add_rmsnorm_kernel(float* __restrict__ h, const elem_t* __restrict__ delta,
                                   const float* __restrict__ weight, elem_t* __restrict__ out,
                                   const int32_t* __restrict__ rows, int width, float eps,
                                   int write_h) {
    __shared__ float scratch[16];
    const int r = blockIdx.x;
    const size_t src = rows ? (size_t)rows[r] : (size_t)r;
    float* hrow = h + src * width;
    const elem_t* drow = delta ? delta + src * width : nullptr;
    float sum = 0.f;
    for (int i = threadIdx.x; i < width; i += blockDim.x) {
        float x = hrow[i];
        if (drow) {
            x += to_float(drow[i]);
            if (write_h) hrow[i] = x;
        }
        sum += x * x;
    }
    sum = block_sum(sum, scratch);
    elem_t* orow = out + (size_t)r * width;
    if (!isfinite(sum)) {                      // (the same in every thread of the workgroup)
        norm_row_rescaled<false>(hrow, (drow && !write_h) ? drow : nullptr, weight, orow, width, eps, scratch);
        return;
    }
    const float scale = 1.0f / sqrtf(sum / (float)width + eps);
    for (int i = threadIdx.x; i < width; i += blockDim.x) {
        float x = hrow[i];
        if (drow && !write_h) x += to_float(drow[i]);
        orow[i] = from_float<elem_t>((x * scale) * weight[i]);
    }
}

// One workgroup per row as above, 16 bytes per thread and access (width a multiple of MLR_VEC): for few
// rows of the bfloat16 engine, where the scalar kernel's latency would show.
__global__ __launch_bounds__(256) void add_rmsnorm_row_vec_kernel(float* __restrict__ h, const elem_t* __restrict__ delta,
                                                                  const float* __restrict__ weight,
                                                                  elem_t* __restrict__ out, const int32_t* __restrict__ rows,
                                                                  int width, float eps, int write_h) {
    __shared__ float scratch[16];
    const int r = blockIdx.x;
    const size_t src = rows ? (size_t)rows[r] : (size_t)r;
    float* hrow = h + src * width;
    const elem_t* drow = delta ? delta + src * width : nullptr;
    float sum = 0.f;
    for (int c = threadIdx.x * MLR_VEC; c < width; c += 256 * MLR_VEC) {
        float x[MLR_VEC];
#pragma unroll
        for (int e = 0; e < MLR_VEC; e += 4) {
            const float4 v = *reinterpret_cast<const float4*>(hrow + c + e);
            x[e] = v.x; x[e + 1] = v.y; x[e + 2] = v.z; x[e + 3] = v.w;
        }
        if (drow) {
            float dv[MLR_VEC];
            load_vec(drow + c, dv);
#pragma unroll
            for (int e = 0; e < MLR_VEC; ++e) x[e] += dv[e];
            if (write_h) {
#pragma unroll
                for (int e = 0; e < MLR_VEC; e += 4)
                    *reinterpret_cast<float4*>(hrow + c + e) = make_float4(x[e], x[e + 1], x[e + 2], x[e + 3]);
            }
        }
#pragma unroll
        for (int e = 0; e < MLR_VEC; ++e) sum += x[e] * x[e];
    }
    sum = block_sum(sum, scratch);
    elem_t* orow = out + (size_t)r * width;
    if (!isfinite(sum)) {
        norm_row_rescaled<false>(hrow, (drow && !write_h) ? drow : nullptr, weight, orow, width, eps, scratch);
        return;
    }
    const float scale = 1.0f / sqrtf(sum / (float)width + eps);
    for (int c = threadIdx.x * MLR_VEC; c < width; c += 256 * MLR_VEC) {
        float x[MLR_VEC], y[MLR_VEC];
#pragma unroll
        for (int e = 0; e < MLR_VEC; e += 4) {
            const float4 v = *reinterpret_cast<const float4*>(hrow + c + e);
            x[e] = v.x; x[e + 1] = v.y; x[e + 2] = v.z; x[e + 3] = v.w;
        }
        if (drow && !write_h) {
            float dv[MLR_VEC];
            load_vec(drow + c, dv);
#pragma unroll
            for (int e = 0; e < MLR_VEC; ++e) x[e] += dv[e];
        }
#pragma unroll
        for (int e = 0; e < MLR_VEC; e += 4) {
            const float4 w = *reinterpret_cast<const float4*>(weight + c + e);
            y[e] = (x[e] * scale) * w.x;
            y[e + 1] = (x[e + 1] * scale) * w.y;
            y[e + 2] = (x[e + 2] * scale) * w.z;
            y[e + 3] = (x[e + 3] * scale) * w.w;
        }
        store_vec(orow + c, y);
    }
}

// The same for widths that are a multiple of 8 (bfloat16) or 4 (float), 16 bytes per lane and access:
// one wavefront per row, four rows per workgroup, the row kept in registers between the two passes
// when it fits (width <= 64 * MLR_VEC * ROW_REGS), else re-read.
#define ROW_REGS 4
__global__ __launch_bounds__(256) void add_rmsnorm_vec_kernel(float* __restrict__ h, const elem_t* __restrict__ delta,
                                                              const float* __restrict__ weight,
                                                              elem_t* __restrict__ out, const int32_t* __restrict__ rows,
                                                              int n_out, int width, float eps, int write_h) {
    const int lane = threadIdx.x & 63;
    const int r = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (r >= n_out) return;
    const size_t src = rows ? (size_t)rows[r] : (size_t)r;
    float* hrow = h + src * width;
    const elem_t* drow = delta ? delta + src * width : nullptr;
    float x[ROW_REGS][MLR_VEC];
    float sum = 0.f;
#pragma unroll
    for (int i = 0; i < ROW_REGS; ++i) {
        const int c = (lane + 64 * i) * MLR_VEC;
        if (c < width) {
#pragma unroll
            for (int e = 0; e < MLR_VEC; e += 4) {
                const float4 v = *reinterpret_cast<const float4*>(hrow + c + e);
                x[i][e] = v.x; x[i][e + 1] = v.y; x[i][e + 2] = v.z; x[i][e + 3] = v.w;
            }
            if (drow) {
                float dv[MLR_VEC];
                load_vec(drow + c, dv);
#pragma unroll
                for (int e = 0; e < MLR_VEC; ++e) x[i][e] += dv[e];
                if (write_h) {
#pragma unroll
                    for (int e = 0; e < MLR_VEC; e += 4)
                        *reinterpret_cast<float4*>(hrow + c + e) = make_float4(x[i][e], x[i][e + 1], x[i][e + 2], x[i][e + 3]);
                }
            }
#pragma unroll
            for (int e = 0; e < MLR_VEC; ++e) sum += x[i][e] * x[i][e];
        }
    }
    sum = wave_sum(sum);
    elem_t* orow = out + (size_t)r * width;
    if (!isfinite(sum)) {                      // (the same in every lane of the wavefront, which serves this row alone)
        norm_row_rescaled<true>(hrow, (drow && !write_h) ? drow : nullptr, weight, orow, width, eps, nullptr);
        return;
    }
    const float scale = 1.0f / sqrtf(sum / (float)width + eps);
#pragma unroll
    for (int i = 0; i < ROW_REGS; ++i) {
        const int c = (lane + 64 * i) * MLR_VEC;
        if (c < width) {
            float y[MLR_VEC];
#pragma unroll
            for (int e = 0; e < MLR_VEC; e += 4) {
                const float4 w = *reinterpret_cast<const float4*>(weight + c + e);
                y[e] = (x[i][e] * scale) * w.x;
                y[e + 1] = (x[i][e + 1] * scale) * w.y;
                y[e + 2] = (x[i][e + 2] * scale) * w.z;
                y[e + 3] = (x[i][e + 3] * scale) * w.w;
            }
            store_vec(orow + c, y);
        }
    }
}

// h[m, :] += delta[m, :] (the last residual sum when nothing is normed afterwards).
__global__ void residual_add_kernel(float* __restrict__ h, const elem_t* __restrict__ delta, size_t count) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < count;
         i += (size_t)gridDim.x * blockDim.x) {
        h[i] += to_float(delta[i]);
    }
}

// The same, 16 bytes per lane and access, for inter % MLR_VEC == 0.
__global__ void silu_mul_vec_kernel(const elem_t* __restrict__ gate_up, elem_t* __restrict__ act, int rows, int inter) {
    const int per_row = inter / MLR_VEC;
    const size_t total = (size_t)rows * per_row;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (size_t)gridDim.x * blockDim.x) {
        const size_t m = i / per_row, f = (i % per_row) * MLR_VEC;
        float g[MLR_VEC], u[MLR_VEC], y[MLR_VEC];
        load_vec(gate_up + m * 2 * inter + f, g);
        load_vec(gate_up + m * 2 * inter + inter + f, u);
#pragma unroll
        for (int e = 0; e < MLR_VEC; ++e) y[e] = (g[e] / (1.0f + expf(-g[e]))) * u[e];
        store_vec(act + m * inter + f, y);
    }
}

// act[m, f] = silu(gate_up[m, f]) * gate_up[m, inter + f]; silu(g) = g / (1 + exp(-g)).
__global__ void silu_mul_kernel(const elem_t* __restrict__ gate_up, elem_t* __restrict__ act,
                                int rows, int inter) {
    const size_t total = (size_t)rows * inter;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total;
         i += (size_t)gridDim.x * blockDim.x) {
        const size_t m = i / inter, f = i % inter;
        const float g = to_float(gate_up[m * 2 * inter + f]);
        const float u = to_float(gate_up[m * 2 * inter + inter + f]);
        act[i] = from_float<elem_t>((g / (1.0f + expf(-g))) * u);
    }
}

// The first half of an RMSNorm whose scale is applied by the projection that follows (few rows): x = h + delta
// (delta may be null; written back to h when write_h), out = elem(x * weight) WITHOUT the scale, and the row's
// sum of squares ss[r] (one "partial" sum a row).  One workgroup per row, sums in a fixed order.
__global__ void rows_prenorm_kernel(float* __restrict__ h, const elem_t* __restrict__ delta,
                                    const float* __restrict__ weight, elem_t* __restrict__ out,
                                    float* __restrict__ ss, int width) {
    __shared__ float scratch[16];
    const int r = blockIdx.x;
    float* hrow = h + (size_t)r * width;
    const elem_t* drow = delta ? delta + (size_t)r * width : nullptr;
    elem_t* orow = out + (size_t)r * width;
    float sum = 0.f;
    for (int i = threadIdx.x; i < width; i += blockDim.x) {
        float x = hrow[i];
        if (drow) {
            x += to_float(drow[i]);
            hrow[i] = x;
        }
        sum += x * x;
        orow[i] = from_float<elem_t>(x * weight[i]);
    }
    sum = block_sum(sum, scratch);
    if (threadIdx.x == 0) ss[r] = sum;
}

// The check of the hidden state (a debug mode; the reference runs the like after every layer and poisons
// its runtime, src/minillm/cuda/layer.cpp:71, src/minillm/cuda/ops.cu:29-43).  status[0] collects bits
// (1: a NaN, 2: an infinity), status[1] the smallest (layer << 20 | row) at which one was seen.
__global__ void status_reset_kernel(int32_t* __restrict__ status) {
    if (threadIdx.x == 0) {
        status[0] = 0;
        status[1] = 0x7fffffff;
    }
}

// One workgroup per row of x = h + delta (delta may be null): which kinds of non-finite values it holds.
__global__ void finite_check_kernel(const float* __restrict__ h, const elem_t* __restrict__ delta, int width, int layer,
                                    int32_t* __restrict__ status) {
    const int r = blockIdx.x;
    const float* hrow = h + (size_t)r * width;
    const elem_t* drow = delta ? delta + (size_t)r * width : nullptr;
    int bits = 0;
    for (int i = threadIdx.x; i < width; i += blockDim.x) {
        const float x = hrow[i] + (drow ? to_float(drow[i]) : 0.f);
        const uint32_t u = __float_as_uint(x) & 0x7fffffffu;
        if (u > 0x7f800000u) bits |= 1;
        else if (u == 0x7f800000u) bits |= 2;
    }
    if (__any(bits != 0)) {                     // (rare: one atomic per wavefront that saw something)
        for (int off = 32; off > 0; off >>= 1) bits |= __shfl_xor(bits, off, MLR_WAVE);
        if ((threadIdx.x & 63) == 0) {
            atomicOr(&status[0], bits);
            atomicMin(&status[1], (layer << 20) | (r < (1 << 20) ? r : (1 << 20) - 1));
        }
    }
}

static int grid_for(size_t count, int block) {
    size_t g = (count + block - 1) / block;
    return (int)(g > 65535 ? 65535 : (g == 0 ? 1 : g));
}

extern "C" {

int mlr_embed_gather(const int32_t* ids, const void* table, float* h, int rows, int width, int vocab,
                     hipStream_t stream) {
    if (rows <= 0) return 0;
    embed_gather_kernel<<<rows, 256, 0, stream>>>(ids, (const elem_t*)table, h, width, vocab);
    return (int)hipGetLastError();
}

int mlr_add_rmsnorm(float* h, const void* delta, const float* weight, void* out, const int32_t* rows,
                    int n_out, int width, float eps, int write_h, hipStream_t stream) {
    if (n_out <= 0) return 0;
    // (the float engine keeps its one order of additions for every batch size)
    if (MLR_BF16 && width % MLR_VEC == 0 && width <= 64 * MLR_VEC * ROW_REGS && n_out >= 64) {
        add_rmsnorm_vec_kernel<<<(n_out + 3) / 4, 256, 0, stream>>>(h, (const elem_t*)delta, weight, (elem_t*)out,
                                                                     rows, n_out, width, eps, write_h);
        return (int)hipGetLastError();
    }
    if (MLR_BF16 && width % MLR_VEC == 0) {
        add_rmsnorm_row_vec_kernel<<<n_out, 256, 0, stream>>>(h, (const elem_t*)delta, weight, (elem_t*)out, rows,
                                                              width, eps, write_h);
        return (int)hipGetLastError();
    }
    add_rmsnorm_kernel<<<n_out, 256, 0, stream>>>(h, (const elem_t*)delta, weight, (elem_t*)out, rows,
                                                  width, eps, write_h);
    return (int)hipGetLastError();
}

int mlr_rows_prenorm(float* h, const void* delta, const float* weight, void* out, float* ss, int rows, int width,
                     hipStream_t stream) {
    if (rows <= 0) return 0;
    rows_prenorm_kernel<<<rows, 256, 0, stream>>>(h, (const elem_t*)delta, weight, (elem_t*)out, ss, width);
    return (int)hipGetLastError();
}

int mlr_status_reset(int32_t* status, hipStream_t stream) {
    status_reset_kernel<<<1, 64, 0, stream>>>(status);
    return (int)hipGetLastError();
}

int mlr_finite_check(const float* h, const void* delta, int rows, int width, int layer, int32_t* status,
                     hipStream_t stream) {
    if (rows <= 0) return 0;
    if (layer < 0 || layer >= 2047) return -1;
    finite_check_kernel<<<rows, 256, 0, stream>>>(h, (const elem_t*)delta, width, layer, status);
    return (int)hipGetLastError();
}

int mlr_residual_add(float* h, const void* delta, size_t count, hipStream_t stream) {
    if (count == 0) return 0;
    residual_add_kernel<<<grid_for(count, 256), 256, 0, stream>>>(h, (const elem_t*)delta, count);
    return (int)hipGetLastError();
}

int mlr_silu_mul(const void* gate_up, void* act, int rows, int inter, hipStream_t stream) {
    if (rows <= 0) return 0;
    if (inter % MLR_VEC == 0) {
        silu_mul_vec_kernel<<<grid_for((size_t)rows * (inter / MLR_VEC), 256), 256, 0, stream>>>(
            (const elem_t*)gate_up, (elem_t*)act, rows, inter);
        return (int)hipGetLastError();
    }
    silu_mul_kernel<<<grid_for((size_t)rows * inter, 256), 256, 0, stream>>>(
        (const elem_t*)gate_up, (elem_t*)act, rows, inter);
    return (int)hipGetLastError();
}

}  // extern "C"
