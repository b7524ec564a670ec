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
    const float scale = 1.0f / sqrtf(sum / (float)width + eps);
    elem_t* orow = out + (size_t)r * width;
    for (int i = threadIdx.x; i < width; i += blockDim.x) {
        float x = hrow[i];
        if (drow && !write_h) x += to_float(drow[i]);
        orow[i] = from_float<elem_t>((x * scale) * weight[i]);
    }
}

// h[m, :] += delta[m, :] (the last residual sum when nothing is normed afterwards).
__global__ void residual_add_kernel(float* __restrict__ h, const elem_t* __restrict__ delta, size_t count) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < count;
         i += (size_t)gridDim.x * blockDim.x) {
        h[i] += to_float(delta[i]);
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
    add_rmsnorm_kernel<<<n_out, 256, 0, stream>>>(h, (const elem_t*)delta, weight, (elem_t*)out, rows,
                                                  width, eps, write_h);
    return (int)hipGetLastError();
}

int mlr_residual_add(float* h, const void* delta, size_t count, hipStream_t stream) {
    if (count == 0) return 0;
    residual_add_kernel<<<grid_for(count, 256), 256, 0, stream>>>(h, (const elem_t*)delta, count);
    return (int)hipGetLastError();
}

int mlr_silu_mul(const void* gate_up, void* act, int rows, int inter, hipStream_t stream) {
    if (rows <= 0) return 0;
    silu_mul_kernel<<<grid_for((size_t)rows * inter, 256), 256, 0, stream>>>(
        (const elem_t*)gate_up, (elem_t*)act, rows, inter);
    return (int)hipGetLastError();
}

}  // extern "C"
