// Per-head RMSNorm of q and k, split-half rotation by position, and the write of k and v
// into their pages of the cache: one kernel, one pass over the projection's output.
//
// Cache layout of one layer: keys pages[num_pages][kv_heads][page_size][head_dim], values transposed
// pages[num_pages][kv_heads][head_dim][page_size]; token position p of the request in slot s lies in
// page block_table[s][p / page_size] at row (values: column) p % page_size.  Norm sums and the rotation are computed in 32-bit; cos/sin come from a
// float table [max_positions][head_dim] (first half cos, second half sin).
#include "common.h"

#define MAX_PAIRS 4   // head_dim / 2 <= 64 * MAX_PAIRS

__global__ void qk_norm_rope_kv_kernel(
    const elem_t* __restrict__ qkv, int ld, elem_t* __restrict__ q_out,
    elem_t* __restrict__ k_pages, elem_t* __restrict__ v_pages,
    const int32_t* __restrict__ block_table, int max_blocks,
    const int32_t* __restrict__ slots, const int32_t* __restrict__ positions,
    const float* __restrict__ q_norm_w, const float* __restrict__ k_norm_w, float eps,
    const float* __restrict__ rope, int q_heads, int kv_heads, int head_dim, int page_size,
    int write_cache) {
    const int m = blockIdx.x;
    const int lane = threadIdx.x & 63, waves = gridDim.y * (blockDim.x >> 6);
    const int wave = blockIdx.y * (blockDim.x >> 6) + (threadIdx.x >> 6);       // heads are dealt out to these
    const int half = head_dim >> 1;
    const int pos = positions[m];
    const int slot = slots[m];
    const elem_t* row = qkv + (size_t)m * ld;
    const float* cs = rope ? rope + (size_t)pos * head_dim : nullptr;

    size_t cache_row = 0, cache_page = 0;
    bool cache_ok = false;
    if (write_cache) {
        const int page = block_table[(size_t)slot * max_blocks + pos / page_size];
        cache_ok = page >= 0;
        cache_page = (size_t)(page < 0 ? 0 : page) * kv_heads;
        cache_row = cache_page * page_size + (pos % page_size);
    }

    const int total = q_heads + 2 * kv_heads;
    for (int head = wave; head < total; head += waves) {
        const elem_t* src = row + (size_t)head * head_dim;
        if (head >= q_heads + kv_heads) {            // a value head: copy into its page
            if (cache_ok) {
                const int kvh = head - q_heads - kv_heads;
                elem_t* dst = v_pages + (cache_page + kvh) * head_dim * page_size + (pos % page_size);
                for (int d = lane; d < head_dim; d += 64) dst[(size_t)d * page_size] = src[d];
            }
            continue;
        }
        const bool is_q = head < q_heads;
        const float* w = is_q ? q_norm_w : k_norm_w;
        float a[MAX_PAIRS], b[MAX_PAIRS];
        float sum = 0.f;
#pragma unroll
        for (int i = 0; i < MAX_PAIRS; ++i) {
            const int j = lane + 64 * i;
            a[i] = b[i] = 0.f;
            if (j < half) {
                a[i] = to_float(src[j]);
                b[i] = to_float(src[j + half]);
                sum += a[i] * a[i] + b[i] * b[i];
            }
        }
        if (w) {
            sum = wave_sum(sum);
            const float scale = 1.0f / sqrtf(sum / (float)head_dim + eps);
#pragma unroll
            for (int i = 0; i < MAX_PAIRS; ++i) {
                const int j = lane + 64 * i;
                if (j < half) {
                    a[i] = (a[i] * scale) * w[j];
                    b[i] = (b[i] * scale) * w[j + half];
                }
            }
        }
        elem_t* dst;
        if (is_q) {
            dst = q_out + ((size_t)m * q_heads + head) * head_dim;
        } else {
            if (!cache_ok) continue;
            dst = k_pages + (cache_row + (size_t)(head - q_heads) * page_size) * head_dim;
        }
#pragma unroll
        for (int i = 0; i < MAX_PAIRS; ++i) {
            const int j = lane + 64 * i;
            if (j < half) {
                float x = a[i], y = b[i];
                if (cs) {
                    const float c = cs[j], s = cs[j + half];
                    x = a[i] * c - b[i] * s;
                    y = a[i] * s + b[i] * c;
                }
                dst[j] = from_float<elem_t>(x);
                dst[j + half] = from_float<elem_t>(y);
            }
        }
    }
}

extern "C" int mlr_qk_norm_rope_kv(
    const void* qkv, int ld, void* q_out, void* k_pages, void* v_pages, const int32_t* block_table,
    int max_blocks, const int32_t* slots, const int32_t* positions, const float* q_norm_w,
    const float* k_norm_w, float eps, const float* rope, int rows, int q_heads, int kv_heads,
    int head_dim, int page_size, int write_cache, hipStream_t stream) {
    if (rows <= 0) return 0;
    if (head_dim % 2 != 0 || head_dim / 2 > 64 * MAX_PAIRS) return -1;
    // few rows: spread a row's heads over several workgroups (a wavefront per head)
    const int total_heads = q_heads + 2 * kv_heads;
    int chunks = 1;
    if (rows < 512) chunks = (total_heads + 3) / 4;
    if (chunks > 64) chunks = 64;
    qk_norm_rope_kv_kernel<<<dim3(rows, chunks), 256, 0, stream>>>(
        (const elem_t*)qkv, ld, (elem_t*)q_out, (elem_t*)k_pages, (elem_t*)v_pages, block_table,
        max_blocks, slots, positions, q_norm_w, k_norm_w, eps, rope, q_heads, kv_heads, head_dim,
        page_size, write_cache);
    return (int)hipGetLastError();
}
