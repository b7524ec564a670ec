// Per-head RMSNorm of q and k, rotation by position, and the write of k and v into their pages
// of the cache: one kernel, one pass over the projection's output.
//
// Cache layout of one layer: keys pages[num_pages][kv_heads][page_size][head_dim], values transposed
// pages[num_pages][kv_heads][head_dim][page_size]; token position p of the request in slot s lies in
// page block_table[s][p / page_size] at row (values: column) p % page_size.  Norm sums and the rotation are
// computed in 32-bit.
//
// What is rotated is the position part's decision, not this kernel's: the first rot_dim channels of a head
// (even, <= head_dim; the rest pass through unrotated), in pairs (j, j + rot_dim / 2) ("split-half") or
// (2 j, 2 j + 1) ("interleaved"); pair j turns by the angle whose cosine is table[p][j] and whose sine is
// table[p][rot_dim / 2 + j], table being float [max_positions][rot_dim].  The general kernel takes any of
// these; the vector kernel for many rows takes the whole head in split-half pairs.
#include "common.h"

#define MAX_PAIRS 4   // head_dim / 2 <= 64 * MAX_PAIRS

__global__ void qk_norm_rope_kv_kernel(
    const elem_t* __restrict__ qkv, int ld, elem_t* __restrict__ q_out,
    elem_t* __restrict__ k_pages, elem_t* __restrict__ v_pages,
    const int32_t* __restrict__ block_table, int max_blocks,
    const int32_t* __restrict__ slots, const int32_t* __restrict__ positions,
    const float* __restrict__ q_norm_w, const float* __restrict__ k_norm_w, float eps,
    const float* __restrict__ rope, int q_heads, int kv_heads, int head_dim, int page_size,
    int write_cache, int rot_dim, int interleaved) {
    const int m = blockIdx.x;
    const int lane = threadIdx.x & 63, waves = gridDim.y * (blockDim.x >> 6);
    const int wave = blockIdx.y * (blockDim.x >> 6) + (threadIdx.x >> 6);       // heads are dealt out to these
    const int half = head_dim >> 1, rot_half = rot_dim >> 1;
    const int pos = positions[m];
    const int slot = slots[m];
    const elem_t* row = qkv + (size_t)m * ld;
    const float* cs = rope ? rope + (size_t)pos * rot_dim : nullptr;
    // pair j of a head: channels (ia, ib); rotated when j < rot_half (split-half) or 2 j < rot_dim (interleaved)
    auto pair_of = [&](int j, int& ia, int& ib, bool& turned) {
        if (interleaved) {
            ia = 2 * j;
            ib = 2 * j + 1;
            turned = 2 * j < rot_dim;
        } else if (j < rot_half) {
            ia = j;
            ib = j + rot_half;
            turned = true;
        } else {
            ia = rot_dim + 2 * (j - rot_half);
            ib = ia + 1;
            turned = false;
        }
    };

    size_t cache_row = 0, cache_page = 0;
    bool cache_ok = false;
    if (write_cache) {
        // (a position beyond the request's row of the table has no page, like an entry of -1)
        const int block = pos / page_size;
        const int page = block < max_blocks ? block_table[(size_t)slot * max_blocks + block] : -1;
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
                int ia, ib;
                bool turned;
                pair_of(j, ia, ib, turned);
                a[i] = to_float(src[ia]);
                b[i] = to_float(src[ib]);
                sum += squares(a[i], b[i]);
            }
        }
        if (w) {
            sum = wave_sum(sum);
            const float scale = 1.0f / sqrtf(sum / (float)head_dim + eps);
#pragma unroll
            for (int i = 0; i < MAX_PAIRS; ++i) {
                const int j = lane + 64 * i;
                if (j < half) {
                    int ia, ib;
                    bool turned;
                    pair_of(j, ia, ib, turned);
                    a[i] = (a[i] * scale) * w[ia];
                    b[i] = (b[i] * scale) * w[ib];
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
                int ia, ib;
                bool turned;
                pair_of(j, ia, ib, turned);
                float x = a[i], y = b[i];
                if (cs && turned) {
                    const float c = cs[j], s = cs[j + rot_half];
                    x = turn_x(a[i], b[i], c, s);
                    y = turn_y(a[i], b[i], c, s);
                }
                dst[ia] = from_float<elem_t>(x);
                dst[ib] = from_float<elem_t>(y);
            }
        }
    }
}

#if MLR_BF16
// The same for many rows of the bfloat16 engine and head sizes 16, 32, 64, 128, 256: head_dim / 16 lanes
// serve a head, each with eight consecutive channels of the first half and their partners of the second
// half (16-byte accesses); a wavefront serves 64 / (head_dim / 16) heads at once.
typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;

// Values into their transposed pages, sixteen batch rows at a time: the rows' values of one kv head go
// through LDS so that a thread ends up with eight consecutive rows of one channel.  When those rows are
// eight consecutive positions of one request inside one page (the usual case in a prompt portion that
// starts at a multiple of eight) they are one 16-byte store; otherwise element by element.  Done by extra
// workgroups of the kernel below (the two jobs share nothing; one launch instead of two).
__device__ __forceinline__ void write_values_transposed(
    const __bf16* __restrict__ qkv, int ld, __bf16* __restrict__ v_pages, const int32_t* __restrict__ block_table,
    int max_blocks, const int32_t* __restrict__ slots, const int32_t* __restrict__ positions, int rows, int q_heads,
    int kv_heads, int head_dim, int page_size, int r0, int kvh) {
    extern __shared__ __attribute__((aligned(16))) __bf16 tile[];   // [16 rows][head_dim + 8]
    __shared__ long long row_base[16];                     // element offset of (page, kv head) for each row, or -1
    __shared__ int row_in_page[16];
    const int pitch = head_dim + 8;
    const int chunks = head_dim / 8;                       // 16-byte chunks per row
    for (int i = threadIdx.x; i < 16 * chunks; i += 256) {
        const int r = i / chunks, c = i % chunks;
        bf16x8 v = {0, 0, 0, 0, 0, 0, 0, 0};
        if (r0 + r < rows)
            v = *reinterpret_cast<const bf16x8*>(qkv + (size_t)(r0 + r) * ld + (size_t)(q_heads + kv_heads + kvh) * head_dim + 8 * c);
        *reinterpret_cast<bf16x8*>(&tile[r * pitch + 8 * c]) = v;
    }
    if (threadIdx.x < 16) {
        const int r = r0 + threadIdx.x;
        long long base = -1;
        int in_page = 0;
        if (r < rows) {
            const int pos = positions[r];
            const int block = pos / page_size;
            const int page = block < max_blocks ? block_table[(size_t)slots[r] * max_blocks + block] : -1;
            if (page >= 0) base = ((long long)page * kv_heads + kvh) * head_dim * page_size;
            in_page = pos % page_size;
        }
        row_base[threadIdx.x] = base;
        row_in_page[threadIdx.x] = in_page;
    }
    __syncthreads();
    // thread -> (channel d, rows 8 h .. 8 h + 7)
    for (int i = threadIdx.x; i < 2 * head_dim; i += 256) {
        const int d = i % head_dim, h = i / head_dim;
        const long long base = row_base[8 * h];
        const int in_page = row_in_page[8 * h];
        bool run = base >= 0 && (in_page & 7) == 0;
#pragma unroll
        for (int e = 1; e < 8; ++e) run = run && row_base[8 * h + e] == base && row_in_page[8 * h + e] == in_page + e;
        if (run) {
            bf16x8 v;
#pragma unroll
            for (int e = 0; e < 8; ++e) v[e] = tile[(8 * h + e) * pitch + d];
            *reinterpret_cast<bf16x8*>(v_pages + base + (long long)d * page_size + in_page) = v;
        } else {
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const long long b = row_base[8 * h + e];
                if (b >= 0) v_pages[b + (long long)d * page_size + row_in_page[8 * h + e]] = tile[(8 * h + e) * pitch + d];
            }
        }
    }
}

// Every load is asked for as early as its address is known and none sits behind a branch, so a thread
// waits for memory twice (the row's position and its own channels; then the page id and the rotation row)
// instead of once per table.
template <bool HAS_NORM, bool HAS_ROPE>
__global__ __launch_bounds__(256) void qk_norm_rope_kv_vec_kernel(
    const __bf16* __restrict__ qkv, int ld, __bf16* __restrict__ q_out, __bf16* __restrict__ k_pages,
    __bf16* __restrict__ v_pages, const int32_t* __restrict__ block_table, int max_blocks,
    const int32_t* __restrict__ slots, const int32_t* __restrict__ positions, const float* __restrict__ q_norm_w,
    const float* __restrict__ k_norm_w, float eps, const float* __restrict__ rope, int q_heads, int kv_heads,
    int head_dim, int page_size, int write_cache, int skip_values, int rows) {
    if (blockIdx.x >= (unsigned)rows) {                    // a workgroup beyond the rows: sixteen rows' values of one kv head
        if (blockIdx.y != 0) return;
        const int job = blockIdx.x - rows;
        write_values_transposed(qkv, ld, v_pages, block_table, max_blocks, slots, positions, rows, q_heads, kv_heads,
                                head_dim, page_size, (job / kv_heads) * 16, job % kv_heads);
        return;
    }
    const int m = blockIdx.x;
    const int lph = head_dim / 16;                         // lanes per head (a power of two)
    const int half = head_dim >> 1;
    const int total = q_heads + (skip_values ? 1 : 2) * kv_heads;
    const int head_raw = (blockIdx.y * blockDim.x + threadIdx.x) / lph;
    const bool active = head_raw < total;
    const int head = active ? head_raw : 0;
    const int c = threadIdx.x % lph;                       // this lane: channels 8c .. 8c + 7 and half + 8c ..
    const int pos = positions[m], slot = slots[m];
    const __bf16* src = qkv + (size_t)m * ld + (size_t)head * head_dim;
    const bf16x8 lo8 = *reinterpret_cast<const bf16x8*>(src + 8 * c);
    const bf16x8 hi8 = *reinterpret_cast<const bf16x8*>(src + half + 8 * c);
    const bool is_q = head < q_heads;
    float wl[8], wh[8];
    if (HAS_NORM) {
        const float* w = is_q ? q_norm_w : k_norm_w;
        const float4 w0 = *reinterpret_cast<const float4*>(w + 8 * c), w1 = *reinterpret_cast<const float4*>(w + 8 * c + 4);
        const float4 w2 = *reinterpret_cast<const float4*>(w + half + 8 * c);
        const float4 w3 = *reinterpret_cast<const float4*>(w + half + 8 * c + 4);
        wl[0] = w0.x; wl[1] = w0.y; wl[2] = w0.z; wl[3] = w0.w; wl[4] = w1.x; wl[5] = w1.y; wl[6] = w1.z; wl[7] = w1.w;
        wh[0] = w2.x; wh[1] = w2.y; wh[2] = w2.z; wh[3] = w2.w; wh[4] = w3.x; wh[5] = w3.y; wh[6] = w3.z; wh[7] = w3.w;
    }
    // what needs the position: the page (entry 0 of the request's row when nothing is written) and the
    // rotation row
    const int block = write_cache ? pos / page_size : 0;       // (beyond the request's row of the table: no page)
    const int page_read = block_table[(size_t)slot * max_blocks + min(block, max_blocks - 1)];
    const int page = block < max_blocks ? page_read : -1;
    float co[8], si[8];
    if (HAS_ROPE) {
        const float* cs = rope + (size_t)pos * head_dim;
        const float4 c0 = *reinterpret_cast<const float4*>(cs + 8 * c), c1 = *reinterpret_cast<const float4*>(cs + 8 * c + 4);
        const float4 s0 = *reinterpret_cast<const float4*>(cs + half + 8 * c);
        const float4 s1 = *reinterpret_cast<const float4*>(cs + half + 8 * c + 4);
        co[0] = c0.x; co[1] = c0.y; co[2] = c0.z; co[3] = c0.w; co[4] = c1.x; co[5] = c1.y; co[6] = c1.z; co[7] = c1.w;
        si[0] = s0.x; si[1] = s0.y; si[2] = s0.z; si[3] = s0.w; si[4] = s1.x; si[5] = s1.y; si[6] = s1.z; si[7] = s1.w;
    }
    float a[8], b[8];
    float sum = 0.f;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        a[e] = (float)lo8[e];
        b[e] = (float)hi8[e];
        sum += squares(a[e], b[e]);
    }
    for (int off = 1; off < lph; off <<= 1) sum += __shfl_xor(sum, off, MLR_WAVE);
    if (!active) return;
    const bool cache_ok = write_cache && page >= 0;
    const size_t cache_page = (size_t)(page < 0 ? 0 : page) * kv_heads;
    const int in_page = pos % page_size;
    if (head >= q_heads + kv_heads) {                      // a value head: into its transposed page
        if (!cache_ok) return;
        __bf16* dst = v_pages + (cache_page + (head - q_heads - kv_heads)) * head_dim * page_size + in_page;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            dst[(size_t)(8 * c + e) * page_size] = lo8[e];
            dst[(size_t)(half + 8 * c + e) * page_size] = hi8[e];
        }
        return;
    }
    if (HAS_NORM) {
        const float scale = 1.0f / sqrtf(sum / (float)head_dim + eps);
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            a[e] = (a[e] * scale) * wl[e];
            b[e] = (b[e] * scale) * wh[e];
        }
    }
    if (HAS_ROPE) {
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const float x = turn_x(a[e], b[e], co[e], si[e]);
            const float y = turn_y(a[e], b[e], co[e], si[e]);
            a[e] = x;
            b[e] = y;
        }
    }
    __bf16* dst;
    if (is_q) {
        dst = q_out + ((size_t)m * q_heads + head) * head_dim;
    } else {
        if (!cache_ok) return;
        dst = k_pages + ((cache_page + (head - q_heads)) * page_size + in_page) * head_dim;
    }
    bf16x8 o_lo, o_hi;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        o_lo[e] = (__bf16)a[e];
        o_hi[e] = (__bf16)b[e];
    }
    *reinterpret_cast<bf16x8*>(dst + 8 * c) = o_lo;
    *reinterpret_cast<bf16x8*>(dst + half + 8 * c) = o_hi;
}

#endif

extern "C" int mlr_qk_norm_rope_kv(
    const void* qkv, int ld, void* q_out, void* k_pages, void* v_pages, const int32_t* block_table,
    int max_blocks, const int32_t* slots, const int32_t* positions, const float* q_norm_w,
    const float* k_norm_w, float eps, const float* rope, int rows, int q_heads, int kv_heads,
    int head_dim, int page_size, int write_cache, int rot_dim, int interleaved, hipStream_t stream) {
    if (rows <= 0) return 0;
    if (head_dim % 2 != 0 || head_dim / 2 > 64 * MAX_PAIRS) return -1;
    if (rope == nullptr) {                                 // (no rotation: any pairing covers the head)
        rot_dim = head_dim;
        interleaved = 0;
    }
    if (rot_dim < 2 || rot_dim > head_dim || rot_dim % 2 != 0) return -2;
    const int total_heads = q_heads + 2 * kv_heads;
#if MLR_BF16
    const int lph = head_dim / 16;
    if (rows >= 64 && head_dim % 16 == 0 && (lph & (lph - 1)) == 0 && ld % 8 == 0 && rot_dim == head_dim && !interleaved) {
        // values take workgroups of their own (stores of 16 bytes into the transposed pages) when pages hold
        // a multiple of eight tokens
        const int split_values = write_cache && page_size % 8 == 0;
        const int threads_needed = (total_heads - (split_values ? kv_heads : 0)) * lph;
        const int value_jobs = split_values ? ((rows + 15) / 16) * kv_heads : 0;
        const dim3 grid(rows + value_jobs, (threads_needed + 255) / 256);
        const size_t lds = split_values ? 16 * (head_dim + 8) * sizeof(__bf16) : 0;
#define MLR_ROPE_VEC(NORM, ROPE)                                                                                   \
        qk_norm_rope_kv_vec_kernel<NORM, ROPE><<<grid, 256, lds, stream>>>(                                        \
            (const __bf16*)qkv, ld, (__bf16*)q_out, (__bf16*)k_pages, (__bf16*)v_pages, block_table, max_blocks,  \
            slots, positions, q_norm_w, k_norm_w, eps, rope, q_heads, kv_heads, head_dim, page_size, write_cache, \
            split_values, rows)
        const bool norm = q_norm_w != nullptr && k_norm_w != nullptr;
        if (norm && rope) MLR_ROPE_VEC(true, true);
        else if (norm) MLR_ROPE_VEC(true, false);
        else if (rope) MLR_ROPE_VEC(false, true);
        else MLR_ROPE_VEC(false, false);
#undef MLR_ROPE_VEC
        return (int)hipGetLastError();
    }
#endif
    // few rows: spread a row's heads over several workgroups (a wavefront per head)
    int chunks = 1;
    if (rows < 512) chunks = (total_heads + 3) / 4;
    if (chunks > 64) chunks = 64;
    qk_norm_rope_kv_kernel<<<dim3(rows, chunks), 256, 0, stream>>>(
        (const elem_t*)qkv, ld, (elem_t*)q_out, (elem_t*)k_pages, (elem_t*)v_pages, block_table,
        max_blocks, slots, positions, q_norm_w, k_norm_w, eps, rope, q_heads, kv_heads, head_dim,
        page_size, write_cache, rot_dim, interleaved);
    return (int)hipGetLastError();
}
