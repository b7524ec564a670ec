// Attention of a batch of tokens over the paged cache.
//
// Every token m of the batch (a prompt portion's token or a decoded one) is a query at
// position positions[m] of the request in slot slots[m]; its keys and values are read from
// the pages of that request, the tokens of this very batch included (they were written
// before this kernel runs).  Keys seen: positions in [max(0, p - window + 1), p]
// (window <= 0: all from 0).  Scores, the softmax and the weighted sum are 32-bit.
//
// Work split: one workgroup per (token, kv head, chunk of the query heads of that kv head,
// key split).  Keys are walked in tiles of 64 whose edges are multiples of 64 in absolute
// position, and key splits are ranges [s * split_keys, (s + 1) * split_keys): the order of
// every sum depends only on the token's own position, never on the batch around it.
// With more than one split the workgroups write partial (max, sum, weighted values) and
// `attention_combine_kernel` merges them in ascending order.
//
// Cache layout of one layer: pages[num_pages][kv_heads][page_size][head_dim].
#include "common.h"

#define TILE_KEYS 64
#define DIM_CHUNK 128
#define HEADS_PER_WAVE 2
#define WAVES 4
#define HEADS_PER_BLOCK (HEADS_PER_WAVE * WAVES)
#define MAX_DIM_REGS 4          // head_dim <= 64 * MAX_DIM_REGS

struct AttnArgs {
    const elem_t* q;            // [M, q_heads, head_dim]
    const elem_t* k_pages;
    const elem_t* v_pages;
    const int32_t* block_table; // [slots, max_blocks]
    const int32_t* slots;       // [M]
    const int32_t* positions;   // [M]
    elem_t* out;                // [M, q_heads, head_dim]
    float* partial;             // [M, q_heads, max_splits, head_dim + 2] when max_splits > 1
    int max_blocks, q_heads, kv_heads, head_dim, page_size, window, split_keys, max_splits;
    float scale;
};

__global__ __launch_bounds__(256) void paged_attention_kernel(AttnArgs a) {
    extern __shared__ float lds[];
    const int D = a.head_dim;
    const int group = a.q_heads / a.kv_heads;
    const int head_chunks = (group + HEADS_PER_BLOCK - 1) / HEADS_PER_BLOCK;
    const int m = blockIdx.x, kvh = blockIdx.y;
    const int chunk = blockIdx.z % head_chunks, split = blockIdx.z / head_chunks;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;

    float* q_lds = lds;                                    // [HEADS_PER_BLOCK][D]
    float* k_lds = q_lds + HEADS_PER_BLOCK * D;            // [TILE_KEYS][DIM_CHUNK + 1]
    float* p_lds = k_lds + TILE_KEYS * (DIM_CHUNK + 1);    // [HEADS_PER_BLOCK][TILE_KEYS]
    __shared__ long long row_off[TILE_KEYS];               // element offset of each key's row

    const int pos = a.positions[m];
    const int slot = a.slots[m];
    int kbegin = a.window > 0 ? max(0, pos - a.window + 1) : 0;
    int kend = pos + 1;
    if (a.max_splits > 1) {
        kbegin = max(kbegin, split * a.split_keys);
        kend = min(kend, (split + 1) * a.split_keys);
    }
    const int head0 = kvh * group + chunk * HEADS_PER_BLOCK;       // first query head of this block
    const int nheads = min(HEADS_PER_BLOCK, group - chunk * HEADS_PER_BLOCK);

    for (int i = threadIdx.x; i < nheads * D; i += blockDim.x) {
        q_lds[i] = to_float(a.q[((size_t)m * a.q_heads + head0) * D + i]);
    }

    float run_max[HEADS_PER_WAVE], run_sum[HEADS_PER_WAVE], acc[HEADS_PER_WAVE][MAX_DIM_REGS];
#pragma unroll
    for (int hh = 0; hh < HEADS_PER_WAVE; ++hh) {
        run_max[hh] = -INFINITY;
        run_sum[hh] = 0.f;
#pragma unroll
        for (int i = 0; i < MAX_DIM_REGS; ++i) acc[hh][i] = 0.f;
    }

    const int32_t* table = a.block_table + (size_t)slot * a.max_blocks;
    for (int t0 = (kbegin / TILE_KEYS) * TILE_KEYS; t0 < kend; t0 += TILE_KEYS) {
        __syncthreads();                       // previous tile's reads of row_off / p_lds are done
        if (threadIdx.x < TILE_KEYS) {
            const int kp = t0 + threadIdx.x;
            long long off = -1;
            if (kp >= kbegin && kp < kend) {
                const int page = table[kp / a.page_size];
                if (page >= 0) {
                    off = (((long long)page * a.kv_heads + kvh) * a.page_size + kp % a.page_size) * D;
                }
            }
            row_off[threadIdx.x] = off;
        }
        float score[HEADS_PER_WAVE];
#pragma unroll
        for (int hh = 0; hh < HEADS_PER_WAVE; ++hh) score[hh] = 0.f;
        for (int dc = 0; dc < D; dc += DIM_CHUNK) {
            const int dw = min(DIM_CHUNK, D - dc);
            __syncthreads();                   // row_off visible; previous chunk's k_lds reads done
            for (int i = threadIdx.x; i < TILE_KEYS * dw; i += blockDim.x) {
                const int key = i / dw, d = i % dw;
                const long long off = row_off[key];
                k_lds[key * (DIM_CHUNK + 1) + d] = off >= 0 ? to_float(a.k_pages[off + dc + d]) : 0.f;
            }
            __syncthreads();
#pragma unroll
            for (int hh = 0; hh < HEADS_PER_WAVE; ++hh) {
                const int hi = wave + WAVES * hh;
                if (hi < nheads) {
                    const float* qh = q_lds + hi * D + dc;
                    const float* kr = k_lds + lane * (DIM_CHUNK + 1);
                    float s = 0.f;
                    for (int d = 0; d < dw; ++d) s += qh[d] * kr[d];
                    score[hh] += s;
                }
            }
        }
        const bool valid = row_off[lane] >= 0;
#pragma unroll
        for (int hh = 0; hh < HEADS_PER_WAVE; ++hh) {
            const int hi = wave + WAVES * hh;
            if (hi < nheads) {
                const float s = valid ? score[hh] * a.scale : -INFINITY;
                const float new_max = fmaxf(run_max[hh], wave_max(s));
                // a tile can be wholly masked only before the window: then new_max stays -inf
                const float p = (valid && new_max > -INFINITY) ? expf(s - new_max) : 0.f;
                const float corr = new_max > -INFINITY ? expf(run_max[hh] - new_max) : 1.f;
                run_sum[hh] = run_sum[hh] * corr + wave_sum(p);
                run_max[hh] = new_max;
#pragma unroll
                for (int i = 0; i < MAX_DIM_REGS; ++i) acc[hh][i] *= corr;
                p_lds[hi * TILE_KEYS + lane] = p;
            }
        }
        __syncthreads();
        const int nkeys = min(TILE_KEYS, kend - t0);
        for (int key = 0; key < nkeys; ++key) {
            const long long off = row_off[key];
            if (off < 0) continue;
            float v[MAX_DIM_REGS];
#pragma unroll
            for (int i = 0; i < MAX_DIM_REGS; ++i) {
                const int d = lane + 64 * i;
                v[i] = d < D ? to_float(a.v_pages[off + d]) : 0.f;
            }
#pragma unroll
            for (int hh = 0; hh < HEADS_PER_WAVE; ++hh) {
                const int hi = wave + WAVES * hh;
                if (hi < nheads) {
                    const float p = p_lds[hi * TILE_KEYS + key];
#pragma unroll
                    for (int i = 0; i < MAX_DIM_REGS; ++i) acc[hh][i] += p * v[i];
                }
            }
        }
    }

#pragma unroll
    for (int hh = 0; hh < HEADS_PER_WAVE; ++hh) {
        const int hi = wave + WAVES * hh;
        if (hi >= nheads) continue;
        const int head = head0 + hi;
        if (a.max_splits > 1) {
            float* dst = a.partial + (((size_t)m * a.q_heads + head) * a.max_splits + split) * (D + 2);
#pragma unroll
            for (int i = 0; i < MAX_DIM_REGS; ++i) {
                const int d = lane + 64 * i;
                if (d < D) dst[d] = acc[hh][i];
            }
            if (lane == 0) {
                dst[D] = run_max[hh];
                dst[D + 1] = run_sum[hh];
            }
        } else {
            // a division, as in the combine kernel: one split gives the same bits either way
            const float den = run_sum[hh];
            elem_t* dst = a.out + ((size_t)m * a.q_heads + head) * D;
#pragma unroll
            for (int i = 0; i < MAX_DIM_REGS; ++i) {
                const int d = lane + 64 * i;
                if (d < D) dst[d] = from_float<elem_t>(den > 0.f ? acc[hh][i] / den : 0.f);
            }
        }
    }
}

// out[m, head, :] = sum_s w_s acc_s / sum_s w_s l_s with w_s = exp(max_s - max), over the
// splits that hold keys of this token, in ascending order.
__global__ void attention_combine_kernel(AttnArgs a) {
    const int m = blockIdx.x, head = blockIdx.y;
    const int D = a.head_dim;
    const int pos = a.positions[m];
    const int nsplit = min(a.max_splits, pos / a.split_keys + 1);
    const float* base = a.partial + ((size_t)m * a.q_heads + head) * a.max_splits * (D + 2);
    float gmax = -INFINITY;
    for (int s = 0; s < nsplit; ++s) gmax = fmaxf(gmax, base[(size_t)s * (D + 2) + D]);
    for (int d = threadIdx.x; d < D; d += blockDim.x) {
        float num = 0.f, den = 0.f;
        for (int s = 0; s < nsplit; ++s) {
            const float* p = base + (size_t)s * (D + 2);
            const float smax = p[D];
            if (smax == -INFINITY) continue;
            const float w = expf(smax - gmax);
            num += w * p[d];
            den += w * p[D + 1];
        }
        a.out[((size_t)m * a.q_heads + head) * D + d] = from_float<elem_t>(den > 0.f ? num / den : 0.f);
    }
}

extern "C" int mlr_paged_attention(
    const void* q, const void* k_pages, const void* v_pages, const int32_t* block_table,
    int max_blocks, const int32_t* slots, const int32_t* positions, void* out, float* partial,
    int rows, int q_heads, int kv_heads, int head_dim, int page_size, int window, float scale,
    int split_keys, int max_splits, hipStream_t stream) {
    if (rows <= 0) return 0;
    if (head_dim > 64 * MAX_DIM_REGS || q_heads % kv_heads != 0) return -1;
    if (max_splits > 1 && (partial == nullptr || split_keys <= 0 || split_keys % TILE_KEYS != 0)) return -2;
    AttnArgs a{(const elem_t*)q, (const elem_t*)k_pages, (const elem_t*)v_pages, block_table, slots,
               positions, (elem_t*)out, partial, max_blocks, q_heads, kv_heads, head_dim, page_size,
               window, split_keys, max_splits < 1 ? 1 : max_splits, scale};
    const int group = q_heads / kv_heads;
    const int head_chunks = (group + HEADS_PER_BLOCK - 1) / HEADS_PER_BLOCK;
    const size_t lds = sizeof(float) * ((size_t)HEADS_PER_BLOCK * head_dim +
                                        TILE_KEYS * (DIM_CHUNK + 1) + HEADS_PER_BLOCK * TILE_KEYS);
    dim3 grid(rows, kv_heads, head_chunks * a.max_splits);
    paged_attention_kernel<<<grid, 256, lds, stream>>>(a);
    int err = (int)hipGetLastError();
    if (err != 0) return err;
    if (a.max_splits > 1) {
        attention_combine_kernel<<<dim3(rows, q_heads), 64, 0, stream>>>(a);
        err = (int)hipGetLastError();
    }
    return err;
}
