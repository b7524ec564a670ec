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
// Cache layout of one layer: keys pages[num_pages][kv_heads][page_size][head_dim]; values transposed,
// pages[num_pages][kv_heads][head_dim][page_size], so that the keys of one channel lie side by side
// (the layout the matrix cores want for probabilities x values).
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
    extern __shared__ __attribute__((aligned(16))) float lds[];
    const int D = a.head_dim;
    const int group = a.q_heads / a.kv_heads;
    const int head_chunks = (group + HEADS_PER_BLOCK - 1) / HEADS_PER_BLOCK;
    const int m = blockIdx.x, kvh = blockIdx.y;
    const int chunk = blockIdx.z % head_chunks, split = blockIdx.z / head_chunks;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;

    float* q_lds = lds;                                    // [HEADS_PER_BLOCK][D]
    float* k_lds = q_lds + HEADS_PER_BLOCK * D;            // [TILE_KEYS][DIM_CHUNK + 1]
    float* p_lds = k_lds + TILE_KEYS * (DIM_CHUNK + 1);    // [HEADS_PER_BLOCK][TILE_KEYS]
    __shared__ long long row_off[TILE_KEYS];               // element offset of each key's row in k_pages
    __shared__ long long val_off[TILE_KEYS];               // element offset of each key's column in v_pages

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
            long long off = -1, voff = -1;
            if (kp >= kbegin && kp < kend) {
                const int block = kp / a.page_size;
                const int page = block < a.max_blocks ? table[block] : -1;     // (beyond the table's row: no page)
                if (page >= 0) {
                    off = (((long long)page * a.kv_heads + kvh) * a.page_size + kp % a.page_size) * D;
                    voff = ((long long)page * a.kv_heads + kvh) * D * a.page_size + kp % a.page_size;
                }
            }
            row_off[threadIdx.x] = off;
            val_off[threadIdx.x] = voff;
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
            const long long off = val_off[key];
            if (off < 0) continue;
            float v[MAX_DIM_REGS];
#pragma unroll
            for (int i = 0; i < MAX_DIM_REGS; ++i) {
                const int d = lane + 64 * i;
                v[i] = d < D ? to_float(a.v_pages[off + (long long)d * a.page_size]) : 0.f;
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
                if (d < D) dst[d] = from_float<elem_t>(den != 0.f ? acc[hh][i] / den : 0.f);
            }
        }
    }
}

// out[m, head, :] = sum_s w_s acc_s / sum_s w_s l_s with w_s = exp(max_s - max), over the splits
// first_split .. last_split that hold keys of this token, in ascending order.  One wavefront per
// (token, head); the splits' weights go through LDS, the channel loads are independent of each other.
#define COMBINE_MAX_SPLITS 1024
__global__ __launch_bounds__(64) void attention_combine_kernel(AttnArgs a) {
    __shared__ float w_lds[COMBINE_MAX_SPLITS];
    __shared__ float l_lds[COMBINE_MAX_SPLITS];
    const int m = blockIdx.x, head = blockIdx.y;
    const int D = a.head_dim;
    const int pos = a.positions[m];
    const int first = a.window > 0 ? max(0, pos + 1 - a.window) / a.split_keys : 0;
    const int last = min(a.max_splits - 1, pos / a.split_keys);
    const int n = last - first + 1;
    const float* base = a.partial + (((size_t)m * a.q_heads + head) * a.max_splits + first) * (D + 2);
    float gmax = -INFINITY;
    for (int s = threadIdx.x; s < n; s += 64) {
        const float smax = base[(size_t)s * (D + 2) + D];
        w_lds[s] = smax;
        l_lds[s] = base[(size_t)s * (D + 2) + D + 1];
        gmax = fmaxf(gmax, smax);
    }
    gmax = wave_max(gmax);
    __syncthreads();
    for (int s = threadIdx.x; s < n; s += 64) {
        const float smax = w_lds[s];
        w_lds[s] = smax > -INFINITY ? expf(smax - gmax) : 0.f;       // an empty split holds zeros
    }
    __syncthreads();
    float den = 0.f;
    for (int s = 0; s < n; ++s) den += w_lds[s] * l_lds[s];
    float num[MAX_DIM_REGS];
#pragma unroll
    for (int i = 0; i < MAX_DIM_REGS; ++i) num[i] = 0.f;
    for (int s = 0; s < n; ++s) {
        const float w = w_lds[s];
        const float* p = base + (size_t)s * (D + 2);
#pragma unroll
        for (int i = 0; i < MAX_DIM_REGS; ++i) {
            const int d = threadIdx.x + 64 * i;
            if (d < D) num[i] += w * p[d];
        }
    }
#pragma unroll
    for (int i = 0; i < MAX_DIM_REGS; ++i) {
        const int d = threadIdx.x + 64 * i;
        if (d < D) a.out[((size_t)m * a.q_heads + head) * D + d] = from_float<elem_t>(den != 0.f ? num[i] / den : 0.f);
    }
}

extern "C" int mlr_paged_attention(
    const void* q, const void* k_pages, const void* v_pages, const int32_t* block_table,
    int max_blocks, const int32_t* slots, const int32_t* positions, void* out, float* partial,
    int rows, int q_heads, int kv_heads, int head_dim, int page_size, int window, float scale,
    int split_keys, int max_splits, hipStream_t stream) {
    if (rows <= 0) return 0;
    if (head_dim > 64 * MAX_DIM_REGS || q_heads % kv_heads != 0) return -1;
    if (max_splits > 1 && (partial == nullptr || split_keys <= 0 || split_keys % TILE_KEYS != 0 ||
                           max_splits > COMBINE_MAX_SPLITS)) return -2;
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

#if MLR_BF16
// ------------------------------------------------------------------------------------------------
// Matrix-core attention for the bfloat16 engine.
//
// A workgroup serves one GROUP of up to 16 query columns that share their keys: `ntok` consecutive
// tokens of one request (rows row0 .. row0 + ntok - 1 of the batch, positions pos0 ..) times the
// `g = q_heads / kv_heads` query heads of one kv head; column c is (token c / g, head c % g).  A decoded
// token is a group of one token.  Keys are walked in tiles of 32 at absolute multiples of 32; the four
// wavefronts of the workgroup take the tiles t with t % 4 == wave, keep (max, sum, weighted values) each
// and are merged in the order 0..3 at the end, so a column's sums depend on its own position only.
// The loads of the next tile are issued before the current one is computed.
//
// Per tile, with v_mfma_f32_16x16x32_bf16 (D = A x B, a lane holds row/column lane % 16 and the eight
// k-slots (lane / 16, 0..7) of A and of B):
//   scores^T[key][column] = K[key][:] . Q[column][:]      A = 16 keys of K (rows as they lie in the page),
//                                                         B = Q; two such products cover the 32 keys;
//   out^T[d][column]     += V^T[d][key] . P^T[key][column]  A = 16 channels of V^T (keys side by side in
//                                                         the transposed page), B = the probabilities,
//                                                         which already sit in B's register layout:
//                                                         k-slot (b, e) is key 4b + e of the first 16 keys
//                                                         for e < 4 and key 4b + e - 4 of the second 16.
//
// With key splits (max_splits > 1) every workgroup that holds keys writes its partial result and
// `attention_combine_kernel` merges them (a second launch: on this GPU partial results of other
// workgroups become visible cheaply at a kernel's end only).
typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(__bf16)))) __bf16 bf16x4;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float floatx4;

#define MFMA_TILE_KEYS 32

template <int NCH>
struct KvTile {
    bf16x8 k[2][NCH];
    bf16x4 v[2 * NCH][2];
    int ok;                  // bit j: the page of keys tb + 16 j .. is mapped
    int tb;
};

#define DECODE_PAGE_CACHE 4096

// Decoding (every group is one new token of a request) without a kernel of its own for the per-head norm,
// the rotation and the cache write: the attention kernel takes the raw projection, norms and rotates its
// queries itself and walks the keys that are cached already (positions below the token's own); the merge
// kernel, which follows anyway, norms and rotates the token's own key, adds the token's own score and
// value as one more summand, and writes key and value into their pages for the steps to come.
// Needs head_dim % 64 == 0 (a lane of the attention kernel then holds both channels of a rotation pair).
struct DecodeFusion {
    const __bf16* qkv;          // [M, ld]: q heads, k heads, v heads of every row
    const float* q_norm_w;      // [head_dim] or null
    const float* k_norm_w;
    const float* rope;          // [positions, head_dim]: cosines | sines, or null
    int ld;
    float eps;
};

template <int NCH, bool FUSED>   // NCH: ceil(head_dim / 32)
__global__ __launch_bounds__(256, (NCH <= 4 ? 2 : 1)) void attention_mfma_kernel(AttnArgs a, const int32_t* __restrict__ group_row0,
                                                             const int32_t* __restrict__ group_ntok, DecodeFusion f) {
    extern __shared__ __attribute__((aligned(16))) float lds[];
    __shared__ int32_t page_lds[DECODE_PAGE_CACHE];    // the request's page ids for this workgroup's key range
    const int D = a.head_dim, P = a.page_size;
    const int g = a.q_heads / a.kv_heads;
    const int grp = blockIdx.x, kvh = blockIdx.y, split = blockIdx.z;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int col = lane & 15, b = lane >> 4;
    // (FUSED: group i is the one token in batch row i; no need to wait for the group vectors)
    const int row0 = FUSED ? grp : group_row0[grp], ntok = FUSED ? 1 : group_ntok[grp];
    const int slot = a.slots[row0], pos0 = a.positions[row0];
    const int tok = col / g, hh = col % g;
    const bool col_valid = tok < ntok;
    const int kend_full = col_valid ? pos0 + tok + 1 : 0;
    int kbegin_c = a.window > 0 ? max(0, kend_full - a.window) : 0;
    const int kend_c = FUSED ? max(kend_full - 1, 0) : kend_full;     // FUSED: the token's own key is not cached yet
    const int glo = a.window > 0 ? max(0, pos0 + 1 - a.window) : 0;   // the group's key range [glo, ke)
    const int ke = pos0 + ntok - (FUSED ? 1 : 0);                      // keys below ke are written
    int lo = glo, hi = ke;
    if (a.max_splits > 1) {
        const int first_split = glo / a.split_keys;
        const int last_split = min(a.max_splits - 1, max(ke - 1, 0) / a.split_keys);
        if (split < first_split || split > last_split) return;          // no keys here: the whole workgroup leaves
        lo = max(lo, split * a.split_keys);
        hi = min(hi, (split + 1) * a.split_keys);
    }
    hi = max(hi, lo);                                                   // (FUSED, first token: no key at all)
    kbegin_c = max(kbegin_c, lo);
    const int kstop_c = min(kend_c, hi);

    const __bf16* q = reinterpret_cast<const __bf16*>(a.q);
    const __bf16* kp_base = reinterpret_cast<const __bf16*>(a.k_pages);
    const __bf16* vp_base = reinterpret_cast<const __bf16*>(a.v_pages);
    const bf16x8 zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
    const int32_t* table = a.block_table + (size_t)slot * a.max_blocks;

    // page ids first, into LDS: a tile's loads then never wait on a load of the block table
    const int t_begin = lo / MFMA_TILE_KEYS, t_end = (hi + MFMA_TILE_KEYS - 1) / MFMA_TILE_KEYS;
    const int first_page = t_begin * MFMA_TILE_KEYS / P;
    {
        const int n_pages = min(DECODE_PAGE_CACHE, (hi + P - 1) / P - first_page);
        // (an entry beyond the request's row of the table is no page, like an entry of -1)
        for (int i = threadIdx.x; i < n_pages; i += 256)
            page_lds[i] = first_page + i < a.max_blocks ? table[first_page + i] : -1;
    }

    // The queries.  FUSED: the raw query of this lane's column, its norm weights and its rotation row are
    // asked for here; the arithmetic waits until the first key tile has been asked for as well (below).
    bf16x8 qf[NCH];
    constexpr int HC = NCH / 2;
    bf16x8 q_raw[FUSED ? NCH : 1];
    float4 q_w[FUSED ? 2 * NCH : 1], q_cs[FUSED ? 2 * NCH : 1];
    if (FUSED) {
        const __bf16* src = f.qkv + (size_t)(row0 + (col_valid ? tok : 0)) * f.ld + (size_t)(kvh * g + (col_valid ? hh : 0)) * D + 8 * b;
        const float* wq = (f.q_norm_w ? f.q_norm_w : reinterpret_cast<const float*>(f.qkv)) + 8 * b;     // (any readable address)
        const float* cs = (f.rope ? f.rope + (size_t)(pos0 + (col_valid ? tok : 0)) * D : reinterpret_cast<const float*>(f.qkv)) + 8 * b;
#pragma unroll
        for (int c = 0; c < NCH; ++c) {
            q_raw[c] = *reinterpret_cast<const bf16x8*>(src + 32 * c);
            q_w[2 * c] = *reinterpret_cast<const float4*>(wq + 32 * c);
            q_w[2 * c + 1] = *reinterpret_cast<const float4*>(wq + 32 * c + 4);
            // cosines of the pairs 32 c + 8 b .. for c < HC, their sines for c >= HC (the table holds cosines | sines)
            q_cs[2 * c] = *reinterpret_cast<const float4*>(cs + 32 * c);
            q_cs[2 * c + 1] = *reinterpret_cast<const float4*>(cs + 32 * c + 4);
        }
    } else {
#pragma unroll
        for (int c = 0; c < NCH; ++c) {
            const int d0 = 32 * c + 8 * b;
            qf[c] = zero8;
            if (col_valid && d0 < D)
                qf[c] = *reinterpret_cast<const bf16x8*>(q + ((size_t)(row0 + tok) * a.q_heads + kvh * g + hh) * D + d0);
        }
    }
    __syncthreads();
    auto finish_queries = [&]() {
        // per-head norm, rotation (a lane holds channels 32 c + 8 b .. of every chunk c, so with head_dim =
        // 32 NCH, NCH even, the partner d + head_dim / 2 of a channel is in chunk c + NCH / 2 of the same
        // lane), rounded to bfloat16 as the cache's keys are
        float x[NCH][8];
        float sq = 0.f;
#pragma unroll
        for (int c = 0; c < NCH; ++c)
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                x[c][e] = (float)q_raw[c][e];
                sq += x[c][e] * x[c][e];
            }
        sq += __shfl_xor(sq, 16, MLR_WAVE);
        sq += __shfl_xor(sq, 32, MLR_WAVE);
        if (f.q_norm_w) {
            const float scale = 1.0f / sqrtf(sq / (float)D + f.eps);
#pragma unroll
            for (int c = 0; c < NCH; ++c) {
                const float w8[8] = {q_w[2 * c].x, q_w[2 * c].y, q_w[2 * c].z, q_w[2 * c].w,
                                     q_w[2 * c + 1].x, q_w[2 * c + 1].y, q_w[2 * c + 1].z, q_w[2 * c + 1].w};
#pragma unroll
                for (int e = 0; e < 8; ++e) x[c][e] = (x[c][e] * scale) * w8[e];
            }
        }
        if (f.rope) {
#pragma unroll
            for (int c = 0; c < HC; ++c) {
                const float co[8] = {q_cs[2 * c].x, q_cs[2 * c].y, q_cs[2 * c].z, q_cs[2 * c].w,
                                     q_cs[2 * c + 1].x, q_cs[2 * c + 1].y, q_cs[2 * c + 1].z, q_cs[2 * c + 1].w};
                const float si[8] = {q_cs[2 * (c + HC)].x, q_cs[2 * (c + HC)].y, q_cs[2 * (c + HC)].z, q_cs[2 * (c + HC)].w,
                                     q_cs[2 * (c + HC) + 1].x, q_cs[2 * (c + HC) + 1].y, q_cs[2 * (c + HC) + 1].z,
                                     q_cs[2 * (c + HC) + 1].w};
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    const float lo_v = x[c][e], hi_v = x[c + HC][e];
                    x[c][e] = turn_x(lo_v, hi_v, co[e], si[e]);
                    x[c + HC][e] = turn_y(lo_v, hi_v, co[e], si[e]);
                }
            }
        }
#pragma unroll
        for (int c = 0; c < NCH; ++c)
#pragma unroll
            for (int e = 0; e < 8; ++e) qf[c][e] = col_valid ? (__bf16)x[c][e] : (__bf16)0.f;
    };

    // Scores are kept in the base-2 domain: s * (scale * log2 e), so that a probability is one v_exp_f32.
    const float c2 = a.scale * 1.44269504088896340736f;
    float m_run = -INFINITY, l_run = 0.f;
    floatx4 o[2 * NCH];
#pragma unroll
    for (int i = 0; i < 2 * NCH; ++i) o[i] = floatx4{0.f, 0.f, 0.f, 0.f};

    // this lane's fixed offsets into a key page (row col, channels 8b ..) and a value page (row col, keys 4b ..)
    // (the channel offset 8 b joins the key row only where it lies inside the head: with head_dim 16 the
    // lane blocks b = 2, 3 have no channels, and col * D + 8 b would reach into the next key's row and, in
    // the last row of the last page, past the end of the cache)
    const int k_lane = col * D, v_lane = col * P + 4 * b;
    const bool d_whole = (D & 31) == 0;
    // No branch around a load: a load behind a branch makes the compiler wait for every load in flight.
    // A missing page reads page 0 instead, channels beyond head_dim read channel block 0; both are
    // discarded when the tile is used.
    auto load = [&](int t, KvTile<NCH>& T) {
        T.tb = t * MFMA_TILE_KEYS;
        T.ok = 0;
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const int key0 = T.tb + 16 * j;
            const int idx = min(max(key0 / P - first_page, 0), DECODE_PAGE_CACHE - 1);
            const int page = key0 < hi ? page_lds[idx] : -1;
            T.ok |= (page >= 0 ? 1 : 0) << j;
            const size_t pk = (size_t)max(page, 0) * a.kv_heads + kvh;
            const __bf16* kptr = kp_base + (pk * P + key0 % P) * D + k_lane;
            const __bf16* vptr = vp_base + pk * D * P + key0 % P + v_lane;
#pragma unroll
            for (int c = 0; c < NCH; ++c)
                T.k[j][c] = *reinterpret_cast<const bf16x8*>(kptr + (32 * c + 8 * b < D ? 32 * c + 8 * b : 0));
#pragma unroll
            for (int db = 0; db < 2 * NCH; ++db)
                T.v[db][j] = *reinterpret_cast<const bf16x4*>(vptr + (size_t)(16 * db < D ? 16 * db : 0) * P);
        }
    };
    auto compute = [&](KvTile<NCH>& T) {
        floatx4 s[2];
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            s[j] = floatx4{0.f, 0.f, 0.f, 0.f};
            if (d_whole) {
#pragma unroll
                for (int c = 0; c < NCH; ++c)
                    s[j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(T.k[j][c], qf[c], s[j], 0, 0, 0);
            } else {
#pragma unroll
                for (int c = 0; c < NCH; ++c) {
                    const bf16x8 kf = (32 * c + 8 * b < D) ? T.k[j][c] : zero8;
                    s[j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf, qf[c], s[j], 0, 0, 0);
                }
            }
        }
        // this lane: keys tb + 16 j + 4 b + r of column `col`
        float sv[2][4];
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int key = T.tb + 16 * j + 4 * b + r;
                const bool ok = ((T.ok >> j) & 1) && key >= kbegin_c && key < kstop_c;
                sv[j][r] = ok ? s[j][r] * c2 : -INFINITY;
            }
        float tile_max = fmaxf(fmaxf(fmaxf(sv[0][0], sv[0][1]), fmaxf(sv[0][2], sv[0][3])),
                               fmaxf(fmaxf(sv[1][0], sv[1][1]), fmaxf(sv[1][2], sv[1][3])));
        tile_max = fmaxf(tile_max, __shfl_xor(tile_max, 16, MLR_WAVE));
        tile_max = fmaxf(tile_max, __shfl_xor(tile_max, 32, MLR_WAVE));
        // the running maximum rarely moves after the first tiles: rescale only when it does, for any column
        if (__builtin_amdgcn_ballot_w64(tile_max > m_run) != 0) {
            const float m_new = fmaxf(m_run, tile_max);
            const float corr = m_new > -INFINITY ? __builtin_amdgcn_exp2f(m_run - m_new) : 1.f;   // -inf - finite: 0
            l_run *= corr;
#pragma unroll
            for (int db = 0; db < 2 * NCH; ++db) o[db] *= corr;
            m_run = m_new;
        }
        const float m_use = fmaxf(m_run, -1e30f);      // a column with no key yet: exp2(-inf - finite) = 0, not NaN
        bf16x8 pf;
        float psum = 0.f;
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const float p = __builtin_amdgcn_exp2f(sv[j][r] - m_use);
                psum += p;
                pf[4 * j + r] = (__bf16)p;
            }
        l_run += psum;
        // values of keys that are not written yet (or of a page that is not there) must count as zero: a
        // probability of zero does not cancel a NaN.  Only a workgroup's last tile can hold such keys.
        const bool ragged = T.ok != 3 || T.tb + MFMA_TILE_KEYS > ke;
#pragma unroll
        for (int db = 0; db < 2 * NCH; ++db) {
            if (16 * db >= D) break;
            bf16x4 v0 = T.v[db][0], v1 = T.v[db][1];
            if (ragged) {
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    if (!(T.ok & 1) || T.tb + 4 * b + r >= ke) v0[r] = (__bf16)0.f;
                    if (!(T.ok & 2) || T.tb + 16 + 4 * b + r >= ke) v1[r] = (__bf16)0.f;
                }
            }
            const bf16x8 vf = {v0[0], v0[1], v0[2], v0[3], v1[0], v1[1], v1[2], v1[3]};
            o[db] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf, pf, o[db], 0, 0, 0);
        }
    };

    {
        // two tiles under way per wavefront: one being multiplied, one in flight; fetches are unconditional
        // (clamped to the wavefront's last tile) for the reason given above
        KvTile<NCH> ta, tb2;
        int t = t_begin + wave;
        const int t_last = t + ((t_end - 1 - t) / 4) * 4;
        if (t < t_end) load(t, ta);
        if (FUSED) finish_queries();
        if (t < t_end) {
            for (;;) {
                load(min(t + 4, t_last), tb2);
                compute(ta);
                if (t + 4 >= t_end) break;
                load(min(t + 8, t_last), ta);
                compute(tb2);
                if (t + 8 >= t_end) break;
                t += 8;
            }
        }
    }
    // per column: the four lane blocks hold partial sums of the same column
    l_run += __shfl_xor(l_run, 16, MLR_WAVE);
    l_run += __shfl_xor(l_run, 32, MLR_WAVE);

    // merge the wavefronts: 1..3 park their state in LDS, 0 merges in ascending order
    const int stride = 16 * D + 32;                        // floats per wavefront: the sums [D / 4][16 columns][4], max[16], sum[16]
    if (wave > 0) {
        float* dst = lds + (size_t)(wave - 1) * stride;
#pragma unroll
        for (int db = 0; db < 2 * NCH; ++db) {
            if (16 * db >= D) break;
            // (a lane's four sums side by side: one 16-byte access, consecutive lanes consecutive addresses)
            *reinterpret_cast<floatx4*>(dst + ((4 * db + b) * 16 + col) * 4) = o[db];
        }
        if (b == 0) {
            dst[16 * D + col] = m_run;
            dst[16 * D + 16 + col] = l_run;
        }
    }
    __syncthreads();
    const size_t out_row = (size_t)(row0 + tok) * a.q_heads + kvh * g + hh;
    if (wave == 0) {
        float m_tot = m_run;
        for (int w = 0; w < 3; ++w) m_tot = fmaxf(m_tot, lds[(size_t)w * stride + 16 * D + col]);
        // (a wavefront that saw no key has sum 0 and is passed over; one whose keys were all NaN -- a page
        // that nobody wrote -- has maximum -inf too, but a NaN sum, and must not be: 0 x NaN stays NaN)
        const float own = m_run > -INFINITY ? __builtin_amdgcn_exp2f(m_run - m_tot) : 0.f;
        float l_tot = l_run * own;
#pragma unroll
        for (int db = 0; db < 2 * NCH; ++db) o[db] *= own;
        for (int w = 0; w < 3; ++w) {
            const float* src = lds + (size_t)w * stride;
            const float mw = src[16 * D + col], lw = src[16 * D + 16 + col];
            if (lw == 0.f) continue;
            const float f = mw > -INFINITY ? __builtin_amdgcn_exp2f(mw - m_tot) : 0.f;
            l_tot += lw * f;
#pragma unroll
            for (int db = 0; db < 2 * NCH; ++db) {
                if (16 * db >= D) break;
                const floatx4 other = *reinterpret_cast<const floatx4*>(src + ((4 * db + b) * 16 + col) * 4);
#pragma unroll
                for (int r = 0; r < 4; ++r) o[db][r] += other[r] * f;
            }
        }
        if (col_valid) {
            if (a.max_splits > 1 || FUSED) {                   // (FUSED: the merge kernel always follows)
                float* dst = a.partial + (out_row * a.max_splits + split) * (D + 2);
#pragma unroll
                for (int db = 0; db < 2 * NCH; ++db) {
                    if (16 * db >= D) break;
#pragma unroll
                    for (int r = 0; r < 4; ++r) dst[16 * db + 4 * b + r] = o[db][r];
                }
                if (b == 0) {
                    dst[D] = m_tot;
                    dst[D + 1] = l_tot;
                }
            } else {
                __bf16* dst = reinterpret_cast<__bf16*>(a.out) + out_row * D;
#pragma unroll
                for (int db = 0; db < 2 * NCH; ++db) {
                    if (16 * db >= D) break;
                    bf16x4 w4;
#pragma unroll
                    for (int r = 0; r < 4; ++r) w4[r] = (__bf16)(l_tot != 0.f ? o[db][r] / l_tot : 0.f);
                    *reinterpret_cast<bf16x4*>(dst + 16 * db + 4 * b) = w4;
                }
            }
        }
    }
}

// ------------------------------------------------------------------------------------------------
// Prompt portions: a workgroup serves up to 4 * (16 / g) consecutive tokens of one request (each
// wavefront 16 columns: 16 / g tokens times g heads).  All four wavefronts walk the same key tiles,
// which are staged once per workgroup through LDS (double-buffered: the next tile's global loads are in
// flight while the current one is multiplied), so keys and values are read from memory once per
// workgroup instead of once per wavefront.  The arithmetic per column is that of
// `attention_mfma_kernel` without key splits, tile by tile in ascending order.
#define PAGE_CACHE 2048
template <int NCH>
__device__ __forceinline__ void prefill_group(const AttnArgs& a, const int32_t* __restrict__ group_row0,
                                              const int32_t* __restrict__ group_ntok, int grp, int kvh,
                                              __bf16 (*k_lds)[32 * (32 * NCH + 8)], __bf16 (*v_lds)[32 * NCH * 36],
                                              int32_t* page_lds) {
    constexpr int DMAX = 32 * NCH;
    constexpr int KPITCH = DMAX + 8;                  // elements per key row in LDS
    constexpr int VPITCH = 32 + 4;                    // elements per channel row in LDS
    constexpr int STAGE = (NCH + 1) / 2;              // 16-byte chunks a thread stages per tile, for K and for V
    const int D = a.head_dim, P = a.page_size;
    const int g = a.q_heads / a.kv_heads, tq = 16 / g;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int col = lane & 15, b = lane >> 4;
    const int row0 = group_row0[grp], ntok = group_ntok[grp];
    const int slot = a.slots[row0], pos0 = a.positions[row0];
    const int tok = wave * tq + col / g, hh = col % g;          // this lane's column: token within the group, head
    const bool col_valid = col / g < tq && tok < ntok;
    const int kend_c = col_valid ? pos0 + tok + 1 : 0;
    const int kbegin_c = a.window > 0 ? max(0, kend_c - a.window) : 0;
    const int lo = a.window > 0 ? max(0, pos0 + 1 - a.window) : 0;
    const int ke = pos0 + ntok;
    // this wavefront's own key range (its tokens wave * tq .. wave * tq + tq - 1)
    const int wtok0 = wave * tq;
    const bool wave_active = wtok0 < ntok;
    const int wave_hi = wave_active ? pos0 + min(ntok, wtok0 + tq) : 0;
    const int wave_lo = a.window > 0 ? max(0, pos0 + wtok0 + 1 - a.window) : 0;

    const __bf16* q = reinterpret_cast<const __bf16*>(a.q);
    const __bf16* kp_base = reinterpret_cast<const __bf16*>(a.k_pages);
    const __bf16* vp_base = reinterpret_cast<const __bf16*>(a.v_pages);
    const bf16x8 zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
    const int32_t* table = a.block_table + (size_t)slot * a.max_blocks;

    bf16x8 qf[NCH];
#pragma unroll
    for (int c = 0; c < NCH; ++c) {
        const int d0 = 32 * c + 8 * b;
        qf[c] = zero8;
        if (col_valid && d0 < D)
            qf[c] = *reinterpret_cast<const bf16x8*>(q + ((size_t)(row0 + tok) * a.q_heads + kvh * g + hh) * D + d0);
    }
    float m_run = -INFINITY, l_run = 0.f;
    floatx4 o[2 * NCH];
#pragma unroll
    for (int i = 0; i < 2 * NCH; ++i) o[i] = floatx4{0.f, 0.f, 0.f, 0.f};

    // page ids first: looked up in LDS, a tile's loads do not have to wait for a load of the block table
    // (the first tile starts at the multiple of 32 at or below lo, so the cache starts at that key's page)
    const int first_page = (lo / MFMA_TILE_KEYS) * MFMA_TILE_KEYS / P;
    {
        const int n_pages = min(PAGE_CACHE, (ke + P - 1) / P - first_page);
        for (int i = threadIdx.x; i < n_pages; i += 256)
            page_lds[i] = first_page + i < a.max_blocks ? table[first_page + i] : -1;
        __syncthreads();
    }
    const int kchunks = 4 * D;                         // 32 keys x D / 8 chunks of 16 bytes; as many for V
    struct Staged {
        bf16x8 k[STAGE], v[STAGE];
        int tb;
        int ok;                                        // bit j: the page of keys tb + 16 j .. is mapped
    };                                                 // (no array indexed at run time: that would live in scratch)
    // what a thread stages does not change from tile to tile: offsets computed once
    int k_goff[STAGE], k_loff[STAGE], v_goff[STAGE], v_loff[STAGE], v_key[STAGE];
    bool st_valid[STAGE], k_sel[STAGE], v_sel[STAGE];
#pragma unroll
    for (int i = 0; i < STAGE; ++i) {
        st_valid[i] = (int)threadIdx.x + 256 * i < kchunks;
        const int ci = min((int)threadIdx.x + 256 * i, kchunks - 1);
        const int key = ci / (D / 8), c8 = ci % (D / 8);
        k_sel[i] = (key >> 4) != 0;
        k_goff[i] = (key & 15) * D + 8 * c8;
        k_loff[i] = key * KPITCH + 8 * c8;
        const int d = ci >> 2, q4 = ci & 3;
        v_sel[i] = (q4 >> 1) != 0;
        v_goff[i] = d * P + 8 * (q4 & 1);
        v_loff[i] = d * VPITCH + 8 * q4;
        v_key[i] = 8 * q4;                             // first key of the chunk within the tile
    }
    // global -> registers.  No branch around a load: a load behind a branch makes the compiler wait for
    // every load in flight.  Addresses are clamped to valid memory (page 0 for a missing page, the last
    // chunk for a thread without one); what must read as zero is zeroed when the registers go to LDS.
    auto fetch = [&](int t, Staged& st) {
        const int tb = t * MFMA_TILE_KEYS;
        st.tb = tb;
        const int idx0 = min(max(tb / P - first_page, 0), PAGE_CACHE - 1);
        const int idx1 = min(max((tb + 16) / P - first_page, 0), PAGE_CACHE - 1);
        const int page0 = tb < ke ? page_lds[idx0] : -1;           // the host keeps the group's pages within the cache
        const int page1 = tb + 16 < ke ? page_lds[idx1] : -1;
        st.ok = (page0 >= 0 ? 1 : 0) | (page1 >= 0 ? 2 : 0);
        const size_t pk0 = (size_t)max(page0, 0) * a.kv_heads + kvh, pk1 = (size_t)max(page1, 0) * a.kv_heads + kvh;
        const __bf16* k0 = kp_base + (pk0 * P + tb % P) * D;
        const __bf16* k1 = kp_base + (pk1 * P + (tb + 16) % P) * D;
        const __bf16* v0 = vp_base + pk0 * D * P + tb % P;
        const __bf16* v1 = vp_base + pk1 * D * P + (tb + 16) % P;
#pragma unroll
        for (int i = 0; i < STAGE; ++i) {
            st.k[i] = *reinterpret_cast<const bf16x8*>((k_sel[i] ? k1 : k0) + k_goff[i]);
            st.v[i] = *reinterpret_cast<const bf16x8*>((v_sel[i] ? v1 : v0) + v_goff[i]);
        }
    };
    auto stash = [&](int buf, const Staged& st) {      // registers -> LDS
        const bool whole = st.ok == 3 && st.tb + MFMA_TILE_KEYS <= ke;    // the usual tile: nothing to zero
#pragma unroll
        for (int i = 0; i < STAGE; ++i) {
            if (!st_valid[i]) continue;
            bf16x8 kv = st.k[i], v = st.v[i];
            if (!whole) {
                if (!((st.ok >> (k_sel[i] ? 1 : 0)) & 1)) kv = zero8;
                if (!((st.ok >> (v_sel[i] ? 1 : 0)) & 1)) v = zero8;
                const int key0 = st.tb + v_key[i];
#pragma unroll
                for (int e = 0; e < 8; ++e)            // keys that are not written yet count as zero
                    if (key0 + e >= ke) v[e] = (__bf16)0.f;
            }
            *reinterpret_cast<bf16x8*>(&k_lds[buf][k_loff[i]]) = kv;
            *reinterpret_cast<bf16x4*>(&v_lds[buf][v_loff[i]]) = bf16x4{v[0], v[1], v[2], v[3]};
            *reinterpret_cast<bf16x4*>(&v_lds[buf][v_loff[i] + 4]) = bf16x4{v[4], v[5], v[6], v[7]};
        }
    };

    // Scores are kept in the base-2 domain: s * (scale * log2 e), so that a probability is one v_exp_f32.
    const float c2 = a.scale * 1.44269504088896340736f;
    const int wave_first_kend = pos0 + wtok0 + 1;                     // key range end of the wavefront's first token
    const int wave_last_kbegin = a.window > 0 ? max(0, wave_hi - a.window) : 0;
    auto compute = [&](int t, int buf) {
        const int tb = t * MFMA_TILE_KEYS;
        if (!wave_active || tb >= wave_hi || tb + MFMA_TILE_KEYS <= wave_lo) return;     // nothing for this wavefront
        floatx4 s[2];
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            s[j] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int c = 0; c < NCH; ++c) {
                // channels at and beyond head_dim were never staged: they must read as zero, not as whatever
                // the LDS held (a NaN there would turn the whole score into NaN)
                bf16x8 kf = zero8;
                if (32 * c + 8 * b < D)
                    kf = *reinterpret_cast<const bf16x8*>(&k_lds[buf][(16 * j + col) * KPITCH + 32 * c + 8 * b]);
                s[j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf, qf[c], s[j], 0, 0, 0);
            }
        }
        float sv[2][4];
        // a tile that every token of this wavefront sees whole needs no mask (all but the last one or two)
        const bool interior = tb + MFMA_TILE_KEYS <= wave_first_kend && tb >= wave_last_kbegin;
        if (interior) {
#pragma unroll
            for (int j = 0; j < 2; ++j)
#pragma unroll
                for (int r = 0; r < 4; ++r) sv[j][r] = s[j][r] * c2;
        } else {
#pragma unroll
            for (int j = 0; j < 2; ++j)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const int key = tb + 16 * j + 4 * b + r;
                    sv[j][r] = (key >= kbegin_c && key < kend_c) ? s[j][r] * c2 : -INFINITY;
                }
        }
        float tile_max = fmaxf(fmaxf(fmaxf(sv[0][0], sv[0][1]), fmaxf(sv[0][2], sv[0][3])),
                               fmaxf(fmaxf(sv[1][0], sv[1][1]), fmaxf(sv[1][2], sv[1][3])));
        tile_max = fmaxf(tile_max, __shfl_xor(tile_max, 16, MLR_WAVE));
        tile_max = fmaxf(tile_max, __shfl_xor(tile_max, 32, MLR_WAVE));
        // the running maximum rarely moves after the first tiles: rescale only when it does, for any column
        if (__builtin_amdgcn_ballot_w64(tile_max > m_run) != 0) {
            const float m_new = fmaxf(m_run, tile_max);
            const float corr = m_new > -INFINITY ? __builtin_amdgcn_exp2f(m_run - m_new) : 1.f;   // -inf - finite: 0
            l_run *= corr;
#pragma unroll
            for (int db = 0; db < 2 * NCH; ++db) o[db] *= corr;
            m_run = m_new;
        }
        const float m_use = fmaxf(m_run, -1e30f);      // a column with no key yet: exp2(-inf - finite) = 0, not NaN
        bf16x8 pf;
        float psum = 0.f;
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const float p = __builtin_amdgcn_exp2f(sv[j][r] - m_use);
                psum += p;
                pf[4 * j + r] = (__bf16)p;
            }
        l_run += psum;
#pragma unroll
        for (int db = 0; db < 2 * NCH; ++db) {
            if (16 * db >= D) break;
            const __bf16* vrow = &v_lds[buf][(16 * db + col) * VPITCH];
            const bf16x4 v0 = *reinterpret_cast<const bf16x4*>(vrow + 4 * b);
            const bf16x4 v1 = *reinterpret_cast<const bf16x4*>(vrow + 16 + 4 * b);
            const bf16x8 vf = {v0[0], v0[1], v0[2], v0[3], v1[0], v1[1], v1[2], v1[3]};
            o[db] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf, pf, o[db], 0, 0, 0);
        }
    };

    // Three tiles are under way at any time: one being multiplied out of LDS, two in flight from memory
    // into registers.  One barrier per tile suffices with two LDS buffers: a wavefront can only reach the
    // second write of a buffer after the barrier that follows every wavefront's read of it.
    const int t_begin = lo / MFMA_TILE_KEYS, t_end = (ke + MFMA_TILE_KEYS - 1) / MFMA_TILE_KEYS;
    // (fetches are unconditional, clamped to the last tile: a fetch behind a branch would again make
    // the compiler drain every load in flight)
    Staged sa, sb, sc;
    const int t_last = t_end - 1;
    fetch(t_begin, sa);
    fetch(min(t_begin + 1, t_last), sb);
    int buf = 0;
    for (int t = t_begin; t < t_end; t += 3) {
        fetch(min(t + 2, t_last), sc);
        stash(buf, sa);
        __syncthreads();
        compute(t, buf);
        buf ^= 1;
        if (t + 1 >= t_end) break;
        fetch(min(t + 3, t_last), sa);
        stash(buf, sb);
        __syncthreads();
        compute(t + 1, buf);
        buf ^= 1;
        if (t + 2 >= t_end) break;
        fetch(min(t + 4, t_last), sb);
        stash(buf, sc);
        __syncthreads();
        compute(t + 2, buf);
        buf ^= 1;
    }
    l_run += __shfl_xor(l_run, 16, MLR_WAVE);
    l_run += __shfl_xor(l_run, 32, MLR_WAVE);
    if (!col_valid) return;
    __bf16* dst = reinterpret_cast<__bf16*>(a.out) + ((size_t)(row0 + tok) * a.q_heads + kvh * g + hh) * D;
#pragma unroll
    for (int db = 0; db < 2 * NCH; ++db) {
        if (16 * db >= D) break;
        bf16x4 w4;
#pragma unroll
        for (int r = 0; r < 4; ++r) w4[r] = (__bf16)(l_run != 0.f ? o[db][r] / l_run : 0.f);
        *reinterpret_cast<bf16x4*>(dst + 16 * db + 4 * b) = w4;
    }
}

// A workgroup takes two groups, one after the other: group i and group (groups - 1 - i).  Within a long
// prompt the groups' key ranges grow with their position, so every workgroup gets about the same work.
template <int NCH>
__global__ __launch_bounds__(256, 2) void attention_prefill_kernel(AttnArgs a, const int32_t* __restrict__ group_row0,
                                                                const int32_t* __restrict__ group_ntok, int groups) {
    __shared__ __attribute__((aligned(16))) __bf16 k_lds[2][32 * (32 * NCH + 8)];
    __shared__ __attribute__((aligned(16))) __bf16 v_lds[2][32 * NCH * 36];
    __shared__ int32_t page_lds[PAGE_CACHE];          // the request's page ids for the group's key range
    const int first = blockIdx.x, second = groups - 1 - first;
    if (second > first) {
        prefill_group<NCH>(a, group_row0, group_ntok, second, blockIdx.y, k_lds, v_lds, page_lds);
        __syncthreads();
    }
    prefill_group<NCH>(a, group_row0, group_ntok, first, blockIdx.y, k_lds, v_lds, page_lds);
}

// The merge of key splits for the groups of `attention_mfma_kernel` (one wavefront per (group, head),
// walking the group's tokens).
__global__ __launch_bounds__(64) void attention_combine_groups_kernel(AttnArgs a, const int32_t* __restrict__ group_row0,
                                                                      const int32_t* __restrict__ group_ntok) {
    __shared__ float w_lds[COMBINE_MAX_SPLITS];
    __shared__ float l_lds[COMBINE_MAX_SPLITS];
    const int grp = blockIdx.x, head = blockIdx.y;
    const int D = a.head_dim;
    for (int j = 0; j < group_ntok[grp]; ++j) {
        const int m = group_row0[grp] + j;
        const int pos = a.positions[m];
        const int first = a.window > 0 ? max(0, pos + 1 - a.window) / a.split_keys : 0;
        const int last = min(a.max_splits - 1, pos / a.split_keys);
        const int n = last - first + 1;
        const float* base = a.partial + (((size_t)m * a.q_heads + head) * a.max_splits + first) * (D + 2);
        float gmax = -INFINITY;
        __syncthreads();
        for (int s = threadIdx.x; s < n; s += 64) {
            const float smax = base[(size_t)s * (D + 2) + D];
            w_lds[s] = smax;
            l_lds[s] = base[(size_t)s * (D + 2) + D + 1];
            gmax = fmaxf(gmax, smax);
        }
        gmax = wave_max(gmax);
        __syncthreads();
        for (int s = threadIdx.x; s < n; s += 64) {
            const float smax = w_lds[s];
            w_lds[s] = smax > -INFINITY ? __builtin_amdgcn_exp2f(smax - gmax) : 0.f;   // maxima are base-2 exponents
        }
        __syncthreads();
        float den = 0.f;
        for (int s = 0; s < n; ++s) den += w_lds[s] * l_lds[s];
        float num[MAX_DIM_REGS];
#pragma unroll
        for (int i = 0; i < MAX_DIM_REGS; ++i) num[i] = 0.f;
#pragma unroll 8
        for (int s = 0; s < n; ++s) {
            const float w = w_lds[s];
            const float* p = base + (size_t)s * (D + 2);
#pragma unroll
            for (int i = 0; i < MAX_DIM_REGS; ++i) {
                const int d = min((int)threadIdx.x + 64 * i, D - 1);      // clamped: no branch around the load
                num[i] += w * p[d];
            }
        }
#pragma unroll
        for (int i = 0; i < MAX_DIM_REGS; ++i) {
            const int d = threadIdx.x + 64 * i;
            if (d < D) a.out[((size_t)m * a.q_heads + head) * D + d] = from_float<elem_t>(den != 0.f ? num[i] / den : 0.f);
        }
    }
}

// The merge for `DecodeFusion`: one wavefront per (token, head).  Besides the splits' partial results it adds
// the token's own key and value (see `DecodeFusion`), and the first head of every kv head writes them
// into the cache.  A lane takes the rotation pairs lane and lane + 64 and the channels lane + 64 i.
__global__ __launch_bounds__(64) void attention_combine_fused_kernel(AttnArgs a, DecodeFusion f) {
    // (group i is batch row i here.)  Loads are asked for as early as their addresses are known: the row's
    // position and slot, its raw q, k, v and the norm weights at once; then what needs the position (the
    // rotation row, the page id, the splits' maxima and sums); then the splits' values, eight at a time.
    __shared__ float w_lds[COMBINE_MAX_SPLITS];
    const int m = blockIdx.x, head = blockIdx.y;
    const int D = a.head_dim, P = a.page_size, half = D >> 1;
    const int g = a.q_heads / a.kv_heads, kvh = head / g;
    const int lane = threadIdx.x;
    const int pos = a.positions[m], slot = a.slots[m];
    const __bf16* row = f.qkv + (size_t)m * f.ld;
    const __bf16* qs = row + (size_t)head * D;
    const __bf16* ks = row + (size_t)(a.q_heads + kvh) * D;
    const __bf16* vs = row + (size_t)(a.q_heads + a.kv_heads + kvh) * D;
    const bool normed = f.q_norm_w != nullptr, rotated = f.rope != nullptr;
    const float* qw = normed ? f.q_norm_w : reinterpret_cast<const float*>(row);      // (any readable address)
    const float* kw = normed ? f.k_norm_w : reinterpret_cast<const float*>(row);
    float qa[2], qb[2], ka[2], kb[2], qwa[2], qwb[2], kwa[2], kwb[2], vv[MAX_DIM_REGS];
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const int j = min(lane + 64 * i, half - 1);
        qa[i] = (float)qs[j];
        qb[i] = (float)qs[j + half];
        ka[i] = (float)ks[j];
        kb[i] = (float)ks[j + half];
        qwa[i] = qw[j];
        qwb[i] = qw[j + half];
        kwa[i] = kw[j];
        kwb[i] = kw[j + half];
    }
#pragma unroll
    for (int i = 0; i < MAX_DIM_REGS; ++i) vv[i] = (float)vs[min(lane + 64 * i, D - 1)];
    // second round: everything that needs the position
    const float* cs = (rotated ? f.rope : reinterpret_cast<const float*>(a.positions)) + (rotated ? (size_t)pos * D : 0);
    float co[2], si[2];
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const int j = rotated ? min(lane + 64 * i, half - 1) : 0;
        co[i] = cs[j];
        si[i] = cs[rotated ? j + half : 0];
    }
    const int page_read = a.block_table[(size_t)slot * a.max_blocks + min(pos / P, a.max_blocks - 1)];
    const int page = pos / P < a.max_blocks ? page_read : -1;    // (beyond the request's row of the table: no page)
    const int glo = a.window > 0 ? max(0, pos + 1 - a.window) : 0;
    const int first = a.max_splits > 1 ? glo / a.split_keys : 0;
    const int last = a.max_splits > 1 ? min(a.max_splits - 1, max(pos - 1, 0) / a.split_keys) : 0;
    const int n = last - first + 1;                     // the same range of splits that the attention kernel served
    const float* base = a.partial + (((size_t)m * a.q_heads + head) * a.max_splits + first) * (D + 2);
    float smax[COMBINE_MAX_SPLITS / 64], ssum[COMBINE_MAX_SPLITS / 64];
    float gmax = -INFINITY;
#pragma unroll
    for (int r = 0; r < COMBINE_MAX_SPLITS / 64; ++r) {
        const int s = lane + 64 * r;
        if (64 * r >= n) break;
        const float* p = base + (size_t)min(s, n - 1) * (D + 2);
        smax[r] = s < n ? p[D] : -INFINITY;
        ssum[r] = p[D + 1];
        gmax = fmaxf(gmax, smax[r]);
    }

    // query and key of this token: norm, rotation, rounded to bfloat16 (what the cache holds)
    float qsum = 0.f, ksum = 0.f;
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        if (lane + 64 * i >= half) qa[i] = qb[i] = ka[i] = kb[i] = 0.f;
        qsum += squares(qa[i], qb[i]);
        ksum += squares(ka[i], kb[i]);
    }
    if (normed) {
        qsum = wave_sum(qsum);
        ksum = wave_sum(ksum);
        const float qscale = 1.0f / sqrtf(qsum / (float)D + f.eps), kscale = 1.0f / sqrtf(ksum / (float)D + f.eps);
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            qa[i] = (qa[i] * qscale) * qwa[i];
            qb[i] = (qb[i] * qscale) * qwb[i];
            ka[i] = (ka[i] * kscale) * kwa[i];
            kb[i] = (kb[i] * kscale) * kwb[i];
        }
    }
    float dot = 0.f;
    __bf16 k_lo[2], k_hi[2];
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        float qx = qa[i], qy = qb[i], kx = ka[i], ky = kb[i];
        if (rotated) {
            qx = turn_x(qa[i], qb[i], co[i], si[i]);
            qy = turn_y(qa[i], qb[i], co[i], si[i]);
            kx = turn_x(ka[i], kb[i], co[i], si[i]);
            ky = turn_y(ka[i], kb[i], co[i], si[i]);
        }
        k_lo[i] = (__bf16)kx;
        k_hi[i] = (__bf16)ky;
        if (lane + 64 * i < half)
            dot += (float)(__bf16)qx * (float)k_lo[i] + (float)(__bf16)qy * (float)k_hi[i];
    }
    const float s_own = wave_sum(dot) * (a.scale * 1.44269504088896340736f);     // base-2 domain, as the partial maxima
    gmax = fmaxf(wave_max(gmax), s_own);
    // the splits' weights (maxima are base-2 exponents) and the denominator, summed in ascending order
#pragma unroll
    for (int r = 0; r < COMBINE_MAX_SPLITS / 64; ++r) {
        const int s = lane + 64 * r;
        if (64 * r >= n) break;
        if (s < n) w_lds[s] = smax[r] > -INFINITY ? __builtin_amdgcn_exp2f(smax[r] - gmax) * 1.0f : 0.f;
    }
    __syncthreads();
    float den = 0.f;
#pragma unroll
    for (int r = 0; r < COMBINE_MAX_SPLITS / 64; ++r) {
        const int s = lane + 64 * r;
        if (64 * r >= n) break;
        den += s < n ? w_lds[s] * ssum[r] : 0.f;
    }
    den = wave_sum(den);
    float num[MAX_DIM_REGS];
#pragma unroll
    for (int i = 0; i < MAX_DIM_REGS; ++i) num[i] = 0.f;
#pragma unroll 8
    for (int s = 0; s < n; ++s) {
        const float w = w_lds[s];
        const float* p = base + (size_t)s * (D + 2);
#pragma unroll
        for (int i = 0; i < MAX_DIM_REGS; ++i) num[i] += w * p[min(lane + 64 * i, D - 1)];     // clamped: no branch around the load
    }
    const float w_own = __builtin_amdgcn_exp2f(s_own - gmax);
    den += w_own;
#pragma unroll
    for (int i = 0; i < MAX_DIM_REGS; ++i) {
        const int d = lane + 64 * i;
        if (d < D) a.out[((size_t)m * a.q_heads + head) * D + d] = from_float<elem_t>((num[i] + w_own * vv[i]) / den);
    }
    // key and value into their pages, once per kv head
    if (head != kvh * g || page < 0) return;
    const size_t pk = (size_t)page * a.kv_heads + kvh;
    __bf16* kdst = reinterpret_cast<__bf16*>(const_cast<elem_t*>(a.k_pages)) + (pk * P + pos % P) * D;
    __bf16* vdst = reinterpret_cast<__bf16*>(const_cast<elem_t*>(a.v_pages)) + pk * D * P + pos % P;
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const int j = lane + 64 * i;
        if (j < half) {
            kdst[j] = k_lo[i];
            kdst[j + half] = k_hi[i];
        }
    }
#pragma unroll
    for (int i = 0; i < MAX_DIM_REGS; ++i) {
        const int d = lane + 64 * i;
        if (d < D) vdst[(size_t)d * P] = (__bf16)vv[i];
    }
}

// Decoding with `DecodeFusion`: group i is the one token in batch row i (group_row0[i] = i, group_ntok[i] = 1);
// qkv holds the raw projections
// [rows, ld].  Key and value of every token are written into the cache.  `partial` holds at least
// rows * q_heads * max(max_splits, 1) * (head_dim + 2) floats, also without splits.
// Needs what `mlr_attention_mfma` needs and head_dim % 64 == 0.
extern "C" int mlr_attention_decode_fused(
    const void* qkv, int ld, const void* k_pages, const void* v_pages, const int32_t* block_table, int max_blocks,
    const int32_t* slots, const int32_t* positions, void* out, float* partial, const int32_t* group_row0,
    const int32_t* group_ntok, int groups, int q_heads, int kv_heads, int head_dim, int page_size, int window,
    float scale, int split_keys, int max_splits, const float* q_norm_w, const float* k_norm_w, float eps,
    const float* rope, hipStream_t stream) {
    if (groups <= 0) return 0;
    if (head_dim % 64 != 0 || head_dim > 256 || page_size % 16 != 0 || q_heads % kv_heads != 0 ||
        q_heads / kv_heads > 16 || partial == nullptr || (q_norm_w == nullptr) != (k_norm_w == nullptr)) return -1;
    if (max_splits < 1) max_splits = 1;
    if (max_splits > 1 && (split_keys <= 0 || split_keys % MFMA_TILE_KEYS != 0 || max_splits > COMBINE_MAX_SPLITS)) return -2;
    if ((max_splits > 1 ? split_keys / page_size + 2 : max_blocks) > DECODE_PAGE_CACHE) return -3;
    AttnArgs a{nullptr, (const elem_t*)k_pages, (const elem_t*)v_pages, block_table, slots,
               positions, (elem_t*)out, partial, max_blocks, q_heads, kv_heads, head_dim, page_size,
               window, split_keys, max_splits, scale};
    DecodeFusion f{(const __bf16*)qkv, q_norm_w, k_norm_w, rope, ld, eps};
    dim3 grid(groups, kv_heads, max_splits);
    const size_t lds = sizeof(float) * 3 * (16 * (size_t)head_dim + 32);
    switch (head_dim / 32) {
        case 2: attention_mfma_kernel<2, true><<<grid, 256, lds, stream>>>(a, group_row0, group_ntok, f); break;
        case 4: attention_mfma_kernel<4, true><<<grid, 256, lds, stream>>>(a, group_row0, group_ntok, f); break;
        case 6: attention_mfma_kernel<6, true><<<grid, 256, lds, stream>>>(a, group_row0, group_ntok, f); break;
        default: attention_mfma_kernel<8, true><<<grid, 256, lds, stream>>>(a, group_row0, group_ntok, f); break;
    }
    int err = (int)hipGetLastError();
    if (err != 0) return err;
    attention_combine_fused_kernel<<<dim3(groups, q_heads), 64, 0, stream>>>(a, f);
    return (int)hipGetLastError();
}

// Groups: group_row0[i] = first batch row of group i, group_ntok[i] = its tokens (consecutive rows of one
// request, ntok * (q_heads / kv_heads) <= 16).  Rows outside the groups are left alone.
// Needs page_size % 16 == 0, head_dim % 16 == 0, q_heads / kv_heads <= 16.
extern "C" int mlr_attention_mfma(
    const void* q, const void* k_pages, const void* v_pages, const int32_t* block_table, int max_blocks,
    const int32_t* slots, const int32_t* positions, void* out, float* partial,
    const int32_t* group_row0, const int32_t* group_ntok, int groups, int rows, int q_heads, int kv_heads,
    int head_dim, int page_size, int window, float scale, int split_keys, int max_splits, hipStream_t stream) {
    (void)rows;
    if (groups <= 0) return 0;
    if (head_dim % 16 != 0 || head_dim > 256 || page_size % 16 != 0 || q_heads % kv_heads != 0 ||
        q_heads / kv_heads > 16) return -1;
    if (max_splits > 1 && (partial == nullptr || split_keys <= 0 || split_keys % MFMA_TILE_KEYS != 0 ||
                           max_splits > COMBINE_MAX_SPLITS)) return -2;
    // a workgroup keeps the page ids of its key range in LDS
    if ((max_splits > 1 ? split_keys / page_size + 2 : max_blocks) > DECODE_PAGE_CACHE) return -3;
    AttnArgs a{(const elem_t*)q, (const elem_t*)k_pages, (const elem_t*)v_pages, block_table, slots,
               positions, (elem_t*)out, partial, max_blocks, q_heads, kv_heads, head_dim, page_size,
               window, split_keys, max_splits < 1 ? 1 : max_splits, scale};
    dim3 grid(groups, kv_heads, a.max_splits);
    const size_t lds = sizeof(float) * 3 * (16 * (size_t)head_dim + 32);
    const int nch = (head_dim + 31) / 32;
    switch (nch) {
        case 1: attention_mfma_kernel<1, false><<<grid, 256, lds, stream>>>(a, group_row0, group_ntok, DecodeFusion{}); break;
        case 2: attention_mfma_kernel<2, false><<<grid, 256, lds, stream>>>(a, group_row0, group_ntok, DecodeFusion{}); break;
        case 3: attention_mfma_kernel<3, false><<<grid, 256, lds, stream>>>(a, group_row0, group_ntok, DecodeFusion{}); break;
        case 4: attention_mfma_kernel<4, false><<<grid, 256, lds, stream>>>(a, group_row0, group_ntok, DecodeFusion{}); break;
        case 5: attention_mfma_kernel<5, false><<<grid, 256, lds, stream>>>(a, group_row0, group_ntok, DecodeFusion{}); break;
        case 6: attention_mfma_kernel<6, false><<<grid, 256, lds, stream>>>(a, group_row0, group_ntok, DecodeFusion{}); break;
        case 7: attention_mfma_kernel<7, false><<<grid, 256, lds, stream>>>(a, group_row0, group_ntok, DecodeFusion{}); break;
        default: attention_mfma_kernel<8, false><<<grid, 256, lds, stream>>>(a, group_row0, group_ntok, DecodeFusion{}); break;
    }
    int err = (int)hipGetLastError();
    if (err != 0) return err;
    if (a.max_splits > 1) {
        attention_combine_groups_kernel<<<dim3(groups, q_heads), 64, 0, stream>>>(a, group_row0, group_ntok);
        err = (int)hipGetLastError();
    }
    return err;
}

// Prompt portions: groups of up to 4 * (16 / g) consecutive tokens of one request each, no key splits.
// A group's keys must span at most PAGE_CACHE (2048) pages: the caller sends longer contexts to
// `mlr_attention_mfma`.
extern "C" int mlr_attention_prefill(
    const void* q, const void* k_pages, const void* v_pages, const int32_t* block_table, int max_blocks,
    const int32_t* slots, const int32_t* positions, void* out, const int32_t* group_row0,
    const int32_t* group_ntok, int groups, int q_heads, int kv_heads, int head_dim, int page_size, int window,
    float scale, hipStream_t stream) {
    if (groups <= 0) return 0;
    if (head_dim % 16 != 0 || head_dim > 192 || page_size % 16 != 0 || q_heads % kv_heads != 0 ||
        q_heads / kv_heads > 16) return -1;            // 192: the two LDS tile buffers and the page ids fit 64 KB
    AttnArgs a{(const elem_t*)q, (const elem_t*)k_pages, (const elem_t*)v_pages, block_table, slots,
               positions, (elem_t*)out, nullptr, max_blocks, q_heads, kv_heads, head_dim, page_size,
               window, 0, 1, scale};
    dim3 grid((groups + 1) / 2, kv_heads);
    const int nch = (head_dim + 31) / 32;
    switch (nch) {
        case 1: attention_prefill_kernel<1><<<grid, 256, 0, stream>>>(a, group_row0, group_ntok, groups); break;
        case 2: attention_prefill_kernel<2><<<grid, 256, 0, stream>>>(a, group_row0, group_ntok, groups); break;
        case 3: attention_prefill_kernel<3><<<grid, 256, 0, stream>>>(a, group_row0, group_ntok, groups); break;
        case 4: attention_prefill_kernel<4><<<grid, 256, 0, stream>>>(a, group_row0, group_ntok, groups); break;
        case 5: attention_prefill_kernel<5><<<grid, 256, 0, stream>>>(a, group_row0, group_ntok, groups); break;
        default: attention_prefill_kernel<6><<<grid, 256, 0, stream>>>(a, group_row0, group_ntok, groups); break;
    }
    return (int)hipGetLastError();
}
#endif
