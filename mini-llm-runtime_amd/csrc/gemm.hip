// out[M, N] = a[M, K] . w[N, K]^T  (both operands row-major with K contiguous, the layout of
// an activation and of a projection's weight), accumulated in 32-bit.
//
// Float engine: a plain tiled FMA kernel; every output element is one sequential sum over k,
// so a row's result does not depend on the other rows of the batch.
// Bfloat16 engine, three families, each with a fixed k order for every output element (so a row's result
// does not depend on the rows beside it): up to 64 rows the weight is streamed once straight into
// v_mfma_f32_16x16x32_bf16 (`gemm_skinny_kernel`, optionally with the residual add and RMSNorm in front
// or silu(gate) * up behind); more rows with k a multiple of 64 go to `gemm_wide_kernel` (32x32 tiles
// out of double-buffered LDS blocks); any other k to the plain 16x16-tile kernel `gemm_bf16_kernel`.
#include "common.h"
#include <type_traits>

#if !MLR_BF16
// ------------------------------------------------------------------------------ float
#define BM 64
#define BN 64
#define BK 16

__global__ __launch_bounds__(256) void gemm_f32_kernel(const float* __restrict__ a,
                                                       const float* __restrict__ w,
                                                       float* __restrict__ out, int M, int N, int K) {
    __shared__ float as[BK][BM + 4];
    __shared__ float ws[BK][BN + 4];
    const int t = threadIdx.x;
    const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
    const int tx = t % 16, ty = t / 16;
    const int lrow = t / 4, lk = (t % 4) * 4;       // this thread stages row lrow, k lk..lk+3
    float acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;

    for (int k0 = 0; k0 < K; k0 += BK) {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int k = k0 + lk + e;
            const int am = m0 + lrow, wn = n0 + lrow;
            as[lk + e][lrow] = (am < M && k < K) ? a[(size_t)am * K + k] : 0.f;
            ws[lk + e][lrow] = (wn < N && k < K) ? w[(size_t)wn * K + k] : 0.f;
        }
        __syncthreads();
#pragma unroll
        for (int k = 0; k < BK; ++k) {
            float av[4], wv[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) av[i] = as[k][ty * 4 + i];
#pragma unroll
            for (int j = 0; j < 4; ++j) wv[j] = ws[k][tx * 4 + j];
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(av[i], wv[j], acc[i][j]);
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int m = m0 + ty * 4 + i;
        if (m >= M) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int n = n0 + tx * 4 + j;
            if (n < N) out[(size_t)m * N + n] = acc[i][j];
        }
    }
}

extern "C" int mlr_gemm(const void* a, const void* w, void* out, int M, int N, int K, int out_float,
                        hipStream_t stream) {
    (void)out_float;                                   // the float engine's outputs are float
    if (M <= 0 || N <= 0) return 0;
    if (K <= 0) return -1;
    dim3 grid((N + BN - 1) / BN, (M + BM - 1) / BM);
    if (grid.y > 65535) return -2;
    gemm_f32_kernel<<<grid, 256, 0, stream>>>((const float*)a, (const float*)w, (float*)out, M, N, K);
    return (int)hipGetLastError();
}

#else
// ------------------------------------------------------------------------------ bfloat16
typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float floatx4;

#define BK 32
#define LDS_STRIDE (BK + 8)      // in elements: rows 80 bytes apart

// Eight consecutive k of one row as a 16-byte vector; zero beyond the matrix.
__device__ __forceinline__ bf16x8 load_k8(const __bf16* base, int row, int rows, int k, int K,
                                          bool vector_ok) {
    bf16x8 v = {0, 0, 0, 0, 0, 0, 0, 0};
    if (row < rows) {
        const __bf16* p = base + (size_t)row * K + k;
        if (vector_ok && k + 8 <= K) {
            v = *reinterpret_cast<const bf16x8*>(p);
        } else {
#pragma unroll
            for (int e = 0; e < 8; ++e)
                if (k + e < K) v[e] = p[e];
        }
    }
    return v;
}

// Workgroup tile (WM * TM * 16) x (WN * TN * 16); WM x WN wavefronts, each TM x TN MFMA tiles.
template <int WM, int WN, int TM, int TN, bool OUT_FLOAT>
__global__ __launch_bounds__(WM * WN * 64) void gemm_bf16_kernel(
    const __bf16* __restrict__ a, const __bf16* __restrict__ w, void* __restrict__ out_raw,
    int M, int N, int K) {
    constexpr int BM = WM * TM * 16, BN = WN * TN * 16, THREADS = WM * WN * 64;
    __shared__ __bf16 as[BM * LDS_STRIDE];
    __shared__ __bf16 ws[BN * LDS_STRIDE];
    const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
    const int wm = wave / WN, wn = wave % WN;
    const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
    const bool vector_ok = (K % 8) == 0;

    floatx4 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) acc[i][j] = floatx4{0.f, 0.f, 0.f, 0.f};

    for (int k0 = 0; k0 < K; k0 += BK) {
        for (int c = t; c < BM * 4; c += THREADS) {           // 4 chunks of 8 per row
            const int r = c >> 2, kc = (c & 3) * 8;
            *reinterpret_cast<bf16x8*>(&as[r * LDS_STRIDE + kc]) =
                load_k8(a, m0 + r, M, k0 + kc, K, vector_ok);
        }
        for (int c = t; c < BN * 4; c += THREADS) {
            const int r = c >> 2, kc = (c & 3) * 8;
            *reinterpret_cast<bf16x8*>(&ws[r * LDS_STRIDE + kc]) =
                load_k8(w, n0 + r, N, k0 + kc, K, vector_ok);
        }
        __syncthreads();
        bf16x8 af[TM], wf[TN];
        const int frag_row = lane & 15, frag_k = (lane >> 4) * 8;
#pragma unroll
        for (int i = 0; i < TM; ++i)
            af[i] = *reinterpret_cast<const bf16x8*>(
                &as[((wm * TM + i) * 16 + frag_row) * LDS_STRIDE + frag_k]);
#pragma unroll
        for (int j = 0; j < TN; ++j)
            wf[j] = *reinterpret_cast<const bf16x8*>(
                &ws[((wn * TN + j) * 16 + frag_row) * LDS_STRIDE + frag_k]);
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j)
                acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(af[i], wf[j], acc[i][j], 0, 0, 0);
        __syncthreads();
    }

    // accumulator element r of a lane: row (lane / 16) * 4 + r, column lane % 16
#pragma unroll
    for (int i = 0; i < TM; ++i) {
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            const int n = n0 + (wn * TN + j) * 16 + (lane & 15);
            if (n >= N) continue;
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int m = m0 + (wm * TM + i) * 16 + (lane >> 4) * 4 + r;
                if (m >= M) continue;
                if (OUT_FLOAT) ((float*)out_raw)[(size_t)m * N + n] = acc[i][j][r];
                else ((__bf16*)out_raw)[(size_t)m * N + n] = (__bf16)acc[i][j][r];
            }
        }
    }
}

// Few rows (M <= 64): the weight is streamed once, straight from memory into the matrix cores.  A
// workgroup owns 16 output columns (16 rows of w); its eight wavefronts each take an eighth of k, and
// their partial sums are added in the order 0..7, so the result does not depend on M.  The weight
// is the A operand (rows n), the activation the B operand (columns m): a lane ends up with four
// consecutive n of one m.
// GATED: w holds two stacked matrices [gate; up] of N rows each; the workgroup computes the same 16
// columns of both and writes silu(gate) * up (the feed-forward's activation fused into the projection).
// STAGE (M <= 16, K a multiple of 64): a wavefront reads its part of the activation as M rows of
// consecutive bytes, puts them into a piece of LDS of its own and takes its operand from there.  Read
// straight into the operand layout, the activation costs as many requests to the cache as the weight
// does to memory, and the weight's rate drops by a tenth to a third (measured; more with more rows).
#define SKINNY_WAVES 8
#define SKINNY_STAGE_PITCH(U) ((U) * 128 + 16)        // bytes a row of the staged activation takes
#define SKINNY_STAGE_LDS (66 * 1024)                  // the most dynamic LDS a workgroup asks for

// What a skinny product of up to 16 rows may do with its sums before it stores them: the two halves of an
// RMSNorm that is handed from the projection before it to the projection after it.
//   EPI_SCALE (the projection after the norm): its input is x * norm_w, rounded, WITHOUT the row's scale
//     rsqrt(mean(x^2) + eps), because whoever produced x knew only partial sums of squares; the scale is a
//     factor per row, so it is applied here, in 32-bit, to the finished sums: out[m] *= rsqrt(sum_p ss[m][p] *
//     inv_size + eps).  The partial sums are added in a fixed order (see the kernel).
//   EPI_RESIDUAL (the projection before the norm, which ends a mixer or a feed-forward): its sums are added
//     to the residual stream, h[m][n] += out[m][n], in 32-bit and in place (every element belongs to one
//     lane); when a norm follows (next_w != null) it also writes x_out = bf16(h * next_w) and, per row and
//     workgroup (16 columns), the sum of squares of its 16 new values of h: ss_out[m][workgroup].
#define EPI_NONE 0
#define EPI_SCALE 1
#define EPI_RESIDUAL 2
struct SkinnyEpilogue {
    const float* ss;          // EPI_SCALE: [M][ss_parts] partial sums of squares of the rows
    int ss_parts;
    int ss_vec;               // ss_parts is a multiple of 4 and ss 16-byte aligned: four sums a load
    float eps, inv_size;
    float* h;                 // EPI_RESIDUAL: [M][N] the residual stream
    const float* next_w;      // [N] weights of the norm that follows, or null
    __bf16* x_out;            // [M][N]
    float* ss_out;            // [M][gridDim.x]
    int cols;                 // PAIR: the output columns of a workgroup, 17..32 (otherwise 16, whatever this says)
    int ss_stride;            // floats between the rows of ss_out (its capacity: a strip of 16 a part)
};

// PAIR: a workgroup owns `cols` (17..32) output columns, two strips side by side, the second one partly
// used: for a number of columns that deals strips of 16 unevenly to the compute units (384 strips on 256
// units take as long as 512), 24 columns a workgroup give every unit the same work.  The second strip
// rides where GATED keeps its second matrix.
template <int MT, bool OUT_FLOAT, bool GATED, int UMAX = 4, bool STAGE = false, int EPI = EPI_NONE, bool PAIR = false>   // UMAX: the most groups of k a turn takes
__global__ __launch_bounds__(SKINNY_WAVES * 64) void gemm_skinny_kernel(const __bf16* __restrict__ a,
                                                               const __bf16* __restrict__ w,
                                                               void* __restrict__ out_raw, int M, int N, int K,
                                                               SkinnyEpilogue epi) {
    constexpr int NW = (GATED || PAIR) ? 2 : 1;
    static_assert(!PAIR || (MT == 1 && !GATED && !STAGE), "two strips: a plain product of few rows");
    static_assert(!STAGE || MT == 1, "the activation is staged for at most 16 rows");
    static_assert(EPI == EPI_NONE || MT == 1, "the norm is handed over for at most 16 rows");
    static_assert(EPI != EPI_RESIDUAL || (!GATED && !OUT_FLOAT), "the residual sum follows a plain projection");
    __shared__ float part[SKINNY_WAVES - 1][NW][MT][64][4];
    __shared__ float ss_lds[SKINNY_WAVES][16];
    extern __shared__ __attribute__((aligned(16))) char staged[];   // [SKINNY_WAVES][M][pitch] when STAGE
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int r16 = lane & 15, b = lane >> 4;
    const int cols = PAIR ? epi.cols : 16;
    const int n0 = blockIdx.x * cols;
    const int last_row = PAIR ? min(N - 1, n0 + cols - 1) : N - 1;     // (PAIR: rows beyond the workgroup's columns read its last one)
    // this lane's weight row for g = 0 and for g = 1 (GATED: the same row of the second matrix; PAIR: 16 rows on)
    const int wrow_of[2] = {min(n0 + r16, N - 1), GATED ? N + min(n0 + r16, N - 1) : min(n0 + 16 + r16, last_row)};
    const bool vector_ok = (K % 8) == 0;
    const int steps = (K + 31) / 32;
    const int per_wave = (steps + SKINNY_WAVES - 1) / SKINNY_WAVES;
    const int s_begin = wave * per_wave, s_end = min(steps, s_begin + per_wave);
    // What the epilogue needs from memory is asked for here, before the weight, by every wavefront alike
    // (no branch around a load); only wavefront 0 uses it.
    float ss_mine = 0.f;                                   // EPI_SCALE: this lane's share of the row's partial sums
    float4 h4 = make_float4(0.f, 0.f, 0.f, 0.f), nw4 = h4;  // EPI_RESIDUAL: h and the next norm's weights at (row r16, columns n0 + 4 b ..)
    float4 h4b = h4, nw4b = h4;                            // ... and, PAIR, at the second strip's columns n0 + 16 + 4 b ..
    if constexpr (EPI == EPI_SCALE) {
        // the row's partial sums are dealt out to the 32 (wavefront, lane block) pairs in runs of q; a run is
        // added in ascending order (four sums that lie side by side as (0 + 1) + (2 + 3) first, when their number
        // allows 16-byte loads), the four runs of a wavefront as (0 + 1) + (2 + 3), the wavefronts in the order
        // 0..7: an order that depends on nothing but the number of partial sums.  Four loads are asked for before
        // the first is used: a load a turn of the loop would cost a trip to the cache each, one after the other,
        // before the workgroup has asked for any of its weight.
        const float* row = epi.ss + (size_t)min(r16, M - 1) * epi.ss_parts;
        const int pair = wave * 4 + b;
        if (epi.ss_vec) {
            const int quads = epi.ss_parts >> 2;
            const int q = (quads + 4 * SKINNY_WAVES - 1) / (4 * SKINNY_WAVES);
            const float4* row4 = reinterpret_cast<const float4*>(row);
            for (int j0 = 0; j0 < q; j0 += 4) {
                float4 v[4];
#pragma unroll
                for (int j = 0; j < 4; ++j) v[j] = row4[min(pair * q + j0 + j, quads - 1)];
                asm volatile("" : "+v"(v[0].x), "+v"(v[1].x), "+v"(v[2].x), "+v"(v[3].x));   // (all four are loaded, none behind a branch)
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const bool mine = j0 + j < q && pair * q + j0 + j < quads;
                    ss_mine += mine ? (v[j].x + v[j].y) + (v[j].z + v[j].w) : 0.f;
                }
            }
        } else {
            const int q = (epi.ss_parts + 4 * SKINNY_WAVES - 1) / (4 * SKINNY_WAVES);
            for (int j0 = 0; j0 < q; j0 += 4) {
                float v[4];
#pragma unroll
                for (int j = 0; j < 4; ++j) v[j] = row[min(pair * q + j0 + j, epi.ss_parts - 1)];
                asm volatile("" : "+v"(v[0]), "+v"(v[1]), "+v"(v[2]), "+v"(v[3]));
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const bool mine = j0 + j < q && pair * q + j0 + j < epi.ss_parts;
                    ss_mine += mine ? v[j] : 0.f;
                }
            }
        }
    }
    if constexpr (EPI == EPI_RESIDUAL) {
        const int n = min(n0 + 4 * b, max(N - 4, 0));      // (clamped: a narrow last strip is handled element by element below)
        const size_t at = (size_t)min(r16, M - 1) * N + n;
        if ((N & 3) == 0) {
            h4 = *reinterpret_cast<const float4*>(epi.h + at);
            if (epi.next_w) nw4 = *reinterpret_cast<const float4*>(epi.next_w + n);
            if constexpr (PAIR) {                         // (PAIR is only launched for N and cols that are multiples of 4)
                const int n2 = min(n0 + 16 + 4 * b, N - 4);
                h4b = *reinterpret_cast<const float4*>(epi.h + (size_t)min(r16, M - 1) * N + n2);
                if (epi.next_w) nw4b = *reinterpret_cast<const float4*>(epi.next_w + n2);
            }
        }
    }
    floatx4 acc[NW][MT];
#pragma unroll
    for (int g = 0; g < NW; ++g)
#pragma unroll
        for (int i = 0; i < MT; ++i) acc[g][i] = floatx4{0.f, 0.f, 0.f, 0.f};
    if ((K & 63) == 0) {
        // The usual case, K a multiple of 64: no branch anywhere near a load (a load behind a branch makes
        // the compiler wait for every load in flight).  Rows beyond N or M read the last valid row; what
        // they produce is never stored.  Two k steps are taken together: a lane reads 32 consecutive bytes
        // of its weight row (four lanes a whole 128-byte line), each 16 of them feed one product; the
        // activation is read the same way, so the k slots of both operands agree.  (Measured: 64 bytes a
        // lane is slower again.)
        constexpr int W = 2;                              // 16-byte chunks per lane and group
        const int groups = steps / W;
        const int per_wave_g = (groups + SKINNY_WAVES - 1) / SKINNY_WAVES;
        const int g_begin = wave * per_wave_g, g_end = min(groups, g_begin + per_wave_g);
        const __bf16* wrow[NW];
#pragma unroll
        for (int g = 0; g < NW; ++g) wrow[g] = w + (size_t)wrow_of[g] * K + b * (8 * W);
        const __bf16* xrow[MT];
#pragma unroll
        for (int i = 0; i < MT; ++i) xrow[i] = a + (size_t)min(16 * i + r16, M - 1) * K + b * (8 * W);
        // Full turns of U groups first: every load of a turn (the activation, which comes from the cache,
        // before the weight that follows it in the queue) is asked for before the first product, with no
        // branch in between.  What is left (fewer than U groups) makes one shorter turn.
        constexpr int U = (MT * NW <= 2 && UMAX >= 4) ? 4 : 2;
        constexpr int PITCH = SKINNY_STAGE_PITCH(U);
        char* mine = staged + (size_t)wave * M * PITCH;
        auto turn = [&](int g0, auto count) {
            constexpr int C = decltype(count)::value;
            constexpr int PPR = C * 8;                        // 16-byte pieces in a row of this turn's chunk
            bf16x8 xf[MT][C][W], wf[NW][C][W], xg[STAGE ? C * W : 1];
            if constexpr (STAGE) {
                // piece p of the chunk: row p / PPR, bytes 16 * (p % PPR); a lane takes pieces lane, lane + 64, ...
#pragma unroll
                for (int i = 0; i < C * W; ++i) {
                    const int p = min(i * 64 + lane, M * PPR - 1);
                    xg[i] = *reinterpret_cast<const bf16x8*>(a + (size_t)(p / PPR) * K + (g0 * (32 * W) + (p % PPR) * 8));
                }
            } else {
#pragma unroll
                for (int u = 0; u < C; ++u)
#pragma unroll
                    for (int i = 0; i < MT; ++i)
#pragma unroll
                        for (int c = 0; c < W; ++c)
                            xf[i][u][c] = *reinterpret_cast<const bf16x8*>(xrow[i] + (g0 + u) * (32 * W) + 8 * c);
            }
#pragma unroll
            for (int u = 0; u < C; ++u)
#pragma unroll
                for (int g = 0; g < NW; ++g)
#pragma unroll
                    for (int c = 0; c < W; ++c)
                        wf[g][u][c] = *reinterpret_cast<const bf16x8*>(wrow[g] + (g0 + u) * (32 * W) + 8 * c);
            __builtin_amdgcn_sched_barrier(0);            // or the compiler spreads the loads among the products
            if constexpr (STAGE) {
                // LDS serves a wavefront's accesses in their order: the reads below see these writes, and
                // the next turn's writes come after these reads.  Rows from M on read row M - 1.
#pragma unroll
                for (int i = 0; i < C * W; ++i) {
                    const int p = i * 64 + lane;
                    if (p < M * PPR) *reinterpret_cast<bf16x8*>(mine + (p / PPR) * PITCH + (p % PPR) * 16) = xg[i];
                }
                const char* row = mine + min(r16, M - 1) * PITCH + b * (16 * W);
#pragma unroll
                for (int u = 0; u < C; ++u)
#pragma unroll
                    for (int c = 0; c < W; ++c)
                        xf[0][u][c] = *reinterpret_cast<const bf16x8*>(row + u * (64 * W) + 16 * c);
            }
#pragma unroll
            for (int u = 0; u < C; ++u)
#pragma unroll
                for (int i = 0; i < MT; ++i)
#pragma unroll
                    for (int c = 0; c < W; ++c)
#pragma unroll
                        for (int g = 0; g < NW; ++g)
                            acc[g][i] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[g][u][c], xf[i][u][c], acc[g][i], 0, 0, 0);
        };
        int g0 = g_begin;
        for (; g0 + U <= g_end; g0 += U) turn(g0, std::integral_constant<int, U>{});
        const int rest = g_end - g0;                      // the same in every lane of a wavefront
        if (U > 2 && rest == 3) turn(g0, std::integral_constant<int, 3>{});
        else if (U > 2 && rest == 2) turn(g0, std::integral_constant<int, 2>{});
        else if (rest == 1) turn(g0, std::integral_constant<int, 1>{});
    } else {
#pragma unroll 4
        for (int s = s_begin; s < s_end; ++s) {
            const int k = s * 32 + b * 8;
            bf16x8 wf[NW];
#pragma unroll
            for (int g = 0; g < NW; ++g) wf[g] = load_k8(w, wrow_of[g], GATED ? 2 * N : N, k, K, vector_ok);
#pragma unroll
            for (int i = 0; i < MT; ++i) {
                const bf16x8 xf = load_k8(a, 16 * i + r16, M, k, K, vector_ok);
#pragma unroll
                for (int g = 0; g < NW; ++g)
                    acc[g][i] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[g], xf, acc[g][i], 0, 0, 0);
            }
        }
    }
    if (wave > 0) {
#pragma unroll
        for (int g = 0; g < NW; ++g)
#pragma unroll
            for (int i = 0; i < MT; ++i)
#pragma unroll
                for (int r = 0; r < 4; ++r) part[wave - 1][g][i][lane][r] = acc[g][i][r];
    }
    if constexpr (EPI == EPI_SCALE) {
        ss_mine += __shfl_xor(ss_mine, 16, MLR_WAVE);
        ss_mine += __shfl_xor(ss_mine, 32, MLR_WAVE);
        if (b == 0) ss_lds[wave][r16] = ss_mine;
    }
    __syncthreads();
    if (wave != 0) return;
    float row_scale = 1.f;
    if constexpr (EPI == EPI_SCALE) {
        float total = 0.f;
#pragma unroll
        for (int i = 0; i < SKINNY_WAVES; ++i) total += ss_lds[i][r16];
        row_scale = 1.0f / sqrtf(total * epi.inv_size + epi.eps);
    }
    float y4[MT][4];
    float y4b[4] = {0.f, 0.f, 0.f, 0.f};                   // PAIR: the second strip's sums of this lane
#pragma unroll
    for (int i = 0; i < MT; ++i) {
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            float v[NW];
#pragma unroll
            for (int g = 0; g < NW; ++g) {
                v[g] = acc[g][i][r];
                for (int p = 0; p < SKINNY_WAVES - 1; ++p) v[g] += part[p][g][i][lane][r];
                if constexpr (EPI == EPI_SCALE) v[g] *= row_scale;
            }
            float y = v[0];
            if (GATED) y = (v[0] / (1.0f + expf(-v[0]))) * v[NW - 1];
            y4[i][r] = y;
            if constexpr (PAIR) y4b[r] = v[1];
            if constexpr (PAIR && EPI != EPI_RESIDUAL) {  // the second strip's sum of this lane: column n0 + 16 + 4 b + r
                const int n = n0 + 16 + 4 * b + r;
                if (r16 < M && n <= last_row) {
                    if (OUT_FLOAT) ((float*)out_raw)[(size_t)r16 * N + n] = v[1];
                    else ((__bf16*)out_raw)[(size_t)r16 * N + n] = (__bf16)v[1];
                }
            }
        }
    }
    if constexpr (EPI == EPI_RESIDUAL) {
        // this lane: row r16, columns n0 + 4 b .. + 3 of h
        const int n = n0 + 4 * b;
        const bool row_ok = r16 < M;
        float x[4];
        float sq = 0.f;
        if ((N & 3) == 0) {
            const bool ok = row_ok && n < N;
            const float hv[4] = {h4.x, h4.y, h4.z, h4.w}, wv[4] = {nw4.x, nw4.y, nw4.z, nw4.w};
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                x[r] = ok ? hv[r] + y4[0][r] : 0.f;
                sq += x[r] * x[r];
            }
            if (ok) {
                *reinterpret_cast<float4*>(epi.h + (size_t)r16 * N + n) = make_float4(x[0], x[1], x[2], x[3]);
                if (epi.next_w) {
                    typedef __attribute__((__vector_size__(4 * sizeof(__bf16)))) __bf16 bf16x4;
                    *reinterpret_cast<bf16x4*>(epi.x_out + (size_t)r16 * N + n) =
                        bf16x4{(__bf16)(x[0] * wv[0]), (__bf16)(x[1] * wv[1]), (__bf16)(x[2] * wv[2]), (__bf16)(x[3] * wv[3])};
                }
            }
        } else {
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const bool ok = row_ok && n + r < N;
                const size_t at = (size_t)min(r16, M - 1) * N + min(n + r, N - 1);
                x[r] = ok ? epi.h[at] + y4[0][r] : 0.f;
                sq += x[r] * x[r];
                if (ok) {
                    epi.h[at] = x[r];
                    if (epi.next_w) epi.x_out[at] = (__bf16)(x[r] * epi.next_w[n + r]);
                }
            }
        }
        if constexpr (PAIR) {
            // the second strip, whole groups of four columns: first its squares on their own, (0 + 1) + (2 + 3)
            // like the first strip's, then added to them
            const int n2 = n0 + 16 + 4 * b;
            const bool ok = row_ok && n2 + 3 <= last_row;
            const float hv[4] = {h4b.x, h4b.y, h4b.z, h4b.w}, wv[4] = {nw4b.x, nw4b.y, nw4b.z, nw4b.w};
            float x2[4], sq2 = 0.f;
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                x2[r] = ok ? hv[r] + y4b[r] : 0.f;
                sq2 += x2[r] * x2[r];
            }
            if (ok) {
                *reinterpret_cast<float4*>(epi.h + (size_t)r16 * N + n2) = make_float4(x2[0], x2[1], x2[2], x2[3]);
                if (epi.next_w) {
                    typedef __attribute__((__vector_size__(4 * sizeof(__bf16)))) __bf16 bf16x4;
                    *reinterpret_cast<bf16x4*>(epi.x_out + (size_t)r16 * N + n2) =
                        bf16x4{(__bf16)(x2[0] * wv[0]), (__bf16)(x2[1] * wv[1]), (__bf16)(x2[2] * wv[2]), (__bf16)(x2[3] * wv[3])};
                }
            }
            if (epi.next_w) {
                sq += __shfl_xor(sq, 16, MLR_WAVE);
                sq += __shfl_xor(sq, 32, MLR_WAVE);
                sq2 += __shfl_xor(sq2, 16, MLR_WAVE);
                sq2 += __shfl_xor(sq2, 32, MLR_WAVE);
                if (b == 0 && row_ok) {
                    // a workgroup a part; the parts beyond the workgroups, up to the buffer's capacity, are zero
                    float* parts = epi.ss_out + (size_t)r16 * epi.ss_stride;
                    parts[blockIdx.x] = sq + sq2;
                    if ((int)(gridDim.x + blockIdx.x) < epi.ss_stride) parts[gridDim.x + blockIdx.x] = 0.f;
                }
            }
            return;
        }
        if (epi.next_w) {
            sq += __shfl_xor(sq, 16, MLR_WAVE);            // (0 + 1) + (2 + 3) over the lane blocks: the strip's 16 columns
            sq += __shfl_xor(sq, 32, MLR_WAVE);
            if (b == 0 && row_ok) epi.ss_out[(size_t)r16 * gridDim.x + blockIdx.x] = sq;
        }
        return;
    }
#pragma unroll
    for (int i = 0; i < MT; ++i) {
        const int m = 16 * i + r16;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int n = n0 + 4 * b + r;
            if (m < M && n < N) {
                if (OUT_FLOAT) ((float*)out_raw)[(size_t)m * N + n] = y4[i][r];
                else ((__bf16*)out_raw)[(size_t)m * N + n] = (__bf16)y4[i][r];
            }
        }
    }
}

// Columns of a workgroup when two strips side by side deal the work out more evenly than strips of 16 do, else 0.
// Only where the weight is long enough for the memory's rate to count (k from 2048).
// Compute units of the current device, asked for once; -1 when the device does not say.
static int compute_units() {
    static int units = 0;
    if (units == 0) {
        int device = 0;
        if (hipGetDevice(&device) != hipSuccess ||
            hipDeviceGetAttribute(&units, hipDeviceAttributeMultiprocessorCount, device) != hipSuccess || units <= 0)
            units = -1;
    }
    return units;
}

static int skinny_pair_columns(int N, int K) {
    const int units = compute_units();
    if (units < 0 || K < 2048 || N % 4 != 0) return 0;
    const int strips = (N + 15) / 16;
    const int turns = (strips + units - 1) / units;       // strips of 16: the busiest unit's share, in strips
    for (int j = 1; j <= 4; ++j) {
        const int cols = (((N + units * j - 1) / (units * j)) + 3) / 4 * 4;
        if (cols > 32) continue;
        if (cols <= 16) break;
        return (double)(j * cols) < 0.9 * 16.0 * turns ? cols : 0;
    }
    return 0;
}

template <int MT, bool OUT_FLOAT, bool GATED, int UMAX, bool STAGE, int EPI>
static int launch_skinny_kernel(const void* a, const void* w, void* out, int M, int N, int K, size_t lds,
                                const SkinnyEpilogue& epi, hipStream_t stream) {
    if constexpr (MT == 1 && !GATED && !STAGE && UMAX == 4) {
        const int cols = skinny_pair_columns(N, K);
        if (cols > 0) {
            SkinnyEpilogue e = epi;
            e.cols = cols;
            e.ss_stride = (N + 15) / 16;
            // (the parts beyond the workgroups are zeroed by the workgroups themselves: there are at most as many)
            gemm_skinny_kernel<MT, OUT_FLOAT, false, 4, false, EPI, true>
                <<<dim3((N + cols - 1) / cols), SKINNY_WAVES * 64, 0, stream>>>((const __bf16*)a, (const __bf16*)w, out, M, N, K, e);
            return (int)hipGetLastError();
        }
    }
    auto* kernel = gemm_skinny_kernel<MT, OUT_FLOAT, GATED, UMAX, STAGE, EPI>;
    if (STAGE) {                                          // static and dynamic LDS together may pass 64 KB
        static const hipError_t allowed = hipFuncSetAttribute(
            reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, SKINNY_STAGE_LDS);
        if (allowed != hipSuccess) return (int)allowed;
    }
    kernel<<<dim3((N + 15) / 16), SKINNY_WAVES * 64, lds, stream>>>((const __bf16*)a, (const __bf16*)w, out, M, N, K, epi);
    return (int)hipGetLastError();
}

template <int MT, bool GATED, int UMAX, bool STAGE, int EPI>
static int launch_skinny_as(const void* a, const void* w, void* out, int M, int N, int K, int out_float,
                            size_t lds, const SkinnyEpilogue& epi, hipStream_t stream) {
    if constexpr (EPI == EPI_NONE) {
        if (out_float) return launch_skinny_kernel<MT, true, GATED, UMAX, STAGE, EPI>(a, w, out, M, N, K, lds, epi, stream);
    }
    return launch_skinny_kernel<MT, false, GATED, UMAX, STAGE, EPI>(a, w, out, M, N, K, lds, epi, stream);
}

template <int MT, bool GATED, int EPI = EPI_NONE>
static int launch_skinny(const void* a, const void* w, void* out, int M, int N, int K, int out_float,
                         hipStream_t stream, const SkinnyEpilogue& epi = SkinnyEpilogue{}) {
    // A short k (at most two groups of 64 a wavefront) takes the variant whose turns hold two groups: it
    // needs fewer registers, so more of its short-lived workgroups fit a compute unit.
    const bool short_k = MT * (GATED ? 2 : 1) <= 2 && K <= 64 * 2 * SKINNY_WAVES;
    if constexpr (MT == 1 && !GATED) {
        // Two rows or more and a long k: the activation goes through LDS.  (Measured: with a short k the
        // extra step costs what it saves, and the gated variant, whose turns would have to shrink to stay
        // within the registers of two workgroups a compute unit, gains nothing.  At k = 2048 it pays where the
        // strips leave half of the compute units idle -- a workgroup's requests go through its unit's cache
        // one after the other, and there the activation's are half of them: 4.9 us for 5.4 on 1024 columns and
        // 8 rows, 5.2 for 6.1 with 16 -- and costs 3-6 % with a strip for every unit.)
        const size_t lds = (size_t)SKINNY_WAVES * M * SKINNY_STAGE_PITCH(4);
        const bool pair = skinny_pair_columns(N, K) > 0;     // (two strips: without the stage)
        const int units = compute_units();
        const bool long_k = K > 2048 || (K == 2048 && units > 0 && 2 * ((N + 15) / 16) <= units);
        if (!pair && M >= 2 && K % 64 == 0 && long_k && lds <= SKINNY_STAGE_LDS)
            return launch_skinny_as<MT, GATED, 4, true, EPI>(a, w, out, M, N, K, out_float, lds, epi, stream);
    }
    if (short_k) return launch_skinny_as<MT, GATED, 2, false, EPI>(a, w, out, M, N, K, out_float, 0, epi, stream);
    return launch_skinny_as<MT, GATED, 4, false, EPI>(a, w, out, M, N, K, out_float, 0, epi, stream);
}

// Many rows (prompt portions), K a multiple of 64: 32x32 tiles of v_mfma_f32_32x32x16_bf16, the operands
// staged through LDS in blocks of 64 k, double-buffered: the loads of block i + 1 are asked for before the
// products of block i and written to the other buffer after them, one barrier per block.
// A workgroup has WM x WN wavefronts, each TM x TN tiles: it owns BM = 32 WM TM rows and BN = 32 WN TN
// columns of the output.  The weight is the A operand of the instruction (its rows are output columns),
// the activation the B operand, so a lane ends up with four consecutive columns n of one row m, as in the
// kernels above (lane = 32 h + i: A holds row i, k slots 8 h .. 8 h + 7, B column i, the same k slots,
// C column i, rows 8 j + 4 h + r in register 4 j + r).
// Rows of a staged block lie 144 bytes apart (128 of data): the eight lanes that the LDS serves in one
// cycle of a 16-byte read then hit different banks.  Every output element is one sum over k in ascending
// order whatever M is.  GATED: w = [gate; up] of N rows each; a wavefront's weight tiles alternate between
// the two, and silu(gate) * up is written (N columns).
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float floatx16;
#define WIDE_BK 64
#define WIDE_PITCH (WIDE_BK + 8)

template <int WM, int WN, int TM, int TN>
struct WideShape {
    static constexpr int BM = 32 * WM * TM, BN = 32 * WN * TN, THREADS = 64 * WM * WN;
    static constexpr int ROWS = BM + BN;                          // staged rows per block: weight, then activation
    static constexpr int PER_THREAD = ROWS * (WIDE_BK / 8) / THREADS;      // 16-byte pieces a thread stages
    static constexpr size_t lds_bytes = 2 * (size_t)ROWS * WIDE_PITCH * sizeof(__bf16);
    static_assert(ROWS * (WIDE_BK / 8) % THREADS == 0, "the staged pieces must divide among the threads");
};

template <int WM, int WN, int TM, int TN, bool OUT_FLOAT, bool GATED>
__global__ __launch_bounds__(64 * WM * WN) void gemm_wide_kernel(const __bf16* __restrict__ a,
                                                                 const __bf16* __restrict__ w,
                                                                 void* __restrict__ out_raw, int M, int N, int K,
                                                                 int tiles_m, int tiles_n) {
    using S = WideShape<WM, WN, TM, TN>;
    constexpr int BM = S::BM, BN = S::BN, THREADS = S::THREADS, ROWS = S::ROWS, PT = S::PER_THREAD;
    static_assert(!GATED || TN % 2 == 0, "gate and up tiles come in pairs");
    extern __shared__ __attribute__((aligned(16))) __bf16 wide_lds[];
    const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
    const int li = lane & 31, h = lane >> 5;
    const int wm = wave / WN, wn = wave % WN;
    // Workgroups go to the 8 XCDs in turn; each XCD gets a contiguous range of tiles, and within it
    // consecutive tiles share their columns, so a strip of the weight is fetched into one L2 once.
    const int total = tiles_m * tiles_n;
    int tile = blockIdx.x;
    if (total % 8 == 0) tile = (tile % 8) * (total / 8) + tile / 8;
    const int m0 = (tile % tiles_m) * BM, n0 = (tile / tiles_m) * BN;
    // In the gated case a workgroup's BN staged weight rows are BN / 2 gate rows and BN / 2 up rows of the
    // same output columns: staged row 32 j + i of wavefront column wn is gate (j even) or up (j odd).
    constexpr int NOUT = GATED ? BN / 2 : BN;                     // output columns of the workgroup
    const int c0 = GATED ? (tile / tiles_m) * NOUT : n0;

    // What a thread stages per block: pieces t, t + THREADS, ... of 16 bytes; piece c is row c / 8 of the
    // staged block (weight rows first), k 8 (c % 8) ..  The first PW pieces of a thread are weight, the
    // others activation; their places are kept as 32-bit element offsets from the matrices' bases (the host
    // refuses matrices of 2^31 elements and more), which keeps the loads' addresses out of the registers.
    constexpr int STEP = THREADS / 8;                             // staged rows between a thread's pieces
    static_assert(BN % STEP == 0, "a thread's pieces must not straddle weight and activation");
    constexpr int PW = BN / STEP;
    uint32_t src[PT];
    const int dst0 = (t >> 3) * WIDE_PITCH + (t & 7) * 8;
#pragma unroll
    for (int i = 0; i < PT; ++i) {
        const int row = (t >> 3) + STEP * i, kc = (t & 7) * 8;
        if (i < PW) {
            int n;
            if (GATED) {
                // staged weight row -> (wavefront column, tile j, row in tile); tile pairs (2 p, 2 p + 1) are
                // gate and up of output columns c0 + wn_ * (TN / 2) * 32 + p * 32 ..
                const int wn_ = row / (32 * TN), j = (row / 32) % TN, r = row % 32;
                const int col = c0 + (wn_ * (TN / 2) + j / 2) * 32 + r;
                n = min(col, N - 1) + (j & 1) * N;
            } else {
                n = min(n0 + row, N - 1);
            }
            src[i] = (uint32_t)n * (uint32_t)K + kc;
        } else {
            src[i] = (uint32_t)min(m0 + row - BN, M - 1) * (uint32_t)K + kc;
        }
    }
    // Two blocks are in flight from memory while a third is multiplied: with one, a compute unit has 64 KB
    // on its way at any time, and the latency of the loads bounds the whole GPU at about 7 TB/s of operands.
    bf16x8 stage0[PT], stage1[PT];
    const int blocks = K / WIDE_BK;
    auto fetch = [&](int kb, auto which) {                    // (blocks past the end fetch the last one again)
        const __bf16* wk = w + (size_t)min(kb, blocks - 1) * WIDE_BK;
        const __bf16* ak = a + (size_t)min(kb, blocks - 1) * WIDE_BK;
#pragma unroll
        for (int i = 0; i < PT; ++i) {
            const bf16x8 v = *reinterpret_cast<const bf16x8*>((i < PW ? wk : ak) + src[i]);
            if constexpr (decltype(which)::value == 0) stage0[i] = v; else stage1[i] = v;
        }
    };
    auto stash = [&](int buf, auto which) {
        __bf16* base = wide_lds + (size_t)buf * ROWS * WIDE_PITCH;
#pragma unroll
        for (int i = 0; i < PT; ++i) {
            if constexpr (decltype(which)::value == 0) *reinterpret_cast<bf16x8*>(base + dst0 + i * STEP * WIDE_PITCH) = stage0[i];
            else *reinterpret_cast<bf16x8*>(base + dst0 + i * STEP * WIDE_PITCH) = stage1[i];
        }
    };
    constexpr std::integral_constant<int, 0> S0{};
    constexpr std::integral_constant<int, 1> S1{};

    floatx16 acc[TN][TM];
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[j][i][e] = 0.f;

    auto products = [&](int buf) {
        const __bf16* base = wide_lds + (size_t)buf * ROWS * WIDE_PITCH;
        const __bf16* wb = base + (wn * TN * 32 + li) * WIDE_PITCH + 8 * h;
        const __bf16* ab = base + (BN + wm * TM * 32 + li) * WIDE_PITCH + 8 * h;
        // the operands of k step ks + 1 are asked for before the products of step ks
        bf16x8 wf[2][TN], af[2][TM];
        auto operands = [&](int ks, int set) {
#pragma unroll
            for (int j = 0; j < TN; ++j) wf[set][j] = *reinterpret_cast<const bf16x8*>(wb + j * 32 * WIDE_PITCH + 16 * ks);
#pragma unroll
            for (int i = 0; i < TM; ++i) af[set][i] = *reinterpret_cast<const bf16x8*>(ab + i * 32 * WIDE_PITCH + 16 * ks);
        };
        operands(0, 0);
#pragma unroll
        for (int ks = 0; ks < WIDE_BK / 16; ++ks) {
            if (ks + 1 < WIDE_BK / 16) operands(ks + 1, (ks + 1) & 1);
#pragma unroll
            for (int j = 0; j < TN; ++j)
#pragma unroll
                for (int i = 0; i < TM; ++i)
                    acc[j][i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(wf[ks & 1][j], af[ks & 1][i], acc[j][i], 0, 0, 0);
        }
    };

    fetch(0, S0);
    fetch(1, S1);
    stash(0, S0);
    fetch(2, S0);
    __syncthreads();
    // block kb is multiplied out of buffer kb % 2; block kb + 1 goes from stage[(kb + 1) % 2] into the other
    // buffer, whose readers passed the last barrier; block kb + 3 takes its place in the registers
    // (two blocks per turn of the loop and no branch inside: the register stages keep their names, and
    // the compiler counts the loads in flight exactly; with a branch it waits for all of them)
    int kb = 0;
#pragma unroll 1
    for (; kb + 2 <= blocks; kb += 2) {
        products(0);
        stash(1, S1);
        fetch(kb + 3, S1);
        __syncthreads();
        products(1);
        stash(0, S0);
        fetch(kb + 4, S0);
        __syncthreads();
    }
    if (kb < blocks) products(0);

    constexpr int TNO = GATED ? TN / 2 : TN;              // 32-column tiles of output per wavefront
    // this lane's results for tile (i, j), rows 8 q + 4 h .. + 3 of the instruction's C (output columns)
    auto result = [&](int i, int j, int q, float* y) {
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            if (GATED) {
                const float gate = acc[2 * j][i][4 * q + r], up = acc[2 * j + 1][i][4 * q + r];
                // silu(g) = g / (1 + 2^(-g log2 e)), with the hardware's exponential and reciprocal (both good
                // to an ulp or so of 32 bits; the result is rounded to bfloat16): a full division costs ten
                // instructions, and a lane has 16 TM TN / 2 of these
                y[r] = gate * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-1.44269504088896340736f * gate)) * up;
            } else {
                y[r] = acc[j][i][4 * q + r];
            }
        }
    };
    const int wave_m0 = m0 + wm * TM * 32, wave_n0 = (GATED ? c0 : n0) + wn * TNO * 32;
    if constexpr (!OUT_FLOAT) {
        // bfloat16 results leave through LDS: a lane holds four columns of one row, which would be stores of
        // 8 bytes to 64 different rows; a piece of LDS of the wavefront's own turns them into rows of 16-byte
        // pieces, eight lanes a 128-byte line (measured on 2048 x 4096 x 1024: the stores took 8 of 28 us).
        constexpr int COLS = TNO * 32, OPITCH = COLS + 8, ROWS_W = TM * 32;
        static_assert((size_t)WM * WN * ROWS_W * OPITCH * sizeof(__bf16) <= S::lds_bytes, "the output tiles must fit the LDS");
        __syncthreads();                                   // every wavefront has read its last operands
        __bf16* mine = wide_lds + (size_t)wave * ROWS_W * OPITCH;
        typedef __attribute__((__vector_size__(4 * sizeof(__bf16)))) __bf16 bf16x4_t;
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TNO; ++j)
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    float y[4];
                    result(i, j, q, y);
                    *reinterpret_cast<bf16x4_t*>(mine + (i * 32 + li) * OPITCH + j * 32 + 8 * q + 4 * h) =
                        bf16x4_t{(__bf16)y[0], (__bf16)y[1], (__bf16)y[2], (__bf16)y[3]};
                }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        constexpr int PIECES = COLS / 8;                   // 16-byte pieces in a row of the wavefront's tile
        const bool whole_n = (N & 7) == 0;
#pragma unroll
        for (int t0 = 0; t0 < ROWS_W * PIECES; t0 += 64) {
            const int c = t0 + lane, row = c / PIECES, piece = c % PIECES;
            const int m = wave_m0 + row, n = wave_n0 + 8 * piece;
            if (m >= M || n >= N) continue;
            const bf16x8 v = *reinterpret_cast<const bf16x8*>(mine + row * OPITCH + 8 * piece);
            __bf16* o = (__bf16*)out_raw + (size_t)m * N + n;
            if (whole_n && n + 8 <= N) {
                *reinterpret_cast<bf16x8*>(o) = v;
            } else {
#pragma unroll
                for (int e = 0; e < 8; ++e) if (n + e < N) o[e] = v[e];
            }
        }
    } else {
#pragma unroll
        for (int i = 0; i < TM; ++i) {
            const int m = wave_m0 + i * 32 + li;
            if (m >= M) continue;
#pragma unroll
            for (int j = 0; j < TNO; ++j)
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const int n = wave_n0 + j * 32 + 8 * q + 4 * h;
                    float y[4];
                    result(i, j, q, y);
                    float* o = (float*)out_raw + (size_t)m * N + n;
                    if (n + 3 < N && (N & 3) == 0) *reinterpret_cast<float4*>(o) = float4{y[0], y[1], y[2], y[3]};
                    else
#pragma unroll
                        for (int r = 0; r < 4; ++r) if (n + r < N) o[r] = y[r];
                }
        }
    }
}

template <int WM, int WN, int TM, int TN, bool GATED>
static int launch_wide(const void* a, const void* w, void* out, int M, int N, int K, int out_float,
                       hipStream_t stream) {
    using S = WideShape<WM, WN, TM, TN>;
    const int tiles_m = (M + S::BM - 1) / S::BM;
    const int tiles_n = GATED ? (N + S::BN / 2 - 1) / (S::BN / 2) : (N + S::BN - 1) / S::BN;
    if ((long long)tiles_m * tiles_n > 0x7fffffffLL) return -2;
    if ((unsigned long long)M * K >= (1ull << 31) || (unsigned long long)N * (GATED ? 2 : 1) * K >= (1ull << 31)) return -3;
#define MLR_WIDE_LAUNCH(OF)                                                                                   \
    {                                                                                                         \
        auto* kernel = gemm_wide_kernel<WM, WN, TM, TN, OF, GATED>;                                           \
        static const hipError_t allowed = hipFuncSetAttribute(                                                \
            reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, (int)S::lds_bytes); \
        if (allowed != hipSuccess) return (int)allowed;                                                       \
        kernel<<<dim3(tiles_m * tiles_n), S::THREADS, S::lds_bytes, stream>>>(                                \
            (const __bf16*)a, (const __bf16*)w, out, M, N, K, tiles_m, tiles_n);                              \
    }
    if (out_float) MLR_WIDE_LAUNCH(true) else MLR_WIDE_LAUNCH(false)
#undef MLR_WIDE_LAUNCH
    return (int)hipGetLastError();
}

// The wide kernel's shapes, largest first: 256 x 256 (8 wavefronts), 128 x 256, 128 x 128 (two workgroups
// a compute unit), 128 x 64 (rows x columns of the output; 64 x 64 in the gated case, whose last shape stages
// 64 gate and 64 up rows).  The largest shape that still gives about a workgroup per compute unit wins:
// measured at 2048 rows, 1.05 PFLOP/s on 24576 x 4096 with the first, 0.93-0.96 on 4096 x 4096 and
// 4096 x 12288 with the second, 0.48-0.53 on 1024 x 2048 and 1024 x 3072 with the last (the vendor library:
// 1.44, 1.18 and 0.56-0.64).
#define WIDE_SHAPES 4
template <bool GATED>
static int launch_wide_shape(int shape, const void* a, const void* w, void* out, int M, int N, int K, int out_float,
                             hipStream_t stream) {
    switch (shape) {
        case 0: return launch_wide<2, 4, 4, 2, GATED>(a, w, out, M, N, K, out_float, stream);
        case 1: return launch_wide<2, 4, 2, 2, GATED>(a, w, out, M, N, K, out_float, stream);
        case 2: return launch_wide<2, 2, 2, 2, GATED>(a, w, out, M, N, K, out_float, stream);
        case 3:
            if constexpr (GATED) return launch_wide<2, 2, 1, 2, true>(a, w, out, M, N, K, out_float, stream);
            else return launch_wide<2, 2, 2, 1, false>(a, w, out, M, N, K, out_float, stream);
        default: return -1;
    }
}

static int wide_shape_for(int M, int N, bool gated) {
    static const int rows[WIDE_SHAPES] = {256, 128, 128, 128}, cols[WIDE_SHAPES] = {256, 256, 128, 64};
    static int units = 0;
    if (units == 0) {
        int dev = 0;
        hipDeviceProp_t prop;
        units = (hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&prop, dev) == hipSuccess)
                    ? prop.multiProcessorCount : 256;
    }
    for (int s = 0; s < WIDE_SHAPES; ++s) {
        const int bm = (gated && s == 3) ? 64 : rows[s], bn = gated ? (s == 3 ? 64 : cols[s] / 2) : cols[s];
        const long long tiles = (long long)((M + bm - 1) / bm) * ((N + bn - 1) / bn);
        if (tiles * 10 >= (long long)units * 7) return s;
    }
    return WIDE_SHAPES - 1;
}

// For tests and measurements: the wide kernel in a given shape (0 .. WIDE_SHAPES - 1; -1: the shape that
// `mlr_gemm` would take), plain or gated.
extern "C" int mlr_gemm_wide(const void* a, const void* w, void* out, int M, int N, int K, int out_float,
                             int shape, int gated, hipStream_t stream) {
    if (M <= 0 || N <= 0) return 0;
    if (K <= 0 || K % WIDE_BK != 0 || (gated && out_float)) return -1;
    if (shape < 0) shape = wide_shape_for(M, N, gated != 0);
    if (gated) return launch_wide_shape<true>(shape, a, w, out, M, N, K, 0, stream);
    return launch_wide_shape<false>(shape, a, w, out, M, N, K, out_float, stream);
}

template <int WM, int WN, int TM, int TN>
static int launch(const void* a, const void* w, void* out, int M, int N, int K, int out_float,
                  hipStream_t stream) {
    constexpr int BM = WM * TM * 16, BN = WN * TN * 16;
    dim3 grid((N + BN - 1) / BN, (M + BM - 1) / BM);
    if (grid.y > 65535) return -2;
    if (out_float)
        gemm_bf16_kernel<WM, WN, TM, TN, true><<<grid, WM * WN * 64, 0, stream>>>(
            (const __bf16*)a, (const __bf16*)w, out, M, N, K);
    else
        gemm_bf16_kernel<WM, WN, TM, TN, false><<<grid, WM * WN * 64, 0, stream>>>(
            (const __bf16*)a, (const __bf16*)w, out, M, N, K);
    return (int)hipGetLastError();
}

extern "C" int mlr_gemm(const void* a, const void* w, void* out, int M, int N, int K, int out_float,
                        hipStream_t stream) {
    if (M <= 0 || N <= 0) return 0;
    if (K <= 0) return -1;
    if (M <= 16) return launch_skinny<1, false>(a, w, out, M, N, K, out_float, stream);
    // 17..64 rows against many columns (the output projection): tiles through LDS re-read the rows less often
    if (M <= 64 && N >= 16384) return launch<2, 2, 2, 2>(a, w, out, M, N, K, out_float, stream);
    if (M <= 32) return launch_skinny<2, false>(a, w, out, M, N, K, out_float, stream);
    if (M <= 64) return launch_skinny<4, false>(a, w, out, M, N, K, out_float, stream);
    if (K % WIDE_BK == 0 && (unsigned long long)M * K < (1ull << 31) && (unsigned long long)N * K < (1ull << 31))
        return launch_wide_shape<false>(wide_shape_for(M, N, false), a, w, out, M, N, K, out_float, stream);
    if (M <= 128) return launch<2, 2, 2, 2>(a, w, out, M, N, K, out_float, stream);  // 64 x 64
    return launch<2, 2, 4, 4>(a, w, out, M, N, K, out_float, stream);                // 128 x 128
}

// out[M, N] = silu(a . w[0:N]^T) * (a . w[N:2N]^T) (w is [2N, K]: gate rows, then up rows): up to 64 rows on
// the weight-streaming kernels, more on the wide kernel when K is a multiple of 64.  Returns 1 when no kernel
// here takes the sizes: the caller then runs the projection and the activation separately.
extern "C" int mlr_gemm_gated_silu(const void* a, const void* w, void* out, int M, int N, int K,
                                   hipStream_t stream) {
    if (M <= 0 || N <= 0) return 0;
    if (K <= 0) return -1;
    if (M <= 16) return launch_skinny<1, true>(a, w, out, M, N, K, 0, stream);
    if (M <= 32) return launch_skinny<2, true>(a, w, out, M, N, K, 0, stream);
    if (M <= 64) return launch_skinny<4, true>(a, w, out, M, N, K, 0, stream);
    if (K % WIDE_BK == 0 && (unsigned long long)M * K < (1ull << 31) && 2ull * N * K < (1ull << 31))
        return launch_wide_shape<true>(wide_shape_for(M, N, true), a, w, out, M, N, K, 0, stream);
    return 1;
}

// The two halves of an RMSNorm handed from one projection to the next, for M <= 16 (see SkinnyEpilogue).
// out = rsqrt(sum_p ss[m][p] / norm_size + eps) * (x . w^T); gated != 0: w is [2N, K] = [gate; up] and
// out = silu(scale * gate) * (scale * up).  x is bf16(h * norm_w) as `mlr_gemm_residual` or the row kernel
// `mlr_rows_prenorm` left it.
extern "C" int mlr_gemm_prenormed(const void* x, const float* ss, int ss_parts, float eps, int norm_size, const void* w,
                                  void* out, int M, int N, int K, int gated, hipStream_t stream) {
    if (M <= 0 || N <= 0) return 0;
    if (M > 16 || K <= 0 || ss_parts <= 0 || norm_size <= 0 || ss == nullptr) return -1;
    SkinnyEpilogue epi{};
    epi.ss = ss;
    epi.ss_parts = ss_parts;
    epi.ss_vec = (ss_parts % 4 == 0 && reinterpret_cast<uintptr_t>(ss) % 16 == 0) ? 1 : 0;
    epi.eps = eps;
    epi.inv_size = 1.0f / (float)norm_size;
    if (gated) return launch_skinny<1, true, EPI_SCALE>(x, w, out, M, N, K, 0, stream, epi);
    return launch_skinny<1, false, EPI_SCALE>(x, w, out, M, N, K, 0, stream, epi);
}

// h[M, N] += a[M, K] . w[N, K]^T in 32-bit, in place.  With next_w != null also x_out[M, N] = bf16(h * next_w)
// and ss_out[M, ceil(N / 16)]: per row and strip of 16 columns the sum of squares of the new h.
extern "C" int mlr_gemm_residual(const void* a, const void* w, float* h, const float* next_w, void* x_out,
                                 float* ss_out, int M, int N, int K, hipStream_t stream) {
    if (M <= 0 || N <= 0) return 0;
    if (M > 16 || K <= 0 || h == nullptr) return -1;
    if (next_w != nullptr && (x_out == nullptr || ss_out == nullptr)) return -2;
    SkinnyEpilogue epi{};
    epi.h = h;
    epi.next_w = next_w;
    epi.x_out = (__bf16*)x_out;
    epi.ss_out = ss_out;
    return launch_skinny<1, false, EPI_RESIDUAL>(a, w, nullptr, M, N, K, 0, stream, epi);
}
#endif
