// Attention for prompt portions on the 32x32 matrix-core tiles of gfx950 (bfloat16 cache and queries).
//
// A workgroup serves one group: consecutive tokens of one request for one kv head, as 32 NQ columns (token,
// head): 32 NQ / g tokens, g = query heads per kv head, NQ = 4 or 2 (the smaller workgroup is for batches
// that would not fill the GPU otherwise).  Its 2 NQ wavefronts are NQ column quarters (32 columns each)
// times two key parities: keys are walked in blocks of 64 at absolute multiples of 64, staged once per
// workgroup through LDS (two buffers, the loads of the next block in flight in registers), and of every
// block the wavefronts of parity 0 take keys 0..31 and those of parity 1 keys 32..63.  The two parities of
// a column are merged through LDS at the end.
//
// What a tile costs (measured): about 2 000 cycles of its SIMD, whether one wavefront or two share the SIMD: the
// last group of a 2 048-token prompt alone on the GPU (one wavefront a SIMD) takes 36.6 us for its 32 blocks, the
// whole prompt 42-44 (two a SIMD most of the time), a prompt of 8 192 tokens 0.95 us a tile and SIMD; and a
// workgroup of eight wavefronts that shares blocks of 128 keys between four key parities (half as many turns
// for a group) takes as long as this one.  Counted per tile at long contexts: 128 vector instructions (a
// dependent one issues every 9 cycles, independent ones every 6, an exponential every 10-13), 16 matrix
// instructions (512 cycles), 47 scalar ones, 16 reads and 8 writes of 16 bytes a lane through the LDS (24 KB;
// a wavefront's read takes 31 cycles) -- which add up rather than overlap (taking the softmax, the matrix
// instructions or the staging out of the kernel shortens it by each one's own time).  So the loop counts its
// instructions: offsets that do not change are computed once, a thread stages 32 contiguous bytes per page
// lookup, blocks whose keys are all written are staged without checks, the maximum of a tile is taken three
// values at a time.
//
// Per tile of 32 keys, with v_mfma_f32_32x32x16_bf16:
//   S^T[key][column]  = K[key][d] . Q^T[d][column]         A = 32 keys x 16 channels from LDS, B = Q (registers)
//   O^T[d][column]   += V^T[d][key] . P^T[key][column]     A = 32 channels x 16 keys from LDS (values are
//                                                           cached transposed), B = the probabilities, which
//                                                           sit in B's register layout already
// Register layouts of that instruction, lane = 32 h + n: A holds row n, k-slots 8 h .. 8 h + 7; B holds
// column n, the same k-slots; C holds column n, rows 8 j + 4 h + r for j, r in 0..3 (register 4 j + r).
// So registers 8 m .. 8 m + 7 of S^T are the keys 16 m + 8 a + 4 h + r (a = 0, 1) of the tile: the values
// are laid out in LDS with those keys side by side (position 16 m + 8 h + 4 a + r), and one 16-byte read
// gives the matching A operand.
//
// Softmax in the base-2 domain, 32-bit.  A column's reference maximum is only raised when a tile's maximum
// exceeds it by more than 2^8 (probabilities then stay below 256, far from overflow; the quotient at the
// end does not depend on the reference): raising it means rescaling 64 accumulators, and with 32 columns
// in a wavefront some column would need it in nearly every tile otherwise.  The decision is taken per
// column from the column's own scores, so a column's arithmetic does not depend on its neighbours.
// The sum of a column's probabilities is taken over their bfloat16 roundings, the values that the second
// product multiplies.
//
// Key splits (max_splits > 1), for a step whose groups alone would not fill the GPU (a short portion of a
// long context): workgroup (group, kv head, split s) takes the keys [s * split_keys, (s + 1) * split_keys),
// split_keys a multiple of 64, and leaves its columns' (values, maximum, sum) unnormalised in `partial`;
// `tiles_combine_kernel` merges a column's splits in ascending order.
//
// Not handled here (the caller uses the other kernels): head sizes above 128, page sizes that are no power
// of two, groups whose keys span more than PAGE_IDS pages.
#include <hip/hip_runtime.h>
#include <stdint.h>

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(__bf16)))) __bf16 bf16x4;
typedef __attribute__((__vector_size__(2 * sizeof(__bf16)))) __bf16 bf16x2;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float floatx16;

#define BLOCK_KEYS 64
#define TILE_KEYS 32
#define PAGE_IDS 2048
#define VPITCH (BLOCK_KEYS + 8)        // elements per channel row of a staged block of values
#define RAISE_BY 8.0f                  // base-2 exponent by which a tile must exceed the reference

struct TileArgs {
    const __bf16* q;             // [M, q_heads, head_dim]
    const __bf16* k_pages;       // [pages][kv_heads][page_size][head_dim]
    const __bf16* v_pages;       // [pages][kv_heads][head_dim][page_size]
    const int32_t* block_table;  // [slots, max_blocks]
    const int32_t* slots;        // [M]
    const int32_t* positions;    // [M]
    __bf16* out;                 // [M, q_heads, head_dim]
    const int32_t* group_row0;   // [groups] first batch row of a group
    const int32_t* group_ntok;   // [groups] its tokens (consecutive rows of one request)
    float* partial;              // [M, q_heads, max_splits, head_dim + 4] when max_splits > 1 (16-byte aligned)
    int groups, max_blocks, q_heads, kv_heads, head_dim, page_size, page_shift, window, split_keys, max_splits;
    float scale;
    int all_resident;            // the grid fits the GPU at once (two workgroups of 64 columns a compute unit)
    int single;                  // host: the caller's `pairing`; kernel: 1 every workgroup takes one group, 0 two (group i and group groups - 1 - i)
};

template <int ND, int NQ>
struct TileShape {
    static constexpr int D = 16 * ND;
    static constexpr int DB = (ND + 1) / 2;               // blocks of 32 channels
    static constexpr int THREADS = 128 * NQ;
    static constexpr int KPITCH = D + 8;                  // elements per key row of a staged block of keys
    static constexpr int KBUF = BLOCK_KEYS * KPITCH;      // elements
    static constexpr int VBUF = 32 * DB * VPITCH;
    static constexpr int KSTEP = THREADS / ND;            // keys that the workgroup stages per pass
    static constexpr int VSTEP = THREADS / D;             // 16-key groups of values per pass
    static constexpr int K_PASSES = (BLOCK_KEYS + KSTEP - 1) / KSTEP;
    static constexpr int V_PASSES = (BLOCK_KEYS / 16 + VSTEP - 1) / VSTEP;
    static constexpr int NO = DB * 16 + 2;                // floats a lane hands over in the merge
    static constexpr size_t kv_bytes = 2 * (size_t)(KBUF + VBUF) * sizeof(__bf16);
    static constexpr size_t merge_bytes = NQ * (size_t)NO * 64 * sizeof(float);
    static constexpr size_t lds_bytes = PAGE_IDS * sizeof(int32_t) + (kv_bytes > merge_bytes ? kv_bytes : merge_bytes);
};

// max(a, b, c) in one instruction (the compiler puts a canonicalising instruction before every fmaxf of a
// matrix-core result; NaN never gets here: masked scores are -inf, others finite)
__device__ __forceinline__ float max3(float a, float b, float c) {
    float r;
    asm("v_max3_f32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
    return r;
}

template <int ND, int NQ>
__device__ __forceinline__ void tile_group(const TileArgs& a, int grp, int kvh, int split, unsigned char* lds_raw) {
    using S = TileShape<ND, NQ>;
    constexpr int D = S::D, DB = S::DB, KPITCH = S::KPITCH, THREADS = S::THREADS;
    int32_t* page_lds = reinterpret_cast<int32_t*>(lds_raw);
    __bf16* k_lds = reinterpret_cast<__bf16*>(lds_raw + PAGE_IDS * sizeof(int32_t));
    __bf16* v_lds = k_lds + 2 * S::KBUF;
    float* merge_lds = reinterpret_cast<float*>(lds_raw + PAGE_IDS * sizeof(int32_t));

    const int P = a.page_size, pshift = a.page_shift;
    const int g = a.q_heads / a.kv_heads, cap = (32 * NQ) / g;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int n = lane & 31, h = lane >> 5;
    const int cq = wave % NQ, kp = wave / NQ;                  // column quarter, key parity
    const int row0 = a.group_row0[grp], ntok = min(a.group_ntok[grp], cap);
    const int slot = a.slots[row0], pos0 = a.positions[row0];
    const int lo = a.window > 0 ? max(0, pos0 + 1 - a.window) : 0;    // first key any token of the group sees
    const int ke = pos0 + ntok;                                      // one past the last
    // the keys of this workgroup: all of them, or those of its split
    const bool splitting = a.max_splits > 1;
    const int lo_s = splitting ? max(lo, split * a.split_keys) : lo;
    const int ke_s = splitting ? min(ke, (split + 1) * a.split_keys) : ke;
    if (lo_s >= ke_s) return;                                        // no column of the group sees this split

    // this wavefront's tokens
    const int tf = (32 * cq) / g;
    const int tl = min(ntok - 1, (32 * cq + 31) / g);
    const bool wave_active = tf < ntok;
    const int wave_first_kend = pos0 + tf + 1;
    const int wave_hi = wave_active ? pos0 + tl + 1 : 0;
    const int wave_lo = a.window > 0 ? max(0, pos0 + tf + 1 - a.window) : 0;
    const int wave_last_kbegin = a.window > 0 ? max(0, pos0 + tl + 1 - a.window) : 0;

    // this lane's column
    const int c = 32 * cq + n;
    const int tok = c / g, hh = c % g;
    const bool col_valid = tok < ntok;
    const int kend_c = col_valid ? pos0 + tok + 1 : 0;
    const int kbegin_c = a.window > 0 ? max(0, kend_c - a.window) : 0;
    const bf16x8 zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
    bf16x8 qf[ND];
    {
        const __bf16* qrow = a.q + ((size_t)(row0 + (col_valid ? tok : 0)) * a.q_heads + kvh * g + hh) * D + 8 * h;
#pragma unroll
        for (int st = 0; st < ND; ++st) {
            const bf16x8 v = *reinterpret_cast<const bf16x8*>(qrow + 16 * st);
            qf[st] = col_valid ? v : zero8;
        }
    }
    float m_ref = -INFINITY, l_run = 0.f;
    floatx16 o[DB];
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int i = 0; i < 16; ++i) o[db][i] = 0.f;

    // page ids of the group's key range, so that a block's loads do not wait for a load of the table
    const int blk_begin = lo_s / BLOCK_KEYS, blk_end = (ke_s + BLOCK_KEYS - 1) / BLOCK_KEYS;
    const int first_page = (blk_begin * BLOCK_KEYS) >> pshift;
    const int32_t* table = a.block_table + (size_t)slot * a.max_blocks;
    bool all_mapped;                                  // every page of the key range is there (none given back, none missing)
    {
        const int n_pages = min(PAGE_IDS, ((ke_s + P - 1) >> pshift) - first_page);
        // (an entry beyond the request's row of the table is no page, like an entry of -1)
        int mine_mapped = 1;
        for (int i = threadIdx.x; i < n_pages; i += THREADS) {
            const int id = first_page + i < a.max_blocks ? table[first_page + i] : -1;
            page_lds[i] = id;
            mine_mapped &= id >= 0 ? 1 : 0;
        }
        all_mapped = __syncthreads_and(mine_mapped) != 0;
    }

    // What a thread stages per block and pass: 32 bytes of the keys (16 channels of one key) and 32 bytes of
    // the values (16 keys of one channel; a page's values of one kv head are contiguous in the order
    // (channel, key)), so one page id and one address serve two 16-byte loads each.
    constexpr int KSTEP = S::KSTEP, VSTEP = S::VSTEP, KN = S::K_PASSES, VN = S::V_PASSES;
    const int k_key0 = threadIdx.x / ND, k_c16 = threadIdx.x % ND;
    const bool k_thread = (int)threadIdx.x < KSTEP * ND;
    const int v_m0 = threadIdx.x / D, v_d = threadIdx.x % D;
    const bool v_thread = (int)threadIdx.x < VSTEP * D;
    const bool big_page = P > BLOCK_KEYS;                   // a block lies within one page
    const uint32_t page_stride = (uint32_t)a.kv_heads * P * D;      // elements; the host keeps offsets within 32 bits
    int k_key[KN], k_pageadd[KN], v_m16[VN], v_pageadd[VN];
    uint32_t k_off0[KN], v_off0[VN];
#pragma unroll
    for (int i = 0; i < KN; ++i) {
        k_key[i] = min(k_key0 + KSTEP * i, BLOCK_KEYS - 1);
        k_pageadd[i] = big_page ? 0 : k_key[i] >> pshift;
        k_off0[i] = (uint32_t)kvh * P * D + (big_page ? k_key[i] : (k_key[i] & (P - 1))) * D + 16 * k_c16;
    }
#pragma unroll
    for (int i = 0; i < VN; ++i) {
        v_m16[i] = min(v_m0 + VSTEP * i, BLOCK_KEYS / 16 - 1);
        v_pageadd[i] = big_page ? 0 : (16 * v_m16[i]) >> pshift;
        v_off0[i] = (uint32_t)kvh * P * D + v_d * P + (big_page ? 16 * v_m16[i] : ((16 * v_m16[i]) & (P - 1)));
    }
    struct Staged {
        bf16x8 k[KN][2], v[VN][2];
        int tb;
        unsigned v_ok;               // bit i: pass i's page is mapped and its first key written
        bool whole;                  // every key of the block is written and mapped: nothing to check or zero
    };
    // global -> registers.  No branch around a load (a load behind a branch makes the compiler wait for
    // every load in flight): addresses are clamped to valid memory, and what must read as zero is zeroed
    // when the registers go to LDS.  Only the pages of written keys were looked up: anything later counts
    // as not mapped.
    auto fetch = [&](int blk, Staged& st) {
        const int tb = blk * BLOCK_KEYS;
        st.tb = tb;
        const int pidx = (tb >> pshift) - first_page;
        const uint32_t inpage = big_page ? (tb & (P - 1)) : 0;
        // (all blocks but a group's last, unless a window has given pages back: the same for every thread)
        st.whole = all_mapped && a.window <= 0 && tb + BLOCK_KEYS <= ke;
        if (st.whole) {
#pragma unroll
            for (int i = 0; i < KN; ++i) {
                const int pg = page_lds[pidx + k_pageadd[i]];
                const __bf16* kptr = a.k_pages + (__umul24(pg, page_stride) + inpage * D + k_off0[i]);
                st.k[i][0] = *reinterpret_cast<const bf16x8*>(kptr);
                st.k[i][1] = *reinterpret_cast<const bf16x8*>(kptr + 8);
            }
#pragma unroll
            for (int i = 0; i < VN; ++i) {
                const int pg = page_lds[pidx + v_pageadd[i]];
                const __bf16* vptr = a.v_pages + (__umul24(pg, page_stride) + inpage + v_off0[i]);
                st.v[i][0] = *reinterpret_cast<const bf16x8*>(vptr);
                st.v[i][1] = *reinterpret_cast<const bf16x8*>(vptr + 8);
            }
            st.v_ok = ~0u;
            return;
        }
        unsigned ok = 0;
#pragma unroll
        for (int i = 0; i < KN; ++i) {
            const int raw = page_lds[min(pidx + k_pageadd[i], PAGE_IDS - 1)];
            const int pg = tb + k_key[i] < ke ? raw : 0;
            const __bf16* kptr = a.k_pages + (__umul24(max(pg, 0), page_stride) + inpage * D + k_off0[i]);
            st.k[i][0] = *reinterpret_cast<const bf16x8*>(kptr);
            st.k[i][1] = *reinterpret_cast<const bf16x8*>(kptr + 8);
        }
#pragma unroll
        for (int i = 0; i < VN; ++i) {
            const int raw = page_lds[min(pidx + v_pageadd[i], PAGE_IDS - 1)];
            const int pg = tb + 16 * v_m16[i] < ke ? raw : -1;
            ok |= (pg >= 0 ? 1u : 0u) << i;
            const __bf16* vptr = a.v_pages + (__umul24(max(pg, 0), page_stride) + inpage + v_off0[i]);
            st.v[i][0] = *reinterpret_cast<const bf16x8*>(vptr);
            st.v[i][1] = *reinterpret_cast<const bf16x8*>(vptr + 8);
        }
        st.v_ok = ok;
    };
    auto stash = [&](int buf, const Staged& st) {      // registers -> LDS
        if (k_thread) {
            __bf16* kb = k_lds + buf * S::KBUF + k_key0 * KPITCH + 16 * k_c16;
#pragma unroll
            for (int i = 0; i < KN; ++i) {
                if (KN * KSTEP > BLOCK_KEYS && k_key0 + KSTEP * i >= BLOCK_KEYS) continue;
                *reinterpret_cast<bf16x8*>(kb + KSTEP * i * KPITCH) = st.k[i][0];
                *reinterpret_cast<bf16x8*>(kb + KSTEP * i * KPITCH + 8) = st.k[i][1];
            }
        }
        if (v_thread) {
            __bf16* vb = v_lds + buf * S::VBUF + v_d * VPITCH + 16 * v_m0;
#pragma unroll
            for (int i = 0; i < VN; ++i) {
                if (VN * VSTEP > BLOCK_KEYS / 16 && v_m0 + VSTEP * i >= BLOCK_KEYS / 16) continue;
                bf16x8 v0 = st.v[i][0], v1 = st.v[i][1];
                const int key0 = st.tb + 16 * (v_m0 + VSTEP * i);
                const bool ok = (st.v_ok >> i) & 1;
                if (!st.whole && !(ok && key0 + 16 <= ke)) {
                    // values of keys that are not written yet, or of a page that was given back (behind a
                    // window), count as zero: their probability is zero, but zero times whatever the
                    // memory holds need not be
#pragma unroll
                    for (int e = 0; e < 8; ++e) {
                        if (!ok || key0 + e >= ke) v0[e] = (__bf16)0.f;
                        if (!ok || key0 + 8 + e >= ke) v1[e] = (__bf16)0.f;
                    }
                }
                // keys 8 a + 4 h + r of the 16 go to position 8 h + 4 a + r
                *reinterpret_cast<bf16x8*>(vb + 16 * VSTEP * i) =
                    bf16x8{v0[0], v0[1], v0[2], v0[3], v1[0], v1[1], v1[2], v1[3]};
                *reinterpret_cast<bf16x8*>(vb + 16 * VSTEP * i + 8) =
                    bf16x8{v0[4], v0[5], v0[6], v0[7], v1[4], v1[5], v1[6], v1[7]};
            }
        }
    };

    const float c2 = a.scale * 1.44269504088896340736f;     // scores in the base-2 domain: one v_exp_f32 each
    // a tile's scores -> probabilities (as B operands), updating the column's reference, sum and accumulators
    auto softmax = [&](floatx16& sc, int tb, bool interior, bf16x8* pf) {
        if (!interior) {
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                const int key = tb + 8 * (i >> 2) + 4 * h + (i & 3);
                sc[i] = (key >= kbegin_c && key < kend_c) ? sc[i] : -INFINITY;
            }
        }
        float mx = max3(max3(sc[0], sc[1], sc[2]), max3(sc[3], sc[4], sc[5]), max3(sc[6], sc[7], sc[8]));
        mx = max3(mx, max3(sc[9], sc[10], sc[11]), max3(sc[12], sc[13], sc[14]));
        mx = fmaxf(mx, sc[15]) * c2;                    // c2 > 0
        if (__builtin_amdgcn_ballot_w64(mx > m_ref + RAISE_BY) != 0) {
            const float full = fmaxf(mx, __shfl_xor(mx, 32, 64));     // the column's maximum in this tile
            if (full > m_ref + RAISE_BY) {                             // the same in both lanes of a column
                const float corr = __builtin_amdgcn_exp2f(m_ref - full);      // -inf - finite: 0
                l_run *= corr;
#pragma unroll
                for (int db = 0; db < DB; ++db)
#pragma unroll
                    for (int i = 0; i < 16; ++i) o[db][i] *= corr;
                m_ref = full;
            }
        }
        const float m_use = fmaxf(m_ref, -1e30f);       // a column with no key yet: exp2(-inf - finite) = 0, not NaN
        // (the sum is taken over the probabilities as the second product sees them, rounded to bfloat16, two
        // at a time: v_dot2c_f32_bf16 with a pair of ones, half the instructions of single additions)
        const bf16x2 ones = {(__bf16)1.0f, (__bf16)1.0f};
        float psum = 0.f;
#pragma unroll
        for (int m = 0; m < 2; ++m) {
#pragma unroll
            for (int e = 0; e < 8; ++e) pf[m][e] = (__bf16)__builtin_amdgcn_exp2f(fmaf(sc[8 * m + e], c2, -m_use));
#pragma unroll
            for (int e = 0; e < 8; e += 2)
                psum = __builtin_amdgcn_fdot2_f32_bf16(bf16x2{pf[m][e], pf[m][e + 1]}, ones, psum, false);
        }
        l_run += psum;
    };

    auto compute = [&](int blk, int buf) {
        const int tb = blk * BLOCK_KEYS + TILE_KEYS * kp;
        if (!wave_active || tb >= wave_hi || tb + TILE_KEYS <= wave_lo) return;      // nothing for this wavefront
        const __bf16* kb = k_lds + buf * S::KBUF + (TILE_KEYS * kp + n) * KPITCH + 8 * h;
        const __bf16* vb = v_lds + buf * S::VBUF + n * VPITCH + TILE_KEYS * kp + 8 * h;
        // all operands of a product are asked for before its first instruction, and the values before
        // the softmax: the LDS answers while the matrix cores and the softmax are busy
        bf16x8 kf[ND];
#pragma unroll
        for (int st = 0; st < ND; ++st) kf[st] = *reinterpret_cast<const bf16x8*>(kb + 16 * st);
        __builtin_amdgcn_sched_barrier(0);
        floatx16 sc;
#pragma unroll
        for (int i = 0; i < 16; ++i) sc[i] = 0.f;
#pragma unroll
        for (int st = 0; st < ND; ++st) sc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf[st], qf[st], sc, 0, 0, 0);
        bf16x8 vf[DB][2];
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
            for (int m = 0; m < 2; ++m) vf[db][m] = *reinterpret_cast<const bf16x8*>(vb + 32 * db * VPITCH + 16 * m);
        __builtin_amdgcn_sched_barrier(0);
        // a tile that every token of this wavefront sees whole needs no mask (all but the last few)
        const bool interior = tb + TILE_KEYS <= wave_first_kend && tb >= wave_last_kbegin;
        bf16x8 pf[2];
        softmax(sc, tb, interior, pf);
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
            for (int m = 0; m < 2; ++m)
                o[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf[db][m], pf[m], o[db], 0, 0, 0);
    };

    // Two blocks are under way at any time: one being multiplied out of LDS, the next in flight from memory
    // into registers.  One barrier per block suffices with two LDS buffers: a wavefront can only reach the
    // second write of a buffer after the barrier that follows every wavefront's read of it.  Fetches are
    // unconditional, clamped to the last block.
    {
        Staged st;
        const int last = blk_end - 1;
        fetch(blk_begin, st);
        int buf = 0;
        for (int blk = blk_begin; blk < blk_end; ++blk) {
            stash(buf, st);
            fetch(min(blk + 1, last), st);
            __syncthreads();
            compute(blk, buf);
            buf ^= 1;
        }
    }

    // merge of the two key parities: parity 1 hands over its state, parity 0 finishes the columns
    l_run += __shfl_xor(l_run, 32, 64);
    __syncthreads();                                     // the staged blocks are not read any more
    float* mine = merge_lds + (size_t)cq * S::NO * 64 + lane;
    if (kp == 1) {
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
            for (int i = 0; i < 16; ++i) mine[(db * 16 + i) * 64] = o[db][i];
        mine[(DB * 16) * 64] = m_ref;
        mine[(DB * 16 + 1) * 64] = l_run;
    }
    __syncthreads();
    if (kp == 0 && col_valid) {
        const float m1 = mine[(DB * 16) * 64], l1 = mine[(DB * 16 + 1) * 64];
        const float m = fmaxf(m_ref, m1);
        const float w0 = m_ref > -INFINITY ? __builtin_amdgcn_exp2f(m_ref - m) : 0.f;
        const float w1 = m1 > -INFINITY ? __builtin_amdgcn_exp2f(m1 - m) : 0.f;
        const float l = l_run * w0 + l1 * w1;
        // A column whose keys all lie in this split is finished here; the merge passes it over.
        const bool whole = !splitting || (split * a.split_keys <= kbegin_c && kend_c <= (split + 1) * a.split_keys);
        if (!whole) {
            // only the splits that hold keys of this column are read by the merge
            if (split * a.split_keys >= kend_c || (split + 1) * a.split_keys <= kbegin_c) return;
            float* dst = a.partial + (((size_t)(row0 + tok) * a.q_heads + kvh * g + hh) * a.max_splits + split) * (D + 4);
#pragma unroll
            for (int db = 0; db < DB; ++db)
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const int d0 = 32 * db + 8 * j + 4 * h;
                    if (d0 >= D) continue;
                    float4 v;                           // (D + 4 floats a split: 16-byte stores)
                    v.x = o[db][4 * j] * w0 + mine[(db * 16 + 4 * j) * 64] * w1;
                    v.y = o[db][4 * j + 1] * w0 + mine[(db * 16 + 4 * j + 1) * 64] * w1;
                    v.z = o[db][4 * j + 2] * w0 + mine[(db * 16 + 4 * j + 2) * 64] * w1;
                    v.w = o[db][4 * j + 3] * w0 + mine[(db * 16 + 4 * j + 3) * 64] * w1;
                    *reinterpret_cast<float4*>(dst + d0) = v;
                }
            if (h == 0) {
                dst[D] = m;
                dst[D + 1] = l;
            }
            return;
        }
        const float inv = l != 0.f ? 1.f / l : 0.f;      // (a NaN sum must show, not read as "no key")
        __bf16* dst = a.out + ((size_t)(row0 + tok) * a.q_heads + kvh * g + hh) * D;
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int d0 = 32 * db + 8 * j + 4 * h;
                if (d0 >= D) continue;
                bf16x4 w4;
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const float other = mine[(db * 16 + 4 * j + r) * 64];
                    w4[r] = (__bf16)((o[db][4 * j + r] * w0 + other * w1) * inv);
                }
                *reinterpret_cast<bf16x4*>(dst + d0) = w4;
            }
    }
}

// The merge of key splits: one wavefront per (group, head, token of the group), four a workgroup; a lane takes
// the channels lane and lane + 64.  Splits are added in ascending order.  A token whose keys lay in one split
// was finished by that split's workgroup.
__global__ __launch_bounds__(256) void tiles_combine_kernel(TileArgs a) {
    const int grp = blockIdx.x, head = blockIdx.y, j = blockIdx.z * 4 + (threadIdx.x >> 6);
    const int lane = threadIdx.x & 63;
    if (j >= a.group_ntok[grp]) return;
    const int D = a.head_dim;
    const int m = a.group_row0[grp] + j;
    const int pos = a.positions[m];
    const int first = a.window > 0 ? max(0, pos + 1 - a.window) / a.split_keys : 0;
    const int last = min(a.max_splits - 1, pos / a.split_keys);
    if (first == last) return;                           // one split held all its keys and wrote the result itself
    const float* base = a.partial + (((size_t)m * a.q_heads + head) * a.max_splits) * (D + 4);
    float gmax = -INFINITY;
    for (int s = first + lane; s <= last; s += 64) gmax = fmaxf(gmax, base[(size_t)s * (D + 4) + D]);
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) gmax = fmaxf(gmax, __shfl_xor(gmax, off, 64));
    const int d0 = min(lane, D - 1), d1 = min(lane + 64, D - 1);
    float den = 0.f, n0 = 0.f, n1 = 0.f;
    for (int s = first; s <= last; ++s) {
        const float* p = base + (size_t)s * (D + 4);
        const float sm = p[D];
        const float w = sm > -INFINITY ? __builtin_amdgcn_exp2f(sm - gmax) : 0.f;   // maxima are base-2 exponents
        den += w * p[D + 1];
        n0 += w * p[d0];
        n1 += w * p[d1];
    }
    const float inv = den != 0.f ? 1.f / den : 0.f;
    __bf16* dst = a.out + ((size_t)m * a.q_heads + head) * D;
    if (lane < D) dst[lane] = (__bf16)(n0 * inv);
    if (lane + 64 < D) dst[lane + 64] = (__bf16)(n1 * inv);
}

// Workgroups of 128 columns take two groups, one after the other: group i and group (groups - 1 - i).
// Within a long prompt the groups' key ranges grow with their position, so every workgroup gets about the
// same work -- unless the pairs would be fewer than the compute units: then every group gets a workgroup of
// its own (a 2 048-token portion of the 0.6B sizes behind 30 000 tokens of context: 20.4 ms for 23.7 with
// workgroups of 64 columns, which load and stage every key twice as often a column).  Workgroups of 64 columns take one group each, the later (longer) groups first, and two of
// them share a compute unit.  When all of them fit the GPU at once, the order is: the later half of the
// groups, longest first, then the earlier half, shortest first, so that the longest group shares its compute
// unit with the shortest (measured at 2 048 tokens: 42.4 us for 44.1; with more workgroups than places the
// longest must simply start first).  Workgroups are dealt to the 8 XCDs round-robin by their linear index; the
// index is remapped so that the workgroups of one kv head, which read the same keys and values, share an
// XCD and its L2.
template <int ND, int NQ>
__global__ __launch_bounds__(128 * NQ, NQ == 2 ? 2 : 1) void attention_tiles_kernel(TileArgs a) {
    extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
    const int per_head = gridDim.x, total = gridDim.x * gridDim.y;
    int lin = blockIdx.x + per_head * blockIdx.y;
    if (total % 8 == 0) lin = (lin % 8) * (total / 8) + lin / 8;
    const int first = lin % per_head, kvh = lin / per_head;
    const int second = a.groups - 1 - first;
    if (a.single) {                                     // one group a workgroup, the later ones first
        // (with splits: split by split, so that the workgroups under way at a time walk the same keys.
        // Measured at 2048 tokens in two splits: 53 us; a group's splits side by side: 60; no split: 44)
        const int half = (a.groups + 1) / 2;
        const int grp = a.max_splits > 1 || !a.all_resident ? second : (first < half ? second : first - half);
        tile_group<ND, NQ>(a, grp, kvh, blockIdx.z, lds_raw);
        return;
    }
    if (second > first) {
        tile_group<ND, NQ>(a, second, kvh, 0, lds_raw);
        __syncthreads();
    }
    tile_group<ND, NQ>(a, first, kvh, 0, lds_raw);
}

template <int ND, int NQ>
static int launch_tiles(const TileArgs& a, hipStream_t stream) {
    static bool prepared = false;
    const size_t lds = TileShape<ND, NQ>::lds_bytes;
    if (!prepared) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&attention_tiles_kernel<ND, NQ>),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return (int)e;
        prepared = true;
    }
    static int compute_units = 0;
    if (compute_units == 0) {
        int device = 0;
        if (hipGetDevice(&device) != hipSuccess ||
            hipDeviceGetAttribute(&compute_units, hipDeviceAttributeMultiprocessorCount, device) != hipSuccess)
            compute_units = -1;
    }
    // (pairs that would leave compute units idle are no gain: then every group gets a workgroup of its own)
    const bool few_pairs = (long)((a.groups + 1) / 2) * a.kv_heads < compute_units;
    const bool single = NQ == 2 || a.max_splits > 1 || a.single == 1 || (a.single == 0 && few_pairs);
    dim3 grid(single ? a.groups : (a.groups + 1) / 2, a.kv_heads, a.max_splits);
    TileArgs b = a;
    b.single = single ? 1 : 0;
    b.all_resident = NQ == 2 && compute_units > 0 && (long)a.groups * a.kv_heads * a.max_splits <= 2L * compute_units;
    attention_tiles_kernel<ND, NQ><<<grid, 128 * NQ, lds, stream>>>(b);
    int err = (int)hipGetLastError();
    if (err != 0 || a.max_splits <= 1) return err;
    tiles_combine_kernel<<<dim3(a.groups, a.q_heads, ((32 * NQ) / (a.q_heads / a.kv_heads) + 3) / 4), 256, 0, stream>>>(a);
    return (int)hipGetLastError();
}

template <int NQ>
static int launch_tiles_dim(const TileArgs& a, hipStream_t stream) {
    switch (a.head_dim / 16) {
        case 1: return launch_tiles<1, NQ>(a, stream);
        case 2: return launch_tiles<2, NQ>(a, stream);
        case 3: return launch_tiles<3, NQ>(a, stream);
        case 4: return launch_tiles<4, NQ>(a, stream);
        case 5: return launch_tiles<5, NQ>(a, stream);
        case 6: return launch_tiles<6, NQ>(a, stream);
        case 7: return launch_tiles<7, NQ>(a, stream);
        default: return launch_tiles<8, NQ>(a, stream);
    }
}

// Groups: group_row0[i] = first batch row of group i, group_ntok[i] = its tokens (consecutive rows of one
// request, at most columns / (q_heads / kv_heads); columns = 128 or 64).  A group's keys must span at most
// PAGE_IDS pages (per key split, with splits).  The cache of num_pages pages must hold fewer than 2^32 elements.
// With max_splits > 1, `partial` holds M * q_heads * max_splits * (head_dim + 4) floats, 16-byte aligned, M the batch's rows.
// `pairing` (workgroups of 128 columns without splits): 0 two groups a workgroup unless that would leave compute
// units idle, 1 always one group a workgroup, 2 always two.  Returns 0, a HIP error
// code, or a negative number for sizes this kernel does not take.
extern "C" int mlr_attention_tiles(
    const void* q, const void* k_pages, const void* v_pages, const int32_t* block_table, int max_blocks,
    const int32_t* slots, const int32_t* positions, void* out, const int32_t* group_row0,
    const int32_t* group_ntok, int groups, int columns, int q_heads, int kv_heads, int head_dim, int page_size,
    int num_pages, int window, float scale, int split_keys, int max_splits, float* partial, int pairing,
    hipStream_t stream) {
    if (groups <= 0) return 0;
    if (head_dim % 16 != 0 || head_dim < 16 || head_dim > 128 || q_heads % kv_heads != 0 ||
        (columns != 128 && columns != 64) || q_heads / kv_heads > columns || pairing < 0 || pairing > 2) return -1;
    if (page_size < 16 || (page_size & (page_size - 1)) != 0) return -2;
    if (max_splits < 1) max_splits = 1;
    if (max_splits > 1 && (partial == nullptr || split_keys <= 0 || split_keys % BLOCK_KEYS != 0 ||
                           max_splits > 65535 || groups > 65535)) return -4;
    // offsets into the cache are 32-bit element counts, a page's stride and id 24-bit factors
    const uint64_t stride = (uint64_t)kv_heads * page_size * head_dim;
    if (stride >= (1u << 24) || num_pages >= (1 << 24) || stride * (uint64_t)num_pages >= (1ull << 32)) return -3;
    int shift = 0;
    while ((1 << shift) < page_size) ++shift;
    TileArgs a{(const __bf16*)q, (const __bf16*)k_pages, (const __bf16*)v_pages, block_table, slots, positions,
               (__bf16*)out, group_row0, group_ntok, partial, groups, max_blocks, q_heads, kv_heads, head_dim,
               page_size, shift, window, split_keys, max_splits, scale, 0, pairing};
    return columns == 128 ? launch_tiles_dim<4>(a, stream) : launch_tiles_dim<2>(a, stream);
}
