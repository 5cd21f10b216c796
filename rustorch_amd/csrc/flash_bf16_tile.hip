// bf16 flash-attention forward for gfx950, the general form: any head dim up to 256 that is a multiple of 8,
// own key count (cross-attention), per-sequence query and key counts (padded batches, chunked decode over a
// cache), causal masks aligned to the last key, the key-padding vector, an additive f32 score bias, and query
// rows that run over (position, head of a GQA group) so that a handful of new positions still fills a tile.
// Device counterpart of flash_forward_masked (crates/rustorch-attention/src/cpu_forward.rs:193-425) for bf16
// tensors: bf16 in, f32 accumulation on the matrix cores, bf16 out rounded once.
//
// Where the 8-wave persistent kernel of flash_bf16.hip hand-schedules two waves per SIMD around one long job
// list, this one is built for many short jobs: a workgroup of four waves owns 128 query rows (32 per wave) of one
// (batch, head) and is gone when they are done; several workgroups share a CU, so one workgroup's set-up, softmax
// and output overlap with another's matrix work without any hand-written interleaving, and the hardware
// dispatcher balances jobs of unequal length.  Keys are walked KT at a time through a double-buffered LDS tile
// (global -> registers -> LDS, one workgroup barrier per tile); per 32-key item a wave computes
//
//   S^T[kv, q]  = K[kv, :] . Q[q, :]      v_mfma_f32_32x32x16_bf16, A = K tile (LDS), B = Q (registers)
//   online softmax on S^T (a lane holds 16 scores of query row lane % 32; row max / sum are in-lane plus one
//                          exchange with lane ^ 32)
//   O^T[d, q]  += V^T[d, kv] . P^T[kv, q]  A = V tile read transposed (ds_read_b64_tr_b16), B = P (registers)
//
// with P fed to the second product straight from the score registers (the accumulator layout of the first
// product is a B operand of the second under a fixed permutation of the contraction slots, which the V operand
// read applies as well).  LDS rows are padded so that the 16-byte K reads and the transposing V reads are free
// of bank conflicts.
#include "rt_common.hpp"
#include "rt_kernels.hpp"

#include <type_traits>

namespace rt {

namespace {

constexpr int TROWS = 128;  // query rows per workgroup: four waves' worth, each wave 32
constexpr float kTileLazyLog2 = 8.0f;

typedef short s16x4t __attribute__((ext_vector_type(4)));
typedef float f32x2t __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2t __attribute__((ext_vector_type(2)));

__device__ __forceinline__ uint32_t t_cvt_pk_bf16(float lo, float hi) {
    f32x2t x = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(x, bf16x2t));  // v_cvt_pk_bf16_f32, RNE
}
// Transposing LDS read: within each group of 16 lanes, lane j receives element (j % 4) of the 8 bytes addressed
// by lanes 4e + j/4, e = 0..3.
__device__ __forceinline__ u32x2_t t_lds_read_tr16(const uint16_t* p) {
    s16x4t v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4t __attribute__((address_space(3)))*)(p));
    return __builtin_bit_cast(u32x2_t, v);
}
__device__ __forceinline__ float t_vmax(float a, float b) {  // plain v_max_f32: returns the non-NaN operand
    float d;
    asm("v_max_f32 %0, %1, %2" : "=v"(d) : "v"(a), "v"(b));
    return d;
}
__device__ __forceinline__ float t_max_with_other_half(float x) {
    auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return t_vmax(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float t_sum_with_other_half(float x) {
    auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}
// Max of the 16 scores a lane holds, as three chains of three-input maxima.  Written with the compiler's own max
// (not inline assembly): the scores come straight out of a matrix instruction, and a vector instruction that reads
// a matrix result needs wait states only the compiler's hazard pass inserts -- it does not look inside assembly.
__device__ __forceinline__ float t_max3(float a, float b, float c) { return __builtin_fmaxf(__builtin_fmaxf(a, b), c); }
__device__ __forceinline__ float t_max16(const f32x16_t& s) {
    float t0 = t_max3(s[0], s[1], s[2]), t1 = t_max3(s[3], s[4], s[5]), t2 = t_max3(s[6], s[7], s[8]);
    t0 = t_max3(t0, s[9], s[10]);
    t1 = t_max3(t1, s[11], s[12]);
    t2 = t_max3(t2, s[13], s[14]);
    return __builtin_fmaxf(t_max3(t0, t1, t2), s[15]);
}
__device__ __forceinline__ int t_wave_max_i(int x) {
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) x = max(x, __shfl_xor(x, off, 64));
    return x;
}
__device__ __forceinline__ int t_wave_min_i(int x) {
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) x = min(x, __shfl_xor(x, off, 64));
    return x;
}

template <int DP>
struct TileCfg {
    static constexpr int KT = DP <= 128 ? 64 : 32;  // keys per LDS tile
    // wave groups: group g takes the g-th share of every tile's 32-key items.  Two groups (eight waves) where the
    // registers allow two such workgroups per CU: the walk over the keys of a query tile is then half as long,
    // which is what a launch of many short sequences waits for at its end.
    static constexpr int NG = 1;
    static constexpr int NI = KT / 32 / NG;                   // items a wave takes per tile
    static constexpr int NWAVES = 4 * NG;
    static constexpr int THREADS = 64 * NWAVES;
    static constexpr int LDK = DP + 8;                        // +16 B: 16 rows x 16 B tile all 64 banks
    static constexpr int LDV = DP + (DP % 64 == 0 ? 32 : 0);  // row pitch = 16 or 48 (mod 64) words: 4 rows x 64 B tile all banks
    static constexpr int OCC = DP <= 64 ? 3 : (DP <= 128 ? 2 : 1);  // workgroups per CU the register budget is set for
    static constexpr int DT = DP / 32;
    static constexpr int PF = DP <= 64 ? 2 : 1;  // register sets of tiles in flight (wider rows take too many registers for more)
    static constexpr int TILE_BYTES = 2 * KT * (LDK + LDV) * 2;           // two stages of K and V
    // one region per query-row wave: the partner group's (O, m, l) when the keys are split two ways, and the
    // staged output rows
    static constexpr int REGION = NG == 2 ? (4 * DT + 1) * 1024 : 32 * LDK * 2;
    static constexpr int LDS_BYTES = TILE_BYTES > 4 * REGION ? TILE_BYTES : 4 * REGION;
    static_assert(REGION >= 32 * LDK * 2, "a region holds a wave's output rows");
};

// MODE: kMaskNone, kMaskCausal, kMaskPadding.  BIAS: an additive f32 score bias is applied (then MODE is kMaskNone).
template <int DP, int MODE, bool BIAS>
__global__ __launch_bounds__(TileCfg<DP>::THREADS, TileCfg<DP>::OCC) void flash_tile_bf16_kernel(FlashTileParams p) {
    using Cfg = TileCfg<DP>;
    constexpr int KT = Cfg::KT, LDK = Cfg::LDK, LDV = Cfg::LDV, NG = Cfg::NG, NI = Cfg::NI, TTHREADS = Cfg::THREADS;
    constexpr int KS = DP / 16;        // contraction steps of the score product
    constexpr int DT = DP / 32;        // 32-row tiles of O^T
    constexpr int CH = DP / 8;         // 16-byte chunks per (padded) row
    constexpr int CHUNKS = KT * CH;    // chunks of one matrix's tile
    constexpr int NL = (CHUNKS + TTHREADS - 1) / TTHREADS;  // chunks a thread moves per matrix per tile
    constexpr bool kCausal = MODE == kMaskCausal;
    constexpr int PF = Cfg::PF;        // register sets of tiles in flight behind the two LDS stages

    __shared__ __attribute__((aligned(16))) unsigned char lds[Cfg::LDS_BYTES];
    uint16_t* const Ks = (uint16_t*)lds;                      // [2][KT * LDK]
    uint16_t* const Vs = (uint16_t*)lds + 2 * KT * LDK;       // [2][KT * LDV]

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int grp = wave >> 2;   // which share of a tile's items this wave takes
    // which 32 query rows of the tile it owns.  Wave w runs on SIMD w % 4, and under a causal mask the rows at the
    // end of a tile see more keys than those at its start: the assignment rotates from workgroup to workgroup so
    // that no SIMD collects the long rows of every tile.
    const int wq = (wave + (int)blockIdx.x) & 3;
    const int col = lane & 31, hh = lane >> 5;

    // ---- which tile.  Workgroups are dealt round-robin to the 8 XCDs (each with its own L2): when the units
    // ((batch, head) pairs, or (batch, kv head) when rows are packed) divide by 8, XCD x gets the units
    // u = x (mod 8), so that all query tiles of a unit share K and V through one L2.  Within an XCD the tiles go
    // out last query tile first: the longest causal rows of every unit, then the next longest, ... -- the
    // dispatcher hands a free slot the next tile in that order, so the long ones start first and the short ones
    // fill the gaps at the end.
    const int G = p.pack;  // heads per packed row block (1: rows are positions of one head)
    const int rows_total = p.seq_q * G;
    const int n_qtiles = (rows_total + TROWS - 1) / TROWS;
    const int heads_u = G > 1 ? p.kv_heads : p.heads;
    const int n_units = p.batch * heads_u;
    int unit, rank;
    {
        const int id = blockIdx.x;
        if ((n_units & 7) == 0) {
            const int x = id & 7, k = id >> 3;
            const int upx = n_units >> 3;
            rank = k / upx;
            unit = (k - rank * upx) * 8 + x;
        } else {
            rank = id / n_units;
            unit = id - rank * n_units;
        }
    }
    const int qtile = n_qtiles - 1 - rank;
    const int q0 = qtile * TROWS;
    const int b = unit / heads_u, hx = unit - b * heads_u;
    const int kvh = G > 1 ? hx : hx / p.group;
    const int h0 = G > 1 ? hx * G : hx;  // head of a row with g = 0

    const int n_q = p.q_lens ? min(max(p.q_lens[b], 0), p.seq_q) : p.seq_q;          // valid query positions
    const int n_keys = p.kv_lens ? min(max(p.kv_lens[b], 0), p.seq_kv) : p.seq_kv;  // keys that exist
    const int off = n_keys - n_q;  // causal: the last valid query sees every key
    const int D = p.dim;

    // keys the workgroup walks
    int kv_end = n_keys;
    {
        const int s_first = G > 1 ? q0 / G : q0;
        const int s_last = min(G > 1 ? (q0 + TROWS - 1) / G : (q0 + TROWS - 1), n_q - 1);
        if (kCausal) kv_end = min(n_keys, s_last + off + 1);
        if (s_first >= n_q) kv_end = 0;  // a tile of padded query rows only
        kv_end = max(kv_end, 0);
    }
    const int n_tiles = (kv_end + KT - 1) / KT;

    f32x16_t acc_o[DT];
#pragma unroll
    for (int t = 0; t < DT; t++)
#pragma unroll
        for (int i = 0; i < 16; i++) acc_o[t][i] = 0.0f;
    float m_run = neg_inf(), l_run = 0.0f;
    bool poison = false;
    bool valid = false;
    const float cc = BIAS ? kLog2e : p.scale_log2e;  // exp2 argument per unit of score

    if (n_tiles > 0) {
        // ---- this lane's query row
        const int r = q0 + 32 * wq + col;
        const int s_pos = G > 1 ? r / G : r;
        const int g = r - s_pos * G;
        const bool exists = r < rows_total;
        valid = exists && s_pos < n_q;
        int lim = n_keys - 1;  // last key this row sees
        if (kCausal) lim = min(lim, s_pos + off);
        if (!valid) lim = -1;
        const int wave_lim_max = __builtin_amdgcn_readfirstlane(t_wave_max_i(lim));  // scalar: the tests on them are wave-uniform
        const int wave_lim_min = __builtin_amdgcn_readfirstlane(t_wave_min_i(lim));

        const size_t q_off = (size_t)b * p.lq.batch_stride + (size_t)(h0 + g) * p.lq.head_stride + (size_t)s_pos * p.lq.row_pitch;
        const uint16_t* __restrict__ Kg = p.k + (size_t)b * p.lkv.batch_stride + (size_t)kvh * p.lkv.head_stride;
        const uint16_t* __restrict__ Vg = p.v + (size_t)b * p.lkv.batch_stride + (size_t)kvh * p.lkv.head_stride;

        // Mask::Padding hiding the reference's whole first key tile: every row NaN (the tiled recurrence of
        // cpu_forward.rs:268-425 takes exp(-inf - (-inf)) on that tile and never recovers)
        if (MODE == kMaskPadding) {
            const int lead = p.ref_bc < n_keys ? p.ref_bc : n_keys;
            bool any = false;
            for (int j = lane; j < lead; j += kWave) any |= (p.keep[j] != 0);
            poison = !__any(any);
        }

        // ---- Q as B operand: column q = lane % 32, contraction slots 16 ks + 8 hh .. + 8
        bf16x8_t qreg[KS];
#pragma unroll
        for (int ks = 0; ks < KS; ks++) {
            u32x4_t z = {0u, 0u, 0u, 0u};
            const int d0 = 16 * ks + 8 * hh;
            if (exists && d0 < D) z = *(const u32x4_t*)(p.q + q_off + d0);
            qreg[ks] = __builtin_bit_cast(bf16x8_t, z);
        }

        // ---- tile movement: chunk c = tid + TTHREADS n of a tile is (row c / CH, 16-byte chunk c % CH).  A tile
        // travels global -> registers -> LDS.  LDS holds two stages; PF register sets hold the tiles behind them, so
        // that a load has PF tile-times to arrive (a workgroup alone on its CU walks a tile in well under the
        // memory latency, and a short sequence is exactly that case at the end of a launch).
        u32x4_t kreg[PF][NL], vreg[PF][NL];
        uint32_t keep_raw[PF];
#pragma unroll
        for (int i = 0; i < PF; i++) {
            keep_raw[i] = 1;
#pragma unroll
            for (int n = 0; n < NL; n++) kreg[i][n] = vreg[i][n] = u32x4_t{0u, 0u, 0u, 0u};
        }
        // per-thread constants of the movement (hoisted: the loop then spends a handful of instructions per tile on it)
        int ld_row[NL];       // row of the tile this thread moves
        uint32_t ld_col[NL];  // element offset inside a row; the same in K and V
        uint32_t st_k[NL], st_v[NL];  // byte offsets of the chunk in an LDS stage
        bool ld_on[NL];
#pragma unroll
        for (int n = 0; n < NL; n++) {
            const int c = tid + TTHREADS * n;
            const int row = c / CH, ch = c - row * CH;
            ld_row[n] = row;
            ld_col[n] = (uint32_t)(8 * ch);
            st_k[n] = (uint32_t)((row * LDK + 8 * ch) * 2);
            st_v[n] = (uint32_t)((2 * KT * LDK + row * LDV + 8 * ch) * 2);
            ld_on[n] = (CHUNKS % TTHREADS == 0 || c < CHUNKS) && 8 * ch < D;
        }
        const uint32_t kv_pitch = (uint32_t)p.lkv.row_pitch;
        auto issue_loads = [&](auto set_c, int kv0) {
            constexpr int SET = decltype(set_c)::value;
#pragma unroll
            for (int n = 0; n < NL; n++) {
                const int key = min(kv0 + ld_row[n], n_keys - 1);  // rows past the end re-read the last key; masked below
                if (ld_on[n]) {  // (the registers of chunks that are never loaded stay at their initial zero)
                    const size_t e = (size_t)(uint32_t)key * kv_pitch + ld_col[n];
                    kreg[SET][n] = *(const u32x4_t*)(Kg + e);
                    vreg[SET][n] = *(const u32x4_t*)(Vg + e);
                }
            }
            // key-padding vector of the tile: one byte per lane, turned into bits with a ballot when the tile is parked
            if (MODE == kMaskPadding) {
                const int j = kv0 + 32 * NI * grp + (lane & (32 * NI - 1));
                keep_raw[SET] = (j < n_keys) ? p.keep[j] : 1u;  // keys past the end are masked by `lim`
            }
        };
        uint64_t keep_bits = ~0ull;  // keep bits of this wave's items of the tile in LDS
        auto park = [&](auto set_c, int st) {
            constexpr int SET = decltype(set_c)::value;
#pragma unroll
            for (int n = 0; n < NL; n++) {
                if (CHUNKS % TTHREADS == 0 || tid + TTHREADS * n < CHUNKS) {
                    *(u32x4_t*)(lds + st * (KT * LDK * 2) + st_k[n]) = kreg[SET][n];
                    *(u32x4_t*)(lds + st * (KT * LDV * 2) + st_v[n]) = vreg[SET][n];
                }
            }
            if (MODE == kMaskPadding) keep_bits = __ballot(keep_raw[SET] != 0);
        };

        const float lazy = kTileLazyLog2 / cc;  // the rescale threshold in score units

        // per-lane LDS offsets (elements): K operand row `col`, slots 8 hh; V operand row (j >> 2) + 4 hh, columns 16 g16 + 4 (j & 3)
        const int k_off = (32 * NI * grp + col) * LDK + 8 * hh;
        const int v_off = (32 * NI * grp + ((lane & 15) >> 2) + 4 * hh) * LDV + 16 * ((lane >> 4) & 1) + 4 * (lane & 3);

        // bias rows of this lane's query: f32 [seq_q, seq_kv] per (batch, head) or one for all
        const float* bias_row = nullptr;
        if (BIAS) bias_row = p.bias + ((size_t)b * p.heads + (h0 + g)) * (size_t)p.bias_bh_stride + (size_t)s_pos * (size_t)p.seq_kv;

        // tile 0 goes straight to LDS; tiles 1 .. PF wait in the register sets (tile i in set i % PF)
        issue_loads(std::integral_constant<int, 0>{}, 0);
        park(std::integral_constant<int, 0>{}, 0);
        {
            auto prefetch = [&](auto i_c) {
                constexpr int I = decltype(i_c)::value;
                if (I < n_tiles) issue_loads(std::integral_constant<int, I % PF>{}, I * KT);
            };
            prefetch(std::integral_constant<int, 1>{});
            if (PF >= 2) prefetch(std::integral_constant<int, 2>{});
            if (PF >= 3) prefetch(std::integral_constant<int, 3>{});
            static_assert(PF <= 3, "prologue covers up to three sets");
        }
        __syncthreads();

        // one tile: this wave's item, then the next tile is parked from register set SET (= (t + 1) % PF) and the
        // set is refilled with tile t + 1 + PF
        // ---- pieces of an item (32 keys against the wave's 32 query rows)
        // bias values of an item: requested ahead of the matrix instructions that hide their latency
        auto bias_fetch = [&](int k0, f32x4_t (&bv)[4]) {
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const int kb = k0 + 8 * j + 4 * hh;
                f32x4_t x = {0.0f, 0.0f, 0.0f, 0.0f};
                if (valid) {
                    if (p.bias_vec4 && kb + 3 < n_keys) {
                        x = *(const f32x4_t*)(bias_row + kb);
                    } else {
#pragma unroll
                        for (int e = 0; e < 4; e++)
                            if (kb + e < n_keys) x[e] = bias_row[kb + e];
                    }
                }
                bv[j] = x;
            }
        };
        auto k_operand = [&](int st, int it, int ks) {
            return *(const bf16x8_t*)(Ks + st * KT * LDK + 32 * it * LDK + k_off + 16 * ks);
        };
        // bias (scores = (q . k) * scale + bias, crates/rustorch-nn/src/attention.rs:378-392, kept in the natural domain
        // so that a bias of -1e4 weighs as it does in the reference), then the masks
        auto mask_item = [&](int it, int k0, f32x16_t& sc, const f32x4_t (&bv)[4]) {
            if (BIAS) {
#pragma unroll
                for (int i = 0; i < 16; i++) sc[i] = __builtin_fmaf(sc[i], p.scale, bv[i >> 2][i & 3]);
            }
            if (k0 + 31 > wave_lim_min) {
#pragma unroll
                for (int i = 0; i < 16; i++) {
                    const int kr = k0 + 8 * (i >> 2) + 4 * hh + (i & 3);
                    sc[i] = (kr > lim) ? neg_inf() : sc[i];
                }
            }
            if (MODE == kMaskPadding) {
                const uint32_t keep_word = (uint32_t)(keep_bits >> (32 * it));
                if (keep_word != 0xffffffffu) {
                    const uint32_t mine = keep_word >> (4 * hh);  // bit 8(i/4) + i%4 of `mine` is key 8(i/4) + 4hh + i%4
#pragma unroll
                    for (int i = 0; i < 16; i++) {
                        const bool kept = (mine >> (8 * (i >> 2) + (i & 3))) & 1u;
                        sc[i] = kept ? sc[i] : neg_inf();
                    }
                }
            }
        };
        // the running max is raised lazily (only when some row's new max exceeds it by 2^8 in the exp2 domain), so the
        // rescale of O leaves the steady state; returns m * cc for the exponentials
        auto raise_max = [&](float m_item) {
            if (__builtin_expect(__any(m_item > m_run + lazy), 0)) {
                const float m_new = t_vmax(m_run, m_item);
                const float m_use = (m_new == neg_inf()) ? 0.0f : m_new;
                const float alpha = __builtin_amdgcn_exp2f((m_run - m_use) * cc);  // m_run = -inf -> 0
                m_run = m_new;
                l_run *= alpha;
#pragma unroll
                for (int tt = 0; tt < DT; tt++)
#pragma unroll
                    for (int i = 0; i < 16; i++) acc_o[tt][i] *= alpha;
            }
            return ((m_run == neg_inf()) ? 0.0f : m_run) * cc;
        };
        // p = exp2(s * cc - mc) in place, P as the two B operands of the item, and the row sum taken from the rounded
        // values (the weights the second product applies are then exactly the ones that are summed): v_dot2_f32_bf16
        // against ones.  (The packed pair stays in a scalar: a bit cast of a vector ELEMENT to bf16x2 as the operand of
        // the dot instruction has been seen to read the wrong element.)
        auto exp_item = [&](f32x16_t& sc, float mc, bf16x8_t (&pB)[2]) {
#pragma unroll
            for (int i = 0; i < 16; i++) sc[i] = __builtin_amdgcn_exp2f(__builtin_fmaf(sc[i], cc, -mc));
            float part0 = 0.0f, part1 = 0.0f;
            const bf16x2t ones = __builtin_bit_cast(bf16x2t, 0x3f803f80u);
#pragma unroll
            for (int u = 0; u < 2; u++) {
                u32x4_t pb;
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    const f32x2t pair = {sc[8 * u + 2 * e], sc[8 * u + 2 * e + 1]};
                    const bf16x2t w = __builtin_convertvector(pair, bf16x2t);  // v_cvt_pk_bf16_f32, RNE
                    pb[e] = __builtin_bit_cast(uint32_t, w);
                    if (e & 1) part1 = __builtin_amdgcn_fdot2_f32_bf16(w, ones, part1, false);
                    else part0 = __builtin_amdgcn_fdot2_f32_bf16(w, ones, part0, false);
                }
                pB[u] = __builtin_bit_cast(bf16x8_t, pb);
            }
            l_run += part0 + part1;
        };
        // O^T += V^T . P^T: contraction slots 0-3 of a lane are keys 16u + 4hh + 0..3, slots 4-7 keys 16u + 8 + 4hh + 0..3
        auto pv_item = [&](int st, int it, const bf16x8_t (&pB)[2]) {
#pragma unroll
            for (int u = 0; u < 2; u++)
#pragma unroll
                for (int dt = 0; dt < DT; dt++) {
                    const uint16_t* vp = Vs + st * KT * LDV + (32 * it + 16 * u) * LDV + v_off + 32 * dt;
                    const u32x2_t lo = t_lds_read_tr16(vp);
                    const u32x2_t hi = t_lds_read_tr16(vp + 8 * LDV);
                    const u32x4_t av = {lo[0], lo[1], hi[0], hi[1]};
                    acc_o[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, av), pB[u], acc_o[dt], 0, 0, 0);
                }
        };
        auto one_item = [&](int st, int it, int k0) {
            f32x4_t bv[4];
            if (BIAS) bias_fetch(k0, bv);
            f32x16_t sc;
#pragma unroll
            for (int i = 0; i < 16; i++) sc[i] = 0.0f;
#pragma unroll
            for (int ks = 0; ks < KS; ks++) sc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(k_operand(st, it, ks), qreg[ks], sc, 0, 0, 0);
            mask_item(it, k0, sc, bv);
            const float mc = raise_max(t_max_with_other_half(t_max16(sc)));
            bf16x8_t pB[2];
            exp_item(sc, mc, pB);
            pv_item(st, it, pB);
        };
        // Two items of a tile as one: their score products are two independent chains of matrix instructions, issued
        // alternately (a chain on one accumulator waits for itself), and one softmax step covers the 64 keys -- one max,
        // one rescale test.  Without it a wave alone on its SIMD spends most of a tile waiting on its own latencies,
        // which is what the last, long query tiles of a launch do.
        auto two_items = [&](int st, int k0) {
            f32x16_t s0, s1;
#pragma unroll
            for (int i = 0; i < 16; i++) s0[i] = s1[i] = 0.0f;
#pragma unroll
            for (int ks = 0; ks < KS; ks++) {
                s0 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(k_operand(st, 0, ks), qreg[ks], s0, 0, 0, 0);
                s1 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(k_operand(st, 1, ks), qreg[ks], s1, 0, 0, 0);
            }
            const f32x4_t no_bias[4] = {};
            mask_item(0, k0, s0, no_bias);
            mask_item(1, k0 + 32, s1, no_bias);
            const float mc = raise_max(t_max_with_other_half(t_vmax(t_max16(s0), t_max16(s1))));
            bf16x8_t pA[2], pC[2];
            exp_item(s0, mc, pA);
            exp_item(s1, mc, pC);
            pv_item(st, 0, pA);
            pv_item(st, 1, pC);
        };

        auto walk_tile = [&](int t, auto set_c) {
            const int st = t & 1;
            const int k0 = t * KT + 32 * NI * grp;  // first key of this wave's items
            if (NI == 2 && !BIAS && DP <= 64 && k0 + 32 <= wave_lim_max) {
                two_items(st, k0);
            } else {
#pragma unroll
                for (int it = 0; it < NI; it++)
                    // else every row of this wave has all of these keys hidden (wave-uniform)
                    if (k0 + 32 * it <= wave_lim_max) one_item(st, it, k0 + 32 * it);
            }
            // ---- the next tile: its registers have been in flight during the last PF tiles' work
            if (t + 1 < n_tiles) {
                park(set_c, st ^ 1);
                if (t + 1 + PF < n_tiles) issue_loads(set_c, (t + 1 + PF) * KT);
            }
            __syncthreads();
        };
        for (int t0 = 0; t0 < n_tiles; t0 += PF) {  // t0 % PF == 0: the set indices below are compile-time
            walk_tile(t0, std::integral_constant<int, 1 % PF>{});
            if (PF >= 2 && t0 + 1 < n_tiles) walk_tile(t0 + 1, std::integral_constant<int, 2 % PF>{});
            if (PF >= 3 && t0 + 2 < n_tiles) walk_tile(t0 + 2, std::integral_constant<int, 3 % PF>{});
        }

        // ---- the two key halves of a row meet: group 1 leaves its (O, m, l) in LDS, group 0 folds it into its own
        // with the online-softmax monoid (crates/rustorch-attention/src/online_softmax.rs:105-131, extended with O).
        // Slot i of a region is 64 lanes x 16 bytes: lane-contiguous, so reads and writes are free of bank conflicts.
        if (NG == 2) {
            f32x4_t* region = (f32x4_t*)(lds + wq * Cfg::REGION);
            if (grp == 1) {
#pragma unroll
                for (int dt = 0; dt < DT; dt++)
#pragma unroll
                    for (int j = 0; j < 4; j++)
                        region[(4 * dt + j) * 64 + lane] =
                            f32x4_t{acc_o[dt][4 * j], acc_o[dt][4 * j + 1], acc_o[dt][4 * j + 2], acc_o[dt][4 * j + 3]};
                region[4 * DT * 64 + lane] = f32x4_t{m_run, l_run, 0.0f, 0.0f};
            }
            __syncthreads();
            if (grp == 1) return;
            const f32x4_t ml = region[4 * DT * 64 + lane];
            const float m_new = t_vmax(m_run, ml[0]);
            const float m_use = (m_new == neg_inf()) ? 0.0f : m_new;
            const float a0 = __builtin_amdgcn_exp2f((m_run - m_use) * cc);  // an empty side (m = -inf) weighs 0
            const float a1 = __builtin_amdgcn_exp2f((ml[0] - m_use) * cc);
            l_run = l_run * a0 + ml[1] * a1;
            m_run = m_new;
#pragma unroll
            for (int dt = 0; dt < DT; dt++)
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    const f32x4_t o1 = region[(4 * dt + j) * 64 + lane];
#pragma unroll
                    for (int e = 0; e < 4; e++) acc_o[dt][4 * j + e] = acc_o[dt][4 * j + e] * a0 + o1[e] * a1;
                }
        }
    } else if (grp == 1) {
        return;  // a tile of padded rows: the first group writes the fill value
    }

    // ---- output: acc_o[dt][4j + e] = O^T[d = 32dt + 8j + 4hh + e][row col of the wave].  A lane holds 8-byte pieces of
    // its row; the wave parks its 32 normalised rows in its own region of LDS (every wave is past the last
    // barrier, and the region's previous content was read by this wave alone) and streams them out as whole rows,
    // 16 bytes per lane.
    const float l = t_sum_with_other_half(l_run);
    const bool good = (l > 0.0f) && (l < __uint_as_float(0x7f800000u)) && !poison;
    const float inv_l = 1.0f / l;
    uint16_t* const obuf = (uint16_t*)(lds + wq * Cfg::REGION);
    const float fill = p.zero_padded_rows ? 0.0f : quiet_nan();
    if (n_tiles > 0) {
#pragma unroll
        for (int dt = 0; dt < DT; dt++)
#pragma unroll
            for (int j = 0; j < 4; j++) {
                float o[4];
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    float x = good ? acc_o[dt][4 * j + e] * inv_l : quiet_nan();
                    if (!valid) x = fill;
                    o[e] = x;
                }
                *(u32x2_t*)(obuf + col * LDK + 32 * dt + 8 * j + 4 * hh) =
                    u32x2_t{t_cvt_pk_bf16(o[0], o[1]), t_cvt_pk_bf16(o[2], o[3])};
            }
    }
    // (the same wave wrote and now reads: no barrier needed, the LDS queue is in order)
    const uint32_t fill2 = t_cvt_pk_bf16(fill, fill);
#pragma unroll
    for (int n = 0; n < CH / 2; n++) {
        const int cidx = lane + 64 * n;
        const int row = cidx / CH, ch = cidx - row * CH;
        const int rr = q0 + 32 * wq + row;
        const int sp = G > 1 ? rr / G : rr;
        const int gg = rr - sp * G;
        // no key tile walked: padded rows get the fill value, valid rows (which then see no key at all) NaN
        const uint32_t f2 = sp < n_q ? 0x7fc07fc0u : fill2;
        u32x4_t val = {f2, f2, f2, f2};
        if (n_tiles > 0) val = *(const u32x4_t*)(obuf + row * LDK + 8 * ch);
        if (rr < rows_total && 8 * ch < D) {
            uint16_t* dst = p.out + (size_t)b * p.lo.batch_stride + (size_t)(h0 + gg) * p.lo.head_stride +
                            (size_t)sp * p.lo.row_pitch + 8 * ch;
            *(u32x4_t*)dst = val;
        }
    }
}

template <int DP, int MODE, bool BIAS>
hipError_t launch_one(hipStream_t stream, const FlashTileParams& p, dim3 grid) {
    hipLaunchKernelGGL((flash_tile_bf16_kernel<DP, MODE, BIAS>), grid, dim3(TileCfg<DP>::THREADS), 0, stream, p);
    return hipGetLastError();
}

template <int DP>
hipError_t launch_dp(hipStream_t stream, const FlashTileParams& p, dim3 grid) {
    if (p.bias) return launch_one<DP, kMaskNone, true>(stream, p, grid);
    switch (p.mask) {
        case kMaskNone: return launch_one<DP, kMaskNone, false>(stream, p, grid);
        case kMaskCausal: return launch_one<DP, kMaskCausal, false>(stream, p, grid);
        case kMaskPadding: return launch_one<DP, kMaskPadding, false>(stream, p, grid);
        default: return hipErrorInvalidValue;
    }
}

}  // namespace

bool flash_tile_bf16_supported(int dim) { return dim > 0 && dim <= 256 && dim % 8 == 0; }

hipError_t launch_flash_tile_bf16(hipStream_t stream, const FlashTileParams& p) {
    if (p.batch == 0 || p.heads == 0 || p.seq_q == 0) return hipSuccess;
    if (!flash_tile_bf16_supported(p.dim) || p.pack < 1) return hipErrorInvalidValue;
    if (p.bias && p.mask != kMaskNone) return hipErrorInvalidValue;
    const long long rows = (long long)p.seq_q * p.pack;
    const long long n_qtiles = (rows + TROWS - 1) / TROWS;
    const long long units = (long long)p.batch * (p.pack > 1 ? p.kv_heads : p.heads);
    if (n_qtiles * units > 0x7fffffffll) return hipErrorInvalidValue;
    dim3 grid((unsigned)(n_qtiles * units));
    if (p.dim <= 32) return launch_dp<32>(stream, p, grid);
    if (p.dim <= 64) return launch_dp<64>(stream, p, grid);
    if (p.dim <= 96) return launch_dp<96>(stream, p, grid);
    if (p.dim <= 128) return launch_dp<128>(stream, p, grid);
    return launch_dp<256>(stream, p, grid);
}

}  // namespace rt
