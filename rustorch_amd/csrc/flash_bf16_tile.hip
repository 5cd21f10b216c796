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

constexpr uint32_t kBufferFlags = 0x00020000u;  // dword 3 of a raw buffer descriptor: 32-bit data format, no swizzle
constexpr int TROWS = 128;  // query rows per workgroup: four waves' worth, each wave 32
constexpr float kTileTrigSum = 65536.0f;  // a lane's 16-key share of a row sum above this sends the wave to the slow path

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

template <int DP>
struct TileCfg {
    static constexpr int KT = DP <= 128 ? 64 : 32;  // keys per LDS tile
    static constexpr int NI = KT / 32;              // 32-key items per tile
    static constexpr int THREADS = 256;
    static constexpr int LDK = DP + 8;                        // +16 B: 16 rows x 16 B tile all 64 banks
    static constexpr int LDV = DP + (DP % 64 == 0 ? 32 : 0);  // row pitch = 16 or 48 (mod 64) words: 4 rows x 64 B tile all banks
    static constexpr int OCC = DP <= 64 ? 3 : (DP <= 128 ? 2 : 1);  // workgroups per CU the register budget is set for
    static constexpr int DT = DP / 32;
    static constexpr int PF = DP <= 32 ? 2 : 1;  // register sets of tiles in flight (wider rows take too many registers for more)
    static constexpr int TILE_BYTES = 2 * KT * (LDK + LDV) * 2;           // two stages of K and V
    static constexpr int REGION = 32 * LDK * 2;                           // a wave's staged output rows
    static constexpr int LDS_BYTES = TILE_BYTES > 4 * REGION ? TILE_BYTES : 4 * REGION;
    // DIRECT: unpadded tiles (rows of DP * 2 bytes, 16-byte slots swizzled), filled by loads that go straight to LDS
    static constexpr int STAGE_BYTES = KT * DP * 2;
    static constexpr int LDS_BYTES_DIRECT = 4 * STAGE_BYTES > 4 * REGION ? 4 * STAGE_BYTES : 4 * REGION;
    static constexpr int OCC_DIRECT = DP <= 64 ? 3 : 2;
};

// 16 bytes per lane from a buffer straight into LDS: lane l lands at LDS byte address lds_block + 16 l (lds_block is
// wave-uniform and goes through M0); a lane whose offset lies past the end of the descriptor lands zeros.  Issued as
// inline assembly so that the compiler's counter bookkeeping does not make every later LDS read wait for it:
// completion is awaited explicitly (s_waitcnt vmcnt(0) before the barrier that publishes the tile).  Loads the
// compiler does not know of can only make its own vmcnt waits longer, never shorter: the counter retires in order.
// (The statement counts as a writer of memory, which keeps the compiler from moving LDS reads across it.)
__device__ __forceinline__ void t_buffer_to_lds(const u32x4_t& rsrc, uint32_t lane_off, uint32_t tile_off, uint32_t lds_block) {
    const uint32_t m = __builtin_amdgcn_readfirstlane(lds_block);
    const uint32_t so = __builtin_amdgcn_readfirstlane(tile_off);
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
                 :
                 : "s"(m), "v"(lane_off), "s"(rsrc), "s"(so)
                 : "memory");
}
// a raw buffer descriptor as four scalars: base, no stride, `bytes` addressable
__device__ __forceinline__ u32x4_t t_make_rsrc(const void* base, uint32_t bytes) {
    const uint64_t a = (uint64_t)(uintptr_t)base;
    return u32x4_t{(uint32_t)__builtin_amdgcn_readfirstlane((uint32_t)a), (uint32_t)__builtin_amdgcn_readfirstlane((uint32_t)(a >> 32) & 0xffffu),
                   (uint32_t)__builtin_amdgcn_readfirstlane(bytes), kBufferFlags};
}

// MODE: kMaskNone, kMaskCausal, kMaskPadding.  BIAS: an additive f32 score bias is applied (then MODE is kMaskNone).
// PACKED: query rows run over (position, head of the GQA group) (then MODE is kMaskCausal and there is no bias).
// The grid is (heads or kv heads, batch, query tiles): no division stands between a workgroup and its first load.
//
// The key walk of a wave is a software pipeline over 32-key items, one step per item j:
//
//   S(j+1) = K(j+1).Q^T           KS matrix instructions   | both independent of the vector work, issued in between
//   O^T   += V(j-1)^T.P(j-1)^T    2 DT matrix instructions | it so that the wave never waits on the matrix pipe
//   P(j)   = softmax step on S(j)  ~60 vector instructions
//
// so a wave that is alone on its SIMD (the long query tiles at the end of a launch of short sequences) keeps the
// matrix pipe and the vector pipe busy at once instead of running the three phases of an item back to back.
// K therefore sits in LDS one tile ahead of V: during tile t the waves read K(t+1) and V(t-1), and after the
// tile's one barrier (behind the step of its first item) K(t+2) and V(t+1) are parked over K(t) and V(t-1).
//
// SPLIT (packed rows only): the keys of a (sequence, kv head) are cut into p.n_splits spans of whole tiles, a
// workgroup walks one span and leaves the unnormalised O, the running max and the row sum of its rows as a partial
// (o, m, l); flash_split_merge_kernel folds the partials with the online-softmax monoid
// (crates/rustorch-attention/src/online_softmax.rs:105-131 extended with o) -- the split over the context of the
// decode kernels, for a chunk of new positions over one long cache, whose few query tiles would otherwise keep a
// handful of CUs busy.
//
// WIN (causal mask, rows of one head): a sliding window, query i sees keys (i + off - window, i + off] -- the
// reference's sliding_window_mask (crates/rustorch-nn/src/masks.rs:41-60) without its [T, T] bias tensor.  The walk
// starts at the tile that holds the first key the workgroup's first row sees (tensor base, key count and causal offset
// moved by that many keys, as for a span of SPLIT), and an item that holds keys below some row's window is masked on
// that side as well.
//
// DIRECT (head dim 64 or 128 exactly, no bias, no key-padding vector): the tiles travel from memory straight into LDS
// (buffer_load_dwordx4 ... lds) instead of through registers and LDS writes.  After a tile's barrier the waves request
// K(t+2) and V(t+1) into the stages K(t) and V(t-1) have just left and wait for their own requests ahead of the next
// tile's barrier.  LDS rows are unpadded (a landing block of 1 KB is contiguous) and their 16-byte slots are XORed
// with bits of the row, as in flash_bf16.hip.  Same instructions on the same operands otherwise: the same bits.
// Measured against the register path, interleaved in one process: 3-5 % on short or padded sequences (B=16 H=16
// N=1024: 52.3 -> 49.3 us), 7-9 % on long ones (B=4 H=32 N=4096: 306 -> 283 us), 4-7 % at head dim 128; three stages
// per matrix or four workgroups per CU (head dim 64) are no faster.
template <int DP, int MODE, bool BIAS, bool PACKED, bool SPLIT = false, bool WIN = false, bool DIRECT = false>
__global__ __launch_bounds__(TileCfg<DP>::THREADS, DIRECT ? TileCfg<DP>::OCC_DIRECT : ((BIAS && DP == 64) ? 2 : TileCfg<DP>::OCC)) void flash_tile_bf16_kernel(FlashTileParams p) {
    static_assert(!SPLIT || (PACKED && !BIAS && MODE == kMaskCausal), "the split over the keys serves the chunked decode");
    static_assert(!WIN || (!PACKED && !BIAS && !SPLIT && MODE == kMaskCausal), "the window is a causal mask's");
    static_assert(!DIRECT || ((DP == 64 || DP == 128) && !BIAS && MODE != kMaskPadding), "tiles straight into LDS: head dim 64 or 128 exactly");
    using Cfg = TileCfg<DP>;
    constexpr int KT = Cfg::KT, LDK = Cfg::LDK, LDV = Cfg::LDV, NI = Cfg::NI, TTHREADS = Cfg::THREADS;
    constexpr int KS = DP / 16;        // contraction steps of the score product
    constexpr int DT = DP / 32;        // 32-row tiles of O^T
    constexpr int NM = 2 * KS;         // matrix instructions of a step: KS for S(j+1), 2 DT = KS for P(j-1).V(j-1)
    constexpr int CH = DP / 8;         // 16-byte chunks per (padded) row
    constexpr int CHUNKS = KT * CH;    // chunks of one matrix's tile
    constexpr int NL = (CHUNKS + TTHREADS - 1) / TTHREADS;  // chunks a thread moves per matrix per tile
    constexpr bool kCausal = MODE == kMaskCausal;
    constexpr int PF = Cfg::PF;        // register sets of tiles in flight behind the two LDS stages
    static_assert(2 * DT == KS, "one P.V matrix instruction per score matrix instruction");
    // Head dims above 128 do not have the registers for two score tiles and their operands in flight (O alone is 128
    // registers), nor does head dim 128 with a bias (two items' bias values) or with a key-padding mask: there an
    // item runs its three phases one after the other, and K is parked with V.
    constexpr bool PIPE = DP <= 128 && !((BIAS || MODE == kMaskPadding) && DP == 128);

    __shared__ alignas(DIRECT ? 1024 : 16) unsigned char lds[DIRECT ? Cfg::LDS_BYTES_DIRECT : Cfg::LDS_BYTES];
    uint16_t* const Ks = (uint16_t*)lds;                      // [2][KT * LDK]
    uint16_t* const Vs = (uint16_t*)lds + 2 * KT * LDK;       // [2][KT * LDV]
    // DIRECT: [K stage 0][K stage 1][V stage 0][V stage 1], rows of ROWB bytes without padding
    constexpr int ROWB = DP * 2, STAGE_B = Cfg::STAGE_BYTES;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int col = lane & 31, hh = lane >> 5;

    // ---- which tile.  The grid is (unit within the batch, batch, rank of the query tile), dispatched x first: all
    // units' tiles of rank 0 (the last query tile, the longest causal rows), then rank 1, ... -- the dispatcher hands a
    // free slot the next tile in that order, so the long ones start first and the short ones fill the gaps at the
    // end.  Workgroups go round-robin to the 8 XCDs (each with its own L2) in the same order: when the units
    // ((batch, head) pairs, or (batch, kv head) when rows are packed) divide by 8, all query tiles of a unit land on
    // one XCD and share K and V through its L2.
    const int G = PACKED ? p.pack : 1;  // heads per packed row block (1: rows are positions of one head)
    const int rows_total = p.seq_q * G;
    const int hx = blockIdx.x, b = blockIdx.y;
    const int zz = (int)gridDim.z - 1 - (int)blockIdx.z;
    // kv head: hx itself when rows are packed, else hx / group (group_magic = 2^32 / group + 1, exact below 2^16 heads)
    const int kvh = (PACKED || p.group_magic == 0) ? hx : (int)__umulhi((uint32_t)hx, p.group_magic);
    const int h0 = PACKED ? hx * G : hx;  // head of a row with g = 0
    const int D = p.dim;

    const uint16_t* __restrict__ Kg = p.k + (size_t)b * p.lkv.batch_stride + (size_t)kvh * p.lkv.head_stride;
    const uint16_t* __restrict__ Vg = p.v + (size_t)b * p.lkv.batch_stride + (size_t)kvh * p.lkv.head_stride;

    // ---- tile movement: chunk c = tid + TTHREADS n of a tile is (row c / CH, 16-byte chunk c % CH).  A tile
    // travels global -> registers -> LDS.  LDS holds two stages of each matrix; PF register sets per matrix hold
    // the tiles behind them, so that a load has PF tile-times to arrive.
    u32x4_t kreg[PF][NL], vreg[PF][NL];
    uint32_t keep_raw[PF];
#pragma unroll
    for (int i = 0; i < PF; i++) {
        keep_raw[i] = 1;
#pragma unroll
        for (int n = 0; n < NL; n++) kreg[i][n] = vreg[i][n] = u32x4_t{0u, 0u, 0u, 0u};  // (only read when there are no keys at all)
    }
    // per-thread constants of the movement (hoisted: the loop then spends a handful of instructions per tile on it)
    uint32_t ld_off[NL];  // byte offset of the thread's chunk from the first byte of a tile; the same in K and V
    uint32_t st_k[NL], st_v[NL];  // byte offsets of the chunk in an LDS stage
    bool ld_on[NL];
    const uint32_t kv_pitch = (uint32_t)p.lkv.row_pitch;
#pragma unroll
    for (int n = 0; n < NL; n++) {
        const int c = tid + TTHREADS * n;
        const int row = c / CH, ch = c - row * CH;
        st_k[n] = (uint32_t)((row * LDK + 8 * ch) * 2);
        st_v[n] = (uint32_t)((2 * KT * LDK + row * LDV + 8 * ch) * 2);
        ld_on[n] = 8 * ch < D;
        // a chunk past the head dim is requested (from column 0) but never parked
        ld_off[n] = ((uint32_t)row * kv_pitch + (ld_on[n] ? (uint32_t)(8 * ch) : 0u)) * 2u;
    }
    u32x4_t k1[NL];
    // DIRECT: a wave's load instruction fills 1 KB of LDS (RPI = 8 rows at head dim 64, 4 at 128), lane l the 16 bytes
    // at 16 l; instruction n of wave w fills block w + 4 n of a stage.  Bank conflicts are avoided by an XOR of the
    // 16-byte slot index with bits of the row (K rows are read 16 at a time at one slot, V rows 4 at a time over 4
    // adjacent slots by the transposing reads), applied on the way in: the lane fetches the slot that belongs at its
    // LDS position.
    constexpr int SPR = DP / 8;                // 16-byte slots per row
    constexpr int RPI = 64 / (SPR > 64 ? 64 : SPR);  // rows per load instruction of a wave
    constexpr int NLD = KT / (4 * RPI);        // load instructions per wave, matrix and tile
    auto swz_k = [](int r) __attribute__((always_inline)) { return DP == 128 ? (r & 15) : ((r >> 1) & 7); };
    auto swz_v = [](int r) __attribute__((always_inline)) { return DP == 128 ? 4 * (r & 3) : 4 * ((r >> 1) & 1); };
    static_assert(!DIRECT || (4 * RPI) % 16 == 0, "the row swizzles must not depend on the load index");
    const uint32_t lds_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) unsigned char*)lds;
    const int dl_row = RPI * wave + lane / SPR;  // row of the lane's chunk in instruction 0; instruction n: + 4 RPI n (the swizzles do not see n)
    const uint32_t dl_k = (uint32_t)dl_row * kv_pitch * 2u + (uint32_t)(((lane % SPR) ^ swz_k(dl_row)) * 16);
    const uint32_t dl_v = (uint32_t)dl_row * kv_pitch * 2u + (uint32_t)(((lane % SPR) ^ swz_v(dl_row)) * 16);
    // the tile whose first row lies tile_off bytes into the descriptor -> the stage at stage_off
    auto dl_tile = [&](const u32x4_t& rs, uint32_t lane_off, uint32_t tile_off, uint32_t stage_off) __attribute__((always_inline)) {
#pragma unroll
        for (int n = 0; n < NLD; n++)
            t_buffer_to_lds(rs, lane_off, tile_off + (uint32_t)(4 * RPI * n) * kv_pitch * 2u, lds_base + stage_off + (uint32_t)((wave + 4 * n) * 1024));
    };
    // Tile 0 (K and V) and K of tile 1 are requested before the sequence lengths have arrived (a dependent load
    // away), through descriptors that end with the tensor's last row: the rows of V(0) past the last key are zeroed
    // once the length is known, those of K are masked in the score tile whatever they hold.  (A span of the keys
    // starts where the sequence's own length puts it: its requests wait for the lengths.)
    const uint32_t tile_bytes_g = (uint32_t)KT * kv_pitch * 2u;  // from a tile's first row to the next tile's, in memory
    if (!SPLIT && !WIN) {
        const uint32_t all_bytes = p.seq_kv > 0 ? ((uint32_t)(p.seq_kv - 1) * kv_pitch + (uint32_t)D) * 2u : 0u;
        if constexpr (DIRECT) {
            const u32x4_t Kall = t_make_rsrc(Kg, all_bytes), Vall = t_make_rsrc(Vg, all_bytes);
            dl_tile(Kall, dl_k, 0u, 0u);
            dl_tile(Vall, dl_v, 0u, 2u * STAGE_B);
            dl_tile(Kall, dl_k, tile_bytes_g, STAGE_B);
        } else {
            const __amdgpu_buffer_rsrc_t Kall = __builtin_amdgcn_make_buffer_rsrc((void*)Kg, 0, all_bytes, kBufferFlags);
            const __amdgpu_buffer_rsrc_t Vall = __builtin_amdgcn_make_buffer_rsrc((void*)Vg, 0, all_bytes, kBufferFlags);
#pragma unroll
            for (int n = 0; n < NL; n++) {
                kreg[0][n] = __builtin_amdgcn_raw_buffer_load_b128(Kall, ld_off[n], 0, 0);
                vreg[0][n] = __builtin_amdgcn_raw_buffer_load_b128(Vall, ld_off[n], 0, 0);
                k1[n] = PIPE ? __builtin_amdgcn_raw_buffer_load_b128(Kall, ld_off[n], tile_bytes_g, 0) : u32x4_t{0u, 0u, 0u, 0u};
            }
        }
    }

    // (DIRECT reads the lengths through the constant address space -- nothing writes them during the launch: behind
    // the assembly statements of the tile requests, which count as writers of memory, the compiler would otherwise
    // fetch them with vector loads, and a wait for a vector load is a wait for every request issued before it: 30.7 us
    // instead of 29.9 on a padded batch of 16 x 16 heads of up to 1024 rows)
    auto len_at = [](const int32_t* a, int i) __attribute__((always_inline)) {
        if constexpr (DIRECT) return ((const __attribute__((address_space(4))) int32_t*)(uintptr_t)a)[i];
        else return a[i];
    };
    const int q_len_raw = p.q_lens ? len_at(p.q_lens, b) : p.seq_q;
    // (a padded batch of self-attention hands over one array for both: one dependent load instead of two in a row)
    const int kv_len_raw = p.kv_lens ? ((DIRECT && p.kv_lens == p.q_lens) ? q_len_raw : len_at(p.kv_lens, b)) : p.seq_kv;
    const int n_q = min(max(q_len_raw, 0), p.seq_q);  // valid query positions
    int n_keys = min(max(kv_len_raw, 0), p.seq_kv);  // keys that exist
    int qtile = SPLIT ? zz / p.n_splits : zz;
    const int split = SPLIT ? zz - qtile * p.n_splits : 0;
    (void)split;
    // A padded batch ranks each sequence's OWN query tiles, last (longest) first: rank 0 is the tile that holds the
    // sequence's last valid row, and the tiles of padded rows only, which have nothing to walk, take the ranks behind
    // the valid ones and so are dispatched last, into the gaps at the end, instead of holding the first slots.
    if (!SPLIT && p.q_lens) {
        const int n_qt = (n_q * G + TROWS - 1) / TROWS;  // tiles with valid rows
        const int rank = (int)blockIdx.z;
        qtile = rank < n_qt ? n_qt - 1 - rank : rank;
    }
    const int q0 = qtile * TROWS;
    // which 32 query rows of the tile a wave owns.  Wave w runs on SIMD w % 4, and under a causal mask the rows at
    // the end of a tile see more keys than those at its start: the assignment rotates from workgroup to workgroup
    // so that no SIMD collects the long rows of every tile.
    const int wq = (wave + hx + b + (int)blockIdx.z) & 3;
    int off = n_keys - n_q;  // causal: the last valid query sees every key

    // keys the workgroup walks
    int kv_end = n_keys;
    {
        const int s_first = G > 1 ? q0 / G : q0;
        const int s_last = min(G > 1 ? (q0 + TROWS - 1) / G : (q0 + TROWS - 1), n_q - 1);
        if (kCausal) kv_end = min(n_keys, s_last + off + 1);
        if (s_first >= n_q) kv_end = 0;  // a tile of padded query rows only
        kv_end = max(kv_end, 0);
    }
    int n_tiles = (kv_end + KT - 1) / KT;
    if (SPLIT) {
        // this workgroup's span of the walk: tiles [t_begin, t_end).  From here on keys are counted from the span's
        // first key: the tensors' base, the key count, the causal offset and the end of the walk all move by it, and
        // the walk below is that of a sequence whose keys are the span's (a row whose last visible key lies before the
        // span gets a negative limit: every score masked, an empty partial).
        const int per = (n_tiles + p.n_splits - 1) / p.n_splits;
        const int t_begin = split * per, t_end = min(n_tiles, t_begin + per);
        const int key0 = t_begin * KT;
        n_tiles = max(t_end - t_begin, 0);
        kv_end = min(kv_end, t_end * KT) - key0;
        n_keys = min(n_keys, t_end * KT) - key0;
        off -= key0;
        Kg += (size_t)key0 * (size_t)p.lkv.row_pitch;
        Vg += (size_t)key0 * (size_t)p.lkv.row_pitch;
    }
    if (WIN) {
        // the first key any row of the workgroup sees, rounded down to a tile: the walk starts there
        const int key0 = (max(q0 + off - p.window + 1, 0) / KT) * KT;
        n_tiles = max(n_tiles - key0 / KT, 0);
        kv_end -= key0;
        n_keys -= key0;
        off -= key0;
        Kg += (size_t)key0 * (size_t)p.lkv.row_pitch;
        Vg += (size_t)key0 * (size_t)p.lkv.row_pitch;
    }
    // A tile of padded query rows only (a padded batch has many: every tile behind a sequence's last row) has nothing
    // to load or walk: its rows get the fill value and the workgroup is done.
    if (!SPLIT && !PACKED && q0 >= n_q) {
        const uint32_t f2 = p.zero_padded_rows ? 0u : 0x7fc07fc0u;
        const u32x4_t val = {f2, f2, f2, f2};
        uint16_t* const ob = p.out + (size_t)b * p.lo.batch_stride + (size_t)h0 * p.lo.head_stride;
        for (int c = tid; c < TROWS * CH; c += TTHREADS) {
            const int row = c / CH, ch = c - row * CH;
            if (q0 + row < rows_total && 8 * ch < D) *(u32x4_t*)(ob + (size_t)(q0 + row) * p.lo.row_pitch + 8 * ch) = val;
        }
        // (the early requests land in this workgroup's LDS: not to be left in flight when it is handed on)
        if constexpr (DIRECT) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        return;
    }
    // K and V are read through buffer descriptors that end with the last key's row: a request for a row behind it
    // returns zeros without touching memory.  Zero rows of V are what the walk needs there (their weights are zero,
    // and zero times a copy of a non-finite row would be NaN); zero rows of K give score 0, masked like any score
    // past the last key.  The lane's offset is a constant of the thread and the tile's offset a scalar, so a request
    // costs no address arithmetic.  (Offsets are 32-bit: the launcher refuses slabs of 4 GiB and more.)
    const uint32_t slab_bytes = n_keys > 0 ? ((uint32_t)(n_keys - 1) * kv_pitch + (uint32_t)D) * 2u : 0u;
    const __amdgpu_buffer_rsrc_t Kbuf = __builtin_amdgcn_make_buffer_rsrc((void*)Kg, 0, slab_bytes, kBufferFlags);
    const __amdgpu_buffer_rsrc_t Vbuf = __builtin_amdgcn_make_buffer_rsrc((void*)Vg, 0, slab_bytes, kBufferFlags);
    const u32x4_t Kd = t_make_rsrc(Kg, slab_bytes), Vd = t_make_rsrc(Vg, slab_bytes);  // (DIRECT: the same descriptors as scalars)
    if (DIRECT && (SPLIT || WIN)) {
        dl_tile(Kd, dl_k, 0u, 0u);
        dl_tile(Vd, dl_v, 0u, 2u * STAGE_B);
        dl_tile(Kd, dl_k, tile_bytes_g, STAGE_B);
    } else if (SPLIT || WIN) {  // tile 0 (K and V) and K of tile 1 of the span / of the window
#pragma unroll
        for (int n = 0; n < NL; n++) {
            kreg[0][n] = __builtin_amdgcn_raw_buffer_load_b128(Kbuf, ld_off[n], 0, 0);
            vreg[0][n] = __builtin_amdgcn_raw_buffer_load_b128(Vbuf, ld_off[n], 0, 0);
            k1[n] = PIPE ? __builtin_amdgcn_raw_buffer_load_b128(Kbuf, ld_off[n], tile_bytes_g, 0) : u32x4_t{0u, 0u, 0u, 0u};
        }
    } else if (!DIRECT && n_keys < KT) {  // the early requests ended with the tensor, not with the sequence
#pragma unroll
        for (int n = 0; n < NL; n++)
            if ((tid + TTHREADS * n) / CH >= n_keys) vreg[0][n] = u32x4_t{0u, 0u, 0u, 0u};
    }

    if (MODE == kMaskPadding && n_keys > 0) {  // keep bytes past the last key count as kept: `lim` masks those keys
        const int j = lane & (KT - 1);
        const uint32_t kb = p.keep[min(j, n_keys - 1)];
        keep_raw[0] = j < n_keys ? kb : 1u;
    }

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
        static_assert(CHUNKS % TTHREADS == 0, "every thread moves NL chunks of every tile");
        // Every request below is unconditional -- a tile index past the last tile is clamped to it, a chunk past the
        // head dim reads column 0 -- and only the LDS write is predicated.  With no branch around a load the compiler
        // counts the loads in flight exactly and waits at a park for the oldest register set only; with one it
        // falls back to waiting for all of them, which empties the prefetch queue at every tile.
        if (!DIRECT && D < DP) {  // the columns that are never parked are zero in both stages
            for (int i = tid; i < Cfg::TILE_BYTES / 16; i += TTHREADS) ((u32x4_t*)lds)[i] = u32x4_t{0u, 0u, 0u, 0u};
            __syncthreads();
        }
        const int last_kv0 = (n_tiles - 1) * KT;
        auto issue_k = [&](u32x4_t (&dst)[NL], int kv0) __attribute__((always_inline)) {
            const uint32_t tile_off = (uint32_t)min(kv0, last_kv0) * (kv_pitch * 2u);
#pragma unroll
            for (int n = 0; n < NL; n++) dst[n] = __builtin_amdgcn_raw_buffer_load_b128(Kbuf, ld_off[n], tile_off, 0);
        };
        auto issue_v = [&](auto set_c, int kv0) __attribute__((always_inline)) {
            constexpr int SET = decltype(set_c)::value;
            kv0 = min(kv0, last_kv0);
            const uint32_t tile_off = (uint32_t)kv0 * (kv_pitch * 2u);
#pragma unroll
            for (int n = 0; n < NL; n++) vreg[SET][n] = __builtin_amdgcn_raw_buffer_load_b128(Vbuf, ld_off[n], tile_off, 0);
            // key-padding vector of the tile: one byte per lane, turned into bits with a ballot when the tile is parked
            if (MODE == kMaskPadding) {
                const int j = kv0 + (lane & (KT - 1));
                const uint32_t kb = p.keep[min(j, n_keys - 1)];
                keep_raw[SET] = (j < n_keys) ? kb : 1u;  // keys past the end are masked by `lim`
            }
        };
        auto park_k = [&](const u32x4_t (&src)[NL], int st) __attribute__((always_inline)) {
#pragma unroll
            for (int n = 0; n < NL; n++)
                if (D == DP || ld_on[n]) *(u32x4_t*)(lds + st * (KT * LDK * 2) + st_k[n]) = src[n];
        };
        uint64_t keep_cur = ~0ull, keep_next = ~0ull;  // keep bits of the tile whose items are in their softmax step, and of the next
        auto park_v = [&](auto set_c, int st) __attribute__((always_inline)) {
            constexpr int SET = decltype(set_c)::value;
#pragma unroll
            for (int n = 0; n < NL; n++)
                if (D == DP || ld_on[n]) *(u32x4_t*)(lds + st * (KT * LDV * 2) + st_v[n]) = vreg[SET][n];
            if (MODE == kMaskPadding) keep_next = __ballot(keep_raw[SET] != 0);
        };

        // ---- this lane's query row
        const int r = q0 + 32 * wq + col;
        const int s_pos = G > 1 ? r / G : r;
        const int g = r - s_pos * G;
        const bool exists = r < rows_total;
        valid = exists && s_pos < n_q;
        int lim = n_keys - 1;  // last key this row sees
        if (kCausal) lim = min(lim, s_pos + off);
        if (!valid) lim = -1;
        // the largest and smallest `lim` of the wave, as scalars (the tests on them are wave-uniform): lim grows with
        // the row, and the rows that are not valid are the last ones
        int wave_lim_max, wave_lim_min;
        {
            const int r_first = q0 + 32 * wq, r_last = r_first + 31;
            const int r_lim = min(rows_total, n_q * G);  // rows below it are valid
            const int r_top = min(r_last, r_lim - 1);
            const int s_top = G > 1 ? r_top / G : r_top, s_bot = G > 1 ? r_first / G : r_first;
            wave_lim_max = r_first < r_lim ? (kCausal ? min(n_keys - 1, s_top + off) : n_keys - 1) : -1;
            wave_lim_min = r_last < r_lim ? (kCausal ? min(n_keys - 1, s_bot + off) : n_keys - 1) : -1;
        }
        // items this wave walks: the ones that hold a key some row of it sees (a prefix of the workgroup's items)
        const int n_it = wave_lim_max < 0 ? 0 : min(n_tiles * NI, (wave_lim_max >> 5) + 1);
        // a window: the first key this row sees, and the largest such key over the wave's rows (its last valid row's)
        const int lo = WIN ? max(lim - p.window + 1, 0) : 0;
        const int wave_lo_max = WIN ? max(wave_lim_max - p.window + 1, 0) : 0;

        // (the query row is read without a test: a row past the tensor reads the tensor's last row)
        const int r_q = min(r, rows_total - 1);
        const int s_q = G > 1 ? r_q / G : r_q;
        const size_t q_off = (size_t)b * p.lq.batch_stride + (size_t)(h0 + (r_q - s_q * G)) * p.lq.head_stride + (size_t)s_q * p.lq.row_pitch;

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
            // Unconditional loads (a row past the tensor is read from the tensor's last row, a chunk past the head dim
            // from its last chunk): a load under a per-lane test costs a branch of its own.  A row that does not exist
            // has every score masked and is not written, so what it holds does not matter; the columns past the head
            // dim must be zero.
            const int d0 = 16 * ks + 8 * hh;
            u32x4_t z = {0u, 0u, 0u, 0u};
            if constexpr (DP <= 128) {
                z = *(const u32x4_t*)(p.q + q_off + min(d0, D - 8));
                if (D < DP && d0 >= D) z = u32x4_t{0u, 0u, 0u, 0u};
            } else {  // (head dim 256 has no register to spare for the clamped addresses)
                if (exists && d0 < D) z = *(const u32x4_t*)(p.q + q_off + d0);
            }
            qreg[ks] = __builtin_bit_cast(bf16x8_t, z);
        }

        // per-lane LDS offsets (elements): K operand row `col`, slots 8 hh; V operand row (j >> 2) + 4 hh, columns 16 g16 + 4 (j & 3)
        const int k_off = col * LDK + 8 * hh;
        const int v_off = (((lane & 15) >> 2) + 4 * hh) * LDV + 16 * ((lane >> 4) & 1) + 4 * (lane & 3);
        // DIRECT (byte offsets): the same operand rows and columns in the swizzled layout.  The swizzles only permute
        // address bits that the operand index also occupies, so operand ks sits at k_base ^ 32 ks, operand dt at
        // v_base ^ 64 dt.
        uint32_t k_base = 0, v_base = 0;
        if constexpr (DIRECT) {
            const int j = lane & 15, g16 = (lane >> 4) & 1, vrow = (j >> 2) + 4 * hh, low = 2 * g16 + ((j & 3) >> 1);
            k_base = (uint32_t)(col * ROWB + ((hh ^ swz_k(col)) * 16));
            v_base = (uint32_t)(2 * STAGE_B + vrow * ROWB + ((low ^ swz_v(vrow)) * 16) + 8 * (j & 1));
        }
        // where the operands of item `item` of stage `st` start: with the lane's own offset (padded layout), or without
        // it (DIRECT: load_op adds the lane's swizzled offset)
        auto k_at = [&](int st, int item) __attribute__((always_inline)) -> const uint16_t* {
            if constexpr (DIRECT) return (const uint16_t*)(lds + st * STAGE_B + item * 32 * ROWB);
            else return Ks + st * KT * LDK + item * 32 * LDK + k_off;
        };
        auto v_at = [&](int st, int item) __attribute__((always_inline)) -> const uint16_t* {
            if constexpr (DIRECT) return (const uint16_t*)(lds + st * STAGE_B + item * 32 * ROWB);
            else return Vs + st * KT * LDV + item * 32 * LDV + v_off;
        };

        // bias rows of this lane's query: f32 [seq_q, seq_kv] per (batch, head) or one for all
        const float* bias_row = nullptr;
        if (BIAS) bias_row = p.bias + ((size_t)b * p.heads + (h0 + g)) * (size_t)p.bias_bh_stride + (size_t)s_pos * (size_t)p.seq_kv;

        // K(0), V(0) -> stage 0, K(1) -> stage 1; then the register sets take K(2) .. K(1 + PF) and V(1) .. V(PF)
        // (K(j) travels in set j % PF, and so does V(j))
        if constexpr (DIRECT) {
            // tile 0 and K(1) have landed (and the queries); V rows of tile 0 past the last key, requested before the
            // lengths were known, are zeroed by the lane that fetched them
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            if (n_keys < KT) {
#pragma unroll
                for (int n = 0; n < NLD; n++)
                    if (dl_row + 4 * RPI * n >= n_keys) *(u32x4_t*)(lds + 2 * STAGE_B + (wave + 4 * n) * 1024 + 16 * lane) = u32x4_t{0u, 0u, 0u, 0u};
            }
        } else {
            park_k(kreg[0], 0);
            park_v(std::integral_constant<int, 0>{}, 0);
            keep_cur = keep_next;
            if (PIPE) park_k(k1, 1);
            {
                auto prefetch = [&](auto i_c) __attribute__((always_inline)) {
                    constexpr int I = decltype(i_c)::value;  // 0 .. PF - 1
                    constexpr int KA = PIPE ? 2 : 1;         // K runs a tile ahead of V in the pipelined walk only
                    issue_k(kreg[(KA + I) % PF], (KA + I) * KT);
                    issue_v(std::integral_constant<int, (1 + I) % PF>{}, (1 + I) * KT);
                };
                prefetch(std::integral_constant<int, 0>{});
                if (PF >= 2) prefetch(std::integral_constant<int, 1>{});
                if (PF >= 3) prefetch(std::integral_constant<int, 2>{});
                static_assert(PF <= 3, "prologue covers up to three sets");
            }
        }
        __syncthreads();

        // ---- pieces of a step
        // bias values of an item (scores = (q . k) * scale + bias, crates/rustorch-nn/src/attention.rs:378-392, kept in
        // the natural domain so that a bias of -1e4 weighs as it does in the reference): requested a step ahead
        auto bias_fetch = [&](int k0, f32x4_t (&bv)[4]) __attribute__((always_inline)) {
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
        // the bias, then the masks, on the scores of the item whose keys start at k0 (item `it` of its tile)
        auto mask_item = [&](int it, int k0, f32x16_t& sc, const f32x4_t (&bv)[4]) __attribute__((always_inline)) {
            if (BIAS) {
#pragma unroll
                for (int i = 0; i < 16; i++) sc[i] = __builtin_fmaf(sc[i], p.scale, bv[i >> 2][i & 3]);
            }
            if (k0 + 31 > wave_lim_min) {
                // key k0 + 8 (i / 4) + 4 hh + i % 4 is hidden when it lies past lim: one subtraction per item, then a
                // comparison with a constant per score
                const int room = lim - k0 - 4 * hh;
#pragma unroll
                for (int i = 0; i < 16; i++) sc[i] = (8 * (i >> 2) + (i & 3) > room) ? neg_inf() : sc[i];
            }
            if (WIN && k0 < wave_lo_max) {
                const int room_lo = lo - k0 - 4 * hh;  // key k0 + 8 (i / 4) + 4 hh + i % 4 lies before the window when below lo
#pragma unroll
                for (int i = 0; i < 16; i++) sc[i] = (8 * (i >> 2) + (i & 3) < room_lo) ? neg_inf() : sc[i];
            }
            if (MODE == kMaskPadding) {
                const uint32_t keep_word = (uint32_t)(keep_cur >> (32 * it));
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
        // operand m of a step: even m = K rows of the next item (A operand of score instruction m / 2), odd m = V of
        // the previous item (contraction slots 0-3 of a lane are keys 16u + 4hh + 0..3, slots 4-7 keys 16u + 8 + 4hh + 0..3)
        auto load_op = [&](int m, const uint16_t* kp, const uint16_t* vp) __attribute__((always_inline)) {
            if constexpr (DIRECT) {
                if ((m & 1) == 0) return *(const u32x4_t*)((const unsigned char*)kp + (k_base ^ (uint32_t)(32 * (m >> 1))));
                const int i = m >> 1, u = i / DT, dt = i - u * DT;
                const unsigned char* const vq = (const unsigned char*)vp + (v_base ^ (uint32_t)(64 * dt)) + 16 * u * ROWB;
                const u32x2_t lo = t_lds_read_tr16((const uint16_t*)vq);
                const u32x2_t hi = t_lds_read_tr16((const uint16_t*)(vq + 8 * ROWB));
                return u32x4_t{lo[0], lo[1], hi[0], hi[1]};
            }
            if ((m & 1) == 0) return *(const u32x4_t*)(kp + 16 * (m >> 1));
            const int i = m >> 1, u = i / DT, dt = i - u * DT;
            const u32x2_t lo = t_lds_read_tr16(vp + 16 * u * LDV + 32 * dt);
            const u32x2_t hi = t_lds_read_tr16(vp + 16 * u * LDV + 32 * dt + 8 * LDV);
            return u32x4_t{lo[0], lo[1], hi[0], hi[1]};
        };
        // An empty assembly statement that takes x as a read-write argument: whatever makes x stays above it, whatever
        // uses x stays below.  A run of them is a fence for exactly the values named.
        auto pin_f = [](float& x) __attribute__((always_inline)) { asm volatile("" : "+v"(x)); };
        auto pin_u = [](uint32_t& x) __attribute__((always_inline)) { asm volatile("" : "+v"(x)); };
        auto pin_b = [](bf16x8_t& x) __attribute__((always_inline)) { asm volatile("" : "+v"(x)); };

        float neg_mc = valid ? __uint_as_float(0x7f800000u) : 0.0f;  // -m_run * cc; +inf while a valid row has no max yet
        // The values that travel from step to step come in pairs: a step reads one of a pair and writes the other, and
        // the next step has them the other way round, so nothing is copied.
        f32x16_t s_a, s_b;        // S(j), made in step j - 1, and S(j + 1)
        bf16x8_t p_a[2], p_b[2];  // P(j - 1) and P(j)
        p_a[0] = p_a[1] = p_b[0] = p_b[1] = __builtin_bit_cast(bf16x8_t, u32x4_t{0u, 0u, 0u, 0u});
        f32x4_t bv_a[4] = {}, bv_b[4] = {};  // bias values of item j and of item j + 1

        // S(0), before the pipeline starts
        {
#pragma unroll
            for (int i = 0; i < 16; i++) s_a[i] = s_b[i] = 0.0f;
            if (BIAS) bias_fetch(0, bv_a);
            if (PIPE && n_it > 0) {
#pragma unroll
                for (int ks = 0; ks < KS; ks++)
                    s_a = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, load_op(2 * ks, k_at(0, 0), nullptr)), qreg[ks], s_a, 0, 0, 0);
                // The running max starts at the max of item 0, taken here, so that the first step already runs the
                // fast path (without it the step would form P twice and rescale an O that is still zero).  The masks
                // are applied first; the step applies them again, which changes nothing.  (Not with a bias: adding it
                // is part of the mask step and must happen once.)
                if (!BIAS) {
                    mask_item(0, 0, s_a, bv_a);
                    const float m0 = t_max_with_other_half(t_max16(s_a));
                    if (m0 > neg_inf()) {  // (false for -inf and for NaN: such a row waits for the slow path)
                        m_run = m0;
                        neg_mc = -m0 * cc;
                    }
                }
            }
        }

        // O^T += V(j-1)^T . P(j-1)^T alone: behind the wave's last item
        auto drain = [&](const uint16_t* vp) __attribute__((always_inline)) {
#pragma unroll
            for (int i = 0; i < KS; i++) {
                const int u = i / DT, dt = i - u * DT;
                const u32x4_t av = load_op(2 * i + 1, nullptr, vp);
                acc_o[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, av), p_a[u], acc_o[dt], 0, 0, 0);
            }
        };
        // P = exp2(s * cc + nmc) of the 16 scores a lane holds as the item's two B operands, and the lane's share of
        // the row sum (plain additions: v_dot2c_f32_bf16 would halve their number but runs on the matrix pipe, where
        // it queues behind the matrix instructions of every wave of the SIMD)
        auto exp_plain = [&](const f32x16_t& sc, float nmc, uint32_t (&w)[8], float& part) __attribute__((always_inline)) {
            float part0 = 0.0f, part1 = 0.0f;
#pragma unroll
            for (int e = 0; e < 8; e++) {
                const float x0 = __builtin_amdgcn_exp2f(__builtin_fmaf(sc[2 * e], cc, nmc));
                const float x1 = __builtin_amdgcn_exp2f(__builtin_fmaf(sc[2 * e + 1], cc, nmc));
                part0 += x0;
                part1 += x1;
                w[e] = t_cvt_pk_bf16(x0, x1);
            }
            part = part0 + part1;
        };

        // the slow path of a softmax step: the item max, O and l rescaled to it, P again from the scores
        auto raise_max_and_redo = [&](const f32x16_t& sc, uint32_t (&w)[8], float& part) __attribute__((always_inline)) {
            const float m_item = t_max_with_other_half(t_max16(sc));
            const float m_new = t_vmax(m_run, m_item);
            const float m_use = (m_new == neg_inf()) ? 0.0f : m_new;
            const float alpha = __builtin_amdgcn_exp2f((m_run - m_use) * cc);  // m_run = -inf -> 0
            m_run = m_new;
            l_run *= alpha;
#pragma unroll
            for (int tt = 0; tt < DT; tt++)
#pragma unroll
                for (int i = 0; i < 16; i++) acc_o[tt][i] *= alpha;
            const float mc = m_use * cc;
            // a valid row that has seen no key yet keeps taking this path (and gets P = 0 from it: exp2(-inf - 0))
            neg_mc = (m_new == neg_inf()) ? (valid ? __uint_as_float(0x7f800000u) : 0.0f) : -mc;
            exp_plain(sc, -mc, w, part);
        };
        // An item whose three phases run one after the other (head dims above 128): S, the softmax step, P.V
        auto step_simple = [&](int it, int k0, const uint16_t* kp, const uint16_t* vp) __attribute__((always_inline)) {
            if (BIAS) bias_fetch(k0, bv_a);
#pragma unroll
            for (int i = 0; i < 16; i++) s_a[i] = 0.0f;
#pragma unroll
            for (int ks = 0; ks < KS; ks++)
                s_a = __builtin_amdgcn_mfma_f32_32x32x16_bf16(*(const bf16x8_t*)(kp + 16 * ks), qreg[ks], s_a, 0, 0, 0);
            mask_item(it, k0, s_a, bv_a);
            uint32_t w[8];
            float part;
            exp_plain(s_a, neg_mc, w, part);
            if (__builtin_expect(__any(!(part <= kTileTrigSum)), 0)) raise_max_and_redo(s_a, w, part);
            l_run += part;
            p_a[0] = __builtin_bit_cast(bf16x8_t, u32x4_t{w[0], w[1], w[2], w[3]});
            p_a[1] = __builtin_bit_cast(bf16x8_t, u32x4_t{w[4], w[5], w[6], w[7]});
            drain(vp);
        };

        // One step of the pipeline: item j (keys k0 .., item `it` of its tile) gets its softmax step; K rows of item
        // j + 1 are at kp, V rows of item j - 1 at vp.
        //
        // The softmax step takes no row max in the steady state: P is formed against the running max as it stands (a
        // stale max scales a row's P, O and l by one common factor, harmless until it overflows), and the lane's share
        // of the row sum, which is needed anyway, bounds every P of the lane.  Only when a share passes kTileTrigSum, or
        // is not a number, or a valid row has no max yet (neg_mc = +inf), does the wave take the item max, rescale O and
        // l and form P again from the scores, which are still in their registers.
        //
        // The vector work is laid out in six groups (arguments, exponentials, sums and conversions, for either half of
        // the scores), the step's matrix instructions are dealt to the groups in order, S and P.V alternating (a chain
        // on one accumulator waits for itself), and an operand is read from LDS one or two groups ahead of its instruction.
        // The fences between the groups name the vector values and the B operands of the matrix instructions on
        // either side, which is what keeps each matrix instruction inside its group.
        auto step = [&](int it, int k0, const uint16_t* kp, const uint16_t* vp, f32x16_t& s_cur, f32x16_t& s_next,
                        bf16x8_t (&p_prev)[2], bf16x8_t (&p_new)[2], f32x4_t (&bv_cur)[4],
                        f32x4_t (&bv_next)[4]) __attribute__((always_inline)) {
            if (BIAS) bias_fetch(k0 + 32, bv_next);
            mask_item(it, k0, s_cur, bv_cur);
#pragma unroll
            for (int i = 0; i < 16; i++) s_next[i] = 0.0f;
            u32x4_t ops[NM];
            auto group_of = [](int m) __attribute__((always_inline)) { return NM >= 6 ? m * 6 / NM : (m * 6 + NM - 1) / NM; };
            auto fetch_group = [&](int gq) __attribute__((always_inline)) {
#pragma unroll
                for (int m = 0; m < NM; m++)
                    if (group_of(m) == gq) ops[m] = load_op(m, kp, vp);
            };
            auto fence_b = [&](int gq) __attribute__((always_inline)) {  // the B operands of the matrix instructions of group gq
#pragma unroll
                for (int m = 0; m < NM; m++) {
                    if (group_of(m) != gq) continue;
                    if (m & 1) pin_b(p_prev[(m >> 1) / DT]);
                    else pin_b(qreg[m >> 1]);
                }
            };
            auto multiply_group = [&](int gq) __attribute__((always_inline)) {
#pragma unroll
                for (int m = 0; m < NM; m++) {
                    if (group_of(m) != gq) continue;
                    const bf16x8_t a_op = __builtin_bit_cast(bf16x8_t, ops[m]);
                    if ((m & 1) == 0) {
                        s_next = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a_op, qreg[m >> 1], s_next, 0, 0, 0);
                    } else {
                        const int i = m >> 1, u = i / DT, dt = i - u * DT;
                        acc_o[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a_op, p_prev[u], acc_o[dt], 0, 0, 0);
                    }
                }
            };
            float t[8];
            uint32_t w[8];
            float part0 = 0.0f, part1 = 0.0f;
            constexpr int LOOK = DP <= 64 ? 2 : 1;  // groups between an operand's LDS read and its matrix instruction
            fetch_group(0);
            if (LOOK > 1) fetch_group(1);
            fence_b(0);
#pragma unroll
            for (int gq = 0; gq < 6; gq++) {
                if (gq + LOOK < 6) fetch_group(gq + LOOK);
                multiply_group(gq);
                const int half = gq / 3;
                if (gq % 3 == 0) {
#pragma unroll
                    for (int i = 0; i < 8; i++) t[i] = __builtin_fmaf(s_cur[8 * half + i], cc, neg_mc);
                } else if (gq % 3 == 1) {
#pragma unroll
                    for (int i = 0; i < 8; i++) t[i] = __builtin_amdgcn_exp2f(t[i]);
                } else {
#pragma unroll
                    for (int i = 0; i < 8; i += 2) {
                        part0 += t[i];
                        part1 += t[i + 1];
                    }
#pragma unroll
                    for (int e = 0; e < 4; e++) w[4 * half + e] = t_cvt_pk_bf16(t[2 * e], t[2 * e + 1]);
                }
                // the fence behind group gq
#pragma unroll
                for (int i = 0; i < 8; i++) pin_f(t[i]);
                if (gq % 3 == 2) {
                    pin_f(part0);
                    pin_f(part1);
#pragma unroll
                    for (int e = 0; e < 4; e++) pin_u(w[4 * half + e]);
                }
                fence_b(gq);
                if (gq + 1 < 6) fence_b(gq + 1);
            }
            float part = part0 + part1;
            if (__builtin_expect(__any(!(part <= kTileTrigSum)), 0)) raise_max_and_redo(s_cur, w, part);
            l_run += part;
            p_new[0] = __builtin_bit_cast(bf16x8_t, u32x4_t{w[0], w[1], w[2], w[3]});
            p_new[1] = __builtin_bit_cast(bf16x8_t, u32x4_t{w[4], w[5], w[6], w[7]});
        };
        // a step whose results are moved back into the first of each pair
        auto step_a = [&](int it, int k0, const uint16_t* kp, const uint16_t* vp) __attribute__((always_inline)) {
            step(it, k0, kp, vp, s_a, s_b, p_a, p_b, bv_a, bv_b);
            s_a = s_b;
            p_a[0] = p_b[0];
            p_a[1] = p_b[1];
            if (BIAS) {
#pragma unroll
                for (int j = 0; j < 4; j++) bv_a[j] = bv_b[j];
            }
        };
        // slot j of the walk: a step while the wave has items left, then once the P.V of its last item
        auto slot = [&](int j, int it, const uint16_t* kp, const uint16_t* vp) __attribute__((always_inline)) {
            if (j < n_it) step_a(it, 32 * j, kp, vp);
            else if (j == n_it && n_it > 0) drain(vp);
        };

        // tile t: the step of its first item, the barrier, K(t+2) and V(t+1) parked from sets KSET and VSET (which
        // are refilled with K(t+2+PF) and V(t+1+PF)), then the steps of its other items
        auto park_next = [&](int t, auto kset_c, auto vset_c, auto st_c) __attribute__((always_inline)) {
            constexpr int KSET = decltype(kset_c)::value;
            const int st = st_c;  // t & 1, as a constant where the caller knows it
            if constexpr (DIRECT) {
                // K(t+2) over K(t), V(t+1) over V(t-1): requested now that every wave is done with those, awaited
                // (vmcnt) ahead of the next tile's barrier
                if (t + 2 < n_tiles) dl_tile(Kd, dl_k, (uint32_t)(t + 2) * tile_bytes_g, (uint32_t)(st * STAGE_B));
                if (t + 1 < n_tiles) dl_tile(Vd, dl_v, (uint32_t)(t + 1) * tile_bytes_g, (uint32_t)((2 + (st ^ 1)) * STAGE_B));
            } else {
                // (behind the last tiles these park and request copies of the last tile, which nobody reads)
                park_k(kreg[KSET], st);
                park_v(vset_c, st ^ 1);
                issue_k(kreg[KSET], (t + 2 + PF) * KT);
                issue_v(vset_c, (t + 1 + PF) * KT);
            }
        };
        // what a wave does ahead of a tile's barrier: DIRECT waits for its own requests of a tile ago
        auto meet = [&]() __attribute__((always_inline)) {
            if constexpr (DIRECT) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            __syncthreads();
        };
        // the same for a tile of which the wave walks every item: straight-line code, the pairs swapped from step to step
        // `st_c` is t & 1, as an integer or as a compile-time constant: with the stage known at compile time every LDS
        // address of the tile is the lane's base plus an immediate, and `later` (t > 0 known) drops the choice of the
        // first tile's stand-in for V(-1)
        auto walk_full = [&](int t, auto kset_c, auto vset_c, auto st_c, auto later_c) __attribute__((always_inline)) {
            const int st = st_c;
            constexpr bool kLater = decltype(later_c)::value;
            const int k0 = t * KT;
            if (NI > 1) {
                step(0, k0, k_at(st, 1), (!kLater && t == 0) ? v_at(st, 0) : v_at(st ^ 1, NI - 1), s_a, s_b, p_a, p_b, bv_a, bv_b);
                meet();
                park_next(t, kset_c, vset_c, st_c);
                step(1, k0 + 32, k_at(st ^ 1, 0), v_at(st, 0), s_b, s_a, p_b, p_a, bv_b, bv_a);
            } else {
                step_a(0, k0, k_at(st ^ 1, 0), (!kLater && t == 0) ? v_at(st, 0) : v_at(st ^ 1, 0));
                __syncthreads();
                park_next(t, kset_c, vset_c, st_c);
                __syncthreads();
            }
            keep_cur = keep_next;
        };
        auto walk_tile = [&](int t, auto kset_c, auto vset_c) __attribute__((always_inline)) {
            const int st = t & 1;  // K(t) and V(t) sit in stage st, K(t+1) and V(t-1) in the other
            // first item: the next item is item 1 of this tile (or item 0 of the next tile when a tile is one item);
            // the previous item is the last of tile t - 1 (at t = 0 there is none: P is zero, and V(0) stands in)
            slot(t * NI, 0, NI > 1 ? k_at(st, 1) : k_at(st ^ 1, 0), t == 0 ? v_at(st, 0) : v_at(st ^ 1, NI - 1));
            meet();
            park_next(t, kset_c, vset_c, st);
            if (NI > 1) {
                slot(t * NI + 1, 1, k_at(st ^ 1, 0), v_at(st, 0));
            } else {
                __syncthreads();  // one item per tile: K(t+2) is read by the very next step
            }
            keep_cur = keep_next;
        };
        int t0 = 0;  // t0 % PF == 0 throughout: the set indices below are compile-time
        if (!PIPE) {
            static_assert(PIPE || PF == 1, "the unpipelined walk keeps one register set");
            for (int t = 0; t < n_tiles; t++) {
                const int st = t & 1;
#pragma unroll
                for (int it = 0; it < NI; it++)
                    if (t * NI + it < n_it)
                        step_simple(it, t * KT + 32 * it, k_at(st, it), v_at(st, it));
                park_k(kreg[0], st ^ 1);
                park_v(std::integral_constant<int, 0>{}, st ^ 1);
                issue_k(kreg[0], (t + 2) * KT);
                issue_v(std::integral_constant<int, 0>{}, (t + 2) * KT);
                __syncthreads();
                keep_cur = keep_next;
            }
            t0 = n_tiles;
        }
        const int t_full = PIPE ? n_it / NI : 0;
        if constexpr (PF == 1 && (DP == 64 || (DIRECT && DP == 128)) && !BIAS && MODE != kMaskPadding) {
            // (head dim 64 only: the wider kernels and the ones with a bias or a padding mask have no register to spare for
            // the second copy of the tile's code)
            // one register set: tile 0 on its own, then the tiles in pairs (odd, even) whose LDS stages are compile-time
            // constants, then what is left of the tiles the wave walks in full
            using IC0 = std::integral_constant<int, 0>;
            using IC1 = std::integral_constant<int, 1>;
            if (PIPE && t0 < t_full) {
                walk_full(0, IC0{}, IC0{}, IC0{}, std::false_type{});
                t0 = 1;
            }
            for (; PIPE && t0 + 2 <= t_full; t0 += 2) {
                walk_full(t0, IC0{}, IC0{}, IC1{}, std::true_type{});
                walk_full(t0 + 1, IC0{}, IC0{}, IC0{}, std::true_type{});
            }
            if (PIPE && t0 < t_full) {
                walk_full(t0, IC0{}, IC0{}, t0 & 1, std::true_type{});
                t0++;
            }
        } else {
            for (; PIPE && t0 + PF <= t_full; t0 += PF) {
                walk_full(t0, std::integral_constant<int, 2 % PF>{}, std::integral_constant<int, 1 % PF>{}, t0 & 1, std::false_type{});
                if (PF >= 2) walk_full(t0 + 1, std::integral_constant<int, 3 % PF>{}, std::integral_constant<int, 2 % PF>{}, (t0 + 1) & 1, std::false_type{});
                if (PF >= 3) walk_full(t0 + 2, std::integral_constant<int, 4 % PF>{}, std::integral_constant<int, 3 % PF>{}, (t0 + 2) & 1, std::false_type{});
            }
        }
        for (; t0 < n_tiles; t0 += PF) {
            walk_tile(t0, std::integral_constant<int, 2 % PF>{}, std::integral_constant<int, 1 % PF>{});
            if (PF >= 2 && t0 + 1 < n_tiles) walk_tile(t0 + 1, std::integral_constant<int, 3 % PF>{}, std::integral_constant<int, 2 % PF>{});
            if (PF >= 3 && t0 + 2 < n_tiles) walk_tile(t0 + 2, std::integral_constant<int, 4 % PF>{}, std::integral_constant<int, 3 % PF>{});
        }
        // a wave that walked every item of the workgroup still owes the last P.V
        if (PIPE && n_it == n_tiles * NI && n_it > 0) drain(v_at((n_tiles - 1) & 1, NI - 1));
        __syncthreads();  // the output rows are staged over the tiles
    }
    // (a workgroup without tiles still has its early requests in flight: they land in its LDS)
    if constexpr (DIRECT) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");

    // ---- output: acc_o[dt][4j + e] = O^T[d = 32dt + 8j + 4hh + e][row col of the wave].  A lane holds 8-byte pieces of
    // its row; the wave parks its 32 normalised rows in its own region of LDS (every wave is past the last
    // barrier, and the region's previous content was read by this wave alone) and streams them out as whole rows,
    // 16 bytes per lane.
    const float l = t_sum_with_other_half(l_run);
    if constexpr (SPLIT) {
        // the partial of this span: O as accumulated (relative to the running max as it stands), that max in the exp2
        // domain, the row sum.  A workgroup without tiles, or a row that saw no key of the span, leaves (0, -inf, 0).
        const int r = q0 + 32 * wq + col;
        if (r < rows_total) {
            const size_t slot = (((size_t)b * p.kv_heads + kvh) * (size_t)rows_total + (size_t)r) * (size_t)p.n_splits + (size_t)split;
            float* const po = p.part_o + slot * (size_t)D;
#pragma unroll
            for (int dt = 0; dt < DT; dt++)
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    const int d0 = 32 * dt + 8 * j + 4 * hh;
                    if (d0 < D)
                        *(f32x4_t*)(po + d0) = f32x4_t{acc_o[dt][4 * j], acc_o[dt][4 * j + 1], acc_o[dt][4 * j + 2], acc_o[dt][4 * j + 3]};
                }
            if (hh == 0) {
                p.part_ml[2 * slot] = m_run * cc;
                p.part_ml[2 * slot + 1] = l;
            }
        }
        return;
    }
    const bool good = (l > 0.0f) && (l < __uint_as_float(0x7f800000u)) && !poison;
    // the hardware reciprocal (1 ulp) instead of the division's dozen instructions: the output is rounded to bf16
    const float inv_l = __builtin_amdgcn_rcpf(l);
    // Packed rows are positions of a chunked decode: one that sees no key at all is a row of zeros, as the reference's
    // decode kernels leave it (crates/rustorch-metal/src/kernels.rs:14504-14514: every loop runs zero times), not the
    // NaN row of flash_forward's l > 0 test.  l == 0 exactly when no key was weighed (a visible key gives P >= 1).
    const float bad = (PACKED && l == 0.0f) ? 0.0f : quiet_nan();
    uint16_t* const obuf = (uint16_t*)(lds + wq * Cfg::REGION);
    const float fill = p.zero_padded_rows ? 0.0f : quiet_nan();
    if (n_tiles > 0) {
        uint16_t* const orow = obuf + col * LDK + 4 * hh;
        if (__all(good && valid)) {
            // the common wave: one multiplication per element (a branch of its own: as a select inside one loop the
            // compiler kept three selects per element for every wave)
#pragma unroll
            for (int dt = 0; dt < DT; dt++)
#pragma unroll
                for (int j = 0; j < 4; j++)
                    *(u32x2_t*)(orow + 32 * dt + 8 * j) =
                        u32x2_t{t_cvt_pk_bf16(acc_o[dt][4 * j] * inv_l, acc_o[dt][4 * j + 1] * inv_l),
                                t_cvt_pk_bf16(acc_o[dt][4 * j + 2] * inv_l, acc_o[dt][4 * j + 3] * inv_l)};
        } else {
#pragma unroll
            for (int dt = 0; dt < DT; dt++)
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    float o[4];
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        float x = good ? acc_o[dt][4 * j + e] * inv_l : bad;
                        if (!valid) x = fill;
                        o[e] = x;
                    }
                    *(u32x2_t*)(orow + 32 * dt + 8 * j) = u32x2_t{t_cvt_pk_bf16(o[0], o[1]), t_cvt_pk_bf16(o[2], o[3])};
                }
        }
    }
    // (the same wave wrote and now reads: no barrier needed, the LDS queue is in order)
    const uint32_t fill2 = t_cvt_pk_bf16(fill, fill);
    if constexpr (!PACKED && 64 % CH == 0 && DP <= 128) {
        // rows of one head, and a wave's store instruction covers whole rows: lane l moves chunk l % CH of the rows
        // l / CH, l / CH + 64 / CH, ... -- one address, then a constant step
        constexpr int RS = 64 / CH;  // rows per store instruction
        const int row0 = (int)((unsigned)lane / (unsigned)CH), ch = (int)((unsigned)lane % (unsigned)CH);
        const int rr0 = q0 + 32 * wq + row0;
        uint16_t* dst = p.out + (size_t)b * p.lo.batch_stride + (size_t)h0 * p.lo.head_stride + (size_t)rr0 * p.lo.row_pitch + 8 * ch;
        const size_t step = (size_t)RS * (size_t)p.lo.row_pitch;
        const uint16_t* src = obuf + row0 * LDK + 8 * ch;
        const bool col_ok = 8 * ch < D;
#pragma unroll
        for (int n = 0; n < CH / 2; n++) {
            const int rr = rr0 + RS * n;
            // no key tile walked: padded rows get the fill value, valid rows (which then see no key at all) NaN
            const uint32_t f2 = rr < n_q ? 0x7fc07fc0u : fill2;
            u32x4_t val = {f2, f2, f2, f2};
            if (n_tiles > 0) val = *(const u32x4_t*)(src + RS * n * LDK);
            if (rr < rows_total && col_ok) *(u32x4_t*)dst = val;
            dst += step;
        }
    } else {
#pragma unroll
        for (int n = 0; n < CH / 2; n++) {
            const int cidx = lane + 64 * n;
            const int row = cidx / CH, ch = cidx - row * CH;
            const int rr = q0 + 32 * wq + row;
            const int sp = G > 1 ? rr / G : rr;
            const int gg = rr - sp * G;
            // no key tile walked: padded rows get the fill value, valid rows (which then see no key at all) NaN -- zeros
            // when the rows are positions of a chunked decode
            const uint32_t f2 = sp < n_q ? (PACKED ? 0u : 0x7fc07fc0u) : fill2;
            u32x4_t val = {f2, f2, f2, f2};
            if (n_tiles > 0) val = *(const u32x4_t*)(obuf + row * LDK + 8 * ch);
            if (rr < rows_total && 8 * ch < D) {
                uint16_t* dst = p.out + (size_t)b * p.lo.batch_stride + (size_t)(h0 + gg) * p.lo.head_stride +
                                (size_t)sp * p.lo.row_pitch + 8 * ch;
                *(u32x4_t*)dst = val;
            }
        }
    }
}

// Folds the partials the SPLIT kernel leaves: thread (row, d) walks the row's n_splits partials (o[d], m, l), weighs each
// by 2^(m - max m) and writes o / l as bf16 where the unsplit kernel would have written the row.  No partial with a
// key (every m is -inf): the position sees no key at all, a row of zeros.
__global__ __launch_bounds__(256) void flash_split_merge_kernel(FlashTileParams p) {
    const int D = p.dim, G = p.pack;
    const size_t rows_total = (size_t)p.seq_q * G;
    const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
    const size_t row_all = idx / (size_t)D;
    const int d = (int)(idx - row_all * (size_t)D);
    if (row_all >= (size_t)p.batch * p.kv_heads * rows_total) return;
    const size_t r = row_all % rows_total, bk = row_all / rows_total;
    const int kvh = (int)(bk % (size_t)p.kv_heads), b = (int)(bk / (size_t)p.kv_heads);
    const float* ml = p.part_ml + 2 * row_all * (size_t)p.n_splits;
    const float* po = p.part_o + row_all * (size_t)p.n_splits * (size_t)D + d;
    // One pass, eight partials at a time: the loads of a group are independent of each other (a dependent load per
    // partial would cost a memory latency each), and the running (m, acc, l) is rescaled once per group.
    constexpr int kGroup = 8;
    float m_all = neg_inf(), acc = 0.0f, l_all = 0.0f;
    bool nan_m = false;
    for (int k0 = 0; k0 < p.n_splits; k0 += kGroup) {
        float mv[kGroup], lv[kGroup], ov[kGroup];
#pragma unroll
        for (int j = 0; j < kGroup; j++) {
            const int k = min(k0 + j, p.n_splits - 1);  // repeats of the last partial get weight 0 below
            mv[j] = ml[2 * k];
            lv[j] = ml[2 * k + 1];
            ov[j] = po[(size_t)k * D];
        }
        float m_new = m_all;
#pragma unroll
        for (int j = 0; j < kGroup; j++) {
            m_new = fmaxf(m_new, mv[j]);
            nan_m |= (mv[j] != mv[j]);
        }
        const float m_use = (m_new == neg_inf()) ? 0.0f : m_new;
        const float rescale = (m_all == neg_inf()) ? 0.0f : __builtin_amdgcn_exp2f(m_all - m_use);
        acc *= rescale;
        l_all *= rescale;
#pragma unroll
        for (int j = 0; j < kGroup; j++) {
            // an empty partial (m = -inf) is the identity
            const float w = (k0 + j < p.n_splits && mv[j] != neg_inf()) ? __builtin_amdgcn_exp2f(mv[j] - m_use) : 0.0f;
            acc += ov[j] * w;
            l_all += lv[j] * w;
        }
        m_all = m_new;
    }
    float x = acc / l_all;
    if (m_all == neg_inf() && !nan_m) x = 0.0f;
    const size_t s_pos = r / (size_t)G;
    const int g = (int)(r - s_pos * (size_t)G);
    p.out[(size_t)b * p.lo.batch_stride + (size_t)(kvh * G + g) * p.lo.head_stride + s_pos * (size_t)p.lo.row_pitch + d] =
        f32_to_bf16_bits(x);
}

// ---------------------------------------------------------------------------------------------------------------
// The same walk with 64 query rows per wave (two blocks of 32), head dim 64, masks none / causal, rows of one head.
// At head dim 64 a 32-key item is only 8 matrix instructions per 32 rows: what paces the tile kernel there is the
// movement of a key tile (LDS parking, the workgroup barrier per tile) and the operand reads, which are the same
// whether a wave multiplies a fragment into one row block or two.  Here every K and V fragment read from LDS feeds
// two matrix instructions, a tile in LDS serves 256 query rows between two barriers, and a workgroup's set-up is
// spread over twice the rows.  Two workgroups share a CU (two O blocks, two score tiles and their operands).
constexpr int WROWS = 256;  // query rows per workgroup: four waves of 64

template <int MODE>
__global__ __launch_bounds__(256, 2) void flash_wide_bf16_kernel(FlashTileParams p) {
    constexpr int DP = 64, KT = 64, LDK = DP + 8, LDV = DP + 32, NI = KT / 32, KS = DP / 16, DT = DP / 32, CH = DP / 8;
    constexpr int TTHREADS = 256, NL = KT * CH / TTHREADS, RB = 2;
    constexpr bool kCausal = MODE == kMaskCausal;
    constexpr int TILE_BYTES = 2 * KT * (LDK + LDV) * 2;  // two stages of K and V
    constexpr int REGION = 64 * LDK * 2;                  // a wave's staged output rows
    static_assert(4 * REGION <= TILE_BYTES, "the staged output rows fit over the tiles");
    static_assert(NI == 2 && KS == 2 * DT, "two items per tile, one P.V instruction per score instruction");

    __shared__ __attribute__((aligned(16))) unsigned char lds[TILE_BYTES];
    uint16_t* const Ks = (uint16_t*)lds;                 // [2][KT * LDK]
    uint16_t* const Vs = (uint16_t*)lds + 2 * KT * LDK;  // [2][KT * LDV]

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int col = lane & 31, hh = lane >> 5;
    const int rows_total = p.seq_q;
    const int hx = blockIdx.x, b = blockIdx.y;
    const int kvh = p.group_magic == 0 ? hx : (int)__umulhi((uint32_t)hx, p.group_magic);
    const uint16_t* const Kg = p.k + (size_t)b * p.lkv.batch_stride + (size_t)kvh * p.lkv.head_stride;
    const uint16_t* const Vg = p.v + (size_t)b * p.lkv.batch_stride + (size_t)kvh * p.lkv.head_stride;

    // ---- tile movement, as in the tile kernel: chunk c = tid + 256 n of a tile is (row c / CH, 16-byte chunk c % CH)
    u32x4_t kreg[NL], vreg[NL], k1[NL];
    uint32_t ld_off[NL], st_k[NL], st_v[NL];
    const uint32_t kv_pitch = (uint32_t)p.lkv.row_pitch;
#pragma unroll
    for (int n = 0; n < NL; n++) {
        const int c = tid + TTHREADS * n;
        const int row = c / CH, ch = c - row * CH;
        st_k[n] = (uint32_t)((row * LDK + 8 * ch) * 2);
        st_v[n] = (uint32_t)((2 * KT * LDK + row * LDV + 8 * ch) * 2);
        ld_off[n] = ((uint32_t)row * kv_pitch + (uint32_t)(8 * ch)) * 2u;
    }
    const uint32_t tile_bytes_g = (uint32_t)KT * kv_pitch * 2u;
    {  // tile 0 (K and V) and K of tile 1, before the lengths have arrived: descriptors that end with the tensor
        const uint32_t all_bytes = p.seq_kv > 0 ? ((uint32_t)(p.seq_kv - 1) * kv_pitch + (uint32_t)DP) * 2u : 0u;
        const __amdgpu_buffer_rsrc_t Kall = __builtin_amdgcn_make_buffer_rsrc((void*)Kg, 0, all_bytes, kBufferFlags);
        const __amdgpu_buffer_rsrc_t Vall = __builtin_amdgcn_make_buffer_rsrc((void*)Vg, 0, all_bytes, kBufferFlags);
#pragma unroll
        for (int n = 0; n < NL; n++) {
            kreg[n] = __builtin_amdgcn_raw_buffer_load_b128(Kall, ld_off[n], 0, 0);
            vreg[n] = __builtin_amdgcn_raw_buffer_load_b128(Vall, ld_off[n], 0, 0);
            k1[n] = __builtin_amdgcn_raw_buffer_load_b128(Kall, ld_off[n], tile_bytes_g, 0);
        }
    }

    const int n_q = p.q_lens ? min(max(p.q_lens[b], 0), p.seq_q) : p.seq_q;          // valid query positions
    const int n_keys = p.kv_lens ? min(max(p.kv_lens[b], 0), p.seq_kv) : p.seq_kv;  // keys that exist
    // rank of the query tile: the last one first; in a padded batch counted from the sequence's own last valid tile
    int qtile = (int)gridDim.z - 1 - (int)blockIdx.z;
    if (p.q_lens) {
        const int n_qt = (n_q + WROWS - 1) / WROWS;
        const int rank = (int)blockIdx.z;
        qtile = rank < n_qt ? n_qt - 1 - rank : rank;
    }
    const int q0 = qtile * WROWS;
    const int wq = (wave + hx + b + (int)blockIdx.z) & 3;  // which 64 rows of the tile: rotated, as in the tile kernel
    const int r0 = q0 + 64 * wq;                           // the wave's first row
    const int off = n_keys - n_q;                          // causal: the last valid query sees every key

    int kv_end = n_keys;
    if (kCausal) kv_end = min(n_keys, min(q0 + WROWS - 1, n_q - 1) + off + 1);
    if (q0 >= n_q) kv_end = 0;
    kv_end = max(kv_end, 0);
    const int n_tiles = (kv_end + KT - 1) / KT;

    const uint32_t fill2 = p.zero_padded_rows ? 0u : 0x7fc07fc0u;
    if (q0 >= n_q) {  // padded rows only: the fill value, and done
        const u32x4_t val = {fill2, fill2, fill2, fill2};
        uint16_t* const ob = p.out + (size_t)b * p.lo.batch_stride + (size_t)hx * p.lo.head_stride;
        for (int c = tid; c < WROWS * CH; c += TTHREADS) {
            const int row = c / CH, ch = c - row * CH;
            if (q0 + row < rows_total) *(u32x4_t*)(ob + (size_t)(q0 + row) * p.lo.row_pitch + 8 * ch) = val;
        }
        return;
    }
    // descriptors that end with the last key's row: rows behind it come back as zeros
    const uint32_t slab_bytes = n_keys > 0 ? ((uint32_t)(n_keys - 1) * kv_pitch + (uint32_t)DP) * 2u : 0u;
    const __amdgpu_buffer_rsrc_t Kbuf = __builtin_amdgcn_make_buffer_rsrc((void*)Kg, 0, slab_bytes, kBufferFlags);
    const __amdgpu_buffer_rsrc_t Vbuf = __builtin_amdgcn_make_buffer_rsrc((void*)Vg, 0, slab_bytes, kBufferFlags);
    if (n_keys < KT) {  // the early requests ended with the tensor, not with the sequence
#pragma unroll
        for (int n = 0; n < NL; n++)
            if ((tid + TTHREADS * n) / CH >= n_keys) vreg[n] = u32x4_t{0u, 0u, 0u, 0u};
    }

    f32x16_t acc_o[RB][DT];
#pragma unroll
    for (int rb = 0; rb < RB; rb++)
#pragma unroll
        for (int t = 0; t < DT; t++)
#pragma unroll
            for (int i = 0; i < 16; i++) acc_o[rb][t][i] = 0.0f;
    float m_run[RB], l_run[RB];
    bool valid[RB];
#pragma unroll
    for (int rb = 0; rb < RB; rb++) {
        m_run[rb] = neg_inf();
        l_run[rb] = 0.0f;
        valid[rb] = false;
    }
    const float cc = p.scale_log2e;  // exp2 argument per unit of score

    if (n_tiles > 0) {
        const int last_kv0 = (n_tiles - 1) * KT;
        auto issue_k = [&](int kv0) __attribute__((always_inline)) {
            const uint32_t tile_off = (uint32_t)min(kv0, last_kv0) * (kv_pitch * 2u);
#pragma unroll
            for (int n = 0; n < NL; n++) kreg[n] = __builtin_amdgcn_raw_buffer_load_b128(Kbuf, ld_off[n], tile_off, 0);
        };
        auto issue_v = [&](int kv0) __attribute__((always_inline)) {
            const uint32_t tile_off = (uint32_t)min(kv0, last_kv0) * (kv_pitch * 2u);
#pragma unroll
            for (int n = 0; n < NL; n++) vreg[n] = __builtin_amdgcn_raw_buffer_load_b128(Vbuf, ld_off[n], tile_off, 0);
        };
        auto park_k = [&](const u32x4_t (&src)[NL], int st) __attribute__((always_inline)) {
#pragma unroll
            for (int n = 0; n < NL; n++) *(u32x4_t*)(lds + st * (KT * LDK * 2) + st_k[n]) = src[n];
        };
        auto park_v = [&](int st) __attribute__((always_inline)) {
#pragma unroll
            for (int n = 0; n < NL; n++) *(u32x4_t*)(lds + st * (KT * LDV * 2) + st_v[n]) = vreg[n];
        };

        // ---- this lane's two query rows, and the wave's limits as scalars
        int lim[RB], wave_lim_min[RB];
        const int r_lim = min(rows_total, n_q);  // rows below it are valid
#pragma unroll
        for (int rb = 0; rb < RB; rb++) {
            const int r = r0 + 32 * rb + col;
            valid[rb] = r < r_lim;
            int l = n_keys - 1;  // last key this row sees
            if (kCausal) l = min(l, r + off);
            lim[rb] = valid[rb] ? l : -1;
            const int r_first = r0 + 32 * rb, r_last = r_first + 31;
            wave_lim_min[rb] = r_last < r_lim ? (kCausal ? min(n_keys - 1, r_first + off) : n_keys - 1) : -1;
        }
        const int r_top = min(r0 + 63, r_lim - 1);
        const int wave_lim_max = r0 < r_lim ? (kCausal ? min(n_keys - 1, r_top + off) : n_keys - 1) : -1;
        // items this wave walks: the ones that hold a key some row of it sees (a prefix of the workgroup's items)
        const int n_it = wave_lim_max < 0 ? 0 : min(n_tiles * NI, (wave_lim_max >> 5) + 1);

        // ---- Q as B operands: column q = lane % 32 of either row block, contraction slots 16 ks + 8 hh .. + 8
        bf16x8_t qreg[RB][KS];
#pragma unroll
        for (int rb = 0; rb < RB; rb++) {
            const int r_q = min(r0 + 32 * rb + col, rows_total - 1);  // (a row past the tensor reads the last row: it is masked and not written)
            const size_t q_off = (size_t)b * p.lq.batch_stride + (size_t)hx * p.lq.head_stride + (size_t)r_q * p.lq.row_pitch;
#pragma unroll
            for (int ks = 0; ks < KS; ks++)
                qreg[rb][ks] = __builtin_bit_cast(bf16x8_t, *(const u32x4_t*)(p.q + q_off + 16 * ks + 8 * hh));
        }
        const int k_off = col * LDK + 8 * hh;
        const int v_off = (((lane & 15) >> 2) + 4 * hh) * LDV + 16 * ((lane >> 4) & 1) + 4 * (lane & 3);

        // K(0), V(0) -> stage 0, K(1) -> stage 1; the register sets then take K(2) and V(1)
        park_k(kreg, 0);
        park_v(0);
        park_k(k1, 1);
        issue_k(2 * KT);
        issue_v(KT);
        __syncthreads();

        auto mask_item = [&](int rb, int k0, f32x16_t& sc) __attribute__((always_inline)) {
            if (k0 + 31 > wave_lim_min[rb]) {
                const int room = lim[rb] - k0 - 4 * hh;  // key k0 + 8 (i / 4) + 4 hh + i % 4 is hidden when it lies past lim
#pragma unroll
                for (int i = 0; i < 16; i++) sc[i] = (8 * (i >> 2) + (i & 3) > room) ? neg_inf() : sc[i];
            }
        };
        auto load_v = [&](int i, const uint16_t* vp) __attribute__((always_inline)) {
            const int u = i / DT, dt = i - u * DT;
            const u32x2_t lo = t_lds_read_tr16(vp + 16 * u * LDV + 32 * dt);
            const u32x2_t hi = t_lds_read_tr16(vp + 16 * u * LDV + 32 * dt + 8 * LDV);
            return u32x4_t{lo[0], lo[1], hi[0], hi[1]};
        };
        auto pin_f = [](float& x) __attribute__((always_inline)) { asm volatile("" : "+v"(x)); };
        auto pin_u = [](uint32_t& x) __attribute__((always_inline)) { asm volatile("" : "+v"(x)); };
        auto pin_b = [](bf16x8_t& x) __attribute__((always_inline)) { asm volatile("" : "+v"(x)); };

        float neg_mc[RB];  // -m_run * cc; +inf while a valid row has no max yet
        f32x16_t s_a[RB];                 // S(j), made at the end of step j - 1
        bf16x8_t p_a[RB][2], p_b[RB][2];  // P(j - 1) and P(j)
#pragma unroll
        for (int rb = 0; rb < RB; rb++) {
            neg_mc[rb] = valid[rb] ? __uint_as_float(0x7f800000u) : 0.0f;
            p_a[rb][0] = p_a[rb][1] = p_b[rb][0] = p_b[rb][1] = __builtin_bit_cast(bf16x8_t, u32x4_t{0u, 0u, 0u, 0u});
#pragma unroll
            for (int i = 0; i < 16; i++) s_a[rb][i] = 0.0f;
        }
        // S(0), and the running max started from it, so that the first step already runs the fast path
        if (n_it > 0) {
#pragma unroll
            for (int ks = 0; ks < KS; ks++) {
                const bf16x8_t kf = *(const bf16x8_t*)(Ks + k_off + 16 * ks);
#pragma unroll
                for (int rb = 0; rb < RB; rb++) s_a[rb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf, qreg[rb][ks], s_a[rb], 0, 0, 0);
            }
#pragma unroll
            for (int rb = 0; rb < RB; rb++) {
                mask_item(rb, 0, s_a[rb]);  // (the step applies the mask again, which changes nothing)
                const float m0 = t_max_with_other_half(t_max16(s_a[rb]));
                if (m0 > neg_inf()) {  // (false for -inf and for NaN: such a row waits for the slow path)
                    m_run[rb] = m0;
                    neg_mc[rb] = -m0 * cc;
                }
            }
        }

        // O^T += V(j-1)^T . P(j-1)^T alone: behind the wave's last item
        auto drain = [&](const uint16_t* vp) __attribute__((always_inline)) {
#pragma unroll
            for (int i = 0; i < KS; i++) {
                const int u = i / DT, dt = i - u * DT;
                const bf16x8_t av = __builtin_bit_cast(bf16x8_t, load_v(i, vp));
#pragma unroll
                for (int rb = 0; rb < RB; rb++)
                    acc_o[rb][dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(av, p_a[rb][u], acc_o[rb][dt], 0, 0, 0);
            }
        };
        auto exp_plain = [&](const f32x16_t& sc, float nmc, uint32_t (&w)[8], float& part) __attribute__((always_inline)) {
            float part0 = 0.0f, part1 = 0.0f;
#pragma unroll
            for (int e = 0; e < 8; e++) {
                const float x0 = __builtin_amdgcn_exp2f(__builtin_fmaf(sc[2 * e], cc, nmc));
                const float x1 = __builtin_amdgcn_exp2f(__builtin_fmaf(sc[2 * e + 1], cc, nmc));
                part0 += x0;
                part1 += x1;
                w[e] = t_cvt_pk_bf16(x0, x1);
            }
            part = part0 + part1;
        };
        // the slow path of a softmax step: the item max, O and l rescaled to it, P again from the scores
        auto raise_max_and_redo = [&](int rb, const f32x16_t& sc, uint32_t (&w)[8], float& part) __attribute__((always_inline)) {
            const float m_item = t_max_with_other_half(t_max16(sc));
            const float m_new = t_vmax(m_run[rb], m_item);
            const float m_use = (m_new == neg_inf()) ? 0.0f : m_new;
            const float alpha = __builtin_amdgcn_exp2f((m_run[rb] - m_use) * cc);  // m_run = -inf -> 0
            m_run[rb] = m_new;
            l_run[rb] *= alpha;
#pragma unroll
            for (int tt = 0; tt < DT; tt++)
#pragma unroll
                for (int i = 0; i < 16; i++) acc_o[rb][tt][i] *= alpha;
            const float mc = m_use * cc;
            neg_mc[rb] = (m_new == neg_inf()) ? (valid[rb] ? __uint_as_float(0x7f800000u) : 0.0f) : -mc;
            exp_plain(sc, -mc, w, part);
        };

        // One step: item j (keys k0 ..) gets its softmax step in both row blocks; K rows of item j + 1 are at kp, V rows
        // of item j - 1 at vp.  The registers hold one score tile per row block (two workgroups per CU), so the row
        // blocks are staggered: while block 0's P(j) is made its P.V instructions of item j - 1 run; while block 1's
        // P(j) is made, block 1's P.V instructions and block 0's S(j+1) run (into the registers block 0's S(j) has
        // just left); block 1's S(j+1) follows, and is still in flight when the next step starts on block 0.  Every V
        // and K fragment is read from LDS once and feeds both row blocks.  No row max in the steady state (see the
        // tile kernel).
        auto step = [&](int k0, const uint16_t* kp, const uint16_t* vp, bf16x8_t (&p_prev)[RB][2],
                        bf16x8_t (&p_new)[RB][2]) __attribute__((always_inline)) {
            mask_item(0, k0, s_a[0]);
            u32x4_t vop[KS], kop[KS];
            constexpr int PER = 16 / KS;  // scores of a row block per group
            const f32x16_t zero16 = {0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f};
            // the vector work of group g of row block rb: a quarter of P(j), fenced
            auto quarter = [&](int rb, int g, float (&part)[2], uint32_t (&w)[8]) __attribute__((always_inline)) {
                float t[PER];
#pragma unroll
                for (int i = 0; i < PER; i++) t[i] = __builtin_fmaf(s_a[rb][PER * g + i], cc, neg_mc[rb]);
#pragma unroll
                for (int i = 0; i < PER; i++) t[i] = __builtin_amdgcn_exp2f(t[i]);
#pragma unroll
                for (int i = 0; i < PER; i += 2) {
                    part[0] += t[i];
                    part[1] += t[i + 1];
                    w[(PER * g + i) / 2] = t_cvt_pk_bf16(t[i], t[i + 1]);
                }
#pragma unroll
                for (int i = 0; i < PER; i++) pin_f(t[i]);
                pin_f(part[0]);
                pin_f(part[1]);
#pragma unroll
                for (int i = 0; i < PER; i += 2) pin_u(w[(PER * g + i) / 2]);
            };
            auto finish = [&](int rb, float (&part)[2], uint32_t (&w)[8]) __attribute__((always_inline)) {
                float pt = part[0] + part[1];
                if (__builtin_expect(__any(!(pt <= kTileTrigSum)), 0)) raise_max_and_redo(rb, s_a[rb], w, pt);
                l_run[rb] += pt;
                p_new[rb][0] = __builtin_bit_cast(bf16x8_t, u32x4_t{w[0], w[1], w[2], w[3]});
                p_new[rb][1] = __builtin_bit_cast(bf16x8_t, u32x4_t{w[4], w[5], w[6], w[7]});
            };
            // ---- row block 0: P(j), with its P.V of item j - 1
            {
                float part[2] = {0.0f, 0.0f};
                uint32_t w[8];
                vop[0] = load_v(0, vp);
#pragma unroll
                for (int g = 0; g < KS; g++) {
                    if (g + 1 < KS) vop[g + 1] = load_v(g + 1, vp);
                    const int u = g / DT, dt = g - u * DT;
                    acc_o[0][dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, vop[g]), p_prev[0][u], acc_o[0][dt], 0, 0, 0);
                    quarter(0, g, part, w);
                    pin_b(p_prev[0][u]);
                }
                finish(0, part, w);
            }
            // ---- row block 1: P(j), with its P.V of item j - 1 and row block 0's S(j+1)
            {
                mask_item(1, k0, s_a[1]);
                float part[2] = {0.0f, 0.0f};
                uint32_t w[8];
                kop[0] = *(const u32x4_t*)(kp);
#pragma unroll
                for (int g = 0; g < KS; g++) {
                    if (g + 1 < KS) kop[g + 1] = *(const u32x4_t*)(kp + 16 * (g + 1));
                    const int u = g / DT, dt = g - u * DT;
                    acc_o[1][dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, vop[g]), p_prev[1][u], acc_o[1][dt], 0, 0, 0);
                    s_a[0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, kop[g]), qreg[0][g], g == 0 ? zero16 : s_a[0], 0, 0, 0);
                    quarter(1, g, part, w);
                    pin_b(p_prev[1][u]);
                    pin_b(qreg[0][g]);
                }
                finish(1, part, w);
            }
            // ---- row block 1's S(j+1)
#pragma unroll
            for (int g = 0; g < KS; g++)
                s_a[1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, kop[g]), qreg[1][g], g == 0 ? zero16 : s_a[1], 0, 0, 0);
        };
        // a step whose results are moved back into the first of each pair
        auto step_a = [&](int k0, const uint16_t* kp, const uint16_t* vp) __attribute__((always_inline)) {
            step(k0, kp, vp, p_a, p_b);
#pragma unroll
            for (int rb = 0; rb < RB; rb++) {
                p_a[rb][0] = p_b[rb][0];
                p_a[rb][1] = p_b[rb][1];
            }
        };
        // slot j of the walk: a step while the wave has items left, then once the P.V of its last item
        auto slot = [&](int j, const uint16_t* kp, const uint16_t* vp) __attribute__((always_inline)) {
            if (j < n_it) step_a(32 * j, kp, vp);
            else if (j == n_it && n_it > 0) drain(vp);
        };
        // behind the barrier of tile t: K(t+2) and V(t+1) parked over K(t) and V(t-1), K(t+3) and V(t+2) requested
        auto park_next = [&](int t, int st) __attribute__((always_inline)) {
            park_k(kreg, st);
            park_v(st ^ 1);
            issue_k((t + 3) * KT);
            issue_v((t + 2) * KT);
        };
        // a tile of which the wave walks both items: straight-line code, the pairs swapped from step to step
        auto walk_full = [&](int t, auto st_c, auto later_c) __attribute__((always_inline)) {
            const int st = st_c;
            constexpr bool kLater = decltype(later_c)::value;
            const uint16_t* const k_st = Ks + st * KT * LDK + k_off;
            const uint16_t* const k_ot = Ks + (st ^ 1) * KT * LDK + k_off;
            const uint16_t* const v_st = Vs + st * KT * LDV + v_off;
            const uint16_t* const v_ot = Vs + (st ^ 1) * KT * LDV + v_off;
            const int k0 = t * KT;
            step(k0, k_st + 32 * LDK, (!kLater && t == 0) ? v_st : v_ot + 32 * LDV, p_a, p_b);
            __syncthreads();
            park_next(t, st);
            step(k0 + 32, k_ot, v_st, p_b, p_a);
        };
        auto walk_tile = [&](int t) __attribute__((always_inline)) {
            const int st = t & 1;
            const uint16_t* const k_st = Ks + st * KT * LDK + k_off;
            const uint16_t* const k_ot = Ks + (st ^ 1) * KT * LDK + k_off;
            const uint16_t* const v_st = Vs + st * KT * LDV + v_off;
            const uint16_t* const v_ot = Vs + (st ^ 1) * KT * LDV + v_off;
            slot(t * NI, k_st + 32 * LDK, t == 0 ? v_st : v_ot + 32 * LDV);
            __syncthreads();
            park_next(t, st);
            slot(t * NI + 1, k_ot, v_st);
        };
        using IC0 = std::integral_constant<int, 0>;
        using IC1 = std::integral_constant<int, 1>;
        const int t_full = n_it / NI;
        int t0 = 0;
        if (t0 < t_full) {
            walk_full(0, IC0{}, std::false_type{});
            t0 = 1;
        }
        for (; t0 + 2 <= t_full; t0 += 2) {
            walk_full(t0, IC1{}, std::true_type{});
            walk_full(t0 + 1, IC0{}, std::true_type{});
        }
        if (t0 < t_full) {
            walk_full(t0, t0 & 1, std::true_type{});
            t0++;
        }
        for (; t0 < n_tiles; t0++) walk_tile(t0);
        // a wave that walked every item of the workgroup still owes the last P.V
        if (n_it == n_tiles * NI && n_it > 0) drain(Vs + ((n_tiles - 1) & 1) * KT * LDV + v_off + 32 * LDV);
        __syncthreads();  // the output rows are staged over the tiles
    }

    // ---- output: the wave parks its 64 normalised rows in its own region of LDS and streams them out as whole rows
    uint16_t* const obuf = (uint16_t*)(lds + wq * REGION);
    const float fill = p.zero_padded_rows ? 0.0f : quiet_nan();
    if (n_tiles > 0) {
#pragma unroll
        for (int rb = 0; rb < RB; rb++) {
            const float l = t_sum_with_other_half(l_run[rb]);
            const bool good = (l > 0.0f) && (l < __uint_as_float(0x7f800000u));
            const float inv_l = __builtin_amdgcn_rcpf(l);
            uint16_t* const orow = obuf + (32 * rb + col) * LDK + 4 * hh;
            if (__all(good && valid[rb])) {
#pragma unroll
                for (int dt = 0; dt < DT; dt++)
#pragma unroll
                    for (int j = 0; j < 4; j++)
                        *(u32x2_t*)(orow + 32 * dt + 8 * j) =
                            u32x2_t{t_cvt_pk_bf16(acc_o[rb][dt][4 * j] * inv_l, acc_o[rb][dt][4 * j + 1] * inv_l),
                                    t_cvt_pk_bf16(acc_o[rb][dt][4 * j + 2] * inv_l, acc_o[rb][dt][4 * j + 3] * inv_l)};
            } else {
#pragma unroll
                for (int dt = 0; dt < DT; dt++)
#pragma unroll
                    for (int j = 0; j < 4; j++) {
                        float o[4];
#pragma unroll
                        for (int e = 0; e < 4; e++) {
                            float x = good ? acc_o[rb][dt][4 * j + e] * inv_l : quiet_nan();
                            if (!valid[rb]) x = fill;
                            o[e] = x;
                        }
                        *(u32x2_t*)(orow + 32 * dt + 8 * j) = u32x2_t{t_cvt_pk_bf16(o[0], o[1]), t_cvt_pk_bf16(o[2], o[3])};
                    }
            }
        }
    }
    // (the same wave wrote and now reads: no barrier needed, the LDS queue is in order)
    {
        constexpr int RS = 64 / CH;  // rows per store instruction
        const int row0 = lane / CH, ch = lane % CH;
        const int rr0 = r0 + row0;
        uint16_t* dst = p.out + (size_t)b * p.lo.batch_stride + (size_t)hx * p.lo.head_stride + (size_t)rr0 * p.lo.row_pitch + 8 * ch;
        const size_t step_e = (size_t)RS * (size_t)p.lo.row_pitch;
        const uint16_t* src = obuf + row0 * LDK + 8 * ch;
#pragma unroll
        for (int n = 0; n < 64 / RS; n++) {
            const int rr = rr0 + RS * n;
            // no key tile walked: padded rows get the fill value, valid rows (which then see no key at all) NaN
            const uint32_t f2 = rr < n_q ? 0x7fc07fc0u : fill2;
            u32x4_t val = {f2, f2, f2, f2};
            if (n_tiles > 0) val = *(const u32x4_t*)(src + RS * n * LDK);
            if (rr < rows_total) *(u32x4_t*)dst = val;
            dst += step_e;
        }
    }
}

template <int DP, int MODE, bool BIAS, bool PACKED, bool SPLIT = false, bool WIN = false, bool DIRECT = false>
hipError_t launch_one(hipStream_t stream, const FlashTileParams& p, dim3 grid) {
    hipLaunchKernelGGL((flash_tile_bf16_kernel<DP, MODE, BIAS, PACKED, SPLIT, WIN, DIRECT>), grid, dim3(TileCfg<DP>::THREADS), 0, stream, p);
    return hipGetLastError();
}

template <int DP>
hipError_t launch_dp(hipStream_t stream, const FlashTileParams& p, dim3 grid) {
    constexpr bool kDirect = DP == 64 || DP == 128;  // head dim 64 or 128 exactly: the tiles go straight to LDS
    const bool direct = kDirect && p.dim == DP;
    if (p.n_splits > 1) {  // (rows packed over a group of one head are rows of that head)
        hipError_t e = direct ? launch_one<DP, kMaskCausal, false, true, true, false, kDirect>(stream, p, grid)
                              : launch_one<DP, kMaskCausal, false, true, true>(stream, p, grid);
        if (e != hipSuccess) return e;
        const size_t total = (size_t)p.batch * p.kv_heads * (size_t)p.seq_q * p.pack * (size_t)p.dim;
        hipLaunchKernelGGL(flash_split_merge_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, stream, p);
        return hipGetLastError();
    }
    if (p.pack > 1 || p.decode_rows) return direct ? launch_one<DP, kMaskCausal, false, true, false, false, kDirect>(stream, p, grid)
                                  : launch_one<DP, kMaskCausal, false, true>(stream, p, grid);
    if (p.window > 0) return direct ? launch_one<DP, kMaskCausal, false, false, false, true, kDirect>(stream, p, grid)
                                    : launch_one<DP, kMaskCausal, false, false, false, true>(stream, p, grid);
    if (p.bias) return launch_one<DP, kMaskNone, true, false>(stream, p, grid);
    if (direct && !p.bias && p.mask == kMaskNone) return launch_one<DP, kMaskNone, false, false, false, false, kDirect>(stream, p, grid);
    if (direct && !p.bias && p.mask == kMaskCausal) return launch_one<DP, kMaskCausal, false, false, false, false, kDirect>(stream, p, grid);
    switch (p.mask) {
        case kMaskNone: return launch_one<DP, kMaskNone, false, false>(stream, p, grid);
        case kMaskCausal: return launch_one<DP, kMaskCausal, false, false>(stream, p, grid);
        case kMaskPadding: return launch_one<DP, kMaskPadding, false, false>(stream, p, grid);
        default: return hipErrorInvalidValue;
    }
}

}  // namespace

bool flash_tile_bf16_supported(int dim) { return dim > 0 && dim <= 256 && dim % 8 == 0; }
int flash_tile_bf16_key_tile(int dim) { return dim <= 128 ? 64 : 32; }
// The kernel addresses the keys of one (batch, kv head) with 32-bit byte offsets (tile offset + lane offset, the
// requests that run a few tiles past the last one included).
bool flash_tile_bf16_addressable(long long seq_kv, long long row_pitch) {
    return seq_kv >= 0 && row_pitch > 0 && (unsigned long long)(seq_kv + 512) * (unsigned long long)row_pitch * 2ull < (1ull << 32);
}

// 64 rows per wave: head dim 64 exactly, rows of one head, masks none / causal (with or without per-sequence lengths)
bool flash_wide_bf16_supported(const FlashTileParams& p) {
    return p.dim == 64 && p.pack <= 1 && !p.bias && p.n_splits <= 1 && (p.mask == kMaskNone || p.mask == kMaskCausal) &&
           flash_tile_bf16_addressable(p.seq_kv, p.lkv.row_pitch);
}

hipError_t launch_flash_wide_bf16(hipStream_t stream, const FlashTileParams& params) {
    FlashTileParams p = params;
    if (p.batch == 0 || p.heads == 0 || p.seq_q == 0) return hipSuccess;
    if (!flash_wide_bf16_supported(p) || p.group < 1) return hipErrorInvalidValue;
    const long long n_qtiles = ((long long)p.seq_q + WROWS - 1) / WROWS;
    if (p.batch > 65535 || n_qtiles > 65535 || p.heads > 65535) return hipErrorInvalidValue;  // grid limits
    p.pack = 1;
    p.group_magic = p.group > 1 ? (uint32_t)(0x100000000ull / (unsigned long long)p.group) + 1u : 0u;
    dim3 grid((unsigned)p.heads, (unsigned)p.batch, (unsigned)n_qtiles);
    if (p.mask == kMaskCausal) hipLaunchKernelGGL(flash_wide_bf16_kernel<kMaskCausal>, grid, dim3(256), 0, stream, p);
    else hipLaunchKernelGGL(flash_wide_bf16_kernel<kMaskNone>, grid, dim3(256), 0, stream, p);
    return hipGetLastError();
}

hipError_t launch_flash_tile_bf16(hipStream_t stream, const FlashTileParams& params) {
    FlashTileParams p = params;
    if (p.batch == 0 || p.heads == 0 || p.seq_q == 0) return hipSuccess;
    if (!flash_tile_bf16_supported(p.dim) || p.pack < 1) return hipErrorInvalidValue;
    if (p.bias && p.mask != kMaskNone) return hipErrorInvalidValue;
    if (!flash_tile_bf16_addressable(p.seq_kv, p.lkv.row_pitch)) return hipErrorInvalidValue;
    if ((p.pack > 1 || p.decode_rows) && (p.bias || p.mask != kMaskCausal)) return hipErrorInvalidValue;  // packed rows: the chunked decode only
    if (p.window < 0 || (p.window > 0 && (p.pack > 1 || p.decode_rows || p.bias || p.mask != kMaskCausal || p.n_splits > 1))) return hipErrorInvalidValue;
    const long long rows = (long long)p.seq_q * p.pack;
    const long long n_qtiles = (rows + TROWS - 1) / TROWS;
    const long long heads_u = (p.pack > 1 || p.decode_rows) ? p.kv_heads : p.heads;
    if (p.n_splits < 1) p.n_splits = 1;
    if (p.n_splits > 1 && (p.pack != p.group || p.bias || p.mask != kMaskCausal || !p.part_o || !p.part_ml))
        return hipErrorInvalidValue;  // the chunked decode only
    if (p.batch > 65535 || n_qtiles * p.n_splits > 65535 || heads_u > 65535 || p.group < 1) return hipErrorInvalidValue;  // grid limits
    p.group_magic = p.group > 1 ? (uint32_t)(0x100000000ull / (unsigned long long)p.group) + 1u : 0u;
    dim3 grid((unsigned)heads_u, (unsigned)p.batch, (unsigned)(n_qtiles * p.n_splits));
    if (p.dim <= 32) return launch_dp<32>(stream, p, grid);
    if (p.dim <= 64) return launch_dp<64>(stream, p, grid);
    if (p.dim <= 96) return launch_dp<96>(stream, p, grid);
    if (p.dim <= 128) return launch_dp<128>(stream, p, grid);
    return launch_dp<256>(stream, p, grid);
}

}  // namespace rt
