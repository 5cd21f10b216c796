// bf16 flash-attention forward (prefill) for gfx950.  Device counterpart of
// flash_forward_masked (crates/rustorch-attention/src/cpu_forward.rs:193-425) for bf16
// tensors: bf16 in, f32 accumulation on the matrix cores, bf16 out rounded once.
//
// Persistent grid, one workgroup of 8 wavefronts (two per SIMD) per CU.  A job is 256 query rows of
// one (batch, head): each wave owns 32 rows, and the workgroup walks the keys 128 at a time through a
// double-buffered LDS tile that the waves fill with direct global->LDS loads (no registers, no LDS
// store instructions).  A wave treats the tile as four 32-key items:
//
//   S^T[kv, q]  = K[kv, :] . Q[q, :]      v_mfma_f32_32x32x16_bf16, A = K tile (LDS), B = Q (registers)
//   online softmax on S^T: lane l holds 16 scores of query row l % 32, so row max / row sum are
//                          in-lane plus one exchange with lane l ^ 32 (v_permlane32_swap)
//   O^T[d, q]  += V^T[d, kv] . P^T[kv, q]  A = V tile, read transposed out of its row-major LDS
//                                          copy by ds_read_b64_tr_b16; B = P (registers)
//
// The C layout of the first product (lane: column q, rows kv = 8j + 4*(l/32) + r) is, read as 8
// consecutive registers, exactly a B operand of the second product under a fixed permutation of
// the 16 contraction slots; the V operand is fetched with the same permutation, so P is never
// written to LDS.
//
// Schedule.  A wave can start one instruction every four to five cycles whatever its kind, and a
// matrix instruction keeps the matrix pipe busy for 32 cycles, so a wave that only multiplies leaves
// most issue slots free while a wave that only does softmax needs all of them.  The two waves of a SIMD
// therefore alternate, one cluster apart:
//
//   C(k): S^T(k) = K(k).Q^T and O^T += V(k-1)^T.P(k-1)^T (16 matrix instructions, operands in registers),
//         with the LDS reads of the NEXT cluster's operands (V(k), K(k+1)) slotted in between and the
//         global->LDS requests of the next tile behind them;
//   S(k): P(k) = exp2(..), row sums, conversion to bf16, overflow check: vector work only.
//
// Waves 0-3 run C(k) while waves 4-7 run S(k-1), then they swap.  The alternation is not enforced cluster
// by cluster: the matrix pipe is the shared resource, a wave in its matrix cluster runs at raised priority,
// and a wave whose partner holds the pipe gets the gaps.  The workgroup meets at two barriers per step only, the two the LDS tile needs:
// "the next tile has landed" before its first read (the matrix cluster of item 3) and "this tile has been
// read" before the requests that overwrite it (item 0 of the next step).  Waves 0-3 pass them behind their
// softmax clusters of items 2 and 3, waves 4-7 behind their matrix clusters of the same items, which also
// puts the two groups one cluster apart again twice per step.
//
// LDS tiles are unpadded; bank conflicts are avoided by an XOR swizzle of the 16-byte slots of a row,
// applied on the global side of the load (lane l of a load instruction always lands at LDS byte 16*l
// of its 1 KB block, so it fetches the slot that belongs there).
//
// The steady-state softmax takes no row max at all: P is formed against the running max as it stands (a
// stale max scales a row's P, O and l by one common factor), and the lane's share of the row sum, which is
// needed anyway, bounds every P of the lane.  Only when a share passes 2^16, or is not a number, or the row
// has no max yet, does the wave compute the item max, rescale O and l and redo P from the scores.
#include "rt_common.hpp"
#include "rt_kernels.hpp"

#include <type_traits>

namespace rt {

namespace {

constexpr int NWAVES = 8;
constexpr int NTHREADS = 64 * NWAVES;
constexpr int BR = 32 * NWAVES;  // query rows per job
constexpr int BC = 128;          // key rows per step (one barrier per step)
constexpr int NITEMS = BC / 32;  // 32-key items per step
constexpr float kTrigSum = 65536.0f;  // a lane's 16-key share of a row sum above this sends the wave to the slow path

typedef short s16x4_t __attribute__((ext_vector_type(4)));
typedef float f32x2_t __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));

__device__ __forceinline__ uint32_t cvt_pk_bf16(float lo, float hi) {
    f32x2_t x = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(x, bf16x2_t));  // v_cvt_pk_bf16_f32, RNE
}

// Transposing LDS read.  Within each group of 16 lanes, lane j receives element (j % 4) of the 8
// bytes addressed by lanes 4e + j/4, e = 0..3.  With lane 4e + c pointing at row k0+e, columns
// n0+4c.., lane j ends up with column n0+j of rows k0..k0+3: a contraction-major MFMA operand
// fragment out of a row-major tile.
__device__ __forceinline__ u32x2_t lds_read_tr16(const unsigned char* p) {
    s16x4_t v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4_t __attribute__((address_space(3)))*)(p));
    return __builtin_bit_cast(u32x2_t, v);
}

// plain v_max_f32: returns the non-NaN operand, without the canonicalising extra instruction fmaxf gets
__device__ __forceinline__ float vmax(float a, float b) {
    float d;
    asm("v_max_f32 %0, %1, %2" : "=v"(d) : "v"(a), "v"(b));
    return d;
}
// max / sum of a value with the one held by lane l ^ 32, without going through LDS:
// v_permlane32_swap leaves (lower half, lower half) in one register and (upper, upper) in the other.
__device__ __forceinline__ float max_with_other_half(float x) {
    auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return vmax(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float sum_with_other_half(float x) {
    auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}
// Max of the 16 scores a lane holds, as three chains of three-input maxima.  Written with the compiler's own max and
// not as inline assembly: the scores are results of matrix instructions, and a vector instruction that reads a
// matrix result needs wait states that only the compiler's hazard pass inserts (it does not look inside assembly).
// Runs on the slow path only.
__device__ __forceinline__ float max3(float a, float b, float c) { return __builtin_fmaxf(__builtin_fmaxf(a, b), c); }
__device__ __forceinline__ float max16(const f32x16_t& s) {
    float t0 = max3(s[0], s[1], s[2]), t1 = max3(s[3], s[4], s[5]), t2 = max3(s[6], s[7], s[8]);
    t0 = max3(t0, s[9], s[10]);
    t1 = max3(t1, s[11], s[12]);
    t2 = max3(t2, s[13], s[14]);
    return __builtin_fmaxf(max3(t0, t1, t2), s[15]);
}
// 16 bytes per lane from global memory straight into LDS: lane l lands at LDS byte address
// lds_block + 16*l (lds_block is wave-uniform and goes through M0).  Issued as inline assembly so that the compiler's counter
// bookkeeping does not treat every later LDS read as dependent on it: completion is awaited explicitly
// (s_waitcnt vmcnt(0) before the barrier that publishes the tile).  Loads the compiler does not know of
// can only make its own vmcnt waits longer, never shorter, because the counter retires in order.
__device__ __forceinline__ void load_to_lds(const void* base, uint32_t byte_off, uint32_t lds_block) {
    // base is wave-uniform (a scalar register pair); the lane's unsigned 32-bit byte offset is added to it
    const uint32_t lds_addr = __builtin_amdgcn_readfirstlane(lds_block);
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                 :
                 : "s"(lds_addr), "v"(byte_off), "s"(base)
                 : "memory");
}

// n / d for 0 <= n < 2^22 and d >= 1 with inv = 1.0f / d: the float quotient is off by at most one.  An integer
// division costs some thirty instructions, and the job bookkeeping does four per job.
__device__ __forceinline__ int div_small(int n, int d, float inv) {
    int q = (int)((float)n * inv);
    const int r = n - q * d;
    q += (r >= d) ? 1 : 0;
    q -= (r < 0) ? 1 : 0;
    return __builtin_amdgcn_readfirstlane(q);  // callers divide wave-uniform values: keep the result scalar
}

// 16-byte LDS read into the register that `dst` already occupies (a read-write argument keeps the register).
// The compiler does not see an LDS read here: the caller waits (s_waitcnt lgkmcnt) before using dst.
template <int OFF>
__device__ __forceinline__ void lds_read_b128_in_place(bf16x8_t& dst, uint32_t addr) {
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "+v"(dst) : "v"(addr), "n"(OFF));
}

template <int HD, int MODE>
__global__ __launch_bounds__(NTHREADS, 1) void flash_fwd_bf16_kernel(FlashBf16Params p) {
    constexpr int ROWB = HD * 2;             // bytes per row
    constexpr int SPR = HD / 8;              // 16-byte slots per row
    constexpr int RPI = 64 / SPR;            // rows covered by one wave load instruction (1 KB)
    constexpr int TILE_B = BC * ROWB;        // bytes of one K (or V) tile
    constexpr int NLD = BC / RPI / NWAVES;   // load instructions per wave, per matrix, per tile
    constexpr int KS = HD / 16;              // contraction steps of the score product
    constexpr int DT = HD / 32;              // 32-row tiles of O^T
    constexpr bool kCausal = (MODE == kMaskCausal) || (MODE == kMaskVarlenCausal);
    // Two barriers per step (see the header) at head dim 128.  At head dim 64 a matrix cluster is half as long as a
    // softmax cluster, the pipe is no longer what paces the waves, and the older scheme measures 2-3 % faster: a
    // barrier behind every cluster, waves 4-7 held one cluster behind waves 0-3 by one extra barrier at either end
    // of a job.
    constexpr bool kLockstep = (HD == 64);
    static_assert(NLD >= 1 && NLD <= NITEMS && BC % (RPI * NWAVES) == 0, "tile load split");

    // [K stage 0][K stage 1][V stage 0][V stage 1]: with this order every operand read of the steady state
    // is one per-lane base address plus an immediate offset below 64 KB
    __shared__ __attribute__((aligned(1024))) unsigned char lds[4 * TILE_B];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // in a scalar register: branches on it are scalar
    const int grp = wave >> 2;                                  // 0: waves 0-3, 1: waves 4-7 (one of each per SIMD)
    const int col = lane & 31, hh = lane >> 5;

    // slot swizzles (see the header): K rows are read 16 at a time at one slot (b128), V rows 4 at a
    // time over 4 adjacent slots (transposing b64 reads)
    auto swz_k = [](int r) { return HD == 128 ? (r & 15) : ((r >> 1) & 7); };
    auto swz_v = [](int r) { return HD == 128 ? 4 * (r & 3) : 4 * ((r >> 1) & 1); };
    auto swz_o = [](int r) { return r & (SPR - 1); };

    // ---- jobs.  A job is one (batch*head, 256-row query tile); every workgroup walks its own list.
    // Jobs are ranked from the longest (causal) rows down and dealt to the workers in boustrophedon
    // rows (a row runs left to right, the next right to left), so every worker gets the same number of
    // key tiles to within one job.  Nothing is relaunched between jobs: the next job's queries and first
    // key tile are requested before the current job's output is stored.
    const int N = p.seq;
    const int n_qtiles = (N + BR - 1) / BR;
    const int n_bh = p.batch * p.heads;
    const int n_jobs = n_qtiles * n_bh;
    const int W = gridDim.x, w = blockIdx.x;
    const float c = p.scale_log2e;
    // bytes between consecutive rows of a (batch, head) slab: ROWB when the slab is contiguous
    const uint32_t q_pitch_b = (uint32_t)p.lq.row_pitch * 2u, kv_pitch_b = (uint32_t)p.lkv.row_pitch * 2u;
    const uint32_t o_pitch_b = (uint32_t)p.lo.row_pitch * 2u;

    bool poison = false;  // a padding mask hiding the reference's whole first key tile: every row NaN
    // The keep vector as one bit per key, a word per 32-key item, built once per workgroup (masks of up to
    // kFlashBf16MaxPaddingKeys keys; the launcher refuses longer ones, which go to the tile kernel).  A word of ones
    // is the common case -- padding sits at the tail -- and costs the softmax cluster nothing.
    constexpr int kKeepWords = kFlashBf16MaxPaddingKeys / 32;
    __shared__ uint32_t keep_bits[MODE == kMaskPadding ? kKeepWords : 1];
    // (the launcher sends longer padding masks to the tile kernel, so the bits are always in LDS here)
    constexpr bool keep_in_lds = (MODE == kMaskPadding);
    if (MODE == kMaskPadding) {
        int lim = p.ref_bc < N ? p.ref_bc : N;
        bool any = false;
        for (int j = lane; j < lim; j += kWave) any |= (p.keep[j] != 0);
        poison = !__any(any);
        if (keep_in_lds) {
            for (int chunk = wave; chunk * 64 < N; chunk += NWAVES) {
                const int j = chunk * 64 + lane;
                // keys past the end count as kept here: they are masked by the length test
                const unsigned long long bits = __ballot(j >= N || p.keep[j] != 0);
                if (lane == 0) {
                    keep_bits[2 * chunk] = (uint32_t)bits;
                    keep_bits[2 * chunk + 1] = (uint32_t)(bits >> 32);
                }
            }
            __syncthreads();
        }
    }

    // ---- per-lane constants of the tile loads: instruction n of this wave fills LDS block
    // wave + NWAVES*n (rows RPI*block ..), lane l fetching the slot that belongs at byte 16*l.  The
    // swizzle only looks at the low bits of the row, which do not depend on n.
    static_assert((NWAVES * RPI) % 16 == 0, "row swizzles must not depend on the load index");
    const int ld_row0 = wave * RPI + lane / SPR;
    const uint32_t ld_k0 = (uint32_t)(((lane % SPR) ^ swz_k(ld_row0)) * 16);  // byte offset inside a global row
    const uint32_t ld_v0 = (uint32_t)(((lane % SPR) ^ swz_v(ld_row0)) * 16);
    const uint32_t ld_off_k = (uint32_t)ld_row0 * kv_pitch_b + ld_k0, ld_off_v = (uint32_t)ld_row0 * kv_pitch_b + ld_v0;
    // ---- per-lane bases of the operand reads.  The swizzles only permute address bits that the operand
    // index also occupies, so operand ks (dt) of a lane sits at base ^ 32*ks (base ^ 64*dt): one register
    // per matrix, one XOR per read.  The stage bit is toggled into the bases once per step; item and
    // half-item offsets are immediates.
    static_assert(HD == 128 || HD == 64, "operand address algebra below");
    // K A-operand: row col of an item, slot (2ks + hh) ^ swz_k(col)
    uint32_t k_base = (uint32_t)(col * ROWB + ((hh ^ swz_k(col)) * 16));
    // V^T A-operand: lane j of a 16-group addresses row j/4 (+4hh), 4 columns; slot (4dt + low) ^ swz_v(row)
    uint32_t v_base;
    {
        const int j = lane & 15, g16 = (lane >> 4) & 1, row = (j >> 2) + 4 * hh;
        const int low = 2 * g16 + ((j & 3) >> 1);
        v_base = (uint32_t)(2 * TILE_B + row * ROWB + ((low ^ swz_v(row)) * 16) + 8 * (j & 1));
    }
    // (2ks + hh) ^ x == (hh ^ x) ^ 2ks and (4dt + low) ^ x == (low ^ x) ^ 4dt bit for bit
    auto v_addr = [&](int dt) { return lds + (v_base ^ (uint32_t)(64 * dt)); };

    // state of the current job
    int q0, qw, q_row, n_keys, n_steps;
    const unsigned char* __restrict__ Kg;
    const unsigned char* __restrict__ Vg;
    uint16_t* __restrict__ Og;
    bf16x8_t qreg[KS];  // Q as B operand, in registers for the whole job
    f32x16_t acc_o[DT];
    float m_run, l_run;
    float neg_mc;  // -m_run * c, or +inf while the row has no max yet
    // operands of the next matrix cluster, and the scores / probabilities that travel between clusters
    bf16x8_t a[KS];      // K(k)
    u32x4_t vreg[2][DT]; // V(k-1): [16-key half][32-row tile of O^T]
    bf16x8_t pB[2];      // P(k-1)
    f32x16_t s;          // S^T(k)

    // This wave issues NLD K loads and NLD V loads per tile; load_part issues the n-th pair, so that a
    // tile's requests can be spread over several clusters (eight waves asking for a whole tile at once
    // queue up behind the CU's one address unit, and a wave cannot issue anything else while it waits).
    // Rows past the last key are read from the last key instead; they are masked in the score tile, so
    // their probabilities are zero.
    const uint32_t lds_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) unsigned char*)lds;
    auto load_part = [&](int n, int kv0, int st) {
        const uint32_t kdst = lds_base + (uint32_t)(st * TILE_B + (wave + NWAVES * n) * 1024);
        // A tile that lies wholly inside the keys (every tile but a ragged last one) needs no per-lane arithmetic:
        // the rows of instruction n start at a wave-uniform offset, which goes into the scalar base, and the lane's
        // own offset is a constant of the kernel.
        if (__builtin_expect(kv0 + BC <= n_keys, 1)) {
            const size_t blk = (size_t)((uint32_t)(kv0 + NWAVES * RPI * n) * kv_pitch_b);
            load_to_lds(Kg + blk, ld_off_k, kdst);
            load_to_lds(Vg + blk, ld_off_v, kdst + 2 * TILE_B);
            return;
        }
        int r = kv0 + ld_row0 + NWAVES * RPI * n;
        asm volatile("" : "+v"(r));  // recompute per call: hoisted copies of these offsets only cost registers
        const bool past_end = r >= n_keys;
        r = min(r, n_keys - 1);
        const uint32_t row_off = (uint32_t)r * kv_pitch_b;  // seq * row pitch stays below 4 GiB (checked by the caller)
        load_to_lds(Kg, row_off + ld_k0, kdst);
        // V rows behind the last key are zeros: their weights are zero, and zero times a copy of a non-finite last
        // row would be NaN.  An ordinary LDS write (lgkmcnt), complete before the barrier that publishes the tile:
        // every cluster starts with lgkmcnt(0), and a job's first tile is published by __syncthreads.
        if (past_end) {
            *(u32x4_t*)(lds + (st * TILE_B + (wave + NWAVES * n) * 1024) + 2 * TILE_B + 16 * lane) = u32x4_t{0u, 0u, 0u, 0u};
        } else {
            load_to_lds(Vg, row_off + ld_v0, kdst + 2 * TILE_B);
        }
    };
    auto load_tile = [&](int kv0, int st) {
#pragma unroll
        for (int n = 0; n < NLD; n++) load_part(n, kv0, st);
    };
    // Job of round i for this worker, or -1, as rank * n_bh + bh (rank 0 = the longest causal rows).
    // Workgroups are dealt round-robin to the 8 XCDs, each with its own L2.  When the heads divide evenly,
    // XCD x owns the heads bh = x (mod 8) and deals ITS job list (head-major, long rows first) to its own
    // workers in boustrophedon rows: the workers of an XCD then sit on one or two heads at a time and
    // share their K/V through that L2, and every worker still gets a long job paired with a short one.
    const bool by_xcd = ((n_bh & 7) == 0) && ((W & 7) == 0);
    const bool small_ids = n_jobs < (1 << 22);  // quotients below come from div_small
    const float inv_qtiles = 1.0f / (float)n_qtiles, inv_bh = 1.0f / (float)n_bh;
    const float inv_heads = 1.0f / (float)p.heads, inv_group = 1.0f / (float)p.group;
    auto quot = [&](int n, int d, float inv) { return small_ids ? div_small(n, d, inv) : n / d; };
    auto job_of_round = [&](int i) {
        if (by_xcd) {
            const int C = W >> 3, x = w & 7, cw = w >> 3;
            const int q = i * C + ((i & 1) ? (C - 1 - cw) : cw);
            if (q >= n_qtiles * (n_bh >> 3)) return -1;
            const int head = quot(q, n_qtiles, inv_qtiles), rank = q - head * n_qtiles;
            return rank * n_bh + head * 8 + x;
        }
        int j = i * W + ((i & 1) ? (W - 1 - w) : w);
        return j < n_jobs ? j : -1;
    };
    // point the state at job j and request its queries and first key tile (into stage 0)
    auto begin_job = [&](int j) {
        const int rank = quot(j, n_bh, inv_bh), bh = j - rank * n_bh;
        const int qtile = n_qtiles - 1 - rank;  // rank 0 = the longest causal rows
        const int b = quot(bh, p.heads, inv_heads), h = bh - b * p.heads;
        const int kvh = quot(h, p.group, inv_group);
        q0 = qtile * BR;
        qw = q0 + wave * 32;
        q_row = qw + col;
        const uint16_t* Qg = p.q + (size_t)b * p.lq.batch_stride + (size_t)h * p.lq.head_stride;
        Kg = (const unsigned char*)(p.k + (size_t)b * p.lkv.batch_stride + (size_t)kvh * p.lkv.head_stride);
        Vg = (const unsigned char*)(p.v + (size_t)b * p.lkv.batch_stride + (size_t)kvh * p.lkv.head_stride);
        Og = p.out + (size_t)b * p.lo.batch_stride + (size_t)h * p.lo.head_stride;
        n_keys = N;  // keys that exist for this sequence
        if (MODE == kMaskVarlenCausal) n_keys = min(N, max(0, p.seq_lens[b]));
        int kv_end = n_keys;
        if (kCausal) kv_end = min(n_keys, q0 + BR);
        if (MODE == kMaskVarlenCausal && q0 >= n_keys) kv_end = 0;  // a tile of padded query rows
        n_steps = (kv_end + BC - 1) / BC;
        // The wave's 32 query rows are one contiguous block: fetched in whole rows (load n, lane l: row
        // RPI*n + l/SPR, slot l%SPR), which costs the address unit a quarter of what row-per-lane loads
        // would; settle_queries() turns the registers into the operand layout once they have landed.
        static_assert(32 / RPI == KS, "one raw query register per operand register");
        {
            int lane_q = lane;
            asm volatile("" : "+v"(lane_q));  // (addresses rebuilt per job: see the note at the output stage)
            const int r0 = lane_q / SPR, slot = lane_q % SPR;
            const unsigned char* qp = (const unsigned char*)Qg + (size_t)(qw + r0) * q_pitch_b + slot * 16;
#pragma unroll
            for (int n = 0; n < KS; n++) {
                u32x4_t z = {0u, 0u, 0u, 0u};
                if (qw + RPI * n + r0 < N) z = *(const u32x4_t*)(qp + (size_t)n * RPI * q_pitch_b);
                qreg[n] = __builtin_bit_cast(bf16x8_t, z);
            }
        }
        if (n_steps > 0) load_tile(0, 0);
    };
    // Raw query registers -> B operands, through the wave's own corner of LDS stage 1 (idle between jobs):
    // rows are written with the K tile's slot swizzle and read back like a K operand, (row col, slot 2ks+hh).
    auto settle_queries = [&]() {
        int lane_q = lane;
        asm volatile("" : "+v"(lane_q));
        const uint32_t qbuf = lds_base + (uint32_t)((grp ? 3 * TILE_B : TILE_B) + (wave & 3) * 32 * ROWB);
        const int r0 = lane_q / SPR, slot = lane_q % SPR;
#pragma unroll
        for (int n = 0; n < KS; n++) {
            const int r = RPI * n + r0;
            *(bf16x8_t __attribute__((address_space(3)))*)(uintptr_t)(qbuf + (uint32_t)(r * ROWB + ((slot ^ swz_k(r)) * 16))) =
                qreg[n];
        }
        const int col_q = lane_q & 31, hh_q = lane_q >> 5;
#pragma unroll
        for (int ks = 0; ks < KS; ks++)
            qreg[ks] = *(const bf16x8_t __attribute__((address_space(3)))*)(uintptr_t)(
                qbuf + (uint32_t)(col_q * ROWB + (((2 * ks + hh_q) ^ swz_k(col_q)) * 16)));
    };

    // ---- pieces of the clusters ------------------------------------------------------------------------
    // operand reads; `off` is an immediate byte offset (item, half item); `flip` = TILE_B reads the other stage
    // The K operand is refilled IN PLACE: the read is written in assembly with the operand register as a
    // read-write argument, so it lands in the register the matrix instruction before it has just read (left
    // to itself the register allocator keeps two sets of K operands and runs out of registers).  The
    // compiler does not see these as LDS reads, so the wait for them is written out (lds_operands_ready).
    auto k_read_one = [&](auto off_c, int flip, int ks) {
        constexpr int OFF = decltype(off_c)::value;
        const uint32_t addr = lds_base + (k_base ^ (uint32_t)(32 * ks + flip));
        lds_read_b128_in_place<OFF>(a[ks], addr);
    };
    auto lds_operands_ready = [&]() { __builtin_amdgcn_s_waitcnt(0xC07F); };  // lgkmcnt(0)
    auto v_read_one = [&](int off, int j) {  // operand of the j-th P.V matrix instruction
        const int u = j / DT, dt = j % DT;
        // contraction slots 0-3 of a lane: keys kv_lo..kv_lo+3; slots 4-7: kv_lo+8..kv_lo+11
        const unsigned char* ptr = v_addr(dt) + off + 16 * u * ROWB;
        u32x2_t lo = lds_read_tr16(ptr);
        u32x2_t hi = lds_read_tr16(ptr + 8 * ROWB);
        vreg[u][dt] = u32x4_t{lo[0], lo[1], hi[0], hi[1]};
    };
    auto mfma_qk = [&](int ks) {
        s = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[ks], qreg[ks], s, 0, 0, 0); };
    auto mfma_pv = [&](int j) {
        const int u = j / DT, dt = j % DT;
        acc_o[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, vreg[u][dt]), pB[u],
                                                            acc_o[dt], 0, 0, 0);
    };
    auto zero_s = [&]() {
#pragma unroll
        for (int i = 0; i < 16; i++) s[i] = 0.0f;
    };
    auto mask_item = [&](int kv_base) {
#pragma unroll
        for (int i = 0; i < 16; i++) {
            int kr = kv_base + 8 * (i >> 2) + 4 * hh + (i & 3);
            bool masked = kr >= n_keys;
            if (kCausal) masked |= kr > q_row;
            s[i] = masked ? neg_inf() : s[i];
        }
    };
    // the same for a padding mask held as bits: `word` covers keys kv_base .. kv_base + 31
    auto mask_item_bits = [&](int kv_base, uint32_t word) {
        const uint32_t mine = word >> (4 * hh);  // bit 8(i/4) + i%4 of `mine` is key 8(i/4) + 4hh + i%4
#pragma unroll
        for (int i = 0; i < 16; i++) {
            const int kr = kv_base + 8 * (i >> 2) + 4 * hh + (i & 3);
            const uint32_t kept = 0u - ((mine >> (8 * (i >> 2) + (i & 3))) & 1u);  // all ones or zero
            uint32_t x = (__float_as_uint(s[i]) & kept) | (0xff800000u & ~kept);
            if (kv_base + 31 >= n_keys) x = (kr >= n_keys) ? 0xff800000u : x;
            s[i] = __uint_as_float(x);
        }
    };
    // The softmax of one item.  Fast path: P = exp2(s*c - m*c) with the running max AS IT STANDS, rounded to
    // bf16 (the two B operands of the item), and the lane's share of the row sum.  No row max is taken: a stale
    // max only scales a row's P, O and l by one common factor, which is harmless until it overflows, and the
    // share of the row sum that falls out anyway bounds every P of the lane from above.  Only when some lane's
    // share is above kTrigSum -- or is NaN, or the row has no max yet (neg_mc = +inf makes the share inf or
    // NaN) -- does the wave take the slow path: the true item max, the rescale of O and l, and P again from
    // the scores, which are still in their registers.
    auto exp_with = [&](float nmc, float& part) {
        float part0 = 0.0f, part1 = 0.0f;
        // Issue order is fixed by hand, eight scores at a time: the exponent arguments, then the exponentials, then the
        // sums and conversions, so that no instruction reads the result of the one or two before it (a dependent
        // instruction waits out the producer's latency, and v_exp_f32's is long).  The empty assembly statements are
        // what holds the order: each takes the values of a stage as read-write arguments, so the stage before it
        // cannot sink below and the one after cannot rise.
        float t[8];
        uint32_t w[8];
        auto pin8 = [&]() {
            asm volatile("" : "+v"(t[0]), "+v"(t[1]), "+v"(t[2]), "+v"(t[3]), "+v"(t[4]), "+v"(t[5]), "+v"(t[6]), "+v"(t[7]));
        };
        auto args = [&](int u) {
#pragma unroll
            for (int i = 0; i < 8; i++) t[i] = __builtin_fmaf(s[8 * u + i], c, nmc);
            pin8();
        };
        auto exps = [&]() {
#pragma unroll
            for (int i = 0; i < 8; i++) t[i] = __builtin_amdgcn_exp2f(t[i]);
            pin8();
        };
        auto convert = [&](int u) {
#pragma unroll
            for (int e = 0; e < 4; e++) w[4 * u + e] = cvt_pk_bf16(t[2 * e], t[2 * e + 1]);
            asm volatile("" : "+v"(w[4 * u]), "+v"(w[4 * u + 1]), "+v"(w[4 * u + 2]), "+v"(w[4 * u + 3]));
        };
        // The lane's share of the row sum is added up with plain v_add_f32 in two chains.  (v_dot2c_f32_bf16 against
        // ones would sum the rounded values in half the instructions, but it runs on the matrix pipe: while the
        // SIMD's other wave is in its matrix cluster each one waits for a gap there, and eight of them cost
        // more than the sixteen additions.)
        auto sum8 = [&]() {
#pragma unroll
            for (int i = 0; i < 8; i += 2) {
                part0 += t[i];
                part1 += t[i + 1];
            }
        };
        args(0);
        exps();
        sum8();
        convert(0);
        asm volatile("" : "+v"(part0), "+v"(part1));
        args(1);
        exps();
        sum8();
        convert(1);
        pB[0] = __builtin_bit_cast(bf16x8_t, u32x4_t{w[0], w[1], w[2], w[3]});
        pB[1] = __builtin_bit_cast(bf16x8_t, u32x4_t{w[4], w[5], w[6], w[7]});
        part = part0 + part1;
    };
    auto softmax_item = [&]() {
        float part;
        exp_with(neg_mc, part);
        if (__builtin_expect(__any(!(part <= kTrigSum)), 0)) {
            const float m_item = max_with_other_half(max16(s));
            const float m_new = vmax(m_run, m_item);
            const float m_use = (m_new == neg_inf()) ? 0.0f : m_new;
            const float alpha = __builtin_amdgcn_exp2f((m_run - m_use) * c);  // m_run = -inf -> 0
            m_run = m_new;
            l_run *= alpha;
#pragma unroll
            for (int t = 0; t < DT; t++)
#pragma unroll
                for (int i = 0; i < 16; i++) acc_o[t][i] *= alpha;
            const float mc = m_use * c;
            // a row that has seen no key yet keeps taking this path (and gets P = 0 from it: exp2(-inf - 0))
            neg_mc = (m_new == neg_inf()) ? __uint_as_float(0x7f800000u) : -mc;
            exp_with(-mc, part);
        }
        l_run += part;
    };
    // a workgroup barrier that nothing may be scheduled across
    auto cluster_barrier = [&]() {
        __builtin_amdgcn_sched_barrier(0);
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_sched_barrier(0);
    };
    // The end of cluster C (after_c) or S of item i: nothing is scheduled across it.  Of the step's two workgroup
    // barriers the first publishes this wave's share of the next tile (vmcnt(0) before it).
    auto cluster_edge = [&](bool after_c, int i) {
        __builtin_amdgcn_sched_barrier(0);
        if (kLockstep) {
            if (after_c && i == 2) __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): this wave's share has landed
            __builtin_amdgcn_s_barrier();
        } else if (i >= 2 && (grp == 1) == after_c) {
            if (i == 2) __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
            __builtin_amdgcn_s_barrier();
        }
        __builtin_amdgcn_sched_barrier(0);
    };
    static_assert(KS == 2 * DT, "one P.V matrix instruction per score matrix instruction");

    // One step = one 128-key tile = four items, each a C cluster and an S cluster.  A wave runs every item of
    // a step it takes part in (an item hidden from all of its rows by the causal mask is scored, masked to
    // -inf and contributes exact zeros): the two waves of a SIMD then stay one cluster apart.  The one exception
    // is taken a whole step at a time, in the job loop: a last key tile that lies wholly past a wave's rows.
    // Barriers: waves 4-7 behind C of items 2 and 3, waves 0-3 behind S of the same items (see the header).
    auto run_item = [&](auto i_c, int kv0, int kv_next, int st, int mask_from) {
        constexpr int i = decltype(i_c)::value;
        constexpr int item_off = 32 * i * ROWB;
        // ---- C: the products, and right after each the read that refills its operand for the next C.
        // Score and P.V instructions alternate: a score instruction accumulates onto the one before it,
        // and back-to-back dependent matrix instructions would wait for each other.
        // the multiplying wave goes first: its next instruction frees the matrix pipe.  (Both groups at the same
        // priority: with waves 0-3 above waves 4-7 a launch took 1.5 % longer, with no priority at all 3.7 %.)
        __builtin_amdgcn_s_setprio(3);
        lds_operands_ready();
        __builtin_amdgcn_sched_barrier(0);  // no matrix instruction may be moved ahead of that wait
        zero_s();
#pragma unroll
        for (int ks = 0; ks < KS; ks++) {
            mfma_qk(ks);
            if (i + 1 < NITEMS) k_read_one(std::integral_constant<int, (i + 1 < NITEMS ? item_off + 32 * ROWB : 0)>{}, 0, ks);
            else k_read_one(std::integral_constant<int, 0>{}, TILE_B, ks);  // item 0 of the next tile, other stage
            mfma_pv(ks);
            v_read_one(item_off, ks);
            // keep this order: two matrix instructions, three reads, and so on (left alone the scheduler
            // bunches the reads, and the matrix pipe runs dry while a wave issues ten of them in a row)
            __builtin_amdgcn_sched_barrier(0);
        }
        // the next tile (or, with none left, this tile again: served from cache into the idle stage,
        // which keeps the cluster free of branches): requested with items 0 and 1, awaited at the first barrier
        if (NLD >= 2) {
            if (i < 2) {
#pragma unroll
                for (int n = 0; n < NLD / 2; n++) load_part(i * (NLD / 2) + n, kv_next, st ^ 1);
            }
        } else if (i == 0) {
            load_part(0, kv_next, st ^ 1);
        }
        if (i == NITEMS - 1) __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0): stage st may be refilled
        __builtin_amdgcn_s_setprio(0);
        cluster_edge(true, i);
        // ---- S
        if (MODE == kMaskPadding) {
            if (keep_in_lds) {
                const uint32_t word = __builtin_amdgcn_readfirstlane(keep_bits[(kv0 + 32 * i) >> 5]);
                if (word != 0xffffffffu || kv0 + 32 * i + 31 >= n_keys) mask_item_bits(kv0 + 32 * i, word);
            } else {
                mask_item(kv0 + 32 * i);
            }
        } else if (__builtin_expect(kv0 + 32 * i + 31 > mask_from, 0)) {
            mask_item(kv0 + 32 * i);
        }
        softmax_item();
        // P is only used by the next matrix cluster, and the compiler would sink the exponentials and
        // conversions that make it down to that use, past the barrier and in between the matrix
        // instructions; pinning the values here keeps the work in this cluster
        asm volatile("" : "+v"(pB[0]), "+v"(pB[1]), "+v"(l_run));
        cluster_edge(false, i);
    };
    auto run_step = [&](int kv0, int kv_next, int st, int mask_from) {
        static_assert(NITEMS == 4, "items per step");
        run_item(std::integral_constant<int, 0>{}, kv0, kv_next, st, mask_from);
        run_item(std::integral_constant<int, 1>{}, kv0, kv_next, st, mask_from);
        run_item(std::integral_constant<int, 2>{}, kv0, kv_next, st, mask_from);
        run_item(std::integral_constant<int, 3>{}, kv0, kv_next, st, mask_from);
    };

#pragma unroll
    for (int ks = 0; ks < KS; ks++) a[ks] = __builtin_bit_cast(bf16x8_t, u32x4_t{0u, 0u, 0u, 0u});
    int round = 0;
    int job = job_of_round(0);
    if (job >= 0) begin_job(job);
    while (job >= 0) {
#pragma unroll
        for (int t = 0; t < DT; t++)
#pragma unroll
            for (int i = 0; i < 16; i++) acc_o[t][i] = 0.0f;
        m_run = neg_inf();
        neg_mc = __uint_as_float(0x7f800000u);
        l_run = 0.0f;
        // the first C of a job has no previous item: it multiplies zeros into O
#pragma unroll
        for (int u = 0; u < 2; u++) {
            pB[u] = __builtin_bit_cast(bf16x8_t, u32x4_t{0u, 0u, 0u, 0u});
#pragma unroll
            for (int dt = 0; dt < DT; dt++) vreg[u][dt] = u32x4_t{0u, 0u, 0u, 0u};
        }
        // the queries and tile 0 have landed; the barrier also ends the previous job's use of LDS
        __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
        settle_queries();
        __syncthreads();

        // an item needs masking when its last key lies past the last existing key or past the wave's first row
        const int mask_from = kCausal ? min(n_keys - 1, qw) : n_keys - 1;
        if (kLockstep && grp == 1) cluster_barrier();  // the second group runs one cluster behind the first
        if (n_steps > 0) {
#pragma unroll
            for (int ks = 0; ks < KS; ks++) k_read_one(std::integral_constant<int, 0>{}, 0, ks);  // K(0)
        }
        if (kLockstep) cluster_barrier();
        __builtin_amdgcn_sched_barrier(0);
        // With a causal mask the job's last key tile starts past the last row of the waves that own the upper
        // half of the query tile: for them every score of that step would be masked.  Such a wave finishes its
        // last live item and then only meets that step's two barriers (no matrix, LDS or vector work: on a
        // part whose clock is set by power the idle wave is worth more than its cycles).
        const bool dead_last = kCausal && n_steps > 0 && (n_steps - 1) * BC > qw + 31;
        const int n_run = n_steps - (dead_last ? 1 : 0);
        for (int step = 0; step < n_run; step++) {
            const int kv0 = step * BC;
            run_step(kv0, step + 1 < n_steps ? kv0 + BC : kv0, step & 1, mask_from);
            k_base ^= (uint32_t)TILE_B;  // the other stage
            v_base ^= (uint32_t)TILE_B;
        }
        // the last item's P.V
        if (n_run > 0) {
#pragma unroll
            for (int j = 0; j < KS; j++) mfma_pv(j);
        }
        if (dead_last) {
#pragma unroll 1
            for (int cl = 0; cl < (kLockstep ? 2 * NITEMS : 2); cl++) cluster_barrier();
            k_base ^= (uint32_t)TILE_B;
            v_base ^= (uint32_t)TILE_B;
        }
        if (n_steps & 1) {  // back to stage 0 for the next job
            k_base ^= (uint32_t)TILE_B;
            v_base ^= (uint32_t)TILE_B;
        }
        cluster_barrier();  // every wave has read its last operands: LDS is free for the output and the next job
        if (kLockstep && grp == 0) cluster_barrier();  // (the first group waits for the second to finish)

        // ---- this job's output.  Stage 1 of LDS is free (the next job's first tile goes to stage 0): each
        // wave parks its 32 normalised rows there, swizzled, and streams them out as whole rows.
        const int qw_out = qw;
        uint16_t* __restrict__ og_out = Og;
        const bool padded_row = (MODE == kMaskVarlenCausal) && (q_row >= n_keys);
        job = job_of_round(++round);
        if (job >= 0) begin_job(job);  // its loads travel while the output is normalised and stored

        // acc_o[dt][i] = O^T[d = 32dt + 8(i/4) + 4hh + i%4][row col of the wave]
        float l = sum_with_other_half(l_run);
        bool good = (l > 0.0f) && (l < __uint_as_float(0x7f800000u)) && !poison;
        float inv_l = 1.0f / l;
        // waves 0-3 park in the K half of stage 1, waves 4-7 in its V half.  All addresses below are built
        // from a copy of the lane index the compiler cannot see through: computed once per kernel they would
        // sit in registers (or scratch) through the whole main loop.
        int lane_e = lane;
        asm volatile("" : "+v"(lane_e));
        const int col_e = lane_e & 31, hh_e = lane_e >> 5;
        const uint32_t obuf = lds_base + (uint32_t)((grp ? 3 * TILE_B : TILE_B) + (wave & 3) * 32 * ROWB);
        // row col_e, slot (4dt + j) ^ swz_o(col_e): the slot bits of the base are XORed with a constant
        const uint32_t park = obuf + (uint32_t)(col_e * ROWB + swz_o(col_e) * 16 + 8 * hh_e);
#pragma unroll
        for (int dt = 0; dt < DT; dt++)
#pragma unroll
            for (int j = 0; j < 4; j++) {
                float o[4];
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    float x = good ? acc_o[dt][4 * j + r] * inv_l : quiet_nan();
                    if (padded_row) x = p.zero_padded_rows ? 0.0f : quiet_nan();
                    o[r] = x;
                }
                u32x2_t wv = {cvt_pk_bf16(o[0], o[1]), cvt_pk_bf16(o[2], o[3])};
                *(u32x2_t __attribute__((address_space(3)))*)(uintptr_t)(park ^ (uint32_t)(16 * (4 * dt + j))) = wv;
            }
        // (the same wave wrote and now reads: no barrier needed, the LDS queue is in order)
        {
            const int r0 = lane_e / SPR, pos = lane_e % SPR;  // instruction n covers rows n*RPI + r0
            const uint32_t rd = obuf + (uint32_t)(r0 * ROWB + pos * 16);
            // global slot pos ^ swz_o(n*RPI + r0); r0 < RPI and RPI is a power of two, so the part of the
            // swizzle that depends on n is a plain XOR into the slot bits of the lane's byte offset
            const uint32_t slot_off = (uint32_t)((pos ^ swz_o(r0)) * 16);
            unsigned char* gp = (unsigned char*)og_out + (size_t)(qw_out + r0) * o_pitch_b;
#pragma unroll
            for (int n = 0; n < 32 / RPI; n++) {
                u32x4_t v = *(const u32x4_t __attribute__((address_space(3)))*)(uintptr_t)(rd + (uint32_t)(n * RPI * ROWB));
                if (qw_out + n * RPI + r0 < N)
                    *(u32x4_t*)(gp + (size_t)n * RPI * o_pitch_b + (slot_off ^ (uint32_t)(swz_o(n * RPI) * 16))) = v;
            }
        }
    }
}

template <int HD>
hipError_t launch_hd(hipStream_t stream, const FlashBf16Params& p, dim3 grid, dim3 block) {
    switch (p.mask) {
        case kMaskNone: hipLaunchKernelGGL((flash_fwd_bf16_kernel<HD, kMaskNone>), grid, block, 0, stream, p); break;
        case kMaskCausal: hipLaunchKernelGGL((flash_fwd_bf16_kernel<HD, kMaskCausal>), grid, block, 0, stream, p); break;
        case kMaskPadding: hipLaunchKernelGGL((flash_fwd_bf16_kernel<HD, kMaskPadding>), grid, block, 0, stream, p); break;
        case kMaskVarlenCausal:
            hipLaunchKernelGGL((flash_fwd_bf16_kernel<HD, kMaskVarlenCausal>), grid, block, 0, stream, p);
            break;
        default: return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

}  // namespace

hipError_t launch_flash_bf16(hipStream_t stream, const FlashBf16Params& p) {
    if (p.batch == 0 || p.heads == 0 || p.seq == 0) return hipSuccess;
    if (p.mask == kMaskPadding && p.seq > kFlashBf16MaxPaddingKeys) return hipErrorInvalidValue;
    int n_qtiles = (p.seq + BR - 1) / BR;
    size_t n_jobs = (size_t)n_qtiles * p.batch * p.heads;
    size_t workers = p.n_workers > 0 ? (size_t)p.n_workers : 256;
    dim3 grid((unsigned)(n_jobs < workers ? n_jobs : workers)), block(NTHREADS);
    switch (p.dim) {
        case 64: return launch_hd<64>(stream, p, grid, block);
        case 128: return launch_hd<128>(stream, p, grid, block);
        default: return hipErrorInvalidValue;
    }
}

}  // namespace rt
