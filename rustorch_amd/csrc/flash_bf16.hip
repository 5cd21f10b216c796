// bf16 flash-attention forward (prefill) for gfx950.  Device counterpart of
// flash_forward_masked (crates/rustorch-attention/src/cpu_forward.rs:193-425) for bf16
// tensors: bf16 in, f32 accumulation on the matrix cores, bf16 out rounded once.
//
// Persistent grid, one workgroup of 8 wavefronts (two per SIMD) per CU.  A job is 256 query rows of
// one (batch, head): each wave owns 32 rows, and the workgroup walks the keys 128 at a time through a
// double-buffered LDS tile that the waves fill with direct global->LDS loads (no registers, no LDS
// store instructions).  A wave treats the tile as four 32-key items and pipelines them so that the
// matrix cores and the vector ALU work at the same time:
//
//   S(i+1) = K(i+1).Q^T  in flight while  P(i) = exp2(S(i) - m)      is computed, then
//   O     += V(i)^T.P(i) in flight while  m   = max(m, rowmax S(i+1)) is computed.
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
// LDS tiles are unpadded; bank conflicts are avoided by an XOR swizzle of the 16-byte slots of a row,
// applied on the global side of the load (lane l of a load instruction always lands at LDS byte 16*l
// of its 1 KB block, so it fetches the slot that belongs there).
//
// The running max is only raised (and O, l rescaled) when some row's item max exceeds it by more
// than 2^8 in the exp2 domain: P then stays below 2^8, harmless in f32/bf16, and the rescale of the
// 64 O registers leaves the steady-state loop.
#include "rt_common.hpp"
#include "rt_kernels.hpp"

// Phase marker for a timing harness that includes this file with its own definition; nothing here.
#ifndef RT_PHASE
#define RT_PHASE(id)
#define RT_PHASE_DECL
#define RT_PHASE_DUMP
#endif

namespace rt {

namespace {

constexpr int NWAVES = 8;
constexpr int NTHREADS = 64 * NWAVES;
constexpr int BR = 32 * NWAVES;  // query rows per job
constexpr int BC = 128;          // key rows per step (one barrier per step)
constexpr int NITEMS = BC / 32;  // 32-key items per step
constexpr float kLazyLog2 = 8.0f;

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
__device__ __forceinline__ float max16(const f32x16_t& s) {
    float a = vmax(vmax(s[0], s[1]), vmax(s[2], s[3]));
    float b = vmax(vmax(s[4], s[5]), vmax(s[6], s[7]));
    float c = vmax(vmax(s[8], s[9]), vmax(s[10], s[11]));
    float d = vmax(vmax(s[12], s[13]), vmax(s[14], s[15]));
    return vmax(vmax(a, b), vmax(c, d));
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
    static_assert(NLD >= 1 && NLD <= NITEMS && BC % (RPI * NWAVES) == 0, "tile load split");

    // [stage 0: K, V][stage 1: K, V]
    __shared__ __attribute__((aligned(1024))) unsigned char lds[4 * TILE_B];

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int col = lane & 31, hh = lane >> 5;
    RT_PHASE_DECL;

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
    const float lazy_raw = kLazyLog2 / c;  // the rescale threshold in raw-score units

    bool poison = false;  // a padding mask hiding the reference's whole first key tile: every row NaN
    if (MODE == kMaskPadding) {
        int lim = p.ref_bc < N ? p.ref_bc : N;
        bool any = false;
        for (int j = lane; j < lim; j += kWave) any |= (p.keep[j] != 0);
        poison = !__any(any);
    }

    // ---- per-lane constants of the tile loads: instruction n of this wave fills LDS block
    // wave + NWAVES*n (rows RPI*block ..), lane l fetching the slot that belongs at byte 16*l.  The
    // swizzle only looks at the low bits of the row, which do not depend on n.
    static_assert((NWAVES * RPI) % 16 == 0, "row swizzles must not depend on the load index");
    const int ld_row0 = wave * RPI + lane / SPR;
    const uint32_t ld_k0 = (uint32_t)(((lane % SPR) ^ swz_k(ld_row0)) * 16);  // byte offset inside a global row
    const uint32_t ld_v0 = (uint32_t)(((lane % SPR) ^ swz_v(ld_row0)) * 16);
    // ---- per-lane constants of the operand reads
    uint32_t koff[KS];  // K A-operand: row col of an item, slot (2ks + hh)
#pragma unroll
    for (int ks = 0; ks < KS; ks++) koff[ks] = (uint32_t)(col * ROWB + (((2 * ks + hh) ^ swz_k(col)) * 16));
    uint32_t voff[DT];  // V^T A-operand: lane j of a 16-group addresses row j/4 (+4hh), 4 columns
#pragma unroll
    for (int dt = 0; dt < DT; dt++) {
        const int j = lane & 15, grp = (lane >> 4) & 1, row = (j >> 2) + 4 * hh;
        const int slot = (4 * dt + 2 * grp + ((j & 3) >> 1)) ^ swz_v(row);
        voff[dt] = (uint32_t)(row * ROWB + slot * 16 + 8 * (j & 1));
    }

    // state of the current job
    int q0, qw, q_row, n_keys, n_steps;
    const unsigned char* __restrict__ Kg;
    const unsigned char* __restrict__ Vg;
    uint16_t* __restrict__ Og;
    bf16x8_t qreg[KS];  // Q as B operand, in registers for the whole job
    f32x16_t acc_o[DT];
    float m_run, l_run;

    // request key tile `kv0` into stage `st`.  Rows past the last key are read from the last key
    // instead; they are masked in the score tile, so their probabilities are zero.
    // This wave issues NLD K loads and NLD V loads per tile; load_part issues the n-th pair, so that a
    // tile's requests can be spread over the step before it (eight waves asking for a whole tile at once
    // queue up behind the CU's one address unit, and a wave cannot issue anything else while it waits).
    const uint32_t lds_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) unsigned char*)lds;
    auto load_part = [&](int n, int kv0, int st) {
        const uint32_t kdst = lds_base + (uint32_t)(st * 2 * TILE_B + (wave + NWAVES * n) * 1024);
        int r = kv0 + ld_row0 + NWAVES * RPI * n;
        asm volatile("" : "+v"(r));  // recompute per call: hoisted copies of these offsets only cost registers
        r = min(r, n_keys - 1);
        const uint32_t row_off = (uint32_t)r * ROWB;  // a (b, h) slab is below 4 GiB: seq * dim * 2 < 2^32
        load_to_lds(Kg, row_off + ld_k0, kdst);
        load_to_lds(Vg, row_off + ld_v0, kdst + TILE_B);
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
    auto job_of_round = [&](int i) {
        if (by_xcd) {
            const int C = W >> 3, x = w & 7, cw = w >> 3;
            const int q = i * C + ((i & 1) ? (C - 1 - cw) : cw);
            if (q >= n_qtiles * (n_bh >> 3)) return -1;
            const int head = q / n_qtiles, rank = q - head * n_qtiles;
            return rank * n_bh + head * 8 + x;
        }
        int j = i * W + ((i & 1) ? (W - 1 - w) : w);
        return j < n_jobs ? j : -1;
    };
    // point the state at job j and request its queries and first key tile (into stage 0)
    auto begin_job = [&](int j) {
        const int rank = j / n_bh, bh = j - rank * n_bh;
        const int qtile = n_qtiles - 1 - rank;  // rank 0 = the longest causal rows
        const int b = bh / p.heads, h = bh - b * p.heads;
        const int kvh = h / p.group;
        q0 = qtile * BR;
        qw = q0 + wave * 32;
        q_row = qw + col;
        const uint16_t* Qg = p.q + ((size_t)b * p.heads + h) * (size_t)N * HD;
        Kg = (const unsigned char*)(p.k + ((size_t)b * p.kv_heads + kvh) * (size_t)N * HD);
        Vg = (const unsigned char*)(p.v + ((size_t)b * p.kv_heads + kvh) * (size_t)N * HD);
        Og = p.out + ((size_t)b * p.heads + h) * (size_t)N * HD;
        n_keys = N;  // keys that exist for this sequence
        if (MODE == kMaskVarlenCausal) n_keys = min(N, max(0, p.seq_lens[b]));
        int kv_end = n_keys;
        if (kCausal) kv_end = min(n_keys, q0 + BR);
        if (MODE == kMaskVarlenCausal && q0 >= n_keys) kv_end = 0;  // a tile of padded query rows
        n_steps = (kv_end + BC - 1) / BC;
#pragma unroll
        for (int ks = 0; ks < KS; ks++) {
            u32x4_t z = {0u, 0u, 0u, 0u};
            if (q_row < N) z = *(const u32x4_t*)(Qg + (size_t)q_row * HD + 16 * ks + 8 * hh);
            qreg[ks] = __builtin_bit_cast(bf16x8_t, z);
        }
        if (n_steps > 0) load_tile(0, 0);
    };

    // ---- pieces of the per-item pipeline -------------------------------------------------------------
    // scores of one 32-key item: KS MFMAs accumulating over the head dim
    auto qk = [&](const unsigned char* Kb, int t, f32x16_t& s) {
        bf16x8_t a[KS];
#pragma unroll
        for (int ks = 0; ks < KS; ks++) a[ks] = *(const bf16x8_t*)(Kb + 32 * t * ROWB + koff[ks]);
#pragma unroll
        for (int i = 0; i < 16; i++) s[i] = 0.0f;
#pragma unroll
        for (int ks = 0; ks < KS; ks++) s = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[ks], qreg[ks], s, 0, 0, 0);
    };
    auto mask_item = [&](int kv_base, f32x16_t& s) {
#pragma unroll
        for (int i = 0; i < 16; i++) {
            int kr = kv_base + 8 * (i >> 2) + 4 * hh + (i & 3);
            bool masked = kr >= n_keys;
            if (kCausal) masked |= kr > q_row;
            if (MODE == kMaskPadding) masked |= (kr < N) && (p.keep[kr] == 0);
            s[i] = masked ? neg_inf() : s[i];
        }
    };
    // raise the running max when it pays (wave-uniform branch; no MFMA inside)
    auto update_max = [&](const f32x16_t& s) {
        float m_item = max_with_other_half(max16(s));
        if (__any(m_item > m_run + lazy_raw)) {
            float m_new = vmax(m_run, m_item);
            float m_use = (m_new == neg_inf()) ? 0.0f : m_new;
            float alpha = __builtin_amdgcn_exp2f((m_run - m_use) * c);  // m_run = -inf -> 0
            m_run = m_new;
            l_run *= alpha;
#pragma unroll
            for (int t = 0; t < DT; t++)
#pragma unroll
                for (int i = 0; i < 16; i++) acc_o[t][i] *= alpha;
        }
    };
    // p = exp2(s*c - m*c) in place, row-sum share, and the two B operands of the item
    auto exp_item = [&](f32x16_t& s, bf16x8_t (&pB)[2]) {
        const float mc = ((m_run == neg_inf()) ? 0.0f : m_run) * c;
        float part[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int i = 0; i < 16; i++) {
            float e = __builtin_amdgcn_exp2f(__builtin_fmaf(s[i], c, -mc));
            s[i] = e;
            part[i & 3] += e;
        }
        l_run += (part[0] + part[1]) + (part[2] + part[3]);
#pragma unroll
        for (int u = 0; u < 2; u++) {
            u32x4_t pb;
#pragma unroll
            for (int e = 0; e < 4; e++) pb[e] = cvt_pk_bf16(s[8 * u + 2 * e], s[8 * u + 2 * e + 1]);
            pB[u] = __builtin_bit_cast(bf16x8_t, pb);
        }
    };
    // O^T += V^T . P^T for one item: 2 contraction steps of 16 keys x DT output tiles
    auto pv = [&](const unsigned char* Vb, int t, const bf16x8_t (&pB)[2]) {
#pragma unroll
        for (int u = 0; u < 2; u++) {
            // contraction slots 0-3 of this lane: keys kv_lo..kv_lo+3; slots 4-7: kv_lo+8..kv_lo+11
            const unsigned char* vp = Vb + (32 * t + 16 * u) * ROWB;
#pragma unroll
            for (int dt = 0; dt < DT; dt++) {
                u32x2_t lo = lds_read_tr16(vp + voff[dt]);
                u32x2_t hi = lds_read_tr16(vp + voff[dt] + 8 * ROWB);
                u32x4_t av = {lo[0], lo[1], hi[0], hi[1]};
                acc_o[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, av), pB[u],
                                                                    acc_o[dt], 0, 0, 0);
            }
        }
    };
    // One 128-key tile = up to four 32-key items.
    // Fast path: all four items visible and unmasked.  Straight-line code, so that each product sits in
    // the same scheduling region as the vector work it is meant to hide (an MFMA only overlaps with the
    // vector instructions issued right behind it; a branch between them would serialise the two).
    auto tile_full = [&](const unsigned char* Kb, const unsigned char* Vb, int kv_next, int st_next) {
        f32x16_t s_a, s_b;
        bf16x8_t pB[2];
        RT_PHASE(1);
        load_part(0, kv_next, st_next);
        qk(Kb, 0, s_a);
        update_max(s_a);
        RT_PHASE(2);
        if (NLD > 1) load_part(1 % NLD, kv_next, st_next);
        qk(Kb, 1, s_b);  exp_item(s_a, pB);      // scores of item 1 | probabilities of item 0
        pv(Vb, 0, pB);   update_max(s_b);        // item 0 into O    | max of item 1 (P(i) is relative to the max
        if (NLD > 2) load_part(2 % NLD, kv_next, st_next);
        qk(Kb, 2, s_a);  exp_item(s_b, pB);      //                  |   BEFORE item i+1 raises it: accumulate first)
        pv(Vb, 1, pB);   update_max(s_a);
        if (NLD > 3) load_part(3 % NLD, kv_next, st_next);
        qk(Kb, 3, s_b);  exp_item(s_a, pB);
        pv(Vb, 2, pB);   update_max(s_b);
        exp_item(s_b, pB);
        pv(Vb, 3, pB);
        RT_PHASE(3);
    };
    // General path: n_act items are visible to this wave (a causal mask hides the rest); only the last
    // visible one can need masking (diagonal or ragged end), unless the mask is a keep vector.
    auto tile_part = [&](const unsigned char* Kb, const unsigned char* Vb, int kv0, int n_act, bool mask_last) {
        f32x16_t s_a, s_b;
        bf16x8_t pB[2];
        qk(Kb, 0, s_a);
        if (MODE == kMaskPadding || (mask_last && n_act == 1)) mask_item(kv0, s_a);
        update_max(s_a);
#pragma unroll
        for (int i = 0; i < NITEMS; i++) {
            f32x16_t& s_cur = (i & 1) ? s_b : s_a;
            f32x16_t& s_nxt = (i & 1) ? s_a : s_b;
            const bool more = i + 1 < n_act;  // wave-uniform
            if (more) qk(Kb, i + 1, s_nxt);
            exp_item(s_cur, pB);
            if (more && (MODE == kMaskPadding || (mask_last && i + 2 == n_act)))
                mask_item(kv0 + 32 * (i + 1), s_nxt);
            pv(Vb, i, pB);
            if (!more) break;
            update_max(s_nxt);
        }
    };

    int round = 0;
    int job = job_of_round(0);
    if (job >= 0) begin_job(job);
    while (job >= 0) {
#pragma unroll
        for (int t = 0; t < DT; t++)
#pragma unroll
            for (int i = 0; i < 16; i++) acc_o[t][i] = 0.0f;
        m_run = neg_inf();
        l_run = 0.0f;
        // the queries and tile 0 have landed; the barrier also ends the previous job's use of LDS
        __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
        __syncthreads();
        RT_PHASE(10);

        for (int step = 0; step < n_steps; step++) {
            const int kv0 = step * BC;
            const int st = step & 1;
            RT_PHASE(0);
            // tile step+1 goes into the other stage (last read in step-1, before the barrier that ended it)
            const bool more = step + 1 < n_steps;
            int n_act = NITEMS;
            if (kCausal) n_act = (kv0 > qw + 31) ? 0 : min(NITEMS, (qw + 31 - kv0) / 32 + 1);  // items starting at or before the wave's last row
            n_act = min(n_act, (n_keys - kv0 + 31) / 32);                // items that hold an existing key
            if (n_act > 0) {
                const int last_kv = kv0 + 32 * n_act - 1;  // last key of the last visible item
                bool mask_last = last_kv >= n_keys;
                if (kCausal) mask_last |= last_kv > qw;
                if (MODE != kMaskPadding && n_act == NITEMS && !mask_last) {
                    // the fast path requests the next tile itself, a quarter per item; with no next tile it
                    // asks for its own tile again (served from cache into the idle stage) to stay branch-free
                    tile_full(lds + st * 2 * TILE_B, lds + st * 2 * TILE_B + TILE_B, more ? kv0 + BC : kv0, st ^ 1);
                } else {
                    if (more) load_tile(kv0 + BC, st ^ 1);
                    tile_part(lds + st * 2 * TILE_B, lds + st * 2 * TILE_B + TILE_B, kv0, n_act, mask_last);
                }
            } else if (more) {
                load_tile(kv0 + BC, st ^ 1);
            }
            RT_PHASE(8);
            __builtin_amdgcn_s_waitcnt(0x0F70);  // this wave's share of tile step+1 has landed
            __syncthreads();                      // stage `st` is free again; stage st^1 is complete
            RT_PHASE(9);
        }

        // ---- this job's output.  Stage 1 of LDS is free (the next job's first tile goes to stage 0): each
        // wave parks its 32 normalised rows there, swizzled, and streams them out as whole rows.
        const int qw_out = qw;
        uint16_t* __restrict__ og_out = Og;
        const bool padded_row = (MODE == kMaskVarlenCausal) && (q_row >= n_keys);
        job = job_of_round(++round);
        RT_PHASE(4);
        if (job >= 0) begin_job(job);  // its loads travel while the output is normalised and stored
        RT_PHASE(5);

        // acc_o[dt][i] = O^T[d = 32dt + 8(i/4) + 4hh + i%4][row col of the wave]
        float l = sum_with_other_half(l_run);
        bool good = (l > 0.0f) && (l < __uint_as_float(0x7f800000u)) && !poison;
        float inv_l = 1.0f / l;
        unsigned char* obuf = lds + 2 * TILE_B + wave * 32 * ROWB;
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
                *(u32x2_t*)(obuf + col * ROWB + (((4 * dt + j) ^ swz_o(col)) * 16) + 8 * hh) = wv;
            }
        RT_PHASE(6);
        // (the same wave wrote and now reads: no barrier needed, the LDS queue is in order)
#pragma unroll
        for (int n = 0; n < 32 / RPI; n++) {
            const int r = n * RPI + lane / SPR, pos = lane % SPR;
            u32x4_t v = *(const u32x4_t*)(obuf + r * ROWB + pos * 16);
            if (qw_out + r < N)
                *(u32x4_t*)((unsigned char*)og_out + (size_t)(qw_out + r) * ROWB + ((pos ^ swz_o(r)) * 16)) = v;
        }
        RT_PHASE(11);
    }
    RT_PHASE_DUMP;
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
