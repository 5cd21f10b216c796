// bf16 flash-attention forward (prefill) for gfx950.  Device counterpart of
// flash_forward_masked (crates/rustorch-attention/src/cpu_forward.rs:193-425) for bf16
// tensors: bf16 in, f32 accumulation on the matrix cores, bf16 out rounded once.
//
// Workgroup = 8 wavefronts (two per SIMD) = 256 query rows of one (batch, head); each wave owns 32
// rows and the workgroup walks the keys 64 at a time through a double-buffered LDS tile.  A wave
// treats the tile as two 32-key items and pipelines them so that the matrix cores and the vector
// ALU work at the same time:
//
//   S0 = K0.Q^T | softmax(S0) with S1 = K1.Q^T in flight | softmax(S1) with O += V0^T.P0 in flight | O += V1^T.P1
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
// The running max is only raised (and O, l rescaled) when some row's item max exceeds it by more
// than 2^8 in the exp2 domain: P then stays below 2^8, harmless in f32/bf16, and the rescale of the
// 64 O registers leaves the steady-state loop.
#include <type_traits>

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

#ifndef RT_FA_WAVES
#define RT_FA_WAVES 8
#endif
#ifndef RT_FA_MIN_BLOCKS
#define RT_FA_MIN_BLOCKS 1
#endif
constexpr int NTHREADS = 64 * RT_FA_WAVES;
constexpr int BR = 32 * RT_FA_WAVES;  // query rows per workgroup
constexpr int BC = 64;                // key rows per step
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
__device__ __forceinline__ u32x2_t lds_read_tr16(const uint16_t* p) {
    s16x4_t v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4_t __attribute__((address_space(3)))*)(p));
    return __builtin_bit_cast(u32x2_t, v);
}

// max / sum of a value with the one held by lane l ^ 32, without going through LDS:
// v_permlane32_swap leaves (lower half, lower half) in one register and (upper, upper) in the other.
__device__ __forceinline__ float max_with_other_half(float x) {
    auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float sum_with_other_half(float x) {
    auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

__device__ __forceinline__ float max16(const f32x16_t& s) {
    float a = fmaxf(fmaxf(s[0], s[1]), fmaxf(s[2], s[3]));
    float b = fmaxf(fmaxf(s[4], s[5]), fmaxf(s[6], s[7]));
    float c = fmaxf(fmaxf(s[8], s[9]), fmaxf(s[10], s[11]));
    float d = fmaxf(fmaxf(s[12], s[13]), fmaxf(s[14], s[15]));
    return fmaxf(fmaxf(a, b), fmaxf(c, d));
}

template <int HD, int MODE>
__global__ __launch_bounds__(NTHREADS, RT_FA_MIN_BLOCKS) void flash_fwd_bf16_kernel(FlashBf16Params p) {
    constexpr int LDK = HD + 8;   // K row stride (bf16): +16 B, 16 rows x 16 B tile all 64 banks
    constexpr int LDV = HD + 32;  // V row stride: = 64 B (mod 256 B), 4 rows x 64 B tile all 64 banks
    constexpr int KS = HD / 16;   // contraction steps of the score product
    constexpr int DT = HD / 32;   // 32-row tiles of O^T
    constexpr int CH = HD / 8;    // 16-byte chunks per row
    constexpr int NCHUNK = BC * CH;  // 16-byte chunks in one K (or V) tile
    constexpr int PASSES = (NCHUNK + NTHREADS - 1) / NTHREADS;
    constexpr bool kCausal = (MODE == kMaskCausal) || (MODE == kMaskVarlenCausal);

    __shared__ __attribute__((aligned(16))) uint16_t Ks[2][BC * LDK];
    __shared__ __attribute__((aligned(16))) uint16_t Vs[2][BC * LDV];

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int col = lane & 31, hh = lane >> 5;
    RT_PHASE_DECL;

    // ---- jobs.  A job is one (batch*head, 256-row query tile); the grid is persistent (one
    // workgroup per CU) and every workgroup walks its own list.  Jobs are ranked from the longest
    // (causal) rows down and dealt to the workers in boustrophedon order (round i: job i*W + w, or
    // i*W + W-1-w when i is odd), so every worker gets the same number of key tiles to within one job,
    // starts on a long job and ends on a short one.  Nothing is relaunched between jobs: the next
    // job's queries and first key tile are requested before the current job's output is stored.
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

    // state of the current job
    int q0, qw, q_row, n_keys, n_steps;
    const uint16_t* __restrict__ Kg;
    const uint16_t* __restrict__ Vg;
    uint16_t* __restrict__ Og;
    bf16x8_t qreg[KS];  // Q as B operand, in registers for the whole job
    u32x4_t kreg[PASSES], vreg[PASSES];
    f32x16_t acc_o[DT];
    float m_run, l_run;

    // ---- global -> register prefetch of one K/V tile, then register -> LDS.  Rows past the last key
    // are read from the last key instead (no branch); they are masked in the score tile, so their
    // probabilities are zero.
    auto prefetch = [&](int kv0) {
#pragma unroll
        for (int i = 0; i < PASSES; i++) {
            const int idx = tid + i * NTHREADS;
            if (NCHUNK % NTHREADS == 0 || idx < NCHUNK) {
                int r = min(kv0 + idx / CH, n_keys - 1);
                kreg[i] = *(const u32x4_t*)(Kg + (size_t)r * HD + 8 * (idx % CH));
                vreg[i] = *(const u32x4_t*)(Vg + (size_t)r * HD + 8 * (idx % CH));
            }
        }
    };
    auto stage = [&](int buf) {
#pragma unroll
        for (int i = 0; i < PASSES; i++) {
            const int idx = tid + i * NTHREADS;
            if (NCHUNK % NTHREADS == 0 || idx < NCHUNK) {
                *(u32x4_t*)(&Ks[buf][(idx / CH) * LDK + 8 * (idx % CH)]) = kreg[i];
                *(u32x4_t*)(&Vs[buf][(idx / CH) * LDV + 8 * (idx % CH)]) = vreg[i];
            }
        }
    };
    // job index of round i for this worker, or -1
    auto job_of_round = [&](int i) {
        int j = i * W + ((i & 1) ? (W - 1 - w) : w);
        return j < n_jobs ? j : -1;
    };
    // point the state at job j and request its queries and first key tile
    auto begin_job = [&](int j) {
        const int rank = j / n_bh, bh = j - rank * n_bh;
        const int qtile = n_qtiles - 1 - rank;  // rank 0 = the longest causal rows
        const int b = bh / p.heads, h = bh - b * p.heads;
        const int kvh = h / p.group;
        q0 = qtile * BR;
        qw = q0 + wave * 32;
        q_row = qw + col;
        const uint16_t* Qg = p.q + ((size_t)b * p.heads + h) * (size_t)N * HD;
        Kg = p.k + ((size_t)b * p.kv_heads + kvh) * (size_t)N * HD;
        Vg = p.v + ((size_t)b * p.kv_heads + kvh) * (size_t)N * HD;
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
        if (n_steps > 0) prefetch(0);
    };

    // per-lane part of the transposing V read: lane -> (row within a group of 4, 4-column chunk)
    const int tr_off = ((lane & 15) >> 2) * LDV + 16 * ((lane >> 4) & 1) + 4 * (lane & 3) + 4 * hh * LDV;
    const int k_off = col * LDK + 8 * hh;

    // ---- pieces of the per-item pipeline -------------------------------------------------------------
    // scores of one 32-key item: 8 (HD=128) MFMAs accumulating over the head dim
    auto qk = [&](const uint16_t* Kb, int t, f32x16_t& s) {
        bf16x8_t a[KS];
#pragma unroll
        for (int ks = 0; ks < KS; ks++) a[ks] = *(const bf16x8_t*)(Kb + 32 * t * LDK + k_off + 16 * ks);
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
            float m_new = fmaxf(m_run, m_item);
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
    auto pv = [&](const uint16_t* Vb, int t, const bf16x8_t (&pB)[2]) {
#pragma unroll
        for (int u = 0; u < 2; u++) {
            // contraction slots 0-3 of this lane: keys kv_lo..kv_lo+3; slots 4-7: kv_lo+8..kv_lo+11
            const uint16_t* vp = Vb + (32 * t + 16 * u) * LDV + tr_off;
#pragma unroll
            for (int dt = 0; dt < DT; dt++) {
                u32x2_t lo = lds_read_tr16(vp + dt * 32);
                u32x2_t hi = lds_read_tr16(vp + dt * 32 + 8 * LDV);
                u32x4_t av = {lo[0], lo[1], hi[0], hi[1]};
                acc_o[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, av), pB[u],
                                                                    acc_o[dt], 0, 0, 0);
            }
        }
    };
    // one 64-key tile; NEED_MASK is a compile-time flag so the steady state carries no mask code
    auto tile = [&](const uint16_t* Kb, const uint16_t* Vb, int kv0, auto need_mask_tag) {
        constexpr bool NEED_MASK = decltype(need_mask_tag)::value;
        f32x16_t s0, s1;
        bf16x8_t p0[2], p1[2];
        RT_PHASE(1);
        qk(Kb, 0, s0);
        if (NEED_MASK) mask_item(kv0, s0);
        RT_PHASE(2);
        update_max(s0);
        RT_PHASE(3);
        qk(Kb, 1, s1);       // matrix cores: scores of item 1 ...
        exp_item(s0, p0);    // ... vector ALU: probabilities of item 0
        if (NEED_MASK) mask_item(kv0 + 32, s1);
        RT_PHASE(4);
        pv(Vb, 0, p0);       // matrix cores: item 0 into O (P0 is relative to the max BEFORE item 1 raises it,
        update_max(s1);      //   so it must be accumulated before a rescale) ... vector ALU: max of item 1
        RT_PHASE(5);
        exp_item(s1, p1);    //   and its probabilities
        RT_PHASE(6);
        pv(Vb, 1, p1);
        RT_PHASE(7);
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
        if (n_steps > 0) {
            stage(0);
            if (n_steps > 1) prefetch(BC);
        }
        // Drain every outstanding global load once per job, here: inside the loop the only loads in
        // flight are then the tile prefetches, and the first MFMA of a step (which reads the Q registers)
        // does not wait for the prefetch issued just before it.
        __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
        __syncthreads();

        for (int step = 0; step < n_steps; step++) {
            const int kv0 = step * BC;
            const int buf = step & 1;
            RT_PHASE(0);
            // tile step+1 goes into the other buffer (last read in step-1, before the barrier that ended it)
            if (step + 1 < n_steps) {
                stage(buf ^ 1);
                if (step + 2 < n_steps) prefetch(kv0 + 2 * BC);
            }
            if (!(kCausal && kv0 > qw + 31)) {  // wave-uniform: this wave's rows see something of the tile
                bool need_mask = (kv0 + BC > n_keys);
                if (kCausal) need_mask |= (kv0 + BC - 1 > qw);
                if (MODE == kMaskPadding) need_mask = true;
                if (need_mask)
                    tile(Ks[buf], Vs[buf], kv0, std::true_type{});
                else
                    tile(Ks[buf], Vs[buf], kv0, std::false_type{});
            }
            RT_PHASE(8);
            __syncthreads();  // tile `buf` is free again; tile buf^1 is complete
            RT_PHASE(9);
        }

        // ---- this job's output rows: remember where they go, then turn the loads over to the next job
        // so that its queries and first key tile travel while the output is normalised and stored
        uint16_t* __restrict__ out_row = Og + (size_t)q_row * HD;
        const bool row_ok = q_row < N;
        const bool padded_row = (MODE == kMaskVarlenCausal) && (q_row >= n_keys);
        job = job_of_round(++round);
        if (job >= 0) begin_job(job);

        // acc_o[dt][i] = O^T[d = 32dt + 8(i/4) + 4hh + i%4][q_row]
        float l = sum_with_other_half(l_run);
        bool good = (l > 0.0f) && (l < __uint_as_float(0x7f800000u)) && !poison;
        float inv_l = 1.0f / l;
        if (row_ok) {
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
                    *(u32x2_t*)(out_row + dt * 32 + 8 * j + 4 * hh) = wv;
                }
        }
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
