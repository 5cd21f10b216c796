// bf16 flash-attention forward (prefill) for gfx950.  Device counterpart of
// flash_forward_masked (crates/rustorch-attention/src/cpu_forward.rs:193-425) for bf16
// tensors: bf16 in, f32 accumulation on the matrix cores, bf16 out rounded once.
//
// Workgroup = 4 wavefronts = 128 query rows of one (batch, head); each wave owns 32 rows and
// the workgroup walks the keys 64 at a time through LDS.  Per wave and step:
//
//   S^T[kv, q]  = K[kv, :] . Q[q, :]      v_mfma_f32_32x32x16_bf16, A = K tile (LDS), B = Q (registers)
//   online softmax on S^T: lane l holds 32 scores of query row l % 32, so row max / row sum are
//                          in-lane plus one exchange with lane l ^ 32
//   O^T[d, q]  += V^T[d, kv] . P^T[kv, q]  A = V tile read transposed from LDS, B = P (registers)
//
// The C layout of the first product (lane: column q, rows kv = 8j + 4*(l/32) + r) is, read as 8
// consecutive registers, exactly a B operand of the second product under a fixed permutation of
// the 16 contraction slots; the V operand is fetched with the same permutation, so P is never
// written to LDS.
#include "rt_common.hpp"
#include "rt_kernels.hpp"

namespace rt {

namespace {

constexpr int BR = 128;  // query rows per workgroup
constexpr int BC = 64;   // key rows per step
constexpr int NTHREADS = 256;

template <int HD>
__global__ __launch_bounds__(NTHREADS, 2) void flash_fwd_bf16_kernel(FlashBf16Params p) {
    constexpr int LDK = HD + 8;   // K tile row stride (bf16): +16 B so 16 rows x 16 B cover all banks once
    constexpr int LDV = BC + 4;   // V^T tile row stride: 34 banks, 32 rows x 8 B cover all banks once
    constexpr int KS = HD / 16;   // contraction steps of the score product
    constexpr int DT = HD / 32;   // 32-row tiles of O^T
    constexpr int CH = HD / 8;    // 16-byte chunks per row
    constexpr int ROWS_PER_PASS = NTHREADS / CH;
    constexpr int PASSES = BC / ROWS_PER_PASS;

    __shared__ __attribute__((aligned(16))) uint16_t Ks[BC * LDK];
    __shared__ __attribute__((aligned(16))) uint16_t Vt[HD * LDV];

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int col = lane & 31, hh = lane >> 5;

    // ---- block -> (batch*head, query tile).  Workgroups are dealt round-robin to the 8 XCDs
    // (each with its own L2); giving XCD x the heads bh = x (mod 8) keeps one head's K/V in one L2.
    const int n_qtiles = (p.seq + BR - 1) / BR;
    const int n_bh = p.batch * p.heads;
    int bh, qt;
    {
        int id = blockIdx.x;
        if ((n_bh & 7) == 0) {
            int xcd = id & 7, slot = id >> 3;
            bh = (slot / n_qtiles) * 8 + xcd;
            qt = slot % n_qtiles;
        } else {
            bh = id / n_qtiles;
            qt = id % n_qtiles;
        }
    }
    const int qtile = n_qtiles - 1 - qt;  // the longest causal rows first
    const int b = bh / p.heads, h = bh % p.heads;
    const int kvh = h / p.group;
    const int N = p.seq;
    const int q0 = qtile * BR;
    const int qw = q0 + wave * 32;  // first query row of this wave
    const int q_row = qw + col;

    const uint16_t* __restrict__ Qg = p.q + ((size_t)b * p.heads + h) * (size_t)N * HD;
    const uint16_t* __restrict__ Kg = p.k + ((size_t)b * p.kv_heads + kvh) * (size_t)N * HD;
    const uint16_t* __restrict__ Vg = p.v + ((size_t)b * p.kv_heads + kvh) * (size_t)N * HD;
    uint16_t* __restrict__ Og = p.out + ((size_t)b * p.heads + h) * (size_t)N * HD;

    const bool causal = (p.mask == kMaskCausal) || (p.mask == kMaskVarlenCausal);
    int n_keys = N;  // keys that exist for this sequence
    if (p.mask == kMaskVarlenCausal) n_keys = min(N, max(0, p.seq_lens[b]));

    bool poison = false;  // see flash_f32.hip: a padding mask hiding the reference's whole first key tile
    if (p.mask == kMaskPadding) {
        int lim = p.ref_bc < N ? p.ref_bc : N;
        bool any = false;
        for (int j = lane; j < lim; j += kWave) any |= (p.keep[j] != 0);
        poison = !__any(any);
    }

    // ---- Q as B operand, in registers for the whole kernel
    bf16x8_t qreg[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ks++) {
        u32x4_t z = {0u, 0u, 0u, 0u};
        if (q_row < N) z = *(const u32x4_t*)(Qg + (size_t)q_row * HD + 16 * ks + 8 * hh);
        qreg[ks] = __builtin_bit_cast(bf16x8_t, z);
    }

    f32x16_t acc_o[DT];
#pragma unroll
    for (int t = 0; t < DT; t++)
#pragma unroll
        for (int i = 0; i < 16; i++) acc_o[t][i] = 0.0f;
    float m_run = neg_inf(), l_run = 0.0f;
    const float c = p.scale_log2e;

    int kv_end = n_keys;
    if (causal) kv_end = min(n_keys, q0 + BR);
    const int n_steps = (kv_end + BC - 1) / BC;

    // ---- global -> register prefetch of one K/V tile
    const int ld_c = tid % CH, ld_r = tid / CH;
    u32x4_t kreg[PASSES], vreg[PASSES];
    auto prefetch = [&](int kv0) {
#pragma unroll
        for (int i = 0; i < PASSES; i++) {
            int r = kv0 + ld_r + i * ROWS_PER_PASS;
            u32x4_t zk = {0u, 0u, 0u, 0u}, zv = {0u, 0u, 0u, 0u};
            if (r < n_keys) {
                zk = *(const u32x4_t*)(Kg + (size_t)r * HD + 8 * ld_c);
                zv = *(const u32x4_t*)(Vg + (size_t)r * HD + 8 * ld_c);
            }
            kreg[i] = zk;
            vreg[i] = zv;
        }
    };
    if (n_steps > 0) prefetch(0);

    for (int step = 0; step < n_steps; step++) {
        const int kv0 = step * BC;
        __syncthreads();  // everyone is done reading the previous tile
#pragma unroll
        for (int i = 0; i < PASSES; i++) {
            int r = ld_r + i * ROWS_PER_PASS;
            *(u32x4_t*)(Ks + r * LDK + 8 * ld_c) = kreg[i];
#pragma unroll
            for (int e = 0; e < 4; e++) {  // V goes in transposed: Vt[d][kv]
                uint32_t w = vreg[i][e];
                Vt[(8 * ld_c + 2 * e) * LDV + r] = (uint16_t)(w & 0xffffu);
                Vt[(8 * ld_c + 2 * e + 1) * LDV + r] = (uint16_t)(w >> 16);
            }
        }
        __syncthreads();
        if (step + 1 < n_steps) prefetch(kv0 + BC);

        if (causal && kv0 > qw + 31) continue;  // this wave's rows see nothing of the tile (wave-uniform)

        // ---- S^T = K . Q^T for the two 32-key halves of the tile
        f32x16_t s[2];
#pragma unroll
        for (int t = 0; t < 2; t++) {
#pragma unroll
            for (int i = 0; i < 16; i++) s[t][i] = 0.0f;
#pragma unroll
            for (int ks = 0; ks < KS; ks++) {
                bf16x8_t a = *(const bf16x8_t*)(Ks + (32 * t + col) * LDK + 16 * ks + 8 * hh);
                s[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, qreg[ks], s[t], 0, 0, 0);
            }
        }

        // ---- mask (only tiles that need it) and row max
        const bool need_mask = (kv0 + BC > n_keys) || (causal && kv0 + BC - 1 > qw) || (p.mask == kMaskPadding);
        float m_tile = neg_inf();
        if (need_mask) {
#pragma unroll
            for (int t = 0; t < 2; t++)
#pragma unroll
                for (int i = 0; i < 16; i++) {
                    int kr = kv0 + 32 * t + 8 * (i >> 2) + 4 * hh + (i & 3);
                    bool masked = kr >= n_keys;
                    if (causal) masked |= kr > q_row;
                    if (p.mask == kMaskPadding) masked |= (kr < N) && (p.keep[kr] == 0);
                    s[t][i] = masked ? neg_inf() : s[t][i];
                }
        }
#pragma unroll
        for (int t = 0; t < 2; t++)
#pragma unroll
            for (int i = 0; i < 16; i++) m_tile = fmaxf(m_tile, s[t][i]);
        m_tile = fmaxf(m_tile, other_half(m_tile));

        // ---- online softmax in the exp2 domain; branch-free (MFMA ignores the exec mask)
        float m_new = fmaxf(m_run, m_tile);
        float m_use = (m_new == neg_inf()) ? 0.0f : m_new;
        float alpha = __builtin_amdgcn_exp2f((m_run - m_use) * c);
        float mc = m_use * c;
        m_run = m_new;
        float tile_l = 0.0f;
#pragma unroll
        for (int t = 0; t < 2; t++)
#pragma unroll
            for (int i = 0; i < 16; i++) {
                float e = __builtin_amdgcn_exp2f(__builtin_fmaf(s[t][i], c, -mc));
                s[t][i] = e;
                tile_l += e;
            }
        l_run = l_run * alpha + tile_l;
#pragma unroll
        for (int t = 0; t < DT; t++)
#pragma unroll
            for (int i = 0; i < 16; i++) acc_o[t][i] *= alpha;

        // ---- O^T += V^T . P^T
#pragma unroll
        for (int t = 0; t < 2; t++)
#pragma unroll
            for (int u = 0; u < 2; u++) {
                u32x4_t pb;
#pragma unroll
                for (int e = 0; e < 4; e++) pb[e] = pack_bf16x2(s[t][8 * u + 2 * e], s[t][8 * u + 2 * e + 1]);
                bf16x8_t pB = __builtin_bit_cast(bf16x8_t, pb);
                const int kv_lo = 32 * t + 16 * u + 4 * hh;
#pragma unroll
                for (int dt = 0; dt < DT; dt++) {
                    const uint16_t* vrow = Vt + (dt * 32 + col) * LDV + kv_lo;
                    u32x2_t lo = *(const u32x2_t*)(vrow);
                    u32x2_t hi = *(const u32x2_t*)(vrow + 8);
                    u32x4_t av = {lo[0], lo[1], hi[0], hi[1]};
                    acc_o[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, av), pB,
                                                                        acc_o[dt], 0, 0, 0);
                }
            }
    }

    // ---- normalise and store.  acc_o[dt][i] = O^T[d = 32dt + 8(i/4) + 4hh + i%4][q_row]
    float l = l_run + other_half(l_run);
    bool good = (l > 0.0f) && (l < __uint_as_float(0x7f800000u)) && !poison;
    float inv_l = 1.0f / l;
    if (q_row < N) {
        const bool padded_row = (p.mask == kMaskVarlenCausal) && (q_row >= n_keys);
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
                u32x2_t w = {pack_bf16x2(o[0], o[1]), pack_bf16x2(o[2], o[3])};
                *(u32x2_t*)(Og + (size_t)q_row * HD + dt * 32 + 8 * j + 4 * hh) = w;
            }
    }
}

}  // namespace

hipError_t launch_flash_bf16(hipStream_t stream, const FlashBf16Params& p) {
    if (p.batch == 0 || p.heads == 0 || p.seq == 0) return hipSuccess;
    int n_qtiles = (p.seq + BR - 1) / BR;
    dim3 grid((unsigned)((size_t)n_qtiles * p.batch * p.heads)), block(NTHREADS);
    switch (p.dim) {
        case 64: hipLaunchKernelGGL(flash_fwd_bf16_kernel<64>, grid, block, 0, stream, p); break;
        case 128: hipLaunchKernelGGL(flash_fwd_bf16_kernel<128>, grid, block, 0, stream, p); break;
        default: return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

}  // namespace rt
