// f32 flash-attention forward for gfx950: the device counterpart of
// flash_forward_masked (crates/rustorch-attention/src/cpu_forward.rs:193-425) and of the
// prefill branch of gqa_forward_f32 (crates/rustorch-nn/src/gqa.rs:151-177).
//
// One wavefront owns 32 query rows and walks the key/value rows 32 at a time.  Both
// products run on the f32 matrix cores (v_mfma_f32_32x32x2_f32, full f32 precision):
//
//   S^T[kv, q]  = sum_d K[kv, d] * Q[q, d]          (A = K tile, B = Q tile)
//   O^T[d, q]  += sum_kv V[kv, d] * P[q, kv]        (A = V tile, B = P from registers)
//
// Computing the transposed score tile leaves every lane holding 16 scores of ONE query row
// (q = lane % 32), so the row max / row sum of the online softmax are in-lane reductions plus
// one exchange with the other half of the wave, and the score registers are already in the
// B-operand layout the second product needs: P never leaves the register file.
//
// Semantics kept from the reference: scale applied to the finished dot product, mask -> -inf
// after scaling, row without a visible key -> NaN row, `out = O * (1/l)`.  Tiles a causal mask
// empties are skipped, not computed.
#include <type_traits>

#include "rt_common.hpp"
#include "rt_kernels.hpp"

namespace rt {

namespace {

constexpr int kRows = 32;  // query rows per workgroup (one wave) and key rows per step

template <int DT>  // DT = ceil(dim / 32); the head dim is zero-padded to DPAD = 32 * DT in LDS
__global__ __launch_bounds__(64) void flash_fwd_f32_kernel(FlashF32Params p) {
    constexpr int DPAD = 32 * DT;
    constexpr int LDQ = DPAD + 1;  // odd row stride: a column read (32 rows, fixed d) hits 32 banks
    __shared__ float Qs[kRows * LDQ];
    __shared__ float Ks[kRows * LDQ];
    __shared__ float Vs[kRows * DPAD];  // read along d: no padding needed

    const int lane = threadIdx.x;
    const int col = lane & 31;  // query row within the tile / MFMA column
    const int hh = lane >> 5;   // which half of the wave
    const int N = p.seq, D = p.dim;
    const int qtile = (int)gridDim.x - 1 - (int)blockIdx.x;  // longest causal rows first
    const int q0 = qtile * kRows;
    const int h = blockIdx.y, b = blockIdx.z;
    const int kvh = h / p.group;
    const float* __restrict__ Qg = p.q + (size_t)b * p.lq.batch_stride + (size_t)h * p.lq.head_stride;
    const float* __restrict__ Kg = p.k + (size_t)b * p.lkv.batch_stride + (size_t)kvh * p.lkv.head_stride;
    const float* __restrict__ Vg = p.v + (size_t)b * p.lkv.batch_stride + (size_t)kvh * p.lkv.head_stride;
    float* __restrict__ Og = p.out + (size_t)b * p.lo.batch_stride + (size_t)h * p.lo.head_stride;
    const size_t q_pitch = p.lq.row_pitch, kv_pitch = p.lkv.row_pitch, o_pitch = p.lo.row_pitch;

    // With a padding mask the reference's recurrence turns every row into NaN when its first
    // key tile [0, bc) holds no visible key (cpu_forward.rs:364-384); reproduce that outcome.
    bool poison = false;
    if (p.mask == kMaskPadding) {
        int lim = p.ref_bc < N ? p.ref_bc : N;
        bool any = false;
        for (int j = lane; j < lim; j += kWave) any |= (p.keep[j] != 0);
        poison = !__any(any);
    }

    // stage the Q tile (zero beyond seq and beyond dim)
    for (int idx = lane; idx < kRows * DPAD; idx += kWave) {
        int r = idx / DPAD, d = idx - r * DPAD;
        int qr = q0 + r;
        Qs[r * LDQ + d] = (qr < N && d < D) ? Qg[(size_t)qr * q_pitch + d] : 0.0f;
    }

    f32x16_t acc_o[DT];
#pragma unroll
    for (int t = 0; t < DT; t++)
#pragma unroll
        for (int i = 0; i < 16; i++) acc_o[t][i] = 0.0f;
    float m_run = neg_inf();
    float l_run = 0.0f;  // this lane's share of the row sum (its 16 keys per step)

    const int q_row = q0 + col;
    int kv_end = N;
    if (p.mask == kMaskCausal) kv_end = min(N, q0 + kRows);  // keys beyond the tile's last row are masked

    for (int kv0 = 0; kv0 < kv_end; kv0 += kRows) {
        __syncthreads();
        for (int idx = lane; idx < kRows * DPAD; idx += kWave) {
            int r = idx / DPAD, d = idx - r * DPAD;
            int kr = kv0 + r;
            bool ok = (kr < N && d < D);
            Ks[r * LDQ + d] = ok ? Kg[(size_t)kr * kv_pitch + d] : 0.0f;
            Vs[r * DPAD + d] = ok ? Vg[(size_t)kr * kv_pitch + d] : 0.0f;
        }
        __syncthreads();

        // S^T = K . Q^T
        f32x16_t s;
#pragma unroll
        for (int i = 0; i < 16; i++) s[i] = 0.0f;
#pragma unroll 8
        for (int ks = 0; ks < DPAD / 2; ks++) {
            float a = Ks[col * LDQ + 2 * ks + hh];
            float bq = Qs[col * LDQ + 2 * ks + hh];
            s = __builtin_amdgcn_mfma_f32_32x32x2f32(a, bq, s, 0, 0, 0);
        }
        // register i of the accumulator holds key row 8*(i/4) + 4*hh + (i%4), query row `col`
        float m_tile = neg_inf();
#pragma unroll
        for (int i = 0; i < 16; i++) {
            int kr = kv0 + 8 * (i >> 2) + 4 * hh + (i & 3);
            float x = s[i] * p.scale;
            bool masked = kr >= N;
            if (p.mask == kMaskCausal) masked |= kr > q_row;
            if (p.mask == kMaskPadding) masked |= (kr < N) && (p.keep[kr] == 0);
            x = masked ? neg_inf() : x;
            s[i] = x;
            m_tile = (x > m_tile) ? x : m_tile;  // NaN never wins, as in the reference's `if x > m`
        }
        {
            float o = other_half(m_tile);
            m_tile = (o > m_tile) ? o : m_tile;
        }
        float m_new = (m_tile > m_run) ? m_tile : m_run;
        // No branch here: MFMA ignores the exec mask, so every lane must reach the products with
        // well-defined operands.  While a row has seen no visible key, subtract 0 instead of -inf:
        // every exp() is then exp(-inf) = 0 and the state stays empty.
        float m_use = (m_new == neg_inf()) ? 0.0f : m_new;
        float alpha = (m_run == neg_inf()) ? 0.0f : expf(m_run - m_use);
        m_run = m_new;
        float tile_l = 0.0f;
#pragma unroll
        for (int i = 0; i < 16; i++) {
            float e = expf(s[i] - m_use);
            s[i] = e;
            tile_l += e;
        }
        l_run = l_run * alpha + tile_l;
#pragma unroll
        for (int t = 0; t < DT; t++)
#pragma unroll
            for (int i = 0; i < 16; i++) acc_o[t][i] *= alpha;

        // O^T += V^T . P^T, two keys per MFMA: the lower half of the wave feeds key 8j+r, the upper 8j+4+r
#pragma unroll
        for (int i = 0; i < 16; i++) {
            int kr = 8 * (i >> 2) + 4 * hh + (i & 3);
#pragma unroll
            for (int t = 0; t < DT; t++) {
                float a = Vs[kr * DPAD + t * 32 + col];
                acc_o[t] = __builtin_amdgcn_mfma_f32_32x32x2f32(a, s[i], acc_o[t], 0, 0, 0);
            }
        }
    }

    float l = l_run + other_half(l_run);
    bool good = (l > 0.0f) && (fabsf(l) != __uint_as_float(0x7f800000u)) && (l == l) && !poison;
    float inv_l = 1.0f / l;
    if (p.lse && hh == 0 && q_row < N) p.lse[((size_t)b * p.heads + h) * (size_t)N + q_row] = m_run + logf(l);
    if (q_row < N) {
#pragma unroll
        for (int t = 0; t < DT; t++)
#pragma unroll
            for (int i = 0; i < 16; i++) {
                int d = t * 32 + 8 * (i >> 2) + 4 * hh + (i & 3);
                if (d < D) Og[(size_t)q_row * o_pitch + d] = good ? acc_o[t][i] * inv_l : quiet_nan();
            }
    }
}


// ---- head dims that are a multiple of 32, 16-byte aligned rows: the fast kernel ---------------------------
//
// One workgroup of four waves owns 32 query rows; wave w walks the key tiles t = w, w+4, ... (32 keys each) on its
// own, with a private LDS tile and no workgroup barrier in the loop, and the four partial (O, m, l) states are
// merged through LDS at the end with the online-softmax monoid (online_softmax.rs:105-131 extended with O).
// Splitting the keys rather than the query rows over the waves shortens the longest chain of dependent steps
// four times, which is what a small problem (8 heads x 2048 rows) is bound by.  The next tile travels from
// global memory into registers (16-byte loads) while the current one is multiplied.
//
// The contraction index of the score product is walked in the order d = 8j + 4*half + i (i = 0..3) for both
// operands, so that a lane fetches its four K values of a chunk with one 16-byte LDS read and Q stays in
// registers for the whole job.
// kExactD: dim == 32 * DT, no column guards anywhere.  kMode: one instantiation per way of masking, so that the tile
// step of each holds only its own tests -- 0 none, 1 causal, 2 Mask::Padding (the only one that carries the keep
// bits in LDS and looks at p.keep), 3 none plus an additive score bias.
template <int DT, bool kExactD, int kMode>
__global__ __launch_bounds__(256, (DT <= 2 ? 2 : 1)) void flash_fwd_f32_splitk_kernel(FlashF32Params p) {
    constexpr bool kCausal = kMode == 1, kPad = kMode == 2, kBias = kMode == 3;
    constexpr int DPAD = 32 * DT;       // dim rounded up to a multiple of 32 (columns beyond dim are zeros in LDS)
    constexpr int LDK = DPAD + 4;       // row stride of the K tile: 16-byte reads of 16 rows tile all banks
    constexpr int CH = DPAD / 4;        // 16-byte chunks per row
    constexpr int NLD = 32 * CH / 64;   // 16-byte loads per lane, per matrix, per tile
    constexpr int KTILE = kRows * LDK, VTILE = kRows * DPAD;
    constexpr int NW = 4;
    __shared__ __attribute__((aligned(16))) float lds[NW * (KTILE + VTILE)];
    __shared__ float red_m[NW][kRows], red_l[NW][kRows];
    __shared__ float fin_inv[kRows];

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int col = lane & 31, hh = lane >> 5;
    const int Nq = p.seq, N = p.seq_kv ? p.seq_kv : p.seq;  // N: keys (== queries unless cross-attention)
    const int D = kExactD ? DPAD : p.dim;
    // Which (batch, head, query tile) this workgroup takes.  Workgroups are dealt round-robin to the 8 XCDs, each
    // with its own L2: when the heads divide evenly, XCD x takes the heads bh = x (mod 8) and walks them one after
    // the other, longest causal rows first, so that a head's K and V are fetched into one L2 only.  When the whole
    // grid is resident at once (p.zigzag) the second half of an XCD's list runs shortest-first, so that the two
    // workgroups that end up sharing a CU (list positions r and r + half) are a long one and a short one.
    const int nq = (int)gridDim.x, n_bh = (int)(gridDim.y * gridDim.z);
    int h = blockIdx.y, b = blockIdx.z;
    int qtile = nq - 1 - (int)blockIdx.x;
    if ((n_bh & 7) == 0) {
        const int lin = (int)blockIdx.x + nq * ((int)blockIdx.y + (int)gridDim.y * (int)blockIdx.z);
        const int xcd = lin & 7, r = lin >> 3, half = (nq * (n_bh >> 3)) >> 1;
        int bh = (r / nq) * 8 + xcd;
        qtile = nq - 1 - r % nq;
        if (p.zigzag && r >= half && (half % nq == 0 || nq == 2 * half)) qtile = (r - half) % nq;
        h = bh % (int)gridDim.y;
        b = bh / (int)gridDim.y;
    } else if (p.zigzag && ((h + b * (int)gridDim.y) * 2 >= n_bh)) {
        qtile = (int)blockIdx.x;
    }
    const int q0 = qtile * kRows;
    const int kvh = h / p.group;
    const float* __restrict__ Qg = p.q + (size_t)b * p.lq.batch_stride + (size_t)h * p.lq.head_stride;
    const float* __restrict__ Kg = p.k + (size_t)b * p.lkv.batch_stride + (size_t)kvh * p.lkv.head_stride;
    const float* __restrict__ Vg = p.v + (size_t)b * p.lkv.batch_stride + (size_t)kvh * p.lkv.head_stride;
    float* __restrict__ Og = p.out + (size_t)b * p.lo.batch_stride + (size_t)h * p.lo.head_stride;
    const size_t q_pitch = p.lq.row_pitch, kv_pitch = p.lkv.row_pitch, o_pitch = p.lo.row_pitch;
    float* Kw = lds + wave * (KTILE + VTILE);
    float* Vw = Kw + KTILE;

    // leading-masked-tile rule of the reference's recurrence (cpu_forward.rs:364-384), as in the kernel above
    bool poison = false;
    // The keep vector as one bit per key in LDS (up to 32 * kKeepWords keys; longer ones are read byte by byte in the
    // loop): a tile step then reads one word, and a tile without a hidden key is not masked at all.
    constexpr int kKeepWords = 1024;
    __shared__ uint32_t keep_bits[kPad ? kKeepWords : 2];
    const bool keep_in_lds = kPad && N <= 32 * kKeepWords;
    if constexpr (kPad) {
        int lim = p.ref_bc < N ? p.ref_bc : N;
        bool any = false;
        for (int j = lane; j < lim; j += kWave) any |= (p.keep[j] != 0);
        poison = !__any(any);
        if (keep_in_lds) {
            for (int base = wave * kWave; base < N; base += NW * kWave) {
                const int key = base + lane;
                const unsigned long long bal = __ballot(key < N && p.keep[key] != 0);
                if (lane == 0) {
                    keep_bits[base >> 5] = (uint32_t)bal;
                    keep_bits[(base >> 5) + 1] = (uint32_t)(bal >> 32);
                }
            }
            __syncthreads();
        }
    }

    // Q as B operand, in registers: qreg[4j + i] = Q[q0 + col][8j + 4hh + i]
    const int q_row = q0 + col;
    float qreg[DPAD / 2];
#pragma unroll
    for (int j = 0; j < DPAD / 8; j++) {
        f32x4_t z = {0.0f, 0.0f, 0.0f, 0.0f};
        if (q_row < Nq && 8 * j + 4 * hh < D) z = *(const f32x4_t*)(Qg + (size_t)q_row * q_pitch + 8 * j + 4 * hh);
#pragma unroll
        for (int i = 0; i < 4; i++) qreg[4 * j + i] = z[i];
    }

    f32x16_t acc_o[DT];
#pragma unroll
    for (int t = 0; t < DT; t++)
#pragma unroll
        for (int i = 0; i < 16; i++) acc_o[t][i] = 0.0f;
    float m_run = neg_inf();
    float l_run = 0.0f;  // this lane's share of the row sum

    int kv_end = N;
    if (kCausal) kv_end = min(N, q0 + kRows);
    const int n_tiles = (kv_end + kRows - 1) / kRows;
    // additive bias row of this lane's query (MultiHeadAttention's attn_mask, added to the scaled scores)
    const float* __restrict__ bias_row = nullptr;
    if (kBias && q_row < Nq)
        bias_row = p.bias + ((size_t)b * p.heads + h) * (size_t)p.bias_bh_stride + (size_t)q_row * (size_t)N;
    const bool bias_vec = ((N & 3) == 0) && ((((uintptr_t)p.bias) & 15) == 0) && ((p.bias_bh_stride & 3) == 0);

    // lane's chunks of a tile: load n covers row (64n + lane) / CH, chunk (64n + lane) % CH.  When CH divides 64
    // that is row n * (64/CH) + lane / CH, chunk lane % CH: one per-lane offset, everything else is uniform.
    constexpr bool kEvenRows = (64 % CH == 0);
    constexpr int RPL = kEvenRows ? 64 / CH : 0;  // rows per load instruction
    const int ld_r = lane / CH, ld_c = lane % CH;
    const bool ld_col_ok = kExactD || 4 * ld_c < D;  // this lane's 16-byte column exists
    const uint32_t ld_off = (uint32_t)ld_r * (uint32_t)kv_pitch * 4u + (uint32_t)ld_c * 16u;  // bytes; a few rows: fits
    f32x4_t kreg[NLD], vreg[NLD];
    auto issue_loads = [&](int tile) {
        if constexpr (kEvenRows) {
            if (tile * kRows + kRows <= N) {  // whole tile present (wave-uniform): no per-load bounds test
                if (!ld_col_ok) {
#pragma unroll
                    for (int n = 0; n < NLD; n++) kreg[n] = vreg[n] = f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};
                    return;
                }
                const char* kb = (const char*)Kg + (size_t)tile * kRows * kv_pitch * sizeof(float) + ld_off;
                const char* vb = (const char*)Vg + (size_t)tile * kRows * kv_pitch * sizeof(float) + ld_off;
#pragma unroll
                for (int n = 0; n < NLD; n++) {
                    const size_t step = (size_t)(RPL * n) * kv_pitch * sizeof(float);  // uniform
                    kreg[n] = *(const f32x4_t*)(kb + step);
                    vreg[n] = *(const f32x4_t*)(vb + step);
                }
                return;
            }
        }
#pragma unroll
        for (int n = 0; n < NLD; n++) {
            f32x4_t zk = {0.0f, 0.0f, 0.0f, 0.0f}, zv = zk;
            if constexpr (kEvenRows) {
                const int row0 = tile * kRows + RPL * n;  // uniform
                const size_t base = (size_t)row0 * kv_pitch * sizeof(float);
                if (row0 + ld_r < N && ld_col_ok) {  // rows past the end are zeros (and masked below)
                    zk = *(const f32x4_t*)((const char*)Kg + base + ld_off);
                    zv = *(const f32x4_t*)((const char*)Vg + base + ld_off);
                }
            } else {
                const int idx = 64 * n + lane, r = idx / CH, c = idx % CH;
                const int kr = tile * kRows + r;
                if (kr < N && 4 * c < D) {
                    zk = *(const f32x4_t*)(Kg + (size_t)kr * kv_pitch + 4 * c);
                    zv = *(const f32x4_t*)(Vg + (size_t)kr * kv_pitch + 4 * c);
                }
            }
            kreg[n] = zk;
            vreg[n] = zv;
        }
    };
    if (wave < n_tiles) issue_loads(wave);

    for (int tile = wave; tile < n_tiles; tile += NW) {
        const int kv0 = tile * kRows;
        // registers -> this wave's LDS tile (its reads of the previous tile are behind it: same wave, in order)
#pragma unroll
        for (int n = 0; n < NLD; n++) {
            const int idx = 64 * n + lane, r = idx / CH, c = idx % CH;
            *(f32x4_t*)(Kw + r * LDK + 4 * c) = kreg[n];
            *(f32x4_t*)(Vw + r * DPAD + 4 * c) = vreg[n];
        }
        // this tile's bias values are requested ahead of the next tile's rows: a wait for them then leaves the
        // prefetch in flight (requests complete in order)
        f32x16_t bias;
#pragma unroll
        for (int i = 0; i < 16; i++) bias[i] = 0.0f;
        if (kBias && bias_row) {
#pragma unroll
            for (int g = 0; g < 4; g++) {
                const int kr0 = kv0 + 8 * g + 4 * hh;
                if (bias_vec && kr0 + 3 < N) {
                    const f32x4_t bv = *(const f32x4_t*)(bias_row + kr0);
#pragma unroll
                    for (int r = 0; r < 4; r++) bias[4 * g + r] = bv[r];
                } else {
#pragma unroll
                    for (int r = 0; r < 4; r++)
                        if (kr0 + r < N) bias[4 * g + r] = bias_row[kr0 + r];
                }
            }
        }
        if (tile + NW < n_tiles) issue_loads(tile + NW);

        // S^T = K . Q^T
        f32x16_t s;
#pragma unroll
        for (int i = 0; i < 16; i++) s[i] = 0.0f;
#pragma unroll
        for (int j = 0; j < DPAD / 8; j++) {
            const f32x4_t a = *(const f32x4_t*)(Kw + col * LDK + 8 * j + 4 * hh);
#pragma unroll
            for (int i = 0; i < 4; i++) s = __builtin_amdgcn_mfma_f32_32x32x2f32(a[i], qreg[4 * j + i], s, 0, 0, 0);
        }
        // register i of the accumulator holds key row 8*(i/4) + 4*hh + (i%4), query row `col`
        float m_tile = neg_inf();
        const uint32_t keep_word = keep_in_lds ? keep_bits[kv0 >> 5] : 0u;  // bit r: key kv0 + r is visible
        const bool edge = (kv0 + kRows > N) || (kCausal && kv0 + kRows - 1 > q0) ||
                          (kPad && keep_word != 0xffffffffu);
#pragma unroll
        for (int i = 0; i < 16; i++) {
            float x = kBias ? s[i] * p.scale + bias[i] : s[i] * p.scale;
            if (edge) {
                int kr = kv0 + 8 * (i >> 2) + 4 * hh + (i & 3);
                bool masked = kr >= N;
                if (kCausal) masked |= kr > q_row;
                if constexpr (kPad) {
                    if (keep_in_lds) masked |= ((keep_word >> (8 * (i >> 2) + 4 * hh + (i & 3))) & 1u) == 0;
                    else masked |= (kr < N) && (p.keep[kr] == 0);
                }
                x = masked ? neg_inf() : x;
            }
            s[i] = x;
            m_tile = (x > m_tile) ? x : m_tile;  // NaN never wins, as in the reference's `if x > m`
        }
        {
            // the two halves of the wave hold the same query rows: v_permlane32_swap leaves the lower halves' values
            // in one register and the upper halves' in the other, without a trip through LDS (neither is NaN)
            auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(m_tile), __float_as_uint(m_tile), false, false);
            const float lo = __uint_as_float(r[0]), hi = __uint_as_float(r[1]);
            m_tile = (hi > lo) ? hi : lo;
        }
        float m_new = (m_tile > m_run) ? m_tile : m_run;
        float m_use = (m_new == neg_inf()) ? 0.0f : m_new;
        float alpha = (m_run == neg_inf()) ? 0.0f : __builtin_amdgcn_exp2f((m_run - m_use) * kLog2e);
        m_run = m_new;
        // exp(x) as exp2(x * log2 e) on the hardware exp2: the difference is taken first (exact for the terms
        // that matter), so the argument carries one rounding, about 1e-7 relative on each weight
        float part[4];
#pragma unroll
        for (int i = 0; i < 16; i++) {
            float e = __builtin_amdgcn_exp2f((s[i] - m_use) * kLog2e);
            s[i] = e;
            if (i < 4) part[i] = e;
            else part[i & 3] += e;
        }
        l_run = l_run * alpha + ((part[0] + part[1]) + (part[2] + part[3]));
        if (__any(alpha != 1.0f)) {  // wave-uniform: the reference also rescales only when alpha != 1 (cpu_forward.rs:372)
#pragma unroll
            for (int t = 0; t < DT; t++)
#pragma unroll
                for (int i = 0; i < 16; i++) acc_o[t][i] *= alpha;
        }
        // O^T += V^T . P^T, two keys per instruction: the lower half of the wave feeds key 8j+r, the upper 8j+4+r
#pragma unroll
        for (int i = 0; i < 16; i++) {
            const int kr = 8 * (i >> 2) + 4 * hh + (i & 3);
#pragma unroll
            for (int t = 0; t < DT; t++) {
                float a = Vw[kr * DPAD + t * 32 + col];
                acc_o[t] = __builtin_amdgcn_mfma_f32_32x32x2f32(a, s[i], acc_o[t], 0, 0, 0);
            }
        }
    }

    // ---- merge the four partial states
    {
        float l = l_run + other_half(l_run);
        if (hh == 0) {
            red_m[wave][col] = m_run;
            red_l[wave][col] = l;
        }
    }
    __syncthreads();  // also: every wave is done with its tiles
    float m_all = neg_inf();
#pragma unroll
    for (int w2 = 0; w2 < NW; w2++) {
        float mw = red_m[w2][col];
        m_all = (mw > m_all) ? mw : m_all;
    }
    float l_all = 0.0f, my_f = 0.0f;
#pragma unroll
    for (int w2 = 0; w2 < NW; w2++) {
        float mw = red_m[w2][col];
        float f = (mw == neg_inf()) ? 0.0f : expf(mw - m_all);  // an empty partial weighs nothing
        l_all += red_l[w2][col] * f;
        if (w2 == wave) my_f = f;
    }
    if (wave == 0 && hh == 0) {
        bool good = (l_all > 0.0f) && (fabsf(l_all) != __uint_as_float(0x7f800000u)) && (l_all == l_all) && !poison;
        fin_inv[col] = good ? 1.0f / l_all : quiet_nan();
        if (p.lse && q0 + col < Nq) p.lse[((size_t)b * p.heads + h) * (size_t)Nq + q0 + col] = m_all + logf(l_all);
    }
    // this wave's weighted O, as rows [col][d], into its own K tile
#pragma unroll
    for (int t = 0; t < DT; t++)
#pragma unroll
        for (int g = 0; g < 4; g++) {
            f32x4_t o = {acc_o[t][4 * g] * my_f, acc_o[t][4 * g + 1] * my_f, acc_o[t][4 * g + 2] * my_f, acc_o[t][4 * g + 3] * my_f};
            *(f32x4_t*)(Kw + col * LDK + t * 32 + 8 * g + 4 * hh) = o;
        }
    __syncthreads();
    // all 256 threads: sum the four partial tiles, normalise, store whole rows
#pragma unroll
    for (int n = 0; n < (kRows * CH + 255) / 256; n++) {
        const int idx = 256 * n + tid;
        if (idx < kRows * CH) {
            const int r = idx / CH, c = idx % CH;
            f32x4_t sum = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
            for (int w2 = 0; w2 < NW; w2++) sum += *(const f32x4_t*)(lds + w2 * (KTILE + VTILE) + r * LDK + 4 * c);
            const float inv = fin_inv[r];
            // a NaN in fin_inv marks a row without a valid sum: the whole row is NaN, whatever O holds
            f32x4_t o;
#pragma unroll
            for (int i = 0; i < 4; i++) o[i] = (inv == inv) ? sum[i] * inv : quiet_nan();
            if (q0 + r < Nq && 4 * c < D) *(f32x4_t*)(Og + (size_t)(q0 + r) * o_pitch + 4 * c) = o;
        }
    }
}

}  // namespace

hipError_t launch_flash_f32(hipStream_t stream, const FlashF32Params& p) {
    if (p.batch == 0 || p.heads == 0 || p.seq == 0) return hipSuccess;
    dim3 grid((p.seq + kRows - 1) / kRows, p.heads, p.batch), block(64);
    int dt = (p.dim + 31) / 32;
    // the fast kernel reads whole 16-byte chunks: head dim a multiple of 4, rows and bases 16-byte aligned
    auto aligned = [](const void* ptr, const TensorLayout& l) {
        return ((uintptr_t)ptr % 16 == 0) && (l.batch_stride % 4 == 0) && (l.head_stride % 4 == 0) && (l.row_pitch % 4 == 0);
    };
    if (p.dim % 4 == 0 && p.dim <= 128 && aligned(p.q, p.lq) && aligned(p.k, p.lkv) && aligned(p.v, p.lkv) && aligned(p.out, p.lo)) {
        dim3 block4(256);
        FlashF32Params pz = p;
        // 8 (dim <= 64) or 4 waves fit on a CU: is every workgroup resident from the start?
        const long long resident = (long long)p.n_cus * (dt <= 2 ? 2 : 1);
        pz.zigzag = (p.mask == kMaskCausal) && ((long long)grid.x * grid.y * grid.z <= resident) ? 1 : 0;
        const bool exact = (p.dim % 32 == 0), pad = (p.mask == kMaskPadding);
        if (p.bias && p.mask != kMaskNone) return hipErrorInvalidValue;  // a bias comes without a mask kind
        const int mode = pad ? 2 : (p.mask == kMaskCausal ? 1 : (p.bias ? 3 : 0));
        auto launch = [&](auto dt_c, auto exact_c) {
            constexpr int kDT = decltype(dt_c)::value;
            constexpr bool kEx = decltype(exact_c)::value;
            switch (mode) {
                case 0: hipLaunchKernelGGL((flash_fwd_f32_splitk_kernel<kDT, kEx, 0>), grid, block4, 0, stream, pz); break;
                case 1: hipLaunchKernelGGL((flash_fwd_f32_splitk_kernel<kDT, kEx, 1>), grid, block4, 0, stream, pz); break;
                case 2: hipLaunchKernelGGL((flash_fwd_f32_splitk_kernel<kDT, kEx, 2>), grid, block4, 0, stream, pz); break;
                default: hipLaunchKernelGGL((flash_fwd_f32_splitk_kernel<kDT, kEx, 3>), grid, block4, 0, stream, pz); break;
            }
        };
        auto launch_dt = [&](auto dt_c) {
            if (exact) launch(dt_c, std::true_type{});
            else launch(dt_c, std::false_type{});
        };
        switch (dt) {
            case 1: launch_dt(std::integral_constant<int, 1>{}); break;
            case 2: launch_dt(std::integral_constant<int, 2>{}); break;
            case 3: launch_dt(std::integral_constant<int, 3>{}); break;
            case 4: launch_dt(std::integral_constant<int, 4>{}); break;
            default: return hipErrorInvalidValue;
        }
        return hipGetLastError();
    }
    if (p.bias || (p.seq_kv && p.seq_kv != p.seq)) return hipErrorInvalidValue;  // only the tiled kernel above does these
    switch (dt) {
        case 1: hipLaunchKernelGGL(flash_fwd_f32_kernel<1>, grid, block, 0, stream, p); break;
        case 2: hipLaunchKernelGGL(flash_fwd_f32_kernel<2>, grid, block, 0, stream, p); break;
        case 3: hipLaunchKernelGGL(flash_fwd_f32_kernel<3>, grid, block, 0, stream, p); break;
        case 4: hipLaunchKernelGGL(flash_fwd_f32_kernel<4>, grid, block, 0, stream, p); break;
        // head dims 129..256: the same kernel with a wider tile (about 100 KB of LDS, one workgroup per CU)
        case 5: hipLaunchKernelGGL(flash_fwd_f32_kernel<5>, grid, block, 0, stream, p); break;
        case 6: hipLaunchKernelGGL(flash_fwd_f32_kernel<6>, grid, block, 0, stream, p); break;
        case 7: hipLaunchKernelGGL(flash_fwd_f32_kernel<7>, grid, block, 0, stream, p); break;
        case 8: hipLaunchKernelGGL(flash_fwd_f32_kernel<8>, grid, block, 0, stream, p); break;
        default: return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

}  // namespace rt
