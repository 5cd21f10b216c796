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

}  // namespace

hipError_t launch_flash_f32(hipStream_t stream, const FlashF32Params& p) {
    if (p.batch == 0 || p.heads == 0 || p.seq == 0) return hipSuccess;
    dim3 grid((p.seq + kRows - 1) / kRows, p.heads, p.batch), block(64);
    int dt = (p.dim + 31) / 32;
    switch (dt) {
        case 1: hipLaunchKernelGGL(flash_fwd_f32_kernel<1>, grid, block, 0, stream, p); break;
        case 2: hipLaunchKernelGGL(flash_fwd_f32_kernel<2>, grid, block, 0, stream, p); break;
        case 3: hipLaunchKernelGGL(flash_fwd_f32_kernel<3>, grid, block, 0, stream, p); break;
        case 4: hipLaunchKernelGGL(flash_fwd_f32_kernel<4>, grid, block, 0, stream, p); break;
        default: return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

}  // namespace rt
