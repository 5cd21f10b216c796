// f32 attention backward for gfx950: the device counterpart of flash_backward
// (crates/rustorch-attention/src/cpu_backward.rs:46-185).
//
// The reference rebuilds the full seq x seq matrices P, dP and dS per (batch, head).  Here nothing of that
// size exists: the forward kernel is run once more to leave O and the row statistic L_i = m_i + ln(l_i), and
//
//   delta_i = sum_j P_ij dP_ij = dO_i . O_i                                   (prologue of flash_bwd_f32_dq_kernel)
//   P_ij    = exp(scale * Q_i.K_j - L_i),   dP_ij = dO_i . V_j,   dS_ij = P_ij (dP_ij - delta_i)
//   dQ_i = scale * sum_j dS_ij K_j                                            (flash_bwd_f32_dq_kernel)
//   dV_j = sum_i P_ij dO_i,   dK_j = scale * sum_i dS_ij Q_i                  (flash_bwd_f32_dkdv_kernel, launched second:
//                                                                              it reads the delta the dQ kernel left)
//
// are recomputed 32 x 32 tile by tile on the f32 matrix cores (v_mfma_f32_32x32x2_f32).  Each output row is owned
// by exactly one workgroup, so there are no atomics and the result does not depend on scheduling.
//
// Both kernels give a workgroup of four waves one tile of 32 "owner" rows (keys for dK/dV, queries for dQ); wave w
// walks the tiles w, w+4, ... of the other side with a private pair of LDS tiles and no workgroup barrier in the
// loop, and the four partial sums are added through LDS at the end.  The owner rows sit in registers as the
// B operand of the two score-shaped products; the accumulator of those products is already in the B-operand
// layout the two gradient products need, so P and dS never leave the register file:
//
//   dK/dV kernel:  S[q, kv] = Q.K^T and dP[q, kv] = dO.V^T   (A = Q / dO tile from LDS, B = K / V registers)
//                  dV^T[d, kv] += dO^T.P,  dK^T[d, kv] += Q^T.dS   (A = the same LDS tiles read along d)
//   dQ kernel:     S^T[kv, q] = K.Q^T and dP^T[kv, q] = V.dO^T     (A = K / V tile from LDS, B = Q / dO registers)
//                  dQ^T[d, q] += K^T.dS^T                          (A = the K tile read along d)
#include "rt_common.hpp"
#include "rt_kernels.hpp"

namespace rt {

namespace {

constexpr int kRows = 32;
constexpr int kNW = 4;  // waves per workgroup

template <int DPAD>
struct TileRegs;
template <int DPAD>
__device__ __forceinline__ void load_tile_regs(TileRegs<DPAD>& t, const float* __restrict__ src, int row0, int N, int D,
                                               int lane);
template <int DPAD, int LD>
__device__ __forceinline__ void store_tile_regs(float* dst, const TileRegs<DPAD>& t, int lane);

// Copies rows [row0, row0 + 32) x [0, dim) of a [seq, dim] matrix into a 32 x LD LDS tile, zero beyond seq and dim.
template <int DPAD, int LD>
__device__ __forceinline__ void stage_tile(float* dst, const float* __restrict__ src, int row0, int N, int D, int lane,
                                           bool vec) {
    if (vec) {
        TileRegs<DPAD> t;
        load_tile_regs<DPAD>(t, src, row0, N, D, lane);
        store_tile_regs<DPAD, LD>(dst, t, lane);
    } else {
        for (int idx = lane; idx < kRows * DPAD; idx += kWave) {
            const int r = idx / DPAD, d = idx - r * DPAD;
            dst[r * LD + d] = (row0 + r < N && d < D) ? src[(size_t)(row0 + r) * D + d] : 0.0f;
        }
    }
}

// The same copy in two halves, so that a tile can travel from global memory into registers while the previous one is
// multiplied: 16-byte loads (rows 16-byte aligned, dim a multiple of 4), then 16-byte LDS stores.
template <int DPAD>
struct TileRegs {
    f32x4_t r[kRows * (DPAD / 4) / kWave];
};
template <int DPAD>
__device__ __forceinline__ void load_tile_regs(TileRegs<DPAD>& t, const float* __restrict__ src, int row0, int N, int D,
                                               int lane) {
    constexpr int CH = DPAD / 4;
    if (D == DPAD && row0 + kRows <= N) {
        // the whole tile is there and contiguous (row pitch == DPAD): one per-lane address, constant offsets, and no
        // per-load bounds test (a wave-uniform condition)
        const f32x4_t* base = (const f32x4_t*)(src + (size_t)row0 * DPAD) + lane;
#pragma unroll
        for (int n = 0; n < kRows * CH / kWave; n++) t.r[n] = base[kWave * n];
        return;
    }
#pragma unroll
    for (int n = 0; n < kRows * CH / kWave; n++) {
        const int idx = kWave * n + lane, r = idx / CH, c = idx % CH;
        f32x4_t z = {0.0f, 0.0f, 0.0f, 0.0f};
        if (row0 + r < N && 4 * c < D) z = *(const f32x4_t*)(src + (size_t)(row0 + r) * D + 4 * c);
        t.r[n] = z;
    }
}
template <int DPAD, int LD>
__device__ __forceinline__ void store_tile_regs(float* dst, const TileRegs<DPAD>& t, int lane) {
    constexpr int CH = DPAD / 4;
#pragma unroll
    for (int n = 0; n < kRows * CH / kWave; n++) {
        const int idx = kWave * n + lane, r = idx / CH, c = idx % CH;
        *(f32x4_t*)(dst + r * LD + 4 * c) = t.r[n];
    }
}

// Adds the four waves' 32 x DPAD partial tiles (each at `tile_off` inside its wave's LDS block) and stores rows
// [row0, row0 + 32) of a [seq, dim] matrix.
template <int DPAD, int LD, int WAVE_STRIDE>
__device__ __forceinline__ void reduce_store(const float* lds, int tile_off, float* __restrict__ dst, int row0, int N,
                                             int D, int tid, bool vec) {
    constexpr int CH = DPAD / 4;
#pragma unroll
    for (int n = 0; n < (kRows * CH + 255) / 256; n++) {
        const int idx = 256 * n + tid;
        if (idx < kRows * CH) {
            const int r = idx / CH, c = idx % CH;
            f32x4_t sum = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
            for (int w = 0; w < kNW; w++) sum += *(const f32x4_t*)(lds + w * WAVE_STRIDE + tile_off + r * LD + 4 * c);
            if (row0 + r < N) {
                float* o = dst + (size_t)(row0 + r) * D + 4 * c;
                if (vec) {
                    if (4 * c < D) *(f32x4_t*)o = sum;
                } else {
#pragma unroll
                    for (int i = 0; i < 4; i++)
                        if (4 * c + i < D) o[i] = sum[i];
                }
            }
        }
    }
}

// accumulator tiles (rows d = 32t + 8g + 4hh + i of column `col`) -> rows [col][d] of an LDS tile
template <int DT, int LD>
__device__ __forceinline__ void spill_transposed(float* tile, const f32x16_t* acc, int col, int hh) {
#pragma unroll
    for (int t = 0; t < DT; t++)
#pragma unroll
        for (int g = 0; g < 4; g++) {
            f32x4_t o = {acc[t][4 * g], acc[t][4 * g + 1], acc[t][4 * g + 2], acc[t][4 * g + 3]};
            *(f32x4_t*)(tile + col * LD + t * 32 + 8 * g + 4 * hh) = o;
        }
}

// Which (batch*head, owner tile) a workgroup takes.  Workgroups are dealt round-robin to the 8 XCDs, each with its own
// L2: when the (batch, head) pairs divide evenly, XCD x takes the pairs bh = x (mod 8) one after the other, so that a
// pair's four input tensors are fetched into one L2 only.
__device__ __forceinline__ void owner_of_block(int& bh, int& tile) {
    const int nt = (int)gridDim.x, n_bh = (int)(gridDim.y * gridDim.z);
    bh = (int)blockIdx.y + (int)gridDim.y * (int)blockIdx.z;
    tile = (int)blockIdx.x;
    if ((n_bh & 7) == 0) {
        const int lin = (int)blockIdx.x + nt * bh;
        const int xcd = lin & 7, r = lin >> 3;
        bh = (r / nt) * 8 + xcd;
        tile = r % nt;
    }
}

template <int DT>  // DT = ceil(dim / 32); the head dim is zero-padded to DPAD = 32 * DT in LDS
__global__ __launch_bounds__(256, (DT <= 2 ? 2 : 1)) void flash_bwd_f32_dkdv_kernel(FlashBwdF32Params p) {
    constexpr int DPAD = 32 * DT;
    constexpr int LD = DPAD + 4;  // 16-byte reads of 16 rows tile all banks
    constexpr int TILE = kRows * LD;
    __shared__ __attribute__((aligned(16))) float lds[kNW * 2 * TILE];
    __shared__ float stat[kNW][2][kRows];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int col = lane & 31, hh = lane >> 5;
    const int N = p.seq, D = p.dim;
    const bool vec = p.vec != 0;
    int bh_i, tile_i;
    owner_of_block(bh_i, tile_i);
    const int kv0 = tile_i * kRows;
    const size_t bh = (size_t)bh_i;
    const size_t base = bh * (size_t)N * D;
    const float* __restrict__ Qg = p.q + base;
    const float* __restrict__ Kg = p.k + base;
    const float* __restrict__ Vg = p.v + base;
    const float* __restrict__ dOg = p.d_out + base;
    const float* __restrict__ lse = p.lse + bh * (size_t)N;
    const float* __restrict__ delta = p.delta + bh * (size_t)N;
    float* Qt = lds + wave * 2 * TILE;  // this wave's Q tile
    float* Ot = Qt + TILE;              // this wave's dO tile

    // the owner rows K[kv0 + col], V[kv0 + col] as B operands; contraction order d = 8j + 4hh + i
    stage_tile<DPAD, LD>(Qt, Kg, kv0, N, D, lane, vec);
    stage_tile<DPAD, LD>(Ot, Vg, kv0, N, D, lane, vec);
    float kreg[DPAD / 2], vreg[DPAD / 2];
#pragma unroll
    for (int j = 0; j < DPAD / 8; j++) {
        const f32x4_t a = *(const f32x4_t*)(Qt + col * LD + 8 * j + 4 * hh);
        const f32x4_t c = *(const f32x4_t*)(Ot + col * LD + 8 * j + 4 * hh);
#pragma unroll
        for (int i = 0; i < 4; i++) {
            kreg[4 * j + i] = a[i];
            vreg[4 * j + i] = c[i];
        }
    }

    f32x16_t acc_dv[DT], acc_dk[DT];
#pragma unroll
    for (int t = 0; t < DT; t++)
#pragma unroll
        for (int i = 0; i < 16; i++) acc_dv[t][i] = acc_dk[t][i] = 0.0f;

    const bool key_ok = kv0 + col < N;
    const int n_qt = (N + kRows - 1) / kRows;
    // at DT == 2 the registers of a second prefetched tile would cost the second wave per SIMD: dO is staged directly
    constexpr bool kPrefetchBoth = (DT != 2);
    // A row beyond seq carries the statistic +inf and a key beyond seq the bias -inf: their weights come out of
    // exp2 as exact zeros and the tile step has no data-dependent branch.
    const float kbias = key_ok ? 0.0f : neg_inf();
    TileRegs<DPAD> ra, rb;
    float nl = 0.0f, nd = 0.0f;  // the next tile's statistic and delta of row `col`
    auto load_stats = [&](int q0n) {
        const bool ok = q0n + col < N;
        nl = ok ? lse[q0n + col] : -neg_inf();
        nd = ok ? delta[q0n + col] : 0.0f;
    };
    if (wave < n_qt) {
        if (vec) {
            load_tile_regs<DPAD>(ra, Qg, wave * kRows, N, D, lane);
            if constexpr (kPrefetchBoth) load_tile_regs<DPAD>(rb, dOg, wave * kRows, N, D, lane);
        }
        load_stats(wave * kRows);
    }
    for (int qt = wave; qt < n_qt; qt += kNW) {
        const int q0 = qt * kRows;
        const bool more = qt + kNW < n_qt;
        if (vec) {
            store_tile_regs<DPAD, LD>(Qt, ra, lane);
            if constexpr (kPrefetchBoth) store_tile_regs<DPAD, LD>(Ot, rb, lane);
            else stage_tile<DPAD, LD>(Ot, dOg, q0, N, D, lane, true);
        } else {
            stage_tile<DPAD, LD>(Qt, Qg, q0, N, D, lane, false);
            stage_tile<DPAD, LD>(Ot, dOg, q0, N, D, lane, false);
        }
        if (hh == 0) {
            stat[wave][0][col] = nl;
            stat[wave][1][col] = nd;
        }
        if (more) {
            if (vec) {
                load_tile_regs<DPAD>(ra, Qg, q0 + kNW * kRows, N, D, lane);
                if constexpr (kPrefetchBoth) load_tile_regs<DPAD>(rb, dOg, q0 + kNW * kRows, N, D, lane);
            }
            load_stats(q0 + kNW * kRows);
        }
        f32x16_t s, dp;
#pragma unroll
        for (int i = 0; i < 16; i++) s[i] = dp[i] = 0.0f;
#pragma unroll
        for (int j = 0; j < DPAD / 8; j++) {
            const f32x4_t a = *(const f32x4_t*)(Qt + col * LD + 8 * j + 4 * hh);
            const f32x4_t c = *(const f32x4_t*)(Ot + col * LD + 8 * j + 4 * hh);
#pragma unroll
            for (int i = 0; i < 4; i++) {
                s = __builtin_amdgcn_mfma_f32_32x32x2f32(a[i], kreg[4 * j + i], s, 0, 0, 0);
                dp = __builtin_amdgcn_mfma_f32_32x32x2f32(c[i], vreg[4 * j + i], dp, 0, 0, 0);
            }
        }
        // register i holds query row 8*(i/4) + 4*hh + (i%4) of the tile, key kv0 + col.  The difference is taken
        // before the change of base, as in the forward kernel: it is exact where it matters (scores near the row
        // maximum), so a weight carries one rounding of its exponent
#pragma unroll
        for (int i = 0; i < 16; i++) {
            const int qr = 8 * (i >> 2) + 4 * hh + (i & 3);
            const float pv = __builtin_amdgcn_exp2f(((s[i] * p.scale - stat[wave][0][qr]) + kbias) * kLog2e);
            s[i] = pv;
            dp[i] = pv * (dp[i] - stat[wave][1][qr]) * p.scale;
        }
        // dV^T += dO^T . P and dK^T += Q^T . dS, two query rows per instruction
#pragma unroll
        for (int i = 0; i < 16; i++) {
            const int qr = 8 * (i >> 2) + 4 * hh + (i & 3);
#pragma unroll
            for (int t = 0; t < DT; t++) {
                acc_dv[t] = __builtin_amdgcn_mfma_f32_32x32x2f32(Ot[qr * LD + t * 32 + col], s[i], acc_dv[t], 0, 0, 0);
                acc_dk[t] = __builtin_amdgcn_mfma_f32_32x32x2f32(Qt[qr * LD + t * 32 + col], dp[i], acc_dk[t], 0, 0, 0);
            }
        }
    }

    spill_transposed<DT, LD>(Ot, acc_dv, col, hh);
    spill_transposed<DT, LD>(Qt, acc_dk, col, hh);
    __syncthreads();
    reduce_store<DPAD, LD, 2 * TILE>(lds, TILE, p.dv + base, kv0, N, D, tid, vec);
    reduce_store<DPAD, LD, 2 * TILE>(lds, 0, p.dk + base, kv0, N, D, tid, vec);
}

template <int DT>
__global__ __launch_bounds__(256, (DT <= 2 ? 2 : 1)) void flash_bwd_f32_dq_kernel(FlashBwdF32Params p) {
    constexpr int DPAD = 32 * DT;
    constexpr int LD = DPAD + 4;
    constexpr int TILE = kRows * LD;
    __shared__ __attribute__((aligned(16))) float lds[kNW * 2 * TILE];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int col = lane & 31, hh = lane >> 5;
    const int N = p.seq, D = p.dim;
    const bool vec = p.vec != 0;
    int bh_i, tile_i;
    owner_of_block(bh_i, tile_i);
    const int q0 = tile_i * kRows;
    const size_t bh = (size_t)bh_i;
    const size_t base = bh * (size_t)N * D;
    const float* __restrict__ Qg = p.q + base;
    const float* __restrict__ Kg = p.k + base;
    const float* __restrict__ Vg = p.v + base;
    const float* __restrict__ dOg = p.d_out + base;
    float* Kt = lds + wave * 2 * TILE;
    float* Vt = Kt + TILE;

    // the owner rows Q[q0 + col], dO[q0 + col] as B operands; the O rows follow them through the tile Q was staged in
    const bool q_ok = q0 + col < N;
    // a row beyond seq carries the statistic +inf: all its weights come out of exp2 as exact zeros
    float lse_q = q_ok ? p.lse[bh * (size_t)N + q0 + col] : -neg_inf();
    const float* __restrict__ Og = p.o + base;
    TileRegs<DPAD> r_o;
    if (vec) {
        TileRegs<DPAD> r_q, r_do;
        load_tile_regs<DPAD>(r_q, Qg, q0, N, D, lane);
        load_tile_regs<DPAD>(r_do, dOg, q0, N, D, lane);
        store_tile_regs<DPAD, LD>(Kt, r_q, lane);
        store_tile_regs<DPAD, LD>(Vt, r_do, lane);
        load_tile_regs<DPAD>(r_o, Og, q0, N, D, lane);  // travels while the operand registers are filled
    } else {
        stage_tile<DPAD, LD>(Kt, Qg, q0, N, D, lane, false);
        stage_tile<DPAD, LD>(Vt, dOg, q0, N, D, lane, false);
    }
    float qreg[DPAD / 2], oreg[DPAD / 2];
#pragma unroll
    for (int j = 0; j < DPAD / 8; j++) {
        const f32x4_t a = *(const f32x4_t*)(Kt + col * LD + 8 * j + 4 * hh);
        const f32x4_t c = *(const f32x4_t*)(Vt + col * LD + 8 * j + 4 * hh);
#pragma unroll
        for (int i = 0; i < 4; i++) {
            qreg[4 * j + i] = a[i];
            oreg[4 * j + i] = c[i];
        }
    }
    // delta of the owner rows, dO_i . O_i: a lane adds up the half of row `col` it holds of dO, the other half sits
    // in lane + 32.  Every wave of the workgroup needs all 32 values and computes them itself; wave 0 leaves them in
    // memory for the dK/dV kernel.  (Rows beyond seq and columns beyond dim are staged as zeros.)
    if (vec) store_tile_regs<DPAD, LD>(Kt, r_o, lane);
    else stage_tile<DPAD, LD>(Kt, Og, q0, N, D, lane, false);
    float delta_q = 0.0f;
#pragma unroll
    for (int j = 0; j < DPAD / 8; j++) {
        const f32x4_t a = *(const f32x4_t*)(Kt + col * LD + 8 * j + 4 * hh);
#pragma unroll
        for (int i = 0; i < 4; i++) delta_q = __builtin_fmaf(a[i], oreg[4 * j + i], delta_q);
    }
    delta_q += __shfl_xor(delta_q, 32, 64);
    if (wave == 0 && hh == 0 && q_ok) p.delta[bh * (size_t)N + q0 + col] = delta_q;
    // have the statistic land here: a wait for it inside the loop would also wait for the tile prefetched there
    asm volatile("" : "+v"(lse_q), "+v"(delta_q));

    f32x16_t acc_dq[DT];
#pragma unroll
    for (int t = 0; t < DT; t++)
#pragma unroll
        for (int i = 0; i < 16; i++) acc_dq[t][i] = 0.0f;

    const int n_kt = (N + kRows - 1) / kRows;
    constexpr bool kPrefetchBoth = (DT != 2);
    TileRegs<DPAD> ra, rb;
    if (vec && wave < n_kt) {
        load_tile_regs<DPAD>(ra, Kg, wave * kRows, N, D, lane);
        if constexpr (kPrefetchBoth) load_tile_regs<DPAD>(rb, Vg, wave * kRows, N, D, lane);
    }
    for (int kt = wave; kt < n_kt; kt += kNW) {
        const int kv0 = kt * kRows;
        if (vec) {
            store_tile_regs<DPAD, LD>(Kt, ra, lane);
            if constexpr (kPrefetchBoth) store_tile_regs<DPAD, LD>(Vt, rb, lane);
            else stage_tile<DPAD, LD>(Vt, Vg, kv0, N, D, lane, true);
            if (kt + kNW < n_kt) {
                load_tile_regs<DPAD>(ra, Kg, kv0 + kNW * kRows, N, D, lane);
                if constexpr (kPrefetchBoth) load_tile_regs<DPAD>(rb, Vg, kv0 + kNW * kRows, N, D, lane);
            }
        } else {
            stage_tile<DPAD, LD>(Kt, Kg, kv0, N, D, lane, false);
            stage_tile<DPAD, LD>(Vt, Vg, kv0, N, D, lane, false);
        }
        f32x16_t s, dp;
#pragma unroll
        for (int i = 0; i < 16; i++) s[i] = dp[i] = 0.0f;
#pragma unroll
        for (int j = 0; j < DPAD / 8; j++) {
            const f32x4_t a = *(const f32x4_t*)(Kt + col * LD + 8 * j + 4 * hh);
            const f32x4_t c = *(const f32x4_t*)(Vt + col * LD + 8 * j + 4 * hh);
#pragma unroll
            for (int i = 0; i < 4; i++) {
                s = __builtin_amdgcn_mfma_f32_32x32x2f32(a[i], qreg[4 * j + i], s, 0, 0, 0);
                dp = __builtin_amdgcn_mfma_f32_32x32x2f32(c[i], oreg[4 * j + i], dp, 0, 0, 0);
            }
        }
        // register i holds key row 8*(i/4) + 4*hh + (i%4) of the tile, query q0 + col
        const bool edge = kv0 + kRows > N;
#pragma unroll
        for (int i = 0; i < 16; i++) {
            const int kr = 8 * (i >> 2) + 4 * hh + (i & 3);
            float arg = s[i] * p.scale - lse_q;
            if (edge) arg = (kv0 + kr < N) ? arg : neg_inf();  // keys beyond seq, last tile only (uniform branch)
            const float pv = __builtin_amdgcn_exp2f(arg * kLog2e);
            dp[i] = pv * (dp[i] - delta_q) * p.scale;
        }
        // dQ^T += K^T . dS^T, two keys per instruction
#pragma unroll
        for (int i = 0; i < 16; i++) {
            const int kr = 8 * (i >> 2) + 4 * hh + (i & 3);
#pragma unroll
            for (int t = 0; t < DT; t++)
                acc_dq[t] = __builtin_amdgcn_mfma_f32_32x32x2f32(Kt[kr * LD + t * 32 + col], dp[i], acc_dq[t], 0, 0, 0);
        }
    }

    spill_transposed<DT, LD>(Kt, acc_dq, col, hh);
    __syncthreads();
    reduce_store<DPAD, LD, 2 * TILE>(lds, 0, p.dq + base, q0, N, D, tid, vec);
}

// ---- any head dim up to 512: one workgroup per row, any speed ------------------------------------------------------
// The gradients of cpu_backward.rs:46-185 for the head dims the tiled kernels above do not hold in registers.  The dQ
// kernel owns a query row i (and leaves delta_i = dO_i . O_i for the second kernel), the dK/dV kernel a key row j;
// each of the four waves takes every fourth row of the other side, forms s = q_i . k_j and dP = dO_i . v_j with the
// lanes strided over the head dim, P = exp(s * scale - L_i), dS = P (dP - delta_i) scale, and adds its products
// into per-lane sums that are folded through LDS at the end.  No atomics: every output row has one owner.
constexpr int kGenDJ = 8;  // 64 lanes x 8 = head dims up to 512

__device__ __forceinline__ float gen_wave_sum(float x) {
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) x += __shfl_xor(x, off, 64);
    return x;
}

__global__ __launch_bounds__(256) void flash_bwd_rows_dq_kernel(FlashBwdF32Params p) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int i = blockIdx.x, h = blockIdx.y, b = blockIdx.z;
    const int N = p.seq, D = p.dim;
    const size_t slab = ((size_t)b * p.heads + h) * (size_t)N;
    const float* qi = p.q + (slab + i) * D;
    const float* doi = p.d_out + (slab + i) * D;
    const float* oi = p.o + (slab + i) * D;
    float qv[kGenDJ], dov[kGenDJ], acc[kGenDJ];
    float dsum = 0.0f;
#pragma unroll
    for (int j = 0; j < kGenDJ; j++) {
        const int d = lane + 64 * j;
        qv[j] = d < D ? qi[d] : 0.0f;
        dov[j] = d < D ? doi[d] : 0.0f;
        acc[j] = 0.0f;
        if (d < D) dsum += dov[j] * oi[d];
    }
    const float delta = gen_wave_sum(dsum);
    const float L = p.lse[slab + i];
    if (threadIdx.x == 0) p.delta[slab + i] = delta;
    for (int t = wave; t < N; t += 4) {
        const float* kt = p.k + (slab + t) * D;
        const float* vt = p.v + (slab + t) * D;
        float ps = 0.0f, pd = 0.0f;
        float kk[kGenDJ];
#pragma unroll
        for (int j = 0; j < kGenDJ; j++) {
            const int d = lane + 64 * j;
            kk[j] = d < D ? kt[d] : 0.0f;
            ps += qv[j] * kk[j];
            if (d < D) pd += dov[j] * vt[d];
        }
        const float sc = gen_wave_sum(ps) * p.scale, dP = gen_wave_sum(pd);
        const float ds = expf(sc - L) * (dP - delta) * p.scale;
#pragma unroll
        for (int j = 0; j < kGenDJ; j++) acc[j] += ds * kk[j];
    }
    __shared__ float part[4][64 * kGenDJ];
#pragma unroll
    for (int j = 0; j < kGenDJ; j++) part[wave][lane + 64 * j] = acc[j];
    __syncthreads();
    for (int d = threadIdx.x; d < D; d += 256) p.dq[(slab + i) * D + d] = (part[0][d] + part[1][d]) + (part[2][d] + part[3][d]);
}

__global__ __launch_bounds__(256) void flash_bwd_rows_dkdv_kernel(FlashBwdF32Params p) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int t = blockIdx.x, h = blockIdx.y, b = blockIdx.z;
    const int N = p.seq, D = p.dim;
    const size_t slab = ((size_t)b * p.heads + h) * (size_t)N;
    const float* kt = p.k + (slab + t) * D;
    const float* vt = p.v + (slab + t) * D;
    float kv[kGenDJ], vv[kGenDJ], acc_k[kGenDJ], acc_v[kGenDJ];
#pragma unroll
    for (int j = 0; j < kGenDJ; j++) {
        const int d = lane + 64 * j;
        kv[j] = d < D ? kt[d] : 0.0f;
        vv[j] = d < D ? vt[d] : 0.0f;
        acc_k[j] = acc_v[j] = 0.0f;
    }
    for (int i = wave; i < N; i += 4) {
        const float* qi = p.q + (slab + i) * D;
        const float* doi = p.d_out + (slab + i) * D;
        float ps = 0.0f, pd = 0.0f;
        float qq[kGenDJ], dd[kGenDJ];
#pragma unroll
        for (int j = 0; j < kGenDJ; j++) {
            const int d = lane + 64 * j;
            qq[j] = d < D ? qi[d] : 0.0f;
            dd[j] = d < D ? doi[d] : 0.0f;
            ps += qq[j] * kv[j];
            pd += dd[j] * vv[j];
        }
        const float sc = gen_wave_sum(ps) * p.scale, dP = gen_wave_sum(pd);
        const float pij = expf(sc - p.lse[slab + i]);
        const float ds = pij * (dP - p.delta[slab + i]) * p.scale;
#pragma unroll
        for (int j = 0; j < kGenDJ; j++) {
            acc_k[j] += ds * qq[j];
            acc_v[j] += pij * dd[j];
        }
    }
    __shared__ float part_k[4][64 * kGenDJ], part_v[4][64 * kGenDJ];
#pragma unroll
    for (int j = 0; j < kGenDJ; j++) {
        part_k[wave][lane + 64 * j] = acc_k[j];
        part_v[wave][lane + 64 * j] = acc_v[j];
    }
    __syncthreads();
    for (int d = threadIdx.x; d < D; d += 256) {
        p.dk[(slab + t) * D + d] = (part_k[0][d] + part_k[1][d]) + (part_k[2][d] + part_k[3][d]);
        p.dv[(slab + t) * D + d] = (part_v[0][d] + part_v[1][d]) + (part_v[2][d] + part_v[3][d]);
    }
}

}  // namespace

size_t flash_bwd_f32_workspace_floats(int batch, int heads, int seq, int dim) {
    return (size_t)batch * heads * seq * ((size_t)dim + 2);
}

hipError_t launch_flash_bwd_f32(hipStream_t stream, const FlashBwdF32Params& p_in, float* workspace, int n_cus) {
    if (p_in.batch == 0 || p_in.heads == 0 || p_in.seq == 0 || p_in.dim == 0) return hipSuccess;
    if (p_in.dim > 256) return hipErrorInvalidValue;  // (the tiled forward stops there; the caller brings O and the statistic)
    const size_t rows = (size_t)p_in.batch * p_in.heads * p_in.seq;
    float* o = workspace;
    float* lse = workspace + rows * p_in.dim;
    float* delta = lse + rows;

    // forward once more: O and the row statistic
    FlashF32Params f{};
    f.q = p_in.q;
    f.k = p_in.k;
    f.v = p_in.v;
    f.out = o;
    f.lse = lse;
    f.batch = p_in.batch;
    f.heads = f.kv_heads = p_in.heads;
    f.group = 1;
    f.seq = p_in.seq;
    f.dim = p_in.dim;
    f.mask = kMaskNone;
    f.ref_bc = 64;
    f.scale = p_in.scale;
    f.n_cus = n_cus;
    f.lq = f.lkv = f.lo = layout_bhnd(p_in.heads, p_in.seq, p_in.dim);
    hipError_t e = launch_flash_f32(stream, f);
    if (e != hipSuccess) return e;
    return launch_flash_bwd_f32_saved(stream, p_in, o, lse, delta);
}

hipError_t launch_flash_bwd_f32_saved(hipStream_t stream, const FlashBwdF32Params& p_in, const float* o, const float* lse,
                                      float* delta) {
    if (p_in.batch == 0 || p_in.heads == 0 || p_in.seq == 0 || p_in.dim == 0) return hipSuccess;
    if (p_in.dim > 64 * kGenDJ) return hipErrorInvalidValue;
    FlashBwdF32Params p = p_in;
    p.o = o;
    p.lse = lse;
    p.delta = delta;
    if (p.dim > 128) {  // beyond the registers of the tiled kernels: a workgroup per row
        if (p.heads > 65535 || p.batch > 65535) return hipErrorInvalidValue;
        dim3 grid_rows(p.seq, p.heads, p.batch);
        hipLaunchKernelGGL(flash_bwd_rows_dq_kernel, grid_rows, dim3(256), 0, stream, p);
        hipLaunchKernelGGL(flash_bwd_rows_dkdv_kernel, grid_rows, dim3(256), 0, stream, p);
        return hipGetLastError();
    }
    auto aligned = [](const void* ptr) { return (uintptr_t)ptr % 16 == 0; };
    p.vec = (p.dim % 4 == 0) && aligned(p.q) && aligned(p.k) && aligned(p.v) && aligned(p.d_out) && aligned(p.dq) &&
            aligned(p.dk) && aligned(p.dv);
    dim3 grid((p.seq + kRows - 1) / kRows, p.heads, p.batch), block(256);
    const int dt = (p.dim + 31) / 32;
    switch (dt) {
        case 1:
            hipLaunchKernelGGL(flash_bwd_f32_dq_kernel<1>, grid, block, 0, stream, p);
            hipLaunchKernelGGL(flash_bwd_f32_dkdv_kernel<1>, grid, block, 0, stream, p);
            break;
        case 2:
            hipLaunchKernelGGL(flash_bwd_f32_dq_kernel<2>, grid, block, 0, stream, p);
            hipLaunchKernelGGL(flash_bwd_f32_dkdv_kernel<2>, grid, block, 0, stream, p);
            break;
        case 3:
            hipLaunchKernelGGL(flash_bwd_f32_dq_kernel<3>, grid, block, 0, stream, p);
            hipLaunchKernelGGL(flash_bwd_f32_dkdv_kernel<3>, grid, block, 0, stream, p);
            break;
        case 4:
            hipLaunchKernelGGL(flash_bwd_f32_dq_kernel<4>, grid, block, 0, stream, p);
            hipLaunchKernelGGL(flash_bwd_f32_dkdv_kernel<4>, grid, block, 0, stream, p);
            break;
        default: return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

}  // namespace rt
