// The steps between the QKV projection and decode attention, in one launch: per-head RMSNorm of q and k
// (model.rs:862-897, Qwen3 q_norm / k_norm), half-split RoPE (rope.rs:162-205: dim k pairs with dim k + D/2,
// cos/sin from the tables of RoPE::new) and the append of k and v to the caches (llm_kernels.rs:353-372) -- steps
// 2a, 2b and 3 of LlamaModel::decode_step (crates/rustorch-llm/src/model.rs:575-636), for a batch of sequences
// with their own positions and `seq` new tokens each (1 when decoding, the prompt length when prefilling: the
// [batch, heads, seq, head_dim] layout and the position_offset + s rule of rope.rs:92-96, the row range
// [current_len, current_len + seq) of kv_cache.rs:97-110), on bf16 storage.
//
// Every value is widened to f32, run through the reference's f32 arithmetic in the reference's order -- the sum
// of squares is taken sequentially, products and sums are rounded separately (this file is compiled with
// floating-point contraction off) -- and rounded to bf16 once, so the result is the bf16 rounding of what the
// CPU path computes on the same bf16 inputs, bit for bit.
#include "rt_common.hpp"
#include "rt_kernels.hpp"

#pragma clang fp contract(off)

namespace rt {

namespace {

constexpr int kPrepMaxD = 512;

// grid (n_heads + n_kv, seq, batch), one wave per head row
__global__ __launch_bounds__(64) void decode_prepare_kernel(DecodePrepareParams p) {
    __shared__ float row[kPrepMaxD];
    const int lane = threadIdx.x;
    const int h = blockIdx.x, sq = blockIdx.y, b = blockIdx.z;
    const int D = p.head_dim, half = D / 2, S = p.seq;
    const int pos0 = p.positions ? p.positions[b] : p.pos;
    // a sequence whose rows would leave the cache or the tables writes nothing (the host checks a scalar position;
    // positions that live on the device are the caller's to keep in range)
    if (pos0 < 0 || pos0 + S > p.max_seq || pos0 + S > p.table_rows) return;
    const int pos = pos0 + sq;
    const bool is_q = h < p.n_heads;
    const int kvh = h - p.n_heads;
    const size_t q_row = (((size_t)b * p.n_heads + h) * S + sq) * D;
    const size_t kv_row = (((size_t)b * p.n_kv + kvh) * S + sq) * D;
    const uint16_t* src = is_q ? p.q + q_row : p.k_in + kv_row;
    const float* gamma = is_q ? p.q_gamma : p.k_gamma;

    for (int i = lane; i < D; i += kWave) row[i] = bf16_bits_to_f32(src[i]);
    __syncthreads();
    if (gamma) {
        // rms_norm_inplace (model.rs:862-885): sq accumulates in index order; every lane walks the whole row
        // (broadcast reads), which keeps the reference's summation order without a serial section
        float sq = 0.0f;
        for (int i = 0; i < D; i++) {
            const float v = row[i];
            sq = sq + v * v;
        }
        const float inv_d = 1.0f / (float)D;
        const float inv_rms = 1.0f / sqrtf(sq * inv_d + p.eps);
        __syncthreads();
        for (int i = lane; i < D; i += kWave) row[i] = row[i] * inv_rms * gamma[i];
        __syncthreads();
    }
    const float* cs = p.cos_table + (size_t)pos * half;
    const float* sn = p.sin_table + (size_t)pos * half;
    uint16_t* dst = is_q ? p.q + q_row
                         : p.k_cache + (((size_t)b * p.n_kv + kvh) * (size_t)p.max_seq + (size_t)pos) * D;
    for (int k = lane; k < half; k += kWave) {
        const float c = cs[k], si = sn[k];
        const float x0 = row[k], x1 = row[k + half];
        dst[k] = f32_to_bf16_bits(x0 * c - x1 * si);
        dst[k + half] = f32_to_bf16_bits(x1 * c + x0 * si);
    }
    if (!is_q) {
        const uint16_t* vs = p.v_in + kv_row;
        uint16_t* vd = p.v_cache + (((size_t)b * p.n_kv + kvh) * (size_t)p.max_seq + (size_t)pos) * D;
        for (int i = lane; i < D; i += kWave) vd[i] = vs[i];
    }
}

// The same arithmetic for a prompt.  With many consecutive tokens per head the one-wave kernel above is bound by its
// own redundancy (all 64 lanes of a wave take the same sum of squares, and a row is moved two bytes per lane): 308 us
// for B=4, 32 + 8 heads, 4096 tokens, D=128 (1.3 TB/s; 84 us = 4.8 TB/s here).  A workgroup takes ROWS consecutive tokens of one
// (sequence, head) -- contiguous rows in q / k_in and in the cache -- through LDS: the rows arrive with 16-byte loads,
// every thread takes the sum of squares of ONE row in index order (the reference's order, model.rs:862-885), and
// the normalised, rotated rows leave with 16-byte stores.  Rows sit in LDS as bf16 with a pitch of D + 2 elements (an odd
// number of 32-bit words: the 64 lanes that walk 64 rows in step hit 64 different banks).  D a multiple of 16, at most
// DMAX; every pointer 16-byte aligned.  Grid (token blocks, heads, batch), token blocks fastest: workgroups go round-robin
// to the 8 XCDs in that order, so all heads of a token block run on one XCD and its cos / sin rows are fetched into one
// L2, once (with the heads fastest every XCD fetched every table row: 76 MB more on the prompt above).
template <int ROWS, int DMAX>
__global__ __launch_bounds__(256) void prompt_prepare_kernel(DecodePrepareParams p) {
    __shared__ uint32_t rows_w[ROWS * (DMAX + 2) / 2];
    __shared__ float inv[ROWS];
    const int tid = threadIdx.x;
    const int h = blockIdx.y, b = blockIdx.z;
    const int sq0 = (int)blockIdx.x * ROWS;
    const int D = p.head_dim, half = D / 2, S = p.seq;
    const int pitch_w = (D + 2) / 2;  // words per row in LDS
    const int CH = D / 8;             // 16-byte chunks per row
    const int pos0 = p.positions ? p.positions[b] : p.pos;
    if (pos0 < 0 || pos0 + S > p.max_seq || pos0 + S > p.table_rows) return;  // as in the one-wave kernel
    const int n_rows = min(ROWS, S - sq0);
    const bool is_q = h < p.n_heads;
    const int kvh = h - p.n_heads;
    const size_t q_row = (((size_t)b * p.n_heads + h) * S + sq0) * D;
    const size_t kv_row = (((size_t)b * p.n_kv + kvh) * S + sq0) * D;
    const uint16_t* src = is_q ? p.q + q_row : p.k_in + kv_row;
    const float* gamma = is_q ? p.q_gamma : p.k_gamma;

    for (int c = tid; c < n_rows * CH; c += 256) {
        const int r = c / CH, ch = c - r * CH;
        const u32x4_t v = *(const u32x4_t*)(src + (size_t)r * D + 8 * ch);
        uint32_t* w = rows_w + r * pitch_w + 4 * ch;  // (rows start on odd words: four 4-byte writes)
        w[0] = v[0];
        w[1] = v[1];
        w[2] = v[2];
        w[3] = v[3];
    }
    __syncthreads();
    if (gamma) {
        for (int r = tid; r < n_rows; r += 256) {
            const uint32_t* w = rows_w + r * pitch_w;
            float sq = 0.0f;
            for (int j = 0; j < half; j++) {  // elements 2j and 2j + 1, in index order
                const uint32_t x = w[j];
                const float v0 = bf16_lo(x), v1 = bf16_hi(x);
                sq = sq + v0 * v0;
                sq = sq + v1 * v1;
            }
            const float inv_d = 1.0f / (float)D;
            inv[r] = 1.0f / sqrtf(sq * inv_d + p.eps);
        }
        __syncthreads();
    }
    uint16_t* dst = is_q ? p.q + q_row
                         : p.k_cache + (((size_t)b * p.n_kv + kvh) * (size_t)p.max_seq + (size_t)(pos0 + sq0)) * D;
    const int HP = half / 8;  // chunk pairs (k .. k + 8, k + half .. k + half + 8) per row
    for (int c = tid; c < n_rows * HP; c += 256) {
        const int r = c / HP, k0 = 8 * (c - r * HP);
        const uint32_t* w = rows_w + r * pitch_w;
        float x0[8], x1[8];
#pragma unroll
        for (int e = 0; e < 4; e++) {
            const uint32_t a = w[k0 / 2 + e], bb = w[(half + k0) / 2 + e];
            x0[2 * e] = bf16_lo(a);
            x0[2 * e + 1] = bf16_hi(a);
            x1[2 * e] = bf16_lo(bb);
            x1[2 * e + 1] = bf16_hi(bb);
        }
        if (gamma) {
            const float inv_rms = inv[r];
            const f32x4_t g0a = *(const f32x4_t*)(gamma + k0), g0b = *(const f32x4_t*)(gamma + k0 + 4);
            const f32x4_t g1a = *(const f32x4_t*)(gamma + half + k0), g1b = *(const f32x4_t*)(gamma + half + k0 + 4);
#pragma unroll
            for (int e = 0; e < 8; e++) {
                x0[e] = x0[e] * inv_rms * (e < 4 ? g0a[e] : g0b[e - 4]);
                x1[e] = x1[e] * inv_rms * (e < 4 ? g1a[e] : g1b[e - 4]);
            }
        }
        const size_t trow = (size_t)(pos0 + sq0 + r) * half + k0;
        const f32x4_t ca = *(const f32x4_t*)(p.cos_table + trow), cb = *(const f32x4_t*)(p.cos_table + trow + 4);
        const f32x4_t sa = *(const f32x4_t*)(p.sin_table + trow), sb = *(const f32x4_t*)(p.sin_table + trow + 4);
        u32x4_t o0, o1;
#pragma unroll
        for (int e = 0; e < 4; e++) {
            const int i0 = 2 * e, i1 = 2 * e + 1;
            const float c0 = i0 < 4 ? ca[i0] : cb[i0 - 4], c1 = i1 < 4 ? ca[i1] : cb[i1 - 4];
            const float s0 = i0 < 4 ? sa[i0] : sb[i0 - 4], s1 = i1 < 4 ? sa[i1] : sb[i1 - 4];
            o0[e] = pack_bf16x2(x0[i0] * c0 - x1[i0] * s0, x0[i1] * c1 - x1[i1] * s1);
            o1[e] = pack_bf16x2(x1[i0] * c0 + x0[i0] * s0, x1[i1] * c1 + x0[i1] * s1);
        }
        *(u32x4_t*)(dst + (size_t)r * D + k0) = o0;
        *(u32x4_t*)(dst + (size_t)r * D + half + k0) = o1;
    }
    if (!is_q) {
        const uint16_t* vs = p.v_in + kv_row;
        uint16_t* vd = p.v_cache + (((size_t)b * p.n_kv + kvh) * (size_t)p.max_seq + (size_t)(pos0 + sq0)) * D;
        for (int c = tid; c < n_rows * CH; c += 256) *(u32x4_t*)(vd + 8 * (size_t)c) = *(const u32x4_t*)(vs + 8 * (size_t)c);
    }
}

bool aligned16(const void* a) { return ((uintptr_t)a & 15) == 0; }

}  // namespace

hipError_t launch_decode_prepare(hipStream_t stream, const DecodePrepareParams& p) {
    if (p.batch == 0 || p.seq == 0 || p.n_heads + p.n_kv == 0 || p.head_dim == 0) return hipSuccess;
    if (p.head_dim > kPrepMaxD || (p.head_dim & 1) || p.seq > 65535 || p.batch > 65535) return hipErrorInvalidValue;
    // a prompt: the kernel that moves 64 consecutive tokens of a head through LDS, where its loads and stores are whole
    // 16-byte chunks (64 rows: 17 or 33 KB of LDS, so that four to eight workgroups share a CU; with 256 rows the same
    // prompt took 113 us instead of 80)
    const bool wide_ok = p.seq >= 32 && p.head_dim % 16 == 0 && p.head_dim <= 256 && aligned16(p.q) && aligned16(p.k_in) &&
                         aligned16(p.v_in) && aligned16(p.k_cache) && aligned16(p.v_cache) && aligned16(p.cos_table) &&
                         aligned16(p.sin_table) && aligned16(p.q_gamma) && aligned16(p.k_gamma) && p.n_heads + p.n_kv <= 65535;
    if (wide_ok) {
        if (p.head_dim <= 128) {
            hipLaunchKernelGGL((prompt_prepare_kernel<64, 128>), dim3((p.seq + 63) / 64, p.n_heads + p.n_kv, p.batch), dim3(256), 0, stream, p);
        } else {
            hipLaunchKernelGGL((prompt_prepare_kernel<64, 256>), dim3((p.seq + 63) / 64, p.n_heads + p.n_kv, p.batch), dim3(256), 0, stream, p);
        }
        return hipGetLastError();
    }
    hipLaunchKernelGGL(decode_prepare_kernel, dim3(p.n_heads + p.n_kv, p.seq, p.batch), dim3(64), 0, stream, p);
    return hipGetLastError();
}

}  // namespace rt
