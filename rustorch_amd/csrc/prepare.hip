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

}  // namespace

hipError_t launch_decode_prepare(hipStream_t stream, const DecodePrepareParams& p) {
    if (p.batch == 0 || p.seq == 0 || p.n_heads + p.n_kv == 0 || p.head_dim == 0) return hipSuccess;
    if (p.head_dim > kPrepMaxD || (p.head_dim & 1) || p.seq > 65535 || p.batch > 65535) return hipErrorInvalidValue;
    hipLaunchKernelGGL(decode_prepare_kernel, dim3(p.n_heads + p.n_kv, p.seq, p.batch), dim3(64), 0, stream, p);
    return hipGetLastError();
}

}  // namespace rt
