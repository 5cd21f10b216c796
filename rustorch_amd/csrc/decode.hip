// Decode-side kernels for gfx950:
//
//   attn_rows_kernel      unmasked attention of single query rows over a key/value prefix, generic in
//                         head dim, grouping and element type: the decode branch of gqa_forward_f32
//                         (crates/rustorch-nn/src/gqa.rs:179-270) and the general case of
//                         gqa_decode_online_bf16 (crates/rustorch-cuda/src/llm_kernels.rs:396-457).
//   decode_split_kernel   split-K GQA decode over a ragged batch: one workgroup per (sequence, kv head,
//   decode_merge_kernel   context chunk) serves every query head of the group from ONE read of the chunk
//                         and leaves an (o, m, l) partial; the merge kernel folds the partials with the
//                         online-softmax monoid (crates/rustorch-attention/src/online_softmax.rs:105-131,
//                         extended with o).
//   kv_append_kernel      llm_kernels.rs:353-372.
#include "rt_common.hpp"
#include "rt_kernels.hpp"

namespace rt {

namespace {

template <typename T>
__device__ __forceinline__ float load_elem(const T* p, size_t i);
template <>
__device__ __forceinline__ float load_elem<float>(const float* p, size_t i) {
    return p[i];
}
template <>
__device__ __forceinline__ float load_elem<uint16_t>(const uint16_t* p, size_t i) {
    return bf16_bits_to_f32(p[i]);
}
__device__ __forceinline__ void store_elem(float* p, size_t i, float x) { p[i] = x; }
__device__ __forceinline__ void store_elem(uint16_t* p, size_t i, float x) { p[i] = f32_to_bf16_bits(x); }

typedef short s16x4v __attribute__((ext_vector_type(4)));
typedef float f32x2v __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2v __attribute__((ext_vector_type(2)));
// transposing LDS read (see flash_bf16.hip): lane j of a 16-lane group gets element j%4 of the 8 bytes
// addressed by lanes 4e + j/4, e = 0..3
__device__ __forceinline__ u32x2_t lds_read_tr16_b64(const uint16_t* p) {
    s16x4v v = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4v __attribute__((address_space(3)))*)(p));
    return __builtin_bit_cast(u32x2_t, v);
}

__device__ __forceinline__ float wave_sum(float x) {
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) x += __shfl_xor(x, off, 64);
    return x;
}

// ------------------------------------------------------------------------------------------------
// Generic single-row attention.  grid (seq_q, heads, batch), 256 threads.  Lane l owns head-dim
// elements l, l+64, ...; each wave walks every 4th key row with its own online-softmax state; the
// four states are merged through LDS at the end.
constexpr int kMaxDJ = 8;  // dim <= 512

template <typename T>
__global__ __launch_bounds__(256) void attn_rows_kernel(AttnRowsParams p) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int qi = blockIdx.x, h = blockIdx.y, b = blockIdx.z;
    const int D = p.dim;
    const int kvh = p.head_map == 0 ? h / (p.heads / p.kv_heads) : (int)(((long)h * p.kv_heads) / p.heads);
    const int kv_len = p.kv_lens ? min(max(p.kv_lens[b], 0), p.kv_stride) : p.kv_len;
    const T* __restrict__ Q = (const T*)p.q + (((size_t)b * p.heads + h) * p.seq_q + qi) * D;
    const T* __restrict__ K = (const T*)p.k + ((size_t)b * p.kv_heads + kvh) * (size_t)p.kv_stride * D;
    const T* __restrict__ V = (const T*)p.v + ((size_t)b * p.kv_heads + kvh) * (size_t)p.kv_stride * D;
    T* __restrict__ O = (T*)p.out + (((size_t)b * p.heads + h) * p.seq_q + qi) * D;

    float qv[kMaxDJ], o[kMaxDJ];
#pragma unroll
    for (int j = 0; j < kMaxDJ; j++) {
        int d = lane + 64 * j;
        qv[j] = d < D ? load_elem<T>(Q, d) : 0.0f;
        o[j] = 0.0f;
    }
    float m = neg_inf(), l = 0.0f;
    for (int t = wave; t < kv_len; t += 4) {
        float part = 0.0f;
#pragma unroll
        for (int j = 0; j < kMaxDJ; j++) {
            int d = lane + 64 * j;
            if (d < D) part += qv[j] * load_elem<T>(K, (size_t)t * D + d);
        }
        float s = wave_sum(part) * p.scale;
        float m_new = s > m ? s : m;
        float m_use = (m_new == neg_inf()) ? 0.0f : m_new;
        float alpha = (m == neg_inf()) ? 0.0f : expf(m - m_use);
        float e = expf(s - m_use);
        l = l * alpha + e;
        m = m_new;
#pragma unroll
        for (int j = 0; j < kMaxDJ; j++) {
            int d = lane + 64 * j;
            if (d < D) o[j] = o[j] * alpha + e * load_elem<T>(V, (size_t)t * D + d);
        }
    }
    __shared__ float sm[4], sl[4];
    __shared__ float so[4][64 * kMaxDJ];
    if (lane == 0) {
        sm[wave] = m;
        sl[wave] = l;
    }
#pragma unroll
    for (int j = 0; j < kMaxDJ; j++) so[wave][lane + 64 * j] = o[j];
    __syncthreads();
    if (wave == 0) {
        float m_all = neg_inf();
#pragma unroll
        for (int w = 0; w < 4; w++) m_all = sm[w] > m_all ? sm[w] : m_all;
        float l_all = 0.0f;
        float cw[4];
#pragma unroll
        for (int w = 0; w < 4; w++) {
            cw[w] = (sm[w] == neg_inf()) ? 0.0f : expf(sm[w] - m_all);  // an empty state is the identity
            l_all += sl[w] * cw[w];
        }
        // kv_len == 0: nothing accumulated; the reference writes zeros (gqa.rs:261, no key to add)
        float inv = kv_len > 0 ? 1.0f / l_all : 0.0f;
#pragma unroll
        for (int j = 0; j < kMaxDJ; j++) {
            int d = lane + 64 * j;
            if (d < D) {
                float acc = 0.0f;
#pragma unroll
                for (int w = 0; w < 4; w++) acc += so[w][d] * cw[w];
                store_elem(O, d, acc * inv);
            }
        }
    }
}

// ------------------------------------------------------------------------------------------------
// Split-K GQA decode, bf16 cache, HD in {64, 128}, up to 16 query heads per kv head.
// grid (n_chunks, kv_heads, batch), ONE wavefront per workgroup: a wave streams `chunk` key rows of
// one (sequence, kv head) and serves every query head of the group from that single read.
//
// Per step of 32 rows the wave loads K and V with fully coalesced 16-byte loads (a load instruction
// covers 4 whole rows), parks them in its private LDS tile, and runs both products on the matrix
// cores with the group's query heads as the (zero-padded) 16-wide column block:
//
//   S^T[kv, h]  = K[kv, :] . Q[h, :]        v_mfma_f32_16x16x32_bf16, A = K tile, B = Q (registers)
//   O^T[d, h]  += V^T[d, kv] . P^T[kv, h]    A = V tile read transposed (ds_read_b64_tr_b16), B = P
//
// Lane l holds column h = l % 16 and the 8 keys 16*rt + 4*(l/16) + i of the step, which as they
// stand are the 8 contraction slots of its B operand for the second product; the V operand is
// fetched with the same slot -> key map.  The memory system sees nothing but long coalesced
// streams; the VALU work per byte is a small fraction of a lane-per-element formulation.
constexpr int kDecRows = 32;  // key rows per step

template <int HD>
__global__ __launch_bounds__(64) void decode_split_kernel(DecodeSplitParams p) {
    constexpr int LDK = HD + 8;    // +16 B: 16 rows x 16 B tile all 64 banks
    constexpr int LDV = HD + 16;   // +32 B: 8 rows x 32 B tile all 64 banks (transposing reads)
    constexpr int KS = HD / 32;    // contraction steps of the score product
    constexpr int DT = HD / 16;    // 16-row tiles of O^T
    constexpr int CH = HD / 8;     // 16-byte chunks per row
    constexpr int RPI = 64 / CH;   // rows covered by one wave load instruction
    constexpr int NLD = kDecRows / RPI;  // load instructions per tile
    __shared__ __attribute__((aligned(16))) uint16_t Kw[kDecRows * LDK];
    __shared__ __attribute__((aligned(16))) uint16_t Vw[kDecRows * LDV];

    const int lane = threadIdx.x;
    const int hcol = lane & 15, g4 = lane >> 4;
    const int chunk = blockIdx.x, kvh = blockIdx.y, b = blockIdx.z;
    const int G = p.heads / p.kv_heads;
    const int kv_len = min(max(p.kv_lens[b], 0), p.max_seq);
    const int r_begin = chunk * p.chunk;
    if (r_begin >= kv_len) return;  // the merge kernel never reads this slot
    const int r_end = min(kv_len, r_begin + p.chunk);

    const size_t cache_base = ((size_t)b * p.kv_heads + kvh) * (size_t)p.max_seq * HD;
    const uint16_t* __restrict__ K = p.k_cache + cache_base;
    const uint16_t* __restrict__ V = p.v_cache + cache_base;

    // Q as B operand: column h = lane % 16 (zero beyond the group), contraction slots 8*(lane/16)..+8
    bf16x8_t qreg[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ks++) {
        u32x4_t z = {0u, 0u, 0u, 0u};
        if (hcol < G) z = *(const u32x4_t*)(p.q + ((size_t)b * p.heads + (size_t)kvh * G + hcol) * HD + 32 * ks + 8 * g4);
        qreg[ks] = __builtin_bit_cast(bf16x8_t, z);
    }
    f32x4_t acc_o[DT];
#pragma unroll
    for (int t = 0; t < DT; t++) acc_o[t] = f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};
    float m_run = neg_inf(), l_run = 0.0f;
    const float c = p.scale_log2e;
    const float lazy_raw = 8.0f / c;

    const int ld_row = lane / CH, ld_c = lane % CH;
    const int k_off = hcol * LDK + 8 * g4;
    const int tr_off = (4 * g4 + (hcol >> 2)) * LDV + 4 * (hcol & 3);

    u32x4_t kreg[NLD], vreg[NLD];
    auto issue_loads = [&](int r0) {
#pragma unroll
        for (int i = 0; i < NLD; i++) {
            int r = min(r0 + RPI * i + ld_row, r_end - 1);  // rows past the end re-read the last row; masked below
            kreg[i] = *(const u32x4_t*)(K + (size_t)r * HD + 8 * ld_c);
            vreg[i] = *(const u32x4_t*)(V + (size_t)r * HD + 8 * ld_c);
        }
    };
    issue_loads(r_begin);

    for (int r0 = r_begin; r0 < r_end; r0 += kDecRows) {
        // registers -> the wave's LDS tile (the previous step's reads have been consumed by its MFMAs)
#pragma unroll
        for (int i = 0; i < NLD; i++) {
            *(u32x4_t*)(Kw + (RPI * i + ld_row) * LDK + 8 * ld_c) = kreg[i];
            *(u32x4_t*)(Vw + (RPI * i + ld_row) * LDV + 8 * ld_c) = vreg[i];
        }
        if (r0 + kDecRows < r_end) issue_loads(r0 + kDecRows);  // next step's rows fly while this one computes

        // ---- S^T = K . Q^T, two 16-key row tiles
        f32x4_t s[2];
#pragma unroll
        for (int rt = 0; rt < 2; rt++) {
            s[rt] = f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
            for (int ks = 0; ks < KS; ks++) {
                bf16x8_t a = *(const bf16x8_t*)(Kw + 16 * rt * LDK + k_off + 32 * ks);
                s[rt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, qreg[ks], s[rt], 0, 0, 0);
            }
        }
        if (r0 + kDecRows > r_end) {  // ragged last step
#pragma unroll
            for (int rt = 0; rt < 2; rt++)
#pragma unroll
                for (int i = 0; i < 4; i++)
                    if (r0 + 16 * rt + 4 * g4 + i >= r_end) s[rt][i] = neg_inf();
        }
        // ---- column max over the 32 keys: in-lane, then across the four 16-lane groups
        float m_step = fmaxf(fmaxf(fmaxf(s[0][0], s[0][1]), fmaxf(s[0][2], s[0][3])),
                             fmaxf(fmaxf(s[1][0], s[1][1]), fmaxf(s[1][2], s[1][3])));
        {
            auto r16 = __builtin_amdgcn_permlane16_swap(__float_as_uint(m_step), __float_as_uint(m_step), false, false);
            m_step = fmaxf(__uint_as_float(r16[0]), __uint_as_float(r16[1]));
            auto r32 = __builtin_amdgcn_permlane32_swap(__float_as_uint(m_step), __float_as_uint(m_step), false, false);
            m_step = fmaxf(__uint_as_float(r32[0]), __uint_as_float(r32[1]));
        }
        if (__any(m_step > m_run + lazy_raw)) {  // raise the running max only when it pays (wave-uniform)
            float m_new = fmaxf(m_run, m_step);
            float m_use = (m_new == neg_inf()) ? 0.0f : m_new;
            float alpha = __builtin_amdgcn_exp2f((m_run - m_use) * c);
            m_run = m_new;
            l_run *= alpha;
#pragma unroll
            for (int t = 0; t < DT; t++) acc_o[t] *= alpha;
        }
        const float mc = ((m_run == neg_inf()) ? 0.0f : m_run) * c;
        float pe[8];
#pragma unroll
        for (int i = 0; i < 8; i++) pe[i] = __builtin_amdgcn_exp2f(__builtin_fmaf(s[i >> 2][i & 3], c, -mc));
        l_run += ((pe[0] + pe[1]) + (pe[2] + pe[3])) + ((pe[4] + pe[5]) + (pe[6] + pe[7]));
        u32x4_t pb;
#pragma unroll
        for (int e = 0; e < 4; e++) {
            f32x2v x = {pe[2 * e], pe[2 * e + 1]};
            pb[e] = __builtin_bit_cast(uint32_t, __builtin_convertvector(x, bf16x2v));
        }
        const bf16x8_t pB = __builtin_bit_cast(bf16x8_t, pb);
        // ---- O^T += V^T . P^T: slots 0-3 of a lane are keys 4g..4g+3, slots 4-7 keys 16+4g..16+4g+3
#pragma unroll
        for (int dt = 0; dt < DT; dt++) {
            const uint16_t* vp = Vw + tr_off + 16 * dt;
            u32x2_t lo = lds_read_tr16_b64(vp);
            u32x2_t hi = lds_read_tr16_b64(vp + 16 * LDV);
            u32x4_t av = {lo[0], lo[1], hi[0], hi[1]};
            acc_o[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, av), pB, acc_o[dt], 0, 0, 0);
        }
    }

    // ---- row sum across the four lane groups, then the partial (o, m, l) of this chunk
    {
        auto r16 = __builtin_amdgcn_permlane16_swap(__float_as_uint(l_run), __float_as_uint(l_run), false, false);
        l_run = __uint_as_float(r16[0]) + __uint_as_float(r16[1]);
        auto r32 = __builtin_amdgcn_permlane32_swap(__float_as_uint(l_run), __float_as_uint(l_run), false, false);
        l_run = __uint_as_float(r32[0]) + __uint_as_float(r32[1]);
    }
    if (hcol < G) {
        float* ws_o = p.ws;
        float* ws_ml = p.ws + (size_t)p.batch * p.heads * p.n_chunks * HD;
        const size_t slot = ((size_t)b * p.heads + (size_t)kvh * G + hcol) * p.n_chunks + chunk;
        // acc_o[dt][i] = O^T[d = 16dt + 4g + i][h]
#pragma unroll
        for (int dt = 0; dt < DT; dt++) *(f32x4_t*)(ws_o + slot * HD + 16 * dt + 4 * g4) = acc_o[dt];
        if (g4 == 0) {
            ws_ml[slot * 2] = m_run * c;  // the merge works in the exp2 domain
            ws_ml[slot * 2 + 1] = l_run;
        }
    }
}

// grid (heads, batch), HD threads.
template <int HD>
__global__ __launch_bounds__(HD) void decode_merge_kernel(DecodeSplitParams p) {
    const int h = blockIdx.x, b = blockIdx.y, d = threadIdx.x;
    const int kv_len = min(max(p.kv_lens[b], 0), p.max_seq);
    const int n_valid = (kv_len + p.chunk - 1) / p.chunk;
    const float* ws_o = p.ws;
    const float* ws_ml = p.ws + (size_t)p.batch * p.heads * p.n_chunks * HD;
    const size_t slot0 = ((size_t)b * p.heads + h) * p.n_chunks;
    float m_all = neg_inf();
    for (int c = 0; c < n_valid; c++) m_all = fmaxf(m_all, ws_ml[(slot0 + c) * 2]);
    float m_use = (m_all == neg_inf()) ? 0.0f : m_all;
    float acc = 0.0f, l_all = 0.0f;
    for (int c = 0; c < n_valid; c++) {
        float cw = __builtin_amdgcn_exp2f(ws_ml[(slot0 + c) * 2] - m_use);
        acc += ws_o[(slot0 + c) * HD + d] * cw;
        l_all += ws_ml[(slot0 + c) * 2 + 1] * cw;
    }
    // kv_len == 0: no key contributes, the output row is zero (gqa.rs:261; llm_kernels.rs:456)
    float r = n_valid > 0 ? acc / l_all : 0.0f;
    p.out[((size_t)b * p.heads + h) * HD + d] = f32_to_bf16_bits(r);
}

__global__ void kv_append_kernel(uint16_t* __restrict__ k_cache, uint16_t* __restrict__ v_cache,
                                 const uint16_t* __restrict__ k_in, const uint16_t* __restrict__ v_in, int pos,
                                 int n_kv, int head_dim, int max_seq) {
    int idx = blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= n_kv * head_dim) return;
    int kv_h = idx / head_dim, i = idx - kv_h * head_dim;
    size_t off = ((size_t)kv_h * max_seq + pos) * head_dim + i;
    k_cache[off] = k_in[idx];
    v_cache[off] = v_in[idx];
}

template <int HD>
hipError_t launch_split_hd(hipStream_t stream, const DecodeSplitParams& p) {
    dim3 grid(p.n_chunks, p.kv_heads, p.batch), block(64);
    hipLaunchKernelGGL(decode_split_kernel<HD>, grid, block, 0, stream, p);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL(decode_merge_kernel<HD>, dim3(p.heads, p.batch), dim3(HD), 0, stream, p);
    return hipGetLastError();
}

}  // namespace

bool decode_split_supported(int heads, int kv_heads, int dim) {
    if (kv_heads <= 0 || heads % kv_heads != 0) return false;
    int g = heads / kv_heads;
    return (dim == 64 || dim == 128) && g <= 16;
}

int decode_split_chunk(int max_seq) {
    (void)max_seq;
    return 512;
}

size_t decode_split_workspace_bytes(int batch, int heads, int dim, int max_seq) {
    int chunk = decode_split_chunk(max_seq);
    size_t n_chunks = ((size_t)max_seq + chunk - 1) / chunk;
    if (n_chunks == 0) n_chunks = 1;
    return (size_t)batch * heads * n_chunks * ((size_t)dim + 2) * sizeof(float);
}

hipError_t launch_decode_split(hipStream_t stream, const DecodeSplitParams& p) {
    if (p.batch == 0 || p.heads == 0) return hipSuccess;
    if (p.dim == 64) return launch_split_hd<64>(stream, p);
    if (p.dim == 128) return launch_split_hd<128>(stream, p);
    return hipErrorInvalidValue;
}

hipError_t launch_attn_rows_f32(hipStream_t stream, const AttnRowsParams& p) {
    if (p.batch == 0 || p.heads == 0 || p.seq_q == 0) return hipSuccess;
    if (p.dim > 64 * kMaxDJ) return hipErrorInvalidValue;
    hipLaunchKernelGGL(attn_rows_kernel<float>, dim3(p.seq_q, p.heads, p.batch), dim3(256), 0, stream, p);
    return hipGetLastError();
}

hipError_t launch_attn_rows_bf16(hipStream_t stream, const AttnRowsParams& p) {
    if (p.batch == 0 || p.heads == 0 || p.seq_q == 0) return hipSuccess;
    if (p.dim > 64 * kMaxDJ) return hipErrorInvalidValue;
    hipLaunchKernelGGL(attn_rows_kernel<uint16_t>, dim3(p.seq_q, p.heads, p.batch), dim3(256), 0, stream, p);
    return hipGetLastError();
}

hipError_t launch_kv_append_bf16(hipStream_t stream, uint16_t* k_cache, uint16_t* v_cache, const uint16_t* k_in,
                                 const uint16_t* v_in, int pos, int n_kv, int head_dim, int max_seq) {
    int n = n_kv * head_dim;
    if (n <= 0) return hipSuccess;
    hipLaunchKernelGGL(kv_append_kernel, dim3((n + 255) / 256), dim3(256), 0, stream, k_cache, v_cache, k_in, v_in,
                       pos, n_kv, head_dim, max_seq);
    return hipGetLastError();
}

}  // namespace rt
