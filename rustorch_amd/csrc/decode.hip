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
// Split-K GQA decode, bf16 cache, HD in {64, 128}, G = query heads per kv head (<= 8).
// grid (n_chunks, kv_heads, batch), 256 threads.  A key row (HD bf16) is read by LPR = HD/8 adjacent
// lanes, 16 bytes each, so a wave load instruction covers 64/LPR whole rows, fully coalesced.
template <int HD, int G>
__global__ __launch_bounds__(256) void decode_split_kernel(DecodeSplitParams p) {
    constexpr int LPR = HD / 8;        // lanes per row
    constexpr int RPW = 64 / LPR;      // rows per wave load
    constexpr int RPB = 4 * RPW;       // rows per workgroup pass
    constexpr int UN = 4;              // passes kept in flight
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int sub = lane % LPR, rsub = lane / LPR;
    const int chunk = blockIdx.x, kvh = blockIdx.y, b = blockIdx.z;
    const int kv_len = min(max(p.kv_lens[b], 0), p.max_seq);
    const int r_begin = chunk * p.chunk;
    if (r_begin >= kv_len) return;  // whole workgroup leaves together; the merge kernel never reads this slot
    const int r_end = min(kv_len, r_begin + p.chunk);

    const size_t cache_base = ((size_t)b * p.kv_heads + kvh) * (size_t)p.max_seq * HD;
    const uint16_t* __restrict__ K = p.k_cache + cache_base;
    const uint16_t* __restrict__ V = p.v_cache + cache_base;

    // this lane's 8 elements of each query head of the group, pre-multiplied by scale*log2(e)
    float qf[G][8];
#pragma unroll
    for (int g = 0; g < G; g++) {
        const uint16_t* qp = p.q + ((size_t)b * p.heads + (size_t)kvh * G + g) * HD + 8 * sub;
        u32x4_t w = *(const u32x4_t*)qp;
#pragma unroll
        for (int e = 0; e < 4; e++) {
            qf[g][2 * e] = bf16_lo(w[e]) * p.scale_log2e;
            qf[g][2 * e + 1] = bf16_hi(w[e]) * p.scale_log2e;
        }
    }
    float m[G], l[G], o[G][8];
#pragma unroll
    for (int g = 0; g < G; g++) {
        m[g] = neg_inf();
        l[g] = 0.0f;
#pragma unroll
        for (int e = 0; e < 8; e++) o[g][e] = 0.0f;
    }

    for (int base = r_begin + wave * RPW; base < r_end; base += UN * RPB) {  // wave-uniform trip count
        u32x4_t kw[UN], vw[UN];
        bool ok[UN];
#pragma unroll
        for (int u = 0; u < UN; u++) {
            int r = base + rsub + u * RPB;
            ok[u] = r < r_end;
            u32x4_t z = {0u, 0u, 0u, 0u};
            kw[u] = ok[u] ? *(const u32x4_t*)(K + (size_t)r * HD + 8 * sub) : z;
            vw[u] = ok[u] ? *(const u32x4_t*)(V + (size_t)r * HD + 8 * sub) : z;
        }
        float s[UN][G];
#pragma unroll
        for (int u = 0; u < UN; u++) {
            float kf[8];
#pragma unroll
            for (int e = 0; e < 4; e++) {
                kf[2 * e] = bf16_lo(kw[u][e]);
                kf[2 * e + 1] = bf16_hi(kw[u][e]);
            }
#pragma unroll
            for (int g = 0; g < G; g++) {
                float acc = 0.0f;
#pragma unroll
                for (int e = 0; e < 8; e++) acc = __builtin_fmaf(qf[g][e], kf[e], acc);
#pragma unroll
                for (int off = LPR / 2; off >= 1; off >>= 1) acc += __shfl_xor(acc, off, 64);
                s[u][g] = ok[u] ? acc : neg_inf();
            }
        }
#pragma unroll
        for (int g = 0; g < G; g++) {
            float m_new = m[g];
#pragma unroll
            for (int u = 0; u < UN; u++) m_new = fmaxf(m_new, s[u][g]);
            float m_use = (m_new == neg_inf()) ? 0.0f : m_new;
            float alpha = __builtin_amdgcn_exp2f(m[g] - m_use);
            m[g] = m_new;
            float pe[UN];
            float lsum = 0.0f;
#pragma unroll
            for (int u = 0; u < UN; u++) {
                pe[u] = __builtin_amdgcn_exp2f(s[u][g] - m_use);
                lsum += pe[u];
            }
            l[g] = l[g] * alpha + lsum;
#pragma unroll
            for (int e = 0; e < 8; e++) o[g][e] *= alpha;
#pragma unroll
            for (int u = 0; u < UN; u++) {
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    o[g][2 * e] = __builtin_fmaf(pe[u], bf16_lo(vw[u][e]), o[g][2 * e]);
                    o[g][2 * e + 1] = __builtin_fmaf(pe[u], bf16_hi(vw[u][e]), o[g][2 * e + 1]);
                }
            }
        }
    }

    // ---- fold the RPW row groups of the wave (lanes differing in rsub), then the 4 waves through LDS
#pragma unroll
    for (int g = 0; g < G; g++) {
#pragma unroll
        for (int off = LPR; off < 64; off <<= 1) {
            float m_o = __shfl_xor(m[g], off, 64);
            float l_o = __shfl_xor(l[g], off, 64);
            float m_new = fmaxf(m[g], m_o);
            float m_use = (m_new == neg_inf()) ? 0.0f : m_new;
            float ca = __builtin_amdgcn_exp2f(m[g] - m_use), cb = __builtin_amdgcn_exp2f(m_o - m_use);
            l[g] = l[g] * ca + l_o * cb;
#pragma unroll
            for (int e = 0; e < 8; e++) {
                float o_o = __shfl_xor(o[g][e], off, 64);
                o[g][e] = o[g][e] * ca + o_o * cb;
            }
            m[g] = m_new;
        }
    }
    __shared__ float sm[4][G], sl[4][G];
    __shared__ float so[4][G][HD];
    if (rsub == 0) {
#pragma unroll
        for (int g = 0; g < G; g++) {
            if (sub == 0) {
                sm[wave][g] = m[g];
                sl[wave][g] = l[g];
            }
#pragma unroll
            for (int e = 0; e < 8; e++) so[wave][g][8 * sub + e] = o[g][e];
        }
    }
    __syncthreads();
    // partial layout: ws_o[(b*heads + h)*n_chunks + chunk][HD], then ws_ml[...][2]
    float* ws_o = p.ws;
    float* ws_ml = p.ws + (size_t)p.batch * p.heads * p.n_chunks * HD;
    for (int idx = threadIdx.x; idx < G * HD; idx += 256) {
        int g = idx / HD, d = idx % HD;
        float m_all = fmaxf(fmaxf(sm[0][g], sm[1][g]), fmaxf(sm[2][g], sm[3][g]));
        float m_use = (m_all == neg_inf()) ? 0.0f : m_all;
        float acc = 0.0f, l_all = 0.0f;
#pragma unroll
        for (int w = 0; w < 4; w++) {
            float cw = __builtin_amdgcn_exp2f(sm[w][g] - m_use);
            acc += so[w][g][d] * cw;
            l_all += sl[w][g] * cw;
        }
        size_t slot = ((size_t)b * p.heads + (size_t)kvh * G + g) * p.n_chunks + chunk;
        ws_o[slot * HD + d] = acc;
        if (d == 0) {
            ws_ml[slot * 2] = m_all;
            ws_ml[slot * 2 + 1] = l_all;
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
    dim3 grid(p.n_chunks, p.kv_heads, p.batch), block(256);
    int g = p.heads / p.kv_heads;
    switch (g) {
        case 1: hipLaunchKernelGGL((decode_split_kernel<HD, 1>), grid, block, 0, stream, p); break;
        case 2: hipLaunchKernelGGL((decode_split_kernel<HD, 2>), grid, block, 0, stream, p); break;
        case 4: hipLaunchKernelGGL((decode_split_kernel<HD, 4>), grid, block, 0, stream, p); break;
        case 8: hipLaunchKernelGGL((decode_split_kernel<HD, 8>), grid, block, 0, stream, p); break;
        default: return hipErrorInvalidValue;
    }
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL(decode_merge_kernel<HD>, dim3(p.heads, p.batch), dim3(HD), 0, stream, p);
    return hipGetLastError();
}

}  // namespace

bool decode_split_supported(int heads, int kv_heads, int dim) {
    if (kv_heads <= 0 || heads % kv_heads != 0) return false;
    int g = heads / kv_heads;
    return (dim == 64 || dim == 128) && (g == 1 || g == 2 || g == 4 || g == 8);
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
