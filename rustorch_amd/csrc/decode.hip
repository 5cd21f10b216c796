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
//   kv_block_append_kernel  KVLayerCache::append, crates/rustorch-nn/src/kv_cache.rs:77-112 (seq_added rows per head).
#include <algorithm>
#include <mutex>

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
    size_t kv_pitch = (size_t)D;  // elements between consecutive key rows
    if (p.use_layout) {
        Q = (const T*)p.q + (size_t)b * p.lq.batch_stride + (size_t)h * p.lq.head_stride + (size_t)qi * p.lq.row_pitch;
        K = (const T*)p.k + (size_t)b * p.lkv.batch_stride + (size_t)kvh * p.lkv.head_stride;
        V = (const T*)p.v + (size_t)b * p.lkv.batch_stride + (size_t)kvh * p.lkv.head_stride;
        O = (T*)p.out + (size_t)b * p.lo.batch_stride + (size_t)h * p.lo.head_stride + (size_t)qi * p.lo.row_pitch;
        kv_pitch = (size_t)p.lkv.row_pitch;
    }
    // scores = (q . k) * scale, then the additive bias (crates/rustorch-nn/src/attention.rs:378-392)
    const float* __restrict__ bias_row =
        p.bias ? p.bias + ((size_t)b * p.heads + h) * (size_t)p.bias_bh_stride + (size_t)qi * (size_t)kv_len : nullptr;

    // rows past a sequence's valid queries: the fill value, nothing else
    const int n_q = p.q_lens ? min(max(p.q_lens[b], 0), p.seq_q) : p.seq_q;
    if (qi >= n_q) {
        const float fill = p.zero_padded_rows ? 0.0f : quiet_nan();
        for (int d = threadIdx.x; d < D; d += 256) store_elem(O, d, fill);
        if (p.lse && threadIdx.x == 0) p.lse[((size_t)b * p.heads + h) * p.seq_q + qi] = fill;
        return;
    }
    // last key this row sees; under the causal mask the last valid query sees every key
    int lim = kv_len - 1;
    if (p.mask == kMaskCausal) lim = min(lim, qi + (kv_len - n_q));
    const uint8_t* __restrict__ keep = p.mask == kMaskPadding ? p.keep : nullptr;
    // Mask::Padding that hides the reference's whole first key tile: every row NaN (cpu_forward.rs:268-425 takes
    // exp(-inf - (-inf)) on that tile and never recovers)
    bool poison = false;
    if (keep) {
        const int lead = min(p.ref_bc, kv_len);
        bool any = false;
        for (int j = lane; j < lead; j += 64) any |= (keep[j] != 0);
        poison = !__any(any);
    }

    float qv[kMaxDJ], o[kMaxDJ];
#pragma unroll
    for (int j = 0; j < kMaxDJ; j++) {
        int d = lane + 64 * j;
        qv[j] = d < D ? load_elem<T>(Q, d) : 0.0f;
        o[j] = 0.0f;
    }
    float m = neg_inf(), l = 0.0f;
    for (int t = wave; t <= lim; t += 4) {
        if (keep && keep[t] == 0) continue;  // (wave-uniform)
        float part = 0.0f;
#pragma unroll
        for (int j = 0; j < kMaxDJ; j++) {
            int d = lane + 64 * j;
            if (d < D) part += qv[j] * load_elem<T>(K, (size_t)t * kv_pitch + d);
        }
        float s = wave_sum(part) * p.scale;
        if (bias_row) s += bias_row[t];
        float m_new = s > m ? s : m;
        float m_use = (m_new == neg_inf()) ? 0.0f : m_new;
        float alpha = (m == neg_inf()) ? 0.0f : expf(m - m_use);
        float e = expf(s - m_use);
        l = l * alpha + e;
        m = m_new;
#pragma unroll
        for (int j = 0; j < kMaxDJ; j++) {
            int d = lane + 64 * j;
            if (d < D) o[j] = o[j] * alpha + e * load_elem<T>(V, (size_t)t * kv_pitch + d);
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
        // flash_forward's rows: out = O * (1 / l) when l > 0 and finite, NaN otherwise (cpu_forward.rs:405-421)
        const bool bad = p.flash_rows && (!(l_all > 0.0f) || !(l_all < __uint_as_float(0x7f800000u)) || poison);
#pragma unroll
        for (int j = 0; j < kMaxDJ; j++) {
            int d = lane + 64 * j;
            if (d < D) {
                float acc = 0.0f;
#pragma unroll
                for (int w = 0; w < 4; w++) acc += so[w][d] * cw[w];
                store_elem(O, d, bad ? quiet_nan() : acc * inv);
            }
        }
        if (p.lse && lane == 0) p.lse[((size_t)b * p.heads + h) * p.seq_q + qi] = bad ? quiet_nan() : m_all + logf(l_all);
    }
}

// ------------------------------------------------------------------------------------------------
// Split-K GQA decode over a ragged batch, bf16 cache, HD in {64, 128}, up to 16 query heads per kv head.
//
// Work is the flat list of 32-row steps of every (sequence, kv head) segment, in (b, kvh, row) order:
// S steps in all.  A fixed grid of one-wave workgroups (as many as the GPU holds at once) cuts that
// list into equal contiguous spans, so every wave streams the same number of bytes whatever the
// lengths are, no workgroup is launched for rows that do not exist, and a segment is split only where
// a span boundary falls inside it.  A wave leaves one partial (o, m, l) per segment it touches, at slot
// (its index - index of the first wave on that segment); the merge kernel folds a head's partials with
// the online-softmax monoid (crates/rustorch-attention/src/online_softmax.rs:105-131, extended with o).
//
// Per step the wave loads K and V with fully coalesced 16-byte loads (a load instruction covers 4
// whole rows), parks them in its private LDS tile, and runs both products on the matrix cores with
// the group's query heads as the (zero-padded) 16-wide column block:
//
//   S^T[kv, h]  = K[kv, :] . Q[h, :]        v_mfma_f32_16x16x32_bf16, A = K tile, B = Q (registers)
//   O^T[d, h]  += V^T[d, kv] . P^T[kv, h]    A = V tile read transposed (ds_read_b64_tr_b16), B = P
//
// Lane l holds column h = l % 16 and the 8 keys 16*rt + 4*(l/16) + i of the step, which as they
// stand are the 8 contraction slots of its B operand for the second product; the V operand is
// fetched with the same slot -> key map.
constexpr int kDecRows = 32;     // key rows per step
constexpr int kDecSpanMin = 8;   // a wave takes at least this many steps (bounds the partials per segment); batches
constexpr int kDecSpanMinOne = 2;  // the same for a single sequence, where the latency of one call is what counts

__device__ __forceinline__ int dec_steps(int len) { return (len + kDecRows - 1) / kDecRows; }
__device__ __forceinline__ int dec_len(const DecodeSplitParams& p, int b) {
    return min(max(p.kv_lens ? p.kv_lens[b] : p.kv_len, 0), p.max_seq);
}

// slots of `ws` (the (m, l) pairs follow the slots' o vectors)
__device__ __forceinline__ size_t dec_slots(const DecodeSplitParams& p) {
    return p.compact ? ((size_t)p.n_waves + (size_t)p.batch * p.kv_heads) * (size_t)(p.heads / p.kv_heads)
                     : (size_t)p.batch * p.heads * p.n_part;
}

__device__ __forceinline__ int wave_sum_i(int x) {
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) x += __shfl_xor(x, off, 64);
    return x;
}
__device__ __forceinline__ int wave_incl_scan_i(int x, int lane) {
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
        int y = __shfl_up(x, off, 64);
        if (lane >= off) x += y;
    }
    return x;
}

// Steps of all sequences (each counted kv_heads times) and the span every wave takes.
__device__ __forceinline__ void dec_total(const DecodeSplitParams& p, int lane, int& total, int& span) {
    int t = 0;
    for (int r = 0; r < p.batch; r += 64) {
        int i = r + lane;
        t += wave_sum_i(i < p.batch ? p.kv_heads * dec_steps(dec_len(p, i)) : 0);
    }
    total = t;
    span = max((t + p.n_waves - 1) / p.n_waves, p.span_min);
}
// First step (in the flat list) of sequence b.
__device__ __forceinline__ int dec_seq_start(const DecodeSplitParams& p, int lane, int b) {
    int t = 0;
    for (int r = 0; r < b; r += 64) {
        int i = r + lane;
        t += wave_sum_i(i < b ? p.kv_heads * dec_steps(dec_len(p, i)) : 0);
    }
    return t;
}

struct DecCursor {  // position in the flat step list
    int b, kvh, st, steps_b, len_b;
};

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
    const int w = blockIdx.x;
    const int G = p.heads / p.kv_heads;
    const int Hkv = p.kv_heads;

    int total, span;
    dec_total(p, lane, total, span);
    const int first = w * span;
    const int last = min(total, first + span);
    if (first >= last) return;

    // ---- locate the sequence that holds step `first`
    DecCursor cur;
    int seq_start;  // flat index of the first step of sequence cur.b
    {
        int base = 0, b = 0, found_start = 0;
        for (int r = 0; r < p.batch; r += 64) {
            int i = r + lane;
            int st = i < p.batch ? Hkv * dec_steps(dec_len(p, i)) : 0;
            int incl = wave_incl_scan_i(st, lane) + base;
            int cnt = __popcll(__ballot(i < p.batch && incl <= first));  // sequences of this round that end before `first`
            if (cnt < 64) {
                b = r + cnt;
                found_start = cnt == 0 ? base : __shfl(incl, cnt - 1, 64);
                break;
            }
            base = __shfl(incl, 63, 64);
        }
        cur.b = b;
        seq_start = found_start;
        cur.len_b = dec_len(p, b);
        cur.steps_b = dec_steps(cur.len_b);
        int local = first - seq_start;
        cur.kvh = local / cur.steps_b;
        cur.st = local - cur.kvh * cur.steps_b;
    }
    auto advance = [&](DecCursor& c) {
        if (++c.st == c.steps_b) {
            c.st = 0;
            if (++c.kvh == Hkv) {
                c.kvh = 0;
                do {  // skip empty sequences; the caller never advances past the last step of the list
                    ++c.b;
                    c.len_b = c.b < p.batch ? dec_len(p, c.b) : kDecRows;
                    c.steps_b = dec_steps(c.len_b);
                } while (c.steps_b == 0);
            }
        }
    };

    const float c = p.scale_log2e;
    const float lazy_raw = 8.0f / c;
    const int ld_row = lane / CH, ld_c = lane % CH;
    const int k_off = hcol * LDK + 8 * g4;
    const int tr_off = (4 * g4 + (hcol >> 2)) * LDV + 4 * (hcol & 3);

    u32x4_t kreg[NLD], vreg[NLD];
    auto issue_loads = [&](const DecCursor& cc) {
        const size_t base = ((size_t)cc.b * Hkv + cc.kvh) * (size_t)p.max_seq * HD;
        const uint16_t* K = p.k_cache + base;
        const uint16_t* V = p.v_cache + base;
#pragma unroll
        for (int i = 0; i < NLD; i++) {
            int r = min(cc.st * kDecRows + RPI * i + ld_row, cc.len_b - 1);  // rows past the end re-read the last row; masked below
            // every cache row is read exactly once per launch: streaming (non-temporal) loads keep the rows from
            // displacing each other and the partials in L2, worth 12 % of the step on a 1.3 GB cache
            kreg[i] = __builtin_nontemporal_load((const u32x4_t*)(K + (size_t)r * HD + 8 * ld_c));
            vreg[i] = __builtin_nontemporal_load((const u32x4_t*)(V + (size_t)r * HD + 8 * ld_c));
        }
    };
    // Q as B operand: column h = lane % 16 (zero beyond the group), contraction slots 8*(lane/16)..+8
    bf16x8_t qreg[KS], qnext[KS];
    auto load_q = [&](const DecCursor& cc, bf16x8_t (&q)[KS]) {
#pragma unroll
        for (int ks = 0; ks < KS; ks++) {
            u32x4_t z = {0u, 0u, 0u, 0u};
            if (hcol < G) z = *(const u32x4_t*)(p.q + ((size_t)cc.b * p.heads + (size_t)cc.kvh * G + hcol) * HD + 32 * ks + 8 * g4);
            q[ks] = __builtin_bit_cast(bf16x8_t, z);
        }
    };

    f32x4_t acc_o[DT];
    float m_run, l_run;
    auto reset_state = [&]() {
#pragma unroll
        for (int t = 0; t < DT; t++) acc_o[t] = f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};
        m_run = neg_inf();
        l_run = 0.0f;
    };
    reset_state();

    DecCursor nxt = cur;  // the prefetch cursor runs one step ahead of `cur`
    load_q(cur, qreg);
    issue_loads(nxt);
    advance(nxt);

    for (int t = first; t < last; t++) {
        // registers -> the wave's LDS tile (the previous step's reads have been consumed by its MFMAs)
#pragma unroll
        for (int i = 0; i < NLD; i++) {
            *(u32x4_t*)(Kw + (RPI * i + ld_row) * LDK + 8 * ld_c) = kreg[i];
            *(u32x4_t*)(Vw + (RPI * i + ld_row) * LDV + 8 * ld_c) = vreg[i];
        }
        const bool more = t + 1 < last;
        if (more) {  // next step's rows (and, on a segment change, its queries) fly while this one computes
            issue_loads(nxt);
            if (nxt.st == 0) load_q(nxt, qnext);
        }

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
        const int r0 = cur.st * kDecRows;
        if (r0 + kDecRows > cur.len_b) {  // ragged last step of a segment
#pragma unroll
            for (int rt = 0; rt < 2; rt++)
#pragma unroll
                for (int i = 0; i < 4; i++)
                    if (r0 + 16 * rt + 4 * g4 + i >= cur.len_b) s[rt][i] = neg_inf();
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
            for (int tt = 0; tt < DT; tt++) acc_o[tt] *= alpha;
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

        // ---- end of a segment (or of this wave's span): leave the partial and start afresh
        const bool seg_end = (cur.st == cur.steps_b - 1);
        if (seg_end || !more) {
            float l_all = l_run;
            {
                auto r16 = __builtin_amdgcn_permlane16_swap(__float_as_uint(l_all), __float_as_uint(l_all), false, false);
                l_all = __uint_as_float(r16[0]) + __uint_as_float(r16[1]);
                auto r32 = __builtin_amdgcn_permlane32_swap(__float_as_uint(l_all), __float_as_uint(l_all), false, false);
                l_all = __uint_as_float(r32[0]) + __uint_as_float(r32[1]);
            }
            const int seg_first = t - cur.st;  // flat index of the segment's first step
            const int part = w - seg_first / span;
            if (hcol < G) {
                float* ws_o = p.ws;
                float* ws_ml = p.ws + dec_slots(p) * HD;
                const size_t slot = p.compact ? ((size_t)w + (size_t)cur.b * Hkv + cur.kvh) * G + hcol
                                              : ((size_t)cur.b * p.heads + (size_t)cur.kvh * G + hcol) * p.n_part + part;
                // acc_o[dt][i] = O^T[d = 16dt + 4g + i][h]
#pragma unroll
                for (int dt = 0; dt < DT; dt++) *(f32x4_t*)(ws_o + slot * HD + 16 * dt + 4 * g4) = acc_o[dt];
                if (g4 == 0) {
                    ws_ml[slot * 2] = m_run * c;  // the merge works in the exp2 domain
                    ws_ml[slot * 2 + 1] = l_all;
                }
            }
            reset_state();
            if (seg_end && more) {
#pragma unroll
                for (int ks = 0; ks < KS; ks++) qreg[ks] = qnext[ks];
            }
        }
        cur = nxt;
        if (more) advance(nxt);
    }
}

// grid (heads, batch), NS * HD threads: thread (d, j) folds element d of the partials j, j + NS, ... (in groups of
// eight) of the head, and the NS running states are combined through LDS.  NS = 1 for batches, where a head has a
// handful of partials; NS = 4 for a single sequence, whose keys are cut into many short spans to keep the latency
// of the call low and whose heads then have up to a hundred partials each.
template <int HD, int NS>
__global__ __launch_bounds__((HD < 64 ? 64 : HD) * NS) void decode_merge_kernel(DecodeSplitParams p) {
    constexpr int TD = HD < 64 ? 64 : HD;  // threads per sub-state
    const int h = blockIdx.x, b = blockIdx.y, d = threadIdx.x % TD, sub = threadIdx.x / TD;
    const int lane = threadIdx.x & 63;
    const int G = p.heads / p.kv_heads;
    const int kvh = h / G;
    int total, span;
    dec_total(p, lane, total, span);
    const int steps_b = dec_steps(dec_len(p, b));
    const int seg_first = dec_seq_start(p, lane, b) + kvh * steps_b;
    const int w_first = seg_first / span;
    const int n_valid = steps_b > 0 ? (seg_first + steps_b - 1) / span - w_first + 1 : 0;
    const float* ws_o = p.ws;
    const float* ws_ml = p.ws + dec_slots(p) * HD;
    // partial k of the head sits at slot0 + k * slot_step
    const size_t slot0 = p.compact ? ((size_t)w_first + (size_t)b * p.kv_heads + kvh) * G + (h - kvh * G)
                                   : ((size_t)b * p.heads + h) * p.n_part;
    const size_t slot_step = p.compact ? (size_t)G : 1;
    const int dd = d < HD ? d : HD - 1;
    // One pass over the partials, eight at a time: the loads of a group are independent of each other (one dependent
    // load after the other would cost more than the split kernel), and the running (m, acc, l) is rescaled once
    // per group.
    constexpr int kGroup = 8;
    float m_all = neg_inf(), acc = 0.0f, l_all = 0.0f;
    for (int k0 = sub * kGroup; k0 < n_valid; k0 += NS * kGroup) {
        float mv[kGroup], lv[kGroup], ov[kGroup];
#pragma unroll
        for (int j = 0; j < kGroup; j++) {
            const int k = min(k0 + j, n_valid - 1);  // repeats of the last partial are given weight 0 below
            const size_t slot = slot0 + (size_t)k * slot_step;
            mv[j] = ws_ml[slot * 2];
            lv[j] = ws_ml[slot * 2 + 1];
            ov[j] = ws_o[slot * HD + dd];
        }
        float m_new = m_all;
#pragma unroll
        for (int j = 0; j < kGroup; j++) m_new = fmaxf(m_new, mv[j]);
        const float m_use = (m_new == neg_inf()) ? 0.0f : m_new;
        const float rescale = (m_all == neg_inf()) ? 0.0f : __builtin_amdgcn_exp2f(m_all - m_use);
        acc *= rescale;
        l_all *= rescale;
#pragma unroll
        for (int j = 0; j < kGroup; j++) {
            const float cw = (k0 + j < n_valid) ? __builtin_amdgcn_exp2f(mv[j] - m_use) : 0.0f;
            acc += ov[j] * cw;
            l_all += lv[j] * cw;
        }
        m_all = m_new;
    }
    if constexpr (NS > 1) {
        __shared__ float sm_acc[NS][TD], sm_m[NS], sm_l[NS];
        sm_acc[sub][d] = acc;
        if (d == 0) {
            sm_m[sub] = m_all;
            sm_l[sub] = l_all;
        }
        __syncthreads();
        if (sub != 0) return;
        float m_tot = neg_inf();
#pragma unroll
        for (int j = 0; j < NS; j++) m_tot = fmaxf(m_tot, sm_m[j]);
        const float m_use = (m_tot == neg_inf()) ? 0.0f : m_tot;
        acc = 0.0f;
        l_all = 0.0f;
#pragma unroll
        for (int j = 0; j < NS; j++) {
            const float cw = (sm_m[j] == neg_inf()) ? 0.0f : __builtin_amdgcn_exp2f(sm_m[j] - m_use);  // empty state
            acc += sm_acc[j][d] * cw;
            l_all += sm_l[j] * cw;
        }
    }
    // kv_len == 0: no key contributes, the output row is zero (gqa.rs:261; llm_kernels.rs:456)
    float r = n_valid > 0 ? acc / l_all : 0.0f;
    if (d < HD) p.out[((size_t)b * p.heads + h) * HD + d] = f32_to_bf16_bits(r);
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

// KVLayerCache::append (kv_cache.rs:97-110): per (b, h) one contiguous run of seq_added * head_dim elements goes
// from new[b, h, 0.., :] to cache[b, h, current_len.., :].  T is the copy unit (16 bytes when everything is
// aligned, else the element); run_units / dst_stride_units / dst_first_unit are in units of T.
template <typename T>
__global__ __launch_bounds__(256) void kv_block_append_kernel(T* __restrict__ k_cache, T* __restrict__ v_cache,
                                                              const T* __restrict__ new_k, const T* __restrict__ new_v,
                                                              size_t run_units, size_t dst_stride_units,
                                                              size_t dst_first_unit) {
    const size_t bh = blockIdx.y;
    const T* sk = new_k + bh * run_units;
    const T* sv = new_v + bh * run_units;
    T* dk = k_cache + bh * dst_stride_units + dst_first_unit;
    T* dv = v_cache + bh * dst_stride_units + dst_first_unit;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < run_units; i += (size_t)gridDim.x * blockDim.x) {
        dk[i] = sk[i];
        dv[i] = sv[i];
    }
}

template <int HD>
hipError_t launch_split_hd(hipStream_t stream, const DecodeSplitParams& p) {
    hipLaunchKernelGGL(decode_split_kernel<HD>, dim3(p.n_waves), dim3(64), 0, stream, p);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    constexpr int TD = HD < 64 ? 64 : HD;
    if (p.batch == 1)
        hipLaunchKernelGGL((decode_merge_kernel<HD, 4>), dim3(p.heads, p.batch), dim3(TD * 4), 0, stream, p);
    else
        hipLaunchKernelGGL((decode_merge_kernel<HD, 1>), dim3(p.heads, p.batch), dim3(TD), 0, stream, p);
    return hipGetLastError();
}

}  // namespace

bool decode_split_supported(int heads, int kv_heads, int dim) {
    if (kv_heads <= 0 || heads % kv_heads != 0) return false;
    int g = heads / kv_heads;
    return (dim == 64 || dim == 128 || dim == 256) && g <= 16;
}

int decode_split_span_min(int batch) { return batch == 1 ? kDecSpanMinOne : kDecSpanMin; }

int decode_split_parts(int batch, int max_seq) {
    int steps_max = (max_seq + kDecRows - 1) / kDecRows;
    int span_min = decode_split_span_min(batch);
    return (steps_max + span_min - 1) / span_min + 1;
}

size_t decode_split_workspace_bytes(int batch, int heads, int dim, int max_seq) {
    return (size_t)batch * heads * decode_split_parts(batch, max_seq) * ((size_t)dim + 2) * sizeof(float);
}

size_t decode_split_compact_bytes(int batch, int heads, int kv_heads, int dim, int n_waves) {
    return ((size_t)n_waves + (size_t)batch * kv_heads) * (size_t)(heads / kv_heads) * ((size_t)dim + 2) * sizeof(float);
}

// ---- the library's own scratch, for callers that cannot allocate ----------------------------------------------
// A fixed block of device memory that exists from the moment the code object is loaded on a GPU until the process
// ends; every GPU holds its own copy at its own address.  The name `static_scratch` is only a handle for
// hipGetSymbolAddress on the host side: kernels are given the address that call returns, never the name.
constexpr size_t kStaticScratchBytes = (size_t)8 << 20;
static __device__ __align__(256) unsigned char static_scratch[kStaticScratchBytes];

namespace {
constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
void* g_scratch_ptr[kMaxDevices] = {};
}  // namespace

hipError_t decode_static_scratch(float** ptr, size_t* bytes) {
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    if (dev < 0 || dev >= kMaxDevices) return hipErrorInvalidDevice;
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        void* addr = nullptr;
        e = hipGetSymbolAddress(&addr, HIP_SYMBOL(static_scratch));
        if (e != hipSuccess) return e;
        if (!addr) return hipErrorInvalidSymbol;
        g_scratch_ptr[dev] = addr;
    }
    *ptr = (float*)g_scratch_ptr[dev];
    *bytes = kStaticScratchBytes;
    return hipSuccess;
}

// ---- scratch slots for entry points whose reference signature has no workspace ----------------------------------
// A second fixed block, cut into kStreamSlots slots of kStreamSlotBytes: the host side hands a slot to a stream the
// first time an entry point needs scratch on it (no allocation, so such a call can be the first one under stream
// capture), and calls on different streams never share a slot.  As above, the array's name is only a handle for
// hipGetSymbolAddress.
static __device__ __align__(256) unsigned char stream_scratch[(size_t)kStreamSlots * kStreamSlotBytes];

namespace {
void* g_stream_scratch_ptr[kMaxDevices] = {};
}  // namespace

hipError_t stream_static_scratch(int slot, float** ptr, size_t* bytes) {
    if (slot < 0 || slot >= kStreamSlots) return hipErrorInvalidValue;
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    if (dev < 0 || dev >= kMaxDevices) return hipErrorInvalidDevice;
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_stream_scratch_ptr[dev]) {
        void* addr = nullptr;
        e = hipGetSymbolAddress(&addr, HIP_SYMBOL(stream_scratch));
        if (e != hipSuccess) return e;
        if (!addr) return hipErrorInvalidSymbol;
        g_stream_scratch_ptr[dev] = addr;
    }
    *ptr = (float*)((unsigned char*)g_stream_scratch_ptr[dev] + (size_t)slot * kStreamSlotBytes);
    *bytes = kStreamSlotBytes;
    return hipSuccess;
}

hipError_t launch_decode_split(hipStream_t stream, const DecodeSplitParams& p) {
    if (p.batch == 0 || p.heads == 0) return hipSuccess;
    if (p.n_waves <= 0 || p.span_min <= 0) return hipErrorInvalidValue;
    if (p.dim == 64) return launch_split_hd<64>(stream, p);
    if (p.dim == 128) return launch_split_hd<128>(stream, p);
    if (p.dim == 256) return launch_split_hd<256>(stream, p);
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

// The reference's outcome for a non-finite V element under the causal mask (cpu_forward.rs:268-425 walks every key
// tile and multiplies the hidden probabilities, exact zeros, into V: 0 * NaN and 0 * Inf are NaN).  The forward kernels
// skip key tiles that no row of a query tile sees, so this pass, run after them on request, restores that outcome:
// one workgroup per (batch, kv head) finds, per column, the last key whose V element is not finite, and writes NaN
// into that column of every query row that does not see that key.  Rows that see it already hold what the reference
// holds (the kernels multiply every key a row sees).  Reads V once; writes only where something was found.
template <typename T>
__global__ __launch_bounds__(256) void strict_hidden_v_kernel(StrictVParams p) {
    const int kvh = blockIdx.x, b = blockIdx.y, tid = threadIdx.x;
    const int group = p.heads / p.kv_heads;
    int n_keys = p.seq, n_q = p.seq;
    if (p.seq_lens) n_keys = n_q = min(max(p.seq_lens[b], 0), p.seq);
    __shared__ int last_bad[512];
    for (int c = tid; c < p.dim; c += 256) last_bad[c] = -1;
    __syncthreads();
    const T* vb = (const T*)p.v + (size_t)b * p.lkv.batch_stride + (size_t)kvh * p.lkv.head_stride;
    // thread t looks at columns t % cw + k * cw of rows t / cw + k * (256 / cw): consecutive lanes, consecutive addresses
    const int cw = p.dim >= 256 ? 256 : (p.dim >= 128 ? 128 : (p.dim >= 64 ? 64 : (p.dim >= 32 ? 32 : 16)));
    const int rows_per_pass = 256 / cw;
    for (int c = tid % cw; c < p.dim; c += cw) {
        int mine = -1;
        for (int j = tid / cw; j < n_keys; j += rows_per_pass) {
            const T x = vb[(size_t)j * p.lkv.row_pitch + c];
            bool bad;
            if constexpr (sizeof(T) == 2) bad = (x & 0x7f80u) == 0x7f80u;
            else bad = (__float_as_uint(x) & 0x7f800000u) == 0x7f800000u;
            mine = bad ? j : mine;
        }
        if (mine >= 0) atomicMax(&last_bad[c], mine);
    }
    __syncthreads();
    const int off = n_keys - n_q;  // query row i sees keys j <= i + off
    for (int c = 0; c < p.dim; c++) {
        const int hidden_rows = min(last_bad[c] - off, n_q);  // rows 0 .. hidden_rows-1 do not see that key
        if (hidden_rows <= 0) continue;
        for (int g = 0; g < group; g++) {
            T* ob = (T*)p.out + (size_t)b * p.lo.batch_stride + (size_t)(kvh * group + g) * p.lo.head_stride + c;
            for (int i = tid; i < hidden_rows; i += 256) {
                if constexpr (sizeof(T) == 2) ob[(size_t)i * p.lo.row_pitch] = (T)0x7fc0u;
                else ob[(size_t)i * p.lo.row_pitch] = __uint_as_float(0x7fc00000u);
            }
        }
    }
}

hipError_t launch_strict_hidden_v(hipStream_t stream, const StrictVParams& p, bool bf16) {
    if (p.batch == 0 || p.heads == 0 || p.seq == 0) return hipSuccess;
    if (p.dim > 512 || p.kv_heads <= 0 || p.heads % p.kv_heads != 0 || p.kv_heads > 65535 || p.batch > 65535) return hipErrorInvalidValue;
    if (bf16) hipLaunchKernelGGL(strict_hidden_v_kernel<uint16_t>, dim3(p.kv_heads, p.batch), dim3(256), 0, stream, p);
    else hipLaunchKernelGGL(strict_hidden_v_kernel<float>, dim3(p.kv_heads, p.batch), dim3(256), 0, stream, p);
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

hipError_t launch_kv_block_append(hipStream_t stream, void* k_cache, void* v_cache, const void* new_k, const void* new_v,
                                  size_t batch_heads, size_t max_seq, size_t head_dim, size_t current_len,
                                  size_t seq_added, size_t elem_bytes) {
    const size_t run_bytes = seq_added * head_dim * elem_bytes;
    if (batch_heads == 0 || run_bytes == 0) return hipSuccess;
    if (batch_heads > 65535) return hipErrorInvalidValue;
    const size_t stride_bytes = max_seq * head_dim * elem_bytes, first_bytes = current_len * head_dim * elem_bytes;
    auto al16 = [](const void* p) { return ((uintptr_t)p & 15) == 0; };
    const bool wide = al16(k_cache) && al16(v_cache) && al16(new_k) && al16(new_v) && run_bytes % 16 == 0 &&
                      stride_bytes % 16 == 0 && first_bytes % 16 == 0;
    const size_t unit = wide ? 16 : elem_bytes;
    const size_t run_units = run_bytes / unit;
    const unsigned gx = (unsigned)std::min<size_t>((run_units + 255) / 256, 1024);
    dim3 grid(gx, (unsigned)batch_heads), block(256);
    if (wide) {
        hipLaunchKernelGGL(kv_block_append_kernel<u32x4_t>, grid, block, 0, stream, (u32x4_t*)k_cache, (u32x4_t*)v_cache,
                           (const u32x4_t*)new_k, (const u32x4_t*)new_v, run_units, stride_bytes / 16, first_bytes / 16);
    } else if (elem_bytes == 2) {
        hipLaunchKernelGGL(kv_block_append_kernel<uint16_t>, grid, block, 0, stream, (uint16_t*)k_cache, (uint16_t*)v_cache,
                           (const uint16_t*)new_k, (const uint16_t*)new_v, run_units, stride_bytes / 2, first_bytes / 2);
    } else if (elem_bytes == 4) {
        hipLaunchKernelGGL(kv_block_append_kernel<uint32_t>, grid, block, 0, stream, (uint32_t*)k_cache, (uint32_t*)v_cache,
                           (const uint32_t*)new_k, (const uint32_t*)new_v, run_units, stride_bytes / 4, first_bytes / 4);
    } else {
        return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

}  // namespace rt
