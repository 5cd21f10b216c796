/*
 * attn_oracle.c -- CPU restatement of rustorch's attention hot path.
 *
 * TEST INFRASTRUCTURE ONLY.  This file is the checker the HIP kernels are
 * compared against (tests, the smoke check and the CPU-baseline leg of the
 * benchmark).  Nothing in the shipped library calls, links or falls back to
 * it.
 *
 * Every function restates one function of the reference and cites it
 * (paths relative to the reference checkout):
 *
 *   ro_flash_forward_masked   crates/rustorch-attention/src/cpu_forward.rs:193-425
 *   ro_flash_forward_scalar   crates/rustorch-attention/src/cpu_forward.rs:594-686
 *   ro_naive_forward_masked   crates/rustorch-attention/src/cpu_forward.rs:702-763
 *   ro_mask_is_masked         crates/rustorch-attention/src/mask.rs:40-46
 *   ro_osm_*                  crates/rustorch-attention/src/online_softmax.rs:44-151
 *   ro_gqa_forward_f32        crates/rustorch-nn/src/gqa.rs:94-270
 *   ro_kv_cache_append        crates/rustorch-nn/src/kv_cache.rs:77-112
 *   ro_kv_trim                crates/rustorch-llm/src/model.rs:638-650
 *   ro_gqa_decode_online_bf16 crates/rustorch-cuda/src/llm_kernels.rs:396-457
 *   ro_kv_append_bf16         crates/rustorch-cuda/src/llm_kernels.rs:353-372
 *   ro_gqa_decode_chunk_bf16  crates/rustorch-metal/src/kernels.rs:14432-14516 (gqa_decode_batched_f32: several
 *                             consecutive query positions over one cache, each causal to itself), per sequence,
 *                             f32 on bf16-rounded inputs
 *   ro_rope_tables            crates/rustorch-nn/src/rope.rs:63-90 (RoPE::new)
 *   ro_rope_half_split        crates/rustorch-nn/src/rope.rs:162-205 (apply_inplace_half_split)
 *   ro_rope_interleaved       crates/rustorch-nn/src/rope.rs:96-142 (apply_inplace)
 *   ro_rms_norm_per_head      crates/rustorch-llm/src/model.rs:862-897
 *   ro_decode_prepare_bf16    crates/rustorch-llm/src/model.rs:575-636 (steps 2a, 2b, 3 of decode_step:
 *                             per-head q/k RMSNorm, half-split RoPE, cache append) on bf16 storage
 *   ro_causal_mask, ro_sliding_window_mask, ro_bool_to_additive
 *                             crates/rustorch-nn/src/masks.rs:22-82
 *   ro_softmax_row            crates/rustorch-cpu/src/kernels/softmax.rs:146-180 (softmax_row_online_f32)
 *   ro_mha_forward_masked     crates/rustorch-nn/src/attention.rs:371-399 (steps 2-8 of the composed
 *                             MultiHeadAttention path: bmm, scale, additive mask, softmax, bmm)
 *   ro_flash_backward         crates/rustorch-attention/src/cpu_backward.rs:46-185
 *   ro_f32_to_bf16            half 2.7.1 bf16::from_f32 (round to nearest even),
 *                             the rule crates/rustorch-amp/src/bf16_kernels.rs:266-267 uses
 *
 * The tile products of the native forward live in the third-party crate
 * `gemm` 0.18.2 (Cargo.lock:1359-1362), which is not vendored.  Its result
 * is restated here as the mathematical product accumulated in f32 in
 * ascending contraction order; agreement with that crate's summation order
 * at the last-bit level is therefore "parity unpinned".  What is pinned: the
 * reference's own flash-vs-naive tolerance (1e-4), the closed forms and the
 * edge/NaN rules (see tests/test_oracle_*.py).
 *
 * Also "parity unpinned": the last bit of powf / cosf / sinf in
 * ro_rope_tables (this file uses the C library's; the reference Rust's
 * std).  One ulp of theta is 5e-4 rad at position 8192.  The tables are an
 * input of everything downstream, which is pinned given the tables.
 *
 * Built with -ffp-contract=off so that mul and add stay separate roundings,
 * as in the reference's scalar Rust loops.
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#define RO_EXPORT __attribute__((visibility("default")))

/* ---- status codes (same numbering as include/rt_attn.h) ----------------- */
enum {
    RO_OK = 0,
    RO_ERR_ZERO_DIM = 1,
    RO_ERR_BUFFER_SHAPE_MISMATCH = 2,
    RO_ERR_OUTPUT_SHAPE_MISMATCH = 3,
    RO_ERR_PADDING_LENGTH_MISMATCH = 4,
    RO_ERR_HEAD_COUNT_MISMATCH = 5,
    RO_ERR_WRONG_INPUT_LEN = 6,
    RO_ERR_KV_OVERFLOW = 7,
    RO_ERR_KV_WRONG_INPUT_LEN = 8,
    RO_ERR_ROPE_WRONG_INPUT_LEN = 9,
    RO_ERR_ROPE_POSITION_OVERFLOW = 10,
};

enum { RO_MASK_NONE = 0, RO_MASK_CAUSAL = 1, RO_MASK_PADDING = 2 };
enum { RO_WHICH_Q = 0, RO_WHICH_K = 1, RO_WHICH_V = 2, RO_WHICH_OUT = 3, RO_WHICH_FLASH = 4, RO_WHICH_DO = 6 };

typedef struct {
    uint64_t batch, heads, seq, dim, br, bc;
} ro_shape;

typedef struct {
    int32_t which;
    uint64_t expected;
    uint64_t got;
    uint64_t got2;
} ro_err;

static void set_err(ro_err *e, int which, uint64_t expected, uint64_t got) {
    if (e) {
        e->which = which;
        e->expected = expected;
        e->got = got;
        e->got2 = 0;
    }
}

/* ---- mask.rs:40-46 ------------------------------------------------------ */
RO_EXPORT int ro_mask_is_masked(int kind, const uint8_t *keep, size_t keep_n, size_t qi, size_t kj) {
    switch (kind) {
    case RO_MASK_CAUSAL:
        return kj > qi;
    case RO_MASK_PADDING:
        return kj < keep_n && !keep[kj];
    default:
        return 0;
    }
}

/* ---- cpu_forward.rs:142-169 (validate) + mask.rs:51-65 ------------------ */
static int validate(const ro_shape *s, size_t qn, size_t kn, size_t vn, size_t on, int kind, size_t keep_n,
                    ro_err *err) {
    if (s->dim == 0) return RO_ERR_ZERO_DIM;
    uint64_t expected = s->batch * s->heads * s->seq * s->dim;
    size_t lens[3] = {qn, kn, vn};
    for (int i = 0; i < 3; i++) {
        if (lens[i] != expected) {
            set_err(err, i, expected, lens[i]);
            return RO_ERR_BUFFER_SHAPE_MISMATCH;
        }
    }
    if (on != expected) {
        set_err(err, RO_WHICH_OUT, expected, on);
        return RO_ERR_OUTPUT_SHAPE_MISMATCH;
    }
    if (kind == RO_MASK_PADDING && keep_n != s->seq) {
        set_err(err, -1, s->seq, keep_n);
        return RO_ERR_PADDING_LENGTH_MISMATCH;
    }
    return RO_OK;
}

/* ---- cpu_forward.rs:268-425, one (b,h) slab ----------------------------- */
static void flash_bh_tiles(const float *q, const float *k, const float *v, float *out_slab, int kind,
                           const uint8_t *keep, size_t keep_n, float scale, size_t seq, size_t dim, size_t br,
                           size_t bc) {
    float *s_buf = (float *)malloc(sizeof(float) * br * bc);
    float *p_buf = (float *)malloc(sizeof(float) * br * bc);
    float *o_buf = (float *)malloc(sizeof(float) * br * dim);
    float *m_buf = (float *)malloc(sizeof(float) * br);
    float *l_buf = (float *)malloc(sizeof(float) * br);
    float *kt = (float *)malloc(sizeof(float) * bc * dim); /* K tile, transposed, for a vectorisable product */

    for (size_t qi = 0; qi < seq; qi += br) {
        size_t qi_end = qi + br < seq ? qi + br : seq;
        size_t br_used = qi_end - qi;
        for (size_t r = 0; r < br_used; r++) {
            m_buf[r] = -INFINITY;
            l_buf[r] = 0.0f;
            for (size_t d = 0; d < dim; d++) o_buf[r * dim + d] = 0.0f;
        }
        /* every kv tile is visited, also those a causal mask empties (:311-313) */
        for (size_t kj = 0; kj < seq; kj += bc) {
            size_t kj_end = kj + bc < seq ? kj + bc : seq;
            size_t bc_used = kj_end - kj;

            /* S = scale * (Q_tile . K_tile^T): dot product first, scale applied to the
             * finished sum (gemm alpha=0, beta=scale; :487-507). */
            for (size_t d = 0; d < dim; d++)
                for (size_t c = 0; c < bc_used; c++) kt[d * bc_used + c] = k[(kj + c) * dim + d];
            for (size_t r = 0; r < br_used; r++) {
                float *s_row = s_buf + r * bc_used;
                const float *q_row = q + (qi + r) * dim;
                for (size_t c = 0; c < bc_used; c++) s_row[c] = 0.0f;
                for (size_t d = 0; d < dim; d++) {
                    float qd = q_row[d];
                    const float *kt_row = kt + d * bc_used;
                    for (size_t c = 0; c < bc_used; c++) s_row[c] += qd * kt_row[c];
                }
                for (size_t c = 0; c < bc_used; c++) s_row[c] *= scale;
            }
            /* mask -> -inf (:342-352) */
            if (kind != RO_MASK_NONE) {
                for (size_t r = 0; r < br_used; r++)
                    for (size_t c = 0; c < bc_used; c++)
                        if (ro_mask_is_masked(kind, keep, keep_n, qi + r, kj + c)) s_buf[r * bc_used + c] = -INFINITY;
            }
            /* per-row online softmax (:355-386) */
            for (size_t r = 0; r < br_used; r++) {
                const float *s_row = s_buf + r * bc_used;
                float m_tile = -INFINITY;
                for (size_t c = 0; c < bc_used; c++)
                    if (s_row[c] > m_tile) m_tile = s_row[c];
                float m_prev = m_buf[r];
                float m_new = m_tile > m_prev ? m_tile : m_prev;
                float alpha = (m_prev == -INFINITY) ? 0.0f : expf(m_prev - m_new);
                if (alpha != 1.0f) {
                    l_buf[r] *= alpha;
                    for (size_t d = 0; d < dim; d++) o_buf[r * dim + d] *= alpha;
                }
                float *p_row = p_buf + r * bc_used;
                float tile_l = 0.0f;
                for (size_t c = 0; c < bc_used; c++) {
                    float p = expf(s_row[c] - m_new);
                    p_row[c] = p;
                    tile_l += p;
                }
                l_buf[r] += tile_l;
                m_buf[r] = m_new;
            }
            /* O += P . V_tile (gemm alpha=1, beta=1; :564-584) */
            for (size_t r = 0; r < br_used; r++) {
                float *o_row = o_buf + r * dim;
                const float *p_row = p_buf + r * bc_used;
                for (size_t c = 0; c < bc_used; c++) {
                    float p = p_row[c];
                    const float *v_row = v + (kj + c) * dim;
                    for (size_t d = 0; d < dim; d++) o_row[d] += p * v_row[d];
                }
            }
        }
        /* normalise or NaN (:405-421) */
        for (size_t r = 0; r < br_used; r++) {
            float *dst = out_slab + (qi + r) * dim;
            float l = l_buf[r];
            if (l > 0.0f && isfinite(l)) {
                float inv_l = 1.0f / l;
                for (size_t d = 0; d < dim; d++) dst[d] = o_buf[r * dim + d] * inv_l;
            } else {
                for (size_t d = 0; d < dim; d++) dst[d] = NAN;
            }
        }
    }
    free(s_buf);
    free(p_buf);
    free(o_buf);
    free(m_buf);
    free(l_buf);
    free(kt);
}

/* ---- cpu_forward.rs:193-242 --------------------------------------------- */
RO_EXPORT int ro_flash_forward_masked(const ro_shape *s, const float *q, size_t qn, const float *k, size_t kn,
                                      const float *v, size_t vn, int mask_kind, const uint8_t *keep, size_t keep_n,
                                      float *out, size_t on, ro_err *err, int threads) {
    int rc = validate(s, qn, kn, vn, on, mask_kind, keep_n, err);
    if (rc) return rc;
    if (s->seq == 0) return RO_OK;
    float scale = 1.0f / sqrtf((float)s->dim);
    size_t s_h = s->seq * s->dim;
    long n_slabs = (long)(s->batch * s->heads);
    if (threads < 1) threads = 1;
    /* one task per (b,h) slab, as rayon's par_chunks_mut(s_h) (:219) */
#pragma omp parallel for schedule(dynamic, 1) num_threads(threads)
    for (long bh = 0; bh < n_slabs; bh++) {
        size_t base = (size_t)bh * s_h;
        flash_bh_tiles(q + base, k + base, v + base, out + base, mask_kind, keep, keep_n, scale, s->seq, s->dim,
                       s->br, s->bc);
    }
    return RO_OK;
}

/* ---- online_softmax.rs:44-151 ------------------------------------------- */
typedef struct {
    float m, l;
} ro_osm_state;

RO_EXPORT void ro_osm_empty(ro_osm_state *st) {
    st->m = -INFINITY;
    st->l = 0.0f;
}
RO_EXPORT void ro_osm_from_scalar(ro_osm_state *st, float x) {
    st->m = x;
    st->l = 1.0f;
}
RO_EXPORT void ro_osm_absorb(ro_osm_state *st, float x) {
    if (x > st->m) {
        st->l = st->l * expf(st->m - x) + 1.0f;
        st->m = x;
    } else {
        st->l += expf(x - st->m);
    }
}
RO_EXPORT int ro_osm_is_empty(const ro_osm_state *st) { return st->m == -INFINITY && st->l == 0.0f; }
RO_EXPORT void ro_osm_combine(const ro_osm_state *a, const ro_osm_state *b, ro_osm_state *r) {
    if (ro_osm_is_empty(a)) {
        *r = *b;
        return;
    }
    if (ro_osm_is_empty(b)) {
        *r = *a;
        return;
    }
    float m_new = a->m > b->m ? a->m : b->m;
    ro_osm_state o;
    o.m = m_new;
    if (a->m == m_new && b->m == m_new)
        o.l = a->l + b->l;
    else if (a->m == m_new)
        o.l = a->l + b->l * expf(b->m - m_new);
    else
        o.l = a->l * expf(a->m - m_new) + b->l;
    *r = o;
}
RO_EXPORT void ro_osm_full(const float *xs, size_t n, ro_osm_state *st) {
    ro_osm_empty(st);
    for (size_t i = 0; i < n; i++) ro_osm_absorb(st, xs[i]);
}

/* ---- cpu_forward.rs:594-686: the row-by-row statement of the same recurrence */
RO_EXPORT int ro_flash_forward_scalar(const ro_shape *s, const float *q, size_t qn, const float *k, size_t kn,
                                      const float *v, size_t vn, int mask_kind, const uint8_t *keep, size_t keep_n,
                                      float *out, size_t on, ro_err *err) {
    int rc = validate(s, qn, kn, vn, on, mask_kind, keep_n, err);
    if (rc) return rc;
    if (s->seq == 0) return RO_OK;
    float scale = 1.0f / sqrtf((float)s->dim);
    size_t seq = s->seq, dim = s->dim, bc = s->bc;
    float *o_row = (float *)malloc(sizeof(float) * dim);
    float *scores = (float *)malloc(sizeof(float) * bc);
    for (size_t bh = 0; bh < s->batch * s->heads; bh++) {
        size_t base = bh * seq * dim;
        for (size_t qi = 0; qi < seq; qi++) {
            ro_osm_state st;
            ro_osm_empty(&st);
            for (size_t d = 0; d < dim; d++) o_row[d] = 0.0f;
            const float *q_row = q + base + qi * dim;
            for (size_t kj = 0; kj < seq; kj += bc) {
                size_t kj_end = kj + bc < seq ? kj + bc : seq;
                size_t bc_used = kj_end - kj;
                for (size_t kk = kj; kk < kj_end; kk++) {
                    const float *k_row = k + base + kk * dim;
                    float acc = 0.0f;
                    for (size_t d = 0; d < dim; d++) acc += q_row[d] * k_row[d];
                    scores[kk - kj] =
                        ro_mask_is_masked(mask_kind, keep, keep_n, qi, kk) ? -INFINITY : acc * scale;
                }
                float m_tile = -INFINITY;
                for (size_t c = 0; c < bc_used; c++) m_tile = fmaxf(m_tile, scores[c]);
                float m_comb = m_tile > st.m ? m_tile : st.m;
                float alpha = (st.m == -INFINITY) ? 0.0f : expf(st.m - m_comb);
                if (alpha != 1.0f) {
                    st.l *= alpha;
                    for (size_t d = 0; d < dim; d++) o_row[d] *= alpha;
                }
                float tile_l = 0.0f;
                for (size_t c = 0; c < bc_used; c++) {
                    float p = expf(scores[c] - m_comb);
                    tile_l += p;
                    const float *v_row = v + base + (kj + c) * dim;
                    for (size_t d = 0; d < dim; d++) o_row[d] += p * v_row[d];
                }
                st.l += tile_l;
                st.m = m_comb;
            }
            float *dst = out + base + qi * dim;
            if (st.l > 0.0f && isfinite(st.l)) {
                for (size_t d = 0; d < dim; d++) dst[d] = o_row[d] / st.l;
            } else {
                for (size_t d = 0; d < dim; d++) dst[d] = NAN;
            }
        }
    }
    free(o_row);
    free(scores);
    return RO_OK;
}

/* ---- cpu_forward.rs:702-763 --------------------------------------------- */
RO_EXPORT int ro_naive_forward_masked(const ro_shape *s, const float *q, size_t qn, const float *k, size_t kn,
                                      const float *v, size_t vn, int mask_kind, const uint8_t *keep, size_t keep_n,
                                      float *out, size_t on, ro_err *err) {
    int rc = validate(s, qn, kn, vn, on, mask_kind, keep_n, err);
    if (rc) return rc;
    float scale = 1.0f / sqrtf((float)s->dim);
    size_t seq = s->seq, dim = s->dim;
    float *scores = (float *)malloc(sizeof(float) * (seq * seq + 1));
    for (size_t bh = 0; bh < s->batch * s->heads; bh++) {
        size_t base = bh * seq * dim;
        for (size_t i = 0; i < seq; i++)
            for (size_t j = 0; j < seq; j++) {
                if (ro_mask_is_masked(mask_kind, keep, keep_n, i, j)) {
                    scores[i * seq + j] = -INFINITY;
                    continue;
                }
                float acc = 0.0f;
                for (size_t d = 0; d < dim; d++) acc += q[base + i * dim + d] * k[base + j * dim + d];
                scores[i * seq + j] = acc * scale;
            }
        for (size_t i = 0; i < seq; i++) {
            float *row = scores + i * seq;
            float m = -INFINITY;
            for (size_t j = 0; j < seq; j++) m = fmaxf(m, row[j]);
            float sum = 0.0f;
            for (size_t j = 0; j < seq; j++) {
                row[j] = expf(row[j] - m);
                sum += row[j];
            }
            float *dst = out + base + i * dim;
            if (sum > 0.0f && isfinite(sum)) {
                for (size_t j = 0; j < seq; j++) row[j] /= sum;
                for (size_t d = 0; d < dim; d++) {
                    float o = 0.0f;
                    for (size_t j = 0; j < seq; j++) o += row[j] * v[base + j * dim + d];
                    dst[d] = o;
                }
            } else {
                for (size_t d = 0; d < dim; d++) dst[d] = NAN;
            }
        }
    }
    free(scores);
    return RO_OK;
}

/* ---- gqa.rs:216-270 ----------------------------------------------------- */
static void decode_attn_row(size_t bh_idx, const float *q, const float *k, const float *v, float *out_block,
                            size_t n_heads, size_t n_kv_heads, size_t seq_q, size_t seq_kv, size_t head_dim,
                            float scale, size_t group_size) {
    size_t b = bh_idx / n_heads, h = bh_idx % n_heads, kv_h = h / group_size;
    const float *q_block = q + b * n_heads * seq_q * head_dim + h * seq_q * head_dim;
    size_t kv_off = b * n_kv_heads * seq_kv * head_dim + kv_h * seq_kv * head_dim;
    const float *k_block = k + kv_off, *v_block = v + kv_off;
    float *scores = (float *)malloc(sizeof(float) * (seq_kv + 1));
    for (size_t q_pos = 0; q_pos < seq_q; q_pos++) {
        const float *q_row = q_block + q_pos * head_dim;
        for (size_t k_pos = 0; k_pos < seq_kv; k_pos++) {
            const float *k_row = k_block + k_pos * head_dim;
            float acc = 0.0f;
            for (size_t d = 0; d < head_dim; d++) acc += q_row[d] * k_row[d];
            scores[k_pos] = acc * scale;
        }
        float max_s = -INFINITY;
        for (size_t t = 0; t < seq_kv; t++) max_s = fmaxf(max_s, scores[t]);
        float sum_exp = 0.0f;
        for (size_t t = 0; t < seq_kv; t++) {
            scores[t] = expf(scores[t] - max_s);
            sum_exp += scores[t];
        }
        float inv_sum = 1.0f / sum_exp;
        for (size_t t = 0; t < seq_kv; t++) scores[t] *= inv_sum;
        float *out_row = out_block + q_pos * head_dim;
        for (size_t d = 0; d < head_dim; d++) out_row[d] = 0.0f;
        for (size_t t = 0; t < seq_kv; t++) {
            const float *v_row = v_block + t * head_dim;
            float w = scores[t];
            for (size_t d = 0; d < head_dim; d++) out_row[d] += w * v_row[d];
        }
    }
    free(scores);
}

/* ---- gqa.rs:94-210 ------------------------------------------------------ */
RO_EXPORT int ro_gqa_forward_f32(const float *q, size_t qn, const float *k, size_t kn, const float *v, size_t vn,
                                 float *out, size_t on, size_t batch, size_t n_heads, size_t n_kv_heads,
                                 size_t seq_q, size_t seq_kv, size_t head_dim, ro_err *err, int threads) {
    if (n_kv_heads == 0 || n_heads % n_kv_heads != 0) {
        set_err(err, -1, n_heads, n_kv_heads);
        return RO_ERR_HEAD_COUNT_MISMATCH;
    }
    size_t q_len = batch * n_heads * seq_q * head_dim;
    size_t kv_len = batch * n_kv_heads * seq_kv * head_dim;
    if (qn != q_len) return set_err(err, RO_WHICH_Q, q_len, qn), RO_ERR_WRONG_INPUT_LEN;
    if (kn != kv_len) return set_err(err, RO_WHICH_K, kv_len, kn), RO_ERR_WRONG_INPUT_LEN;
    if (vn != kv_len) return set_err(err, RO_WHICH_V, kv_len, vn), RO_ERR_WRONG_INPUT_LEN;
    if (on != q_len) return set_err(err, RO_WHICH_OUT, q_len, on), RO_ERR_WRONG_INPUT_LEN;
    size_t group_size = n_heads / n_kv_heads;

    if (seq_q == seq_kv) {
        /* prefill: replicate K/V to n_heads, then unmasked flash (:151-177) */
        size_t kv_h_size = seq_kv * head_dim, kv_block = batch * n_heads * kv_h_size;
        float *k_rep = (float *)malloc(sizeof(float) * (kv_block + 1));
        float *v_rep = (float *)malloc(sizeof(float) * (kv_block + 1));
        for (size_t b = 0; b < batch; b++)
            for (size_t h = 0; h < n_heads; h++) {
                size_t kv_h = h / group_size;
                size_t src = b * n_kv_heads * kv_h_size + kv_h * kv_h_size;
                size_t dst = b * n_heads * kv_h_size + h * kv_h_size;
                memcpy(k_rep + dst, k + src, sizeof(float) * kv_h_size);
                memcpy(v_rep + dst, v + src, sizeof(float) * kv_h_size);
            }
        ro_shape s = {batch, n_heads, seq_q, head_dim, 64, 64};
        int rc = ro_flash_forward_masked(&s, q, qn, k_rep, kv_block, v_rep, kv_block, RO_MASK_NONE, NULL, 0, out, on,
                                         NULL, threads);
        free(k_rep);
        free(v_rep);
        if (rc) {
            /* any flash error is reported as WrongInputLen{which:"flash_forward",0,0} (:171-175) */
            set_err(err, RO_WHICH_FLASH, 0, 0);
            return RO_ERR_WRONG_INPUT_LEN;
        }
        return RO_OK;
    }
    float scale = 1.0f / sqrtf((float)head_dim);
    long n = (long)(batch * n_heads);
    if (seq_q == 1 || threads <= 1) {
        /* single-thread loop for seq_q == 1 (:190-198) */
        for (long i = 0; i < n; i++)
            decode_attn_row((size_t)i, q, k, v, out + (size_t)i * seq_q * head_dim, n_heads, n_kv_heads, seq_q,
                            seq_kv, head_dim, scale, group_size);
        return RO_OK;
    }
#pragma omp parallel for schedule(dynamic, 1) num_threads(threads)
    for (long i = 0; i < n; i++)
        decode_attn_row((size_t)i, q, k, v, out + (size_t)i * seq_q * head_dim, n_heads, n_kv_heads, seq_q, seq_kv,
                        head_dim, scale, group_size);
    return RO_OK;
}

/* ---- kv_cache.rs:77-112: append [B,H,s_new,D] at current_len into [B,H,max_seq,D] */
RO_EXPORT int ro_kv_cache_append(float *k_cache, float *v_cache, size_t batch, size_t n_heads, size_t max_seq,
                                 size_t head_dim, size_t current_len, size_t seq_added, const float *new_k,
                                 size_t nk, const float *new_v, size_t nv, ro_err *err) {
    if (current_len + seq_added > max_seq) {
        set_err(err, -1, max_seq, current_len + seq_added);
        return RO_ERR_KV_OVERFLOW;
    }
    size_t bhsd = batch * n_heads * seq_added * head_dim;
    if (nk != bhsd || nv != bhsd) {
        set_err(err, -1, bhsd, nk);
        if (err) err->got2 = nv;
        return RO_ERR_KV_WRONG_INPUT_LEN;
    }
    for (size_t b = 0; b < batch; b++)
        for (size_t h = 0; h < n_heads; h++) {
            size_t src = b * n_heads * seq_added * head_dim + h * seq_added * head_dim;
            size_t dst = b * n_heads * max_seq * head_dim + h * max_seq * head_dim + current_len * head_dim;
            memcpy(k_cache + dst, new_k + src, sizeof(float) * seq_added * head_dim);
            memcpy(v_cache + dst, new_v + src, sizeof(float) * seq_added * head_dim);
        }
    return RO_OK;
}

/* ---- model.rs:638-650: copy the valid prefix [..kv_len] of every head out of the
 * [H,max_seq,D] slab into a contiguous [H,kv_len,D] buffer */
RO_EXPORT void ro_kv_trim(const float *cache, float *trimmed, size_t n_kv_heads, size_t max_seq, size_t kv_len,
                          size_t head_dim) {
    for (size_t h = 0; h < n_kv_heads; h++)
        memcpy(trimmed + h * kv_len * head_dim, cache + h * max_seq * head_dim, sizeof(float) * kv_len * head_dim);
}

/* ---- bf16 <-> f32, round to nearest even (half 2.7.1 bf16::from_f32) ------ */
RO_EXPORT uint16_t ro_f32_to_bf16(float x) {
    uint32_t u;
    memcpy(&u, &x, 4);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u); /* NaN stays NaN (quiet) */
    uint32_t round_bit = 0x00008000u;
    if ((u & round_bit) != 0 && (u & (3 * round_bit - 1)) != 0) return (uint16_t)((u >> 16) + 1);
    return (uint16_t)(u >> 16);
}
RO_EXPORT float ro_bf16_to_f32(uint16_t h) {
    uint32_t u = (uint32_t)h << 16;
    float f;
    memcpy(&f, &u, 4);
    return f;
}
RO_EXPORT void ro_f32_to_bf16_array(const float *x, uint16_t *y, size_t n) {
    for (size_t i = 0; i < n; i++) y[i] = ro_f32_to_bf16(x[i]);
}
RO_EXPORT void ro_bf16_to_f32_array(const uint16_t *x, float *y, size_t n) {
    for (size_t i = 0; i < n; i++) y[i] = ro_bf16_to_f32(x[i]);
}

/* ---- llm_kernels.rs:353-372 --------------------------------------------- */
RO_EXPORT void ro_kv_append_bf16(uint16_t *k_cache, uint16_t *v_cache, const uint16_t *k_in, const uint16_t *v_in,
                                 int pos, int n_kv, int head_dim, int max_seq) {
    for (int kv_h = 0; kv_h < n_kv; kv_h++)
        for (int i = 0; i < head_dim; i++) {
            size_t cache_off = (size_t)kv_h * max_seq * head_dim + (size_t)pos * head_dim + i;
            size_t in_off = (size_t)kv_h * head_dim + i;
            k_cache[cache_off] = k_in[in_off];
            v_cache[cache_off] = v_in[in_off];
        }
}

/* ---- llm_kernels.rs:396-457: one pass, f32 state (m=-1e30, l, o), bf16 in/out.
 * The block-wide tree reduction of the dot product is restated as an
 * ascending f32 sum. */
RO_EXPORT void ro_gqa_decode_online_bf16(const uint16_t *q, const uint16_t *k_cache, const uint16_t *v_cache,
                                         uint16_t *out, int n_heads, int n_kv, int kv_len, int head_dim,
                                         int max_seq) {
    float scale = 1.0f / sqrtf((float)head_dim);
    float *o = (float *)malloc(sizeof(float) * head_dim);
    for (int h = 0; h < n_heads; h++) {
        int kv_h = h * n_kv / n_heads;
        float m = -1e30f, l = 0.0f;
        for (int i = 0; i < head_dim; i++) o[i] = 0.0f;
        for (int t = 0; t < kv_len; t++) {
            size_t row = ((size_t)kv_h * max_seq + t) * head_dim;
            float dot = 0.0f;
            for (int i = 0; i < head_dim; i++)
                dot += ro_bf16_to_f32(q[(size_t)h * head_dim + i]) * ro_bf16_to_f32(k_cache[row + i]);
            float s_t = dot * scale;
            float new_m = fmaxf(m, s_t);
            float correction = expf(m - new_m);
            float p = expf(s_t - new_m);
            for (int i = 0; i < head_dim; i++) o[i] = o[i] * correction + p * ro_bf16_to_f32(v_cache[row + i]);
            l = l * correction + p;
            m = new_m;
        }
        for (int i = 0; i < head_dim; i++) out[(size_t)h * head_dim + i] = ro_f32_to_bf16(o[i] / fmaxf(l, 1e-12f));
    }
    free(o);
}

/* ---- Batched, ragged decode: the CPU path (model.rs:638-668 trim + gqa.rs
 * decode_attn_row) applied per sequence b with its own kv_len, in f32 on
 * bf16-rounded inputs.  q [B,Hq,D] bf16, caches [B,Hkv,max_seq,D] bf16,
 * out [B,Hq,D] f32.  kv_len == 0 gives a row of zeros: gqa.rs:260-261 fills the row with 0
 * and the key loop is empty (the bf16 kernel's o / fmaxf(l, 1e-12f) gives the same). */
RO_EXPORT void ro_gqa_decode_batched_bf16(const uint16_t *q, const uint16_t *k_cache, const uint16_t *v_cache,
                                          const int32_t *kv_lens, float *out, int batch, int n_heads, int n_kv,
                                          int head_dim, int max_seq, int threads) {
    size_t group = (size_t)n_heads / n_kv;
    float scale = 1.0f / sqrtf((float)head_dim);
    if (threads < 1) threads = 1;
    long n_tasks = (long)batch * n_kv;
#pragma omp parallel for schedule(dynamic, 1) num_threads(threads)
    for (long task = 0; task < n_tasks; task++) {
        size_t b = (size_t)task / n_kv, kv_h = (size_t)task % n_kv;
        size_t kv_len = (size_t)kv_lens[b];
        size_t D = (size_t)head_dim;
        float *kf = (float *)malloc(sizeof(float) * (kv_len * D + 1));
        float *vf = (float *)malloc(sizeof(float) * (kv_len * D + 1));
        float *qf = (float *)malloc(sizeof(float) * D);
        size_t base = (b * n_kv + kv_h) * (size_t)max_seq * D;
        ro_bf16_to_f32_array(k_cache + base, kf, kv_len * D);
        ro_bf16_to_f32_array(v_cache + base, vf, kv_len * D);
        for (size_t g = 0; g < group; g++) {
            size_t h = kv_h * group + g;
            ro_bf16_to_f32_array(q + (b * n_heads + h) * D, qf, D);
            /* a 1-batch, 1-head, 1-kv-head call of the row kernel on the trimmed prefix */
            decode_attn_row(0, qf, kf, vf, out + (b * n_heads + h) * D, 1, 1, 1, kv_len, D, scale, 1);
        }
        free(kf);
        free(vf);
        free(qf);
    }
}

/* ---- gqa_decode_batched_f32 (crates/rustorch-metal/src/kernels.rs:14432-14516), per sequence of a batch.
 * Query position s (0 <= s < seq_new) of sequence b sits at absolute position pos_base_b + s with
 * pos_base_b = kv_lens[b] - seq_new and attends to keys [0, pos_base_b + s] (kv_len = pos_base + b + 1 in the
 * shader).  Phases as in the shader: scores = dot * inv_sqrt_d; max; e = exp(score - max); sum; weights =
 * e * (1 / sum); out[d] = sum_p weights[p] * v[p][d] in ascending p.  q/out [B,seq_new,Hq,D] (position-major, the
 * shader's q + b * n_heads * head_dim + q_h * head_dim), caches [B,Hkv,max_seq,D]; kv head = q_h / (Hq / Hkv).
 * bf16 bit patterns in, f32 out.  A position with no visible key (kv_lens[b] - seq_new + s < 0; cannot happen in
 * the reference, whose kv_len is at least 1) runs every loop of the shader zero times: inv_sum = 1/0 is formed but
 * never multiplied into anything, and phase D writes acc = 0.0 -- a row of zeros, the same outcome as
 * decode_attn_row's and the CUDA kernel's for an empty context (gqa.rs:260-261, llm_kernels.rs:456). */
RO_EXPORT void ro_gqa_decode_chunk_bf16(const uint16_t *q, const uint16_t *k_cache, const uint16_t *v_cache,
                                        const int32_t *kv_lens, float *out, int batch, int seq_new, int n_heads,
                                        int n_kv, int head_dim, int max_seq, int threads) {
    const size_t D = (size_t)head_dim, group = (size_t)n_heads / n_kv;
    const float inv_sqrt_d = 1.0f / sqrtf((float)head_dim);
    if (threads < 1) threads = 1;
    long n_tasks = (long)batch * n_heads;
#pragma omp parallel for schedule(dynamic, 1) num_threads(threads)
    for (long task = 0; task < n_tasks; task++) {
        const size_t b = (size_t)task / n_heads, q_h = (size_t)task % n_heads, kv_h = q_h / group;
        const long pos_base = (long)kv_lens[b] - seq_new;
        const uint16_t *kb = k_cache + (b * n_kv + kv_h) * (size_t)max_seq * D;
        const uint16_t *vb = v_cache + (b * n_kv + kv_h) * (size_t)max_seq * D;
        float *shared = (float *)malloc(sizeof(float) * ((size_t)max_seq + 1));
        for (int s = 0; s < seq_new; s++) {
            const uint16_t *qp = q + ((b * seq_new + s) * n_heads + q_h) * D;
            float *op = out + ((b * seq_new + s) * n_heads + q_h) * D;
            long kv_len = pos_base + s + 1;
            if (kv_len > max_seq) kv_len = max_seq;
            if (kv_len <= 0) {
                for (size_t d = 0; d < D; d++) op[d] = 0.0f;
                continue;
            }
            float max_score = -INFINITY;
            for (long p = 0; p < kv_len; p++) {
                float dot = 0.0f;
                for (size_t d = 0; d < D; d++) dot += ro_bf16_to_f32(qp[d]) * ro_bf16_to_f32(kb[(size_t)p * D + d]);
                shared[p] = dot * inv_sqrt_d;
                if (shared[p] > max_score) max_score = shared[p];
            }
            float sum = 0.0f;
            for (long p = 0; p < kv_len; p++) {
                shared[p] = expf(shared[p] - max_score);
                sum += shared[p];
            }
            const float inv_sum = 1.0f / sum;
            for (long p = 0; p < kv_len; p++) shared[p] *= inv_sum;
            for (size_t d = 0; d < D; d++) {
                float acc = 0.0f;
                for (long p = 0; p < kv_len; p++) acc += shared[p] * ro_bf16_to_f32(vb[(size_t)p * D + d]);
                op[d] = acc;
            }
        }
        free(shared);
    }
}

RO_EXPORT int ro_max_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}


/* ---- RoPE and per-head RMSNorm: the steps between the QKV projection and decode attention ------------- */

/* RoPE::new (rope.rs:63-90): theta_k = 1 / base^(2k / head_dim), angle = p * theta_k, all in f32. */
RO_EXPORT void ro_rope_tables(int head_dim, int max_seq, float base, float *cos_t, float *sin_t) {
    const int half = head_dim / 2;
    for (int p = 0; p < max_seq; p++)
        for (int k = 0; k < half; k++) {
            float inv_theta = 1.0f / powf(base, (float)(2 * k) / (float)head_dim);
            float angle = (float)p * inv_theta;
            cos_t[(size_t)p * half + k] = cosf(angle);
            sin_t[(size_t)p * half + k] = sinf(angle);
        }
}

static int rope_check(size_t x_len, size_t batch, size_t n_heads, size_t seq, size_t d, size_t position_offset,
                      size_t table_rows, ro_err *err) {
    size_t expected = batch * n_heads * seq * d;
    if (x_len != expected) { /* rope.rs:173-178 */
        set_err(err, -1, expected, x_len);
        return RO_ERR_ROPE_WRONG_INPUT_LEN;
    }
    if (position_offset + seq > table_rows) { /* rope.rs:179-184: expected = max_seq, got = requested */
        set_err(err, -1, table_rows, position_offset + seq);
        return RO_ERR_ROPE_POSITION_OVERFLOW;
    }
    return RO_OK;
}

/* apply_inplace_half_split (rope.rs:162-205): dim k pairs with dim k + D/2. */
RO_EXPORT int ro_rope_half_split(float *x, size_t x_len, size_t batch, size_t n_heads, size_t seq, size_t head_dim,
                                 size_t position_offset, const float *cos_t, const float *sin_t, size_t table_rows,
                                 ro_err *err) {
    int rc = rope_check(x_len, batch, n_heads, seq, head_dim, position_offset, table_rows, err);
    if (rc != RO_OK) return rc;
    const size_t d = head_dim, half = d / 2;
    for (size_t b = 0; b < batch; b++)
        for (size_t h = 0; h < n_heads; h++)
            for (size_t s = 0; s < seq; s++) {
                size_t p = position_offset + s;
                size_t row_off = b * n_heads * seq * d + h * seq * d + s * d;
                size_t table_off = p * half;
                for (size_t k = 0; k < half; k++) {
                    float c = cos_t[table_off + k], si = sin_t[table_off + k];
                    float x0 = x[row_off + k], x1 = x[row_off + k + half];
                    x[row_off + k] = x0 * c - x1 * si;
                    x[row_off + k + half] = x1 * c + x0 * si;
                }
            }
    return RO_OK;
}

/* apply_inplace (rope.rs:96-142): pairs (2k, 2k+1). */
RO_EXPORT int ro_rope_interleaved(float *x, size_t x_len, size_t batch, size_t n_heads, size_t seq, size_t head_dim,
                                  size_t position_offset, const float *cos_t, const float *sin_t, size_t table_rows,
                                  ro_err *err) {
    int rc = rope_check(x_len, batch, n_heads, seq, head_dim, position_offset, table_rows, err);
    if (rc != RO_OK) return rc;
    const size_t d = head_dim, half = d / 2;
    for (size_t b = 0; b < batch; b++)
        for (size_t h = 0; h < n_heads; h++)
            for (size_t s = 0; s < seq; s++) {
                size_t p = position_offset + s;
                size_t row_off = b * n_heads * seq * d + h * seq * d + s * d;
                size_t table_off = p * half;
                for (size_t k = 0; k < half; k++) {
                    float c = cos_t[table_off + k], si = sin_t[table_off + k];
                    float x0 = x[row_off + 2 * k], x1 = x[row_off + 2 * k + 1];
                    x[row_off + 2 * k] = x0 * c - x1 * si;
                    x[row_off + 2 * k + 1] = x0 * si + x1 * c;
                }
            }
    return RO_OK;
}

/* rms_norm_inplace (model.rs:862-885, default convention) on one head. */
static void rms_norm_head(float *x, const float *gamma, size_t d, float eps) {
    float inv_d = 1.0f / (float)d;
    float sq = 0.0f;
    for (size_t i = 0; i < d; i++) sq += x[i] * x[i];
    float inv_rms = 1.0f / sqrtf(sq * inv_d + eps);
    for (size_t i = 0; i < d; i++) x[i] = x[i] * inv_rms * gamma[i];
}

/* rms_norm_per_head (model.rs:890-897): gamma [head_dim] shared by the heads. */
RO_EXPORT void ro_rms_norm_per_head(float *x, const float *gamma, size_t n_heads, size_t head_dim, float eps) {
    for (size_t h = 0; h < n_heads; h++) rms_norm_head(x + h * head_dim, gamma, head_dim, eps);
}

/* Steps 2a, 2b and 3 of decode_step (model.rs:575-636) for a batch of sequences with `seq` new tokens each, on bf16
 * storage: every value is widened to f32, normalised per head (when a gamma is given), rotated (half-split) at
 * position positions[b] + s (rope.rs:192-193) and rounded to bf16 once; q [batch, n_heads, seq, head_dim] is
 * rewritten in place, k and v [batch, n_kv, seq, head_dim] go to rows positions[b] .. + seq - 1 of the caches
 * [batch, n_kv, max_seq, head_dim] (KVLayerCache::append, kv_cache.rs:97-110; for seq == 1 the index rule of
 * kv_append_bf16, llm_kernels.rs:353-372).  Every sequence must satisfy 0 <= p and p + seq <= min(max_seq,
 * table_rows); returns the overflow error otherwise, having written nothing. */
RO_EXPORT int ro_decode_prepare_bf16(uint16_t *q, const uint16_t *k_in, const uint16_t *v_in, uint16_t *k_cache,
                                     uint16_t *v_cache, const int32_t *positions, const float *q_gamma,
                                     const float *k_gamma, float eps, const float *cos_t, const float *sin_t, int batch,
                                     int seq, int n_heads, int n_kv, int head_dim, int max_seq, int table_rows,
                                     ro_err *err) {
    const size_t d = (size_t)head_dim;
    for (int b = 0; b < batch; b++) {
        int64_t p = positions[b];
        if (p < 0 || p + seq > table_rows) { /* rope.rs:179-184 */
            set_err(err, -1, (uint64_t)table_rows, (uint64_t)(p + seq));
            return RO_ERR_ROPE_POSITION_OVERFLOW;
        }
        if (p + seq > max_seq) { /* kv_cache.rs:84-89 */
            set_err(err, -1, (uint64_t)max_seq, (uint64_t)(p + seq));
            return RO_ERR_KV_OVERFLOW;
        }
    }
    float *row = (float *)malloc(d * sizeof(float));
    if (!row) return -1;
    ro_err e2;
    for (int b = 0; b < batch; b++)
        for (int h = 0; h < n_heads + n_kv; h++)
            for (int s = 0; s < seq; s++) {
                const size_t p = (size_t)positions[b] + (size_t)s;
                const int is_q = h < n_heads;
                const int kvh = h - n_heads;
                uint16_t *src = is_q ? q + (((size_t)b * n_heads + h) * seq + s) * d
                                     : (uint16_t *)k_in + (((size_t)b * n_kv + kvh) * seq + s) * d;
                const float *gamma = is_q ? q_gamma : k_gamma;
                for (size_t i = 0; i < d; i++) row[i] = ro_bf16_to_f32(src[i]);
                if (gamma) rms_norm_head(row, gamma, d, eps);
                ro_rope_half_split(row, d, 1, 1, 1, d, p, cos_t, sin_t, (size_t)table_rows, &e2);
                if (is_q) {
                    for (size_t i = 0; i < d; i++) src[i] = ro_f32_to_bf16(row[i]);
                } else {
                    const size_t off = (((size_t)b * n_kv + kvh) * (size_t)max_seq + p) * d;
                    const uint16_t *vs = v_in + (((size_t)b * n_kv + kvh) * seq + s) * d;
                    for (size_t i = 0; i < d; i++) {
                        k_cache[off + i] = ro_f32_to_bf16(row[i]);
                        v_cache[off + i] = vs[i];
                    }
                }
            }
    free(row);
    return RO_OK;
}


/* ---- MultiHeadAttention's composed path: additive masks, row softmax, the two batched products ---------------- */

#define RO_MASK_NEG (-1.0e4f) /* masks.rs:22 */

/* causal_mask (masks.rs:30-40) */
RO_EXPORT void ro_causal_mask(size_t seq_len, float *out) {
    for (size_t i = 0; i < seq_len; i++)
        for (size_t j = 0; j < seq_len; j++) out[i * seq_len + j] = (j > i) ? RO_MASK_NEG : 0.0f;
}

/* sliding_window_mask (masks.rs:52-65); window >= 1 is the caller's to guarantee (an assert there) */
RO_EXPORT void ro_sliding_window_mask(size_t seq_len, size_t window, float *out) {
    for (size_t i = 0; i < seq_len; i++)
        for (size_t j = 0; j < seq_len; j++) {
            int inside_causal = j <= i;
            size_t back = i >= j ? i - j : 0; /* saturating_sub */
            int inside_window = back < window;
            out[i * seq_len + j] = (inside_causal && inside_window) ? 0.0f : RO_MASK_NEG;
        }
}

/* bool_to_additive (masks.rs:73-82) */
RO_EXPORT void ro_bool_to_additive(const float *mask, float *out, size_t n) {
    for (size_t i = 0; i < n; i++) out[i] = (mask[i] >= 0.5f) ? 0.0f : RO_MASK_NEG;
}

/* softmax_row_online_f32 (softmax.rs:146-180), the non-log form */
RO_EXPORT void ro_softmax_row(const float *row_in, float *row_out, size_t n) {
    if (n == 0) return;
    float mx = -INFINITY, sum = 0.0f;
    for (size_t i = 0; i < n; i++) {
        float x = row_in[i];
        if (x > mx) {
            sum *= expf(mx - x);
            mx = x;
        }
        sum += expf(x - mx);
    }
    float inv_sum = 1.0f / sum;
    for (size_t i = 0; i < n; i++) row_out[i] = expf(row_in[i] - mx) * inv_sum;
}

/* Steps 2-8 of MultiHeadAttention::forward's composed path (attention.rs:371-399) on the projected tensors
 * q [batch, t_q, heads*hd], k, v [batch, t_kv, heads*hd]: per (b, h) raw = Q.K^T (the two bmm calls go to the `gemm`
 * crate, restated as ascending-order f32 sums), scores = raw * (1/sqrt(hd)), + mask (broadcast over the leading
 * batch*heads axis when mask_bh_stride == 0), softmax over the last axis, context = attn.V, heads merged back.
 * mask may be NULL. */
RO_EXPORT void ro_mha_forward_masked(const float *q, const float *k, const float *v, const float *mask,
                                     size_t mask_bh_stride, float *out, size_t batch, size_t t_q, size_t t_kv,
                                     size_t heads, size_t hd) {
    const size_t e = heads * hd;
    const float inv_scale = 1.0f / sqrtf((float)hd);
    float *scores = (float *)malloc((t_kv ? t_kv : 1) * sizeof(float));
    float *attn = (float *)malloc((t_kv ? t_kv : 1) * sizeof(float));
    for (size_t b = 0; b < batch; b++)
        for (size_t h = 0; h < heads; h++)
            for (size_t i = 0; i < t_q; i++) {
                const float *qr = q + (b * t_q + i) * e + h * hd;
                const float *mrow = mask ? mask + (b * heads + h) * mask_bh_stride + i * t_kv : NULL;
                for (size_t j = 0; j < t_kv; j++) {
                    const float *kr = k + (b * t_kv + j) * e + h * hd;
                    float dot = 0.0f;
                    for (size_t d = 0; d < hd; d++) dot += qr[d] * kr[d];
                    float s = dot * inv_scale;
                    if (mrow) s = s + mrow[j];
                    scores[j] = s;
                }
                ro_softmax_row(scores, attn, t_kv);
                float *o = out + (b * t_q + i) * e + h * hd;
                for (size_t d = 0; d < hd; d++) {
                    float acc = 0.0f;
                    for (size_t j = 0; j < t_kv; j++) acc += attn[j] * v[(b * t_kv + j) * e + h * hd + d];
                    o[d] = acc;
                }
            }
    free(scores);
    free(attn);
}

/* ---- cpu_backward.rs:46-185 ----------------------------------------------
 * (dQ, dK, dV) of unmasked attention from Q, K, V and the upstream gradient
 * dO.  P is recomputed per (b,h) as a full seq x seq matrix, exactly as the
 * reference does; every sum runs in the reference's loop order.  The length
 * checks come first and in the reference's order (q, k, v, "do", then the
 * three outputs with got = the longest); seq == 0 returns before anything is
 * written. */
RO_EXPORT int ro_flash_backward(const ro_shape *s, const float *q, size_t qn, const float *k, size_t kn,
                                const float *v, size_t vn, const float *d_out, size_t don, float *dq, size_t dqn,
                                float *dk, size_t dkn, float *dv, size_t dvn, ro_err *err) {
    const size_t n = s->seq, d = s->dim;
    const uint64_t expected = s->batch * s->heads * s->seq * s->dim;
    const size_t lens[4] = {qn, kn, vn, don};
    const int which[4] = {RO_WHICH_Q, RO_WHICH_K, RO_WHICH_V, RO_WHICH_DO};
    for (int i = 0; i < 4; i++)
        if (lens[i] != expected) {
            set_err(err, which[i], expected, lens[i]);
            return RO_ERR_BUFFER_SHAPE_MISMATCH;
        }
    if (dqn != expected || dkn != expected || dvn != expected) {
        size_t got = dqn > dkn ? dqn : dkn;
        if (dvn > got) got = dvn;
        set_err(err, RO_WHICH_OUT, expected, got);
        return RO_ERR_OUTPUT_SHAPE_MISMATCH;
    }
    if (n == 0) return RO_OK;
    const float scale = 1.0f / sqrtf((float)d);
    for (size_t i = 0; i < expected; i++) dq[i] = dk[i] = dv[i] = 0.0f;
    float *p = (float *)malloc(sizeof(float) * n * n);
    float *dp = (float *)malloc(sizeof(float) * n * n);
    float *ds = (float *)malloc(sizeof(float) * n * n);
    for (size_t bh = 0; bh < s->batch * s->heads; bh++) {
        const size_t base = bh * n * d;
        for (size_t i = 0; i < n; i++) {
            float row_max = -INFINITY;
            const float *qi = q + base + i * d;
            for (size_t j = 0; j < n; j++) {
                const float *kj = k + base + j * d;
                float acc = 0.0f;
                for (size_t t = 0; t < d; t++) acc += qi[t] * kj[t];
                float scaled = acc * scale;
                p[i * n + j] = scaled;
                if (scaled > row_max) row_max = scaled;
            }
            float row_sum = 0.0f;
            for (size_t j = 0; j < n; j++) {
                float e = expf(p[i * n + j] - row_max);
                p[i * n + j] = e;
                row_sum += e;
            }
            if (row_sum > 0.0f && isfinite(row_sum))
                for (size_t j = 0; j < n; j++) p[i * n + j] /= row_sum;
        }
        for (size_t j = 0; j < n; j++) {
            float *dvj = dv + base + j * d;
            for (size_t i = 0; i < n; i++) {
                const float pij = p[i * n + j];
                const float *doi = d_out + base + i * d;
                for (size_t t = 0; t < d; t++) dvj[t] += pij * doi[t];
            }
        }
        for (size_t i = 0; i < n; i++) {
            const float *doi = d_out + base + i * d;
            for (size_t j = 0; j < n; j++) {
                const float *vj = v + base + j * d;
                float acc = 0.0f;
                for (size_t t = 0; t < d; t++) acc += doi[t] * vj[t];
                dp[i * n + j] = acc;
            }
        }
        for (size_t i = 0; i < n; i++) {
            float row_dot = 0.0f;
            for (size_t j = 0; j < n; j++) row_dot += p[i * n + j] * dp[i * n + j];
            for (size_t j = 0; j < n; j++) ds[i * n + j] = p[i * n + j] * (dp[i * n + j] - row_dot);
        }
        for (size_t i = 0; i < n; i++) {
            float *dqi = dq + base + i * d;
            for (size_t j = 0; j < n; j++) {
                const float *kj = k + base + j * d;
                const float dsij = ds[i * n + j];
                for (size_t t = 0; t < d; t++) dqi[t] += scale * dsij * kj[t];
            }
        }
        for (size_t j = 0; j < n; j++) {
            float *dkj = dk + base + j * d;
            for (size_t i = 0; i < n; i++) {
                const float *qi = q + base + i * d;
                const float dsij = ds[i * n + j];
                for (size_t t = 0; t < d; t++) dkj[t] += scale * dsij * qi[t];
            }
        }
    }
    free(p);
    free(dp);
    free(ds);
    return RO_OK;
}
