/*
 * rt_attn.h -- C ABI of librt_attn_hip.so, the MI355X (gfx950) attention engine that stands
 * in for rustorch's attention hot path.
 *
 * Every entry point replaces one call surface of the reference (paths relative to the
 * reference checkout) and keeps its argument meaning and its error order.  Plain pointers and
 * sizes only; `stream` is a hipStream_t passed as void* (NULL = the default stream).
 *
 * Host-slice entry points (rt_flash_forward*_f32, rt_gqa_forward_f32) are synchronous, like
 * the Rust functions they replace: they stage the slices to HBM, run the kernels and copy the
 * result back before returning.  Device entry points (*_dev, rt_gqa_decode_*, rt_kv_append_*)
 * take device addresses, enqueue on `stream` and return without synchronising, like the
 * reference's `LlmKernels` launchers.
 *
 * There is no CPU fallback: with no usable gfx950 device every compute entry point returns
 * RT_ERR_NO_DEVICE / RT_ERR_HIP.
 */
#ifndef RT_ATTN_H
#define RT_ATTN_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* AttentionShape -- crates/rustorch-attention/src/cpu_forward.rs:49-89.  Row-major
 * [batch, heads, seq, dim].  br/bc are the reference's CPU tile sizes (64 by default); the
 * GPU kernels choose their own tiling and use bc only to reproduce the reference's result for
 * a padding mask whose first bc keys are all masked (every row NaN, see rt_flash_forward_masked_f32). */
typedef struct rt_attention_shape {
    uint64_t batch;
    uint64_t heads;
    uint64_t seq;
    uint64_t dim;
    uint64_t br;
    uint64_t bc;
} rt_attention_shape;

/* Return codes.  1-4 mirror AttentionError / MaskError (cpu_forward.rs:93-114, mask.rs:70-78),
 * 5-6 GQAError (crates/rustorch-nn/src/gqa.rs:37-55), 7-8 KVCacheError
 * (crates/rustorch-nn/src/kv_cache.rs:229-256); the rest are this library's own. */
enum rt_status {
    RT_OK = 0,
    RT_ERR_ZERO_DIM = 1,                /* AttentionError::ZeroDim */
    RT_ERR_BUFFER_SHAPE_MISMATCH = 2,   /* AttentionError::BufferShapeMismatch{which,expected,got} */
    RT_ERR_OUTPUT_SHAPE_MISMATCH = 3,   /* AttentionError::OutputShapeMismatch{expected,got} */
    RT_ERR_PADDING_LENGTH_MISMATCH = 4, /* AttentionError::Mask(PaddingLengthMismatch{expected,got}) */
    RT_ERR_HEAD_COUNT_MISMATCH = 5,     /* GQAError::HeadCountMismatch{n_heads=expected,n_kv_heads=got} */
    RT_ERR_WRONG_INPUT_LEN = 6,         /* GQAError::WrongInputLen{which,expected,got} */
    RT_ERR_KV_OVERFLOW = 7,             /* KVCacheError::Overflow{requested=got,max=expected} */
    RT_ERR_KV_WRONG_INPUT_LEN = 8,      /* KVCacheError::WrongInputLen{expected,got_k=got,got_v=got2} */
    RT_ERR_ROPE_WRONG_INPUT_LEN = 9,    /* RoPEError::WrongInputLen{expected,got} */
    RT_ERR_ROPE_POSITION_OVERFLOW = 10, /* RoPEError::PositionOverflow{max_seq=expected,requested=got} */
    RT_ERR_NULL_POINTER = 20,
    RT_ERR_UNSUPPORTED = 21,            /* shape outside what the kernels cover; message says which */
    RT_ERR_WORKSPACE_TOO_SMALL = 22,    /* expected = bytes needed, got = bytes given */
    RT_ERR_NO_DEVICE = 30,              /* no HIP device, or the device is not gfx950 */
    RT_ERR_HIP = 31                     /* a HIP call failed; hip_error holds its code */
};

/* Mask -- crates/rustorch-attention/src/mask.rs:26-46. */
enum rt_mask_kind {
    RT_MASK_NONE = 0,
    RT_MASK_CAUSAL = 1, /* masked iff kj > qi */
    RT_MASK_PADDING = 2 /* masked iff !keep[kj]; one keep vector of length seq for all batches/heads */
};

/* `which` of BufferShapeMismatch / WrongInputLen. */
enum rt_which {
    RT_WHICH_Q = 0,
    RT_WHICH_K = 1,
    RT_WHICH_V = 2,
    RT_WHICH_OUT = 3,
    RT_WHICH_FLASH = 4,
    RT_WHICH_MASK = 5,
    RT_WHICH_DO = 6 /* the upstream gradient of rt_flash_backward_f32 */
};

/* Payload of the error enums above.  May be NULL. */
typedef struct rt_err_detail {
    int32_t which; /* rt_which, or -1 */
    uint64_t expected;
    uint64_t got;
    uint64_t got2;
    int32_t hip_error; /* hipError_t when the status is RT_ERR_HIP */
    char message[160];
} rt_err_detail;

/* ---- library ------------------------------------------------------------------------------ */

/* Selects `device`, checks that it is gfx950 and warms the kernels' module.  Optional: every
 * compute entry point does the same lazily on first use (the reference compiles its kernels
 * lazily behind a OnceLock, crates/rustorch-cuda/src/llm_kernels.rs:578-641). */
int rt_init(int device, rt_err_detail *err);
/* Frees what the library keeps between calls (the per-stream scratch of rt_gqa_decode_online_bf16, the pinned
 * staging buffer of the host-slice entries).  Optional; no call may be in flight.  The library stays usable: the
 * buffers come back on demand. */
int rt_shutdown(rt_err_detail *err);
const char *rt_version(void);
const char *rt_status_name(int status);
/* No counterpart in the reference: the path of the HIP runtime library this library is bound to (dladdr of one of its
 * entry points), "" if it cannot be told.  A host that creates streams, events or graphs of its own for the `stream`
 * arguments below must create them in this runtime; a process can hold a second copy of the runtime (PyTorch wheels
 * ship one) and dlopen("libamdhip64.so") may hand back that one. */
const char *rt_hip_runtime_path(void);

/* ---- prefill, host slices ------------------------------------------------------------------- */

/* rustorch_attention::flash_forward -- cpu_forward.rs:175-183. */
int rt_flash_forward_f32(const rt_attention_shape *shape, const float *q, size_t q_len, const float *k,
                         size_t k_len, const float *v, size_t v_len, float *out, size_t out_len,
                         rt_err_detail *err);

/* rustorch_attention::flash_forward_masked -- cpu_forward.rs:193-242.  Check order: ZeroDim,
 * q, k, v lengths, out length, padding length; seq == 0 returns RT_OK without touching `out`.
 * A row with no visible key is NaN (cpu_forward.rs:411-420); with RT_MASK_PADDING, when none of
 * keep[0 .. min(bc, seq)) is set every row is NaN, as the reference's tiled recurrence gives.
 * dim <= 256 (RT_ERR_UNSUPPORTED beyond). */
int rt_flash_forward_masked_f32(const rt_attention_shape *shape, const float *q, size_t q_len, const float *k,
                                size_t k_len, const float *v, size_t v_len, int mask_kind, const uint8_t *keep,
                                size_t keep_len, float *out, size_t out_len, rt_err_detail *err);

/* rustorch_nn::gqa::gqa_forward_f32 -- crates/rustorch-nn/src/gqa.rs:94-210.  q/out
 * [batch,n_heads,seq_q,head_dim], k/v [batch,n_kv_heads,seq_kv,head_dim]; query head h reads kv
 * head h / (n_heads / n_kv_heads).  seq_q == seq_kv runs the unmasked flash forward (without
 * materialising the replicated K/V); otherwise unmasked attention of every query row over all
 * seq_kv keys (the decode branch).  Check order: head counts, then q, k, v, out lengths. */
int rt_gqa_forward_f32(const float *q, size_t q_len, const float *k, size_t k_len, const float *v, size_t v_len,
                       float *out, size_t out_len, size_t batch, size_t n_heads, size_t n_kv_heads, size_t seq_q,
                       size_t seq_kv, size_t head_dim, rt_err_detail *err);

/* gqa_forward_f32 (gqa.rs:94-210) on device-resident f32 tensors, enqueued on `stream`: the head-count check and the
 * same kernels; the tensor lengths cannot be checked. */
int rt_gqa_forward_f32_dev(void *stream, const float *q, const float *k, const float *v, float *out, size_t batch,
                           size_t n_heads, size_t n_kv_heads, size_t seq_q, size_t seq_kv, size_t head_dim,
                           rt_err_detail *err);

/* rustorch_nn::attention::mha_flash_forward_f32 -- crates/rustorch-nn/src/attention.rs:452-495.  q, k, v
 * [batch, seq, heads, head_dim] host slices, out [batch, seq, heads*head_dim]; unmasked attention per
 * (batch, head) with the checks of flash_forward on the shape (batch, heads, seq, head_dim), in its order. */
int rt_mha_flash_forward_f32(const float *q, size_t q_len, const float *k, size_t k_len, const float *v, size_t v_len,
                             float *out, size_t out_len, size_t batch, size_t seq, size_t heads, size_t head_dim,
                             rt_err_detail *err);

/* rustorch_attention::flash_backward -- crates/rustorch-attention/src/cpu_backward.rs:46-185.  (dQ, dK, dV) of
 * unmasked attention from q, k, v and the upstream gradient d_out, all [batch,heads,seq,dim] host slices.
 * Check order: q, k, v, d_out lengths (RT_ERR_BUFFER_SHAPE_MISMATCH, which = q/k/v/do), then the three outputs
 * (RT_ERR_OUTPUT_SHAPE_MISMATCH, got = the longest of them); seq == 0 returns RT_OK without touching the outputs.
 * The outputs are overwritten, not accumulated into.  dim <= 128. */
int rt_flash_backward_f32(const rt_attention_shape *shape, const float *q, size_t q_len, const float *k,
                          size_t k_len, const float *v, size_t v_len, const float *d_out, size_t d_out_len, float *dq,
                          size_t dq_len, float *dk, size_t dk_len, float *dv, size_t dv_len, rt_err_detail *err);

/* ---- prefill, device pointers ---------------------------------------------------------------- */

/* flash_backward (cpu_backward.rs:46-185) on device-resident f32 tensors.  `workspace` is device memory of at least
 * rt_flash_backward_workspace_bytes(shape) bytes, 16-byte aligned (the recomputed forward output and two per-row
 * statistics); RT_ERR_WORKSPACE_TOO_SMALL otherwise.  Everything runs on `stream`. */
size_t rt_flash_backward_workspace_bytes(const rt_attention_shape *shape);
int rt_flash_backward_f32_dev(void *stream, const rt_attention_shape *shape, const float *q, const float *k,
                              const float *v, const float *d_out, float *dq, float *dk, float *dv, void *workspace,
                              size_t workspace_bytes, rt_err_detail *err);

/* The saved-forward form of the backward, which the header of cpu_backward.rs describes for a GPU path
 * (cpu_backward.rs:3-4, :29-35: "from a saved forward pass (Q, K, V, the softmax statistics m and l, and the upstream
 * gradient dO)"; the reference's CPU function recomputes instead).  rt_flash_forward_stats_f32_dev is the unmasked
 * forward that also writes the row statistic lse[b,h,i] = m_i + ln(l_i) ([batch,heads,seq] f32);
 * rt_flash_backward_saved_f32_dev takes that `out` and `lse` back and skips the recomputation.  `workspace`:
 * batch*heads*seq floats (RT_ERR_WORKSPACE_TOO_SMALL otherwise).  dim <= 128 for the backward. */
int rt_flash_forward_stats_f32_dev(void *stream, const rt_attention_shape *shape, const float *q, const float *k,
                                   const float *v, float *out, float *lse, rt_err_detail *err);
int rt_flash_backward_saved_f32_dev(void *stream, const rt_attention_shape *shape, const float *q, const float *k,
                                    const float *v, const float *out, const float *lse, const float *d_out, float *dq,
                                    float *dk, float *dv, void *workspace, size_t workspace_bytes, rt_err_detail *err);

/* flash_forward_masked on device-resident f32 tensors (same semantics; keep is a device
 * pointer to `seq` bytes).  n_kv_heads = 0 means n_kv_heads = heads.
 *
 * One divergence from the reference, for non-finite V under the causal mask (it holds for every prefill entry of
 * this library, host-slice or device, f32 or bf16): the reference walks every key tile and multiplies the hidden
 * probabilities (exact zeros) into V, so a NaN or Inf in V row j makes EVERY query row NaN in that column
 * (0 * NaN; cpu_forward.rs:268-425 skips no tile).  The kernels skip key tiles that lie wholly past a query tile
 * and never read those rows: query rows i >= j are NaN as in the reference, rows i <= j - 256 are finite (the value
 * the reference gives with V row j zeroed), rows in between may be either.  Finite inputs are unaffected.
 * rt_set_strict_non_finite_v(1) removes the divergence at the cost of one more pass over V. */
int rt_flash_forward_f32_dev(void *stream, const rt_attention_shape *shape, uint64_t n_kv_heads, const float *q,
                             const float *k, const float *v, int mask_kind, const uint8_t *keep, float *out,
                             rt_err_detail *err);

/* The bf16 counterpart (bf16 in, f32 accumulate, bf16 out rounded once, to nearest even):
 * q/out [batch,heads,seq,dim], k/v [batch,n_kv_heads,seq,dim].  Any dim up to 512 (the reference's forward takes
 * any dim != 0, cpu_forward.rs:142-169; above 512: RT_ERR_UNSUPPORTED with expected = 512).  Three MFMA kernels serve
 * dims up to 256 that are a multiple of 8 on 16-byte aligned tensors: a persistent 8-wave kernel for dim 128 (and
 * dim 64 under a key-padding mask) on unpadded batches of at least 512 rows per sequence and one job of 256 rows
 * per compute unit, a 4-wave tile kernel for everything else (dim 64 with no mask or the causal one, short or few
 * sequences, padded batches, other dims), and a form of the tile kernel with 64 query rows per wave for dim 64, which
 * runs only when it is asked for;
 * rt_debug_force_bf16_prefill_kernel forces one of them where it applies.  The remaining dims and alignments run on
 * a one-workgroup-per-row kernel with the same masks and row rules (correct at any speed, not tuned). */
int rt_flash_forward_bf16_dev(void *stream, const rt_attention_shape *shape, uint64_t n_kv_heads, const void *q,
                              const void *k, const void *v, int mask_kind, const uint8_t *keep, void *out,
                              rt_err_detail *err);

/* Causal self-attention with a sliding window, on bf16 device tensors: position i sees keys j with j <= i and
 * i - j < window -- what MultiHeadAttention computes with sliding_window_mask(seq, window) as its additive mask
 * (crates/rustorch-nn/src/masks.rs:41-60, applied at crates/rustorch-nn/src/attention.rs:378-392), without the
 * [seq, seq] f32 tensor (64 MB at seq = 4096, re-read per head) and without scoring the pairs it hides: a query tile
 * walks window + 128 keys.  The reference adds -1e4 to the hidden scores where this entry leaves the keys out; the
 * weights agree exactly (exp underflows to 0) as long as scaled scores stay far below 1e4 in magnitude.  window >= 1
 * (0: RT_ERR_UNSUPPORTED, the reference asserts); window >= seq is the causal mask.  Tensors [batch, heads, seq, dim]
 * (k, v: n_kv_heads; 0 = heads) or, for the _bnhd_ entry, [batch, seq, heads, dim]; head dims up to 256 that are a
 * multiple of 8 and 16-byte aligned tensors (others: RT_ERR_UNSUPPORTED; rt_mha_forward_masked_bf16_dev with the
 * mask tensor serves them). */
int rt_flash_forward_window_bf16_dev(void *stream, const rt_attention_shape *shape, uint64_t n_kv_heads, const void *q,
                                     const void *k, const void *v, uint64_t window, void *out, rt_err_detail *err);
int rt_flash_forward_window_bnhd_bf16_dev(void *stream, const rt_attention_shape *shape, uint64_t n_kv_heads,
                                          const void *q, const void *k, const void *v, uint64_t window, void *out,
                                          rt_err_detail *err);

/* No counterpart in the reference: a switch for measurements and tests.  which = 0 lets the library choose between
 * its bf16 prefill kernels (the default), 1 forces the tile kernel, 2 the persistent kernel where it applies (head
 * dim 64 / 128, no per-sequence lengths), 3 the kernel with 64 query rows per wave where it applies (head dim 64,
 * mask none or causal; elsewhere the tile kernel).  Process-wide; until it is called the value is taken, once, from
 * RT_ATTN_BF16_PREFILL=tile|persistent|wide in the environment.  Returns RT_ERR_UNSUPPORTED for another value. */
int rt_debug_force_bf16_prefill_kernel(int which);

/* No counterpart in the reference, whose CPU loop needs none: on != 0 makes every causal prefill entry (f32 and bf16,
 * every layout, padded batches included) follow its kernel with a pass that reads V once and writes NaN into each
 * (query row, column) for which a key the row does not see holds a NaN or Inf in that column of V -- the outcome of
 * cpu_forward.rs:268-425, which multiplies the hidden zeros into every V tile.  Off by default: the pass costs a
 * read of V (a few percent of a long prefill, more of a short one) and changes nothing for finite V.  Process-wide;
 * returns the previous setting. */
int rt_set_strict_non_finite_v(int on);

/* The same two calls on tensors laid out [batch, seq, heads, dim] (k/v: [batch, seq, n_kv_heads, dim]),
 * the layout rustorch_nn::MultiHeadAttention holds its projections in: the kernels walk the rows with a
 * pitch of heads*dim elements, so the four host-side transposes of
 * crates/rustorch-nn/src/attention.rs:466-486 (transpose_BTHD_to_BHTD_f32 x3, transpose_BHTD_to_BTHD_f32)
 * have no counterpart here.  out has the layout of q, i.e. [batch, seq, heads*dim]. */
int rt_flash_forward_bnhd_f32_dev(void *stream, const rt_attention_shape *shape, uint64_t n_kv_heads, const float *q,
                                  const float *k, const float *v, int mask_kind, const uint8_t *keep, float *out,
                                  rt_err_detail *err);
int rt_flash_forward_bnhd_bf16_dev(void *stream, const rt_attention_shape *shape, uint64_t n_kv_heads, const void *q,
                                   const void *k, const void *v, int mask_kind, const uint8_t *keep, void *out,
                                   rt_err_detail *err);

/* bf16 counterpart of rt_mha_forward_masked_f32_dev -- steps 2-8 of MultiHeadAttention::forward's composed path
 * (crates/rustorch-nn/src/attention.rs:371-399; masks crates/rustorch-nn/src/masks.rs:22-80): q/out bf16
 * [batch,t_q,heads*head_dim], k/v bf16 [batch,t_kv,heads*head_dim] (t_q != t_kv is cross-attention), `mask` an
 * additive f32 bias on the device with t_q*t_kv ([T,T] / [1,T,T]) or batch*heads*t_q*t_kv ([B*H,T,T]) elements,
 * or NULL.  scores = (q.k)/sqrt(head_dim) + mask in f32, softmax, .V; bf16 out rounded once.  A row masked with
 * -1e4 everywhere comes out uniform, a row of -inf as NaN, as in the f32 entry.  head_dim up to 256, a multiple
 * of 8; tensors 16-byte aligned.  Asynchronous on `stream`. */
int rt_mha_forward_masked_bf16_dev(void *stream, const void *q, const void *k, const void *v, const float *mask,
                                   size_t mask_len, void *out, size_t batch, size_t t_q, size_t t_kv, size_t heads,
                                   size_t head_dim, rt_err_detail *err);

/* Padded-batch causal prefill: sequence b has seq_lens[b] <= seq valid positions (device
 * int32[batch]); key j of sequence b is masked iff j > i or j >= seq_lens[b].  Valid rows equal
 * flash_forward_masked(Mask::Causal) on the truncated problem; rows i >= seq_lens[b] are written
 * as 0 when zero_padded_rows != 0, as NaN (the reference's no-visible-key rule) otherwise.
 * No counterpart in the reference, whose padding mask is one per-key vector for the whole batch. */
int rt_flash_forward_varlen_bf16_dev(void *stream, const rt_attention_shape *shape, uint64_t n_kv_heads,
                                     const void *q, const void *k, const void *v, const int32_t *seq_lens,
                                     int zero_padded_rows, void *out, rt_err_detail *err);

/* The masked / cross-attention core of MultiHeadAttention::forward, steps 2-8 of the composed path --
 * crates/rustorch-nn/src/attention.rs:371-399: scores = (Q.K^T) * (1/sqrt(head_dim)), + additive mask, softmax over
 * the keys (crates/rustorch-cpu/src/kernels/softmax.rs:146-180), . V -- on the projected tensors as the module holds
 * them: q, out [batch, t_q, heads*head_dim], k, v [batch, t_kv, heads*head_dim] (t_q != t_kv is cross-attention).
 * `mask` is the additive bias the module adds (crates/rustorch-nn/src/masks.rs:22-80 builds them: 0 keeps, -1e4
 * masks): NULL / mask_len 0 for none, t_q*t_kv elements for [T,T] or [1,T,T], batch*heads*t_q*t_kv for [B*H,T,T].
 * No transposed copies are made and the score matrix is never materialised.  Checks, in order: head_dim == 0 ->
 * RT_ERR_ZERO_DIM; q, k, v lengths -> RT_ERR_BUFFER_SHAPE_MISMATCH{which}; out length ->
 * RT_ERR_OUTPUT_SHAPE_MISMATCH; mask length -> RT_ERR_WRONG_INPUT_LEN{which = 5 ("mask"), expected = t_q*t_kv}.
 * t_kv == 0 gives rows of zeros (an empty softmax times an empty V, as the composed path computes it).
 * Synchronous, host slices. */
int rt_mha_forward_masked_f32(const float *q, size_t q_len, const float *k, size_t k_len, const float *v, size_t v_len,
                              const float *mask, size_t mask_len, float *out, size_t out_len, size_t batch,
                              size_t t_q, size_t t_kv, size_t heads, size_t head_dim, rt_err_detail *err);

/* The same attention on device-resident tensors, enqueued on `stream` (no host checks of the tensor lengths are
 * possible; the mask length is checked as above). */
int rt_mha_forward_masked_f32_dev(void *stream, const float *q, const float *k, const float *v, const float *mask,
                                  size_t mask_len, float *out, size_t batch, size_t t_q, size_t t_kv, size_t heads,
                                  size_t head_dim, rt_err_detail *err);

/* ---- decode, device pointers ------------------------------------------------------------------ */

/* LlmKernels::kv_append_bf16 -- crates/rustorch-cuda/src/llm_kernels.rs:353-372, :874-910.
 * cache[kv_h*max_seq*head_dim + pos*head_dim + i] = in[kv_h*head_dim + i] for K and V. */
int rt_kv_append_bf16(void *stream, void *k_cache, void *v_cache, const void *k_in, const void *v_in, int32_t pos,
                      int32_t n_kv, int32_t head_dim, int32_t max_seq, rt_err_detail *err);

/* KVLayerCache::append -- crates/rustorch-nn/src/kv_cache.rs:77-112 -- on device buffers: new_k / new_v
 * [batch, n_heads, seq_added, head_dim] are written at row current_len of the caches [batch, n_heads, max_seq,
 * head_dim]; elem_bytes is 2 (bf16) or 4 (f32).  Checks in the reference's order: current_len + seq_added > max_seq
 * -> RT_ERR_KV_OVERFLOW {requested = got, max = expected}; new_k_len or new_v_len (elements) != batch * n_heads *
 * seq_added * head_dim -> RT_ERR_KV_WRONG_INPUT_LEN {expected, got_k = got, got_v = got2}.  Asynchronous on `stream`. */
int rt_kv_cache_append_dev(void *stream, void *k_cache, void *v_cache, const void *new_k, size_t new_k_len,
                           const void *new_v, size_t new_v_len, size_t batch, size_t n_heads, size_t max_seq,
                           size_t head_dim, size_t current_len, size_t seq_added, size_t elem_bytes,
                           rt_err_detail *err);

/* Steps 2a, 2b and 3 of LlamaModel::decode_step -- crates/rustorch-llm/src/model.rs:575-636 -- in one launch,
 * for a batch of sequences on bf16 storage: per-head RMSNorm of q and k (rms_norm_per_head, model.rs:862-897;
 * gamma f32[head_dim] shared by the heads, NULL = no norm), half-split RoPE (RoPE::apply_inplace_half_split,
 * crates/rustorch-nn/src/rope.rs:162-205; cos/sin f32[table_rows, head_dim/2] as RoPE::new builds them,
 * rope.rs:63-90) and the cache append (KVLayerCache::append, crates/rustorch-nn/src/kv_cache.rs:77-112; for
 * seq == 1 the index rule of kv_append_bf16, llm_kernels.rs:353-372).  Replaces the rope_half_split_bf16 x2 +
 * kv_append_bf16 launches of crates/rustorch-llm/src/cuda_backend.rs:486-540.
 * `seq` new tokens per sequence (1 when decoding, the prompt length when prefilling): q [batch,n_heads,seq,
 * head_dim] is rewritten in place; k_in/v_in [batch,n_kv,seq,head_dim]; caches [batch,n_kv,max_seq,head_dim].
 * Token s of sequence b sits at position p_b + s, with p_b = positions[b] (device int32[batch]) or, with
 * positions == NULL, `pos`; k and v go to cache rows p_b .. p_b + seq - 1.  f32 arithmetic in the reference's
 * order, one rounding to bf16 at the end.
 * Errors (host `pos` only): pos + seq > table_rows -> RT_ERR_ROPE_POSITION_OVERFLOW (RoPEError::PositionOverflow
 * {max_seq = expected, requested = got}, rope.rs:179-184); pos + seq > max_seq -> RT_ERR_KV_OVERFLOW
 * (kv_cache.rs:84-89); odd head_dim or head_dim > 512 -> RT_ERR_UNSUPPORTED (RoPE::new panics on an odd head_dim).
 * Positions on the device cannot be checked by the host: a sequence whose rows would leave the tables or the
 * cache is left untouched. */
int rt_qk_norm_rope_kv_append_bf16(void *stream, void *q, const void *k_in, const void *v_in, void *k_cache,
                                   void *v_cache, const int32_t *positions, int32_t pos, const float *q_gamma,
                                   const float *k_gamma, float eps, const float *cos_table, const float *sin_table,
                                   int32_t table_rows, int32_t batch, int32_t seq, int32_t n_heads, int32_t n_kv,
                                   int32_t head_dim, int32_t max_seq, rt_err_detail *err);

/* LlmKernels::gqa_decode_online_bf16 -- llm_kernels.rs:396-457, :915-958.  q/out
 * [n_heads,head_dim] bf16, caches [n_kv,max_seq,head_dim] bf16 of which [..kv_len] is read;
 * kv head = h*n_kv/n_heads; f32 accumulation, output rounded once.  Runs the split-K kernels of the batched entry on
 * a batch of one (head_dim 64, 128 or 256, at most 16 query heads per kv head; other shapes take a one-workgroup-per-head
 * kernel).  The reference's signature has no workspace and its launcher allocates nothing (llm_kernels.rs:915-958):
 * the partials go to a slot of a fixed 64 MiB block of device memory inside the library (8 slots of 8 MiB; a
 * (device, stream) pair takes a free slot on its first call and keeps it until rt_stream_destroy / rt_shutdown, so
 * calls on different streams never share scratch), and the call allocates nothing: it may be the first call on a
 * stream and may be recorded into a HIP graph.  Only a ninth concurrent stream, or a shape whose partials do not fit a
 * slot (more than ~500 kv heads at 16 query heads each and head_dim 256), falls back to a buffer the library allocates
 * per (device, stream) on that stream's first call (then not under capture; a grown buffer replaces the old one,
 * which is kept until rt_stream_destroy / rt_shutdown).  q and the caches should be
 * 16-byte aligned: the split-K kernels move 16 bytes per lane, and tensors that are not aligned take the
 * one-workgroup-per-head kernel instead (same results, slower). */
int rt_gqa_decode_online_bf16(void *stream, const void *q, const void *k_cache, const void *v_cache, void *out,
                              int32_t n_heads, int32_t n_kv, int32_t kv_len, int32_t head_dim, int32_t max_seq,
                              rt_err_detail *err);

/* LlmKernels::gqa_decode_naive_bf16 -- llm_kernels.rs:461-545 (kernel), :990-1042 (launcher): the reference's first
 * decode kernel, the same function of the same arguments as gqa_decode_online_bf16 (softmax(q.K^T * scale).V over the
 * first kv_len cache rows, kv head = h*n_kv/n_heads) computed in three passes over a score buffer instead of one pass
 * with a running max.  Here both names run the same kernels and give the same bits. */
int rt_gqa_decode_naive_bf16(void *stream, const void *q, const void *k_cache, const void *v_cache, void *out,
                             int32_t n_heads, int32_t n_kv, int32_t kv_len, int32_t head_dim, int32_t max_seq,
                             rt_err_detail *err);

/* The batched, ragged form of the same call: q/out [batch,n_heads,head_dim], caches
 * [batch,n_kv,max_seq,head_dim], kv_lens device int32[batch] (sequence b reads [..kv_lens[b]]).
 * Split-K over the context with a second-pass (m, l, o) merge; `workspace` (device, at least
 * rt_gqa_decode_workspace_bytes(...) bytes, 16-byte aligned or the call fails with RT_ERR_WORKSPACE_TOO_SMALL)
 * holds the partial results.  q and the caches should be 16-byte aligned too (tensors that are not take the
 * one-workgroup-per-head kernel: same results, slower, no workspace).  The split-K kernels cover
 * head_dim 64, 128 and 256 with at most 16 query heads per kv head; other shapes take a one-workgroup-per-head kernel
 * (head_dim <= 512) that needs no workspace (rt_gqa_decode_workspace_bytes returns 0 for them).
 * batch = 1 with kv_lens = [kv_len] is the reference call.  A sequence with kv_lens[b] == 0
 * gives rows of +0.0 (the reference kernel ends with o / fmaxf(l, 1e-12f) = 0, llm_kernels.rs:456;
 * crates/rustorch-nn/src/gqa.rs:260-261 fills the row with 0 before an empty key loop). */
int rt_gqa_decode_batched_bf16(void *stream, const void *q, const void *k_cache, const void *v_cache, void *out,
                               const int32_t *kv_lens, int32_t batch, int32_t n_heads, int32_t n_kv,
                               int32_t head_dim, int32_t max_seq, void *workspace, size_t workspace_bytes,
                               rt_err_detail *err);

/* gqa_decode_batched_f32 -- crates/rustorch-metal/src/kernels.rs:14432-14516 (launcher :14522-14570) in bf16 and over
 * a batch of sequences: `seq_new` consecutive new positions per sequence attend to the cache, each up to and
 * including itself.  q/out bf16 [batch,seq_new,n_heads,head_dim] (position-major, as the reference's
 * [B,n_heads,head_dim]); caches bf16 [batch,n_kv,max_seq,head_dim], already holding the new positions' keys and
 * values (rt_qk_norm_rope_kv_append_bf16 with seq = seq_new puts them there); kv_lens device int32[batch] = keys in
 * the cache INCLUDING the new ones, or NULL: every sequence has `kv_len`.  Position s of sequence b sees keys
 * [0, kv_lens[b] - seq_new + s]: pos_base of the reference is kv_lens[b] - seq_new.  batch = 1, kv_lens = NULL,
 * kv_len = pos_base + B is the reference call; seq_new = 1 is rt_gqa_decode_batched_bf16.  kv head = h / (n_heads /
 * n_kv).  A position that sees no key (kv_lens[b] < seq_new - s) gives a row of +0.0, as the batched entry does for
 * kv_lens[b] == 0 (the shader's loops run zero times and leave acc = 0.0); kv_lens[b] above max_seq counts as
 * max_seq.  head_dim up to 256, a multiple of 8; tensors 16-byte aligned.  When the batch has fewer (sequence, kv
 * head, 128-row tile) units than the GPU has CUs and the cache is at least four key tiles long -- one sequence over
 * a long cache, the reference's call -- the keys are cut into spans, each span's (o, m, l) partials go to the
 * stream's slot of the library's fixed scratch block (see rt_gqa_decode_online_bf16: no allocation) and a second
 * kernel folds them.  Asynchronous on `stream`. */
int rt_gqa_decode_chunk_bf16(void *stream, const void *q, const void *k_cache, const void *v_cache, void *out,
                             const int32_t *kv_lens, int32_t kv_len, int32_t batch, int32_t seq_new, int32_t n_heads,
                             int32_t n_kv, int32_t head_dim, int32_t max_seq, rt_err_detail *err);

/* No counterpart in the reference.  rt_gqa_decode_batched_bf16 for callers that cannot allocate device memory
 * (code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc): same arguments without
 * the workspace, same kernels, same results bit for bit.  The split-K partials go to a fixed 8 MiB block of device
 * memory inside the library (one per GPU, there from the moment the library's code is loaded on that GPU until the
 * process ends); the call allocates and frees nothing.  rt_init(device) looks the block's address up; without it
 * the first call on a device does.
 *   - Limit: (4 * CUs + batch * n_kv) * (n_heads / n_kv) * (head_dim + 2) * 4 bytes must fit in 8 MiB (the headline
 *     decode workload, batch 64, 32 / 8 heads, head_dim 128, needs 3.2 MB); beyond it RT_ERR_WORKSPACE_TOO_SMALL
 *     (expected = bytes needed, got = 8 MiB).  Only the split-K shapes (head_dim 64 / 128 / 256, at most 16 query
 *     heads per kv head, 16-byte aligned q and caches); others RT_ERR_UNSUPPORTED.
 *   - Every call on a GPU uses that GPU's one block: calls that overlap on one GPU (two streams, two threads) race
 *     and give wrong results.  Calls on one stream are ordered and safe.  Nothing needs clearing between calls:
 *     every partial a call reads was written by the same call. */
int rt_gqa_decode_batched_bf16_noalloc(void *stream, const void *q, const void *k_cache, const void *v_cache, void *out,
                                       const int32_t *kv_lens, int32_t batch, int32_t n_heads, int32_t n_kv,
                                       int32_t head_dim, int32_t max_seq, rt_err_detail *err);
size_t rt_gqa_decode_workspace_bytes(int32_t batch, int32_t n_heads, int32_t n_kv, int32_t head_dim,
                                     int32_t max_seq);

/* ---- device buffers (the slot of Storage::Cuda, crates/rustorch-core/src/tensor/storage.rs:776-817) */
void *rt_buf_alloc(size_t bytes, rt_err_detail *err);
int rt_buf_free(void *ptr, rt_err_detail *err);
/* Zero-fills `bytes` bytes at `ptr` (a multiple of 4, `ptr` 4-byte aligned), asynchronously on `stream`, with a
 * fill kernel (safe to record into a HIP graph).  The reference's caches start as vec![0.0; n]
 * (crates/rustorch-nn/src/kv_cache.rs:63-66). */
int rt_buf_zero(void *ptr, size_t bytes, void *stream, rt_err_detail *err);
/* No counterpart in the reference (its decode loop keeps the position on the host, crates/rustorch-llm/src/
 * cuda_backend.rs:516-556): adds `delta` to each of the `n` int32 values at device address `ptr`, asynchronously on
 * `stream`.  A decode loop recorded into a HIP graph keeps its positions and context lengths on the device (the
 * `positions` of rt_qk_norm_rope_kv_append_bf16, the `kv_lens` of the batched decode entries) and advances them
 * with this call at the end of every token. */
int rt_i32_add_dev(void *stream, int32_t *ptr, size_t n, int32_t delta, rt_err_detail *err);
int rt_memcpy_h2d(void *dst, const void *src, size_t bytes, void *stream, rt_err_detail *err);
int rt_memcpy_d2h(void *dst, const void *src, size_t bytes, void *stream, rt_err_detail *err);
int rt_stream_synchronize(void *stream, rt_err_detail *err);
/* A stream at the default priority for the device entry points (the place of the reference's Arc<CudaStream>,
 * crates/rustorch-cuda/src/llm_kernels.rs:874-880); NULL and err filled on failure. */
void *rt_stream_create(rt_err_detail *err);
int rt_stream_destroy(void *stream, rt_err_detail *err);

#ifdef __cplusplus
}
#endif
#endif /* RT_ATTN_H */
