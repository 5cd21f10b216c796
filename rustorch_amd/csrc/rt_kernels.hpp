// Kernel parameter blocks and launchers shared between the kernel files and the C ABI.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace rt {

// 0..2 are rt_mask_kind of the C ABI; 3 is the padded-batch mode (per-sequence length + causal).
enum MaskKind : int { kMaskNone = 0, kMaskCausal = 1, kMaskPadding = 2, kMaskVarlenCausal = 3 };
constexpr float kLog2eHost = 1.4426950408889634f;

// Where element [b, h, row, 0] of a 4-D attention tensor sits (in elements): rows of `dim` contiguous
// elements, `row_pitch` apart.  [B,H,N,D] row-major: {H*N*D, N*D, D}; [B,N,H,D] row-major (the layout
// MultiHeadAttention holds its projections in): {N*H*D, D, H*D}.
struct TensorLayout {
    long long batch_stride;
    long long head_stride;
    int row_pitch;
};
inline TensorLayout layout_bhnd(long long heads, long long seq, int dim) {
    return TensorLayout{heads * seq * dim, seq * dim, dim};
}
inline TensorLayout layout_bnhd(long long heads, long long seq, int dim) {
    return TensorLayout{seq * heads * dim, (long long)dim, (int)(heads * dim)};
}

struct FlashF32Params {
    const float* q;
    const float* k;
    const float* v;
    float* out;
    const uint8_t* keep;  // device, `seq` bytes, for kMaskPadding
    int batch, heads, kv_heads, group;
    int seq, dim;
    int seq_kv;  // keys per (batch, kv head) when they differ from `seq` (cross-attention; mask none only); 0: == seq
    int mask;
    int ref_bc;  // the reference's key-tile size, for the leading-masked-tile rule
    float scale;
    TensorLayout lq, lkv, lo;  // layouts of q, of k and v, of out
    int n_cus;   // CUs of the device (0: unknown)
    int zigzag;  // set by the launcher
    // optional additive score bias, rows of `seq` f32 per query row, added after scaling (zero-initialise to leave off)
    const float* bias;
    long long bias_bh_stride;  // elements between the biases of consecutive (batch, head) pairs; 0 = one for all
    // optional [batch, heads, seq] output: the row statistic m + ln(l) of the softmax (what a backward pass needs)
    float* lse;
};
// dim <= 256 (the tiled four-wave kernel up to 128).  Returns hipErrorInvalidValue for an unsupported dim.
hipError_t launch_flash_f32(hipStream_t stream, const FlashF32Params& p);

// Backward of unmasked f32 attention; every tensor is [batch, heads, seq, dim] row-major and contiguous.
struct FlashBwdF32Params {
    const float* q;
    const float* k;
    const float* v;
    const float* d_out;
    float* dq;
    float* dk;
    float* dv;
    int batch, heads, seq, dim;
    float scale;
    // filled by the launcher
    const float* o;
    const float* lse;
    float* delta;  // written by the dQ kernel (its owner rows), read by the dK/dV kernel that runs after it
    int vec;
};
// Floats of scratch launch_flash_bwd_f32 needs (O, the row statistic and delta).
size_t flash_bwd_f32_workspace_floats(int batch, int heads, int seq, int dim);
// dim <= 128.  Runs the forward kernel, then dQ (which also leaves delta) and dK/dV on `stream`.
hipError_t launch_flash_bwd_f32(hipStream_t stream, const FlashBwdF32Params& p, float* workspace, int n_cus);
// The same from a saved forward: `o` [B,H,N,D] and `lse` [B,H,N] as launch_flash_f32 leaves them (FlashF32Params::lse);
// `delta` is B*H*N floats of scratch.  Runs dQ (which also leaves delta), then dK/dV.
hipError_t launch_flash_bwd_f32_saved(hipStream_t stream, const FlashBwdF32Params& p, const float* o, const float* lse,
                                      float* delta);

struct FlashBf16Params {
    const uint16_t* q;
    const uint16_t* k;
    const uint16_t* v;
    uint16_t* out;
    const uint8_t* keep;      // kMaskPadding
    const int32_t* seq_lens;  // kMaskVarlenCausal: device int32[batch]
    int batch, heads, kv_heads, group;
    int seq, dim;
    int mask;
    int ref_bc;
    int zero_padded_rows;
    float scale_log2e;  // (1/sqrt(dim)) * log2(e)
    int n_workers;      // persistent workgroups to launch: the number of CUs
    TensorLayout lq, lkv, lo;  // layouts of q, of k and v, of out; seq * row_pitch * 2 bytes must stay below 2^32
};
// dim in {64, 128}; a padding mask (kMaskPadding) of at most kFlashBf16MaxPaddingKeys keys.
constexpr int kFlashBf16MaxPaddingKeys = 65536;
hipError_t launch_flash_bf16(hipStream_t stream, const FlashBf16Params& p);

// The general bf16 forward (flash_bf16_tile.hip): any dim <= 256 that is a multiple of 8, own key count, per-sequence
// query / key counts, causal mask aligned to the last key, key-padding vector, additive f32 bias, packed GQA rows.
struct FlashTileParams {
    const uint16_t* q;
    const uint16_t* k;
    const uint16_t* v;
    uint16_t* out;
    const uint8_t* keep;      // kMaskPadding: device, seq_kv bytes
    const int32_t* q_lens;    // optional device int32[batch]: valid query positions (rows past them are padding)
    const int32_t* kv_lens;   // optional device int32[batch]: keys that exist
    const float* bias;        // optional additive score bias, f32 rows of seq_kv per query position, added after scaling
    long long bias_bh_stride; // elements between the biases of consecutive (batch, head) pairs; 0 = one for all
    int bias_vec4;            // bias rows may be read 16 bytes at a time (base and seq_kv * 4 bytes both 16-byte aligned)
    int batch, heads, kv_heads, group;
    uint32_t group_magic;     // set by the launcher: 2^32 / group + 1 (0 when group is 1), for head / group by a multiply
    // 1: a tile's rows are positions of one head.  group: rows run over (position, head of the GQA group), row
    // r = position * group + head-in-group, so that all heads of a kv head share one pass over its keys.
    int pack;
    // rows are positions of a chunked decode over a cache: a position that sees no key is a row of zeros (the
    // reference's decode kernels leave it so), not the NaN row of flash_forward.  Implied by pack > 1; a group of one
    // head sets it.
    int decode_rows;
    int seq_q, seq_kv, dim;
    int mask;   // kMaskNone, kMaskCausal (key j visible to position i iff j <= i + (keys - valid queries)), kMaskPadding
    int ref_bc;
    int zero_padded_rows;  // rows past q_lens[b]: +0.0 (else NaN)
    float scale_log2e;     // (1/sqrt(dim)) * log2(e)
    float scale;           // 1/sqrt(dim)
    TensorLayout lq, lkv, lo;
    // Split over the keys (packed rows only; zero-initialise to leave it off): n_splits > 1 cuts every (sequence, kv
    // head)'s walk into that many spans of whole tiles; each leaves a partial per packed row in part_o
    // ([batch, kv_heads, seq_q * pack, n_splits, dim] f32) and part_ml (the same index, (m, l) pairs), and a second
    // kernel folds them into `out`.
    int n_splits;
    float* part_o;
    float* part_ml;
    // Sliding window (causal mask only, unpacked rows, no bias; 0 = none): position i sees the `window` keys that end
    // with key i + (keys - valid queries), as sliding_window_mask builds it (crates/rustorch-nn/src/masks.rs:41-60).
    int window;
};
bool flash_tile_bf16_supported(int dim);
// keys per LDS tile of the tile kernel at head dim `dim` (the unit the split over the keys is cut in)
int flash_tile_bf16_key_tile(int dim);
hipError_t launch_flash_tile_bf16(hipStream_t stream, const FlashTileParams& p);
bool flash_tile_bf16_addressable(long long seq_kv, long long row_pitch);  // K/V slabs below 4 GiB (32-bit offsets)
// the same walk with 64 query rows per wave: head dim 64, masks none / causal, rows of one head
bool flash_wide_bf16_supported(const FlashTileParams& p);
hipError_t launch_flash_wide_bf16(hipStream_t stream, const FlashTileParams& p);

// Unmasked attention of every query row over all keys; generic in dim (<= 512), head
// grouping, kv_len and query count.  T is float or uint16_t (bf16 bits).
struct AttnRowsParams {
    const void* q;    // [batch, heads, seq_q, dim]
    const void* k;    // [batch, kv_heads, kv_stride, dim]
    const void* v;
    void* out;        // [batch, heads, seq_q, dim]
    const int32_t* kv_lens;  // device int32[batch] or nullptr (then kv_len)
    int batch, heads, kv_heads;
    int seq_q, kv_len, kv_stride, dim;
    int head_map;  // 0: kv_h = h / (heads/kv_heads) (gqa.rs:233); 1: kv_h = h*kv_heads/heads (llm_kernels.rs:410)
    float scale;
    // optional (zero-initialise the struct to leave them off):
    const float* bias;         // additive score bias [seq_q, kv_len] rows, added after scaling; f32 tensors only
    long long bias_bh_stride;  // elements between the biases of consecutive (batch, head) pairs; 0 = one bias for all
    int use_layout;            // != 0: q/out and k/v are addressed through the layouts below instead of [B,H,S,D]
    TensorLayout lq, lkv, lo;
    // the masks and row rules of flash_forward_masked (crates/rustorch-attention/src/cpu_forward.rs:193-425), for the
    // head dims the tiled kernels do not cover (zero-initialise to leave them off: plain attention over kv_len keys,
    // a row without keys is a row of zeros as in the decode kernels)
    int mask;                  // kMaskNone, kMaskCausal (key t visible to query i iff t <= i + (keys - valid queries)), kMaskPadding
    const uint8_t* keep;       // kMaskPadding: device, kv_len bytes
    int ref_bc;                // kMaskPadding: the reference's key-tile size (a wholly hidden first tile makes every row NaN)
    int flash_rows;            // != 0: a row that sees no key, or whose sum is not finite, is NaN (the l > 0 && finite test)
    const int32_t* q_lens;     // optional device int32[batch]: valid query rows; rows past them get the fill value
    int zero_padded_rows;      // the fill value: +0.0 (else NaN)
    float* lse;                // optional f32 [batch, heads, seq_q]: m + ln(l) of every row (f32 tensors only)
};
hipError_t launch_attn_rows_f32(hipStream_t stream, const AttnRowsParams& p);
hipError_t launch_attn_rows_bf16(hipStream_t stream, const AttnRowsParams& p);

// The pass behind rt_set_strict_non_finite_v: NaN into every (query row, column) whose causally hidden keys hold a
// non-finite V element in that column.  Tensors f32 or bf16 bits ([batch, heads | kv_heads, seq, dim] through the
// layouts); head_map as in flash_forward (kv_h = h / (heads / kv_heads)); seq_lens optional (padded batches).
struct StrictVParams {
    const void* v;
    void* out;
    const int32_t* seq_lens;
    int batch, heads, kv_heads, seq, dim;
    TensorLayout lkv, lo;
};
hipError_t launch_strict_hidden_v(hipStream_t stream, const StrictVParams& p, bool bf16);

struct DecodeSplitParams {
    const uint16_t* q;        // [batch, heads, dim]
    const uint16_t* k_cache;  // [batch, kv_heads, max_seq, dim]
    const uint16_t* v_cache;
    uint16_t* out;            // [batch, heads, dim]
    const int32_t* kv_lens;   // device int32[batch], or nullptr: every sequence has kv_len keys
    int kv_len;
    float* ws;                // partial (o, m, l) per (b, head, chunk)
    int batch, heads, kv_heads, dim, max_seq;
    int n_part;   // partial slots per (sequence, head): decode_split_parts(batch, max_seq)
    int span_min;  // a wave takes at least this many 32-key steps: decode_split_span_min(batch)
    int n_waves;  // one-wave workgroups launched (all resident at once)
    float scale_log2e;
    // Where a partial sits in `ws`.  0: slot (sequence, head, k-th wave on the segment), n_part slots per head --
    // sized for the worst case of every segment at max_seq.  1: slot (wave index + segment index, head of the
    // group): along the flat step list every partial advances the wave, the segment or both, so the sum numbers
    // them without collisions, and (n_waves + batch * kv_heads) * group slots hold any batch whatever its lengths.
    int compact;
};
bool decode_split_supported(int heads, int kv_heads, int dim);
int decode_split_span_min(int batch);
int decode_split_parts(int batch, int max_seq);
size_t decode_split_workspace_bytes(int batch, int heads, int dim, int max_seq);
// bytes of `ws` in the compact layout
size_t decode_split_compact_bytes(int batch, int heads, int kv_heads, int dim, int n_waves);
// The library's own scratch block for callers that cannot allocate: a fixed array in device memory (one per GPU,
// held until the process ends).  Looks its address up once per device (the device must be current) and returns it
// with its size.
hipError_t decode_static_scratch(float** ptr, size_t* bytes);
// A second fixed block, cut into slots: scratch for the entry points whose reference signature has no workspace
// argument.  The host side hands one slot to each (device, stream) that needs one, so calls on different streams
// never share scratch.  Returns the address of a slot on the current device and its size.
constexpr int kStreamSlots = 8;
constexpr size_t kStreamSlotBytes = (size_t)8 << 20;
hipError_t stream_static_scratch(int slot, float** ptr, size_t* bytes);
hipError_t launch_decode_split(hipStream_t stream, const DecodeSplitParams& p);

// KVLayerCache::append on device buffers of 2- or 4-byte elements: [batch_heads, seq_added, head_dim] into
// [batch_heads, max_seq, head_dim] at row current_len.
hipError_t launch_kv_block_append(hipStream_t stream, void* k_cache, void* v_cache, const void* new_k, const void* new_v,
                                  size_t batch_heads, size_t max_seq, size_t head_dim, size_t current_len,
                                  size_t seq_added, size_t elem_bytes);

// Per-head q/k RMSNorm, half-split RoPE and the cache append of one decode step (prepare.hip).
struct DecodePrepareParams {
    uint16_t* q;              // [batch, n_heads, seq, head_dim], rewritten in place
    const uint16_t* k_in;     // [batch, n_kv, seq, head_dim]
    const uint16_t* v_in;
    uint16_t* k_cache;        // [batch, n_kv, max_seq, head_dim]
    uint16_t* v_cache;
    const int32_t* positions; // device int32[batch] (position of a sequence's first new token), or null: `pos` for all
    const float* q_gamma;     // f32[head_dim] or null (no norm)
    const float* k_gamma;
    const float* cos_table;   // f32[table_rows, head_dim / 2]
    const float* sin_table;
    float eps;
    int pos;
    int batch, seq, n_heads, n_kv, head_dim, max_seq, table_rows;
};
// head_dim even and <= 512; seq, batch <= 65535
hipError_t launch_decode_prepare(hipStream_t stream, const DecodePrepareParams& p);

hipError_t launch_kv_append_bf16(hipStream_t stream, uint16_t* k_cache, uint16_t* v_cache, const uint16_t* k_in,
                                 const uint16_t* v_in, int pos, int n_kv, int head_dim, int max_seq);

}  // namespace rt
