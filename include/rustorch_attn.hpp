// rustorch_attn.hpp -- C++ host-side mirror of rustorch's attention call surface over the C ABI of
// librt_attn_hip.so (rt_attn.h).  Header only; link with -lrt_attn_hip.
//
// The names, argument meaning and error behaviour follow the Rust items they stand for (paths relative to
// the reference checkout):
//
//   rustorch_attn::AttentionShape, AttentionError, flash_forward, flash_forward_masked
//                                   crates/rustorch-attention/src/cpu_forward.rs:49-242
//   rustorch_attn::flash_backward   crates/rustorch-attention/src/cpu_backward.rs:46-185
//   rustorch_attn::Mask             crates/rustorch-attention/src/mask.rs:26-78
//   rustorch_attn::gqa_forward_f32, GQAError
//                                   crates/rustorch-nn/src/gqa.rs:36-210
//   rustorch_attn::mha_flash_forward_f32, mha_forward_masked_f32
//                                   crates/rustorch-nn/src/attention.rs:371-399, :452-495
//   rustorch_attn::causal_mask, sliding_window_mask, bool_to_additive
//                                   crates/rustorch-nn/src/masks.rs:22-82
//   rustorch_attn::LlmKernels       crates/rustorch-cuda/src/llm_kernels.rs:874-958 (attention part)
//   rustorch_attn::KVCache          crates/rustorch-nn/src/kv_cache.rs:49-256, buffers in HBM
//   rustorch_attn::RoPE, RoPEError  crates/rustorch-nn/src/rope.rs:33-241 (tables and errors; the rotation runs on the device)
//   rustorch_attn::HipStorage       the slot of Storage::Cuda, crates/rustorch-core/src/tensor/storage.rs:776-817
//
// Where Rust returns Result<(), E>, these functions throw E (a std::exception carrying the enum's fields).
// There is no CPU fallback: on a machine without a gfx950 device compute calls throw DeviceError.
#ifndef RUSTORCH_ATTN_HPP
#define RUSTORCH_ATTN_HPP

#include <array>
#include <cmath>
#include <cstddef>
#include <cstdint>
#include <stdexcept>
#include <string>
#include <utility>
#include <vector>

#include "rt_attn.h"

namespace rustorch_attn {

// ---- errors ------------------------------------------------------------------------------------------

// AttentionError (cpu_forward.rs:93-114) with MaskError folded in as the Mask variant (mask.rs:70-78).
struct AttentionError : std::runtime_error {
    enum class Kind { ZeroDim, BufferShapeMismatch, OutputShapeMismatch, MaskPaddingLengthMismatch };
    Kind kind;
    std::string which;  // "q" | "k" | "v" for BufferShapeMismatch
    size_t expected = 0, got = 0;
    AttentionError(Kind k, std::string w, size_t e, size_t g, const std::string& msg)
        : std::runtime_error(msg), kind(k), which(std::move(w)), expected(e), got(g) {}
};

// GQAError (gqa.rs:37-55).
struct GQAError : std::runtime_error {
    enum class Kind { HeadCountMismatch, WrongInputLen };
    Kind kind;
    std::string which;  // "q" | "k" | "v" | "out" | "flash_forward"
    size_t expected = 0, got = 0;  // HeadCountMismatch: expected = n_heads, got = n_kv_heads
    GQAError(Kind k, std::string w, size_t e, size_t g, const std::string& msg)
        : std::runtime_error(msg), kind(k), which(std::move(w)), expected(e), got(g) {}
};

// RoPEError (crates/rustorch-nn/src/rope.rs:208-241) and KVCacheError::Overflow (kv_cache.rs:229-256), the two
// errors the decode preparation step can return.
struct RoPEError : std::runtime_error {
    enum class Kind { WrongInputLen, PositionOverflow };
    Kind kind;
    size_t expected = 0, got = 0;  // PositionOverflow: expected = max_seq, got = requested
    RoPEError(Kind k, size_t e, size_t g, const std::string& msg) : std::runtime_error(msg), kind(k), expected(e), got(g) {}
};
struct KVCacheOverflow : std::runtime_error {
    size_t requested = 0, max = 0;
    KVCacheOverflow(size_t r, size_t m)
        : std::runtime_error("kv_cache overflow: requested " + std::to_string(r) + " positions, max " + std::to_string(m)),
          requested(r), max(m) {}
};
// The other two variants of KVCacheError.
struct KVCacheWrongInputLen : std::runtime_error {
    size_t expected = 0, got_k = 0, got_v = 0;
    KVCacheWrongInputLen(size_t e, size_t k, size_t v)
        : std::runtime_error("kv_cache append: expected " + std::to_string(e) + ", got K=" + std::to_string(k) +
                             " V=" + std::to_string(v)),
          expected(e), got_k(k), got_v(v) {}
};
struct KVCacheLayerOutOfRange : std::runtime_error {
    size_t layer = 0, num_layers = 0;
    KVCacheLayerOutOfRange(size_t l, size_t n)
        : std::runtime_error("kv_cache layer " + std::to_string(l) + " out of range (have " + std::to_string(n) + ")"),
          layer(l), num_layers(n) {}
};

// Stands where the reference has CudaError: no device, a failed HIP call, a shape the kernels do not cover.
struct DeviceError : std::runtime_error {
    int status;     // rt_status
    int hip_error;  // hipError_t when status == RT_ERR_HIP
    DeviceError(int st, int he, const std::string& msg) : std::runtime_error(msg), status(st), hip_error(he) {}
};

namespace detail {
inline const char* which_name(int w) {
    static const char* names[] = {"q", "k", "v", "out", "flash_forward", "mask", "do"};
    return (w >= 0 && w < 7) ? names[w] : "";
}
[[noreturn]] inline void throw_device(int rc, const rt_err_detail& e) {
    throw DeviceError(rc, e.hip_error, std::string(rt_status_name(rc)) + ": " + e.message);
}
inline void check_attention(int rc, const rt_err_detail& e) {
    using K = AttentionError::Kind;
    switch (rc) {
        case RT_OK: return;
        case RT_ERR_ZERO_DIM: throw AttentionError(K::ZeroDim, "", 0, 0, "dim must be > 0");
        case RT_ERR_BUFFER_SHAPE_MISMATCH: {
            std::string w = which_name(e.which);
            throw AttentionError(K::BufferShapeMismatch, w, e.expected, e.got,
                                 w + " buffer has " + std::to_string(e.got) + " elements, expected " +
                                     std::to_string(e.expected));
        }
        case RT_ERR_OUTPUT_SHAPE_MISMATCH:
            throw AttentionError(K::OutputShapeMismatch, "", e.expected, e.got,
                                 "output buffer has " + std::to_string(e.got) + " elements, expected " +
                                     std::to_string(e.expected));
        case RT_ERR_PADDING_LENGTH_MISMATCH:
            throw AttentionError(K::MaskPaddingLengthMismatch, "", e.expected, e.got,
                                 "mask error: padding mask len " + std::to_string(e.got) + ", expected " +
                                     std::to_string(e.expected));
        default: throw_device(rc, e);
    }
}
inline void check_gqa(int rc, const rt_err_detail& e) {
    using K = GQAError::Kind;
    switch (rc) {
        case RT_OK: return;
        case RT_ERR_HEAD_COUNT_MISMATCH:
            throw GQAError(K::HeadCountMismatch, "", e.expected, e.got,
                           "gqa: n_heads " + std::to_string(e.expected) + " not divisible by n_kv_heads " +
                               std::to_string(e.got));
        case RT_ERR_WRONG_INPUT_LEN: {
            std::string w = which_name(e.which);
            throw GQAError(K::WrongInputLen, w, e.expected, e.got,
                           "gqa: " + w + " expected " + std::to_string(e.expected) + " f32, got " +
                               std::to_string(e.got));
        }
        default: throw_device(rc, e);
    }
}
inline void check_device(int rc, const rt_err_detail& e) {
    if (rc != RT_OK) throw_device(rc, e);
}
inline void check_prepare(int rc, const rt_err_detail& e) {
    switch (rc) {
        case RT_OK: return;
        case RT_ERR_ROPE_WRONG_INPUT_LEN:
            throw RoPEError(RoPEError::Kind::WrongInputLen, e.expected, e.got,
                            "rope: expected buffer of " + std::to_string(e.expected) + " f32, got " + std::to_string(e.got));
        case RT_ERR_ROPE_POSITION_OVERFLOW:
            throw RoPEError(RoPEError::Kind::PositionOverflow, e.expected, e.got,
                            "rope: position " + std::to_string(e.got) + " exceeds max_seq " + std::to_string(e.expected));
        case RT_ERR_KV_OVERFLOW: throw KVCacheOverflow(e.got, e.expected);
        case RT_ERR_KV_WRONG_INPUT_LEN: throw KVCacheWrongInputLen(e.expected, e.got, e.got2);
        default: throw_device(rc, e);
    }
}
}  // namespace detail

// ---- shapes and masks ------------------------------------------------------------------------------------

// AttentionShape (cpu_forward.rs:49-89): row-major [batch, heads, seq, dim]; br = bc = 64 by default.
struct AttentionShape {
    size_t batch = 0, heads = 0, seq = 0, dim = 0, br = 64, bc = 64;
    static AttentionShape make(size_t batch, size_t heads, size_t seq, size_t dim) {
        return AttentionShape{batch, heads, seq, dim, 64, 64};
    }
    AttentionShape with_tiles(size_t br_, size_t bc_) const {
        AttentionShape s = *this;
        s.br = br_;
        s.bc = bc_;
        return s;
    }
    size_t buffer_len() const { return batch * heads * seq * dim; }
    std::array<size_t, 4> strides() const { return {heads * seq * dim, seq * dim, dim, 1}; }
    rt_attention_shape c() const { return rt_attention_shape{batch, heads, seq, dim, br, bc}; }
};

// Mask (mask.rs:26-65).
struct Mask {
    enum class Kind { None = RT_MASK_NONE, Causal = RT_MASK_CAUSAL, Padding = RT_MASK_PADDING };
    Kind kind = Kind::None;
    std::vector<uint8_t> keep;  // Padding: one byte per key, non-zero = visible
    static Mask none() { return Mask{}; }
    static Mask causal() {
        Mask m;
        m.kind = Kind::Causal;
        return m;
    }
    static Mask padding(const std::vector<bool>& keep_mask) {
        Mask m;
        m.kind = Kind::Padding;
        m.keep.assign(keep_mask.begin(), keep_mask.end());
        return m;
    }
    bool is_masked(size_t qi, size_t kj) const {
        if (kind == Kind::Causal) return kj > qi;
        if (kind == Kind::Padding) return kj < keep.size() && keep[kj] == 0;
        return false;
    }
};

// ---- prefill on host slices (synchronous, like the Rust functions) ----------------------------------------

inline void flash_forward_masked(const AttentionShape& shape, const float* q, size_t q_len, const float* k,
                                 size_t k_len, const float* v, size_t v_len, const Mask& mask, float* out,
                                 size_t out_len) {
    rt_attention_shape s = shape.c();
    rt_err_detail e;
    int rc = rt_flash_forward_masked_f32(&s, q, q_len, k, k_len, v, v_len, (int)mask.kind,
                                         mask.keep.empty() ? nullptr : mask.keep.data(), mask.keep.size(), out,
                                         out_len, &e);
    detail::check_attention(rc, e);
}
inline void flash_forward_masked(const AttentionShape& shape, const std::vector<float>& q,
                                 const std::vector<float>& k, const std::vector<float>& v, const Mask& mask,
                                 std::vector<float>& out) {
    flash_forward_masked(shape, q.data(), q.size(), k.data(), k.size(), v.data(), v.size(), mask, out.data(),
                         out.size());
}
inline void flash_forward(const AttentionShape& shape, const std::vector<float>& q, const std::vector<float>& k,
                          const std::vector<float>& v, std::vector<float>& out) {
    flash_forward_masked(shape, q, k, v, Mask::none(), out);
}

// flash_backward (cpu_backward.rs:46-185): (dQ, dK, dV) of unmasked attention; the three outputs are overwritten.
inline void flash_backward(const AttentionShape& shape, const std::vector<float>& q, const std::vector<float>& k,
                           const std::vector<float>& v, const std::vector<float>& d_out, std::vector<float>& dq,
                           std::vector<float>& dk, std::vector<float>& dv) {
    rt_attention_shape s = shape.c();
    rt_err_detail e;
    int rc = rt_flash_backward_f32(&s, q.data(), q.size(), k.data(), k.size(), v.data(), v.size(), d_out.data(),
                                   d_out.size(), dq.data(), dq.size(), dk.data(), dk.size(), dv.data(), dv.size(), &e);
    detail::check_attention(rc, e);
}

// gqa_forward_f32 (gqa.rs:94-210).
inline void gqa_forward_f32(const std::vector<float>& q, const std::vector<float>& k, const std::vector<float>& v,
                            std::vector<float>& out, size_t batch, size_t n_heads, size_t n_kv_heads, size_t seq_q,
                            size_t seq_kv, size_t head_dim) {
    rt_err_detail e;
    int rc = rt_gqa_forward_f32(q.data(), q.size(), k.data(), k.size(), v.data(), v.size(), out.data(), out.size(),
                                batch, n_heads, n_kv_heads, seq_q, seq_kv, head_dim, &e);
    detail::check_gqa(rc, e);
}

// mha_flash_forward_f32 (attention.rs:452-495): q, k, v [B,T,H,hd]; returns [B,T,H*hd].
inline std::vector<float> mha_flash_forward_f32(const std::vector<float>& q, const std::vector<float>& k,
                                                const std::vector<float>& v, size_t batch, size_t seq, size_t heads,
                                                size_t head_dim) {
    std::vector<float> out(batch * seq * heads * head_dim);
    rt_err_detail e;
    int rc = rt_mha_flash_forward_f32(q.data(), q.size(), k.data(), k.size(), v.data(), v.size(), out.data(),
                                      out.size(), batch, seq, heads, head_dim, &e);
    detail::check_attention(rc, e);
    return out;
}

// Additive attention masks (crates/rustorch-nn/src/masks.rs:22-82): 0 keeps, kMaskNeg masks.
constexpr float kMaskNeg = -1.0e4f;
inline std::vector<float> causal_mask(size_t seq_len) {
    std::vector<float> m(seq_len * seq_len, 0.0f);
    for (size_t i = 0; i < seq_len; i++)
        for (size_t j = i + 1; j < seq_len; j++) m[i * seq_len + j] = kMaskNeg;
    return m;
}
inline std::vector<float> sliding_window_mask(size_t seq_len, size_t window) {
    if (window < 1) throw std::invalid_argument("sliding_window_mask: window must be >= 1");
    std::vector<float> m(seq_len * seq_len, kMaskNeg);
    for (size_t i = 0; i < seq_len; i++)
        for (size_t j = 0; j <= i; j++)
            if (i - j < window) m[i * seq_len + j] = 0.0f;
    return m;
}
inline std::vector<float> bool_to_additive(const std::vector<float>& keep) {
    std::vector<float> m(keep.size());
    for (size_t i = 0; i < keep.size(); i++) m[i] = keep[i] >= 0.5f ? 0.0f : kMaskNeg;
    return m;
}

// Steps 2-8 of MultiHeadAttention::forward's composed path (attention.rs:371-399): softmax(Q.K^T/sqrt(hd) + mask).V on
// the projected tensors q [B,t_q,H*hd], k, v [B,t_kv,H*hd]; `attn_mask` empty, t_q*t_kv or B*H*t_q*t_kv elements.
inline std::vector<float> mha_forward_masked_f32(const std::vector<float>& q, const std::vector<float>& k,
                                                 const std::vector<float>& v, size_t batch, size_t t_q, size_t t_kv,
                                                 size_t heads, size_t head_dim,
                                                 const std::vector<float>& attn_mask = std::vector<float>()) {
    std::vector<float> out(batch * t_q * heads * head_dim);
    rt_err_detail e;
    int rc = rt_mha_forward_masked_f32(q.data(), q.size(), k.data(), k.size(), v.data(), v.size(),
                                       attn_mask.empty() ? nullptr : attn_mask.data(), attn_mask.size(), out.data(),
                                       out.size(), batch, t_q, t_kv, heads, head_dim, &e);
    if (rc == RT_ERR_WRONG_INPUT_LEN) detail::check_gqa(rc, e);  // which = "mask"
    detail::check_attention(rc, e);
    return out;
}

// gqa_forward_f32 on device-resident tensors, enqueued on `stream`.
inline void gqa_forward_f32_dev(const float* q, const float* k, const float* v, float* out, size_t batch,
                                size_t n_heads, size_t n_kv_heads, size_t seq_q, size_t seq_kv, size_t head_dim,
                                void* stream = nullptr) {
    rt_err_detail e;
    detail::check_gqa(rt_gqa_forward_f32_dev(stream, q, k, v, out, batch, n_heads, n_kv_heads, seq_q, seq_kv, head_dim, &e),
                      e);
}

// mha_forward_masked_f32 on device-resident tensors, enqueued on `stream`; `mask` is a device buffer of mask_len
// elements (t_q*t_kv or batch*heads*t_q*t_kv) or nullptr.
inline void mha_forward_masked_f32_dev(const float* q, const float* k, const float* v, float* out, size_t batch,
                                       size_t t_q, size_t t_kv, size_t heads, size_t head_dim,
                                       const float* mask = nullptr, size_t mask_len = 0, void* stream = nullptr) {
    rt_err_detail e;
    int rc = rt_mha_forward_masked_f32_dev(stream, q, k, v, mask, mask_len, out, batch, t_q, t_kv, heads, head_dim, &e);
    if (rc == RT_ERR_WRONG_INPUT_LEN) detail::check_gqa(rc, e);  // which = "mask"
    detail::check_attention(rc, e);
}

// The same composed path on bf16 device tensors (bit patterns, [B,t,H*hd]) with an f32 device mask; bf16 out.
inline void mha_forward_masked_bf16_dev(const void* q, const void* k, const void* v, void* out, size_t batch, size_t t_q,
                                        size_t t_kv, size_t heads, size_t head_dim, const float* mask = nullptr,
                                        size_t mask_len = 0, void* stream = nullptr) {
    rt_err_detail e;
    int rc = rt_mha_forward_masked_bf16_dev(stream, q, k, v, mask, mask_len, out, batch, t_q, t_kv, heads, head_dim, &e);
    if (rc == RT_ERR_WRONG_INPUT_LEN) detail::check_gqa(rc, e);  // which = "mask"
    detail::check_attention(rc, e);
}

// The branch MultiHeadAttention::forward takes for the attention between its projections, under no_grad on contiguous
// f32 tensors (attention.rs:325-333, :347-356).
enum class MhaRoute { Identity, Flash, Composed };
inline MhaRoute mha_attention_route(size_t t_q, size_t t_kv, bool has_mask) {
    if (!has_mask && t_q == 1 && t_kv == 1) return MhaRoute::Identity;  // softmax over one position is 1
    if (!has_mask && t_q == t_kv) return MhaRoute::Flash;
    return MhaRoute::Composed;
}
// Projected q [B,t_q,H*hd], k, v [B,t_kv,H*hd] -> context [B,t_q,H*hd] with that routing.
inline std::vector<float> mha_attention_f32(const std::vector<float>& q, const std::vector<float>& k,
                                            const std::vector<float>& v, size_t batch, size_t t_q, size_t t_kv,
                                            size_t heads, size_t head_dim,
                                            const std::vector<float>& attn_mask = std::vector<float>()) {
    switch (mha_attention_route(t_q, t_kv, !attn_mask.empty())) {
        case MhaRoute::Identity: return v;
        case MhaRoute::Flash: return mha_flash_forward_f32(q, k, v, batch, t_q, heads, head_dim);
        default: return mha_forward_masked_f32(q, k, v, batch, t_q, t_kv, heads, head_dim, attn_mask);
    }
}

// ---- device memory --------------------------------------------------------------------------------------

class HipStorage {
public:
    HipStorage() = default;
    explicit HipStorage(size_t bytes) : bytes_(bytes) {
        rt_err_detail e;
        ptr_ = rt_buf_alloc(bytes, &e);
        if (!ptr_ && bytes) detail::throw_device(e.hip_error ? RT_ERR_HIP : RT_ERR_NO_DEVICE, e);
    }
    template <typename T>
    static HipStorage from_host(const std::vector<T>& host) {
        HipStorage s(host.size() * sizeof(T));
        s.upload(host.data(), host.size() * sizeof(T));
        return s;
    }
    HipStorage(const HipStorage&) = delete;
    HipStorage& operator=(const HipStorage&) = delete;
    HipStorage(HipStorage&& o) noexcept : ptr_(o.ptr_), bytes_(o.bytes_) { o.ptr_ = nullptr; o.bytes_ = 0; }
    HipStorage& operator=(HipStorage&& o) noexcept {
        if (this != &o) {
            release();
            ptr_ = o.ptr_;
            bytes_ = o.bytes_;
            o.ptr_ = nullptr;
            o.bytes_ = 0;
        }
        return *this;
    }
    ~HipStorage() { release(); }
    void* ptr() const { return ptr_; }
    size_t byte_len() const { return bytes_; }
    void upload(const void* src, size_t bytes, void* stream = nullptr) {
        rt_err_detail e;
        detail::check_device(rt_memcpy_h2d(ptr_, src, bytes, stream, &e), e);
    }
    void download(void* dst, size_t bytes, void* stream = nullptr) const {
        rt_err_detail e;
        detail::check_device(rt_memcpy_d2h(dst, ptr_, bytes, stream, &e), e);
    }
    template <typename T>
    std::vector<T> to_host() const {
        std::vector<T> h(bytes_ / sizeof(T));
        download(h.data(), h.size() * sizeof(T));
        return h;
    }

private:
    void release() {
        if (ptr_) (void)rt_buf_free(ptr_, nullptr);
        ptr_ = nullptr;
    }
    void* ptr_ = nullptr;
    size_t bytes_ = 0;
};

// A stream at the default priority (the place of the reference's Arc<CudaStream>); get() is what the device entry
// points take.
class Stream {
public:
    Stream() {
        rt_err_detail e;
        h_ = rt_stream_create(&e);
        if (!h_) detail::throw_device(e.hip_error ? RT_ERR_HIP : RT_ERR_NO_DEVICE, e);
    }
    Stream(const Stream&) = delete;
    Stream& operator=(const Stream&) = delete;
    ~Stream() {
        rt_err_detail e;
        if (h_) (void)rt_stream_destroy(h_, &e);
    }
    void* get() const { return h_; }

private:
    void* h_ = nullptr;
};

inline void synchronize(void* stream = nullptr) {
    rt_err_detail e;
    detail::check_device(rt_stream_synchronize(stream, &e), e);
}

// ---- device-resident prefill (bf16 bit patterns) ------------------------------------------------------------

inline void flash_forward_bf16_dev(const AttentionShape& shape, const void* q, const void* k, const void* v, void* out,
                                   Mask::Kind mask = Mask::Kind::None, const uint8_t* keep_dev = nullptr,
                                   size_t n_kv_heads = 0, void* stream = nullptr) {
    rt_attention_shape s = shape.c();
    rt_err_detail e;
    detail::check_attention(rt_flash_forward_bf16_dev(stream, &s, n_kv_heads, q, k, v, (int)mask, keep_dev, out, &e), e);
}
inline void flash_forward_varlen_bf16_dev(const AttentionShape& shape, const void* q, const void* k, const void* v,
                                          const int32_t* seq_lens_dev, void* out, bool zero_padded_rows = true,
                                          size_t n_kv_heads = 0, void* stream = nullptr) {
    rt_attention_shape s = shape.c();
    rt_err_detail e;
    detail::check_attention(
        rt_flash_forward_varlen_bf16_dev(stream, &s, n_kv_heads, q, k, v, seq_lens_dev, zero_padded_rows ? 1 : 0, out, &e),
        e);
}

// Causal attention with a sliding window (key j visible to query i iff j <= i and i - j < window: sliding_window_mask,
// crates/rustorch-nn/src/masks.rs:41-60) without the mask tensor; bnhd: [batch, seq, heads, dim] tensors.
inline void flash_forward_window_bf16_dev(const AttentionShape& shape, const void* q, const void* k, const void* v,
                                          void* out, size_t window, size_t n_kv_heads = 0, bool bnhd = false,
                                          void* stream = nullptr) {
    rt_attention_shape s = shape.c();
    rt_err_detail e;
    detail::check_attention(bnhd ? rt_flash_forward_window_bnhd_bf16_dev(stream, &s, n_kv_heads, q, k, v, window, out, &e)
                                 : rt_flash_forward_window_bf16_dev(stream, &s, n_kv_heads, q, k, v, window, out, &e),
                            e);
}

// ---- device-resident f32 backward (cpu_backward.rs:46-185; the saved-forward form of its header comment) ----------

inline size_t flash_backward_workspace_bytes(const AttentionShape& shape) {
    rt_attention_shape s = shape.c();
    return rt_flash_backward_workspace_bytes(&s);
}
inline void flash_backward_f32_dev(const AttentionShape& shape, const float* q, const float* k, const float* v,
                                   const float* d_out, float* dq, float* dk, float* dv, void* workspace,
                                   size_t workspace_bytes, void* stream = nullptr) {
    rt_attention_shape s = shape.c();
    rt_err_detail e;
    detail::check_attention(
        rt_flash_backward_f32_dev(stream, &s, q, k, v, d_out, dq, dk, dv, workspace, workspace_bytes, &e), e);
}
// out and lse ([batch, heads, seq], m + ln l) as flash_forward_stats_f32_dev leaves them
inline void flash_forward_stats_f32_dev(const AttentionShape& shape, const float* q, const float* k, const float* v,
                                        float* out, float* lse, void* stream = nullptr) {
    rt_attention_shape s = shape.c();
    rt_err_detail e;
    detail::check_attention(rt_flash_forward_stats_f32_dev(stream, &s, q, k, v, out, lse, &e), e);
}
// workspace: batch * heads * seq floats
inline void flash_backward_saved_f32_dev(const AttentionShape& shape, const float* q, const float* k, const float* v,
                                         const float* out, const float* lse, const float* d_out, float* dq, float* dk,
                                         float* dv, void* workspace, size_t workspace_bytes, void* stream = nullptr) {
    rt_attention_shape s = shape.c();
    rt_err_detail e;
    detail::check_attention(rt_flash_backward_saved_f32_dev(stream, &s, q, k, v, out, lse, d_out, dq, dk, dv, workspace,
                                                            workspace_bytes, &e),
                            e);
}

// ---- KVCache (crates/rustorch-nn/src/kv_cache.rs:49-256) with its buffers in HBM ---------------------------
//
// Same protocol as the reference: append(layer, seq_added, new_k, new_v) for every layer, then advance(seq_added).
// Buffers are [batch, n_heads, max_seq, head_dim] of 2-byte (bf16, the decode kernels' storage) or 4-byte (f32)
// elements, zero-filled at construction; new_k / new_v are device buffers and their element counts are checked
// as the reference checks slice lengths.  k_buffer / v_buffer are what the decode entry points take as caches.
class KVCache {
public:
    KVCache(size_t num_layers, size_t batch, size_t n_heads, size_t head_dim, size_t max_seq, size_t elem_bytes = 2)
        : batch_(batch), n_heads_(n_heads), head_dim_(head_dim), max_seq_(max_seq), elem_bytes_(elem_bytes) {
        const size_t bytes = batch * n_heads * max_seq * head_dim * elem_bytes;
        for (size_t i = 0; i < num_layers; i++) {
            k_.emplace_back(bytes);
            v_.emplace_back(bytes);
            rt_err_detail e;
            detail::check_device(rt_buf_zero(k_.back().ptr(), bytes, nullptr, &e), e);
            detail::check_device(rt_buf_zero(v_.back().ptr(), bytes, nullptr, &e), e);
        }
    }
    size_t num_layers() const { return k_.size(); }
    size_t max_seq() const { return max_seq_; }
    size_t current_len() const { return current_len_; }
    void clear() { current_len_ = 0; }
    void append(size_t layer_idx, size_t seq_added, const HipStorage& new_k, const HipStorage& new_v, void* stream = nullptr) {
        if (layer_idx >= k_.size()) throw KVCacheLayerOutOfRange(layer_idx, k_.size());
        rt_err_detail e;
        detail::check_prepare(
            rt_kv_cache_append_dev(stream, k_[layer_idx].ptr(), v_[layer_idx].ptr(), new_k.ptr(), new_k.byte_len() / elem_bytes_,
                                   new_v.ptr(), new_v.byte_len() / elem_bytes_, batch_, n_heads_, max_seq_, head_dim_,
                                   current_len_, seq_added, elem_bytes_, &e),
            e);
    }
    void advance(size_t seq_added) {
        if (current_len_ + seq_added > max_seq_) throw KVCacheOverflow(current_len_ + seq_added, max_seq_);
        current_len_ += seq_added;
    }
    const HipStorage* k_buffer(size_t layer_idx) const { return layer_idx < k_.size() ? &k_[layer_idx] : nullptr; }
    const HipStorage* v_buffer(size_t layer_idx) const { return layer_idx < v_.size() ? &v_[layer_idx] : nullptr; }
    std::array<size_t, 4> dims() const { return {batch_, n_heads_, max_seq_, head_dim_}; }

private:
    size_t batch_, n_heads_, head_dim_, max_seq_, elem_bytes_, current_len_ = 0;
    std::vector<HipStorage> k_, v_;
};

// ---- RoPE tables (crates/rustorch-nn/src/rope.rs:33-90) ----------------------------------------------------
//
// RoPE::new: theta_k = 1 / base^(2k / head_dim), angle = p * theta_k, cos and sin per (position, k), all in f32.
// The tables are uploaded on first use and read by LlmKernels::qk_norm_rope_kv_append_bf16.
class RoPE {
public:
    RoPE(size_t head_dim, size_t max_seq, float base = 10000.0f) : head_dim_(head_dim), max_seq_(max_seq) {
        if (head_dim % 2 != 0) throw std::invalid_argument("RoPE: head_dim must be even, got " + std::to_string(head_dim));
        const size_t half = head_dim / 2;
        cos_.resize(max_seq * half);
        sin_.resize(max_seq * half);
        for (size_t p = 0; p < max_seq; p++)
            for (size_t k = 0; k < half; k++) {
                const float inv_theta = 1.0f / std::pow(base, (float)(2 * k) / (float)head_dim);
                const float angle = (float)p * inv_theta;
                cos_[p * half + k] = std::cos(angle);
                sin_[p * half + k] = std::sin(angle);
            }
    }
    size_t head_dim() const { return head_dim_; }
    size_t max_seq() const { return max_seq_; }
    const std::vector<float>& cos_table() const { return cos_; }
    const std::vector<float>& sin_table() const { return sin_; }
    const void* device_cos() { upload(); return dcos_.ptr(); }
    const void* device_sin() { upload(); return dsin_.ptr(); }

private:
    void upload() {
        if (dcos_.ptr() || cos_.empty()) return;
        dcos_ = HipStorage::from_host(cos_);
        dsin_ = HipStorage::from_host(sin_);
    }
    size_t head_dim_, max_seq_;
    std::vector<float> cos_, sin_;
    HipStorage dcos_, dsin_;
};

// ---- LlmKernels: the attention launchers (llm_kernels.rs:874-958), raw device addresses and i32 dims ----------

struct LlmKernels {
    static void kv_append_bf16(void* stream, void* k_cache, void* v_cache, const void* k_in, const void* v_in, int32_t pos,
                               int32_t n_kv, int32_t head_dim, int32_t max_seq) {
        rt_err_detail e;
        detail::check_device(rt_kv_append_bf16(stream, k_cache, v_cache, k_in, v_in, pos, n_kv, head_dim, max_seq, &e), e);
    }
    // Steps 2a, 2b, 3 of LlamaModel::decode_step (crates/rustorch-llm/src/model.rs:575-636) in one launch: per-head
    // q/k RMSNorm (device f32 gammas or nullptr), half-split RoPE, cache append, for `seq` new tokens per sequence
    // ([batch, heads, seq, head_dim] buffers; 1 when decoding).  `positions` is a device int32[batch] array (position
    // of each sequence's first new token), or nullptr to use `pos` for every sequence (then checked here, like the
    // reference).
    static void qk_norm_rope_kv_append_bf16(void* stream, void* q, const void* k_in, const void* v_in, void* k_cache,
                                            void* v_cache, const int32_t* positions, int32_t pos, const float* q_gamma,
                                            const float* k_gamma, float eps, RoPE& rope, int32_t batch, int32_t n_heads,
                                            int32_t n_kv, int32_t head_dim, int32_t max_seq, int32_t seq = 1) {
        if (!positions) {  // the reference's checks, before anything touches the device (rope.rs:179-184, kv_cache.rs:84-89)
            const int64_t end = (int64_t)pos + seq;
            if (pos < 0 || end > (int64_t)rope.max_seq())
                throw RoPEError(RoPEError::Kind::PositionOverflow, rope.max_seq(), (size_t)end,
                                "rope: position " + std::to_string(end) + " exceeds max_seq " + std::to_string(rope.max_seq()));
            if (end > max_seq) throw KVCacheOverflow((size_t)end, (size_t)max_seq);
        }
        rt_err_detail e;
        detail::check_prepare(
            rt_qk_norm_rope_kv_append_bf16(stream, q, k_in, v_in, k_cache, v_cache, positions, pos, q_gamma, k_gamma, eps,
                                           (const float*)rope.device_cos(), (const float*)rope.device_sin(),
                                           (int32_t)rope.max_seq(), batch, seq, n_heads, n_kv, head_dim, max_seq, &e),
            e);
    }
    static void gqa_decode_online_bf16(void* stream, const void* q, const void* k_cache, const void* v_cache, void* out,
                                       int32_t n_heads, int32_t n_kv, int32_t kv_len, int32_t head_dim, int32_t max_seq) {
        rt_err_detail e;
        detail::check_gqa(
            rt_gqa_decode_online_bf16(stream, q, k_cache, v_cache, out, n_heads, n_kv, kv_len, head_dim, max_seq, &e), e);
    }
    // llm_kernels.rs:990-1042: the three-pass launcher of the same function
    static void gqa_decode_naive_bf16(void* stream, const void* q, const void* k_cache, const void* v_cache, void* out,
                                      int32_t n_heads, int32_t n_kv, int32_t kv_len, int32_t head_dim, int32_t max_seq) {
        rt_err_detail e;
        detail::check_gqa(
            rt_gqa_decode_naive_bf16(stream, q, k_cache, v_cache, out, n_heads, n_kv, kv_len, head_dim, max_seq, &e), e);
    }
    static size_t gqa_decode_workspace_bytes(int32_t batch, int32_t n_heads, int32_t n_kv, int32_t head_dim,
                                             int32_t max_seq) {
        return rt_gqa_decode_workspace_bytes(batch, n_heads, n_kv, head_dim, max_seq);
    }
    static void gqa_decode_batched_bf16(void* stream, const void* q, const void* k_cache, const void* v_cache, void* out,
                                        const int32_t* kv_lens, int32_t batch, int32_t n_heads, int32_t n_kv,
                                        int32_t head_dim, int32_t max_seq, void* workspace, size_t workspace_bytes) {
        rt_err_detail e;
        detail::check_gqa(rt_gqa_decode_batched_bf16(stream, q, k_cache, v_cache, out, kv_lens, batch, n_heads, n_kv,
                                                     head_dim, max_seq, workspace, workspace_bytes, &e),
                          e);
    }
    // The same without a workspace: the partials go to a fixed block of device memory inside the library, and the call
    // allocates nothing (for callers under graph capture or in loops that must not allocate).
    static void gqa_decode_batched_bf16_noalloc(void* stream, const void* q, const void* k_cache, const void* v_cache,
                                                void* out, const int32_t* kv_lens, int32_t batch, int32_t n_heads,
                                                int32_t n_kv, int32_t head_dim, int32_t max_seq) {
        rt_err_detail e;
        detail::check_gqa(rt_gqa_decode_batched_bf16_noalloc(stream, q, k_cache, v_cache, out, kv_lens, batch, n_heads,
                                                             n_kv, head_dim, max_seq, &e),
                          e);
    }
    // gqa_decode_batched_f32 (crates/rustorch-metal/src/kernels.rs:14432-14516) in bf16 over a batch: seq_new consecutive
    // new positions per sequence, position s seeing keys [0, kv_lens[b] - seq_new + s]; q/out [B,seq_new,Hq,D].
    // kv_lens == nullptr: every sequence has kv_len keys.
    static void gqa_decode_chunk_bf16(void* stream, const void* q, const void* k_cache, const void* v_cache, void* out,
                                      const int32_t* kv_lens, int32_t kv_len, int32_t batch, int32_t seq_new,
                                      int32_t n_heads, int32_t n_kv, int32_t head_dim, int32_t max_seq) {
        rt_err_detail e;
        detail::check_gqa(rt_gqa_decode_chunk_bf16(stream, q, k_cache, v_cache, out, kv_lens, kv_len, batch, seq_new,
                                                   n_heads, n_kv, head_dim, max_seq, &e),
                          e);
    }
    // No counterpart in the reference: adds `delta` to n int32 values on the device, on `stream` -- the positions and
    // context lengths of a decode loop recorded into a HIP graph advance inside the graph.
    static void i32_add_dev(void* stream, int32_t* values, size_t n, int32_t delta) {
        rt_err_detail e;
        detail::check_gqa(rt_i32_add_dev(stream, values, n, delta, &e), e);
    }
};

// Process-wide: causal prefill entries follow their kernel with a pass that gives rows the reference's NaN for
// non-finite V elements at keys they do not see (cpu_forward.rs:268-425 multiplies the hidden zeros into every V tile).
// Returns the previous setting.
inline bool set_strict_non_finite_v(bool on) { return rt_set_strict_non_finite_v(on ? 1 : 0) != 0; }

}  // namespace rustorch_attn

#endif  // RUSTORCH_ATTN_HPP
