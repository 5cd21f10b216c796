// C ABI of librt_attn_hip.so (declared in include/rt_attn.h): argument checks in the
// reference's order, device selection, host staging for the slice entry points, kernel dispatch.
// There is no CPU path in this library.
#include <dlfcn.h>
#include <hip/hip_runtime.h>
#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <algorithm>
#include <atomic>
#include <map>
#include <mutex>
#include <vector>

#include "../../include/rt_attn.h"
#include "rt_kernels.hpp"

#define RT_API extern "C" __attribute__((visibility("default")))

namespace {

void clear_err(rt_err_detail* e) {
    if (e) {
        e->which = -1;
        e->expected = e->got = e->got2 = 0;
        e->hip_error = 0;
        e->message[0] = 0;
    }
}

int fail(rt_err_detail* e, int status, int which, uint64_t expected, uint64_t got, const char* msg, uint64_t got2 = 0) {
    if (e) {
        e->which = which;
        e->expected = expected;
        e->got = got;
        e->got2 = got2;
        e->hip_error = 0;
        snprintf(e->message, sizeof(e->message), "%s", msg ? msg : "");
    }
    return status;
}

int fail_hip(rt_err_detail* e, hipError_t code, const char* where) {
    if (e) {
        e->which = -1;
        e->expected = e->got = e->got2 = 0;
        e->hip_error = (int32_t)code;
        snprintf(e->message, sizeof(e->message), "%s: %s", where, hipGetErrorString(code));
    }
    return RT_ERR_HIP;
}

#define HIP_TRY(expr, where)                                  \
    do {                                                      \
        hipError_t _e = (expr);                               \
        if (_e != hipSuccess) return fail_hip(err, _e, where); \
    } while (0)

int g_num_cus = 0;
int g_decode_waves = 0;  // one-wave workgroups one launch of the decode kernel keeps resident
std::mutex g_init_mutex;
int g_init_status = -1;  // -1: not tried
char g_init_msg[160];

// Finds a gfx950 device once per process.  Never falls back to anything else.
int ensure_device(rt_err_detail* err, int device = -1) {
    std::lock_guard<std::mutex> lock(g_init_mutex);
    if (g_init_status == RT_OK && device < 0) return RT_OK;
    int count = 0;
    hipError_t e = hipGetDeviceCount(&count);
    if (e != hipSuccess || count == 0) {
        (void)hipGetLastError();
        snprintf(g_init_msg, sizeof(g_init_msg), "no HIP device visible (%s)",
                 e == hipSuccess ? "count is 0" : hipGetErrorString(e));
        g_init_status = RT_ERR_NO_DEVICE;
        return fail(err, RT_ERR_NO_DEVICE, -1, 0, 0, g_init_msg);
    }
    int dev = device >= 0 ? device : 0;
    if (device < 0) (void)hipGetDevice(&dev);
    if (dev >= count) {
        snprintf(g_init_msg, sizeof(g_init_msg), "device %d requested, %d visible", dev, count);
        return fail(err, RT_ERR_NO_DEVICE, -1, (uint64_t)count, (uint64_t)dev, g_init_msg);
    }
    hipDeviceProp_t prop;
    e = hipGetDeviceProperties(&prop, dev);
    if (e != hipSuccess) return fail_hip(err, e, "hipGetDeviceProperties");
    if (strncmp(prop.gcnArchName, "gfx950", 6) != 0) {
        snprintf(g_init_msg, sizeof(g_init_msg), "device %d is %s; this library holds gfx950 code only", dev,
                 prop.gcnArchName);
        g_init_status = RT_ERR_NO_DEVICE;
        return fail(err, RT_ERR_NO_DEVICE, -1, 0, 0, g_init_msg);
    }
    if (device >= 0) {
        e = hipSetDevice(dev);
        if (e != hipSuccess) return fail_hip(err, e, "hipSetDevice");
    }
    // the decode kernel (one wave, ~18 KB LDS, <= 256 VGPRs) fits 8 times on a CU; one wave per SIMD already
    // streams at the rate the memory system gives, and fewer waves leave fewer partials to merge
    g_num_cus = prop.multiProcessorCount;
    g_decode_waves = prop.multiProcessorCount * 4;
    g_init_status = RT_OK;
    return RT_OK;
}

// validate() of cpu_forward.rs:142-169 followed by Mask::validate (mask.rs:51-65)
int validate_flash(const rt_attention_shape* s, size_t qn, size_t kn, size_t vn, size_t on, int mask_kind,
                   size_t keep_n, rt_err_detail* err) {
    if (s->dim == 0) return fail(err, RT_ERR_ZERO_DIM, -1, 0, 0, "dim must be > 0");
    uint64_t expected = s->batch * s->heads * s->seq * s->dim;
    const size_t lens[3] = {qn, kn, vn};
    static const char* names[3] = {"q", "k", "v"};
    for (int i = 0; i < 3; i++)
        if (lens[i] != expected) {
            char msg[96];
            snprintf(msg, sizeof(msg), "%s buffer has %zu elements, expected %llu", names[i], lens[i],
                     (unsigned long long)expected);
            return fail(err, RT_ERR_BUFFER_SHAPE_MISMATCH, i, expected, lens[i], msg);
        }
    if (on != expected) return fail(err, RT_ERR_OUTPUT_SHAPE_MISMATCH, RT_WHICH_OUT, expected, on, "output buffer length");
    if (mask_kind == RT_MASK_PADDING && keep_n != s->seq)
        return fail(err, RT_ERR_PADDING_LENGTH_MISMATCH, -1, s->seq, keep_n, "padding mask length");
    if (mask_kind != RT_MASK_NONE && mask_kind != RT_MASK_CAUSAL && mask_kind != RT_MASK_PADDING)
        return fail(err, RT_ERR_UNSUPPORTED, -1, 0, (uint64_t)mask_kind, "unknown mask kind");
    return RT_OK;
}

bool fits_int(uint64_t x) { return x <= 0x7fffffffull; }

int check_flash_dims(const rt_attention_shape* s, uint64_t n_kv_heads, rt_err_detail* err) {
    if (!fits_int(s->batch) || !fits_int(s->heads) || !fits_int(s->seq) || !fits_int(s->dim) || s->batch > 65535 ||
        s->heads > 65535)
        return fail(err, RT_ERR_UNSUPPORTED, -1, 0, 0, "shape too large for the launch grid");
    if (n_kv_heads == 0 || s->heads % n_kv_heads != 0)
        return fail(err, RT_ERR_HEAD_COUNT_MISMATCH, -1, s->heads, n_kv_heads, "heads not divisible by n_kv_heads");
    return RT_OK;
}

// bnhd: tensors are [batch, seq, heads, dim] instead of [batch, heads, seq, dim]
// rt_set_strict_non_finite_v: off by default
std::atomic<int> g_strict_v{0};

// After a causal forward, when the strict switch is on: the pass that gives query rows the reference's NaN for
// non-finite V elements at keys they do not see (the forward kernels skip those key tiles).
int strict_pass(hipStream_t stream, const rt_attention_shape* s, uint64_t n_kv_heads, const void* v, void* out,
                const int32_t* seq_lens, int mask_kind, bool bnhd, bool bf16, rt_err_detail* err) {
    if (mask_kind != rt::kMaskCausal && mask_kind != rt::kMaskVarlenCausal) return RT_OK;
    if (!g_strict_v.load(std::memory_order_relaxed)) return RT_OK;
    rt::StrictVParams p{};
    p.v = v;
    p.out = out;
    p.seq_lens = seq_lens;
    p.batch = (int)s->batch;
    p.heads = (int)s->heads;
    p.kv_heads = (int)n_kv_heads;
    p.seq = (int)s->seq;
    p.dim = (int)s->dim;
    if (bnhd) {
        p.lo = rt::layout_bnhd((long long)s->heads, (long long)s->seq, p.dim);
        p.lkv = rt::layout_bnhd((long long)n_kv_heads, (long long)s->seq, p.dim);
    } else {
        p.lo = rt::layout_bhnd((long long)s->heads, (long long)s->seq, p.dim);
        p.lkv = rt::layout_bhnd((long long)n_kv_heads, (long long)s->seq, p.dim);
    }
    HIP_TRY(rt::launch_strict_hidden_v(stream, p, bf16), "strict_hidden_v launch");
    return RT_OK;
}

int flash_f32_device(hipStream_t stream, const rt_attention_shape* s, uint64_t n_kv_heads, const float* q,
                     const float* k, const float* v, int mask_kind, const uint8_t* keep, float* out,
                     rt_err_detail* err, bool bnhd = false, const float* bias = nullptr, long long bias_bh_stride = 0,
                     float* lse = nullptr, uint64_t seq_kv = 0) {
    if (s->dim > 512) return fail(err, RT_ERR_UNSUPPORTED, -1, 512, s->dim, "f32 flash kernels cover dim <= 512");
    if (s->dim > 256) {
        // beyond the tiled kernels: one workgroup per query row (any speed), with flash_forward's masks and row rules
        if (s->seq > 0x7fffffffull || seq_kv > 0x7fffffffull) return fail(err, RT_ERR_UNSUPPORTED, -1, 0, 0, "shape too large for the launch grid");
        rt::AttnRowsParams r{};
        r.q = q;
        r.k = k;
        r.v = v;
        r.out = out;
        r.batch = (int)s->batch;
        r.heads = (int)s->heads;
        r.kv_heads = (int)n_kv_heads;
        r.seq_q = (int)s->seq;
        r.kv_len = r.kv_stride = (int)(seq_kv ? seq_kv : s->seq);
        r.dim = (int)s->dim;
        r.head_map = 0;
        r.scale = 1.0f / sqrtf((float)s->dim);
        r.bias = bias;
        r.bias_bh_stride = bias_bh_stride;
        r.use_layout = 1;
        if (bnhd) {
            r.lq = r.lo = rt::layout_bnhd((long long)s->heads, (long long)s->seq, r.dim);
            r.lkv = rt::layout_bnhd((long long)n_kv_heads, (long long)r.kv_len, r.dim);
        } else {
            r.lq = r.lo = rt::layout_bhnd((long long)s->heads, (long long)s->seq, r.dim);
            r.lkv = rt::layout_bhnd((long long)n_kv_heads, (long long)r.kv_len, r.dim);
        }
        r.mask = mask_kind;
        r.keep = keep;
        r.ref_bc = (int)(s->bc == 0 ? 1 : (s->bc > 0x7fffffffull ? 0x7fffffff : s->bc));
        r.flash_rows = 1;
        r.lse = lse;
        HIP_TRY(rt::launch_attn_rows_f32(stream, r), "attn_rows_f32 launch");
        return seq_kv ? RT_OK : strict_pass(stream, s, n_kv_heads, v, out, nullptr, mask_kind, bnhd, false, err);
    }
    rt::FlashF32Params p{};
    p.bias = bias;
    p.bias_bh_stride = bias_bh_stride;
    p.lse = lse;
    p.q = q;
    p.k = k;
    p.v = v;
    p.out = out;
    p.keep = keep;
    p.batch = (int)s->batch;
    p.heads = (int)s->heads;
    p.kv_heads = (int)n_kv_heads;
    p.group = (int)(s->heads / n_kv_heads);
    p.seq = (int)s->seq;
    p.dim = (int)s->dim;
    p.seq_kv = (int)seq_kv;
    p.mask = mask_kind;
    p.ref_bc = (int)(s->bc == 0 ? 1 : (s->bc > 0x7fffffffull ? 0x7fffffff : s->bc));
    p.scale = 1.0f / sqrtf((float)s->dim);
    p.n_cus = g_num_cus;
    const long long kv_rows = (long long)(seq_kv ? seq_kv : s->seq);
    if (bnhd) {
        p.lq = p.lo = rt::layout_bnhd((long long)s->heads, (long long)s->seq, p.dim);
        p.lkv = rt::layout_bnhd((long long)n_kv_heads, kv_rows, p.dim);
    } else {
        p.lq = p.lo = rt::layout_bhnd((long long)s->heads, (long long)s->seq, p.dim);
        p.lkv = rt::layout_bhnd((long long)n_kv_heads, kv_rows, p.dim);
    }
    HIP_TRY(rt::launch_flash_f32(stream, p), "flash_fwd_f32 launch");
    return seq_kv ? RT_OK : strict_pass(stream, s, n_kv_heads, v, out, nullptr, mask_kind, bnhd, false, err);
}

// Scratch the library keeps for entry points whose reference signature has no workspace argument: one buffer per
// (device, stream), allocated on the first call that needs it and kept until rt_stream_destroy / rt_shutdown.
// Calls on one stream are ordered, so they can share it; calls on different streams get different buffers.  When a
// later call needs more, a larger block is allocated and the old one is RETIRED, not freed: another thread may have
// been handed the old pointer and not yet enqueued its kernels (the lock below covers the bookkeeping only, not
// the caller's launches), and kernels already enqueued may still use it.  Retired blocks are freed with the
// stream's entry.  The first call on a stream allocates (hipMalloc): not for use under stream capture.
struct StreamWs {
    void* ptr = nullptr;
    size_t bytes = 0;
    std::vector<void*> retired;
};
std::mutex g_ws_mutex;
std::map<std::pair<int, hipStream_t>, StreamWs> g_ws;

int stream_workspace(hipStream_t stream, size_t bytes, float** out, rt_err_detail* err) {
    int dev = 0;
    HIP_TRY(hipGetDevice(&dev), "hipGetDevice");
    std::lock_guard<std::mutex> lock(g_ws_mutex);
    StreamWs& w = g_ws[{dev, stream}];
    if (w.bytes < bytes) {
        // grow geometrically, so that a context that lengthens token by token retires a handful of blocks at most
        size_t want = std::max<size_t>(std::max<size_t>(bytes, (size_t)1 << 20), 2 * w.bytes);
        void* fresh = nullptr;
        HIP_TRY(hipMalloc(&fresh, want), "hipMalloc workspace");
        if (w.ptr) w.retired.push_back(w.ptr);
        w.ptr = fresh;
        w.bytes = want;
    }
    *out = (float*)w.ptr;
    return RT_OK;
}

// frees what a stream's entry holds; the caller holds g_ws_mutex and has made sure the stream is idle
void release_stream_ws(StreamWs& w) {
    if (w.ptr) (void)hipFree(w.ptr);
    for (void* r : w.retired) (void)hipFree(r);
    w.ptr = nullptr;
    w.bytes = 0;
    w.retired.clear();
}

// Scratch that needs no allocation: the library's second fixed block is cut into rt::kStreamSlots slots, and a
// (device, stream) pair is given one the first time it asks (host bookkeeping only: nothing is allocated, so the
// call may be the first one under stream capture).  A stream keeps its slot until rt_stream_destroy / rt_shutdown;
// when all slots are taken the caller falls back to stream_workspace.
struct SlotTable {
    hipStream_t owner[rt::kStreamSlots] = {};
    bool used[rt::kStreamSlots] = {};
};
std::map<int, SlotTable> g_slots;  // per device; guarded by g_ws_mutex

// The slot of `stream` on the current device (taking a free one if it has none yet): its scratch and size, or
// *ptr = nullptr when no slot is free.
int stream_slot_scratch(hipStream_t stream, float** ptr, size_t* bytes, rt_err_detail* err) {
    *ptr = nullptr;
    *bytes = 0;
    int dev = 0;
    HIP_TRY(hipGetDevice(&dev), "hipGetDevice");
    int slot = -1;
    {
        std::lock_guard<std::mutex> lock(g_ws_mutex);
        SlotTable& t = g_slots[dev];
        for (int i = 0; i < rt::kStreamSlots && slot < 0; i++)
            if (t.used[i] && t.owner[i] == stream) slot = i;
        for (int i = 0; i < rt::kStreamSlots && slot < 0; i++)
            if (!t.used[i]) {
                t.used[i] = true;
                t.owner[i] = stream;
                slot = i;
            }
    }
    if (slot < 0) return RT_OK;
    HIP_TRY(rt::stream_static_scratch(slot, ptr, bytes), "hipGetSymbolAddress(stream scratch)");
    return RT_OK;
}

// the caller holds g_ws_mutex
void release_stream_slot(int dev, hipStream_t stream) {
    auto it = g_slots.find(dev);
    if (it == g_slots.end()) return;
    for (int i = 0; i < rt::kStreamSlots; i++)
        if (it->second.used[i] && it->second.owner[i] == stream) it->second.used[i] = false;
}

struct DevPtr {  // a device address inside a Stage's block
    void* p = nullptr;
};

struct DevBuf {
    void* p = nullptr;
    ~DevBuf() {
        if (p) (void)hipFree(p);
    }
};

// Staging of one host-slice call: every input, output and scratch buffer of the call sits in ONE device block.
// Small calls (inputs + outputs within kPinnedBytes) travel through a pinned host buffer the library keeps, as one
// host-to-device and one device-to-host transfer: a pageable hipMemcpy costs about 60 us whatever its size below
// a megabyte, and a call has four of them.  One call at a time can hold the pinned buffer; a call that finds it
// taken (another thread is inside a host-slice entry) or that is larger copies buffer by buffer instead.
constexpr size_t kPinnedBytes = (size_t)4 << 20;
std::mutex g_pinned_mutex;
void* g_pinned = nullptr;

class Stage {
public:
    void in(const void* host, size_t bytes, void** dev) { items_.push_back({host, nullptr, bytes, dev, 0, 0}); }
    void out(void* host, size_t bytes, void** dev) { items_.push_back({nullptr, host, bytes, dev, 0, 1}); }
    void scratch(size_t bytes, void** dev) { items_.push_back({nullptr, nullptr, bytes, dev, 0, 2}); }

    // Allocates the block, hands out the device pointers and uploads the inputs (register inputs, then outputs,
    // then scratch).
    int commit(rt_err_detail* err) {
        size_t off = 0;
        for (auto& it : items_) {
            it.off = off;
            off += (it.bytes + 255) & ~(size_t)255;
            if (it.kind == 0) in_end_ = off;
            if (it.kind == 1) io_end_ = off;
        }
        if (io_end_ < in_end_) io_end_ = in_end_;
        HIP_TRY(hipMalloc(&block_.p, off ? off : 256), "hipMalloc staging block");
        for (auto& it : items_) *it.dev = (char*)block_.p + it.off;
        if (io_end_ <= kPinnedBytes) {
            lock_ = std::unique_lock<std::mutex>(g_pinned_mutex, std::try_to_lock);
            if (lock_.owns_lock() && !g_pinned && hipHostMalloc(&g_pinned, kPinnedBytes, hipHostMallocDefault) != hipSuccess) {
                (void)hipGetLastError();
                g_pinned = nullptr;
                lock_.unlock();
            }
        }
        if (lock_.owns_lock()) {
            for (auto& it : items_)
                if (it.kind == 0 && it.bytes) memcpy((char*)g_pinned + it.off, it.host_in, it.bytes);
            if (in_end_) HIP_TRY(hipMemcpyAsync(block_.p, g_pinned, in_end_, hipMemcpyHostToDevice, nullptr), "upload");
        } else {
            for (auto& it : items_)
                if (it.kind == 0 && it.bytes)
                    HIP_TRY(hipMemcpy((char*)block_.p + it.off, it.host_in, it.bytes, hipMemcpyHostToDevice), "copy input");
        }
        return RT_OK;
    }

    // Brings the outputs back; returns after they are in the caller's buffers.
    int fetch(rt_err_detail* err) {
        fetched_ = true;  // every path below ends with the stream idle (or reports the failure of the attempt)
        if (lock_.owns_lock()) {
            if (io_end_ > in_end_)
                HIP_TRY(hipMemcpyAsync((char*)g_pinned + in_end_, (char*)block_.p + in_end_, io_end_ - in_end_,
                                       hipMemcpyDeviceToHost, nullptr),
                        "download");
            HIP_TRY(hipStreamSynchronize(nullptr), "hipStreamSynchronize");
            for (auto& it : items_)
                if (it.kind == 1 && it.bytes) memcpy(it.host_out, (char*)g_pinned + it.off, it.bytes);
        } else {
            for (auto& it : items_)
                if (it.kind == 1 && it.bytes)
                    HIP_TRY(hipMemcpy(it.host_out, (char*)block_.p + it.off, it.bytes, hipMemcpyDeviceToHost), "copy output");
        }
        return RT_OK;
    }

    ~Stage() {
        // an early return (a failed launch) may leave work in flight that still reads the block or the pinned buffer
        if (block_.p && !fetched_) (void)hipStreamSynchronize(nullptr);
    }

private:
    struct Item {
        const void* host_in;
        void* host_out;
        size_t bytes;
        void** dev;
        size_t off;
        int kind;  // 0 input, 1 output, 2 scratch
    };
    std::vector<Item> items_;
    size_t in_end_ = 0, io_end_ = 0;
    bool fetched_ = false;
    std::unique_lock<std::mutex> lock_;  // declared before block_: the block is freed first, then the pinned buffer released
    DevBuf block_;
};

}  // namespace

RT_API const char* rt_version(void) { return "rt_attn_hip 0.1 (gfx950)"; }

// The file the HIP runtime this library is bound to was loaded from.  A host that wants streams, events or graphs of
// its own must talk to the same runtime instance; a process can hold a second copy (PyTorch wheels ship one), and a
// dlopen by bare name may return that one, whose calls do not know this library's streams.
RT_API const char* rt_hip_runtime_path(void) {
    Dl_info info;
    if (dladdr((void*)&hipGetDeviceCount, &info) && info.dli_fname) return info.dli_fname;
    return "";
}

RT_API const char* rt_status_name(int status) {
    switch (status) {
        case RT_OK: return "Ok";
        case RT_ERR_ZERO_DIM: return "ZeroDim";
        case RT_ERR_BUFFER_SHAPE_MISMATCH: return "BufferShapeMismatch";
        case RT_ERR_OUTPUT_SHAPE_MISMATCH: return "OutputShapeMismatch";
        case RT_ERR_PADDING_LENGTH_MISMATCH: return "PaddingLengthMismatch";
        case RT_ERR_HEAD_COUNT_MISMATCH: return "HeadCountMismatch";
        case RT_ERR_WRONG_INPUT_LEN: return "WrongInputLen";
        case RT_ERR_KV_OVERFLOW: return "Overflow";
        case RT_ERR_KV_WRONG_INPUT_LEN: return "KvWrongInputLen";
        case RT_ERR_ROPE_WRONG_INPUT_LEN: return "RopeWrongInputLen";
        case RT_ERR_ROPE_POSITION_OVERFLOW: return "PositionOverflow";
        case RT_ERR_NULL_POINTER: return "NullPointer";
        case RT_ERR_UNSUPPORTED: return "Unsupported";
        case RT_ERR_WORKSPACE_TOO_SMALL: return "WorkspaceTooSmall";
        case RT_ERR_NO_DEVICE: return "NoDeviceFound";
        case RT_ERR_HIP: return "Driver";
        default: return "Unknown";
    }
}

RT_API int rt_init(int device, rt_err_detail* err) {
    clear_err(err);
    int rc = ensure_device(err, device < 0 ? 0 : device);
    if (rc) return rc;
    // the address of the library's fixed scratch block on this device, looked up here so that the first call of
    // rt_gqa_decode_batched_bf16_noalloc has nothing left to set up
    float* scratch = nullptr;
    size_t scratch_bytes = 0;
    HIP_TRY(rt::decode_static_scratch(&scratch, &scratch_bytes), "hipGetSymbolAddress(static scratch)");
    HIP_TRY(rt::stream_static_scratch(0, &scratch, &scratch_bytes), "hipGetSymbolAddress(stream scratch)");
    return RT_OK;
}

// ---- prefill, host slices -------------------------------------------------------------------------

RT_API int rt_flash_forward_masked_f32(const rt_attention_shape* shape, const float* q, size_t q_len, const float* k,
                                       size_t k_len, const float* v, size_t v_len, int mask_kind,
                                       const uint8_t* keep, size_t keep_len, float* out, size_t out_len,
                                       rt_err_detail* err) {
    clear_err(err);
    if (!shape) return fail(err, RT_ERR_NULL_POINTER, -1, 0, 0, "shape is NULL");
    int rc = validate_flash(shape, q_len, k_len, v_len, out_len, mask_kind, keep_len, err);
    if (rc) return rc;
    if (shape->seq == 0) return RT_OK;  // cpu_forward.rs:203-206
    size_t n = q_len;
    if (n == 0) return RT_OK;  // batch or heads is 0
    if (!q || !k || !v || !out || (mask_kind == RT_MASK_PADDING && !keep))
        return fail(err, RT_ERR_NULL_POINTER, -1, 0, 0, "NULL buffer");
    rc = check_flash_dims(shape, shape->heads, err);
    if (rc) return rc;
    rc = ensure_device(err);
    if (rc) return rc;

    Stage st;
    void *dq, *dk, *dv, *dout, *dkeep = nullptr;
    size_t bytes = n * sizeof(float);
    st.in(q, bytes, &dq);
    st.in(k, bytes, &dk);
    st.in(v, bytes, &dv);
    if (mask_kind == RT_MASK_PADDING) st.in(keep, keep_len, &dkeep);
    st.out(out, bytes, &dout);
    rc = st.commit(err);
    if (rc) return rc;
    rc = flash_f32_device(nullptr, shape, shape->heads, (const float*)dq, (const float*)dk, (const float*)dv, mask_kind,
                          (const uint8_t*)dkeep, (float*)dout, err);
    if (rc) return rc;
    return st.fetch(err);
}

RT_API int rt_flash_forward_f32(const rt_attention_shape* shape, const float* q, size_t q_len, const float* k,
                                size_t k_len, const float* v, size_t v_len, float* out, size_t out_len,
                                rt_err_detail* err) {
    return rt_flash_forward_masked_f32(shape, q, q_len, k, k_len, v, v_len, RT_MASK_NONE, nullptr, 0, out, out_len,
                                       err);
}

namespace {

// The attention of rt_gqa_forward_f32 on device-resident tensors (arguments already checked).
int gqa_device(hipStream_t stream, const float* q, const float* k, const float* v, float* out, size_t batch,
               size_t n_heads, size_t n_kv_heads, size_t seq_q, size_t seq_kv, size_t head_dim, rt_err_detail* err) {
    auto aligned16 = [](const void* ptr) { return ((uintptr_t)ptr & 15) == 0; };
    if (seq_q == seq_kv) {
        // prefill: unmasked flash; the kernel maps query head -> kv head itself (no replicated copy)
        rt_attention_shape s = {batch, n_heads, seq_q, head_dim, 64, 64};
        return flash_f32_device(stream, &s, n_kv_heads, q, k, v, RT_MASK_NONE, nullptr, out, err);
    }
    if (seq_kv > 0 && head_dim % 4 == 0 && head_dim <= 128 && aligned16(q) && aligned16(k) && aligned16(v) &&
        aligned16(out)) {
        // decode / chunked prefill: every query row attends to all seq_kv keys (gqa.rs:179-208); the tiled kernel
        // with its own key count
        rt_attention_shape s = {batch, n_heads, seq_q, head_dim, 64, 64};
        return flash_f32_device(stream, &s, n_kv_heads, q, k, v, RT_MASK_NONE, nullptr, out, err, false, nullptr, 0,
                                nullptr, seq_kv);
    }
    if (head_dim > 512) return fail(err, RT_ERR_UNSUPPORTED, -1, 512, head_dim, "decode rows kernel covers dim <= 512");
    if (seq_q > 65535 * 32ull) return fail(err, RT_ERR_UNSUPPORTED, -1, 0, seq_q, "seq_q too large");
    rt::AttnRowsParams p{};
    p.q = q;
    p.k = k;
    p.v = v;
    p.out = out;
    p.kv_lens = nullptr;
    p.batch = (int)batch;
    p.heads = (int)n_heads;
    p.kv_heads = (int)n_kv_heads;
    p.seq_q = (int)seq_q;
    p.kv_len = (int)seq_kv;
    p.kv_stride = (int)seq_kv;
    p.dim = (int)head_dim;
    p.head_map = 0;
    p.scale = 1.0f / sqrtf((float)head_dim);
    HIP_TRY(rt::launch_attn_rows_f32(stream, p), "attn_rows_f32 launch");
    return RT_OK;
}

}  // namespace

RT_API int rt_gqa_forward_f32(const float* q, size_t q_len, const float* k, size_t k_len, const float* v,
                              size_t v_len, float* out, size_t out_len, size_t batch, size_t n_heads,
                              size_t n_kv_heads, size_t seq_q, size_t seq_kv, size_t head_dim, rt_err_detail* err) {
    clear_err(err);
    // gqa.rs:106-141
    if (n_kv_heads == 0 || n_heads % n_kv_heads != 0)
        return fail(err, RT_ERR_HEAD_COUNT_MISMATCH, -1, n_heads, n_kv_heads, "n_heads not divisible by n_kv_heads");
    size_t q_expected = batch * n_heads * seq_q * head_dim;
    size_t kv_expected = batch * n_kv_heads * seq_kv * head_dim;
    if (q_len != q_expected) return fail(err, RT_ERR_WRONG_INPUT_LEN, RT_WHICH_Q, q_expected, q_len, "q length");
    if (k_len != kv_expected) return fail(err, RT_ERR_WRONG_INPUT_LEN, RT_WHICH_K, kv_expected, k_len, "k length");
    if (v_len != kv_expected) return fail(err, RT_ERR_WRONG_INPUT_LEN, RT_WHICH_V, kv_expected, v_len, "v length");
    if (out_len != q_expected) return fail(err, RT_ERR_WRONG_INPUT_LEN, RT_WHICH_OUT, q_expected, out_len, "out length");
    if (seq_q == seq_kv && head_dim == 0)
        // the prefill branch's flash_forward fails with ZeroDim, reported as WrongInputLen{"flash_forward",0,0} (gqa.rs:171-175)
        return fail(err, RT_ERR_WRONG_INPUT_LEN, RT_WHICH_FLASH, 0, 0, "flash_forward");
    if (q_expected == 0) return RT_OK;
    if (!q || !out || (kv_expected && (!k || !v))) return fail(err, RT_ERR_NULL_POINTER, -1, 0, 0, "NULL buffer");
    if (!fits_int(batch) || !fits_int(n_heads) || !fits_int(seq_q) || !fits_int(seq_kv) || !fits_int(head_dim) ||
        batch > 65535 || n_heads > 65535)
        return fail(err, RT_ERR_UNSUPPORTED, -1, 0, 0, "shape too large for the launch grid");
    int rc = ensure_device(err);
    if (rc) return rc;

    Stage st;
    DevPtr dq, dk, dv, dout;
    st.in(q, q_expected * 4, &dq.p);
    st.in(k, kv_expected * 4, &dk.p);
    st.in(v, kv_expected * 4, &dv.p);
    st.out(out, q_expected * 4, &dout.p);
    rc = st.commit(err);
    if (rc) return rc;
    rc = gqa_device(nullptr, (const float*)dq.p, (const float*)dk.p, (const float*)dv.p, (float*)dout.p, batch, n_heads,
                    n_kv_heads, seq_q, seq_kv, head_dim, err);
    if (rc) return rc;
    return st.fetch(err);
}

RT_API int rt_gqa_forward_f32_dev(void* stream, const float* q, const float* k, const float* v, float* out, size_t batch,
                                  size_t n_heads, size_t n_kv_heads, size_t seq_q, size_t seq_kv, size_t head_dim,
                                  rt_err_detail* err) {
    clear_err(err);
    if (n_kv_heads == 0 || n_heads % n_kv_heads != 0)
        return fail(err, RT_ERR_HEAD_COUNT_MISMATCH, -1, n_heads, n_kv_heads, "n_heads not divisible by n_kv_heads");
    if (seq_q == seq_kv && head_dim == 0) return fail(err, RT_ERR_WRONG_INPUT_LEN, RT_WHICH_FLASH, 0, 0, "flash_forward");
    const size_t q_expected = batch * n_heads * seq_q * head_dim, kv_expected = batch * n_kv_heads * seq_kv * head_dim;
    if (q_expected == 0) return RT_OK;
    if (!q || !out || (kv_expected && (!k || !v))) return fail(err, RT_ERR_NULL_POINTER, -1, 0, 0, "NULL buffer");
    if (!fits_int(batch) || !fits_int(n_heads) || !fits_int(seq_q) || !fits_int(seq_kv) || !fits_int(head_dim) ||
        batch > 65535 || n_heads > 65535)
        return fail(err, RT_ERR_UNSUPPORTED, -1, 0, 0, "shape too large for the launch grid");
    int rc = ensure_device(err);
    if (rc) return rc;
    return gqa_device((hipStream_t)stream, q, k, v, out, batch, n_heads, n_kv_heads, seq_q, seq_kv, head_dim, err);
}

// ---- backward (cpu_backward.rs:46-185) ----------------------------------------------------------------

namespace {

// saved_out / saved_lse non-NULL: the forward is not recomputed and `workspace` holds delta only
int flash_bwd_device(hipStream_t stream, const rt_attention_shape* s, const float* q, const float* k, const float* v,
                     const float* d_out, float* dq, float* dk, float* dv, float* workspace, rt_err_detail* err,
                     const float* saved_out = nullptr, const float* saved_lse = nullptr) {
    if (s->dim > 512) return fail(err, RT_ERR_UNSUPPORTED, -1, 512, s->dim, "f32 backward kernels cover dim <= 512");
    rt::FlashBwdF32Params p{};
    p.q = q;
    p.k = k;
    p.v = v;
    p.d_out = d_out;
    p.dq = dq;
    p.dk = dk;
    p.dv = dv;
    p.batch = (int)s->batch;
    p.heads = (int)s->heads;
    p.seq = (int)s->seq;
    p.dim = (int)s->dim;
    p.scale = 1.0f / sqrtf((float)s->dim);
    if (saved_out) {
        HIP_TRY(rt::launch_flash_bwd_f32_saved(stream, p, saved_out, saved_lse, workspace), "flash_bwd_f32 launch");
    } else if (s->dim > 256) {
        // the recomputed forward of a head dim the tiled forward kernels do not cover: O and the row statistic from
        // the one-workgroup-per-row kernel, then the backward from them
        const size_t rows = (size_t)(s->batch * s->heads * s->seq);
        float* o = workspace;
        float* lse_ws = workspace + rows * s->dim;
        int rc = flash_f32_device(stream, s, s->heads, q, k, v, RT_MASK_NONE, nullptr, o, err, false, nullptr, 0, lse_ws);
        if (rc) return rc;
        HIP_TRY(rt::launch_flash_bwd_f32_saved(stream, p, o, lse_ws, lse_ws + rows), "flash_bwd_f32 launch");
    } else {
        HIP_TRY(rt::launch_flash_bwd_f32(stream, p, workspace, g_num_cus), "flash_bwd_f32 launch");
    }
    return RT_OK;
}

}  // namespace

RT_API size_t rt_flash_backward_workspace_bytes(const rt_attention_shape* shape) {
    if (!shape) return 0;
    if (!fits_int(shape->batch) || !fits_int(shape->heads) || !fits_int(shape->seq) || !fits_int(shape->dim)) return 0;
    return rt::flash_bwd_f32_workspace_floats((int)shape->batch, (int)shape->heads, (int)shape->seq, (int)shape->dim) *
           sizeof(float);
}

RT_API int rt_flash_backward_f32(const rt_attention_shape* shape, const float* q, size_t q_len, const float* k,
                                 size_t k_len, const float* v, size_t v_len, const float* d_out, size_t d_out_len,
                                 float* dq, size_t dq_len, float* dk, size_t dk_len, float* dv, size_t dv_len,
                                 rt_err_detail* err) {
    clear_err(err);
    if (!shape) return fail(err, RT_ERR_NULL_POINTER, -1, 0, 0, "shape is NULL");
    // cpu_backward.rs:59-74: no ZeroDim check here, unlike the forward
    const uint64_t expected = shape->batch * shape->heads * shape->seq * shape->dim;
    const size_t lens[4] = {q_len, k_len, v_len, d_out_len};
    static const char* names[4] = {"q", "k", "v", "do"};
    static const int which[4] = {RT_WHICH_Q, RT_WHICH_K, RT_WHICH_V, RT_WHICH_DO};
    for (int i = 0; i < 4; i++)
        if (lens[i] != expected) {
            char msg[96];
            snprintf(msg, sizeof(msg), "%s buffer has %zu elements, expected %llu", names[i], lens[i],
                     (unsigned long long)expected);
            return fail(err, RT_ERR_BUFFER_SHAPE_MISMATCH, which[i], expected, lens[i], msg);
        }
    if (dq_len != expected || dk_len != expected || dv_len != expected) {
        size_t got = dq_len > dk_len ? dq_len : dk_len;
        if (dv_len > got) got = dv_len;
        return fail(err, RT_ERR_OUTPUT_SHAPE_MISMATCH, RT_WHICH_OUT, expected, got, "gradient buffer length");
    }
    if (shape->seq == 0 || expected == 0) return RT_OK;
    if (!q || !k || !v || !d_out || !dq || !dk || !dv) return fail(err, RT_ERR_NULL_POINTER, -1, 0, 0, "NULL buffer");
    int rc = check_flash_dims(shape, shape->heads, err);
    if (rc) return rc;
    rc = ensure_device(err);
    if (rc) return rc;

    const size_t bytes = (size_t)expected * sizeof(float);
    Stage st;
    DevPtr in[4], out[3], ws;
    const float* host_in[4] = {q, k, v, d_out};
    float* host_out[3] = {dq, dk, dv};
    for (int i = 0; i < 4; i++) st.in(host_in[i], bytes, &in[i].p);
    for (int i = 0; i < 3; i++) st.out(host_out[i], bytes, &out[i].p);
    st.scratch(rt_flash_backward_workspace_bytes(shape), &ws.p);
    rc = st.commit(err);
    if (rc) return rc;
    rc = flash_bwd_device(nullptr, shape, (const float*)in[0].p, (const float*)in[1].p, (const float*)in[2].p,
                          (const float*)in[3].p, (float*)out[0].p, (float*)out[1].p, (float*)out[2].p, (float*)ws.p, err);
    if (rc) return rc;
    return st.fetch(err);
}

RT_API int rt_flash_backward_f32_dev(void* stream, const rt_attention_shape* shape, const float* q, const float* k,
                                     const float* v, const float* d_out, float* dq, float* dk, float* dv,
                                     void* workspace, size_t workspace_bytes, rt_err_detail* err) {
    clear_err(err);
    if (!shape) return fail(err, RT_ERR_NULL_POINTER, -1, 0, 0, "shape is NULL");
    if (shape->seq == 0 || shape->batch == 0 || shape->heads == 0 || shape->dim == 0) return RT_OK;
    int rc = check_flash_dims(shape, shape->heads, err);
    if (rc) return rc;
    if (!q || !k || !v || !d_out || !dq || !dk || !dv || !workspace)
        return fail(err, RT_ERR_NULL_POINTER, -1, 0, 0, "NULL buffer");
    const size_t need = rt_flash_backward_workspace_bytes(shape);
    if (workspace_bytes < need || ((uintptr_t)workspace & 15))
        return fail(err, RT_ERR_WORKSPACE_TOO_SMALL, -1, need, workspace_bytes, "backward workspace");
    rc = ensure_device(err);
    if (rc) return rc;
    return flash_bwd_device((hipStream_t)stream, shape, q, k, v, d_out, dq, dk, dv, (float*)workspace, err);
}

RT_API int rt_flash_forward_stats_f32_dev(void* stream, const rt_attention_shape* shape, const float* q, const float* k,
                                          const float* v, float* out, float* lse, rt_err_detail* err) {
    clear_err(err);
    if (!shape) return fail(err, RT_ERR_NULL_POINTER, -1, 0, 0, "shape is NULL");
    if (shape->dim == 0) return fail(err, RT_ERR_ZERO_DIM, -1, 0, 0, "dim must be > 0");
    if (shape->seq == 0 || shape->batch == 0 || shape->heads == 0) return RT_OK;
    int rc = check_flash_dims(shape, shape->heads, err);
    if (rc) return rc;
    if (!q || !k || !v || !out || !lse) return fail(err, RT_ERR_NULL_POINTER, -1, 0, 0, "NULL buffer");
    rc = ensure_device(err);
    if (rc) return rc;
    return flash_f32_device((hipStream_t)stream, shape, shape->heads, q, k, v, RT_MASK_NONE, nullptr, out, err, false,
                            nullptr, 0, lse);
}

RT_API int rt_flash_backward_saved_f32_dev(void* stream, const rt_attention_shape* shape, const float* q, const float* k,
                                           const float* v, const float* out, const float* lse, const float* d_out,
                                           float* dq, float* dk, float* dv, void* workspace, size_t workspace_bytes,
                                           rt_err_detail* err) {
    clear_err(err);
    if (!shape) return fail(err, RT_ERR_NULL_POINTER, -1, 0, 0, "shape is NULL");
    if (shape->seq == 0 || shape->batch == 0 || shape->heads == 0 || shape->dim == 0) return RT_OK;
    int rc = check_flash_dims(shape, shape->heads, err);
    if (rc) return rc;
    if (!q || !k || !v || !out || !lse || !d_out || !dq || !dk || !dv || !workspace)
        return fail(err, RT_ERR_NULL_POINTER, -1, 0, 0, "NULL buffer");
    const size_t need = (size_t)(shape->batch * shape->heads * shape->seq) * sizeof(float);
    if (workspace_bytes < need)
        return fail(err, RT_ERR_WORKSPACE_TOO_SMALL, -1, need, workspace_bytes, "backward workspace (delta)");
    rc = ensure_device(err);
    if (rc) return rc;
    return flash_bwd_device((hipStream_t)stream, shape, q, k, v, d_out, dq, dk, dv, (float*)workspace, err, out, lse);
}

// ---- prefill, device pointers -----------------------------------------------------------------------

RT_API int rt_flash_forward_f32_dev(void* stream, const rt_attention_shape* shape, uint64_t n_kv_heads,
                                    const float* q, const float* k, const float* v, int mask_kind,
                                    const uint8_t* keep, float* out, rt_err_detail* err) {
    clear_err(err);
    if (!shape) return fail(err, RT_ERR_NULL_POINTER, -1, 0, 0, "shape is NULL");
    if (shape->dim == 0) return fail(err, RT_ERR_ZERO_DIM, -1, 0, 0, "dim must be > 0");
    if (mask_kind < RT_MASK_NONE || mask_kind > RT_MASK_PADDING)
        return fail(err, RT_ERR_UNSUPPORTED, -1, 0, (uint64_t)mask_kind, "unknown mask kind");
    if (n_kv_heads == 0) n_kv_heads = shape->heads;
    if (shape->seq == 0 || shape->batch == 0 || shape->heads == 0) return RT_OK;
    int rc = check_flash_dims(shape, n_kv_heads, err);
    if (rc) return rc;
    if (!q || !k || !v || !out || (mask_kind == RT_MASK_PADDING && !keep))
        return fail(err, RT_ERR_NULL_POINTER, -1, 0, 0, "NULL buffer");
    rc = ensure_device(err);
    if (rc) return rc;
    return flash_f32_device((hipStream_t)stream, shape, n_kv_heads, q, k, v, mask_kind, keep, out, err);
}

// Which bf16 prefill kernel serves a call.  RT_ATTN_BF16_PREFILL=tile|persistent|wide in the environment forces one
// where it applies (for measurements and tests); otherwise the persistent 8-wave kernel takes head dim 128 (and head
// dim 64 under a key-padding mask) on unpadded batches with at least 512 rows per sequence and a job for every CU,
// and the 4-wave tile kernel everything else.
enum class PrefillKernel { kAuto, kTile, kPersistent, kWide };
// A debug switch for measurements and tests, not part of the reference's surface: rt_debug_force_bf16_prefill_kernel
// sets it; until that is called, the value is what RT_ATTN_BF16_PREFILL=tile|persistent held when the library made its
// first bf16 prefill call (read once: a later change of the environment does not change which kernel a caller gets).
static PrefillKernel parse_prefill_kernel(const char* e) {
    if (!e) return PrefillKernel::kAuto;
    if (strcmp(e, "tile") == 0) return PrefillKernel::kTile;
    if (strcmp(e, "persistent") == 0) return PrefillKernel::kPersistent;
    if (strcmp(e, "wide") == 0) return PrefillKernel::kWide;
    return PrefillKernel::kAuto;
}
static std::atomic<int> g_prefill_forced{-1};  // -1: not set through the API
static PrefillKernel prefill_kernel_override() {
    const int f = g_prefill_forced.load(std::memory_order_relaxed);
    if (f >= 0) return (PrefillKernel)f;
    static const PrefillKernel once = parse_prefill_kernel(getenv("RT_ATTN_BF16_PREFILL"));
    return once;
}
RT_API int rt_debug_force_bf16_prefill_kernel(int which) {
    if (which < 0 || which > 3) return RT_ERR_UNSUPPORTED;
    g_prefill_forced.store(which, std::memory_order_relaxed);
    return RT_OK;
}

RT_API int rt_set_strict_non_finite_v(int on) { return g_strict_v.exchange(on ? 1 : 0); }

static int flash_bf16_common(void* stream, const rt_attention_shape* shape, uint64_t n_kv_heads, const void* q,
                             const void* k, const void* v, int mask, const uint8_t* keep, const int32_t* seq_lens,
                             int zero_padded_rows, void* out, rt_err_detail* err, bool bnhd = false) {
    clear_err(err);
    if (!shape) return fail(err, RT_ERR_NULL_POINTER, -1, 0, 0, "shape is NULL");
    if (shape->dim == 0) return fail(err, RT_ERR_ZERO_DIM, -1, 0, 0, "dim must be > 0");
    if (n_kv_heads == 0) n_kv_heads = shape->heads;
    if (shape->seq == 0 || shape->batch == 0 || shape->heads == 0) return RT_OK;
    int rc = check_flash_dims(shape, n_kv_heads, err);
    if (rc) return rc;
    if (shape->dim > 512)
        return fail(err, RT_ERR_UNSUPPORTED, -1, 512, shape->dim, "bf16 flash kernels cover head dims up to 512");
    // the tile kernel's grid is (heads, batch, query tiles of 128 rows), each dimension below 2^16
    if (shape->heads > 65535 || shape->batch > 65535 || (shape->seq + 127) / 128 > 65535)
        return fail(err, RT_ERR_UNSUPPORTED, -1, 0, 0, "shape too large for the launch grid");
    if (!q || !k || !v || !out || (mask == rt::kMaskPadding && !keep) || (mask == rt::kMaskVarlenCausal && !seq_lens))
        return fail(err, RT_ERR_NULL_POINTER, -1, 0, 0, "NULL buffer");
    rc = ensure_device(err);
    if (rc) return rc;
    // The matrix-core kernels move 16 bytes at a time: head dims up to 256 that are a multiple of 8, tensors 16-byte
    // aligned.  Everything else (the reference takes any dim != 0, cpu_forward.rs:142-169) goes to the
    // one-workgroup-per-row kernel: same masks, same row rules, any speed.
    // (so does a K/V slab of 4 GiB or more per (batch, kv head): the tile kernel addresses it with 32-bit offsets)
    const bool tile_addressable = rt::flash_tile_bf16_addressable((long long)shape->seq, (long long)((bnhd ? n_kv_heads : 1) * shape->dim));
    if (shape->dim > 256 || shape->dim % 8 != 0 || (((uintptr_t)q | (uintptr_t)k | (uintptr_t)v | (uintptr_t)out) & 15) != 0 ||
        !tile_addressable) {
        rt::AttnRowsParams r{};
        r.q = q;
        r.k = k;
        r.v = v;
        r.out = out;
        r.kv_lens = mask == rt::kMaskVarlenCausal ? seq_lens : nullptr;
        r.q_lens = r.kv_lens;
        r.batch = (int)shape->batch;
        r.heads = (int)shape->heads;
        r.kv_heads = (int)n_kv_heads;
        r.seq_q = r.kv_len = r.kv_stride = (int)shape->seq;
        r.dim = (int)shape->dim;
        r.head_map = 0;
        r.scale = 1.0f / sqrtf((float)shape->dim);
        r.use_layout = 1;
        if (bnhd) {
            r.lq = r.lo = rt::layout_bnhd((long long)shape->heads, (long long)shape->seq, r.dim);
            r.lkv = rt::layout_bnhd((long long)n_kv_heads, (long long)shape->seq, r.dim);
        } else {
            r.lq = r.lo = rt::layout_bhnd((long long)shape->heads, (long long)shape->seq, r.dim);
            r.lkv = rt::layout_bhnd((long long)n_kv_heads, (long long)shape->seq, r.dim);
        }
        r.mask = mask == rt::kMaskVarlenCausal ? rt::kMaskCausal : mask;
        r.keep = keep;
        r.ref_bc = (int)(shape->bc == 0 ? 1 : (shape->bc > 0x7fffffffull ? 0x7fffffff : shape->bc));
        r.flash_rows = 1;
        r.zero_padded_rows = zero_padded_rows;
        HIP_TRY(rt::launch_attn_rows_bf16((hipStream_t)stream, r), "attn_rows_bf16 launch");
        return strict_pass((hipStream_t)stream, shape, n_kv_heads, v, out, seq_lens, mask, bnhd, true, err);
    }
    // the persistent kernel needs a job (256 query rows of one head) for every CU and gains on the tile kernel as the
    // rows get longer; a padded batch is a set of jobs of very different lengths, which the tile kernel's
    // dispatcher-balanced workgroups handle better
    const bool persistent_dim = shape->dim == 64 || shape->dim == 128;
    const uint64_t jobs256 = (shape->seq + 255) / 256 * shape->batch * shape->heads;
    bool persistent = persistent_dim && shape->seq >= 512 && jobs256 >= (uint64_t)g_num_cus && mask != rt::kMaskVarlenCausal;
    const PrefillKernel forced = prefill_kernel_override();
    if (forced == PrefillKernel::kTile || forced == PrefillKernel::kWide) persistent = false;
    // head dim 64 exactly, no mask or the causal one: the tile kernel (whose K/V tiles go straight from memory to LDS
    // at this head dim) measured ahead of the persistent kernel on every shape tried (N = 1024 .. 32768, 4-9 %) and
    // level with the kernel of 64 query rows per wave, which therefore runs only when it is asked for
    if (forced == PrefillKernel::kAuto && shape->dim == 64 && (mask == rt::kMaskNone || mask == rt::kMaskCausal)) persistent = false;
    if (forced == PrefillKernel::kPersistent && persistent_dim) persistent = true;
    if (mask == rt::kMaskPadding && shape->seq > (uint64_t)rt::kFlashBf16MaxPaddingKeys) persistent = false;
    if (persistent) {  // that kernel addresses the rows of one (batch, head) slab with 32-bit byte offsets
        const uint64_t pitch_b = (bnhd ? shape->heads : 1) * shape->dim * 2;
        if (shape->seq * pitch_b >= (1ull << 32)) persistent = false;
    }
    const int dim = (int)shape->dim;
    rt::TensorLayout lq, lkv;
    if (bnhd) {
        lq = rt::layout_bnhd((long long)shape->heads, (long long)shape->seq, dim);
        lkv = rt::layout_bnhd((long long)n_kv_heads, (long long)shape->seq, dim);
    } else {
        lq = rt::layout_bhnd((long long)shape->heads, (long long)shape->seq, dim);
        lkv = rt::layout_bhnd((long long)n_kv_heads, (long long)shape->seq, dim);
    }
    const int ref_bc = (int)(shape->bc == 0 ? 1 : (shape->bc > 0x7fffffffull ? 0x7fffffff : shape->bc));
    const float scale = 1.0f / sqrtf((float)shape->dim);
    if (!persistent) {
        rt::FlashTileParams t{};
        t.q = (const uint16_t*)q;
        t.k = (const uint16_t*)k;
        t.v = (const uint16_t*)v;
        t.out = (uint16_t*)out;
        t.keep = keep;
        // a padded batch: sequence b has seq_lens[b] query positions and as many keys, masked causally
        t.q_lens = mask == rt::kMaskVarlenCausal ? seq_lens : nullptr;
        t.kv_lens = t.q_lens;
        t.batch = (int)shape->batch;
        t.heads = (int)shape->heads;
        t.kv_heads = (int)n_kv_heads;
        t.group = (int)(shape->heads / n_kv_heads);
        t.pack = 1;
        t.seq_q = t.seq_kv = (int)shape->seq;
        t.dim = dim;
        t.mask = mask == rt::kMaskVarlenCausal ? rt::kMaskCausal : mask;
        t.ref_bc = ref_bc;
        t.zero_padded_rows = zero_padded_rows;
        t.scale = scale;
        t.scale_log2e = scale * rt::kLog2eHost;
        t.lq = t.lo = lq;
        t.lkv = lkv;
        if (forced == PrefillKernel::kWide && rt::flash_wide_bf16_supported(t)) {
            HIP_TRY(rt::launch_flash_wide_bf16((hipStream_t)stream, t), "flash_wide_bf16 launch");
            return strict_pass((hipStream_t)stream, shape, n_kv_heads, v, out, seq_lens, mask, bnhd, true, err);
        }
        HIP_TRY(rt::launch_flash_tile_bf16((hipStream_t)stream, t), "flash_tile_bf16 launch");
        return strict_pass((hipStream_t)stream, shape, n_kv_heads, v, out, seq_lens, mask, bnhd, true, err);
    }
    rt::FlashBf16Params p;
    p.q = (const uint16_t*)q;
    p.k = (const uint16_t*)k;
    p.v = (const uint16_t*)v;
    p.out = (uint16_t*)out;
    p.keep = keep;
    p.seq_lens = seq_lens;
    p.batch = (int)shape->batch;
    p.heads = (int)shape->heads;
    p.kv_heads = (int)n_kv_heads;
    p.group = (int)(shape->heads / n_kv_heads);
    p.seq = (int)shape->seq;
    p.dim = dim;
    p.mask = mask;
    p.ref_bc = ref_bc;
    p.zero_padded_rows = zero_padded_rows;
    p.scale_log2e = scale * rt::kLog2eHost;
    p.n_workers = g_num_cus;
    p.lq = p.lo = lq;
    p.lkv = lkv;
    HIP_TRY(rt::launch_flash_bf16((hipStream_t)stream, p), "flash_fwd_bf16 launch");
    return strict_pass((hipStream_t)stream, shape, n_kv_heads, v, out, seq_lens, mask, bnhd, true, err);
}

RT_API int rt_flash_forward_bf16_dev(void* stream, const rt_attention_shape* shape, uint64_t n_kv_heads,
                                     const void* q, const void* k, const void* v, int mask_kind, const uint8_t* keep,
                                     void* out, rt_err_detail* err) {
    if (mask_kind < RT_MASK_NONE || mask_kind > RT_MASK_PADDING) {
        clear_err(err);
        return fail(err, RT_ERR_UNSUPPORTED, -1, 0, (uint64_t)mask_kind, "unknown mask kind");
    }
    return flash_bf16_common(stream, shape, n_kv_heads, q, k, v, mask_kind, keep, nullptr, 0, out, err);
}

RT_API int rt_flash_forward_bnhd_bf16_dev(void* stream, const rt_attention_shape* shape, uint64_t n_kv_heads,
                                          const void* q, const void* k, const void* v, int mask_kind,
                                          const uint8_t* keep, void* out, rt_err_detail* err) {
    if (mask_kind < RT_MASK_NONE || mask_kind > RT_MASK_PADDING) {
        clear_err(err);
        return fail(err, RT_ERR_UNSUPPORTED, -1, 0, (uint64_t)mask_kind, "unknown mask kind");
    }
    return flash_bf16_common(stream, shape, n_kv_heads, q, k, v, mask_kind, keep, nullptr, 0, out, err, true);
}

RT_API int rt_flash_forward_bnhd_f32_dev(void* stream, const rt_attention_shape* shape, uint64_t n_kv_heads,
                                         const float* q, const float* k, const float* v, int mask_kind,
                                         const uint8_t* keep, float* out, rt_err_detail* err) {
    clear_err(err);
    if (!shape) return fail(err, RT_ERR_NULL_POINTER, -1, 0, 0, "shape is NULL");
    if (shape->dim == 0) return fail(err, RT_ERR_ZERO_DIM, -1, 0, 0, "dim must be > 0");
    if (mask_kind < RT_MASK_NONE || mask_kind > RT_MASK_PADDING)
        return fail(err, RT_ERR_UNSUPPORTED, -1, 0, (uint64_t)mask_kind, "unknown mask kind");
    if (n_kv_heads == 0) n_kv_heads = shape->heads;
    if (shape->seq == 0 || shape->batch == 0 || shape->heads == 0) return RT_OK;
    int rc = check_flash_dims(shape, n_kv_heads, err);
    if (rc) return rc;
    if (!q || !k || !v || !out || (mask_kind == RT_MASK_PADDING && !keep))
        return fail(err, RT_ERR_NULL_POINTER, -1, 0, 0, "NULL buffer");
    rc = ensure_device(err);
    if (rc) return rc;
    return flash_f32_device((hipStream_t)stream, shape, n_kv_heads, q, k, v, mask_kind, keep, out, err, true);
}

RT_API int rt_mha_flash_forward_f32(const float* q, size_t q_len, const float* k, size_t k_len, const float* v,
                                    size_t v_len, float* out, size_t out_len, size_t batch, size_t seq, size_t heads,
                                    size_t head_dim, rt_err_detail* err) {
    clear_err(err);
    // the reference transposes to [B,H,T,hd] and calls flash_forward (attention.rs:474-483): same checks, same order
    rt_attention_shape shape = {batch, heads, seq, head_dim, 64, 64};
    int rc = validate_flash(&shape, q_len, k_len, v_len, out_len, RT_MASK_NONE, 0, err);
    if (rc) return rc;
    if (seq == 0 || q_len == 0) return RT_OK;
    if (!q || !k || !v || !out) return fail(err, RT_ERR_NULL_POINTER, -1, 0, 0, "NULL buffer");
    rc = check_flash_dims(&shape, heads, err);
    if (rc) return rc;
    rc = ensure_device(err);
    if (rc) return rc;
    Stage st;
    DevPtr dq, dk, dv, dout;
    size_t bytes = q_len * sizeof(float);
    st.in(q, bytes, &dq.p);
    st.in(k, bytes, &dk.p);
    st.in(v, bytes, &dv.p);
    st.out(out, bytes, &dout.p);
    rc = st.commit(err);
    if (rc) return rc;
    rc = flash_f32_device(nullptr, &shape, heads, (const float*)dq.p, (const float*)dk.p, (const float*)dv.p,
                          RT_MASK_NONE, nullptr, (float*)dout.p, err, true);
    if (rc) return rc;
    return st.fetch(err);
}

namespace {

// The attention of rt_mha_forward_masked_f32 on device-resident tensors (arguments already checked).
int mha_masked_device(hipStream_t stream, const float* q, const float* k, const float* v, const float* mask,
                      size_t mask_len, float* out, size_t batch, size_t t_q, size_t t_kv, size_t heads,
                      size_t head_dim, rt_err_detail* err) {
    const size_t one_mask = t_q * t_kv, all_masks = batch * heads * one_mask;
    int rc = RT_OK;
    const long long bias_bh_stride = (mask_len == all_masks && all_masks != one_mask) ? (long long)one_mask : 0;
    auto aligned16 = [](const void* ptr) { return ((uintptr_t)ptr & 15) == 0; };
    if (t_kv > 0 && head_dim % 4 == 0 && head_dim <= 128 && fits_int(t_kv) && aligned16(q) && aligned16(k) &&
        aligned16(v) && aligned16(out)) {
        // a head dim the tiled f32 kernel covers (and 16-byte aligned tensors): the same kernel as the unmasked path,
        // with the mask's row added to the scaled scores and, for cross-attention, its own number of keys
        rt_attention_shape shape = {batch, heads, t_q, head_dim, 64, 64};
        rc = flash_f32_device(stream, &shape, heads, q, k, v, RT_MASK_NONE, nullptr, out, err, true,
                              mask_len ? mask : nullptr, bias_bh_stride, nullptr, t_kv);
        return rc;
    }
    rt::AttnRowsParams p{};
    p.q = q;
    p.k = k;
    p.v = v;
    p.out = out;
    p.kv_lens = nullptr;
    p.batch = (int)batch;
    p.heads = (int)heads;
    p.kv_heads = (int)heads;
    p.seq_q = (int)t_q;
    p.kv_len = (int)t_kv;
    p.kv_stride = (int)t_kv;
    p.dim = (int)head_dim;
    p.head_map = 0;
    p.scale = 1.0f / sqrtf((float)head_dim);
    p.bias = mask_len ? mask : nullptr;
    p.bias_bh_stride = bias_bh_stride;
    p.use_layout = 1;
    p.lq = p.lo = rt::layout_bnhd((long long)heads, (long long)t_q, (int)head_dim);
    p.lkv = rt::layout_bnhd((long long)heads, (long long)t_kv, (int)head_dim);
    HIP_TRY(rt::launch_attn_rows_f32(stream, p), "attn_rows_f32 launch");
    return RT_OK;
}

}  // namespace

RT_API int rt_mha_forward_masked_f32(const float* q, size_t q_len, const float* k, size_t k_len, const float* v,
                                     size_t v_len, const float* mask, size_t mask_len, float* out, size_t out_len,
                                     size_t batch, size_t t_q, size_t t_kv, size_t heads, size_t head_dim,
                                     rt_err_detail* err) {
    clear_err(err);
    if (head_dim == 0) return fail(err, RT_ERR_ZERO_DIM, -1, 0, 0, "dim must be > 0");
    const size_t embed = heads * head_dim;
    const size_t q_expected = batch * t_q * embed, kv_expected = batch * t_kv * embed;
    if (q_len != q_expected) return fail(err, RT_ERR_BUFFER_SHAPE_MISMATCH, RT_WHICH_Q, q_expected, q_len, "q length");
    if (k_len != kv_expected) return fail(err, RT_ERR_BUFFER_SHAPE_MISMATCH, RT_WHICH_K, kv_expected, k_len, "k length");
    if (v_len != kv_expected) return fail(err, RT_ERR_BUFFER_SHAPE_MISMATCH, RT_WHICH_V, kv_expected, v_len, "v length");
    if (out_len != q_expected) return fail(err, RT_ERR_OUTPUT_SHAPE_MISMATCH, -1, q_expected, out_len, "out length");
    const size_t one_mask = t_q * t_kv, all_masks = batch * heads * one_mask;
    if (!mask) mask_len = 0;
    if (mask_len != 0 && mask_len != one_mask && mask_len != all_masks)
        return fail(err, RT_ERR_WRONG_INPUT_LEN, RT_WHICH_MASK, one_mask, mask_len, "mask length");
    if (q_expected == 0) return RT_OK;
    if (!q || !out || (kv_expected && (!k || !v))) return fail(err, RT_ERR_NULL_POINTER, -1, 0, 0, "NULL buffer");
    if (head_dim > 512) return fail(err, RT_ERR_UNSUPPORTED, -1, 512, head_dim, "rows kernel covers dim <= 512");
    if (heads > 65535 || batch > 65535 || t_q > 0x7fffffffull || t_kv > 0x7fffffffull || embed > 0x7fffffffull)
        return fail(err, RT_ERR_UNSUPPORTED, -1, 0, 0, "shape too large for the launch grid");
    int rc = ensure_device(err);
    if (rc) return rc;
    Stage st;
    DevPtr dq, dk, dv, dm, dout;
    st.in(q, q_expected * 4, &dq.p);
    st.in(k, kv_expected * 4, &dk.p);
    st.in(v, kv_expected * 4, &dv.p);
    st.in(mask, mask_len * 4, &dm.p);
    st.out(out, q_expected * 4, &dout.p);
    rc = st.commit(err);
    if (rc) return rc;
    rc = mha_masked_device(nullptr, (const float*)dq.p, (const float*)dk.p, (const float*)dv.p,
                           mask_len ? (const float*)dm.p : nullptr, mask_len, (float*)dout.p, batch, t_q, t_kv, heads,
                           head_dim, err);
    if (rc) return rc;
    return st.fetch(err);
}

RT_API int rt_mha_forward_masked_f32_dev(void* stream, const float* q, const float* k, const float* v, const float* mask,
                                         size_t mask_len, float* out, size_t batch, size_t t_q, size_t t_kv,
                                         size_t heads, size_t head_dim, rt_err_detail* err) {
    clear_err(err);
    if (head_dim == 0) return fail(err, RT_ERR_ZERO_DIM, -1, 0, 0, "dim must be > 0");
    const size_t embed = heads * head_dim;
    const size_t q_expected = batch * t_q * embed, kv_expected = batch * t_kv * embed;
    const size_t one_mask = t_q * t_kv, all_masks = batch * heads * one_mask;
    if (!mask) mask_len = 0;
    if (mask_len != 0 && mask_len != one_mask && mask_len != all_masks)
        return fail(err, RT_ERR_WRONG_INPUT_LEN, RT_WHICH_MASK, one_mask, mask_len, "mask length");
    if (q_expected == 0) return RT_OK;
    if (!q || !out || (kv_expected && (!k || !v))) return fail(err, RT_ERR_NULL_POINTER, -1, 0, 0, "NULL buffer");
    if (head_dim > 512) return fail(err, RT_ERR_UNSUPPORTED, -1, 512, head_dim, "rows kernel covers dim <= 512");
    if (heads > 65535 || batch > 65535 || t_q > 0x7fffffffull || t_kv > 0x7fffffffull || embed > 0x7fffffffull)
        return fail(err, RT_ERR_UNSUPPORTED, -1, 0, 0, "shape too large for the launch grid");
    int rc = ensure_device(err);
    if (rc) return rc;
    return mha_masked_device((hipStream_t)stream, q, k, v, mask_len ? mask : nullptr, mask_len, out, batch, t_q, t_kv,
                             heads, head_dim, err);
}

// bf16 counterpart of rt_mha_forward_masked_f32_dev: steps 2-8 of MultiHeadAttention::forward's composed path
// (crates/rustorch-nn/src/attention.rs:371-399) on bf16 [B,T,H*hd] tensors with an f32 additive mask.
RT_API int rt_mha_forward_masked_bf16_dev(void* stream, const void* q, const void* k, const void* v, const float* mask,
                                          size_t mask_len, void* out, size_t batch, size_t t_q, size_t t_kv,
                                          size_t heads, size_t head_dim, rt_err_detail* err) {
    clear_err(err);
    if (head_dim == 0) return fail(err, RT_ERR_ZERO_DIM, -1, 0, 0, "dim must be > 0");
    const size_t embed = heads * head_dim;
    const size_t q_expected = batch * t_q * embed, kv_expected = batch * t_kv * embed;
    const size_t one_mask = t_q * t_kv, all_masks = batch * heads * one_mask;
    if (!mask) mask_len = 0;
    if (mask_len != 0 && mask_len != one_mask && mask_len != all_masks)
        return fail(err, RT_ERR_WRONG_INPUT_LEN, RT_WHICH_MASK, one_mask, mask_len, "mask length");
    if (q_expected == 0) return RT_OK;
    if (!q || !out || (kv_expected && (!k || !v))) return fail(err, RT_ERR_NULL_POINTER, -1, 0, 0, "NULL buffer");
    if (head_dim > 512) return fail(err, RT_ERR_UNSUPPORTED, -1, 512, head_dim, "bf16 kernels cover head dims up to 512");
    if (heads > 65535 || batch > 65535 || t_q > 0x7fffffffull || t_kv > 0x7fffffffull || embed > 0x7fffffffull ||
        (t_q + 127) / 128 > 65535)
        return fail(err, RT_ERR_UNSUPPORTED, -1, 0, 0, "shape too large for the launch grid");
    if (((uintptr_t)mask & 3) != 0) return fail(err, RT_ERR_UNSUPPORTED, -1, 4, 0, "the mask must be 4-byte aligned");
    int rc = ensure_device(err);
    if (rc) return rc;
    if (!rt::flash_tile_bf16_supported((int)head_dim) || (((uintptr_t)q | (uintptr_t)k | (uintptr_t)v | (uintptr_t)out) & 15) != 0 ||
        !rt::flash_tile_bf16_addressable((long long)t_kv, (long long)(heads * head_dim))) {
        // head dims and alignments the matrix-core kernel does not cover: one workgroup per query row, any speed
        if (t_kv == 0) return rt_buf_zero(out, q_expected * 2, stream, err);
        rt::AttnRowsParams r{};
        r.q = q;
        r.k = k;
        r.v = v;
        r.out = out;
        r.batch = (int)batch;
        r.heads = r.kv_heads = (int)heads;
        r.seq_q = (int)t_q;
        r.kv_len = r.kv_stride = (int)t_kv;
        r.dim = (int)head_dim;
        r.head_map = 0;
        r.scale = 1.0f / sqrtf((float)head_dim);
        r.bias = mask_len ? mask : nullptr;
        r.bias_bh_stride = (mask_len == all_masks && all_masks != one_mask) ? (long long)one_mask : 0;
        r.use_layout = 1;
        r.lq = r.lo = rt::layout_bnhd((long long)heads, (long long)t_q, (int)head_dim);
        r.lkv = rt::layout_bnhd((long long)heads, (long long)t_kv, (int)head_dim);
        HIP_TRY(rt::launch_attn_rows_bf16((hipStream_t)stream, r), "attn_rows_bf16 launch");
        return RT_OK;
    }
    rt::FlashTileParams t{};
    t.q = (const uint16_t*)q;
    t.k = (const uint16_t*)k;
    t.v = (const uint16_t*)v;
    t.out = (uint16_t*)out;
    t.bias = mask_len ? mask : nullptr;
    t.bias_bh_stride = (mask_len == all_masks && all_masks != one_mask) ? (long long)one_mask : 0;
    t.bias_vec4 = (((uintptr_t)mask & 15) == 0 && t_kv % 4 == 0) ? 1 : 0;
    t.batch = (int)batch;
    t.heads = t.kv_heads = (int)heads;
    t.group = 1;
    t.pack = 1;
    t.seq_q = (int)t_q;
    t.seq_kv = (int)t_kv;
    t.dim = (int)head_dim;
    t.mask = rt::kMaskNone;
    t.ref_bc = 64;
    t.zero_padded_rows = 0;
    t.scale = 1.0f / sqrtf((float)head_dim);
    t.scale_log2e = t.scale * rt::kLog2eHost;
    t.lq = t.lo = rt::layout_bnhd((long long)heads, (long long)t_q, (int)head_dim);
    t.lkv = rt::layout_bnhd((long long)heads, (long long)t_kv, (int)head_dim);
    if (t_kv == 0)  // no key to weigh: the reference's products over an empty axis leave rows of zeros
        return rt_buf_zero(out, q_expected * 2, stream, err);
    HIP_TRY(rt::launch_flash_tile_bf16((hipStream_t)stream, t), "flash_tile_bf16 launch");
    return RT_OK;
}

// Causal attention with a sliding window on bf16 tensors, the mask itself never built: position i sees keys
// (i - window, i].  bnhd: [batch, seq, heads, dim] tensors (MultiHeadAttention's), else [batch, heads, seq, dim].
static int flash_window_bf16(void* stream, const rt_attention_shape* shape, uint64_t n_kv_heads, const void* q, const void* k,
                             const void* v, uint64_t window, void* out, rt_err_detail* err, bool bnhd) {
    clear_err(err);
    if (!shape) return fail(err, RT_ERR_NULL_POINTER, -1, 0, 0, "shape is NULL");
    if (shape->dim == 0) return fail(err, RT_ERR_ZERO_DIM, -1, 0, 0, "dim must be > 0");
    if (window == 0) return fail(err, RT_ERR_UNSUPPORTED, -1, 1, 0, "window must be >= 1 (masks.rs:51)");
    if (n_kv_heads == 0) n_kv_heads = shape->heads;
    if (shape->seq == 0 || shape->batch == 0 || shape->heads == 0) return RT_OK;
    int rc = check_flash_dims(shape, n_kv_heads, err);
    if (rc) return rc;
    if (shape->heads > 65535 || shape->batch > 65535 || (shape->seq + 127) / 128 > 65535)
        return fail(err, RT_ERR_UNSUPPORTED, -1, 0, 0, "shape too large for the launch grid");
    if (!q || !k || !v || !out) return fail(err, RT_ERR_NULL_POINTER, -1, 0, 0, "NULL buffer");
    if (!rt::flash_tile_bf16_supported((int)shape->dim))
        return fail(err, RT_ERR_UNSUPPORTED, -1, 256, shape->dim,
                    "the windowed kernel covers head dims up to 256 that are a multiple of 8 (others: the additive-mask entry)");
    if ((((uintptr_t)q | (uintptr_t)k | (uintptr_t)v | (uintptr_t)out) & 15) != 0)
        return fail(err, RT_ERR_UNSUPPORTED, -1, 16, 0, "bf16 kernels need 16-byte aligned tensors");
    if (!rt::flash_tile_bf16_addressable((long long)shape->seq, (long long)((bnhd ? n_kv_heads : 1) * shape->dim)))
        return fail(err, RT_ERR_UNSUPPORTED, -1, 0, shape->seq, "a K/V slab of one (batch, kv head) must stay below 4 GiB");
    rc = ensure_device(err);
    if (rc) return rc;
    const int dim = (int)shape->dim;
    rt::FlashTileParams t{};
    t.q = (const uint16_t*)q;
    t.k = (const uint16_t*)k;
    t.v = (const uint16_t*)v;
    t.out = (uint16_t*)out;
    t.batch = (int)shape->batch;
    t.heads = (int)shape->heads;
    t.kv_heads = (int)n_kv_heads;
    t.group = (int)(shape->heads / n_kv_heads);
    t.pack = 1;
    t.seq_q = t.seq_kv = (int)shape->seq;
    t.dim = dim;
    t.mask = rt::kMaskCausal;
    t.ref_bc = 64;
    t.scale = 1.0f / sqrtf((float)dim);
    t.scale_log2e = t.scale * rt::kLog2eHost;
    t.window = (int)(window > shape->seq ? shape->seq : window);  // a window of the whole sequence and more is the causal mask
    if (bnhd) {
        t.lq = t.lo = rt::layout_bnhd((long long)shape->heads, (long long)shape->seq, dim);
        t.lkv = rt::layout_bnhd((long long)n_kv_heads, (long long)shape->seq, dim);
    } else {
        t.lq = t.lo = rt::layout_bhnd((long long)shape->heads, (long long)shape->seq, dim);
        t.lkv = rt::layout_bhnd((long long)n_kv_heads, (long long)shape->seq, dim);
    }
    HIP_TRY(rt::launch_flash_tile_bf16((hipStream_t)stream, t), "flash_tile_bf16 (window) launch");
    return RT_OK;
}

RT_API int rt_flash_forward_window_bf16_dev(void* stream, const rt_attention_shape* shape, uint64_t n_kv_heads, const void* q,
                                            const void* k, const void* v, uint64_t window, void* out, rt_err_detail* err) {
    return flash_window_bf16(stream, shape, n_kv_heads, q, k, v, window, out, err, false);
}

RT_API int rt_flash_forward_window_bnhd_bf16_dev(void* stream, const rt_attention_shape* shape, uint64_t n_kv_heads,
                                                 const void* q, const void* k, const void* v, uint64_t window, void* out,
                                                 rt_err_detail* err) {
    return flash_window_bf16(stream, shape, n_kv_heads, q, k, v, window, out, err, true);
}

RT_API int rt_flash_forward_varlen_bf16_dev(void* stream, const rt_attention_shape* shape, uint64_t n_kv_heads,
                                            const void* q, const void* k, const void* v, const int32_t* seq_lens,
                                            int zero_padded_rows, void* out, rt_err_detail* err) {
    return flash_bf16_common(stream, shape, n_kv_heads, q, k, v, rt::kMaskVarlenCausal, nullptr, seq_lens,
                             zero_padded_rows, out, err);
}

// ---- decode, device pointers -------------------------------------------------------------------------

RT_API int rt_kv_append_bf16(void* stream, void* k_cache, void* v_cache, const void* k_in, const void* v_in,
                             int32_t pos, int32_t n_kv, int32_t head_dim, int32_t max_seq, rt_err_detail* err) {
    clear_err(err);
    if (n_kv < 0 || head_dim < 0 || max_seq < 0) return fail(err, RT_ERR_UNSUPPORTED, -1, 0, 0, "negative dimension");
    if (pos < 0 || pos >= max_seq)
        return fail(err, RT_ERR_KV_OVERFLOW, -1, (uint64_t)max_seq, (uint64_t)(int64_t)pos + 1, "position outside the cache");
    if (n_kv == 0 || head_dim == 0) return RT_OK;
    if (!k_cache || !v_cache || !k_in || !v_in) return fail(err, RT_ERR_NULL_POINTER, -1, 0, 0, "NULL buffer");
    int rc = ensure_device(err);
    if (rc) return rc;
    HIP_TRY(rt::launch_kv_append_bf16((hipStream_t)stream, (uint16_t*)k_cache, (uint16_t*)v_cache,
                                      (const uint16_t*)k_in, (const uint16_t*)v_in, pos, n_kv, head_dim, max_seq),
            "kv_append_bf16 launch");
    return RT_OK;
}

RT_API int rt_kv_cache_append_dev(void* stream, void* k_cache, void* v_cache, const void* new_k, size_t new_k_len,
                                  const void* new_v, size_t new_v_len, size_t batch, size_t n_heads, size_t max_seq,
                                  size_t head_dim, size_t current_len, size_t seq_added, size_t elem_bytes,
                                  rt_err_detail* err) {
    clear_err(err);
    if (current_len + seq_added > max_seq)  // kv_cache.rs:84-89
        return fail(err, RT_ERR_KV_OVERFLOW, -1, (uint64_t)max_seq, (uint64_t)(current_len + seq_added), "append beyond max_seq");
    const size_t bhsd = batch * n_heads * seq_added * head_dim;
    if (new_k_len != bhsd || new_v_len != bhsd) {  // kv_cache.rs:90-97
        int rc = fail(err, RT_ERR_KV_WRONG_INPUT_LEN, -1, (uint64_t)bhsd, (uint64_t)new_k_len, "new_k / new_v length");
        if (err) err->got2 = (uint64_t)new_v_len;
        return rc;
    }
    if (elem_bytes != 2 && elem_bytes != 4) return fail(err, RT_ERR_UNSUPPORTED, -1, 0, (uint64_t)elem_bytes, "elem_bytes must be 2 or 4");
    if (batch * n_heads > 65535) return fail(err, RT_ERR_UNSUPPORTED, -1, 0, 0, "shape too large for the launch grid");
    if (bhsd == 0) return RT_OK;
    if (!k_cache || !v_cache || !new_k || !new_v) return fail(err, RT_ERR_NULL_POINTER, -1, 0, 0, "NULL buffer");
    int rc = ensure_device(err);
    if (rc) return rc;
    HIP_TRY(rt::launch_kv_block_append((hipStream_t)stream, k_cache, v_cache, new_k, new_v, batch * n_heads, max_seq, head_dim,
                                       current_len, seq_added, elem_bytes),
            "kv_cache_append launch");
    return RT_OK;
}

RT_API int rt_qk_norm_rope_kv_append_bf16(void* stream, void* q, const void* k_in, const void* v_in, void* k_cache,
                                          void* v_cache, const int32_t* positions, int32_t pos, const float* q_gamma,
                                          const float* k_gamma, float eps, const float* cos_table,
                                          const float* sin_table, int32_t table_rows, int32_t batch, int32_t seq,
                                          int32_t n_heads, int32_t n_kv, int32_t head_dim, int32_t max_seq,
                                          rt_err_detail* err) {
    clear_err(err);
    if (batch < 0 || seq < 0 || n_heads < 0 || n_kv < 0 || head_dim < 0 || max_seq < 0 || table_rows < 0)
        return fail(err, RT_ERR_UNSUPPORTED, -1, 0, 0, "negative dimension");
    if ((head_dim & 1) || head_dim > 512)
        return fail(err, RT_ERR_UNSUPPORTED, -1, 512, (uint64_t)head_dim, "head_dim must be even and <= 512");
    if (batch > 65535 || seq > 65535 || n_heads + n_kv > 65535)
        return fail(err, RT_ERR_UNSUPPORTED, -1, 0, 0, "shape too large for the launch grid");
    if (!positions) {
        // the checks of RoPE::apply_inplace_half_split (rope.rs:179-184), then of KVLayerCache::append (kv_cache.rs:84-89)
        if (pos < 0 || (int64_t)pos + seq > table_rows)
            return fail(err, RT_ERR_ROPE_POSITION_OVERFLOW, -1, (uint64_t)table_rows, (uint64_t)((int64_t)pos + seq),
                        "positions outside the RoPE tables");
        if ((int64_t)pos + seq > max_seq)
            return fail(err, RT_ERR_KV_OVERFLOW, -1, (uint64_t)max_seq, (uint64_t)((int64_t)pos + seq), "rows outside the cache");
    }
    if (batch == 0 || seq == 0 || n_heads + n_kv == 0 || head_dim == 0) return RT_OK;
    if ((n_heads > 0 && !q) || (n_kv > 0 && (!k_in || !v_in || !k_cache || !v_cache)) || !cos_table || !sin_table)
        return fail(err, RT_ERR_NULL_POINTER, -1, 0, 0, "NULL buffer");
    int rc = ensure_device(err);
    if (rc) return rc;
    rt::DecodePrepareParams p;
    p.q = (uint16_t*)q;
    p.k_in = (const uint16_t*)k_in;
    p.v_in = (const uint16_t*)v_in;
    p.k_cache = (uint16_t*)k_cache;
    p.v_cache = (uint16_t*)v_cache;
    p.positions = positions;
    p.q_gamma = q_gamma;
    p.k_gamma = k_gamma;
    p.cos_table = cos_table;
    p.sin_table = sin_table;
    p.eps = eps;
    p.pos = pos;
    p.batch = batch;
    p.seq = seq;
    p.n_heads = n_heads;
    p.n_kv = n_kv;
    p.head_dim = head_dim;
    p.max_seq = max_seq;
    p.table_rows = table_rows;
    HIP_TRY(rt::launch_decode_prepare((hipStream_t)stream, p), "decode_prepare launch");
    return RT_OK;
}

static int check_decode_dims(int32_t batch, int32_t n_heads, int32_t n_kv, int32_t head_dim, int32_t max_seq,
                             rt_err_detail* err) {
    if (batch < 0 || n_heads < 0 || n_kv < 0 || head_dim < 0 || max_seq < 0)
        return fail(err, RT_ERR_UNSUPPORTED, -1, 0, 0, "negative dimension");
    if (n_kv == 0 || n_heads % n_kv != 0)
        return fail(err, RT_ERR_HEAD_COUNT_MISMATCH, -1, (uint64_t)n_heads, (uint64_t)n_kv,
                    "n_heads not divisible by n_kv");
    if (head_dim == 0) return fail(err, RT_ERR_ZERO_DIM, -1, 0, 0, "head_dim must be > 0");
    if (batch > 65535 || n_heads > 65535) return fail(err, RT_ERR_UNSUPPORTED, -1, 0, 0, "shape too large for the launch grid");
    return RT_OK;
}

RT_API int rt_gqa_decode_online_bf16(void* stream, const void* q, const void* k_cache, const void* v_cache,
                                     void* out, int32_t n_heads, int32_t n_kv, int32_t kv_len, int32_t head_dim,
                                     int32_t max_seq, rt_err_detail* err) {
    clear_err(err);
    int rc = check_decode_dims(1, n_heads, n_kv, head_dim, max_seq, err);
    if (rc) return rc;
    if (kv_len < 0 || kv_len > max_seq)
        return fail(err, RT_ERR_KV_OVERFLOW, -1, (uint64_t)max_seq, (uint64_t)(int64_t)kv_len, "kv_len outside the cache");
    if (n_heads == 0) return RT_OK;
    if (head_dim > 512) return fail(err, RT_ERR_UNSUPPORTED, -1, 512, (uint64_t)head_dim, "decode rows kernel covers dim <= 512");
    if (!q || !out || (kv_len > 0 && (!k_cache || !v_cache))) return fail(err, RT_ERR_NULL_POINTER, -1, 0, 0, "NULL buffer");
    rc = ensure_device(err);
    if (rc) return rc;
    // the split-K kernels move q, K and V 16 bytes at a time; tensors that are not 16-byte aligned take the
    // element-wise kernel below
    const bool aligned = ((((uintptr_t)q | (uintptr_t)k_cache | (uintptr_t)v_cache) & 15) == 0);
    if (aligned && rt::decode_split_supported(n_heads, n_kv, head_dim)) {
        // the split-K kernels of the batched entry, on a batch of one.  The reference's signature has no workspace
        // argument: the partials go to this stream's slot of the library's fixed scratch block (nothing is allocated,
        // so the call can be captured into a graph), in the compact slot numbering; only when no slot is free, or the
        // slot cannot hold a useful number of partials, to a buffer the library allocates per stream
        rt::DecodeSplitParams sp{};
        sp.span_min = rt::decode_split_span_min(1);
        // no more one-wave workgroups than there are spans of the minimum length (short contexts)
        const long long steps = (long long)n_kv * ((kv_len + 31) / 32);
        const long long spans = (steps + sp.span_min - 1) / sp.span_min;
        sp.n_waves = (int)std::min<long long>(g_decode_waves, std::max<long long>(spans, 1));
        float* ws = nullptr;
        size_t slot_bytes = 0;
        rc = stream_slot_scratch((hipStream_t)stream, &ws, &slot_bytes, err);
        if (rc) return rc;
        if (ws) {
            // compact numbering: (waves + n_kv) * group partials of head_dim + 2 floats
            const size_t per_wave = (size_t)(n_heads / n_kv) * ((size_t)head_dim + 2) * sizeof(float);
            const long long fit = (long long)(slot_bytes / per_wave) - n_kv;
            if (fit >= std::min<long long>(sp.n_waves, 256)) {
                sp.n_waves = (int)std::min<long long>(sp.n_waves, fit);
                sp.compact = 1;
            } else {
                ws = nullptr;
            }
        }
        if (!ws) {
            rc = stream_workspace((hipStream_t)stream, rt::decode_split_workspace_bytes(1, n_heads, head_dim, max_seq), &ws, err);
            if (rc) return rc;
        }
        sp.q = (const uint16_t*)q;
        sp.k_cache = (const uint16_t*)k_cache;
        sp.v_cache = (const uint16_t*)v_cache;
        sp.out = (uint16_t*)out;
        sp.kv_lens = nullptr;
        sp.kv_len = kv_len;
        sp.ws = ws;
        sp.batch = 1;
        sp.heads = n_heads;
        sp.kv_heads = n_kv;
        sp.dim = head_dim;
        sp.max_seq = max_seq;
        sp.n_part = rt::decode_split_parts(1, max_seq);
        sp.scale_log2e = (1.0f / sqrtf((float)head_dim)) * rt::kLog2eHost;
        HIP_TRY(rt::launch_decode_split((hipStream_t)stream, sp), "decode_split launch");
        return RT_OK;
    }
    rt::AttnRowsParams p{};
    p.q = q;
    p.k = k_cache;
    p.v = v_cache;
    p.out = out;
    p.kv_lens = nullptr;
    p.batch = 1;
    p.heads = n_heads;
    p.kv_heads = n_kv;
    p.seq_q = 1;
    p.kv_len = kv_len;
    p.kv_stride = max_seq;
    p.dim = head_dim;
    p.head_map = 1;
    p.scale = 1.0f / sqrtf((float)head_dim);
    HIP_TRY(rt::launch_attn_rows_bf16((hipStream_t)stream, p), "attn_rows_bf16 launch");
    return RT_OK;
}

RT_API int rt_gqa_decode_naive_bf16(void* stream, const void* q, const void* k_cache, const void* v_cache, void* out,
                                    int32_t n_heads, int32_t n_kv, int32_t kv_len, int32_t head_dim, int32_t max_seq,
                                    rt_err_detail* err) {
    return rt_gqa_decode_online_bf16(stream, q, k_cache, v_cache, out, n_heads, n_kv, kv_len, head_dim, max_seq, err);
}

// Several new positions per sequence against the cache, causally masked: the bf16 form of gqa_decode_batched_f32
// (crates/rustorch-metal/src/kernels.rs:14432-14516), batched over sequences with their own context lengths.
RT_API int rt_gqa_decode_chunk_bf16(void* stream, const void* q, const void* k_cache, const void* v_cache, void* out,
                                    const int32_t* kv_lens, int32_t kv_len, int32_t batch, int32_t seq_new,
                                    int32_t n_heads, int32_t n_kv, int32_t head_dim, int32_t max_seq,
                                    rt_err_detail* err) {
    clear_err(err);
    int rc = check_decode_dims(batch, n_heads, n_kv, head_dim, max_seq, err);
    if (rc) return rc;
    if (seq_new < 0) return fail(err, RT_ERR_UNSUPPORTED, -1, 0, 0, "negative dimension");
    if (!kv_lens && (kv_len < seq_new || kv_len > max_seq))
        return fail(err, RT_ERR_KV_OVERFLOW, -1, (uint64_t)max_seq, (uint64_t)(int64_t)kv_len,
                    "kv_len must cover the new positions and fit the cache");
    if (batch == 0 || n_heads == 0 || seq_new == 0) return RT_OK;
    if (!q || !out || !k_cache || !v_cache) return fail(err, RT_ERR_NULL_POINTER, -1, 0, 0, "NULL buffer");
    if (!rt::flash_tile_bf16_supported(head_dim))
        return fail(err, RT_ERR_UNSUPPORTED, -1, 256, (uint64_t)head_dim,
                    "bf16 kernels cover head dims up to 256 that are a multiple of 8");
    if ((((uintptr_t)q | (uintptr_t)k_cache | (uintptr_t)v_cache | (uintptr_t)out) & 15) != 0)
        return fail(err, RT_ERR_UNSUPPORTED, -1, 16, 0, "bf16 kernels need 16-byte aligned tensors");
    if (!rt::flash_tile_bf16_addressable((long long)max_seq, (long long)head_dim))
        return fail(err, RT_ERR_UNSUPPORTED, -1, 0, (uint64_t)max_seq, "a cache slab of one (sequence, kv head) must stay below 4 GiB");
    const int group = n_heads / n_kv;
    if (((int64_t)seq_new * group + 127) / 128 > 65535 || batch > 65535 || n_kv > 65535)
        return fail(err, RT_ERR_UNSUPPORTED, -1, 0, 0, "shape too large for the launch grid");
    rc = ensure_device(err);
    if (rc) return rc;
    rt::FlashTileParams t{};
    t.q = (const uint16_t*)q;
    t.k = (const uint16_t*)k_cache;
    t.v = (const uint16_t*)v_cache;
    t.out = (uint16_t*)out;
    t.kv_lens = kv_lens;
    t.batch = batch;
    t.heads = n_heads;
    t.kv_heads = n_kv;
    t.group = group;
    t.pack = group;  // rows of a tile run over (position, head of the group): one pass over a kv head's keys serves them all
    t.decode_rows = 1;  // (also with one head per group: a position without keys is a row of zeros)
    t.seq_q = seq_new;
    t.seq_kv = kv_lens ? max_seq : kv_len;
    t.dim = head_dim;
    t.mask = rt::kMaskCausal;  // position s sees keys [0, kv_len - seq_new + s]
    t.ref_bc = 64;
    t.zero_padded_rows = 0;
    t.scale = 1.0f / sqrtf((float)head_dim);
    t.scale_log2e = t.scale * rt::kLog2eHost;
    t.lq = t.lo = rt::layout_bnhd((long long)n_heads, (long long)seq_new, head_dim);
    t.lkv = rt::layout_bhnd((long long)n_kv, (long long)max_seq, head_dim);
    // Few (sequence, kv head, query tile) units and a long cache -- the reference's own call shape, one sequence:
    // cut the keys into spans so that every CU has a workgroup (two per CU measured 20 % slower at four new positions,
    // the same at sixteen), each span at least two key tiles long.  The
    // partials go to this stream's slot of the library's fixed scratch block (nothing is allocated); with no slot free,
    // to the buffer the library allocates per stream.
    const long long units = (long long)batch * n_kv * (((long long)seq_new * group + 127) / 128);
    const int key_tile = rt::flash_tile_bf16_key_tile(head_dim);
    const long long tiles_max = ((long long)t.seq_kv + key_tile - 1) / key_tile;
    long long n_splits = 1;
    if (units < g_num_cus && tiles_max >= 4)
        n_splits = std::min<long long>(std::min<long long>((g_num_cus + units - 1) / units, tiles_max / 2), 64);
    if (n_splits > 1) {
        const size_t per_split = (size_t)batch * n_kv * (size_t)seq_new * group * ((size_t)head_dim + 2) * sizeof(float);
        float* ws = nullptr;
        size_t slot_bytes = 0;
        rc = stream_slot_scratch((hipStream_t)stream, &ws, &slot_bytes, err);
        if (rc) return rc;
        if (ws && slot_bytes / per_split >= 2) {
            n_splits = std::min<long long>(n_splits, (long long)(slot_bytes / per_split));
        } else {
            rc = stream_workspace((hipStream_t)stream, per_split * (size_t)n_splits, &ws, err);
            if (rc) return rc;
        }
        t.n_splits = (int)n_splits;
        t.part_o = ws;
        t.part_ml = ws + (size_t)batch * n_kv * (size_t)seq_new * group * (size_t)n_splits * (size_t)head_dim;
    }
    HIP_TRY(rt::launch_flash_tile_bf16((hipStream_t)stream, t), "flash_tile_bf16 launch");
    return RT_OK;
}

RT_API size_t rt_gqa_decode_workspace_bytes(int32_t batch, int32_t n_heads, int32_t n_kv, int32_t head_dim,
                                            int32_t max_seq) {
    if (batch <= 0 || n_heads <= 0 || n_kv <= 0 || head_dim <= 0 || max_seq < 0) return 0;
    if (!rt::decode_split_supported(n_heads, n_kv, head_dim)) return 0;
    return rt::decode_split_workspace_bytes(batch, n_heads, head_dim, max_seq);
}

RT_API int rt_gqa_decode_batched_bf16(void* stream, const void* q, const void* k_cache, const void* v_cache,
                                      void* out, const int32_t* kv_lens, int32_t batch, int32_t n_heads,
                                      int32_t n_kv, int32_t head_dim, int32_t max_seq, void* workspace,
                                      size_t workspace_bytes, rt_err_detail* err) {
    clear_err(err);
    int rc = check_decode_dims(batch, n_heads, n_kv, head_dim, max_seq, err);
    if (rc) return rc;
    if (batch == 0 || n_heads == 0) return RT_OK;
    if (!q || !out || !kv_lens || (max_seq > 0 && (!k_cache || !v_cache)))
        return fail(err, RT_ERR_NULL_POINTER, -1, 0, 0, "NULL buffer");
    rc = ensure_device(err);
    if (rc) return rc;
    // the split-K kernels move q, K, V and the partials 16 bytes at a time; tensors that are not 16-byte aligned
    // take the element-wise kernel below, which needs no workspace
    const bool aligned = ((((uintptr_t)q | (uintptr_t)k_cache | (uintptr_t)v_cache) & 15) == 0);
    if (aligned && rt::decode_split_supported(n_heads, n_kv, head_dim)) {
        size_t need = rt::decode_split_workspace_bytes(batch, n_heads, head_dim, max_seq);
        if (!workspace || workspace_bytes < need)
            return fail(err, RT_ERR_WORKSPACE_TOO_SMALL, -1, need, workspace ? workspace_bytes : 0, "workspace too small");
        if ((uintptr_t)workspace & 15)
            return fail(err, RT_ERR_WORKSPACE_TOO_SMALL, -1, 16, (uint64_t)((uintptr_t)workspace & 15),
                        "workspace must be 16-byte aligned");
        rt::DecodeSplitParams p{};
        p.q = (const uint16_t*)q;
        p.k_cache = (const uint16_t*)k_cache;
        p.v_cache = (const uint16_t*)v_cache;
        p.out = (uint16_t*)out;
        p.kv_lens = kv_lens;
        p.ws = (float*)workspace;
        p.batch = batch;
        p.heads = n_heads;
        p.kv_heads = n_kv;
        p.dim = head_dim;
        p.max_seq = max_seq;
        p.n_part = rt::decode_split_parts(batch, max_seq);
        p.span_min = rt::decode_split_span_min(batch);
        p.n_waves = g_decode_waves;
        p.scale_log2e = (1.0f / sqrtf((float)head_dim)) * rt::kLog2eHost;
        HIP_TRY(rt::launch_decode_split((hipStream_t)stream, p), "decode_split launch");
        return RT_OK;
    }
    // shapes outside the split-K kernel: one workgroup per (sequence, head), no workspace
    if (head_dim > 512) return fail(err, RT_ERR_UNSUPPORTED, -1, 512, (uint64_t)head_dim, "decode rows kernel covers dim <= 512");
    rt::AttnRowsParams p{};
    p.q = q;
    p.k = k_cache;
    p.v = v_cache;
    p.out = out;
    p.kv_lens = kv_lens;
    p.batch = batch;
    p.heads = n_heads;
    p.kv_heads = n_kv;
    p.seq_q = 1;
    p.kv_len = 0;
    p.kv_stride = max_seq;
    p.dim = head_dim;
    p.head_map = 1;
    p.scale = 1.0f / sqrtf((float)head_dim);
    HIP_TRY(rt::launch_attn_rows_bf16((hipStream_t)stream, p), "attn_rows_bf16 launch");
    return RT_OK;
}

// The batched decode for callers that cannot allocate (under HIP graph capture, in serving loops or harnesses that
// forbid hipMalloc): the partials go to the library's fixed scratch block in device memory instead of a workspace
// argument.  Calls nothing that allocates or frees.
RT_API int rt_gqa_decode_batched_bf16_noalloc(void* stream, const void* q, const void* k_cache, const void* v_cache,
                                              void* out, const int32_t* kv_lens, int32_t batch, int32_t n_heads,
                                              int32_t n_kv, int32_t head_dim, int32_t max_seq, rt_err_detail* err) {
    clear_err(err);
    int rc = check_decode_dims(batch, n_heads, n_kv, head_dim, max_seq, err);
    if (rc) return rc;
    if (batch == 0 || n_heads == 0) return RT_OK;
    if (!q || !out || !kv_lens || (max_seq > 0 && (!k_cache || !v_cache)))
        return fail(err, RT_ERR_NULL_POINTER, -1, 0, 0, "NULL buffer");
    rc = ensure_device(err);
    if (rc) return rc;
    if (!rt::decode_split_supported(n_heads, n_kv, head_dim))
        return fail(err, RT_ERR_UNSUPPORTED, -1, 0, (uint64_t)head_dim,
                    "the no-allocation decode covers head_dim 64, 128, 256 with at most 16 query heads per kv head");
    if ((((uintptr_t)q | (uintptr_t)k_cache | (uintptr_t)v_cache) & 15) != 0)
        return fail(err, RT_ERR_UNSUPPORTED, -1, 16, 0, "the no-allocation decode needs 16-byte aligned q and caches");
    float* scratch = nullptr;
    size_t scratch_bytes = 0;
    HIP_TRY(rt::decode_static_scratch(&scratch, &scratch_bytes), "hipGetSymbolAddress(static scratch)");
    const size_t need = rt::decode_split_compact_bytes(batch, n_heads, n_kv, head_dim, g_decode_waves);
    if (need > scratch_bytes)
        return fail(err, RT_ERR_WORKSPACE_TOO_SMALL, -1, (uint64_t)need, (uint64_t)scratch_bytes,
                    "batch too large for the library's fixed scratch block; use rt_gqa_decode_batched_bf16 with a workspace");
    rt::DecodeSplitParams p{};
    p.q = (const uint16_t*)q;
    p.k_cache = (const uint16_t*)k_cache;
    p.v_cache = (const uint16_t*)v_cache;
    p.out = (uint16_t*)out;
    p.kv_lens = kv_lens;
    p.ws = scratch;
    p.batch = batch;
    p.heads = n_heads;
    p.kv_heads = n_kv;
    p.dim = head_dim;
    p.max_seq = max_seq;
    p.n_part = rt::decode_split_parts(batch, max_seq);
    p.span_min = rt::decode_split_span_min(batch);
    p.n_waves = g_decode_waves;
    p.scale_log2e = (1.0f / sqrtf((float)head_dim)) * rt::kLog2eHost;
    p.compact = 1;
    HIP_TRY(rt::launch_decode_split((hipStream_t)stream, p), "decode_split launch");
    return RT_OK;
}

// ---- device buffers ------------------------------------------------------------------------------------

RT_API void* rt_buf_alloc(size_t bytes, rt_err_detail* err) {
    clear_err(err);
    if (ensure_device(err) != RT_OK) return nullptr;
    void* p = nullptr;
    hipError_t e = hipMalloc(&p, bytes ? bytes : 1);
    if (e != hipSuccess) {
        fail_hip(err, e, "hipMalloc");
        return nullptr;
    }
    return p;
}

RT_API int rt_buf_free(void* ptr, rt_err_detail* err) {
    clear_err(err);
    if (!ptr) return RT_OK;
    HIP_TRY(hipFree(ptr), "hipFree");
    return RT_OK;
}

namespace {
__global__ __launch_bounds__(256) void zero_fill_kernel(uint32_t* p, size_t n_words) {
    const size_t n4 = n_words / 4;
    uint4* p4 = (uint4*)p;
    const size_t stride = (size_t)gridDim.x * blockDim.x, t = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (((uintptr_t)p & 15) == 0) {
        for (size_t i = t; i < n4; i += stride) p4[i] = make_uint4(0u, 0u, 0u, 0u);
        for (size_t i = 4 * n4 + t; i < n_words; i += stride) p[i] = 0u;
    } else {
        for (size_t i = t; i < n_words; i += stride) p[i] = 0u;
    }
}
}  // namespace

RT_API int rt_buf_zero(void* ptr, size_t bytes, void* stream, rt_err_detail* err) {
    clear_err(err);
    if (bytes == 0) return RT_OK;
    if (!ptr) return fail(err, RT_ERR_NULL_POINTER, -1, 0, 0, "NULL buffer");
    if ((bytes & 3) || ((uintptr_t)ptr & 3)) return fail(err, RT_ERR_UNSUPPORTED, -1, 0, (uint64_t)bytes, "zero fill works on 4-byte words");
    int rc = ensure_device(err);
    if (rc) return rc;
    const size_t n_words = bytes / 4;
    const unsigned blocks = (unsigned)std::min<size_t>((n_words / 4 + 255) / 256 + 1, 4096);
    hipLaunchKernelGGL(zero_fill_kernel, dim3(blocks), dim3(256), 0, (hipStream_t)stream, (uint32_t*)ptr, n_words);
    HIP_TRY(hipGetLastError(), "zero_fill launch");
    return RT_OK;
}

namespace {
__global__ __launch_bounds__(256) void i32_add_kernel(int32_t* p, size_t n, int32_t delta) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] += delta;
}
}  // namespace

RT_API int rt_i32_add_dev(void* stream, int32_t* ptr, size_t n, int32_t delta, rt_err_detail* err) {
    clear_err(err);
    if (n == 0) return RT_OK;
    if (!ptr) return fail(err, RT_ERR_NULL_POINTER, -1, 0, 0, "NULL buffer");
    if (((uintptr_t)ptr & 3) || n > ((size_t)1 << 30)) return fail(err, RT_ERR_UNSUPPORTED, -1, 0, (uint64_t)n, "int32 add works on up to 2^30 aligned values");
    int rc = ensure_device(err);
    if (rc) return rc;
    hipLaunchKernelGGL(i32_add_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, (hipStream_t)stream, ptr, n, delta);
    HIP_TRY(hipGetLastError(), "i32_add launch");
    return RT_OK;
}

RT_API int rt_memcpy_h2d(void* dst, const void* src, size_t bytes, void* stream, rt_err_detail* err) {
    clear_err(err);
    if (bytes == 0) return RT_OK;
    if (!dst || !src) return fail(err, RT_ERR_NULL_POINTER, -1, 0, 0, "NULL buffer");
    HIP_TRY(hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, (hipStream_t)stream), "hipMemcpyAsync h2d");
    return RT_OK;
}

RT_API int rt_memcpy_d2h(void* dst, const void* src, size_t bytes, void* stream, rt_err_detail* err) {
    clear_err(err);
    if (bytes == 0) return RT_OK;
    if (!dst || !src) return fail(err, RT_ERR_NULL_POINTER, -1, 0, 0, "NULL buffer");
    HIP_TRY(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, (hipStream_t)stream), "hipMemcpyAsync d2h");
    return RT_OK;
}

RT_API int rt_stream_synchronize(void* stream, rt_err_detail* err) {
    clear_err(err);
    HIP_TRY(hipStreamSynchronize((hipStream_t)stream), "hipStreamSynchronize");
    return RT_OK;
}

RT_API void* rt_stream_create(rt_err_detail* err) {
    clear_err(err);
    if (ensure_device(err) != RT_OK) return nullptr;
    hipStream_t s = nullptr;
    hipError_t e = hipStreamCreate(&s);
    if (e != hipSuccess) {
        fail_hip(err, e, "hipStreamCreate");
        return nullptr;
    }
    return (void*)s;
}

RT_API int rt_stream_destroy(void* stream, rt_err_detail* err) {
    clear_err(err);
    if (!stream) return RT_OK;
    {
        // the library's scratch for this stream goes with it
        std::lock_guard<std::mutex> lock(g_ws_mutex);
        int dev = 0;
        if (hipGetDevice(&dev) == hipSuccess) {
            auto it = g_ws.find({dev, (hipStream_t)stream});
            if (it != g_ws.end()) {
                (void)hipStreamSynchronize((hipStream_t)stream);
                release_stream_ws(it->second);
                g_ws.erase(it);
            }
            release_stream_slot(dev, (hipStream_t)stream);
        }
    }
    HIP_TRY(hipStreamDestroy((hipStream_t)stream), "hipStreamDestroy");
    return RT_OK;
}

RT_API int rt_shutdown(rt_err_detail* err) {
    clear_err(err);
    // what the library keeps between calls: the per-stream scratch of rt_gqa_decode_online_bf16 and the pinned staging
    // buffer of the host-slice entries.  The caller makes sure no call is in flight.
    {
        std::lock_guard<std::mutex> lock(g_ws_mutex);
        for (auto& kv : g_ws) {
            if (kv.second.ptr) (void)hipStreamSynchronize(kv.first.second);
            release_stream_ws(kv.second);
        }
        g_ws.clear();
        g_slots.clear();
    }
    {
        std::lock_guard<std::mutex> lock(g_pinned_mutex);
        if (g_pinned) (void)hipHostFree(g_pinned);
        g_pinned = nullptr;
    }
    (void)hipGetLastError();
    return RT_OK;
}
