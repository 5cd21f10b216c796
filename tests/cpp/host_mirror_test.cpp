// Tests of the C++ host mirror (include/rustorch_attn.hpp), written after the reference's own unit tests
// (crates/rustorch-attention/src/cpu_forward.rs tests module, crates/rustorch-nn/src/gqa.rs tests).
//   host_mirror_test errors   error enums and their order: needs no GPU
//   host_mirror_test gpu      small forwards against a double-precision loop and the reference's closed forms
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <limits>
#include <vector>

#include "rustorch_attn.hpp"

using namespace rustorch_attn;

static int g_failed = 0;
#define CHECK(cond)                                                          \
    do {                                                                     \
        if (!(cond)) {                                                       \
            std::printf("FAIL %s:%d: %s\n", __FILE__, __LINE__, #cond);      \
            ++g_failed;                                                      \
        }                                                                    \
    } while (0)

template <typename E, typename F>
static bool throws(F&& f, E* out = nullptr) {
    try {
        f();
    } catch (const E& e) {
        if (out) *out = e;
        return true;
    } catch (...) {
        return false;
    }
    return false;
}

static std::vector<float> lcg(size_t n, uint64_t seed) {  // uniform in [-1, 1)
    std::vector<float> v(n);
    uint64_t s = seed * 6364136223846793005ull + 1442695040888963407ull;
    for (size_t i = 0; i < n; i++) {
        s = s * 6364136223846793005ull + 1442695040888963407ull;
        v[i] = (float)((double)(s >> 11) / 9007199254740992.0 * 2.0 - 1.0);
    }
    return v;
}

// softmax(q k^T / sqrt(d)) v in double, with the reference's "no visible key -> NaN row" rule
static std::vector<float> naive(const AttentionShape& s, const std::vector<float>& q, const std::vector<float>& k,
                                const std::vector<float>& v, const Mask& mask) {
    std::vector<float> out(s.buffer_len());
    const double scale = 1.0 / std::sqrt((double)s.dim);
    std::vector<double> sc(s.seq);
    for (size_t bh = 0; bh < s.batch * s.heads; bh++) {
        const float* Q = q.data() + bh * s.seq * s.dim;
        const float* K = k.data() + bh * s.seq * s.dim;
        const float* V = v.data() + bh * s.seq * s.dim;
        for (size_t i = 0; i < s.seq; i++) {
            double m = -std::numeric_limits<double>::infinity();
            for (size_t j = 0; j < s.seq; j++) {
                double d = 0;
                for (size_t t = 0; t < s.dim; t++) d += (double)Q[i * s.dim + t] * K[j * s.dim + t];
                sc[j] = mask.is_masked(i, j) ? -std::numeric_limits<double>::infinity() : d * scale;
                if (sc[j] > m) m = sc[j];
            }
            double l = 0;
            for (size_t j = 0; j < s.seq; j++) l += std::isinf(m) ? 0.0 : std::exp(sc[j] - m);
            for (size_t t = 0; t < s.dim; t++) {
                double o = 0;
                for (size_t j = 0; j < s.seq; j++) o += (std::isinf(m) ? 0.0 : std::exp(sc[j] - m)) * V[j * s.dim + t];
                out[(bh * s.seq + i) * s.dim + t] = l > 0 ? (float)(o / l) : std::numeric_limits<float>::quiet_NaN();
            }
        }
    }
    return out;
}

static void test_errors() {
    {   // the strict switch needs no device and returns the previous setting
        CHECK(set_strict_non_finite_v(true) == false);
        CHECK(set_strict_non_finite_v(false) == true);
        CHECK(set_strict_non_finite_v(false) == false);
    }
    {   // ZeroDim comes first (cpu_forward.rs:142-169)
        std::vector<float> e, out;
        AttentionError err(AttentionError::Kind::ZeroDim, "", 0, 0, "");
        CHECK(throws<AttentionError>([&] { flash_forward(AttentionShape::make(1, 1, 4, 0), e, e, e, out); }, &err));
        CHECK(err.kind == AttentionError::Kind::ZeroDim);
    }
    {   // then q, k, v lengths, then the output, then the padding mask
        AttentionShape s = AttentionShape::make(1, 1, 4, 8);
        std::vector<float> good(32), bad(16), out(32);
        const char* which[3] = {"q", "k", "v"};
        for (int i = 0; i < 3; i++) {
            AttentionError err(AttentionError::Kind::ZeroDim, "", 0, 0, "");
            const std::vector<float>& a = i == 0 ? bad : good;
            const std::vector<float>& b = i <= 1 ? bad : good;
            CHECK(throws<AttentionError>([&] { flash_forward(s, a, b, bad, out); }, &err));
            CHECK(err.kind == AttentionError::Kind::BufferShapeMismatch && err.which == which[i]);
            CHECK(err.expected == 32 && err.got == 16);
            CHECK(std::string(err.what()) == std::string(which[i]) + " buffer has 16 elements, expected 32");
        }
        std::vector<float> short_out(31);
        AttentionError err(AttentionError::Kind::ZeroDim, "", 0, 0, "");
        CHECK(throws<AttentionError>([&] { flash_forward(s, good, good, good, short_out); }, &err));
        CHECK(err.kind == AttentionError::Kind::OutputShapeMismatch && err.expected == 32 && err.got == 31);
        AttentionShape s4 = AttentionShape::make(1, 1, 4, 4);
        std::vector<float> out16(16);
        CHECK(throws<AttentionError>(
            [&] { flash_forward_masked(s4, bad, bad, bad, Mask::padding({true, true, true}), out16); }, &err));
        CHECK(err.kind == AttentionError::Kind::MaskPaddingLengthMismatch && err.expected == 4 && err.got == 3);
    }
    {   // seq == 0 is Ok and touches nothing (cpu_forward.rs:203-206)
        std::vector<float> e, out;
        flash_forward(AttentionShape::make(2, 4, 0, 16), e, e, e, out);
    }
    {   // backward: q, k, v, "do" in that order, then the outputs with got = the longest (cpu_backward.rs:59-77)
        AttentionShape s = AttentionShape::make(1, 1, 4, 4);
        std::vector<float> good(16), bad(10), g16(16), g20(20), g7(7);
        const char* which[4] = {"q", "k", "v", "do"};
        for (int i = 0; i < 4; i++) {
            const std::vector<float>& a = i > 0 ? good : bad;
            const std::vector<float>& b = i > 1 ? good : bad;
            const std::vector<float>& c = i > 2 ? good : bad;
            AttentionError err(AttentionError::Kind::ZeroDim, "", 0, 0, "");
            CHECK(throws<AttentionError>([&] { flash_backward(s, a, b, c, bad, g7, g7, g7); }, &err));
            CHECK(err.kind == AttentionError::Kind::BufferShapeMismatch && err.which == which[i]);
            CHECK(err.expected == 16 && err.got == 10);
        }
        AttentionError err(AttentionError::Kind::ZeroDim, "", 0, 0, "");
        CHECK(throws<AttentionError>([&] { flash_backward(s, good, good, good, good, g16, g20, g7); }, &err));
        CHECK(err.kind == AttentionError::Kind::OutputShapeMismatch && err.expected == 16 && err.got == 20);
        std::vector<float> e;
        flash_backward(AttentionShape::make(1, 1, 0, 4), e, e, e, e, e, e, e);  // cpu_backward.rs:252-260
    }
    {   // the routing of MultiHeadAttention::forward (attention.rs:325-333, :347-356)
        CHECK(mha_attention_route(1, 1, false) == MhaRoute::Identity);
        CHECK(mha_attention_route(1, 1, true) == MhaRoute::Composed);
        CHECK(mha_attention_route(64, 64, false) == MhaRoute::Flash);
        CHECK(mha_attention_route(64, 64, true) == MhaRoute::Composed);
        CHECK(mha_attention_route(1, 64, false) == MhaRoute::Composed);
        std::vector<float> v = {1, 2, 3, 4, 5, 6, 7, 8};
        CHECK(mha_attention_f32(v, v, v, 2, 1, 1, 2, 2) == v);  // needs no device
    }
    {   // GQA: head counts first, then q, k, v, out (gqa.rs:106-141)
        std::vector<float> q(20), kv(8), out(20);
        GQAError err(GQAError::Kind::WrongInputLen, "", 0, 0, "");
        CHECK(throws<GQAError>([&] { gqa_forward_f32(q, kv, kv, out, 1, 5, 2, 1, 1, 4); }, &err));
        CHECK(err.kind == GQAError::Kind::HeadCountMismatch && err.expected == 5 && err.got == 2);
        std::vector<float> q16(16), q7(7), kv9(9), out15(15);
        CHECK(throws<GQAError>([&] { gqa_forward_f32(q7, kv, kv, q16, 1, 4, 2, 1, 1, 4); }, &err));
        CHECK(err.which == "q" && err.expected == 16 && err.got == 7);
        CHECK(throws<GQAError>([&] { gqa_forward_f32(q16, kv9, kv, q16, 1, 4, 2, 1, 1, 4); }, &err));
        CHECK(err.which == "k" && err.expected == 8 && err.got == 9);
        CHECK(throws<GQAError>([&] { gqa_forward_f32(q16, kv, kv9, q16, 1, 4, 2, 1, 1, 4); }, &err));
        CHECK(err.which == "v");
        CHECK(throws<GQAError>([&] { gqa_forward_f32(q16, kv, kv, out15, 1, 4, 2, 1, 1, 4); }, &err));
        CHECK(err.which == "out" && err.expected == 16 && err.got == 15);
    }
    {   // shape helpers
        AttentionShape s = AttentionShape::make(2, 3, 5, 7);
        CHECK(s.buffer_len() == 210 && s.br == 64 && s.bc == 64);
        auto st = s.strides();
        CHECK(st[0] == 105 && st[1] == 35 && st[2] == 7 && st[3] == 1);
        CHECK(Mask::causal().is_masked(1, 2) && !Mask::causal().is_masked(2, 2));
        CHECK(Mask::padding({true, false}).is_masked(0, 1) && !Mask::padding({true, false}).is_masked(0, 0));
    }
    {   // additive masks (masks.rs:88-208)
        auto c = causal_mask(3);
        CHECK(c[0] == 0 && c[1] == kMaskNeg && c[3] == 0 && c[4] == 0 && c[5] == kMaskNeg && c[8] == 0);
        CHECK(sliding_window_mask(5, 100) == causal_mask(5));
        auto w = sliding_window_mask(4, 1);
        for (int i = 0; i < 4; i++)
            for (int j = 0; j < 4; j++) CHECK((w[i * 4 + j] == 0.0f) == (i == j));
        auto a = bool_to_additive({1.0f, 0.0f, 1.0f, 1.0f});
        CHECK(a[0] == 0 && a[1] == kMaskNeg && a[2] == 0 && a[3] == 0);
    }
    {   // RoPE::new: position 0 is cos 1 / sin 0, theta_0 = 1, odd head_dim refused (rope.rs:63-90)
        RoPE rope(4, 8);
        CHECK(rope.cos_table().size() == 16 && rope.cos_table()[0] == 1.0f && rope.sin_table()[1] == 0.0f);
        CHECK(std::fabs(rope.cos_table()[2 * 3] - std::cos(3.0f)) < 1e-6f);
        bool threw = false;
        try { RoPE bad(5, 4); } catch (const std::invalid_argument&) { threw = true; }
        CHECK(threw);
    }
    {   // a host position is checked like the reference: the RoPE tables first, then the cache (no device needed)
        RoPE rope(8, 16);
        uint16_t dummy[8] = {0};
        bool ok = false;
        try {
            LlmKernels::qk_norm_rope_kv_append_bf16(nullptr, dummy, dummy, dummy, dummy, dummy, nullptr, 16, nullptr, nullptr,
                                                    1e-6f, rope, 1, 1, 1, 8, 32);
        } catch (const RoPEError& e) {
            ok = e.kind == RoPEError::Kind::PositionOverflow && e.expected == 16 && e.got == 17;
        } catch (const DeviceError&) {
        }
        CHECK(ok);
    }
}

static float max_abs_diff(const std::vector<float>& a, const std::vector<float>& b, bool* nan_same) {
    float m = 0;
    *nan_same = true;
    for (size_t i = 0; i < a.size(); i++) {
        if (std::isnan(a[i]) != std::isnan(b[i])) *nan_same = false;
        if (!std::isnan(a[i]) && !std::isnan(b[i])) m = std::fmax(m, std::fabs(a[i] - b[i]));
    }
    return m;
}

static void test_gpu() {
    const size_t shapes[][4] = {{1, 1, 1, 4}, {1, 2, 7, 8}, {2, 3, 33, 16}, {1, 2, 130, 64}, {1, 1, 65, 128}};
    for (auto& sh : shapes) {
        AttentionShape s = AttentionShape::make(sh[0], sh[1], sh[2], sh[3]);
        auto q = lcg(s.buffer_len(), 1), k = lcg(s.buffer_len(), 2), v = lcg(s.buffer_len(), 3);
        std::vector<bool> keep(s.seq);
        for (size_t j = 0; j < s.seq; j++) keep[j] = (j % 3 != 1);
        const Mask masks[3] = {Mask::none(), Mask::causal(), Mask::padding(keep)};
        for (const Mask& m : masks) {
            std::vector<float> out(s.buffer_len(), -7.0f);
            flash_forward_masked(s, q, k, v, m, out);
            bool nan_same;
            float d = max_abs_diff(out, naive(s, q, k, v, m), &nan_same);
            CHECK(nan_same);
            CHECK(d <= 1e-5f);
        }
    }
    {   // backward against central differences of the forward (cpu_backward.rs:230-250) and its closed forms
        AttentionShape s = AttentionShape::make(1, 2, 6, 4);
        auto q = lcg(s.buffer_len(), 1), k = lcg(s.buffer_len(), 2), v = lcg(s.buffer_len(), 3), d_out = lcg(s.buffer_len(), 4);
        std::vector<float> dq(s.buffer_len(), -7.0f), dk(dq), dv(dq);
        flash_backward(s, q, k, v, d_out, dq, dk, dv);
        std::vector<float>* ins[3] = {&q, &k, &v};
        std::vector<float>* grads[3] = {&dq, &dk, &dv};
        for (int w = 0; w < 3; w++)
            for (size_t idx : {size_t(0), size_t(5), size_t(10), size_t(29), size_t(47)}) {
                const float saved = (*ins[w])[idx], eps = 1e-2f;
                std::vector<float> op(s.buffer_len()), om(s.buffer_len());
                (*ins[w])[idx] = saved + eps;
                flash_forward(s, q, k, v, op);
                (*ins[w])[idx] = saved - eps;
                flash_forward(s, q, k, v, om);
                (*ins[w])[idx] = saved;
                double g = 0.0;
                for (size_t i = 0; i < op.size(); i++) g += (double)d_out[i] * ((double)op[i] - om[i]) / (2.0 * eps);
                CHECK(std::fabs((*grads[w])[idx] - g) < 2e-3);
            }
        std::vector<float> zero(s.buffer_len(), 0.0f);
        flash_backward(s, q, k, v, zero, dq, dk, dv);  // cpu_backward.rs:279-299
        for (size_t i = 0; i < dq.size(); i++) CHECK(dq[i] == 0.0f && dk[i] == 0.0f && dv[i] == 0.0f);
        // a single key: P == 1, so dV = dO exactly; dQ = dK = 0 up to the rounding of dO.V summed in two orders
        AttentionShape one = AttentionShape::make(2, 2, 1, 16);
        auto q1 = lcg(one.buffer_len(), 5), g1 = lcg(one.buffer_len(), 6);
        std::vector<float> a(one.buffer_len()), b(a), c(a);
        flash_backward(one, q1, q1, q1, g1, a, b, c);
        for (size_t i = 0; i < a.size(); i++) CHECK(std::fabs(a[i]) < 1e-6f && std::fabs(b[i]) < 1e-6f && c[i] == g1[i]);
    }
    {   // the device-resident backward on a stream of its own, recomputing and from a saved forward: the host entry's bits
        AttentionShape s = AttentionShape::make(2, 2, 70, 32);
        const size_t n = s.buffer_len(), bytes = n * sizeof(float);
        auto q = lcg(n, 11), k = lcg(n, 12), v = lcg(n, 13), g = lcg(n, 14);
        std::vector<float> dq(n), dk(n), dv(n);
        flash_backward(s, q, k, v, g, dq, dk, dv);
        Stream st;
        HipStorage hq(bytes), hk(bytes), hv(bytes), hg(bytes), ho(bytes), hl(2 * 2 * 70 * sizeof(float));
        HipStorage gq(bytes), gk(bytes), gv(bytes), ws(flash_backward_workspace_bytes(s));
        hq.upload(q.data(), bytes, st.get());
        hk.upload(k.data(), bytes, st.get());
        hv.upload(v.data(), bytes, st.get());
        hg.upload(g.data(), bytes, st.get());
        auto f = [](const HipStorage& h) { return (float*)h.ptr(); };
        flash_backward_f32_dev(s, f(hq), f(hk), f(hv), f(hg), f(gq), f(gk), f(gv), ws.ptr(), ws.byte_len(), st.get());
        synchronize(st.get());
        CHECK(gq.to_host<float>() == dq && gk.to_host<float>() == dk && gv.to_host<float>() == dv);
        HipStorage sq(bytes), sk(bytes), sv(bytes);
        flash_forward_stats_f32_dev(s, f(hq), f(hk), f(hv), f(ho), f(hl), st.get());
        flash_backward_saved_f32_dev(s, f(hq), f(hk), f(hv), f(ho), f(hl), f(hg), f(sq), f(sk), f(sv), ws.ptr(),
                                     ws.byte_len(), st.get());
        synchronize(st.get());
        CHECK(sq.to_host<float>() == dq && sk.to_host<float>() == dk && sv.to_host<float>() == dv);
    }
    {   // N == 1: out == v (reference test single_token_returns_v)
        AttentionShape s = AttentionShape::make(1, 1, 1, 4);
        std::vector<float> q = {1, 2, 3, 4}, k = {4, 3, 2, 1}, v = {0.5f, -1.5f, 2.5f, 7.0f}, out(4);
        flash_forward(s, q, k, v, out);
        for (int i = 0; i < 4; i++) CHECK(out[i] == v[i]);
    }
    {   // keep = [T, F, F, T] with equal scores: the mean of V rows 0 and 3
        AttentionShape s = AttentionShape::make(1, 1, 4, 1);
        std::vector<float> q(4, 0.0f), k(4, 0.0f), v = {10, 99, 99, 30}, out(4);
        flash_forward_masked(s, q, k, v, Mask::padding({true, false, false, true}), out);
        for (int i = 0; i < 4; i++) CHECK(std::fabs(out[i] - 20.0f) <= 1e-5f);
    }
    {   // mha_flash_forward_f32 == flash_forward on transposed copies
        size_t b = 2, t = 9, h = 3, d = 8;
        auto q = lcg(b * t * h * d, 5), k = lcg(b * t * h * d, 6), v = lcg(b * t * h * d, 7);
        auto tr = [&](const std::vector<float>& x) {  // [B,T,H,D] -> [B,H,T,D]
            std::vector<float> y(x.size());
            for (size_t bi = 0; bi < b; bi++)
                for (size_t ti = 0; ti < t; ti++)
                    for (size_t hi = 0; hi < h; hi++)
                        for (size_t di = 0; di < d; di++)
                            y[((bi * h + hi) * t + ti) * d + di] = x[((bi * t + ti) * h + hi) * d + di];
            return y;
        };
        AttentionShape s = AttentionShape::make(b, h, t, d);
        auto want = naive(s, tr(q), tr(k), tr(v), Mask::none());
        auto got = mha_flash_forward_f32(q, k, v, b, t, h, d);
        float m = 0;
        for (size_t bi = 0; bi < b; bi++)
            for (size_t ti = 0; ti < t; ti++)
                for (size_t hi = 0; hi < h; hi++)
                    for (size_t di = 0; di < d; di++)
                        m = std::fmax(m, std::fabs(got[((bi * t + ti) * h + hi) * d + di] -
                                                    want[((bi * h + hi) * t + ti) * d + di]));
        CHECK(m <= 1e-5f);
    }
    {   // decode preparation: at position 0 without norms the rotation is the identity (rope.rs:247-256), so q is
        // unchanged and row 0 of the caches holds k_in / v_in; at position 1, theta_0 = 1 rotates the pair (0, D/2)
        // of a unit vector to (cos 1, sin 1)
        const int hq = 2, hkv = 1, d = 8, lmax = 4;
        auto bf = [](float x) { uint32_t u; std::memcpy(&u, &x, 4); return (uint16_t)(u >> 16); };
        auto fb = [](uint16_t h) { uint32_t u = (uint32_t)h << 16; float f; std::memcpy(&f, &u, 4); return f; };
        std::vector<uint16_t> q(hq * d), k(hkv * d), v(hkv * d), cache(hkv * lmax * d, bf(9.0f));
        for (int i = 0; i < hq * d; i++) q[i] = bf(0.25f * (float)(i % 7) - 0.5f);
        for (int i = 0; i < hkv * d; i++) { k[i] = bf(i == 0 ? 1.0f : 0.0f); v[i] = bf(0.5f * (float)i); }
        RoPE rope(d, 16);
        HipStorage dq = HipStorage::from_host(q), dk = HipStorage::from_host(k), dv = HipStorage::from_host(v);
        HipStorage dkc = HipStorage::from_host(cache), dvc = HipStorage::from_host(cache);
        LlmKernels::qk_norm_rope_kv_append_bf16(nullptr, dq.ptr(), dk.ptr(), dv.ptr(), dkc.ptr(), dvc.ptr(), nullptr, 0, nullptr,
                                                nullptr, 1e-6f, rope, 1, hq, hkv, d, lmax);
        synchronize();
        CHECK(dq.to_host<uint16_t>() == q);
        auto kc = dkc.to_host<uint16_t>(), vc = dvc.to_host<uint16_t>();
        for (int i = 0; i < d; i++) CHECK(kc[i] == k[i] && vc[i] == v[i] && kc[d + i] == bf(9.0f));
        LlmKernels::qk_norm_rope_kv_append_bf16(nullptr, dq.ptr(), dk.ptr(), dv.ptr(), dkc.ptr(), dvc.ptr(), nullptr, 1, nullptr,
                                                nullptr, 1e-6f, rope, 1, hq, hkv, d, lmax);
        synchronize();
        kc = dkc.to_host<uint16_t>();
        CHECK(std::fabs(fb(kc[d + 0]) - std::cos(1.0f)) < 4e-3f && std::fabs(fb(kc[d + d / 2]) - std::sin(1.0f)) < 4e-3f);
        for (int i = 1; i < d / 2; i++) CHECK(kc[d + i] == 0 && kc[d + d / 2 + i] == 0);
    }
    {   // masked core of MultiHeadAttention: zero q/k + causal mask gives prefix means of V; sliding window 1 gives V itself
        size_t b = 1, t = 5, h = 2, d = 4;
        std::vector<float> z(b * t * h * d, 0.0f), v = lcg(b * t * h * d, 13);
        auto got = mha_forward_masked_f32(z, z, v, b, t, t, h, d, causal_mask(t));
        for (size_t i = 0; i < t; i++)
            for (size_t c = 0; c < h * d; c++) {
                double mean = 0;
                for (size_t j = 0; j <= i; j++) mean += v[j * h * d + c];
                CHECK(std::fabs(got[i * h * d + c] - (float)(mean / (double)(i + 1))) <= 1e-5f);
            }
        auto diag = mha_forward_masked_f32(z, z, v, b, t, t, h, d, sliding_window_mask(t, 1));
        for (size_t i = 0; i < v.size(); i++) CHECK(std::fabs(diag[i] - v[i]) <= 1e-6f);
        bool threw = false;
        try { mha_forward_masked_f32(z, z, v, b, t, t, h, d, std::vector<float>(7)); }
        catch (const GQAError& e) { threw = e.which == "mask" && e.expected == t * t && e.got == 7; }
        CHECK(threw);
    }
    {   // KVCache: the reference's index table (kv_cache.rs:306-322) and errors (:326-348) on device buffers
        KVCache c(1, 1, 1, 2, 4, 4);
        std::vector<float> k1 = {1, 2}, v1 = {10, 20}, k2 = {3, 4}, v2 = {30, 40};
        c.append(0, 1, HipStorage::from_host(k1), HipStorage::from_host(v1));
        c.advance(1);
        c.append(0, 1, HipStorage::from_host(k2), HipStorage::from_host(v2));
        c.advance(1);
        synchronize();
        auto kb = c.k_buffer(0)->to_host<float>(), vb = c.v_buffer(0)->to_host<float>();
        CHECK(kb[0] == 1 && kb[1] == 2 && kb[2] == 3 && kb[3] == 4 && kb[4] == 0);
        CHECK(vb[0] == 10 && vb[1] == 20 && vb[2] == 30 && vb[3] == 40 && c.current_len() == 2);
        bool overflow = false, wrong = false, layer = false;
        std::vector<float> six(6, 0.0f), three(3, 0.0f);
        try { c.append(0, 3, HipStorage::from_host(six), HipStorage::from_host(six)); }
        catch (const KVCacheOverflow& e) { overflow = e.requested == 5 && e.max == 4; }
        try { c.append(0, 1, HipStorage::from_host(three), HipStorage::from_host(k1)); }
        catch (const KVCacheWrongInputLen& e) { wrong = e.expected == 2 && e.got_k == 3 && e.got_v == 2; }
        try { c.append(7, 1, HipStorage::from_host(k1), HipStorage::from_host(v1)); }
        catch (const KVCacheLayerOutOfRange& e) { layer = e.layer == 7 && e.num_layers == 1; }
        CHECK(overflow && wrong && layer && c.k_buffer(3) == nullptr);
    }
    {   // device buffers round-trip
        std::vector<float> h = lcg(1000, 9);
        HipStorage s = HipStorage::from_host(h);
        auto back = s.to_host<float>();
        CHECK(back == h);
    }
}

int main(int argc, char** argv) {
    const char* mode = argc > 1 ? argv[1] : "errors";
    try {
        if (!std::strcmp(mode, "errors")) test_errors();
        else if (!std::strcmp(mode, "gpu")) test_gpu();
        else {
            std::printf("usage: %s errors|gpu\n", argv[0]);
            return 2;
        }
    } catch (const std::exception& e) {
        std::printf("FAIL: unexpected exception: %s\n", e.what());
        return 1;
    }
    std::printf(g_failed ? "%d check(s) failed\n" : "ok\n", g_failed);
    return g_failed ? 1 : 0;
}
