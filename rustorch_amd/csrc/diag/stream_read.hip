// What the memory system delivers to a kernel that only reads: one-wave workgroups, eight 16-byte loads per lane
// and matrix in flight, every byte read once.  Two address patterns:
//
//   contiguous   one 1.25 GiB array cut into equal spans
//   cache        the decode workload's: two arrays (K and V) of 512 segments of 2 MiB (64 sequences x 8 kv heads x
//                8192 rows x 256 B), a prefix of U[512, 8192] rows of each segment read, the flat list of 8 KiB +
//                8 KiB steps cut into equal spans; three sets rotated so that no launch finds its rows in the
//                last-level cache
//
//   stream_read [contiguous|cache = cache] [workgroups = 1024] [launches = 60]
//
// Prints the rate with plain loads and with non-temporal loads.  The decode kernel's fraction of the 8 TB/s data
// sheet figure is bounded by what this program reaches on the cache pattern.
#include <hip/hip_runtime.h>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <random>
#include <vector>

typedef unsigned u32x4 __attribute__((ext_vector_type(4)));

#define CHECK(x)                                                                              \
    do {                                                                                      \
        hipError_t e_ = (x);                                                                  \
        if (e_ != hipSuccess) {                                                               \
            fprintf(stderr, "%s:%d: %s: %s\n", __FILE__, __LINE__, #x, hipGetErrorString(e_)); \
            return 1;                                                                         \
        }                                                                                     \
    } while (0)

// step t of the flat list lies in segment seg (seg_start[seg] <= t < seg_start[seg + 1]), at 8 KiB * (t - seg_start[seg])
template <bool NT>
__global__ __launch_bounds__(64) void read_steps(const u32x4* __restrict__ k, const u32x4* __restrict__ v,
                                                 const int* __restrict__ seg_start, int n_seg, size_t seg_vecs, int total,
                                                 unsigned* out) {
    const int span = (total + (int)gridDim.x - 1) / (int)gridDim.x;
    const int first = (int)blockIdx.x * span, last = min(total, first + span);
    if (first >= last) return;
    int seg = 0;
    while (seg + 1 < n_seg && seg_start[seg + 1] <= first) seg++;
    unsigned acc = 0;
    for (int t = first; t < last; t++) {
        while (seg + 1 < n_seg && seg_start[seg + 1] <= t) seg++;
        const size_t off = (size_t)seg * seg_vecs + (size_t)(t - seg_start[seg]) * 512 + threadIdx.x;
        u32x4 a[8], b[8];
#pragma unroll
        for (int u = 0; u < 8; u++) {
            if (NT) {
                a[u] = __builtin_nontemporal_load(k + off + u * 64);
                b[u] = __builtin_nontemporal_load(v + off + u * 64);
            } else {
                a[u] = k[off + u * 64];
                b[u] = v[off + u * 64];
            }
        }
#pragma unroll
        for (int u = 0; u < 8; u++) acc += a[u][0] ^ a[u][3] ^ b[u][1] ^ b[u][2];
    }
    if (acc == 0x12345678u) out[0] = acc;  // keeps the loads alive
}

int main(int argc, char** argv) {
    const bool contiguous = argc > 1 && !strcmp(argv[1], "contiguous");
    const int waves = argc > 2 ? atoi(argv[2]) : 1024;
    const int iters = argc > 3 ? atoi(argv[3]) : 60;
    if (waves < 1 || waves > 65535 || iters < 1) {
        fprintf(stderr, "usage: stream_read [contiguous|cache] [workgroups] [launches]\n");
        return 2;
    }
    const int sets = 3;
    int n_seg;
    size_t seg_bytes;
    std::vector<int> start;
    int total = 0;
    if (contiguous) {  // one segment per matrix, all of it read: 2 x 640 MiB
        n_seg = 1;
        seg_bytes = (size_t)640 << 20;
        total = (int)(seg_bytes / 8192);
        start = {0, total};
    } else {
        n_seg = 512;
        seg_bytes = (size_t)2 << 20;
        start.resize(n_seg + 1);
        std::mt19937 rng(4);
        for (int b = 0; b < 64; b++) {
            const int len = 512 + (int)(rng() % (8192 - 512 + 1));
            for (int h = 0; h < 8; h++) {
                start[b * 8 + h] = total;
                total += (len + 31) / 32;
            }
        }
        start[n_seg] = total;
    }
    const size_t arr = (size_t)n_seg * seg_bytes;
    std::vector<u32x4*> ks(sets), vs(sets);
    for (int s = 0; s < sets; s++) {
        CHECK(hipMalloc(&ks[s], arr));
        CHECK(hipMalloc(&vs[s], arr));
        CHECK(hipMemset(ks[s], 1, arr));
        CHECK(hipMemset(vs[s], 2, arr));
    }
    int* ds;
    CHECK(hipMalloc(&ds, (n_seg + 1) * sizeof(int)));
    CHECK(hipMemcpy(ds, start.data(), (n_seg + 1) * sizeof(int), hipMemcpyHostToDevice));
    unsigned* out;
    CHECK(hipMalloc(&out, 4));
    hipEvent_t e0, e1;
    CHECK(hipEventCreate(&e0));
    CHECK(hipEventCreate(&e1));
    for (int nt = 0; nt < 2; nt++) {
        auto launch = [&](int i) {
            if (nt)
                hipLaunchKernelGGL(read_steps<true>, dim3(waves), dim3(64), 0, 0, ks[i % sets], vs[i % sets], ds, n_seg,
                                   seg_bytes / 16, total, out);
            else
                hipLaunchKernelGGL(read_steps<false>, dim3(waves), dim3(64), 0, 0, ks[i % sets], vs[i % sets], ds, n_seg,
                                   seg_bytes / 16, total, out);
        };
        for (int i = 0; i < 5; i++) launch(i);
        CHECK(hipGetLastError());
        CHECK(hipEventRecord(e0));
        for (int i = 0; i < iters; i++) launch(i);
        CHECK(hipEventRecord(e1));
        CHECK(hipEventSynchronize(e1));
        float ms;
        CHECK(hipEventElapsedTime(&ms, e0, e1));
        ms /= iters;
        const double bytes = (double)total * 16384.0;
        printf("%s pattern, %d workgroups, %s loads: %.3e bytes in %.1f us = %.0f GB/s\n", contiguous ? "contiguous" : "cache",
               waves, nt ? "non-temporal" : "plain", bytes, ms * 1e3, bytes / (ms * 1e-3) / 1e9);
    }
    return 0;
}
