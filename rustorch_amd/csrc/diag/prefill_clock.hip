// The bf16 prefill kernel, timed the way a serving loop runs it (back to back, for a second or more), with
// the shader clock it ran at: the first and the last workgroup read the shader-clock counter and the
// constant 100 MHz counter at their start and end.  Compiles the kernel source of the library itself with
// its phase hooks filled in; nothing else differs from the shipped kernel.
//
//   prefill_clock [seq = 4096] [batch = 4] [mask: 0 none | 1 causal = 1] [launches = 1000] [warm-up launches = 300]
//
// heads = 32, head dim = 128, (B, H, N, D) layout, one persistent workgroup per CU.
#include <hip/hip_runtime.h>
#include <cmath>
#include <cstdio>
#include <cstdlib>

__device__ long long* g_clk;
#define RT_PHASE_DECL const long long clk_c0 = clock64(), clk_w0 = wall_clock64();
#define RT_PHASE(id)
#define RT_PHASE_DUMP                                                                         \
    do {                                                                                      \
        if ((blockIdx.x == 0 || blockIdx.x == gridDim.x - 1) && threadIdx.x == 0) {           \
            long long* o_ = g_clk + (blockIdx.x == 0 ? 0 : 2);                                \
            o_[0] = clock64() - clk_c0;                                                       \
            o_[1] = wall_clock64() - clk_w0;                                                  \
        }                                                                                     \
    } while (0)
#include "../flash_bf16.hip"

#define CHECK(x)                                                                              \
    do {                                                                                      \
        hipError_t e_ = (x);                                                                  \
        if (e_ != hipSuccess) {                                                               \
            fprintf(stderr, "%s:%d: %s: %s\n", __FILE__, __LINE__, #x, hipGetErrorString(e_)); \
            return 1;                                                                         \
        }                                                                                     \
    } while (0)

__global__ void fill_normalish(uint16_t* p, size_t n, uint32_t seed) {
    size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x;
    for (; i < n; i += (size_t)gridDim.x * blockDim.x) {
        uint32_t x = (uint32_t)i * 2654435761u + seed;
        x ^= x >> 15; x *= 2246822519u; x ^= x >> 13;
        float f = ((x & 0xffff) / 65536.0f - 0.5f) * 3.4f;  // roughly unit variance
        p[i] = (uint16_t)(__float_as_uint(f) >> 16);
    }
}

int main(int argc, char** argv) {
    const int H = 32, D = 128;
    const int N = argc > 1 ? atoi(argv[1]) : 4096;
    const int B = argc > 2 ? atoi(argv[2]) : 4;
    const int mask = argc > 3 ? atoi(argv[3]) : 1;
    const int iters = argc > 4 ? atoi(argv[4]) : 1000;
    const int warm = argc > 5 ? atoi(argv[5]) : 300;
    if (N < 1 || N > (1 << 20) || B < 1 || (mask != 0 && mask != 1) || iters < 1 || warm < 0) {
        fprintf(stderr, "usage: prefill_clock [seq] [batch] [mask 0|1] [launches] [warm-up launches]\n");
        return 2;
    }
    hipDeviceProp_t prop;
    CHECK(hipGetDeviceProperties(&prop, 0));
    const size_t n = (size_t)B * H * N * D;
    uint16_t *q, *k, *v, *o;
    CHECK(hipMalloc(&q, n * 2));
    CHECK(hipMalloc(&k, n * 2));
    CHECK(hipMalloc(&v, n * 2));
    CHECK(hipMalloc(&o, n * 2));
    hipLaunchKernelGGL(fill_normalish, dim3(1024), dim3(256), 0, 0, q, n, 1u);
    hipLaunchKernelGGL(fill_normalish, dim3(1024), dim3(256), 0, 0, k, n, 2u);
    hipLaunchKernelGGL(fill_normalish, dim3(1024), dim3(256), 0, 0, v, n, 3u);
    CHECK(hipGetLastError());
    rt::FlashBf16Params p{};
    p.q = q; p.k = k; p.v = v; p.out = o;
    p.batch = B; p.heads = H; p.kv_heads = H; p.group = 1; p.seq = N; p.dim = D;
    p.mask = mask; p.ref_bc = 64;
    p.scale_log2e = 1.4426950408889634f / sqrtf((float)D);
    p.n_workers = prop.multiProcessorCount;
    p.lq = p.lkv = p.lo = rt::layout_bhnd(H, N, D);
    long long* clk;
    CHECK(hipMalloc(&clk, 4 * sizeof(long long)));
    CHECK(hipMemset(clk, 0, 4 * sizeof(long long)));
    CHECK(hipMemcpyToSymbol(HIP_SYMBOL(g_clk), &clk, sizeof(clk)));
    for (int i = 0; i < warm; i++) CHECK(rt::launch_flash_bf16(0, p));
    CHECK(hipDeviceSynchronize());
    hipEvent_t e0, e1;
    CHECK(hipEventCreate(&e0));
    CHECK(hipEventCreate(&e1));
    CHECK(hipEventRecord(e0));
    for (int i = 0; i < iters; i++) CHECK(rt::launch_flash_bf16(0, p));
    CHECK(hipEventRecord(e1));
    CHECK(hipEventSynchronize(e1));
    float ms;
    CHECK(hipEventElapsedTime(&ms, e0, e1));
    ms /= iters;
    long long h[4];
    CHECK(hipMemcpy(h, clk, sizeof(h), hipMemcpyDeviceToHost));
    const double fl = mask == 1 ? 4.0 * B * H * D * ((double)N * (N + 1) / 2) : 4.0 * B * H * D * (double)N * N;
    for (int b = 0; b < 2; b++)
        printf("%s workgroup of the last launch: %lld shader clocks in %.1f us -> %.0f MHz\n", b ? "last" : "first", h[2 * b],
               h[2 * b + 1] / 100.0, 100.0 * (double)h[2 * b] / (double)h[2 * b + 1]);
    printf("B=%d H=%d N=%d D=%d mask=%d: %.4f ms per launch over %d launches, %.1f TFLOP/s; at 2400 MHz the same clocks would be %.1f TFLOP/s\n",
           B, H, N, D, mask, ms, iters, fl / ms / 1e9, fl / ((double)h[0] / 2.4e9) / 1e12);
    return 0;
}
