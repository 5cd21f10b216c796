// What the matrix cores of this GPU sustain, as opposed to their data-sheet peak: a loop of nothing but
// v_mfma_f32_32x32x16_bf16 on operands that change from instruction to instruction (N(0,1)-like bf16
// values, so the multipliers see realistic switching activity), launched back to back for seconds.
// Prints, per group of 100 launches, the rate and the shader clock the part settled at.  Under load the
// clock is governed by the power limit, and a kernel's fraction of the data-sheet peak (2.5 PFLOP/s at
// 2.4 GHz) is bounded by what this loop reaches.
//
//   mfma_sustained [workgroups per CU = 2] [groups of 100 launches = 20] [operands: random | constant = random]
//
// With `constant` every instruction multiplies the same two values in every lane (little switching in the
// multipliers): the comparison shows how much of the limit is power.
//
// Last line: "sustained <TFLOP/s> <MHz>" (median over the second half of the groups), for scripts.
#include <hip/hip_runtime.h>
#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <vector>

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef unsigned u32x4 __attribute__((ext_vector_type(4)));

#define CHECK(x)                                                                              \
    do {                                                                                      \
        hipError_t e_ = (x);                                                                  \
        if (e_ != hipSuccess) {                                                               \
            fprintf(stderr, "%s:%d: %s: %s\n", __FILE__, __LINE__, #x, hipGetErrorString(e_)); \
            return 1;                                                                         \
        }                                                                                     \
    } while (0)

__device__ inline unsigned mix(unsigned x) {
    x *= 2654435761u; x ^= x >> 15; x *= 2246822519u; x ^= x >> 13;
    return x;
}
// two bf16 values, roughly unit variance
__device__ inline unsigned bf16_pair(unsigned h) {
    float a = ((h & 0xffff) / 65536.0f - 0.5f) * 3.4f, b = ((h >> 16) / 65536.0f - 0.5f) * 3.4f;
    return (__float_as_uint(a) >> 16) | (__float_as_uint(b) & 0xffff0000u);
}

constexpr int kAcc = 4;          // independent accumulators per wave: no instruction waits for the one before
constexpr int kPerIter = 8 * kAcc;

__global__ __launch_bounds__(256) void mfma_loop(float* out, long long* clk, int iters, int constant) {
    const long long c0 = clock64(), w0 = wall_clock64();
    f32x16 acc[kAcc];
    for (int a = 0; a < kAcc; a++)
        for (int i = 0; i < 16; i++) acc[a][i] = 0.0f;
    bf16x8 av[8], bv[8];
    for (int r = 0; r < 8; r++) {
        u32x4 x, y;
        for (int i = 0; i < 4; i++) {
            x[i] = constant ? 0x3f003f00u : bf16_pair(mix(threadIdx.x * 64 + r * 8 + i));
            y[i] = constant ? 0x3e803e80u : bf16_pair(mix(threadIdx.x * 64 + r * 8 + i + 4 + blockIdx.x * 77777));
        }
        av[r] = __builtin_bit_cast(bf16x8, x);
        bv[r] = __builtin_bit_cast(bf16x8, y);
    }
    for (int it = 0; it < iters; it++) {
#pragma unroll
        for (int r = 0; r < 8; r++)
#pragma unroll
            for (int a = 0; a < kAcc; a++)
                acc[a] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(av[(r + a) & 7], bv[r], acc[a], 0, 0, 0);
    }
    float s = 0.0f;
    for (int a = 0; a < kAcc; a++)
        for (int i = 0; i < 16; i++) s += acc[a][i];
    out[blockIdx.x * 256 + threadIdx.x] = s;
    if (blockIdx.x == 0 && threadIdx.x == 0) {
        clk[0] = clock64() - c0;        // shader clocks
        clk[1] = wall_clock64() - w0;   // ticks of the constant 100 MHz counter
    }
}

int main(int argc, char** argv) {
    const int wg_per_cu = argc > 1 ? atoi(argv[1]) : 2;
    const int groups = argc > 2 ? atoi(argv[2]) : 20;
    const bool constant = argc > 3 && argv[3][0] == 'c';
    if (wg_per_cu < 1 || wg_per_cu > 2 || groups < 2 || groups > 200) {
        fprintf(stderr, "usage: mfma_sustained [workgroups per CU: 1|2] [groups of 100 launches: 2..200] [random|constant]\n");
        return 2;
    }
    hipDeviceProp_t prop;
    CHECK(hipGetDeviceProperties(&prop, 0));
    const int cus = prop.multiProcessorCount;
    float* d;
    long long* c;
    CHECK(hipMalloc(&d, (size_t)cus * wg_per_cu * 256 * sizeof(float)));
    CHECK(hipMalloc(&c, 2 * sizeof(long long)));
    const int iters = 400;
    hipEvent_t e0, e1;
    CHECK(hipEventCreate(&e0));
    CHECK(hipEventCreate(&e1));
    std::vector<double> tf, mhz;
    for (int g = 0; g < groups; g++) {
        CHECK(hipEventRecord(e0));
        for (int i = 0; i < 100; i++) hipLaunchKernelGGL(mfma_loop, dim3(cus * wg_per_cu), dim3(256), 0, 0, d, c, iters, constant ? 1 : 0);
        CHECK(hipGetLastError());
        CHECK(hipEventRecord(e1));
        CHECK(hipEventSynchronize(e1));
        float ms;
        CHECK(hipEventElapsedTime(&ms, e0, e1));
        long long h[2];
        CHECK(hipMemcpy(h, c, sizeof(h), hipMemcpyDeviceToHost));
        const double flops = 100.0 * cus * wg_per_cu * 4 * (double)iters * kPerIter * 32768.0;  // 2*32*32*16 per instruction
        tf.push_back(flops / (ms * 1e-3) / 1e12);
        mhz.push_back(100.0 * (double)h[0] / (double)h[1]);
        printf("launches %4d-%4d: %.3f ms each  %7.1f TFLOP/s  shader clock %4.0f MHz\n", 100 * g, 100 * g + 99, ms / 100,
               tf.back(), mhz.back());
    }
    std::vector<double> t2(tf.begin() + groups / 2, tf.end()), m2(mhz.begin() + groups / 2, mhz.end());
    std::sort(t2.begin(), t2.end());
    std::sort(m2.begin(), m2.end());
    printf("sustained %.1f %.0f\n", t2[t2.size() / 2], m2[m2.size() / 2]);
    return 0;
}
