// Measurement aid: what the matrix pipes of this device sustain when they do
// nothing but v_mfma_f32_32x32x16_f16 back to back (one wave per SIMD, four
// independent accumulators, eight operand pairs taking turns), and how much of
// that depends on the operand DATA.  The published F16 peak (2.5 PFLOP/s dense)
// is 256 CUs x 4 pipes x 1024 flop per clock at 2.4 GHz; the device holds that
// clock only while the instruction is cheap to execute.  With all-zero or
// all-one operands the loop runs at 2.4 GHz; with operands drawn from N(0, 1),
// which is what attention multiplies, the clock the device grants falls to
// 1.5-1.7 GHz for the same instruction stream.  The second figure, not the
// first, bounds a real MFMA-bound kernel on this device.
//
//   calib_mfma [MFMAs per wave in thousands, default 32]
//
// One line per operand kind: launch time (events around 5 launches, after 2
// untimed), the rate, and the shader clock = cycles the loop took (s_memtime)
// over its wall time (the 100 MHz counter).
#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <vector>

#define CK(x)                                                              \
    do {                                                                   \
        hipError_t e_ = (x);                                               \
        if (e_ != hipSuccess) {                                            \
            fprintf(stderr, "%s: %s\n", #x, hipGetErrorString(e_));        \
            return 1;                                                      \
        }                                                                  \
    } while (0)

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

constexpr int kThreads = 256;        // four waves: one per SIMD
constexpr int kPairs = 8;

__global__ __launch_bounds__(kThreads, 1) void mfma_only(const half8* __restrict__ src, float* __restrict__ out,
                                                          unsigned long long* __restrict__ clk, int iters)
{
    half8 a[kPairs], b[kPairs];
    for (int i = 0; i < kPairs; i++) {
        a[i] = src[(2 * i) * kThreads + threadIdx.x];
        b[i] = src[(2 * i + 1) * kThreads + threadIdx.x];
    }
    f32x16 acc[4];
    for (int j = 0; j < 4; j++)
        for (int r = 0; r < 16; r++) acc[j][r] = 0.f;
    const unsigned long long c0 = __builtin_readcyclecounter(), w0 = wall_clock64();
    for (int it = 0; it < iters; it++) {
#pragma unroll
        for (int u = 0; u < kPairs; u++)
            acc[u & 3] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a[u], b[u], acc[u & 3], 0, 0, 0);
    }
    const unsigned long long c1 = __builtin_readcyclecounter(), w1 = wall_clock64();
    float x = 0.f;
    for (int j = 0; j < 4; j++)
        for (int r = 0; r < 16; r++) x += acc[j][r];
    out[blockIdx.x * kThreads + threadIdx.x] = x;
    if (threadIdx.x == 0 && blockIdx.x == 0) {
        clk[0] = c1 - c0;
        clk[1] = w1 - w0;
    }
}

static float gauss()
{
    const float u1 = (float)((rand() + 1.0) / (RAND_MAX + 2.0)), u2 = (float)((rand() + 1.0) / (RAND_MAX + 2.0));
    return sqrtf(-2.f * logf(u1)) * cosf(6.2831853f * u2);
}

int main(int argc, char** argv)
{
    const long kilo = argc > 1 ? atol(argv[1]) : 32;
    if (kilo < 1 || kilo > 4096) {
        fprintf(stderr, "usage: calib_mfma [MFMAs per wave in thousands, 1..4096]\n");
        return 2;
    }
    const int iters = (int)(kilo * 1000 / kPairs);
    hipDeviceProp_t prop;
    CK(hipGetDeviceProperties(&prop, 0));
    const int cus = prop.multiProcessorCount;
    const size_t n = (size_t)2 * kPairs * kThreads * 8;
    std::vector<_Float16> h(n);
    _Float16* d;
    float* out;
    unsigned long long* clk;
    CK(hipMalloc(&d, n * sizeof(_Float16)));
    CK(hipMalloc(&out, (size_t)cus * kThreads * sizeof(float)));
    CK(hipMalloc(&clk, 2 * sizeof(unsigned long long)));
    hipEvent_t e0, e1;
    CK(hipEventCreate(&e0));
    CK(hipEventCreate(&e1));
    const char* names[3] = {"zeros", "ones", "normal"};
    srand(12345);
    for (int kind = 0; kind < 3; kind++) {
        for (size_t i = 0; i < n; i++)
            h[i] = kind == 0 ? (_Float16)0.f : kind == 1 ? (_Float16)1.f : (_Float16)gauss();
        CK(hipMemcpy(d, h.data(), n * sizeof(_Float16), hipMemcpyHostToDevice));
        const int reps = 5;
        for (int r = 0; r < 2; r++)
            hipLaunchKernelGGL(mfma_only, dim3(cus), dim3(kThreads), 0, 0, (const half8*)d, out, clk, iters);
        CK(hipDeviceSynchronize());
        CK(hipEventRecord(e0));
        for (int r = 0; r < reps; r++)
            hipLaunchKernelGGL(mfma_only, dim3(cus), dim3(kThreads), 0, 0, (const half8*)d, out, clk, iters);
        CK(hipEventRecord(e1));
        CK(hipEventSynchronize(e1));
        CK(hipGetLastError());
        float ms = 0.f;
        CK(hipEventElapsedTime(&ms, e0, e1));
        unsigned long long c[2];
        CK(hipMemcpy(c, clk, sizeof c, hipMemcpyDeviceToHost));
        const double us = ms * 1e3 / reps;
        const double flops = (double)cus * 4 * iters * kPairs * 2.0 * 32 * 32 * 16;
        printf("operands %-6s grid %4d  launch_us %9.1f  TFLOP/s %7.1f  GHz %5.3f\n", names[kind], cus, us,
               flops / us * 1e-6, c[1] ? (double)c[0] / ((double)c[1] * 10.0) : 0.0);
        fflush(stdout);
    }
    return 0;
}
