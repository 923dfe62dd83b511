// Measurement aid: what ONE launch costs inside a chain of dependent launches
// on one stream, which is what a decode step of the device walk is (about 140
// launches that each wait for the one before).  Every kernel here does what a
// one-row projection must do at the least -- read the row its predecessor
// wrote, reduce it across the workgroup, write 16 outputs -- and nothing else,
// so the figures are a floor for such a launch, not a model of it.
//
//   calib_chain [launches per chain, default 400]
//
// Lines:
//   empty                     a kernel with no instructions: the dispatch itself;
//   constant row              every workgroup reads a 16 KiB row that nobody
//                             writes (it stays in the caches), reduces, stores;
//   predecessor's row         the row is the output of the launch before (two
//                             buffers take turns): same instructions, but the
//                             lines were written a moment ago by workgroups on
//                             other XCDs; with 4 KiB / 16 KiB rows and 64 / 256
//                             workgroups (the cost follows rows x workgroups);
//   ... + 8 MiB of weights    plus a stream of 8 MiB, shared out over the
//                             workgroups, asked for before the row is read.
// Time per launch = elapsed time between two events around the whole chain,
// divided by its length; the best of five chains.
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstdlib>

#define CK(x)                                                              \
    do {                                                                   \
        hipError_t e_ = (x);                                               \
        if (e_ != hipSuccess) {                                            \
            fprintf(stderr, "%s: %s\n", #x, hipGetErrorString(e_));        \
            return 1;                                                      \
        }                                                                  \
    } while (0)

__global__ __launch_bounds__(256) void chain_empty(const float*, float*) {}

// W16 = 16-byte units of "weights" per workgroup (0 = none)
__global__ __launch_bounds__(256) void chain_row(const float* __restrict__ in, float* __restrict__ out, int n,
                                                 const float4* __restrict__ w, int w16)
{
    float4 acc = {0.f, 0.f, 0.f, 0.f};
    const float4* wp = w + (size_t)blockIdx.x * w16;
    for (int i = threadIdx.x; i < w16; i += 256) {
        const float4 v = wp[i];
        acc.x += v.x;
        acc.y += v.y;
        acc.z += v.z;
        acc.w += v.w;
    }
    float s = 0.f;
    for (int i = threadIdx.x; i < n; i += 256) s += in[i];
    s += (acc.x + acc.y + acc.z + acc.w) * 1e-30f;
    for (int off = 32; off; off >>= 1) s += __shfl_xor(s, off);
    __shared__ float s4[4];
    if ((threadIdx.x & 63) == 0) s4[threadIdx.x >> 6] = s;
    __syncthreads();
    s = (s4[0] + s4[1]) + (s4[2] + s4[3]);
    if (threadIdx.x < 16) {
        const int o = blockIdx.x * 16 + threadIdx.x;
        if (o < n) out[o] = s * 1e-3f + 1.0f;
    }
}

int main(int argc, char** argv)
{
    const int reps = argc > 1 ? atoi(argv[1]) : 400;
    if (reps < 1 || reps > 100000) {
        fprintf(stderr, "usage: calib_chain [launches per chain, 1..100000]\n");
        return 2;
    }
    const int nmax = 4096;
    float *a, *b, *cst;
    float4* w;
    const size_t wbytes = 8u << 20;
    CK(hipMalloc(&a, nmax * 4));
    CK(hipMalloc(&b, nmax * 4));
    CK(hipMalloc(&cst, nmax * 4));
    CK(hipMalloc(&w, wbytes));
    CK(hipMemset(a, 0, nmax * 4));
    CK(hipMemset(b, 0, nmax * 4));
    CK(hipMemset(cst, 0, nmax * 4));
    CK(hipMemset(w, 0, wbytes));
    hipStream_t st;
    CK(hipStreamCreate(&st));
    hipEvent_t e0, e1;
    CK(hipEventCreate(&e0));
    CK(hipEventCreate(&e1));

    struct Case {
        const char* name;
        int grid, n, fresh, weights;      // n = 0: the empty kernel
    };
    const Case cases[] = {
        {"empty", 256, 0, 0, 0},
        {"constant row, 16 KiB", 256, 4096, 0, 0},
        {"predecessor's row, 4 KiB", 64, 1024, 1, 0},
        {"predecessor's row, 4 KiB", 256, 1024, 1, 0},
        {"predecessor's row, 16 KiB", 64, 4096, 1, 0},
        {"predecessor's row, 16 KiB", 256, 4096, 1, 0},
        {"predecessor's row, 4 KiB + 8 MiB of weights", 256, 1024, 1, 1},
        {"predecessor's row, 16 KiB + 8 MiB of weights", 256, 4096, 1, 1},
    };
    for (const Case& c : cases) {
        float best = 1e30f;
        for (int rep = 0; rep < 5; rep++) {
            CK(hipEventRecord(e0, st));
            for (int i = 0; i < reps; i++) {
                const float* in = c.fresh ? ((i & 1) ? b : a) : cst;
                float* out = (i & 1) ? a : b;
                if (c.n == 0)
                    hipLaunchKernelGGL(chain_empty, dim3(c.grid), dim3(256), 0, st, in, out);
                else
                    hipLaunchKernelGGL(chain_row, dim3(c.grid), dim3(256), 0, st, in, out, c.n, w,
                                       c.weights ? (int)(wbytes / 16 / c.grid) : 0);
            }
            CK(hipGetLastError());
            CK(hipEventRecord(e1, st));
            CK(hipEventSynchronize(e1));
            float ms = 0.f;
            CK(hipEventElapsedTime(&ms, e0, e1));
            if (ms < best) best = ms;
        }
        printf("%-46s grid %4d  us per launch %6.2f\n", c.name, c.grid, best * 1000.f / reps);
    }
    return 0;
}
