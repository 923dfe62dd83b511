// Measurement aid: a plain device-to-device copy of a known size, used to
// calibrate the rocprofv3 FETCH_SIZE / WRITE_SIZE counters (what the counter
// reads for N bytes known to be fetched / written) before they are applied to
// the attention kernels.
//
//   calib_copy [MiB per launch, default 256] [launches, default 10]
//
// Each launch reads MiB and writes MiB (16 bytes per lane, grid-stride).
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstdlib>

typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

__global__ __launch_bounds__(256) void calib_copy_kernel(const u32x4* __restrict__ src,
                                                         u32x4* __restrict__ dst, size_t n_vec)
{
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n_vec; i += stride)
        dst[i] = src[i];
}

int main(int argc, char** argv)
{
    const size_t mib = argc > 1 ? strtoull(argv[1], nullptr, 10) : 256;
    const int launches = argc > 2 ? atoi(argv[2]) : 10;
    const size_t bytes = mib << 20;
    void *src = nullptr, *dst = nullptr;
    if (hipMalloc(&src, bytes) != hipSuccess || hipMalloc(&dst, bytes) != hipSuccess) {
        fprintf(stderr, "calib_copy: allocation failed\n");
        return 1;
    }
    (void)hipMemset(src, 1, bytes);
    (void)hipMemset(dst, 0, bytes);
    hipEvent_t e0, e1;
    (void)hipEventCreate(&e0);
    (void)hipEventCreate(&e1);
    (void)hipEventRecord(e0, 0);
    for (int i = 0; i < launches; i++)
        hipLaunchKernelGGL(calib_copy_kernel, dim3(2048), dim3(256), 0, 0, (const u32x4*)src,
                           (u32x4*)dst, bytes / 16);
    (void)hipEventRecord(e1, 0);
    if (hipEventSynchronize(e1) != hipSuccess) {
        fprintf(stderr, "calib_copy: launch failed\n");
        return 1;
    }
    float ms = 0.f;
    (void)hipEventElapsedTime(&ms, e0, e1);
    printf("calib_copy: %d launches, each reads %zu and writes %zu bytes; %.1f us per launch, "
           "%.0f GB/s read+write\n", launches, bytes, bytes, ms * 1e3 / launches,
           2.0 * bytes * launches / (ms * 1e-3) / 1e9);
    (void)hipFree(src);
    (void)hipFree(dst);
    return 0;
}
