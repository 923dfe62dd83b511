// Measurement aid: what a kernel that ONLY reads can get out of HBM on this
// device, for the access patterns that matter to the decode kernel.  The decode
// kernel's roofline fraction is quoted against the published 8 TB/s; these
// figures say how much of the gap any reader of the same bytes would have.
//
//   calib_read [MiB per launch, default 256] [launches per pattern, default 24]
//
// Successive launches walk eight distinct windows, so nothing is served from
// the 256 MB last-level cache.  Patterns:
//   stride   grid-stride, 16 bytes per lane, UNROLL loads in flight per lane:
//            all waves read one narrow moving window (the friendliest pattern
//            for DRAM pages);
//   tiles    the decode kernel's: W workgroups of four waves, each workgroup
//            owns a run of 16 KiB tiles (8 KiB of "K" in one region, 8 KiB of
//            "V" in another, as the cache stores them), waves take tiles
//            round-robin with two tiles in flight each, 256 registers a wave
//            so that two workgroups share a compute unit (the decode kernel's
//            earlier form); and the same with one tile per wave and three
//            workgroups to a compute unit (its present form at head dim 128).
// Every figure is the average kernel time between the kernel's own start and
// stop events (hipExtLaunchKernelGGL), as the bench times the decode kernel.
#include <hip/hip_runtime.h>
#include <hip/hip_ext.h>

#include <cstdio>
#include <cstdlib>

typedef float f4 __attribute__((ext_vector_type(4)));

template <int UNROLL>
__global__ __launch_bounds__(256) void read_stride_kernel(const f4* __restrict__ p, size_t n16, float* sink)
{
    const size_t stride = (size_t)gridDim.x * 256;
    size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    f4 acc = {0, 0, 0, 0};
    for (; i + (UNROLL - 1) * stride < n16; i += UNROLL * stride) {
        f4 v[UNROLL];
#pragma unroll
        for (int u = 0; u < UNROLL; u++) v[u] = __builtin_nontemporal_load(&p[i + u * stride]);
#pragma unroll
        for (int u = 0; u < UNROLL; u++) acc += v[u];
    }
    if (acc[0] + acc[1] + acc[2] + acc[3] == 12345.678f) *sink = 1.f;     // keeps the loads
}

// tiles_per_wave tiles per wave, 4 * tiles_per_wave per workgroup; the
// workgroup's bytes are [K tiles][V tiles]
__global__ __launch_bounds__(256, 2) void read_tiles_kernel(const f4* __restrict__ base, int tiles_per_wave,
                                                            float* sink)
{
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int tiles = 4 * tiles_per_wave;
    const f4* wg = base + (size_t)blockIdx.x * tiles * 1024;
    f4 acc = {0, 0, 0, 0};
    f4 a[16], b[16];
    auto load = [&](f4 (&r)[16], int t) {
        const f4* k = wg + (size_t)t * 512;
        const f4* v = wg + (size_t)tiles * 512 + (size_t)t * 512;
#pragma unroll
        for (int i = 0; i < 8; i++) r[i] = __builtin_nontemporal_load(&k[i * 64 + lane]);
#pragma unroll
        for (int i = 0; i < 8; i++) r[8 + i] = __builtin_nontemporal_load(&v[i * 64 + lane]);
    };
    auto use = [&](f4 (&r)[16]) {
#pragma unroll
        for (int i = 0; i < 16; i++) acc += r[i];
    };
    int t = wave;
    load(a, t);
    load(b, t + 4);
#pragma unroll 1
    for (; t + 12 < tiles; t += 8) {
        use(a);
        load(a, t + 8);
        use(b);
        load(b, t + 12);
    }
    use(a);
    use(b);
    if (acc[0] + acc[1] + acc[2] + acc[3] == 12345.678f) *sink = 1.f;
}

// The same run of tiles with ONE tile per wave in registers, the next one asked
// for once the present one has been used, and three workgroups to a compute
// unit: what the decode kernel does at head dim 128.
__global__ __launch_bounds__(256, 3) void read_tiles1_kernel(const f4* __restrict__ base, int tiles_per_wave,
                                                             float* sink)
{
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int tiles = 4 * tiles_per_wave;
    const f4* wg = base + (size_t)blockIdx.x * tiles * 1024;
    f4 acc = {0, 0, 0, 0};
    f4 a[16];
    auto load_k = [&](int t) {
        const f4* k = wg + (size_t)t * 512;
#pragma unroll
        for (int i = 0; i < 8; i++) a[i] = __builtin_nontemporal_load(&k[i * 64 + lane]);
    };
    auto load_v = [&](int t) {
        const f4* v = wg + (size_t)tiles * 512 + (size_t)t * 512;
#pragma unroll
        for (int i = 0; i < 8; i++) a[8 + i] = __builtin_nontemporal_load(&v[i * 64 + lane]);
    };
    int t = wave;
    load_k(t);
    load_v(t);
#pragma unroll 1
    for (; t + 4 < tiles; t += 4) {
#pragma unroll
        for (int i = 0; i < 8; i++) acc += a[i];          // the K half is used, and refilled, first
        load_k(t + 4);
#pragma unroll
        for (int i = 8; i < 16; i++) acc += a[i];
        load_v(t + 4);
    }
#pragma unroll
    for (int i = 0; i < 16; i++) acc += a[i];
    if (acc[0] + acc[1] + acc[2] + acc[3] == 12345.678f) *sink = 1.f;
}

int main(int argc, char** argv)
{
    const size_t mib = argc > 1 ? strtoull(argv[1], nullptr, 10) : 256;
    const int reps = argc > 2 ? atoi(argv[2]) : 24;
    const size_t window = mib << 20;
    const int nwin = 8;
    char* buf = nullptr;
    float* sink = nullptr;
    if (hipMalloc(&buf, window * nwin) != hipSuccess || hipMalloc(&sink, 4) != hipSuccess) {
        fprintf(stderr, "calib_read: allocation failed\n");
        return 1;
    }
    (void)hipMemset(buf, 1, window * nwin);
    hipEvent_t e0, e1;
    hipStream_t st;
    (void)hipEventCreate(&e0);
    (void)hipEventCreate(&e1);
    (void)hipStreamCreate(&st);
    const size_t n16 = window / 16;

    auto report = [&](const char* name, int grid, double sum_ms, double best_ms, double bytes) {
        const double avg = sum_ms / reps;
        printf("%-40s grid %5d  avg %7.2f us  %6.0f GB/s (%.3f of 8 TB/s)   best %7.2f us\n", name, grid,
               avg * 1e3, bytes / (avg * 1e-3) / 1e9, bytes / (avg * 1e-3) / 8e12, best_ms * 1e3);
        fflush(stdout);
    };
#define TIMED(launch, name, grid, bytes)                                                   \
    do {                                                                                   \
        double sum = 0, best = 1e9;                                                        \
        for (int r = 0; r < reps + 4; r++) {                                               \
            const f4* p = reinterpret_cast<const f4*>(buf + (size_t)(r % nwin) * window);  \
            launch;                                                                        \
            if (hipStreamSynchronize(st) != hipSuccess) return 1;                          \
            float ms = 0;                                                                  \
            (void)hipEventElapsedTime(&ms, e0, e1);                                        \
            if (r >= 4) {                                                                  \
                sum += ms;                                                                 \
                if (ms < best) best = ms;                                                  \
            }                                                                              \
        }                                                                                  \
        report(name, grid, sum, best, bytes);                                              \
    } while (0)

    for (int grid : {256, 512, 2048})
        TIMED(hipExtLaunchKernelGGL(read_stride_kernel<8>, dim3(grid), dim3(256), 0, st, e0, e1, 0, p, n16, sink),
              "stride, 8 loads in flight per lane", grid, (double)window);
    for (int tpw : {16, 8, 4}) {
        const int grid = (int)(window / ((size_t)4 * tpw * 16384));
        char name[64];
        snprintf(name, sizeof name, "tiles, %d per workgroup (decode-like)", 4 * tpw);
        TIMED(hipExtLaunchKernelGGL(read_tiles_kernel, dim3(grid), dim3(256), 0, st, e0, e1, 0, p, tpw, sink),
              name, grid, (double)grid * 4 * tpw * 16384);
    }
    for (int tpw : {8, 4}) {
        const int grid = (int)(window / ((size_t)4 * tpw * 16384));
        char name[64];
        snprintf(name, sizeof name, "tiles, %d per workgroup, one in flight", 4 * tpw);
        TIMED(hipExtLaunchKernelGGL(read_tiles1_kernel, dim3(grid), dim3(256), 0, st, e0, e1, 0, p, tpw, sink),
              name, grid, (double)grid * 4 * tpw * 16384);
    }
    return 0;
}
