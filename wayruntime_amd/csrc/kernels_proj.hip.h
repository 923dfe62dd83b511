// Row projections  Y[R][N] = X[R][K] . W[N][K]^T  with F16 weights and F32
// activations: the Q/K/V/output projections either side of the attention
// path (reference: wri_op_matmul at src/core/session.c:446-457 and :499-506,
// inner loops src/core/kernels.c:124-137; weights are W[out][in] with `in`
// contiguous, src/core/internal.h:113-118, and F16 tensors are widened to F32
// before the multiply, src/core/loader.c:164-190).
//
// Decode sends 1..16 rows through a projection, so the work is reading W once:
// HBM-bound, algorithmic bytes per launch = 2 * N * K.  The multiply-adds run
// on v_mfma_f32_16x16x32_f16 to keep them off the vector ALUs, as in the decode
// kernel, and F32 accuracy is kept the same way: each row is scaled by a power
// of two into [1, 2) (by its largest magnitude), split into two half-precision
// terms x = hi + lo * 2^-11, and the two terms take two COLUMNS of the same MFMA
// (column c = hi of row c, column c + 8 = lo of row c, eight rows per MFMA).
// The columns are combined and the scale undone at the end; sums are F32.
//
// Layouts on the device (both private to the library):
//
//   W   [N/16][K/32][64][8] halves: tile (nt, kt) is the MFMA A operand of
//       outputs 16nt..16nt+15 and inputs 32kt..32kt+31 in lane order (lane =
//       16g + m holds W[16nt + m][32kt + 8g .. +8]), one contiguous KiB per
//       operand load; a wave streams the K/32 consecutive KiBs of its outputs.
//   X   fragments [ceil(R/8)][K/32][64][8] halves, the matching B operands
//       (lane 16g + c: column c, inputs 32kt + 8g .. +8), and one F32 scale
//       per row, written by proj_prep_kernel, read by every wave (L2 / L1 hits).
//
// Kernels, by row count of a launch:
//   1 row        proj_row1_kernel: the fragment step inside the product;
//   2 .. 63      proj_prep_kernel, then proj_rows_kernel (a wave owns one to four
//                16-output tiles for one to four row groups; HBM-bound);
//   64 .. 4096   proj_prep_group_kernel, then an MFMA-bound GEMM:
//                proj_gemm_lds_kernel (operands staged through LDS) where its
//                tiles fill the chip, proj_gemm_split_kernel below that.
// N must be a multiple of 16 and K a multiple of 32.
#pragma once

#include "common.hip.h"

namespace wr {

constexpr int kProjThreads = 256;
constexpr int kProjMaxRows = 4096;                // rows per launch (512 row groups)
constexpr int kProjKBatch = 8;                    // k-steps (KiBs of W) a wave keeps in flight per buffer

// Row-major F16 W[N][K] -> tile order.  One thread per 16-byte unit.
__global__ __launch_bounds__(256) void proj_pack_weights_kernel(const uint16_t* __restrict__ w,
                                                                u32x4* __restrict__ tiles,
                                                                uint32_t N, uint32_t K)
{
    const size_t unit = (size_t)blockIdx.x * blockDim.x + threadIdx.x;     // destination unit
    const size_t total = (size_t)N * K / 8;
    if (unit >= total) return;
    const uint32_t lane = (uint32_t)(unit & 63);
    const size_t tile = unit >> 6;
    const uint32_t kt = (uint32_t)(tile % (K / 32));
    const uint32_t nt = (uint32_t)(tile / (K / 32));
    const uint32_t m = lane & 15, g = lane >> 4;
    const u32x4* src = reinterpret_cast<const u32x4*>(w + ((size_t)(nt * 16 + m) * K + kt * 32 + g * 8));
    tiles[unit] = *src;
}

// X rows -> B-operand fragments and per-row scales, one workgroup per row
// (rows past R, which pad the last group of eight, get zero fragments).
//
// The row is first brought to its final F32 values v[k] by one of three
// sources, so that a normalisation or activation that only feeds a projection
// never has to be written out:
//   kProjSrcPlain    v = x
//   kProjSrcRmsNorm  v = x * (1 / sqrt(mean x^2 + eps)) * w     (RMSNorm,
//                    src/core/kernels.c:1276-1316, same expressions and the
//                    same reduction tree as rmsnorm_rows_kernel)
//   kProjSrcSwiglu   v = silu(g) * u, g = x[k], u = x[K + k]   (kernels.c:963-967)
//   kProjSrcGeglu    v = gelu_tanh(g) * u, same operands      (kernels.c:969-976)
// Then scales[row] = 2^e with 2^e <= max|v| < 2^(e+1) (1 for a row of zeros),
// v is divided by it (exact), so its largest magnitude lies in [1, 2), and
// split into
//   hi = binary16(v), flushed to zero below the normal range, and
//   lo = binary16((v - hi) * 2^11),
// i.e. v = hi + lo * 2^-11 to about 2^-22 |v| (2^-25 of the row's largest value
// for elements so small that hi is flushed).  Keeping lo scaled up keeps both
// terms in the normal binary16 range, so the result does not depend on how the
// matrix cores treat subnormal inputs.
constexpr float kProjLoScale = 2048.0f;
constexpr int kProjSrcPlain = 0, kProjSrcRmsNorm = 1, kProjSrcSwiglu = 2, kProjSrcGeglu = 3;

struct ProjPrepArgs {
    const float* x;          // [R][ldx]
    const float* norm_w;     // kProjSrcRmsNorm: [K]
    half8* frag;             // [groups][K/32][64]
    float* scales;           // [R]
    uint32_t ldx, R, K;
    float eps;
};

// (The barriers in these two wait for LDS traffic only: __syncthreads() would
// also wait for every global load in flight, and the one-row product has its
// weights on the way while it reduces.)
// s4 must not be written again before the workgroup's next barrier (the two
// reductions of a row use the two halves of an array of eight): one barrier
// each, not two.
__device__ __forceinline__ float block_sum_256(float v, float* s4)
{
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) v += wave_xor_f32(v, off);
    if ((threadIdx.x & 63) == 0) s4[threadIdx.x >> 6] = v;
    lds_barrier();
    return (s4[0] + s4[1]) + (s4[2] + s4[3]);
}

__device__ __forceinline__ float block_max_256(float v, float* s4)
{
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) v = fmaxf(v, wave_xor_f32(v, off));
    if ((threadIdx.x & 63) == 0) s4[threadIdx.x >> 6] = v;
    lds_barrier();
    return fmaxf(fmaxf(s4[0], s4[1]), fmaxf(s4[2], s4[3]));
}

// Sum of squares of a row by a 256-thread workgroup.  Thread t takes the
// chunks of eight values t, t + 256, ... in order; the partial sums go through
// a wave tree and the four waves are added pairwise.  Every kernel that
// normalises a row uses this order, so a norm computed inside the fragment
// kernel has the bits of rmsnorm_rows_kernel.
__device__ __forceinline__ float row_sumsq_256(const float* __restrict__ xr, uint32_t K, float* s4)
{
    float ss = 0.f;
    for (uint32_t k0 = threadIdx.x * 8; k0 < K; k0 += 2048) {
#pragma unroll
        for (int j = 0; j < 8; j++) {
            const float v = (k0 + j < K) ? xr[k0 + j] : 0.f;
            ss = fmaf(v, v, ss);          // explicit, so every copy of this sum rounds alike
        }
    }
    return block_sum_256(ss, s4);
}

// the two gated activations: SiLU(g) * u and the tanh form of GELU(g) * u
template <int SRC>
__device__ __forceinline__ float proj_gated(float g, float u)
{
    if constexpr (SRC == kProjSrcGeglu) {
        const float x3 = g * g * g;
        const float z = 0.7978845608f * (g + 0.044715f * x3);
        const float th = 2.0f / (1.0f + expf(-2.0f * z)) - 1.0f;
        return 0.5f * g * (1.0f + th) * u;
    } else {
        return silu_mul(g, u);
    }
}

template <int SRC>
__device__ __forceinline__ float proj_src_value(const ProjPrepArgs& a, const float* xr, uint32_t k,
                                                float inv_rms)
{
    if constexpr (SRC == kProjSrcRmsNorm) {
        return xr[k] * inv_rms * a.norm_w[k];
    } else if constexpr (SRC == kProjSrcSwiglu || SRC == kProjSrcGeglu) {
        return proj_gated<SRC>(xr[k], xr[a.K + k]);
    } else {
        return xr[k];
    }
}

__device__ __forceinline__ void proj_write_chunk(half8* frow, uint32_t q, uint32_t c,
                                                 const float (&v)[8], float inv)
{
    half8 hi, lo;
#pragma unroll
    for (int j = 0; j < 8; j++) {
        const float s = v[j] * inv;
        _Float16 h = (_Float16)s;
        if (fabsf((float)h) < 6.103515625e-05f) h = (_Float16)0.0f;      // 2^-14
        hi[j] = h;
        lo[j] = (_Float16)((s - (float)h) * kProjLoScale);
    }
    const uint32_t kt = q >> 2, g = q & 3;
    frow[(size_t)kt * 64 + 16 * g + c] = hi;
    frow[(size_t)kt * 64 + 16 * g + c + 8] = lo;
}

// CH > 0: K <= 2048 * CH and the row's values are held in registers between
// the passes (one read of the row: a single-row call is pure latency, and each
// pass over global memory is a round trip).  CH = 0: any K, the passes re-read
// (and re-compute) the row.
template <int SRC, int CH>
__global__ __launch_bounds__(256) void proj_prep_kernel(const ProjPrepArgs a)
{
    __shared__ float s4[8];
    const uint32_t row = blockIdx.x, t = threadIdx.x;
    const uint32_t ktiles = a.K / 32, nchunks = a.K / 8;
    const uint32_t grp = row / 8, c = row % 8;
    half8* frow = a.frag + (size_t)grp * ktiles * 64;
    if (row >= a.R) {                                     // padding row of the last group
        half8 z;
#pragma unroll
        for (int j = 0; j < 8; j++) z[j] = (_Float16)0.0f;
        for (uint32_t q = t; q < nchunks; q += 256) {
            const uint32_t kt = q >> 2, g = q & 3;
            frow[(size_t)kt * 64 + 16 * g + c] = z;
            frow[(size_t)kt * 64 + 16 * g + c + 8] = z;
        }
        return;
    }
    const float* xr = a.x + (size_t)row * a.ldx;

    if constexpr (CH > 0) {
        float v[CH][8];
        float ss = 0.f;
#pragma unroll
        for (int i = 0; i < CH; i++) {
            const uint32_t q = t + 256 * i;
#pragma unroll
            for (int j = 0; j < 8; j++) v[i][j] = (q < nchunks) ? xr[q * 8 + j] : 0.f;
            if constexpr (SRC == kProjSrcRmsNorm) {
#pragma unroll
                for (int j = 0; j < 8; j++) ss = fmaf(v[i][j], v[i][j], ss);
            }
        }
        float mx = 0.f;
        if constexpr (SRC == kProjSrcRmsNorm) {
            const float inv_rms = 1.0f / sqrtf(block_sum_256(ss, s4) / (float)a.K + a.eps);
#pragma unroll
            for (int i = 0; i < CH; i++) {
                const uint32_t q = t + 256 * i;
#pragma unroll
                for (int j = 0; j < 8; j++)
                    v[i][j] = (q < nchunks) ? v[i][j] * inv_rms * a.norm_w[q * 8 + j] : 0.f;
            }
        } else if constexpr (SRC == kProjSrcSwiglu || SRC == kProjSrcGeglu) {
#pragma unroll
            for (int i = 0; i < CH; i++) {
                const uint32_t q = t + 256 * i;
#pragma unroll
                for (int j = 0; j < 8; j++) {
                    const float u = (q < nchunks) ? xr[a.K + q * 8 + j] : 0.f;
                    v[i][j] = proj_gated<SRC>(v[i][j], u);
                }
            }
        }
#pragma unroll
        for (int i = 0; i < CH; i++)
#pragma unroll
            for (int j = 0; j < 8; j++) mx = fmaxf(mx, fabsf(v[i][j]));
        mx = block_max_256(mx, s4 + 4);
        uint32_t ex = (__float_as_uint(mx) >> 23) & 0xFFu;
        if (ex == 0 || ex == 0xFF) ex = 127;              // zeros, subnormals, inf / NaN rows: no scaling
        if (ex > 253) ex = 253;                           // keeps the inverse 2^-e a normal number
        if (t == 0) a.scales[row] = __uint_as_float(ex << 23);
        const float inv = __uint_as_float((254u - ex) << 23);
#pragma unroll
        for (int i = 0; i < CH; i++) {
            const uint32_t q = t + 256 * i;
            if (q < nchunks) proj_write_chunk(frow, q, c, v[i], inv);
        }
    } else {
        float inv_rms = 1.0f;
        if constexpr (SRC == kProjSrcRmsNorm)
            inv_rms = 1.0f / sqrtf(row_sumsq_256(xr, a.K, s4) / (float)a.K + a.eps);
        float mx = 0.f;
        for (uint32_t k = t; k < a.K; k += 256) mx = fmaxf(mx, fabsf(proj_src_value<SRC>(a, xr, k, inv_rms)));
        mx = block_max_256(mx, s4 + 4);
        uint32_t ex = (__float_as_uint(mx) >> 23) & 0xFFu;
        if (ex == 0 || ex == 0xFF) ex = 127;
        if (ex > 253) ex = 253;
        if (t == 0) a.scales[row] = __uint_as_float(ex << 23);
        const float inv = __uint_as_float((254u - ex) << 23);
        for (uint32_t q = t; q < nchunks; q += 256) {     // 8 consecutive inputs per thread
            float v[8];
#pragma unroll
            for (int j = 0; j < 8; j++) v[j] = proj_src_value<SRC>(a, xr, q * 8 + j, inv_rms);
            proj_write_chunk(frow, q, c, v, inv);
        }
    }
}

// The fragment kernel for many rows: one workgroup per row GROUP of eight.
// Thread t serves row t % 8 of the group and the chunks of eight inputs t / 8,
// t / 8 + 32, ...: a wave reads 256 contiguous bytes of each of its eight rows
// per step and writes the hi and lo terms of eight chunks as whole 128-byte
// lines (the eight rows' 16-byte units of one chunk are neighbours in the
// fragment), where the one-row kernel's writes touch 16 bytes of a line each.
// Same sources, expressions and scaling as proj_prep_kernel; the row sums are
// formed in a different order (each thread over its own chunks, then the 32
// threads of the row), so a normalised row agrees with the one-row kernel's to
// rounding, not bit for bit: only launches of 64 rows and more come here.
//
// CH > 0: K <= 256 * CH and the row group's values stay in registers between
// the passes; CH = 0: any K, the passes re-read and re-compute.
__device__ __forceinline__ float group_rows_sum(float v, float (*s)[8], int lane, int wave, int c)
{
    v += wave_xor_f32(v, 8);
    v += wave_xor_f32(v, 16);
    v += wave_xor_f32(v, 32);
    if (lane < 8) s[wave][lane] = v;
    __syncthreads();
    const float t = (s[0][c] + s[1][c]) + (s[2][c] + s[3][c]);
    __syncthreads();
    return t;
}

__device__ __forceinline__ float group_rows_max(float v, float (*s)[8], int lane, int wave, int c)
{
    v = fmaxf(v, wave_xor_f32(v, 8));
    v = fmaxf(v, wave_xor_f32(v, 16));
    v = fmaxf(v, wave_xor_f32(v, 32));
    if (lane < 8) s[wave][lane] = v;
    __syncthreads();
    const float t = fmaxf(fmaxf(s[0][c], s[1][c]), fmaxf(s[2][c], s[3][c]));
    __syncthreads();
    return t;
}

// the eight values of chunk q of a row, from the row's source
template <int SRC>
__device__ __forceinline__ void proj_src_chunk(const ProjPrepArgs& a, const float* xr, uint32_t q,
                                               float inv_rms, float (&v)[8])
{
    const f32x4 lo = *reinterpret_cast<const f32x4*>(xr + q * 8), hi = *reinterpret_cast<const f32x4*>(xr + q * 8 + 4);
#pragma unroll
    for (int j = 0; j < 4; j++) {
        v[j] = lo[j];
        v[4 + j] = hi[j];
    }
    if constexpr (SRC == kProjSrcRmsNorm) {
        const f32x4 wl = *reinterpret_cast<const f32x4*>(a.norm_w + q * 8),
                    wh = *reinterpret_cast<const f32x4*>(a.norm_w + q * 8 + 4);
#pragma unroll
        for (int j = 0; j < 4; j++) {
            v[j] = v[j] * inv_rms * wl[j];
            v[4 + j] = v[4 + j] * inv_rms * wh[j];
        }
    } else if constexpr (SRC == kProjSrcSwiglu || SRC == kProjSrcGeglu) {
        const f32x4 ul = *reinterpret_cast<const f32x4*>(xr + a.K + q * 8),
                    uh = *reinterpret_cast<const f32x4*>(xr + a.K + q * 8 + 4);
#pragma unroll
        for (int j = 0; j < 8; j++) v[j] = proj_gated<SRC>(v[j], j < 4 ? ul[j] : uh[j - 4]);
    }
}

template <int SRC, int CH>
__global__ __launch_bounds__(256) void proj_prep_group_kernel(const ProjPrepArgs a)
{
    __shared__ float s48[4][8];
    const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
    const int c = t & 7;
    const uint32_t col = t >> 3;                                  // 0..31
    const uint32_t grp = blockIdx.x, row = grp * 8 + c;
    const uint32_t ktiles = a.K / 32, nchunks = a.K / 8;
    half8* frow = a.frag + (size_t)grp * ktiles * 64;
    const bool live = row < a.R;                                  // rows past R pad the last group with zeros
    const float* xr = a.x + (size_t)(live ? row : a.R - 1) * a.ldx;

    // rows need 16-byte alignment for the vector loads: ldx and K are multiples
    // of four floats (the host checks), the base comes from the allocator
    float inv_rms = 1.0f;
    if constexpr (SRC == kProjSrcRmsNorm) {
        float ss = 0.f;
        for (uint32_t q = col; q < nchunks; q += 32) {
            const f32x4 lo = *reinterpret_cast<const f32x4*>(xr + q * 8), hi = *reinterpret_cast<const f32x4*>(xr + q * 8 + 4);
#pragma unroll
            for (int j = 0; j < 4; j++) ss = fmaf(lo[j], lo[j], ss);
#pragma unroll
            for (int j = 0; j < 4; j++) ss = fmaf(hi[j], hi[j], ss);
        }
        inv_rms = 1.0f / sqrtf(group_rows_sum(ss, s48, lane, wave, c) / (float)a.K + a.eps);
    }

    float held[CH > 0 ? CH : 1][8];
    float mx = 0.f;
    if constexpr (CH > 0) {
#pragma unroll
        for (int i = 0; i < CH; i++) {
            const uint32_t q = col + 32 * i;
            if (q < nchunks) {
                proj_src_chunk<SRC>(a, xr, q, inv_rms, held[i]);
#pragma unroll
                for (int j = 0; j < 8; j++) mx = fmaxf(mx, fabsf(held[i][j]));
            }
        }
    } else {
        for (uint32_t q = col; q < nchunks; q += 32) {
            float v[8];
            proj_src_chunk<SRC>(a, xr, q, inv_rms, v);
#pragma unroll
            for (int j = 0; j < 8; j++) mx = fmaxf(mx, fabsf(v[j]));
        }
    }
    mx = group_rows_max(mx, s48, lane, wave, c);
    uint32_t ex = (__float_as_uint(mx) >> 23) & 0xFFu;
    if (ex == 0 || ex == 0xFF) ex = 127;              // zeros, subnormals, inf / NaN rows: no scaling
    if (ex > 253) ex = 253;                           // keeps the inverse 2^-e a normal number
    if (col == 0 && live) a.scales[row] = __uint_as_float(ex << 23);
    const float inv = __uint_as_float((254u - ex) << 23);

    if constexpr (CH > 0) {
#pragma unroll
        for (int i = 0; i < CH; i++) {
            const uint32_t q = col + 32 * i;
            if (q < nchunks) {
                if (!live) {
#pragma unroll
                    for (int j = 0; j < 8; j++) held[i][j] = 0.f;
                }
                proj_write_chunk(frow, q, c, held[i], inv);
            }
        }
    } else {
        for (uint32_t q = col; q < nchunks; q += 32) {
            float v[8];
            proj_src_chunk<SRC>(a, xr, q, inv_rms, v);
            if (!live) {
#pragma unroll
                for (int j = 0; j < 8; j++) v[j] = 0.f;
            }
            proj_write_chunk(frow, q, c, v, inv);
        }
    }
}

struct ProjArgs {
    const half8* w;          // tile order
    const half8* xfrag;      // [groups][K/32][64]
    const float* scales;     // [R]
    const float* bias_rows;  // optional [R][ldy] added to the result (residual), or nullptr
    float* y;                // [R][ldy]
    uint32_t N, K, R, ldy;
    uint32_t ksplit;         // waves of a workgroup that share one run of outputs: 1, 2 or 4
};

// Writes one accumulator tile.  Layout: lane 16g + c holds outputs 16nt + 4g .. +3
// of column c; column c (< 8) is the hi term of row c of the group, column c + 8
// its lo term.  The two are combined, the row's scale undone, the optional
// residual added.  Tiles past N and rows past R are dropped.
__device__ __forceinline__ void proj_store_tile(const ProjArgs& a, f32x4 v, uint32_t nt, uint32_t group,
                                                int lane, const float* scales = nullptr,
                                                const f32x4* residual = nullptr)
{
    if (!scales) scales = a.scales;
    const int c = lane & 15, g = lane >> 4;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        // the lo column of row c is eight lanes on in the same row of sixteen: a
        // rotation by eight inside the row (DPP row_ror:8), no trip through LDS
        const float other = __int_as_float(
            __builtin_amdgcn_update_dpp(0, __float_as_int(v[i]), 0x128, 0xF, 0xF, false));
        v[i] += other * (1.0f / kProjLoScale);      // meaningful in the hi columns only
    }
    const uint32_t row = group * 8 + (c & 7);
    if (c < 8 && row < a.R && nt < a.N / 16) {
        const float sc = scales[row];
        const size_t o = (size_t)row * a.ldy + nt * 16 + g * 4;
        f32x4 r;
#pragma unroll
        for (int i = 0; i < 4; i++) r[i] = v[i] * sc;
        if (a.bias_rows) {
            // (residual: the same values, read earlier by the caller)
            const f32x4 b = residual ? *residual : *reinterpret_cast<const f32x4*>(a.bias_rows + o);
#pragma unroll
            for (int i = 0; i < 4; i++) r[i] += b[i];
        }
        *reinterpret_cast<f32x4*>(a.y + o) = r;
    }
}

// One wave-step: NT weight tiles against GROUPS operand fragments.
template <int GROUPS, int NT>
__device__ __forceinline__ void proj_step(f32x4 (&acc)[NT][GROUPS], const half8 (&wv)[NT],
                                          const half8* __restrict__ xp, uint32_t ktiles, uint32_t kt)
{
#pragma unroll
    for (int gi = 0; gi < GROUPS; gi++) {
        const half8 xb = xp[((size_t)gi * ktiles + kt) * 64];
#pragma unroll
        for (int t = 0; t < NT; t++)
            acc[t][gi] = __builtin_amdgcn_mfma_f32_16x16x32_f16(wv[t], xb, acc[t][gi], 0, 0, 0);
    }
}

// GROUPS = row groups of eight per wave, NT = 16-output tiles per wave
// (templates, so the accumulators stay in registers); grid.y walks further
// runs of GROUPS row groups when a launch carries more rows than that.  A workgroup is four
// waves.  With ksplit = 1 they own four consecutive runs of 16*NT outputs; with
// ksplit = 2 or 4 that many waves share a run and take contiguous parts of the
// input range (a narrow weight then still puts a thousand waves on the chip),
// and their sums are added through LDS in part order, so the result does not
// depend on timing.  Every X fragment a wave loads serves NT weight tiles:
// with two row groups (9..16 rows) NT = 2 keeps the operand traffic through
// the vector cache at the two bytes per weight byte of the one-group case.
template <int GROUPS, int NT>
__global__ __launch_bounds__(kProjThreads) void proj_rows_kernel(const ProjArgs a)
{
    constexpr int KB = kProjKBatch / NT;                               // k-steps per register batch
    // partial sums of the waves with part > 0: (4 / S) runs x (S - 1) parts <= 3 entries
    __shared__ f32x4 s_part[(GROUPS <= 2) ? 3 * NT * GROUPS * 64 : 1];

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const uint32_t S = a.ksplit;
    const uint32_t slot = wave / S, part = wave % S;
    const uint32_t run = blockIdx.x * (4 / S) + slot;            // this wave's run of 16*NT outputs
    const uint32_t nt0 = run * NT;
    const uint32_t ntiles = a.N / 16;
    const bool live = nt0 < ntiles;                              // N/16 need not be a multiple of the runs per block
    const uint32_t ktiles = a.K / 32;
    const uint32_t kper = ktiles / S;                            // host guarantees divisibility
    const uint32_t k_begin = part * kper, k_end = k_begin + kper;
    // blockIdx.y: which run of GROUPS row groups (prefill-sized row counts only)
    const uint32_t group0 = blockIdx.y * GROUPS;
    const half8* xp = a.xfrag + (size_t)group0 * ktiles * 64 + lane;

    f32x4 acc[NT][GROUPS];
#pragma unroll
    for (int t = 0; t < NT; t++)
#pragma unroll
        for (int gi = 0; gi < GROUPS; gi++) acc[t][gi] = f32x4{0.f, 0.f, 0.f, 0.f};

    if (live) {
        // tile t of this wave; a run that sticks out past N re-reads the last tile and drops the result
        const half8* wp[NT];
#pragma unroll
        for (int t = 0; t < NT; t++) {
            const uint32_t nt = (nt0 + t < ntiles) ? nt0 + t : ntiles - 1;
            wp[t] = a.w + (size_t)nt * ktiles * 64 + lane;
        }
        // W is read exactly once per launch (non-temporal); X fragments are
        // shared by every wave of the grid and stay cached.  Loads inside the
        // loop are unconditional and the last batch is peeled, so the
        // compiler's load counting keeps the prefetched batch in flight.
        half8 wa[KB][NT], wb[KB][NT];
        // The operand fragments travel a batch ahead with the weights: read when
        // needed they are cache hits, but a round trip to L2 per batch on a
        // chain of four to thirty batches that is the launch's critical path.
        half8 xa[KB][GROUPS], xb[KB][GROUPS];
        auto load_x = [&](half8 (&xv)[KB][GROUPS], uint32_t k0) {
#pragma unroll
            for (int u = 0; u < KB; u++)
#pragma unroll
                for (int gi = 0; gi < GROUPS; gi++) xv[u][gi] = xp[((size_t)gi * ktiles + k0 + u) * 64];
        };
        auto step = [&](const half8 (&wv)[NT], const half8 (&xv)[GROUPS]) {
#pragma unroll
            for (int gi = 0; gi < GROUPS; gi++)
#pragma unroll
                for (int t = 0; t < NT; t++)
                    acc[t][gi] = __builtin_amdgcn_mfma_f32_16x16x32_f16(wv[t], xv[gi], acc[t][gi], 0, 0, 0);
        };
        uint32_t kt = k_begin;
        const uint32_t full_end = k_begin + kper / KB * KB;
        if (kt < full_end) {
#pragma unroll
            for (int u = 0; u < KB; u++)
#pragma unroll
                for (int t = 0; t < NT; t++)
                    wa[u][t] = __builtin_nontemporal_load(&wp[t][(size_t)(kt + u) * 64]);
            load_x(xa, kt);
            while (kt + 2 * KB <= full_end) {
#pragma unroll
                for (int u = 0; u < KB; u++)
#pragma unroll
                    for (int t = 0; t < NT; t++)
                        wb[u][t] = __builtin_nontemporal_load(&wp[t][(size_t)(kt + KB + u) * 64]);
                load_x(xb, kt + KB);
#pragma unroll
                for (int u = 0; u < KB; u++) step(wa[u], xa[u]);
#pragma unroll
                for (int u = 0; u < KB; u++) {
#pragma unroll
                    for (int t = 0; t < NT; t++) wa[u][t] = wb[u][t];
#pragma unroll
                    for (int gi = 0; gi < GROUPS; gi++) xa[u][gi] = xb[u][gi];
                }
                kt += KB;
            }
#pragma unroll
            for (int u = 0; u < KB; u++) step(wa[u], xa[u]);
            kt += KB;
        }
        for (; kt < k_end; kt++) {                               // part not a multiple of the batch
            half8 wv[NT];
#pragma unroll
            for (int t = 0; t < NT; t++) wv[t] = __builtin_nontemporal_load(&wp[t][(size_t)kt * 64]);
            proj_step<GROUPS, NT>(acc, wv, xp, ktiles, kt);
        }
    }

    if constexpr (GROUPS <= 2) {
        if (S > 1) {                                             // uniform over the workgroup
            if (part > 0) {
#pragma unroll
                for (int t = 0; t < NT; t++)
#pragma unroll
                    for (int gi = 0; gi < GROUPS; gi++)
                        s_part[(((slot * (S - 1) + (part - 1)) * NT + t) * GROUPS + gi) * 64 + lane] = acc[t][gi];
            }
            __syncthreads();
            if (part > 0) return;
            for (uint32_t p = 1; p < S; p++) {
#pragma unroll
                for (int t = 0; t < NT; t++)
#pragma unroll
                    for (int gi = 0; gi < GROUPS; gi++) {
                        const f32x4 o = s_part[(((slot * (S - 1) + (p - 1)) * NT + t) * GROUPS + gi) * 64 + lane];
#pragma unroll
                        for (int i = 0; i < 4; i++) acc[t][gi][i] += o[i];
                    }
            }
        }
    }
    if (!live) return;

#pragma unroll
    for (int t = 0; t < NT; t++)
#pragma unroll
        for (int gi = 0; gi < GROUPS; gi++) proj_store_tile(a, acc[t][gi], nt0 + t, group0 + gi, lane);
}

// One row (a decode step): proj_rows_kernel<1, 1> with the fragment kernel
// folded in.  Every workgroup builds the row's operand terms in its own LDS
// (4 bytes per input: hi and lo of the one live column pair) while its first
// batches of weights are on the way, instead of reading fragments a launch before
// it wrote: a decode step is a chain of dependent launches of a few
// microseconds each, and this removes four of ten per layer.  The row's values,
// the scale and the order of every sum are those of proj_prep_kernel followed
// by proj_rows_kernel<1, 1> (same helpers, same loops), so the result has the
// same bits: a serial step still equals its row of a batched step.
//
// Order of the requests: the row (with the norm's weights, the gate's partner
// values and the residual) FIRST, then up to three batches of weights (24
// k-steps: the whole share of a wave for inputs up to 3072 at four waves per
// tile).  A wave's loads come back in the order they were asked for, so a row
// asked for after the weights is not there before them (2.0 us after the
// workgroup's start, measured, against 0.8); asked for first, the sums over the
// row run while the weights travel.  NB0 = batches asked for up front, a
// template parameter so that every load before the first wait is unconditional
// and the compiler's count of loads in flight is exact.
template <int SRC, int NB0>
__device__ __forceinline__ void proj_row1_body(const ProjArgs& a, const ProjPrepArgs& p, half8* sfrag,
                                               f32x4* s_part, float* s4, float* s_scale)
{
    constexpr int KB = kProjKBatch;
    constexpr int CH = 2;                                        // chunks of eight inputs a thread can hold
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const uint32_t t = threadIdx.x;
    const uint32_t S = a.ksplit;
    const uint32_t slot = wave / S, part = wave % S;
    const uint32_t nt0 = blockIdx.x * (4 / S) + slot;
    const uint32_t ntiles = a.N / 16;
    const bool live = nt0 < ntiles;
    const uint32_t ktiles = a.K / 32, nchunks = a.K / 8;
    const uint32_t kper = ktiles / S;
    const uint32_t k_begin = part * kper, k_end = k_begin + kper;
    const half8* wp = a.w + (size_t)(live ? nt0 : ntiles - 1) * ktiles * 64 + lane;
    const float* xr = p.x;
    const bool in_regs = a.K <= 2048u * CH;                      // uniform

    // 1. the row and what goes with it (a chunk past the end re-reads the last one; dropped below)
    f32x4 xl[CH], xh[CH];
    f32x4 el[SRC == kProjSrcPlain ? 1 : CH], eh[SRC == kProjSrcPlain ? 1 : CH];     // norm weights / gate partners
    if (in_regs) {
#pragma unroll
        for (int i = 0; i < CH; i++) {
            const uint32_t qc = min(t + 256u * i, nchunks - 1);
            xl[i] = *reinterpret_cast<const f32x4*>(xr + qc * 8);
            xh[i] = *reinterpret_cast<const f32x4*>(xr + qc * 8 + 4);
            if constexpr (SRC == kProjSrcRmsNorm) {
                el[i] = *reinterpret_cast<const f32x4*>(p.norm_w + qc * 8);
                eh[i] = *reinterpret_cast<const f32x4*>(p.norm_w + qc * 8 + 4);
            } else if constexpr (SRC == kProjSrcSwiglu || SRC == kProjSrcGeglu) {
                el[i] = *reinterpret_cast<const f32x4*>(xr + a.K + qc * 8);
                eh[i] = *reinterpret_cast<const f32x4*>(xr + a.K + qc * 8 + 4);
            }
        }
    }

    // 1b. the residual values the store at the very end will add, for every lane
    // and whether or not there is a residual (the row's start stands in): a load
    // that is only sometimes issued would turn the exact waits below into waits
    // for everything in flight
    f32x4 resid;
    {
        const int rc = lane & 15, rg = lane >> 4;
        const uint32_t rrow = min((uint32_t)(rc & 7), a.R - 1), rnt = min(nt0, ntiles - 1);
        const float* rp = a.bias_rows ? a.bias_rows + (size_t)rrow * a.ldy + rnt * 16 + rg * 4 : xr + rg * 4;
        resid = *reinterpret_cast<const f32x4*>(rp);
    }

    // 2. the weights: NB0 batches now, the rest as the buffers come free
    half8 wa[KB], wb[KB], wc[KB];
    const uint32_t nb = kper / KB;                               // whole batches of this wave (>= NB0)
    auto load_batch = [&](half8 (&w)[KB], uint32_t b) {
#pragma unroll
        for (int u = 0; u < KB; u++) w[u] = __builtin_nontemporal_load(&wp[(size_t)(k_begin + b * KB + u) * 64]);
    };
    if constexpr (NB0 > 0) load_batch(wa, 0);
    if constexpr (NB0 > 1) load_batch(wb, 1);
    if constexpr (NB0 > 2) load_batch(wc, 2);

    // 3. the row's terms, as proj_prep_kernel forms them
    auto put_chunk = [&](uint32_t q, const float (&v)[8], float inv) {
        half8 hi, lo;
#pragma unroll
        for (int j = 0; j < 8; j++) {
            const float sv = v[j] * inv;
            _Float16 h = (_Float16)sv;
            if (fabsf((float)h) < 6.103515625e-05f) h = (_Float16)0.0f;      // 2^-14
            hi[j] = h;
            lo[j] = (_Float16)((sv - (float)h) * kProjLoScale);
        }
        sfrag[q * 2] = hi;
        sfrag[q * 2 + 1] = lo;
    };
    if (in_regs) {
        // One read of the row: its values stay in registers between the passes
        // (sum of squares, largest magnitude, terms).  Same values, same order of
        // the sum as the passes of the other branch (thread t takes the chunks t,
        // t + 256, ... in order).
        float v[CH][8];
        float ss = 0.f;
#pragma unroll
        for (int i = 0; i < CH; i++) {
            const bool has = t + 256u * i < nchunks;
#pragma unroll
            for (int j = 0; j < 4; j++) {
                v[i][j] = has ? xl[i][j] : 0.f;
                v[i][4 + j] = has ? xh[i][j] : 0.f;
            }
            if constexpr (SRC == kProjSrcRmsNorm) {
#pragma unroll
                for (int j = 0; j < 8; j++) ss = fmaf(v[i][j], v[i][j], ss);
            }
        }
        if constexpr (SRC == kProjSrcRmsNorm) {
            const float inv_rms = 1.0f / sqrtf(block_sum_256(ss, s4) / (float)a.K + p.eps);
#pragma unroll
            for (int i = 0; i < CH; i++) {
                if (t + 256u * i < nchunks) {
#pragma unroll
                    for (int j = 0; j < 4; j++) {
                        v[i][j] = v[i][j] * inv_rms * el[i][j];
                        v[i][4 + j] = v[i][4 + j] * inv_rms * eh[i][j];
                    }
                }
            }
        } else if constexpr (SRC == kProjSrcSwiglu || SRC == kProjSrcGeglu) {
#pragma unroll
            for (int i = 0; i < CH; i++) {
                if (t + 256u * i < nchunks) {
#pragma unroll
                    for (int j = 0; j < 8; j++) v[i][j] = proj_gated<SRC>(v[i][j], j < 4 ? el[i][j] : eh[i][j - 4]);
                }
            }
        }
        float mx = 0.f;
#pragma unroll
        for (int i = 0; i < CH; i++)
#pragma unroll
            for (int j = 0; j < 8; j++) mx = fmaxf(mx, fabsf(v[i][j]));
        mx = block_max_256(mx, s4 + 4);
        uint32_t ex = (__float_as_uint(mx) >> 23) & 0xFFu;
        if (ex == 0 || ex == 0xFF) ex = 127;
        if (ex > 253) ex = 253;
        if (t == 0) *s_scale = __uint_as_float(ex << 23);
        const float inv = __uint_as_float((254u - ex) << 23);
#pragma unroll
        for (int i = 0; i < CH; i++) {
            const uint32_t q = t + 256u * i;
            if (q < nchunks) put_chunk(q, v[i], inv);
        }
    } else {
        float inv_rms = 1.0f;
        if constexpr (SRC == kProjSrcRmsNorm)
            inv_rms = 1.0f / sqrtf(row_sumsq_256(xr, a.K, s4) / (float)a.K + p.eps);
        float mx = 0.f;
        for (uint32_t k = t; k < a.K; k += 256) mx = fmaxf(mx, fabsf(proj_src_value<SRC>(p, xr, k, inv_rms)));
        mx = block_max_256(mx, s4 + 4);
        uint32_t ex = (__float_as_uint(mx) >> 23) & 0xFFu;
        if (ex == 0 || ex == 0xFF) ex = 127;
        if (ex > 253) ex = 253;
        if (t == 0) *s_scale = __uint_as_float(ex << 23);
        const float inv = __uint_as_float((254u - ex) << 23);
        for (uint32_t q = t; q < nchunks; q += 256) {
            float v[8];
#pragma unroll
            for (int j = 0; j < 8; j++) v[j] = proj_src_value<SRC>(p, xr, q * 8 + j, inv_rms);
            put_chunk(q, v, inv);
        }
    }
    lds_barrier();                                              // the terms are in LDS (the weights may still be on their way)

    // B operand of k-step kt: column 0 = hi, column 8 = lo of row 0, the rest zero
    const int c = lane & 15, g = lane >> 4;
    const bool has = (c & 7) == 0;
    const half8* my = sfrag + g * 2 + (c >> 3);
    half8 zero;
#pragma unroll
    for (int j = 0; j < 8; j++) zero[j] = (_Float16)0.0f;
    f32x4 acc = f32x4{0.f, 0.f, 0.f, 0.f};
    auto step = [&](const half8& wv, uint32_t k) {
        const half8 xb = has ? my[(size_t)k * 8] : zero;
        acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(wv, xb, acc, 0, 0, 0);
    };
    // k-steps in ascending order, whatever buffer holds them (the order of the sum
    // is that of proj_rows_kernel<1, 1>)
    auto steps = [&](const half8 (&w)[KB], uint32_t b) {
#pragma unroll
        for (int u = 0; u < KB; u++) step(w[u], k_begin + b * KB + u);
    };
    if constexpr (NB0 > 0) {
        steps(wa, 0);
        if (NB0 > 2 && nb > 3) load_batch(wa, 3);
    }
    if constexpr (NB0 > 1) {
        steps(wb, 1);
        if (NB0 > 2 && nb > 4) load_batch(wb, 4);
    }
    if constexpr (NB0 > 2) {
        steps(wc, 2);
        for (uint32_t b = 3; b < nb; b += 2) {                   // wa holds batch b, wb batch b + 1
            steps(wa, b);
            if (b + 2 < nb) load_batch(wa, b + 2);
            if (b + 1 < nb) {
                steps(wb, b + 1);
                if (b + 3 < nb) load_batch(wb, b + 3);
            }
        }
    }
    for (uint32_t kt = k_begin + nb * KB; kt < k_end; kt++) step(__builtin_nontemporal_load(&wp[(size_t)kt * 64]), kt);

    if (S > 1) {                                                 // uniform over the workgroup
        if (part > 0) s_part[(slot * (S - 1) + (part - 1)) * 64 + lane] = acc;
        __syncthreads();
        if (part > 0) return;
        for (uint32_t pp = 1; pp < S; pp++) {
            const f32x4 o = s_part[(slot * (S - 1) + (pp - 1)) * 64 + lane];
#pragma unroll
            for (int i = 0; i < 4; i++) acc[i] += o[i];
        }
    }
    if (!live) return;
    proj_store_tile(a, acc, nt0, 0, lane, s_scale, &resid);
}

template <int SRC>
__global__ __launch_bounds__(kProjThreads) void proj_row1_kernel(const ProjArgs a, const ProjPrepArgs p)
{
    extern __shared__ __attribute__((aligned(16))) unsigned char row1_smem[];
    half8* sfrag = reinterpret_cast<half8*>(row1_smem);           // [K/8][2]: hi, lo of chunk q
    __shared__ f32x4 s_part[3 * 64];
    __shared__ float s4[8];
    __shared__ float s_scale;
    const uint32_t nb = a.K / 32 / a.ksplit / kProjKBatch;        // whole batches of weights per wave: uniform
    if (nb >= 3)
        proj_row1_body<SRC, 3>(a, p, sfrag, s_part, s4, &s_scale);
    else if (nb == 2)
        proj_row1_body<SRC, 2>(a, p, sfrag, s_part, s4, &s_scale);
    else if (nb == 1)
        proj_row1_body<SRC, 1>(a, p, sfrag, s_part, s4, &s_scale);
    else
        proj_row1_body<SRC, 0>(a, p, sfrag, s_part, s4, &s_scale);
}

// Many rows (prefill chunks), products too small to fill the chip with the
// LDS-staged tiles below: a register-tiled GEMM on the same two layouts.  The
// four waves of a workgroup share one tile of NT x GROUPS accumulator tiles
// (16 NT outputs x 8 GROUPS rows) and take a quarter of the input range each;
// their sums are added through LDS in wave order.  Every k-step loads NT weight
// tiles and GROUPS operand fragments, one KiB each and both already in operand
// order, and feeds NT x GROUPS MFMAs; the next k-step's operands are requested
// while this one's MFMAs run (two register sets, the loop unrolled by two so no
// set is copied).  Small tiles and the split range put several waves on every
// SIMD and keep the chains of dependent k-steps short: these products are
// bound by load latency, not by bytes.  grid.x walks the outputs, so the
// workgroups the dispatcher deals round-robin to the eight XCDs differ in
// output tile.  At least three workgroups per CU (<= 168 registers), which
// also keeps the accumulators in ordinary vector registers.
template <int GROUPS, int NT>
__global__ __launch_bounds__(kProjThreads, 3) void proj_gemm_split_kernel(const ProjArgs a)
{
    __shared__ f32x4 s_red[3 * NT * GROUPS * 64];
    const int lane = threadIdx.x & 63;
    const uint32_t wave = (uint32_t)__builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t ktiles = a.K / 32, ntiles = a.N / 16, ngroups = (a.R + 7) / 8;
    const uint32_t nt0 = blockIdx.x * NT, group0 = blockIdx.y * GROUPS;
    const uint32_t k_begin = ktiles * wave / 4, k_end = ktiles * (wave + 1) / 4;

    // a tile or group past the end re-reads the last one; its result is dropped
    const half8* wp[NT];
    const half8* xp[GROUPS];
#pragma unroll
    for (int t = 0; t < NT; t++)
        wp[t] = a.w + (size_t)min(nt0 + t, ntiles - 1) * ktiles * 64;
#pragma unroll
    for (int gi = 0; gi < GROUPS; gi++)
        xp[gi] = a.xfrag + (size_t)min(group0 + gi, ngroups - 1) * ktiles * 64;

    f32x4 acc[NT][GROUPS];
#pragma unroll
    for (int t = 0; t < NT; t++)
#pragma unroll
        for (int gi = 0; gi < GROUPS; gi++) acc[t][gi] = f32x4{0.f, 0.f, 0.f, 0.f};

    half8 w0[NT], x0[GROUPS], w1[NT], x1[GROUPS];
    auto load_set = [&](half8 (&wv)[NT], half8 (&xv)[GROUPS], uint32_t kt) {
        const size_t o = (size_t)kt * 64 + lane;
#pragma unroll
        for (int t = 0; t < NT; t++) wv[t] = wp[t][o];
#pragma unroll
        for (int gi = 0; gi < GROUPS; gi++) xv[gi] = xp[gi][o];
    };
    auto mfma_set = [&](const half8 (&wv)[NT], const half8 (&xv)[GROUPS]) {
#pragma unroll
        for (int gi = 0; gi < GROUPS; gi++)
#pragma unroll
            for (int t = 0; t < NT; t++)
                acc[t][gi] = __builtin_amdgcn_mfma_f32_16x16x32_f16(wv[t], xv[gi], acc[t][gi], 0, 0, 0);
    };

    // loads inside the loop are unconditional (a k-step past the end re-reads the
    // last one, unused), so the load counter the compiler waits on stays exact;
    // a wave whose part of the range is empty (fewer than four k-steps) adds zeros
    const uint32_t klast = ktiles - 1;
    load_set(w0, x0, min(k_begin, klast));
    uint32_t kt = k_begin;
    for (; kt + 2 <= k_end; kt += 2) {
        load_set(w1, x1, kt + 1);
        mfma_set(w0, x0);
        load_set(w0, x0, min(kt + 2, klast));
        mfma_set(w1, x1);
    }
    if (kt < k_end) mfma_set(w0, x0);                     // odd number of k-steps

    if (wave > 0) {
#pragma unroll
        for (int t = 0; t < NT; t++)
#pragma unroll
            for (int gi = 0; gi < GROUPS; gi++)
                s_red[(((wave - 1) * NT + t) * GROUPS + gi) * 64 + lane] = acc[t][gi];
    }
    __syncthreads();
    if (wave > 0) return;
    // wave order: 0 + 1 + 2 + 3; a real loop over the waves, so that at most
    // one wave's partial tiles are in registers beside the accumulators
#pragma unroll 1
    for (int p = 0; p < 3; p++) {
        const f32x4* from = s_red + (size_t)p * NT * GROUPS * 64 + lane;
#pragma unroll
        for (int t = 0; t < NT; t++)
#pragma unroll
            for (int gi = 0; gi < GROUPS; gi++) {
                const f32x4 o = from[(t * GROUPS + gi) * 64];
#pragma unroll
                for (int i = 0; i < 4; i++) acc[t][gi][i] += o[i];
            }
    }
#pragma unroll
    for (int t = 0; t < NT; t++)
#pragma unroll
        for (int gi = 0; gi < GROUPS; gi++) proj_store_tile(a, acc[t][gi], nt0 + t, group0 + gi, lane);
}

// Many rows, products that fill the chip with 128-output x 128-row workgroup
// tiles (2 x 2 waves of 64 x 64): operands staged through LDS.  Per k-step the
// workgroup needs 8 weight tiles and 16 operand fragments, 24 KiB that are
// already in operand order: every wave copies six of them with direct-to-LDS
// loads (no registers, so the copies run two k-steps ahead of the MFMAs in a
// ring of three stages), and reads the 4 + 8 KiB of its own wave tile back with
// 128-bit LDS reads, lane i at 16 i: conflict free.  Against loading the wave
// tile's operands into registers directly the vector cache moves half the
// bytes per MFMA and the prefetch depth costs no registers.  grid.x walks the
// output panels, so one XCD's L2 holds an eighth of the weight and all of the
// fragments.
//
// Step kt: wait for this wave's copies of stage kt (the six of stage kt + 1 may
// still be in flight), workgroup barrier (everybody's copies of stage kt have
// landed, and everybody has finished reading stage kt - 1), start the copies
// of stage kt + 2 into the slot of stage kt - 1, then read and multiply.
//
// GROUPS = 8 is the tile described above; GROUPS = 4 halves the rows (128
// outputs x 64 rows, 16 KiB per stage) for products with too few rows to fill
// the chip with the large one.
// WN = waves side by side along the outputs (2 or 4; two wave rows always),
// RING = stages.  <8, 2, 3>: the tile above.  <4, 2, 3>: 128 x 64 for products
// with too few rows to fill the chip with the large one.  <8, 4, 4>: eight
// waves, 256 outputs x 128 rows, 32 KiB per stage copied three k-steps ahead,
// one workgroup per CU: a third fewer bytes per MFMA than the four-wave tile.
template <int GROUPS, int WN, int RING, int KS = 1>
constexpr size_t gemm_lds_bytes()
{
    return (size_t)KS * RING * (WN * 4 + 2 * GROUPS) * 1024;   // KiB per stage and set of waves: 4 WN weight tiles, 2 GROUPS fragments
}

// PIPE: the operand reads of the next k-step are issued before this one's MFMAs
// (two register sets), for launches that leave a SIMD with a single wave and
// nobody else to cover its LDS latency; needs one more ring stage, because a
// stage is now read one k-step before it is used.
//
// KS = 2: two such sets of waves in one workgroup, each with its own ring, take
// one half of the input range each (the host asks for it only when the number of
// k-steps is even); the upper half's sums pass through LDS at the end and the
// lower half adds them to its own, always in that order.  For products whose
// tiles give every CU one workgroup and no more (a SIMD would hold a single wave
// for a long chain of k-steps): twice the waves per SIMD, half the chain.
template <int GROUPS, int WN, int RING, bool PIPE = false, int KS = 1>
__global__ __launch_bounds__(128 * WN * KS, (WN == 2 && KS == 1) ? 2 : 1) void proj_gemm_lds_kernel(const ProjArgs a)
{
    extern __shared__ __attribute__((aligned(16))) unsigned char gemm_smem[];
    constexpr int NT = 4, WAVES = 2 * WN, CHUNKS = WN * NT + 2 * GROUPS, CPW = CHUNKS / WAVES;
    static_assert(CHUNKS % WAVES == 0, "every wave copies the same number of chunks");
    static_assert(KS == 1 || KS == 2, "one set of waves, or two that halve the input range");
    constexpr uint32_t STAGE = CHUNKS * 1024;
    const int lane = threadIdx.x & 63;
    const uint32_t wave_wg = (uint32_t)__builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t kh = wave_wg / WAVES, wave = wave_wg % WAVES;      // half of the input range, wave of the set
    const uint32_t wn = wave % WN, wr = wave / WN;
    const uint32_t ktiles_row = a.K / 32, ntiles = a.N / 16, ngroups = (a.R + 7) / 8;
    const uint32_t ktiles = ktiles_row / KS, kfirst = kh * ktiles;    // this set's k-steps
    const uint32_t klast = ktiles - 1;
    // Workgroup -> tile.  The dispatcher deals consecutive workgroups round-robin
    // to the eight XCDs; XCD x takes the output panels x, x + 8, ..., and runs
    // through all row panels of one before the next, so the workgroups resident
    // on an XCD at one time share a few weight panels (fetched once into its L2)
    // and the fragments of all rows.
    const uint32_t nx = (ntiles + WN * NT - 1) / (WN * NT), ny = (ngroups + 2 * GROUPS - 1) / (2 * GROUPS);
    const uint32_t xcd = blockIdx.x % 8, slot = blockIdx.x / 8;
    const uint32_t px = (slot / ny) * 8 + xcd, py = slot % ny;
    if (px >= nx) return;                                 // the grid is padded to eight equal shares
    const uint32_t nt_wg = px * WN * NT, g_wg = py * 2 * GROUPS;
    const uint32_t lds0 = (uint32_t)__builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)gemm_smem);

    // chunk c of a stage: weight tile nt_wg + c (c < WN * NT) or fragment group
    // g_wg + c - WN * NT; one past the end re-reads the last one, and its results are dropped
    const unsigned char* src[CPW];
#pragma unroll
    for (int i = 0; i < CPW; i++) {
        const uint32_t c = wave * CPW + i;
        const unsigned char* p =
            c < WN * NT ? reinterpret_cast<const unsigned char*>(a.w) + (size_t)min(nt_wg + c, ntiles - 1) * ktiles_row * 1024
                        : reinterpret_cast<const unsigned char*>(a.xfrag) +
                              (size_t)min(g_wg + c - WN * NT, ngroups - 1) * ktiles_row * 1024;
        src[i] = uniform_ptr(p + (size_t)kfirst * 1024);
    }
    const uint32_t lane_off = lane * 16;
    auto issue = [&](uint32_t kt) {                        // a k-step past the end copies the last one again
        const size_t k = (size_t)min(kt, klast) * 1024;
        const uint32_t to = lds0 + ((kt % RING) * KS + kh) * STAGE + wave * CPW * 1024;
#pragma unroll
        for (int i = 0; i < CPW; i++) lds_direct_load(to + i * 1024, src[i] + k, lane_off);
    };

    f32x4 acc[NT][GROUPS];
#pragma unroll
    for (int t = 0; t < NT; t++)
#pragma unroll
        for (int gi = 0; gi < GROUPS; gi++) acc[t][gi] = f32x4{0.f, 0.f, 0.f, 0.f};

#pragma unroll
    for (int st0 = 0; st0 < RING - 1; st0++) issue(st0);
    const uint32_t w_off = wn * NT * 1024 + lane * 16;
    const uint32_t x_off = (WN * NT + wr * GROUPS) * 1024 + lane * 16;
    if constexpr (PIPE) {
        static_assert(RING >= 4, "a stage is read while the one before it is multiplied");
        half8 w0[NT], x0[GROUPS], w1[NT], x1[GROUPS];
        auto read_ops = [&](half8 (&wv)[NT], half8 (&xv)[GROUPS], uint32_t kt) {
            const unsigned char* st = gemm_smem + ((kt % RING) * KS + kh) * STAGE;
#pragma unroll
            for (int t = 0; t < NT; t++) wv[t] = *reinterpret_cast<const half8*>(st + w_off + t * 1024);
#pragma unroll
            for (int gi = 0; gi < GROUPS; gi++) xv[gi] = *reinterpret_cast<const half8*>(st + x_off + gi * 1024);
        };
        auto mfmas = [&](const half8 (&wv)[NT], const half8 (&xv)[GROUPS]) {
#pragma unroll
            for (int gi = 0; gi < GROUPS; gi++)
#pragma unroll
                for (int t = 0; t < NT; t++)
                    acc[t][gi] = __builtin_amdgcn_mfma_f32_16x16x32_f16(wv[t], xv[gi], acc[t][gi], 0, 0, 0);
        };
        // stage 0 into the first register set
        asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"(CPW * (RING - 2)) : "memory");
        read_ops(w0, x0, 0);
        // Step kt: everybody's copies of stage kt + 1 have landed (the barrier),
        // the copies of stage kt + RING - 1 go to the slot of stage kt - 1, whose
        // last reads were waited for before the MFMAs of step kt - 1 were issued;
        // then the reads of stage kt + 1, then the MFMAs of stage kt.  Two steps
        // per iteration so that no register set is copied; a step past the end
        // reads a stage that holds a repeat of the last one and is not used.
        uint32_t kt = 0;
        for (; kt + 2 <= ktiles; kt += 2) {
            asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"(CPW * (RING - 3)) : "memory");
            issue(kt + RING - 1);
            read_ops(w1, x1, kt + 1);
            mfmas(w0, x0);
            asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"(CPW * (RING - 3)) : "memory");
            issue(kt + RING);
            read_ops(w0, x0, kt + 2);
            mfmas(w1, x1);
        }
        if (kt < ktiles) mfmas(w0, x0);                   // odd number of k-steps
    } else
    for (uint32_t kt = 0; kt < ktiles; kt++) {
        // this wave's copies of stage kt have landed; those of the RING - 2 stages after it may be in flight
        asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"(CPW * (RING - 2)) : "memory");
        issue(kt + RING - 1);
        const unsigned char* st = gemm_smem + ((kt % RING) * KS + kh) * STAGE;
        half8 wv[NT], xv[GROUPS];
#pragma unroll
        for (int t = 0; t < NT; t++) wv[t] = *reinterpret_cast<const half8*>(st + w_off + t * 1024);
#pragma unroll
        for (int gi = 0; gi < GROUPS; gi++) xv[gi] = *reinterpret_cast<const half8*>(st + x_off + gi * 1024);
#pragma unroll
        for (int gi = 0; gi < GROUPS; gi++)
#pragma unroll
            for (int t = 0; t < NT; t++)
                acc[t][gi] = __builtin_amdgcn_mfma_f32_16x16x32_f16(wv[t], xv[gi], acc[t][gi], 0, 0, 0);
        // all operand reads first (their latency overlaps, and the first MFMAs
        // hide the rest), then the MFMAs: left alone the scheduler reads two
        // fragments at a time and waits for each pair
        __builtin_amdgcn_sched_group_barrier(0x100, NT + GROUPS, 0);
        __builtin_amdgcn_sched_group_barrier(0x008, NT * GROUPS, 0);
    }
    // the last steps' copies still target the ring
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");

    if constexpr (KS == 2) {
        // the upper half's sums through LDS (the rings are done with: every wave's
        // copies have landed and, past the barrier, every wave's reads are over),
        // added to the lower half's in a fixed order
        static_assert((size_t)WAVES * NT * GROUPS * 1024 <= (size_t)RING * KS * STAGE, "the partial tiles fit the rings");
        f32x4* red = reinterpret_cast<f32x4*>(gemm_smem) + (size_t)wave * NT * GROUPS * 64 + lane;
        asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
        if (kh == 1) {
#pragma unroll
            for (int t = 0; t < NT; t++)
#pragma unroll
                for (int gi = 0; gi < GROUPS; gi++) red[(t * GROUPS + gi) * 64] = acc[t][gi];
        }
        asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
        if (kh == 1) return;
#pragma unroll
        for (int t = 0; t < NT; t++)
#pragma unroll
            for (int gi = 0; gi < GROUPS; gi++) {
                const f32x4 o = red[(t * GROUPS + gi) * 64];
#pragma unroll
                for (int i = 0; i < 4; i++) acc[t][gi][i] += o[i];
            }
    }

    const uint32_t nt0 = nt_wg + wn * NT, group0 = g_wg + wr * GROUPS;
    if (nt0 >= ntiles || group0 >= ngroups) return;
#pragma unroll
    for (int t = 0; t < NT; t++)
#pragma unroll
        for (int gi = 0; gi < GROUPS; gi++) proj_store_tile(a, acc[t][gi], nt0 + t, group0 + gi, lane);
}

}  // namespace wr
