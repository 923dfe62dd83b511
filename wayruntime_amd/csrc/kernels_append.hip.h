// Cache append / import / export kernels.
//
// append: F32 rows [n_rows][nkv][hd] -> truncated F16 into rows pos.. of K and
// of the block-transposed Vt (layout in common.hip.h).  The conversion is the
// reference's truncating rule (reference: src/core/session.c:139-154 calling
// src/core/quant.c:121-136), done with integer ops so the stored bits equal
// the reference's bit for bit.  HBM-bound byte work: 6 bytes moved per element
// (4 read, 2 written).
#pragma once

#include "common.hip.h"

namespace wr {

template <typename Src>
__device__ __forceinline__ uint16_t to_cache_bits(Src v);
template <>
__device__ __forceinline__ uint16_t to_cache_bits<float>(float v) { return f32_to_f16_trunc(v); }
template <>
__device__ __forceinline__ uint16_t to_cache_bits<uint16_t>(uint16_t v) { return v; }

// K side: one thread per element; reads are unit-stride in d, writes go out in
// 16-byte chunks (eight consecutive d of one position).
template <typename Src>
__global__ __launch_bounds__(256) void append_k_kernel(const Src* __restrict__ src,
                                                       uint16_t* __restrict__ k, uint32_t pos,
                                                       uint32_t n_rows, uint32_t nkv, uint32_t hd,
                                                       uint32_t ctx_pad)
{
    const size_t total = (size_t)n_rows * nkv * hd;
    const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= total) return;
    const uint32_t d = (uint32_t)(idx % hd);
    const uint32_t kvh = (uint32_t)((idx / hd) % nkv);
    const uint32_t r = (uint32_t)(idx / ((size_t)hd * nkv));
    k[k_offset(kvh, ctx_pad, pos + r, d, hd)] = to_cache_bits<Src>(src[idx]);
}

// V side: a workgroup owns a 32-position x 64-dimension tile of one KV head.
// It reads the source unit-stride in d, turns the tile through LDS and writes
// each dimension's 32 positions as one contiguous 64-byte run.  Positions of
// the block that lie outside [pos, pos + n_rows) are left untouched, so a
// one-row decode append never disturbs its neighbours.
template <typename Src>
__global__ __launch_bounds__(256) void append_v_kernel(const Src* __restrict__ src,
                                                       uint16_t* __restrict__ vt, uint32_t pos,
                                                       uint32_t n_rows, uint32_t nkv, uint32_t hd,
                                                       uint32_t ctx_pad)
{
    __shared__ uint16_t tile[64][kVBlock + 2];
    const uint32_t d0 = blockIdx.x * 64;
    const uint32_t kvh = blockIdx.y;
    const uint32_t blk = pos / kVBlock + blockIdx.z;
    const uint32_t t = threadIdx.x;
    const uint32_t end = pos + n_rows;

    const uint32_t dl = t & 63;
#pragma unroll
    for (int i = 0; i < 8; i++) {
        const uint32_t pl = i * 4 + (t >> 6);
        const uint32_t p = blk * kVBlock + pl;
        uint16_t bits = 0;
        if (p >= pos && p < end && d0 + dl < hd)
            bits = to_cache_bits<Src>(src[((size_t)(p - pos) * nkv + kvh) * hd + d0 + dl]);
        tile[dl][pl] = bits;
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < 8; i++) {
        const uint32_t idx = i * 256 + t;
        const uint32_t dl2 = idx / kVBlock;
        const uint32_t pl2 = idx % kVBlock;
        const uint32_t p = blk * kVBlock + pl2;
        if (p >= pos && p < end && d0 + dl2 < hd)
            vt[vt_offset(kvh, ctx_pad, p, d0 + dl2, hd)] = tile[dl2][pl2];
    }
}

// Rotary position embedding in place on F32 rows [rows][heads][hd], split-half
// pairing (element j with element j + hd/2, j < n_rot), as the reference
// applies it before the append (reference: src/core/kernels.c:1356-1412):
//   r[j] = x0*c - x1*s,  r[j + hd/2] = x0*s + x1*c
// with c = cs[row][j][0], s = cs[row][j][1], the table rope_table_kernel below
// (or the caller) makes.  The products and the sum are rounded separately (no
// fused multiply-add), so the rotated values, and with them the cache bits,
// equal the reference's bit for bit.
__global__ __launch_bounds__(256) void rope_rows_kernel(float* __restrict__ x,
                                                        const float* __restrict__ cs,
                                                        uint32_t rows, uint32_t heads,
                                                        uint32_t hd, uint32_t n_rot)
{
// The products and their sum must round one by one.  The pragma covers the
// operators written in this function; the __fmul_rn / __fadd_rn intrinsics do
// not help, they are plain operators defined under the default contraction.
#pragma clang fp contract(off)
    const size_t total = (size_t)rows * heads * n_rot;
    const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= total) return;
    const uint32_t j = (uint32_t)(idx % n_rot);
    const uint32_t h = (uint32_t)((idx / n_rot) % heads);
    const uint32_t r = (uint32_t)(idx / ((size_t)n_rot * heads));
    const uint32_t half = hd / 2;
    float* row = x + ((size_t)r * heads + h) * hd;
    const float c = cs[((size_t)r * n_rot + j) * 2], sn = cs[((size_t)r * n_rot + j) * 2 + 1];
    const float x0 = row[j], x1 = row[j + half];
    const float a0 = x0 * c, b0 = x1 * sn, a1 = x0 * sn, b1 = x1 * c;
    row[j] = a0 - b0;
    row[j + half] = a1 + b1;
}

// ---- rotary angles ---------------------------------------------------------
// (cos, sin) of angle(p, j) = p / base^(2j/hd) for `rows` positions and n_rot
// pairs, out [rows][n_rot][2], through the reference's own scalar forms
// operation for operation (reference: src/core/kernels.c:1384-1404 for the
// angle, src/core/mathx.c:37-57 exp, :72-86 log, :112-147 range reduction, sine
// and cosine), every operator rounded by itself, division and int conversion
// as C has them: the table's bytes equal the reference's.
//
// The reference folds an angle into [-pi, pi] by subtracting 2*pi once per
// turn, and each subtraction rounds: only the same loop gives the same bits,
// thousands of dependent steps for the low pairs of a late position.  The
// lanes of a wave therefore take 64 consecutive ROWS of one pair: their angles
// differ by at most 63 / base^(2j/hd), so all 64 leave the loop within a few
// turns of each other and a wave costs what its slowest lane costs; a launch
// has (rows / 64) x n_rot such waves, and the higher pairs (the angle shrinks
// geometrically with j) finish early and free their slots.
struct RopeTableArgs {
    float* out;
    uint32_t rows, hd, n_rot;
    float theta;
    uint32_t pos0;
    uint32_t listed;          // rows <= 16 positions given one by one
    uint32_t pos[16];
};

__device__ __forceinline__ float ref_exp(float x)
{
#pragma clang fp contract(off)
    if (x < -88.0f) return 0.0f;
    if (x > 88.0f) return 1e38f;
    const float ln2 = 0.6931471805599453f;
    const int k = (int)(x / ln2 + (x >= 0 ? 0.5f : -0.5f));
    const float r = x - (float)k * ln2;
    const float r2 = r * r;
    float e = 1.0f + r + r2 * 0.5f + r2 * r * (1.0f / 6.0f) + r2 * r2 * (1.0f / 24.0f) +
              r2 * r2 * r * (1.0f / 120.0f);
    if (k >= -126 && k <= 127) e = __uint_as_float(__float_as_uint(e) + ((uint32_t)k << 23));
    return e;
}

__device__ __forceinline__ float ref_log(float x)
{
#pragma clang fp contract(off)
    if (x <= 0.0f) return -1e38f;
    const uint32_t u = __float_as_uint(x);
    const int e = (int)((u >> 23) & 0xFF) - 127;
    const float m = __uint_as_float((u & 0x007FFFFFu) | 0x3F800000u);
    const float t = (m - 1.0f) / (m + 1.0f);
    const float t2 = t * t;
    const float lnm =
        2.0f * t * (1.0f + t2 * (1.0f / 3.0f + t2 * (1.0f / 5.0f + t2 * (1.0f / 7.0f))));
    return lnm + (float)e * 0.6931471805599453f;
}

__global__ __launch_bounds__(64) void rope_table_kernel(const RopeTableArgs a)
{
#pragma clang fp contract(off)
    const uint32_t r = blockIdx.x * 64u + threadIdx.x;
    const uint32_t j = blockIdx.y;
    if (r >= a.rows) return;
    const uint32_t p = a.listed ? a.pos[r & 15u] : a.pos0 + r;
    const float lnb = ref_log(a.theta);
    const float exponent = (float)(2u * j) / (float)a.hd;
    const float powv = ref_exp(exponent * lnb);
    float x = (float)p / powv;
    const float pi = 3.14159265358979f, two_pi = 6.28318530717958f;
    while (x > pi) x -= two_pi;
    while (x < -pi) x += two_pi;
    const float x2 = x * x;
    const float x3 = x2 * x, x5 = x3 * x2, x7 = x5 * x2;
    const float sn = x - x3 * (1.0f / 6.0f) + x5 * (1.0f / 120.0f) - x7 * (1.0f / 5040.0f);
    const float x4 = x2 * x2, x6 = x4 * x2;
    const float cs = 1.0f - x2 * 0.5f + x4 * (1.0f / 24.0f) - x6 * (1.0f / 720.0f);
    float2* o = reinterpret_cast<float2*>(a.out) + ((size_t)r * a.n_rot + j);
    *o = make_float2(cs, sn);
}

// One new row for each of up to 16 sessions in one launch (the batched decode
// step appends one position per session and layer).  grid = sessions.
struct AppendBatchArgs {
    uint16_t* k[16];
    uint16_t* vt[16];
    uint32_t pos[16];
    uint32_t ctx_pad[16];
    const float* k_src;      // [n][nkv][hd]
    const float* v_src;
    uint32_t nkv, hd;
};

__global__ __launch_bounds__(256) void append_batch_kernel(const AppendBatchArgs a)
{
    const uint32_t i = blockIdx.x;
    const uint32_t row = a.nkv * a.hd;
    const uint32_t pos = a.pos[i], ctx_pad = a.ctx_pad[i];
    for (uint32_t idx = threadIdx.x; idx < row; idx += 256) {
        const uint32_t kvh = idx / a.hd, d = idx % a.hd;
        a.k[i][k_offset(kvh, ctx_pad, pos, d, a.hd)] = f32_to_f16_trunc(a.k_src[(size_t)i * row + idx]);
        a.vt[i][vt_offset(kvh, ctx_pad, pos, d, a.hd)] = f32_to_f16_trunc(a.v_src[(size_t)i * row + idx]);
    }
}

// Export rows back in position-major order [n_rows][nkv][hd] (tests, tooling).
__global__ __launch_bounds__(256) void export_kv_kernel(const uint16_t* __restrict__ k,
                                                        const uint16_t* __restrict__ vt,
                                                        uint16_t* __restrict__ k_out,
                                                        uint16_t* __restrict__ v_out, uint32_t pos,
                                                        uint32_t n_rows, uint32_t nkv, uint32_t hd,
                                                        uint32_t ctx_pad)
{
    const size_t total = (size_t)n_rows * nkv * hd;
    const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= total) return;
    const uint32_t d = (uint32_t)(idx % hd);
    const uint32_t kvh = (uint32_t)((idx / hd) % nkv);
    const uint32_t r = (uint32_t)(idx / ((size_t)hd * nkv));
    k_out[idx] = k[k_offset(kvh, ctx_pad, pos + r, d, hd)];
    v_out[idx] = vt[vt_offset(kvh, ctx_pad, pos + r, d, hd)];
}

}  // namespace wr
