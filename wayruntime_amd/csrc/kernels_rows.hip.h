// Row-wise steps around the attention path for callers that keep a layer's
// activations on the device: RMS normalisation, the split of a stacked Q/K/V
// projection into rotated Q, rotated K and V (per-head RMSNorm and rotary
// embedding fused, the steps the reference runs between the projections and
// the cache append, src/core/session.c:459-486), and the gated activation.
// All are tiny byte-moving kernels; none is on the timed attention path.
//
// Arithmetic follows the reference's formulas (src/core/kernels.c:1276-1316
// RMSNorm, :1356-1412 rotary, :963-967 SiLU); sums over a row are tree
// reductions here, sequential there, so results agree to F32 rounding.
#pragma once

#include "common.hip.h"
#include "kernels_proj.hip.h"      // row_sumsq_256: the one summation order of every row norm
#include "row8.hip.h"              // a head's norm and rotation with eight lanes per position

namespace wr {

constexpr int kRowsMaxHd = 1024;      // largest head_dim (reference: WR_FLASH_D_MAX)

__device__ __forceinline__ float wave_sum_f32(float v)
{
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) v += wave_xor_f32(v, off);
    return v;
}

// out[r][j] = x[r][j] * (1 / sqrt(mean_j x^2 + eps)) * w[j % wn]   (wn == 0: no weight),
// or out[r][j] += that when `accumulate` (a normalised sublayer output joining the residual)
// One workgroup of 256 threads per row.
__global__ __launch_bounds__(256) void rmsnorm_rows_kernel(const float* __restrict__ x, uint32_t ldx,
                                                           const float* __restrict__ w, uint32_t wn,
                                                           float* __restrict__ out, uint32_t ldo,
                                                           uint32_t dim, float eps, int accumulate)
{
    __shared__ float s_sum[4];
    const uint32_t r = blockIdx.x;
    const float* xr = x + (size_t)r * ldx;
    const float total = row_sumsq_256(xr, dim, s_sum);
    const float inv_rms = 1.0f / sqrtf(total / (float)dim + eps);
    float* orow = out + (size_t)r * ldo;
    for (uint32_t j = threadIdx.x; j < dim; j += 256) {
        const float ww = wn ? w[j % wn] : 1.0f;
        const float v = xr[j] * inv_rms * ww;
        orow[j] = accumulate ? orow[j] + v : v;
    }
}

struct QkvPrepArgs {
    const float* qkv;        // [rows][ld]: nq query heads, then nkv key heads, then nkv value heads
    const float* q_norm;     // [hd] per-head RMSNorm weights, or nullptr for no Q/K norm
    const float* k_norm;
    const float* cos_sin;    // [rows][n_rot][2]
    float* q_out;            // [rows][nq][hd]
    float* k_out;            // [rows][nkv][hd]
    float* v_out;            // [rows][nkv][hd]
    uint32_t ld, nq, nkv, hd, n_rot;
    float eps;
};

// grid = (rows, nq + 2 nkv), one wave per (row, head).  Q and K heads: optional
// RMSNorm over the head, then the rotary embedding (split-half pairing, element
// j with j + hd/2 for j < n_rot, products and sums rounded one by one as in
// rope_rows_kernel); V heads are copied.
__global__ __launch_bounds__(64) void qkv_prep_kernel(const QkvPrepArgs a)
{
#pragma clang fp contract(off)
    __shared__ float s[kRowsMaxHd];
    const uint32_t r = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
    const uint32_t hd = a.hd, half = hd / 2;
    const float* src = a.qkv + (size_t)r * a.ld + (size_t)h * hd;
    if (h >= a.nq + a.nkv) {
        float* dst = a.v_out + ((size_t)r * a.nkv + (h - a.nq - a.nkv)) * hd;
        for (uint32_t j = lane; j < hd; j += 64) dst[j] = src[j];
        return;
    }
    const bool is_q = h < a.nq;
    const float* nw = is_q ? a.q_norm : a.k_norm;
    float* dst = is_q ? a.q_out + ((size_t)r * a.nq + h) * hd
                      : a.k_out + ((size_t)r * a.nkv + (h - a.nq)) * hd;
    float ss = 0.f;
    for (uint32_t j = lane; j < hd; j += 64) {
        const float v = src[j];
        s[j] = v;
        ss += v * v;
    }
    if (nw) {
        ss = wave_sum_f32(ss);
        const float inv_rms = 1.0f / sqrtf(ss / (float)hd + a.eps);
        for (uint32_t j = lane; j < hd; j += 64) s[j] = s[j] * inv_rms * nw[j];
    }
    __syncthreads();
    const float* cs = a.cos_sin + (size_t)r * a.n_rot * 2;
    for (uint32_t j = lane; j < half; j += 64) {
        const float x0 = s[j], x1 = s[j + half];
        if (j < a.n_rot) {
            const float c = cs[2 * j], sn = cs[2 * j + 1];
            const float a0 = x0 * c, b0 = x1 * sn, a1 = x0 * sn, b1 = x1 * c;
            dst[j] = a0 - b0;
            dst[j + half] = a1 + b1;
        } else {
            dst[j] = x0;
            dst[j + half] = x1;
        }
    }
}

// qkv_prep and the cache append in one launch: Q heads leave as rotated F32
// rows, K heads go through the same norm and rotation and are truncated to F16
// straight into the cache's K tiles, V heads are truncated and turned into the
// block-transposed Vt.  The arithmetic is qkv_prep_kernel's (one wave per row
// and head, the same wave sum) and the conversion is the append kernels', so Q
// and the cache bits equal the two-step path's bit for bit.
//
// Two shapes of call:
//   rows of ONE session at consecutive positions pos[0] ... (prefill, a step):
//     grid.x walks the cache's 32-position blocks the rows touch;
//   ONE row for each of n sessions (batched step): grid.x = session.
// grid.y = head (nq + 2 nkv), 256 threads: wave w takes the block's positions
// w, w + 4, ...  A V workgroup gathers its block in LDS and writes each
// dimension's positions as one run, like append_v_kernel.
struct QkvAppendArgs {
    const float* qkv;        // [rows][ld]
    const float* q_norm;
    const float* k_norm;
    const float* cos_sin;    // [rows][n_rot][2]
    float* q_out;            // [rows][nq][hd]
    uint16_t* q16_out;       // or (eight-lane form only): the Q rows as binary16, multiplied by q16_scale
    float q16_scale;
    uint16_t* k[16];
    uint16_t* vt[16];
    uint32_t pos[16];
    uint32_t ctx_pad[16];
    uint32_t ld, nq, nkv, hd, n_rot, rows;
    uint32_t per_session;    // 1: row i belongs to session i; 0: all rows to session 0 from pos[0]
    uint32_t v_norm;         // 1: V heads get a weightless RMSNorm before they are stored
    uint32_t row8;           // hd / 64 (2 or 4) when qkv_append_row8 may serve the call, else 0
    float eps;
};

// One workgroup's share of qkv_append_kernel for head dims of 128 and 256
// (NJ = hd / 64) with everything 16-byte aligned: eight lanes per position, all
// 32 positions of the block at once.  Lane `part` of a position holds the
// elements 64 c + 8 part + e (c < NJ, e < 8), i.e. what the lanes 8 part .. + 7
// of qkv_append_kernel's wave hold, so the sum of squares runs through the same
// additions, a rotation pair (j, j + hd/2) is in one lane, and every load and
// store is a run of 32 bytes (16 for a K chunk).  No loop over positions and no
// barrier on the Q and K paths: one round trip to memory instead of eight.
template <int NJ>
__device__ __forceinline__ void qkv_append_row8(const QkvAppendArgs& a, unsigned char* smem, uint32_t h,
                                                uint32_t sess, uint32_t ctx_pad, uint32_t p_begin,
                                                uint32_t np, uint32_t row0)
{
#pragma clang fp contract(off)
    constexpr uint32_t HD = 64 * NJ;
    const uint32_t i = threadIdx.x >> 3, part = threadIdx.x & 7;
    const bool live = i < np;
    const uint32_t r = row0 + (live ? i : 0);
    const float* src = a.qkv + (size_t)r * a.ld + (size_t)h * HD + part * 8;
    const bool is_v = h >= a.nq + a.nkv, is_q = h < a.nq;
    float x[NJ][8];
    row8_head_values<NJ>(x, src, live, is_v ? nullptr : (is_q ? a.q_norm : a.k_norm), is_v && a.v_norm != 0,
                         a.eps, part, is_v ? nullptr : a.cos_sin + (size_t)r * a.n_rot * 2, a.n_rot);

    if (is_v) {
        const uint32_t kvh = h - a.nq - a.nkv;
        uint16_t (*tile)[kVBlock + 2] = reinterpret_cast<uint16_t (*)[kVBlock + 2]>(smem);
        if (live) {
#pragma unroll
            for (int c = 0; c < NJ; c++)
#pragma unroll
                for (int e = 0; e < 8; e++) tile[c * 64 + part * 8 + e][i] = f32_to_f16_trunc(x[c][e]);
        }
        __syncthreads();
        uint16_t* vt = a.vt[sess];
        for (uint32_t idx = threadIdx.x; idx < HD * np; idx += 256) {
            const uint32_t d = idx / np, ii = idx % np;
            vt[vt_offset(kvh, ctx_pad, p_begin + ii, d, HD)] = tile[d][ii];
        }
        return;
    }

    if (!live) return;
    if (is_q && a.q16_out != nullptr) {
        // what the prefill kernel would make of the F32 row itself (q_scaled_f16)
        uint16_t* dst = a.q16_out + ((size_t)r * a.nq + h) * HD + part * 8;
#pragma unroll
        for (int c = 0; c < NJ; c++) {
            const half4 lo = q_scaled_f16(make_float4(x[c][0], x[c][1], x[c][2], x[c][3]), a.q16_scale);
            const half4 hi = q_scaled_f16(make_float4(x[c][4], x[c][5], x[c][6], x[c][7]), a.q16_scale);
            *reinterpret_cast<half4*>(dst + c * 64) = lo;
            *reinterpret_cast<half4*>(dst + c * 64 + 4) = hi;
        }
    } else if (is_q) {
        float* dst = a.q_out + ((size_t)r * a.nq + h) * HD + part * 8;
#pragma unroll
        for (int c = 0; c < NJ; c++) {
            *reinterpret_cast<f32x4*>(dst + c * 64) = f32x4{x[c][0], x[c][1], x[c][2], x[c][3]};
            *reinterpret_cast<f32x4*>(dst + c * 64 + 4) = f32x4{x[c][4], x[c][5], x[c][6], x[c][7]};
        }
    } else {
        uint16_t* k = a.k[sess];
        const uint32_t kvh = h - a.nq, p = p_begin + i;
#pragma unroll
        for (int c = 0; c < NJ; c++) {
            uint32_t w[4];
#pragma unroll
            for (int e = 0; e < 4; e++)
                w[e] = (uint32_t)f32_to_f16_trunc(x[c][2 * e]) | ((uint32_t)f32_to_f16_trunc(x[c][2 * e + 1]) << 16);
            *reinterpret_cast<u32x4*>(k + k_offset(kvh, ctx_pad, p, c * 64 + part * 8, HD)) =
                u32x4{w[0], w[1], w[2], w[3]};
        }
    }
}

__global__ __launch_bounds__(256) void qkv_append_kernel(const QkvAppendArgs a)
{
#pragma clang fp contract(off)
    extern __shared__ __attribute__((aligned(16))) unsigned char qkv_smem[];
    const uint32_t h = blockIdx.y, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const uint32_t hd = a.hd, half = hd / 2;
    const uint32_t sess = a.per_session ? blockIdx.x : 0;
    const uint32_t pos0 = a.pos[sess], ctx_pad = a.ctx_pad[sess];
    // positions of this workgroup: [p_begin, p_end), rows row0 ...
    uint32_t p_begin, p_end, row0;
    if (a.per_session) {
        p_begin = pos0;
        p_end = pos0 + 1;
        row0 = blockIdx.x;
    } else {
        const uint32_t blk = pos0 / kVBlock + blockIdx.x;
        p_begin = max(blk * kVBlock, pos0);
        p_end = min((blk + 1) * kVBlock, pos0 + a.rows);
        row0 = p_begin - pos0;
    }
    const uint32_t np = p_end - p_begin;                  // 1 .. 32

    if (a.row8 == 2) return qkv_append_row8<2>(a, qkv_smem, h, sess, ctx_pad, p_begin, np, row0);
    if (a.row8 == 4) return qkv_append_row8<4>(a, qkv_smem, h, sess, ctx_pad, p_begin, np, row0);

    if (h >= a.nq + a.nkv) {
        // V head: rows -> F16 -> tile[d][position in block] -> runs along positions
        const uint32_t kvh = h - a.nq - a.nkv;
        uint16_t (*tile)[kVBlock + 2] = reinterpret_cast<uint16_t (*)[kVBlock + 2]>(qkv_smem);
        for (uint32_t i = wave; i < np; i += 4) {
            const float* src = a.qkv + (size_t)(row0 + i) * a.ld + (size_t)h * hd;
            float inv_rms = 1.0f;
            if (a.v_norm) {                               // wave-uniform
                float ss = 0.f;
                for (uint32_t j = lane; j < hd; j += 64) {
                    const float v = src[j];
                    ss += v * v;
                }
                ss = wave_sum_f32(ss);
                inv_rms = 1.0f / sqrtf(ss / (float)hd + a.eps);
            }
            for (uint32_t j = lane; j < hd; j += 64)
                tile[j][i] = f32_to_f16_trunc(a.v_norm ? src[j] * inv_rms : src[j]);
        }
        __syncthreads();
        uint16_t* vt = a.vt[sess];
        for (uint32_t idx = threadIdx.x; idx < hd * np; idx += 256) {
            const uint32_t d = idx / np, i = idx % np;
            vt[vt_offset(kvh, ctx_pad, p_begin + i, d, hd)] = tile[d][i];
        }
        return;
    }

    const bool is_q = h < a.nq;
    const float* nw = is_q ? a.q_norm : a.k_norm;
    float* s = reinterpret_cast<float*>(qkv_smem) + (size_t)wave * hd;   // this wave's row
    // the same trip count in every wave (the barrier needs it); a wave past its
    // positions repeats the block's last one and stores nothing
    for (uint32_t i0 = 0; i0 < np; i0 += 4) {
        const bool mine = i0 + wave < np;
        const uint32_t i = mine ? i0 + wave : np - 1;
        const uint32_t r = row0 + i;
        const float* src = a.qkv + (size_t)r * a.ld + (size_t)h * hd;
        float ss = 0.f;
        for (uint32_t j = lane; j < hd; j += 64) {
            const float v = src[j];
            s[j] = v;
            ss += v * v;
        }
        if (nw) {
            ss = wave_sum_f32(ss);
            const float inv_rms = 1.0f / sqrtf(ss / (float)hd + a.eps);
            for (uint32_t j = lane; j < hd; j += 64) s[j] = s[j] * inv_rms * nw[j];
        }
        __syncthreads();
        const float* cs = a.cos_sin + (size_t)r * a.n_rot * 2;
        for (uint32_t j = lane; j < half; j += 64) {
            const float x0 = s[j], x1 = s[j + half];
            float y0 = x0, y1 = x1;
            if (j < a.n_rot) {
                const float c = cs[2 * j], sn = cs[2 * j + 1];
                const float a0 = x0 * c, b0 = x1 * sn, a1 = x0 * sn, b1 = x1 * c;
                y0 = a0 - b0;
                y1 = a1 + b1;
            }
            if (!mine) continue;
            if (is_q) {
                float* dst = a.q_out + ((size_t)r * a.nq + h) * hd;
                dst[j] = y0;
                dst[j + half] = y1;
            } else {
                uint16_t* k = a.k[sess];
                const uint32_t kvh = h - a.nq, p = p_begin + i;
                k[k_offset(kvh, ctx_pad, p, j, hd)] = f32_to_f16_trunc(y0);
                k[k_offset(kvh, ctx_pad, p, j + half, hd)] = f32_to_f16_trunc(y1);
            }
        }
        __syncthreads();                                  // s is rewritten by the next position
    }
}

// act[r][j] = silu(gu[r][j]) * gu[r][ffn + j],  silu(x) = x / (1 + exp(-x))
__global__ __launch_bounds__(256) void swiglu_rows_kernel(const float* __restrict__ gu, uint32_t ld,
                                                          float* __restrict__ act, uint32_t ldo,
                                                          uint32_t rows, uint32_t ffn)
{
    const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= (size_t)rows * ffn) return;
    const uint32_t r = (uint32_t)(idx / ffn), j = (uint32_t)(idx % ffn);
    const float g = gu[(size_t)r * ld + j], u = gu[(size_t)r * ld + ffn + j];
    act[(size_t)r * ldo + j] = silu_mul(g, u);
}

}  // namespace wr
