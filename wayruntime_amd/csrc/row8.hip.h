// A head's values of one position, normalised and rotated, with eight lanes per
// position: the arithmetic shared by the cache append of whole rows
// (qkv_append_kernel) and the decode kernel that does the new row's append
// itself.  Lane `part` of the eight holds the elements 64 c + 8 part + e
// (c < NJ = hd / 64, e < 8): a rotation pair (j, j + hd/2) is in one lane, every
// load is a run of 32 bytes, and the sum of squares runs through the additions
// of a wave sum over the row (below), so the bits are those of the one-wave-
// per-row kernels (reference: per-head RMSNorm src/core/session.c:459-474 over
// src/core/kernels.c:1276-1316, rotation kernels.c:1356-1412).
#pragma once

#include "common.hip.h"

namespace wr {

// wave_sum_f32 over a row whose 64 partial sums sit eight to a lane in eight
// neighbouring lanes (lane `part` of the eight holds partial sums 8 part ..
// 8 part + 7).  The wave sum pairs partial sums 32, 16, 8, 4, 2, 1 apart, in
// that order: the first three are the lanes 4, 2, 1 away, the last three are
// in the lane.  The same additions, hence the same bits.
__device__ __forceinline__ float row8_sum_f32(float (&s)[8])
{
#pragma unroll
    for (int m = 4; m >= 1; m >>= 1)
#pragma unroll
        for (int e = 0; e < 8; e++) s[e] += wave_xor_f32(s[e], m);
    const float b0 = s[0] + s[4], b1 = s[1] + s[5], b2 = s[2] + s[6], b3 = s[3] + s[7];
    const float c0 = b0 + b2, c1 = b1 + b3;
    return c0 + c1;
}

// x: the head's elements of this lane, read from src (the head's row + 8 part)
// when live, zero otherwise.  nw: the norm's weight vector or null; weightless:
// an RMSNorm without weights (V heads of the Gemma family); cs: the position's
// (cos, sin) table or null for no rotation; n_rot a multiple of eight.  All
// eight lanes of a position must call together (the sum crosses them).
template <int NJ>
__device__ __forceinline__ void row8_head_values(float (&x)[NJ][8], const float* src, bool live,
                                                 const float* nw, bool weightless, float eps, uint32_t part,
                                                 const float* cs, uint32_t n_rot)
{
#pragma clang fp contract(off)
    constexpr uint32_t HD = 64 * NJ;
#pragma unroll
    for (int c = 0; c < NJ; c++) {
        f32x4 lo = {0.f, 0.f, 0.f, 0.f}, hi = lo;
        if (live) {
            lo = *reinterpret_cast<const f32x4*>(src + c * 64);
            hi = *reinterpret_cast<const f32x4*>(src + c * 64 + 4);
        }
#pragma unroll
        for (int e = 0; e < 4; e++) {
            x[c][e] = lo[e];
            x[c][4 + e] = hi[e];
        }
    }
    if (weightless || nw != nullptr) {                    // uniform over the eight lanes
        float s[8];
#pragma unroll
        for (int e = 0; e < 8; e++) {
            float ss = 0.f;
#pragma unroll
            for (int c = 0; c < NJ; c++) ss += x[c][e] * x[c][e];
            s[e] = ss;
        }
        const float inv_rms = 1.0f / sqrtf(row8_sum_f32(s) / (float)HD + eps);
#pragma unroll
        for (int c = 0; c < NJ; c++) {
            if (weightless) {
#pragma unroll
                for (int e = 0; e < 8; e++) x[c][e] = x[c][e] * inv_rms;
            } else {
                const f32x4 wl = *reinterpret_cast<const f32x4*>(nw + c * 64 + part * 8);
                const f32x4 wh = *reinterpret_cast<const f32x4*>(nw + c * 64 + part * 8 + 4);
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    x[c][e] = x[c][e] * inv_rms * wl[e];
                    x[c][4 + e] = x[c][4 + e] * inv_rms * wh[e];
                }
            }
        }
    }
    if (cs == nullptr) return;
    // rotation of the pairs (j, j + hd/2), j = 64 c + 8 part + e for c < NJ / 2
#pragma unroll
    for (int c = 0; c < NJ / 2; c++) {
        const uint32_t j0 = c * 64 + part * 8;
        if (live && j0 < n_rot) {
#pragma unroll
            for (int q = 0; q < 4; q++) {
                const f32x4 t = *reinterpret_cast<const f32x4*>(cs + 2 * j0 + 4 * q);
#pragma unroll
                for (int u = 0; u < 2; u++) {
                    const float co = t[2 * u], sn = t[2 * u + 1];
                    const float x0 = x[c][2 * q + u], x1 = x[c + NJ / 2][2 * q + u];
                    const float a0 = x0 * co, b0 = x1 * sn, a1 = x0 * sn, b1 = x1 * co;
                    x[c][2 * q + u] = a0 - b0;
                    x[c + NJ / 2][2 * q + u] = a1 + b1;
                }
            }
        }
    }
}

}  // namespace wr
