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

// What a lane reads for one head of one position: its 8 NJ elements, the
// norm's weights for them and the (cos, sin) pairs of its rotation pairs.  All
// three are asked for together, before anything is waited for: read where they
// are used they are three dependent trips to memory (row -> sum -> weights ->
// rotation table), and a caller with other loads to start (the decode kernel's
// tiles) can start them in between.
template <int NJ>
struct Row8Loads {
    f32x4 x[NJ][2];
    f32x4 w[NJ][2];
    f32x4 t[NJ / 2 > 0 ? NJ / 2 : 1][4];
};

// src: the head's row + 8 part; nw: the norm's weight vector or null; cs: the
// position's (cos, sin) table or null; n_rot a multiple of eight.  EVERY load
// is issued whatever the lane goes on to use, from an address that is valid:
// without weights or a table the head's own row is read in their place (its
// 64 NJ floats cover every offset used below), and pairs past n_rot read the
// table's last eight.  Loads that are only sometimes issued would make the
// compiler wait for everything in flight where it now waits for these alone.
template <int NJ>
__device__ __forceinline__ void row8_head_request(Row8Loads<NJ>& L, const float* src, const float* nw,
                                                  uint32_t part, const float* cs, uint32_t n_rot)
{
    const float* head = src - part * 8;
    const float* nwp = nw != nullptr ? nw : head;
    const float* csp = cs != nullptr ? cs : head;
    const uint32_t last = (cs != nullptr && n_rot >= 8) ? n_rot - 8 : 64u * (NJ / 2 > 0 ? NJ / 2 : 1) - 8;
#pragma unroll
    for (int c = 0; c < NJ; c++) {
        L.x[c][0] = *reinterpret_cast<const f32x4*>(src + c * 64);
        L.x[c][1] = *reinterpret_cast<const f32x4*>(src + c * 64 + 4);
    }
#pragma unroll
    for (int c = 0; c < NJ; c++) {
        L.w[c][0] = *reinterpret_cast<const f32x4*>(nwp + c * 64 + part * 8);
        L.w[c][1] = *reinterpret_cast<const f32x4*>(nwp + c * 64 + part * 8 + 4);
    }
#pragma unroll
    for (int c = 0; c < NJ / 2; c++) {
        const uint32_t j0 = min((uint32_t)(c * 64 + part * 8), last);
#pragma unroll
        for (int q = 0; q < 4; q++) L.t[c][q] = *reinterpret_cast<const f32x4*>(csp + 2 * j0 + 4 * q);
    }
}

// x: the head's elements of this lane from what row8_head_request read.
// norm: RMSNorm with the weights read (weightless: without weights, the V heads
// of the Gemma family); rotate: apply the rotation read.  All eight lanes of a
// position must call together with the same flags (the sum crosses them).
template <int NJ>
__device__ __forceinline__ void row8_head_finish(float (&x)[NJ][8], const Row8Loads<NJ>& L, bool norm,
                                                 bool weightless, float eps, uint32_t part, bool rotate,
                                                 uint32_t n_rot)
{
#pragma clang fp contract(off)
    constexpr uint32_t HD = 64 * NJ;
#pragma unroll
    for (int c = 0; c < NJ; c++)
#pragma unroll
        for (int e = 0; e < 4; e++) {
            x[c][e] = L.x[c][0][e];
            x[c][4 + e] = L.x[c][1][e];
        }
    // No branches from here on (values are selected, not skipped): a load whose
    // value is only used inside a branch gets moved down into that branch,
    // behind whatever the caller has asked for in between.
    {
        float s[8];
#pragma unroll
        for (int e = 0; e < 8; e++) {
            float ss = 0.f;
#pragma unroll
            for (int c = 0; c < NJ; c++) ss += x[c][e] * x[c][e];
            s[e] = ss;
        }
        const float inv_rms = 1.0f / sqrtf(row8_sum_f32(s) / (float)HD + eps);
        const bool scaled = weightless || norm;
#pragma unroll
        for (int c = 0; c < NJ; c++) {
#pragma unroll
            for (int e = 0; e < 4; e++) {
                // weightless: times one, which changes no bit
                const float w0 = weightless ? 1.0f : L.w[c][0][e], w1 = weightless ? 1.0f : L.w[c][1][e];
                const float y0 = x[c][e] * inv_rms * w0, y1 = x[c][4 + e] * inv_rms * w1;
                x[c][e] = scaled ? y0 : x[c][e];
                x[c][4 + e] = scaled ? y1 : x[c][4 + e];
            }
        }
    }
    // rotation of the pairs (j, j + hd/2), j = 64 c + 8 part + e for c < NJ / 2
#pragma unroll
    for (int c = 0; c < NJ / 2; c++) {
        const uint32_t j0 = c * 64 + part * 8;
        const bool turn = rotate && j0 < n_rot;
#pragma unroll
        for (int q = 0; q < 4; q++) {
            const f32x4 t = L.t[c][q];
#pragma unroll
            for (int u = 0; u < 2; u++) {
                const float co = t[2 * u], sn = t[2 * u + 1];
                const float x0 = x[c][2 * q + u], x1 = x[c + NJ / 2][2 * q + u];
                const float a0 = x0 * co, b0 = x1 * sn, a1 = x0 * sn, b1 = x1 * co;
                x[c][2 * q + u] = turn ? a0 - b0 : x0;
                x[c + NJ / 2][2 * q + u] = turn ? a1 + b1 : x1;
            }
        }
    }
}

// Both steps in one call.  x: the head's elements of this lane, read from src
// (the head's row + 8 part) when live, zero otherwise.  nw: the norm's weight
// vector or null; weightless: an RMSNorm without weights; cs: the position's
// (cos, sin) table or null for no rotation.  All eight lanes of a position must
// call together.
template <int NJ>
__device__ __forceinline__ void row8_head_values(float (&x)[NJ][8], const float* src, bool live,
                                                 const float* nw, bool weightless, float eps, uint32_t part,
                                                 const float* cs, uint32_t n_rot)
{
    Row8Loads<NJ> L;
    if (live) {
        row8_head_request<NJ>(L, src, nw, part, cs, n_rot);
    } else {
#pragma unroll
        for (int c = 0; c < NJ; c++) L.x[c][0] = L.x[c][1] = L.w[c][0] = L.w[c][1] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int c = 0; c < NJ / 2; c++)
#pragma unroll
            for (int q = 0; q < 4; q++) L.t[c][q] = f32x4{0.f, 0.f, 0.f, 0.f};
    }
    row8_head_finish<NJ>(x, L, nw != nullptr, weightless, eps, part, live && cs != nullptr, n_rot);
}

}  // namespace wr
