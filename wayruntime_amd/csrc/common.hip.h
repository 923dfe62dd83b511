// Shared device helpers and the HBM layout of the per-session KV cache.
//
// Layout of one layer of one session (all F16 bit patterns):
//
//   K   [nkv][ctx_pad][hd]            head-major, one row per cached position
//   Vt  [nkv][ctx_pad/32][hd][32]     head-major, transposed in blocks of 32
//                                     positions: the 32 values of one
//                                     dimension are contiguous (64 bytes)
//
// ctx_pad is max_ctx rounded up to 32.  Head-major K makes the stream one
// (session, kv head) workgroup reads fully contiguous.  The blocked transpose
// of V puts the contraction index of P.V (positions) innermost, which is what
// an MFMA operand wants, so neither kernel has to transpose V on the fly.
// The slab is zero-filled at creation; rows above the caller's cursor are
// never trusted (kernels mask them), only required to be addressable.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace wr {

constexpr int kVBlock = 32;           // positions per transposed V block

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half4 __attribute__((ext_vector_type(4)));
typedef _Float16 half2v __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

// Truncating float32 -> binary16, the rule of the reference's cache append
// (reference: src/core/quant.c:121-136): drop the low 13 mantissa bits, flush
// results below the normal range to signed zero, saturate overflow and NaN to
// signed infinity.  Integer arithmetic only, so it is bit-exact by construction.
__device__ __forceinline__ uint16_t f32_to_f16_trunc(float f)
{
    const uint32_t bits = __float_as_uint(f);
    const uint32_t sign = (bits >> 16) & 0x8000u;
    const int32_t e = (int32_t)((bits >> 23) & 0xFFu) - 112;
    const uint32_t mant = (bits >> 13) & 0x3FFu;
    uint32_t r = sign | ((uint32_t)e << 10) | mant;
    if (e <= 0) r = sign;
    if (e >= 31) r = sign | 0x7C00u;
    return (uint16_t)r;
}

__device__ __forceinline__ size_t k_row_offset(uint32_t kvh, uint32_t ctx_pad, uint32_t pos,
                                               uint32_t hd)
{
    return ((size_t)kvh * ctx_pad + pos) * hd;
}

// element offset of (kvh, pos, d) inside Vt
__device__ __forceinline__ size_t vt_offset(uint32_t kvh, uint32_t ctx_pad, uint32_t pos,
                                            uint32_t d, uint32_t hd)
{
    const uint32_t blocks = ctx_pad / kVBlock;
    return (((size_t)kvh * blocks + pos / kVBlock) * hd + d) * kVBlock + (pos % kVBlock);
}

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

__device__ __forceinline__ float wave_xor_f32(float v, int mask)
{
    return __shfl_xor(v, mask, 64);
}

// The value lane ^ 32 holds, without going through LDS: v_permlane32_swap
// exchanges the upper half of its first operand with the lower half of its
// second, so with the same value in both the two results together hold, in
// every lane, this lane's value and its partner's.
__device__ __forceinline__ float wave_partner32(float v)
{
    const uint32_t u = __float_as_uint(v);
    const auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
    const bool upper = (__builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u)) & 32u) != 0;
    return __uint_as_float(upper ? r[0] : r[1]);
}

// max / sum of this lane's value and lane ^ 32's (order-insensitive, so no
// select is needed)
__device__ __forceinline__ float wave_pair32_max(float v)
{
    const uint32_t u = __float_as_uint(v);
    const auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
    return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}

__device__ __forceinline__ float wave_pair32_sum(float v)
{
    const uint32_t u = __float_as_uint(v);
    const auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

}  // namespace wr
