// Shared device helpers and the HBM layout of the per-session KV cache.
//
// Layout of one layer of one session (all F16 bit patterns):
//
//   K   [nkv][ctx_pad/32][2][hdp/8][16][8]   head-major, in tiles of 32 positions
//   Vt  [nkv][ctx_pad/32][hd][32]            head-major, transposed in blocks of
//                                            32 positions: the 32 values of one
//                                            dimension are contiguous (64 bytes)
//
// ctx_pad is max_ctx rounded up to 32; hdp is head_dim rounded up to 8.
//
// A K tile is stored in the order the decode kernel's matrix instruction eats
// it.  Position p of a tile belongs to half t = (p >> 2) & 1 and slot
// m = (p >> 3) * 4 + (p & 3) of that half; inside a half, the 16-byte chunk
// c = d / 8 of all 16 slots is contiguous: unit (t, c, m) sits at
// ((t * hdp/8 + c) * 16 + m) * 16 bytes.  One MFMA operand load (row m of 16,
// lane group g reads chunk 4s + g) is then 64 lanes x 16 bytes = one contiguous
// KiB.  With position-major rows the same load touches sixteen rows for 64
// bytes each, and a compute unit streams that pattern at a third of the rate
// (33 against 80-90 GB/s measured for one workgroup), which is what a ragged
// batch's longest workgroups and a single session's few workgroups run at.
// The halves and slots are the permutation that leaves each lane group's
// scores on eight consecutive positions, the order Vt is read in.
//
// The blocked transpose of V puts the contraction index of P.V (positions)
// innermost, which is what an MFMA operand wants, so neither kernel has to
// transpose V on the fly.  The slab is zero-filled at creation; rows above the
// caller's cursor are never trusted (kernels mask them), only required to be
// addressable.
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

constexpr int kKTile = 32;            // positions per K tile

__host__ __device__ __forceinline__ uint32_t k_padded_hd(uint32_t hd) { return (hd + 7u) & ~7u; }

// half and slot of a position inside its K tile, and back
__device__ __forceinline__ uint32_t k_tile_half(uint32_t p) { return (p >> 2) & 1u; }
__device__ __forceinline__ uint32_t k_tile_slot(uint32_t p) { return ((p >> 3) << 2) | (p & 3u); }
__device__ __forceinline__ uint32_t k_tile_pos(uint32_t half, uint32_t slot)
{
    return ((slot >> 2) << 3) | (half << 2) | (slot & 3u);
}

// element offset of (kvh, pos, d) inside K
__device__ __forceinline__ size_t k_offset(uint32_t kvh, uint32_t ctx_pad, uint32_t pos, uint32_t d,
                                           uint32_t hd)
{
    const uint32_t hdp = k_padded_hd(hd);
    const uint32_t p = pos % kKTile;
    const uint32_t unit = (k_tile_half(p) * (hdp / 8) + d / 8) * 16 + k_tile_slot(p);
    return ((size_t)kvh * ctx_pad + (pos - p)) * hdp + (size_t)unit * 8 + (d & 7u);
}

// element offset of (kvh, pos, d) inside Vt
__device__ __forceinline__ size_t vt_offset(uint32_t kvh, uint32_t ctx_pad, uint32_t pos,
                                            uint32_t d, uint32_t hd)
{
    const uint32_t blocks = ctx_pad / kVBlock;
    return (((size_t)kvh * blocks + pos / kVBlock) * hd + d) * kVBlock + (pos % kVBlock);
}

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// silu(g) * u, silu(g) = g / (1 + exp(-g)) (reference: src/core/kernels.c:963-967),
// with exp(-g) = 2^(-g log2 e) from the hardware's exp2 and the reciprocal from
// v_rcp_f32: six instructions where expf and an IEEE division are about forty,
// in kernels whose time IS their instruction count (the gated products of a decode
// step spend a microsecond of vector ALU on sixteen of these per lane, and the
// unrolled library calls are a third of the code they have to fetch).  Relative
// error about 2^-23 + |g| 2^-24 (the rounded product in the exponent): for the
// |g| < 20 that contribute anything, within 1.3e-6.  One definition for every
// kernel that gates: the fused and the separate forms must agree bit for bit.
__device__ __forceinline__ float silu_mul(float g, float u)
{
    const float e = __builtin_amdgcn_exp2f(-g * 1.44269504088896340736f);
    const float sig = __builtin_amdgcn_rcpf(1.0f + e);        // e = inf: 0
    return (g * sig) * u;
}

// The value lane ^ mask holds, mask a power of two below 64.  Through the
// vector ALU's own lane crossings where there is one (a swap of wave halves or
// of rows of sixteen, a rotation inside a row, a quad permutation), not through
// the LDS crossbar: a reduction over the wave is six of these in a dependent
// chain, each about a hundred cycles by way of ds_bpermute and about ten this
// way, and the kernels of a decode step are chains of exactly such things.  The
// partner is the same lane either way, so every sum keeps its bits.  (Callers
// pass literal masks or unrolled loop counters: the switch folds away.)
__device__ __forceinline__ float wave_xor_f32(float v, int mask)
{
    const uint32_t u = __float_as_uint(v);
    const uint32_t lane = __builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u));
    switch (mask) {
    case 32: {
        const auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
        return __uint_as_float((lane & 32u) ? r[0] : r[1]);
    }
    case 16: {
        const auto r = __builtin_amdgcn_permlane16_swap(u, u, false, false);
        return __uint_as_float((lane & 16u) ? r[0] : r[1]);
    }
    case 8:                                               // row_ror:8
        return __int_as_float(__builtin_amdgcn_update_dpp(0, (int)u, 0x128, 0xF, 0xF, false));
    case 4: {
        // banks 0 and 2 of a row (lanes 0-3, 8-11) take the lane four up (row_shl:4),
        // banks 1 and 3 the lane four down (row_shr:4)
        const int up = __builtin_amdgcn_update_dpp(0, (int)u, 0x104, 0xF, 0x5, false);
        return __int_as_float(__builtin_amdgcn_update_dpp(up, (int)u, 0x114, 0xF, 0xA, false));
    }
    case 2:                                               // quad_perm:[2,3,0,1]
        return __int_as_float(__builtin_amdgcn_update_dpp(0, (int)u, 0x4E, 0xF, 0xF, false));
    case 1:                                               // quad_perm:[1,0,3,2]
        return __int_as_float(__builtin_amdgcn_update_dpp(0, (int)u, 0xB1, 0xF, 0xF, false));
    default:
        return __shfl_xor(v, mask, 64);
    }
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

// Tells the compiler that a pointer is the same in every lane (keeps the
// arithmetic on it in scalar registers).
__device__ __forceinline__ const unsigned char* uniform_ptr(const unsigned char* p)
{
    const uint64_t b = reinterpret_cast<uint64_t>(p);
    // the builtin returns a signed int: widen through uint32_t, or a low half
    // with its top bit set would smear ones over the high half
    const uint32_t lo = (uint32_t)__builtin_amdgcn_readfirstlane((uint32_t)b);
    const uint32_t hi = (uint32_t)__builtin_amdgcn_readfirstlane((uint32_t)(b >> 32));
    return reinterpret_cast<const unsigned char*>((uint64_t)lo | ((uint64_t)hi << 32));
}

// One 64 x 16-byte load from global memory straight into LDS.  The LDS address
// (wave-uniform, in M0) receives lane 0's 16 bytes, lane i's go 16*i further.
__device__ __forceinline__ void lds_direct_load(uint32_t lds_addr, const unsigned char* base,
                                                uint32_t lane_off)
{
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                 :
                 : "s"(lds_addr), "v"(lane_off), "s"(base)
                 : "memory");
}

// Four query values multiplied by the softmax scale (times log2 e) and rounded
// to binary16: what the prefill kernel's first contraction takes.  One
// function for the kernel that is handed F32 rows and for the row kernel that
// writes the rounded form for it, so that the two give the same bits.
__device__ __forceinline__ half4 q_scaled_f16(float4 x, float qscale)
{
#pragma clang fp contract(off)
    // Two roundings, product then conversion.  The products pass through an empty
    // statement: where it cannot pair two conversions the compiler otherwise
    // folds product and conversion into one mixed-precision instruction
    // (v_fma_mixlo_f16), which rounds once and differs in the tie cases.
    float p0 = x.x * qscale, p1 = x.y * qscale, p2 = x.z * qscale, p3 = x.w * qscale;
    asm("" : "+v"(p0), "+v"(p1), "+v"(p2), "+v"(p3));
    half4 h;
    h[0] = (_Float16)p0;
    h[1] = (_Float16)p1;
    h[2] = (_Float16)p2;
    h[3] = (_Float16)p3;
    return h;
}

// Workgroup barrier that waits for this wave's LDS traffic only.  __syncthreads()
// also drains outstanding global loads, which would pull the tiles being
// prefetched for later iterations back onto the critical path.
__device__ __forceinline__ void lds_barrier()
{
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

}  // namespace wr
