// Causal prefill attention on the matrix cores for head dim 256
// (v_mfma_f32_32x32x16_f16, F32 accumulate).  MFMA-bound: 4 * nq * hd flops per
// (query row, visible key).
//
// Semantics: kernels_prefill.hip.h (reference: the prefill loop
// src/core/session.c:615-625 over src/core/kernels.c:1475-1523).
//
// The step of kernels_prefill_il.hip.h with the two wave sets dividing the head
// DIMENSIONS instead of the keys.  A wave that owned all 256 dimensions of its 32
// rows would hold 128 accumulator registers and a 64-register Q operand, which
// leaves no room for two waves per SIMD; here
//
//   workgroup = 8 waves = one KV head x 4 (head, 32-row block) pairs x 2 halves:
//   waves 0-3 own dimensions 0-127, waves 4-7 dimensions 128-255, of every tile.
//
// Per wave and tile:
//   S'^T[key][row] = K[key][own dims] . Q^T[own dims][row]    8 MFMAs (half the contraction)
//   the two halves' partial scores meet through LDS: S = S'(own) + S'(other)
//       (one addition of two floats, the same two in both waves, so both hold
//        the same bits and everything derived from them -- maximum, reference,
//        probabilities, normaliser -- is the same in both without more traffic)
//   online softmax on the 16 scores a lane holds
//   O^T[own dims][row] += Vt[own dims][key] . P^T[key][row]   8 MFMAs
// so a wave carries what a wave of the 128-dimension kernel carries (64
// accumulator registers, a 32-register Q operand), the matrix work per tile is
// not duplicated, the halves' outputs are disjoint and nothing is merged at the
// end.  Each half streams its own half of every K tile (two runs of 4 KiB in the
// cache's tile layout) and of every Vt block (8 KiB) into its own ring of three
// slots: the ring geometry, the slot permutations, the operand reads and the
// copy schedule are those of the 128-dimension kernel (SplitLds<128>).
//
// Step j.  On entry `cur` holds the wave's partial scores of tile j, kf the K
// operands of tile j+1; the other half's partial scores of tile j are in the
// exchange buffer of parity j.
//   first half:   the partial chain S'(j+1); behind its first links the scores of
//                 tile j are completed (sum of the two partials, row maximum,
//                 masks, reference), behind the others go the Vt operand reads of
//                 tile j and the exponentials and packs of S(j);
//   second half:  O^T += Vt(j).P(j)^T, and between the products the K operand
//                 reads of tile j+2, the step's copies and the partial scores of
//                 tile j+1 on their way to the exchange buffer of parity j+1;
//   one hardware barrier per step, as in the 128-dimension kernel: it publishes
//   the copies that have landed and the partial scores, and frees the ring slots
//   and the exchange buffer the next step overwrites.  A buffer of either parity
//   is written in one step, read in the next and written again in the step after
//   that, with a barrier between each two: nothing here depends on how far one
//   wave runs ahead of another.
//
// The chain of tile j+1 has started (from the block of -m) when the reference of
// tile j is settled.  If that moves m by delta, the scores of tile j+1 come out
// delta too high; the move leaves delta in `pend`, and the completion of tile j+1
// subtracts it (rare, wave-uniform branch; the same in both halves).
//
// The halves share the accumulated reference: the chain of the lower half starts
// from the block of -m, the upper half's from zero, and their sum is S - m.
#pragma once

#include "kernels_prefill_il.hip.h"

namespace wr {

constexpr int kIldHalf = 128;                             // dimensions a wave owns

struct IldLds {
    using L = SplitLds<kIldHalf>;
    static constexpr int X_OFF = 2 * L::SET_BYTES;        // exchange of partial scores: [2 parities][4 pairs][2 halves][16][64] floats
    static constexpr int X_WAVE = 16 * 64 * 4;
    static constexpr int X_PARITY = 8 * X_WAVE;
    static constexpr int X_BYTES = 2 * X_PARITY;
    // rows leave through LDS, row-major, once the rings are quiet: [8 waves][32][128 + 4] floats from 0
    static constexpr int O_WAVE = 32 * (kIldHalf + 4) * 4;
    static constexpr int TOTAL = (X_OFF + X_BYTES > 8 * O_WAVE) ? X_OFF + X_BYTES : 8 * O_WAVE;
    static_assert(TOTAL <= 160 * 1024, "fits a CU's LDS");
};

constexpr size_t ild_smem_bytes() { return IldLds::TOTAL; }

// tile jt of the block (both halves walk every tile), clamped to its last one
__device__ __forceinline__ uint32_t ild_tile(const IlCtx<kIldHalf>& cx, uint32_t jt)
{
    return min(cx.t0 + jt, cx.t_last);
}

// One of this wave's two copies of its half of K tile jt / Vt block jt into ring
// slot SLOT.  A K tile of 256 dimensions is 16 KiB in the cache, a Vt block too;
// the half's share of the latter is contiguous, of the former two runs (one per
// half of the tile's keys) that gk_off addresses.
template <int SLOT>
__device__ __forceinline__ void ild_issue_k1(const IlCtx<kIldHalf>& cx, uint32_t jt, int u)
{
    using L = SplitLds<kIldHalf>;
    const unsigned char* src = cx.kbase + (size_t)ild_tile(cx, jt) * (2 * L::KTILE);
    lds_direct_load(cx.m0k + SLOT * L::KTILE + u * 4096, src + u * 128, cx.gk_off);
}

template <int SLOT>
__device__ __forceinline__ void ild_issue_v1(const IlCtx<kIldHalf>& cx, uint32_t jt, int u)
{
    using L = SplitLds<kIldHalf>;
    const unsigned char* src = cx.vtbase + (size_t)ild_tile(cx, jt) * (2 * L::VTILE);
    lds_direct_load(cx.m0v + SLOT * L::VTILE + u * 4096, src + u * 4096, cx.gv_off);
}

template <int SLOT>
__device__ __forceinline__ void ild_issue_k(const IlCtx<kIldHalf>& cx, uint32_t jt)
{
    ild_issue_k1<SLOT>(cx, jt, 0);
    ild_issue_k1<SLOT>(cx, jt, 1);
}

template <int SLOT>
__device__ __forceinline__ void ild_issue_v(const IlCtx<kIldHalf>& cx, uint32_t jt)
{
    ild_issue_v1<SLOT>(cx, jt, 0);
    ild_issue_v1<SLOT>(cx, jt, 1);
}

// il_patch_tail for this kernel's tile walk.
template <int SLOT>
__device__ __forceinline__ void ild_patch_tail(unsigned char* smem, const IlCtx<kIldHalf>& cx, uint32_t jt,
                                               int sub, int lane, uint32_t kv_valid)
{
    using L = SplitLds<kIldHalf>;
    const uint32_t tile = ild_tile(cx, jt);
    if (tile < cx.tail_tile) return;
#pragma unroll
    for (int u = 0; u < L::NL; u++) {
        const int q = sub + 4 * u;
        const int row = q * 16 + lane / 4;                // Vt row (dimension of the half)
        const int c = (lane & 3) ^ L::fv(row);            // key chunk this slot holds
        const uint32_t key0 = tile * kTileKeys + c * 8;
        u32x4* at = reinterpret_cast<u32x4*>(smem + cx.ring + L::V_IN_SET + SLOT * L::VTILE + q * 1024 +
                                             lane * 16);
        u32x4 v = *at;
        uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
        for (int e = 0; e < 4; e++) {
            if (key0 + 2 * e >= kv_valid) w[e] &= 0xFFFF0000u;
            if (key0 + 2 * e + 1 >= kv_valid) w[e] &= 0x0000FFFFu;
        }
        *at = u32x4{w[0], w[1], w[2], w[3]};
    }
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");    // the patch is in LDS before the barrier that follows
}

// il_move_reference with the upper half's chain starting from zero: only the
// lower half keeps -m in the block its chain starts from.
__device__ __forceinline__ void ild_move_reference(PrefillRows<kIldHalf>& R, IlCtx<kIldHalf>& cx, f32x16& negm,
                                                   f32x16& c, float tmax, bool jump, bool upper, float& pend,
                                                   uint32_t& pend_on)
{
    const bool unset = (R.m_run == -INFINITY);
    const float delta = jump ? tmax : 0.f;
    const float alpha = jump ? (unset ? 0.f : fast_exp2(-delta)) : 1.0f;
    R.l_run *= alpha;
#pragma unroll
    for (int dt = 0; dt < kIldHalf / 32; dt++)
#pragma unroll
        for (int r = 0; r < 16; r++) R.o[dt][r] *= alpha;
#pragma unroll
    for (int r = 0; r < 16; r++) asm volatile("v_sub_f32 %0, %0, %1" : "+v"(c[r]) : "v"(delta));
    // the chain in flight started from the reference as it was (from zero while
    // the row had none): its scores come out delta too high
    pend = delta;
    pend_on = 1;
    if (jump) R.m_run = (unset ? 0.f : R.m_run) + delta;
    const bool still = (R.m_run == -INFINITY);
    const float nm = (still || upper) ? 0.f : -R.m_run;
#pragma unroll
    for (int r = 0; r < 16; r++) asm volatile("v_mov_b32 %0, %1" : "+v"(negm[r]) : "v"(nm));
    asm volatile("v_mov_b32 %0, %1" : "+v"(cx.thr) : "v"(still ? -INFINITY : kLazyLog2));
}

__device__ __forceinline__ void ild_settle(PrefillRows<kIldHalf>& R, IlCtx<kIldHalf>& cx, f32x16& negm, f32x16& c,
                                           float tmax, bool upper, float& pend, uint32_t& pend_on)
{
    {
        const uint32_t u = __float_as_uint(tmax);
        const auto sw = __builtin_amdgcn_permlane32_swap(u, u, false, false);
        tmax = max3_raw(__uint_as_float(sw[0]), __uint_as_float(sw[1]), tmax);   // same in both lanes of a row
    }
    const bool jump = tmax > cx.thr;
    if (__builtin_amdgcn_ballot_w64(jump) != 0) ild_move_reference(R, cx, negm, c, tmax, jump, upper, pend, pend_on);
}

// The wave's partial scores into the exchange buffer, register r of lane l at
// float (r / 4 * 64 + l) * 4 + r % 4: 16-byte writes, lane-contiguous.
__device__ __forceinline__ void ild_send1(float* xw, const f32x16& c, int lane, int q4)
{
    *reinterpret_cast<f32x4*>(xw + (q4 * 64 + lane) * 4) = f32x4{c[4 * q4], c[4 * q4 + 1], c[4 * q4 + 2],
                                                              c[4 * q4 + 3]};
}

__device__ __forceinline__ void ild_send(float* xw, const f32x16& c, int lane)
{
#pragma unroll
    for (int q4 = 0; q4 < 4; q4++) ild_send1(xw, c, lane, q4);
}

// Step j of a wave (P == j % kRing, XB == j % 2).  On entry `cur` holds the
// wave's partial scores of tile j and kf the K operands of tile j+1; on exit
// `nxt` holds the partial scores of tile j+1 (sent to the exchange buffer of the
// other parity) and kf the operands of tile j+2.
template <int P, int XB>
__device__ __forceinline__ void ild_step(PrefillRows<kIldHalf>& R, IlCtx<kIldHalf>& cx, f32x16& negm, f32x16& cur,
                                         f32x16& nxt, u32x4 (&pop)[2], half8 (&kf)[8], half8 (&vf)[8],
                                         unsigned char* smem, float* xw, const float* xr_at, uint32_t j, int sub,
                                         int lane, int g, uint32_t kv_valid, bool upper, float& pend,
                                         uint32_t& pend_on)
{
    using L = SplitLds<kIldHalf>;
    constexpr int NS = 8, ND = 4;
    constexpr int VS = P;                 // slot of Vt of tile j
    constexpr int KS = (P + 2) % 3;       // slot of K of tile j+2
    constexpr int KC = (P + 1) % 3;       // K of tile j+4 replaces K of tile j+1 (read in the previous step)
    constexpr int VC = (P + 2) % 3;       // Vt of tile j+2 replaces Vt of tile j-1 (read in the previous step)
    constexpr int TS = (P + 1) % 3;       // slot of Vt of tile j+1, whose tail is patched once it has landed
    constexpr int XF = IldLds::X_PARITY / 4;              // floats between the two exchange buffers

    float psum = 0.f;
    const half2v ones = {(_Float16)1.0f, (_Float16)1.0f};
    auto pair = [&](int p) {
        // two exp2, one pack to F16, one dot product with (1, 1): the normaliser
        // is the sum of exactly the rounded values P.V multiplies
        const int r = 2 * p;
        const half2v ph = {(_Float16)fast_exp2(cur[r]), (_Float16)fast_exp2(cur[r + 1])};
        psum = __builtin_amdgcn_fdot2(ph, ones, psum, false);
        pop[r >> 3][(r & 7) >> 1] = __builtin_bit_cast(uint32_t, ph);
    };
    f32x4 xr[4];
#pragma unroll
    for (int q4 = 0; q4 < 4; q4++)
        xr[q4] = *reinterpret_cast<const f32x4*>(xr_at + XB * XF + (q4 * 64 + lane) * 4);
    // the completion of tile j's scores is spread behind links 1 to 3 (the other
    // half's partial scores, asked for above, are on their way during links 0 and
    // 1), so that neither wave of the SIMD leaves the matrix pipe waiting for it
    nxt = __builtin_amdgcn_mfma_f32_32x32x16_f16(kf[0], R.qop[0], negm, 0, 0, 0);
    vf[0] = *reinterpret_cast<const half8*>(cx.vop[0] + VS * L::VTILE);
    __builtin_amdgcn_sched_barrier(0);
    nxt = __builtin_amdgcn_mfma_f32_32x32x16_f16(kf[1], R.qop[1], nxt, 0, 0, 0);
    vf[1] = *reinterpret_cast<const half8*>(cx.vop[0] + VS * L::VTILE + 2048);
#pragma unroll
    for (int r = 0; r < 16; r++) cur[r] += xr[r >> 2][r & 3];
    if (pend_on) {
#pragma unroll
        for (int r = 0; r < 16; r++) asm volatile("v_sub_f32 %0, %0, %1" : "+v"(cur[r]) : "v"(pend));
        pend_on = 0;
    }
    __builtin_amdgcn_sched_barrier(0);
    nxt = __builtin_amdgcn_mfma_f32_32x32x16_f16(kf[2], R.qop[2], nxt, 0, 0, 0);
    vf[2] = *reinterpret_cast<const half8*>(cx.vop[0] + VS * L::VTILE + 2 * 2048);
    float tmax = il_max16(cur);
    if (j < cx.pl_lo || j > cx.pl_hi) {
        il_mask_special<kIldHalf>(R, cx, cur, cx.t0 + j, j, g, tmax);
        tmax = il_max16(cur);
    }
    __builtin_amdgcn_sched_barrier(0);
    nxt = __builtin_amdgcn_mfma_f32_32x32x16_f16(kf[3], R.qop[3], nxt, 0, 0, 0);
    vf[3] = *reinterpret_cast<const half8*>(cx.vop[0] + VS * L::VTILE + 3 * 2048);
    ild_settle(R, cx, negm, cur, tmax, upper, pend, pend_on);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int i = 4; i < NS; i++) {
        nxt = __builtin_amdgcn_mfma_f32_32x32x16_f16(kf[i], R.qop[i], nxt, 0, 0, 0);
        vf[i] = *reinterpret_cast<const half8*>(cx.vop[i / ND] + VS * L::VTILE + (i % ND) * 2048);
        pair(i - 4);
        if (i == NS - 1) pair(4);                         // the first half of P is complete before the first product
        __builtin_amdgcn_sched_barrier(0);
    }
    // products; the partial scores of tile j+1 leave behind the first of them, ahead
    // of the last operand reads, so that the wait before the barrier can name them
#pragma unroll
    for (int i = 0; i < NS; i++) {
        const int t = i / ND, dt = i % ND;
        R.o[dt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(vf[i], __builtin_bit_cast(half8, pop[t]), R.o[dt], 0, 0,
                                                           0);
        kf[i] = *reinterpret_cast<const half8*>(cx.kop[i] + KS * L::KTILE);
        if (i < 3) pair(5 + i);                           // the second half of P is first used by product 4
        if (i >= 1 && i <= 4) ild_send1(xw + (XB ^ 1) * XF, nxt, lane, i - 1);
        if (i < L::NL) ild_issue_k1<KC>(cx, j + 4, i);
        else if (i < 2 * L::NL) ild_issue_v1<VC>(cx, j + 2, i - L::NL);
        __builtin_amdgcn_sched_barrier(0);
    }
    R.l_run += psum;
    // all copies but this step's have landed: K of tile j+3 and Vt of tile j+1,
    // which the next step reads once the barrier has published them
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * L::NL) : "memory");
    ild_patch_tail<TS>(smem, cx, j + 1, sub, lane, kv_valid);
    __builtin_amdgcn_sched_barrier(0);
    // LDS operations complete in the order issued: with at most the three operand
    // reads issued after the last piece of the partial scores outstanding, those
    // are in the exchange buffer (the operand reads' slot is not refilled before
    // the next step's products, long after the next chain has consumed them).
    // The last piece leaves with product 4, and products 5, 6 and 7 each issue one
    // operand read behind a scheduling barrier that nothing crosses: three reads
    // follow it whatever the scheduler does inside a product's group.
    asm volatile("s_waitcnt lgkmcnt(3)\n\ts_barrier" ::: "memory");
    __builtin_amdgcn_sched_barrier(0);
}

// One position block.
__device__ __forceinline__ void ild_block(const PrefillArgs& a, unsigned char* smem, uint32_t pb, uint32_t kvh,
                                          uint32_t hc, const unsigned char* kbase, const unsigned char* vtbase)
{
    using L = SplitLds<kIldHalf>;
    constexpr int HD = 2 * kIldHalf, H = kIldHalf;
    const int tid = threadIdx.x;
    const int lane = il_fresh_lane();
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int kg = wave >> 2;                             // the half of the dimensions owned
    const bool upper = kg != 0;
    const int n = lane & 31, g = lane >> 5;
    const int sub = wave & 3;                             // the (head, 32-row block) pair served
    const uint32_t G = a.group;
    const uint32_t Gw = G < 4 ? G : 4;
    const uint32_t BP = 32 * (4 / Gw);                    // positions per block
    const uint32_t head = (uint32_t)__builtin_amdgcn_readfirstlane(kvh * G + hc * Gw + (sub % Gw));
    const uint32_t sub_rows = (uint32_t)__builtin_amdgcn_readfirstlane((sub / Gw) * 32);
    const uint32_t row0 = pb * BP + sub_rows;             // first chunk row of this wave
    const uint32_t kv_valid = a.p0 + a.T;                 // rows of the cache that hold data
    uint32_t t_first, t_last;

    PrefillRows<H> R;
    prefill_rows_init<H, false>(R, a, row0, head, n, g);

    IlCtx<H> cx;
    prefill_block_tiles(a, pb, BP, t_first, t_last);
    cx.t0 = t_first;
    cx.nt = t_last - t_first + 1;
    cx.t_last = t_last;
    cx.tail_tile = kv_valid / kTileKeys;
    cx.kbase = kbase;
    cx.vtbase = vtbase + kg * L::VTILE;                   // the half's dimensions of every Vt block
    cx.ring = kg * L::SET_BYTES;
    {
        const uint32_t lds0 = (uint32_t)__builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)smem);
        cx.m0k = lds0 + cx.ring + sub * 1024;
        cx.m0v = lds0 + cx.ring + L::V_IN_SET + sub * 1024;
        // block-local tile indices this wave's rows take part in
        const uint32_t lo_t = max(R.wt_first, t_first), hi_t = min(R.wt_last, t_last);
        if (R.wave_ok && lo_t <= hi_t) {
            cx.jt_lo = lo_t - t_first;
            cx.jt_hi = hi_t - t_first;
        } else {
            cx.jt_lo = 1;
            cx.jt_hi = 0;
        }
        // Tile kb holds an invisible (row, key) pair if kb + 31 > the first row's
        // position (diagonal), i.e. from tile edge_hi on, or kb < the last row's
        // window floor, i.e. below tile edge_lo.  The others are plain.
        const uint32_t edge_hi = (R.w_first_pos + 1) / kTileKeys;
        const uint32_t edge_lo = (R.w_hi_lo + kTileKeys - 1) / kTileKeys;
        cx.pl_lo = 1;
        cx.pl_hi = 0;
        if (cx.jt_lo <= cx.jt_hi && edge_hi >= 1 && edge_hi - 1 >= t_first) {
            const uint32_t lo = edge_lo > t_first ? max(cx.jt_lo, edge_lo - t_first) : cx.jt_lo;
            const uint32_t hi = min(cx.jt_hi, edge_hi - 1 - t_first);
            if (lo <= hi) {
                cx.pl_lo = lo;
                cx.pl_hi = hi;
            }
        }
        cx.jt_lo = (uint32_t)__builtin_amdgcn_readfirstlane(cx.jt_lo);
        cx.jt_hi = (uint32_t)__builtin_amdgcn_readfirstlane(cx.jt_hi);
        cx.pl_lo = (uint32_t)__builtin_amdgcn_readfirstlane(cx.pl_lo);
        cx.pl_hi = (uint32_t)__builtin_amdgcn_readfirstlane(cx.pl_hi);
    }
    {
        // K: lane -> (row of the tile, slot of the half's 16 chunks); the cache keeps
        // 32 chunks per key and half-tile, this half's are 16 kg .. 16 kg + 15
        const int row = sub * (1024 / L::RB) + lane / L::CPR;
        const int chunk = (lane % L::CPR) ^ L::fk(row);
        cx.gk_off = ((k_tile_half(row) * (2 * L::CPR) + kg * L::CPR + chunk) * 16 + k_tile_slot(row)) * 16;
        const int vrow = sub * 16 + lane / 4;
        cx.gv_off = vrow * 64 + ((lane & 3) ^ L::fv(vrow)) * 16;
        const int krow = prefill_key_perm(n);             // tile row this lane feeds to MFMA row n
        const uint32_t kread = krow * L::RB + ((g ^ L::fk(krow)) * 16);
        const uint32_t vread = n * 64 + ((g ^ L::fv(n)) * 16);
#pragma unroll
        for (int i = 0; i < H / 16; i++) cx.kop[i] = smem + ((cx.ring + kread) ^ (i * 32));
#pragma unroll
        for (int t = 0; t < 2; t++) cx.vop[t] = smem + cx.ring + L::V_IN_SET + (vread ^ (t * 32));
    }
    cx.thr = -INFINITY;
    const uint32_t nsteps = cx.nt;                        // the same in every wave

    // everything the first two vector blocks read, in order of need
    ild_issue_k<0>(cx, 0);
    ild_issue_k<1>(cx, 1);
    ild_issue_v<0>(cx, 0);
    ild_issue_k<2>(cx, 2);
    ild_issue_v<1>(cx, 1);
    // The wave's Q: 32 rows x its 128 dimensions, read in whole half rows (512
    // contiguous bytes per 32 lanes)
    float4 qx[16];
#pragma unroll
    for (int jj = 0; jj < 16; jj++) {
        const uint32_t row = min(row0 + 2 * jj + (lane >> 5), a.T - 1);   // idle rows re-read the last one
        qx[jj] = *reinterpret_cast<const float4*>(a.q + ((size_t)row * a.nq + head) * HD + kg * H + (lane & 31) * 4);
    }
    float* xw = reinterpret_cast<float*>(smem + IldLds::X_OFF + (sub * 2 + kg) * IldLds::X_WAVE);
    const float* xr_at = reinterpret_cast<const float*>(smem + IldLds::X_OFF + (sub * 2 + (kg ^ 1)) * IldLds::X_WAVE);

    f32x16 sa, sb, negm;
    u32x4 pop[2];
    half8 kf[8], vf[8];
#pragma unroll
    for (int r = 0; r < 16; r++) sa[r] = sb[r] = negm[r] = 0.f;
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    {
        // Q is scaled, rounded once and turned into the per-lane operand layout
        // (contraction slots (g, j) of link i = dims 128 kg + 16 i + 8 g + j of the
        // lane's own row) through the wave's share of the exchange buffers, which
        // nothing uses before the first step: rows of 256 bytes, the 16-byte chunk
        // c of row r at slot c ^ (r % 16).  Nobody else reads it: no barrier.
        unsigned char* qs = smem + IldLds::X_OFF + wave * 8192;
        static_assert(8 * 8192 <= IldLds::X_BYTES, "the staged Q operands fit the exchange buffers");
#pragma unroll
        for (int jj = 0; jj < 16; jj++) {
            const int r = 2 * jj + (lane >> 5), c = (lane & 31) >> 1;
            *reinterpret_cast<half4*>(qs + r * 256 + ((c ^ (r & 15)) * 16) + (lane & 1) * 8) =
                q_scaled_f16(qx[jj], a.qscale);
        }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
        for (int i = 0; i < H / 16; i++)
            R.qop[i] = *reinterpret_cast<const half8*>(qs + n * 256 + (((2 * i + g) ^ (n & 15)) * 16));
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");   // read back before the first partial scores land there
    }
    ild_patch_tail<0>(smem, cx, 0, sub, lane, kv_valid);
    il_barrier();                                         // first tiles visible to all
    // scores of the first tile
#pragma unroll
    for (int i = 0; i < 8; i++) kf[i] = *reinterpret_cast<const half8*>(cx.kop[i]);
#pragma unroll
    for (int i = 0; i < 8; i++) sa = __builtin_amdgcn_mfma_f32_32x32x16_f16(kf[i], R.qop[i], sa, 0, 0, 0);
    ild_send(xw, sa, lane);                               // tile 0: the exchange buffer of parity 0
    il_barrier();                                         // partial scores out; slot 0 of K has been read by all
    ild_issue_k<0>(cx, 3);
#pragma unroll
    for (int i = 0; i < 8; i++) kf[i] = *reinterpret_cast<const half8*>(cx.kop[i] + L::KTILE);
    il_barrier();                                         // slot 1 of K has been read by all: step 0 refills it
    float pend = 0.f;
    uint32_t pend_on = 0;

#define WR_ILD_STEP(PHASE, XB, CUR, NXT)                                                                     \
    ild_step<PHASE, XB>(R, cx, negm, CUR, NXT, pop, kf, vf, smem, xw, xr_at, j, sub, lane, g, kv_valid, upper, \
                        pend, pend_on);                                                                      \
    if (++j >= nsteps) break;
#pragma unroll 1
    for (uint32_t j = 0;;) {
        WR_ILD_STEP(0, 0, sa, sb)
        WR_ILD_STEP(1, 1, sb, sa)
        WR_ILD_STEP(2, 0, sa, sb)
        WR_ILD_STEP(0, 1, sb, sa)
        WR_ILD_STEP(1, 0, sa, sb)
        WR_ILD_STEP(2, 1, sb, sa)
    }
#undef WR_ILD_STEP

    // the ring must be quiet before the rows are staged over it (the last steps'
    // copies still target it)
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    const int lane_e = il_fresh_lane();
    const int n_e = lane_e & 31, g_e = lane_e >> 5;
    const float l_tot = wave_pair32_sum(R.l_run);
    const float inv = (l_tot > 0.f) ? 1.0f / l_tot : 0.f;
    // rows leave through LDS: the wave's tile row-major in its own scratch, then
    // whole half rows (512 contiguous bytes) per 32 lanes
    float (*os)[H + 4] = reinterpret_cast<float (*)[H + 4]>(smem + (size_t)wave * IldLds::O_WAVE);
#pragma unroll
    for (int dt = 0; dt < H / 32; dt++)
#pragma unroll
        for (int q4 = 0; q4 < 4; q4++) {
            float4 v;
            v.x = R.o[dt][4 * q4 + 0] * inv;
            v.y = R.o[dt][4 * q4 + 1] * inv;
            v.z = R.o[dt][4 * q4 + 2] * inv;
            v.w = R.o[dt][4 * q4 + 3] * inv;
            *reinterpret_cast<float4*>(&os[n_e][dt * 32 + 8 * q4 + 4 * g_e]) = v;
        }
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");    // the wave reads back what it wrote itself
    {
        constexpr int LPR = H / 4;                        // lanes per half row (one float4 each)
        constexpr int RPI = 64 / LPR;                     // rows per store instruction
#pragma unroll
        for (int jj = 0; jj < 32 / RPI; jj++) {
            const int r = jj * RPI + lane_e / LPR;
            const float4 v = *reinterpret_cast<const float4*>(&os[r][(lane_e % LPR) * 4]);
            if (row0 + r < a.T)
                *reinterpret_cast<float4*>(a.out + ((size_t)(row0 + r) * a.nq + head) * HD + kg * H +
                                           (lane_e % LPR) * 4) = v;
        }
    }
}

// grid = (KV heads x head chunks, ceil(blocks / 2)), as prefill_il_kernel.
__global__ __launch_bounds__(kSplitThreads, 1) void prefill_ild_kernel(const PrefillArgs a)
{
    extern __shared__ __attribute__((aligned(16))) unsigned char prefill_smem_raw[];
    constexpr int HD = 2 * kIldHalf;
    const uint32_t G = a.group;
    const uint32_t Gw = G < 4 ? G : 4;
    const uint32_t chunks = G / Gw;
    const uint32_t kvh = (uint32_t)__builtin_amdgcn_readfirstlane(blockIdx.x / chunks);
    const uint32_t hc = (uint32_t)__builtin_amdgcn_readfirstlane(blockIdx.x % chunks);
    const uint32_t BP = 32 * (4 / Gw);
    const uint32_t nblk = (uint32_t)__builtin_amdgcn_readfirstlane((a.T + BP - 1) / BP);
    const uint32_t lo = blockIdx.y, hi = nblk - 1 - blockIdx.y;
    const unsigned char* kbase =
        uniform_ptr(reinterpret_cast<const unsigned char*>(a.k + (size_t)kvh * a.ctx_pad * HD));
    const unsigned char* vtbase = uniform_ptr(reinterpret_cast<const unsigned char*>(
        a.vt + (size_t)kvh * (a.ctx_pad / kVBlock) * HD * kVBlock));
    ild_block(a, prefill_smem_raw, hi, kvh, hc, kbase, vtbase);
    if (!a.single && hi != lo) {
        __syncthreads();                                  // LDS changes hands
        ild_block(a, prefill_smem_raw, lo, kvh, hc, kbase, vtbase);
    }
}

}  // namespace wr
