// Causal prefill attention on the matrix cores, one wave per SIMD, two 32-row
// units per wave (head dims 64 and 128; v_mfma_f32_32x32x16_f16, F32 accumulate).
// MFMA-bound: 4 * nq * hd flops per (query row, visible key).
//
// Semantics: kernels_prefill.hip.h (reference: the prefill loop
// src/core/session.c:615-625 over src/core/kernels.c:1475-1523).
//
// Workgroup = 4 waves = one KV head x 4 units x 2 key sets.  A unit is one head of
// the GQA group at one 32-row sub-block (unit u: head u % Gw, sub-block u / Gw,
// Gw = min(group, 4)).  Wave w serves the TWO units 2 * (w & 1) and 2 * (w & 1) + 1
// over the 32-key tiles of parity (w >> 1) of the block's key range: split-K inside
// the workgroup, the two partial (m, l, O) triples of a unit exchanged through LDS
// at the end, where each wave of a pair finishes one of the pair's two units.
//
// Why two units per wave: every K and Vt operand a wave reads out of LDS feeds two
// matrix instructions instead of one (half the LDS bytes per flop), and the two
// score chains alternate, so no matrix instruction waits for the one before it.
// The accumulators of two units (128 registers at head dim 128) plus two score
// buffers each do not fit 256 registers: the kernel runs one wave per SIMD with
// the whole register file, and everything that hides latency is in the wave's own
// instruction stream.
//
// Per wave, unit and tile, with the query row as the MFMA COLUMN (lane % 32):
//   S^T[key][row]  = K[key][:] . Q^T[:][row]          HD/16 MFMAs, a dependent chain
//   online softmax on the 16 scores a lane holds (+ one exchange with lane^32)
//   O^T[dim][row] += Vt[dim][key] . P^T[key][row]     HD/16 MFMAs
// Operand layouts, the K row permutation, the lazy softmax reference, the chain
// that starts from a block of -m, the LDS tile image (chunks of a row permuted so
// that 128-bit reads are conflict free) and the copies from global memory straight
// into LDS are those of kernels_prefill_il.hip.h.
//
// Shape of a step (set-local tile j -> j + 1), one instruction stream:
//   first half:   the score chains S(j+1) of both units, link by link in turn, and
//                 behind each link a Vt operand read of tile j and a share of the
//                 exponentials and packs of S(j);
//   second half:  O^T += Vt(j).P(j)^T for both units, and between the products the
//                 K operand reads of tile j+2, the step's copies and the row maxima
//                 of S(j+1);
//   one hardware barrier per step publishes the copies that have landed and
//   frees the ring slots the next step overwrites.
//
// Ends of a block.  Q rows are read straight into operand layout (each lane its
// own row, 32 contiguous bytes per contraction step); nothing is staged.  After
// the loop the wave of key set s keeps unit s of its pair and hands the other
// unit's partial to its partner through LDS; each then merges, normalises and
// stores its unit's rows from registers (16 bytes per lane and store, the four
// stores of a 128-byte line back to back).  The next block's first copies and Q
// rows are asked for before the exchange.
#pragma once

#include "kernels_prefill_il.hip.h"

#ifndef WR_PAIR_PROBE
#define WR_PAIR_PROBE 0
#endif

namespace wr {

constexpr int kPairThreads = 256;

template <int HD>
struct PairLds {
    static constexpr int RB = 2 * HD;                     // bytes per K row
    static constexpr int CPR = HD / 8;                    // 16-byte chunks per K row
    static constexpr int RPB = 256 / RB > 0 ? 256 / RB : 1;   // K rows per 256-byte bank row
    static constexpr int KTILE = kTileKeys * RB;          // bytes of one tile's K
    static constexpr int VTILE = HD * kVBlock * 2;        // bytes of one tile's Vt block
    static constexpr int PIECES = KTILE / 1024;           // KiB pieces per tile, each of K and Vt
    static constexpr int NLW = PIECES / 2;                // copies per wave and tile, each of K and Vt
    static constexpr int SET_BYTES = kRing * (KTILE + VTILE);
    static constexpr int V_IN_SET = kRing * KTILE;
    // exchange scratch: per wave the accumulators of one unit, [HD/8][64 lanes][4]
    static constexpr int X_OFF = 2 * SET_BYTES;
    static constexpr int X_WAVE = (HD / 2) * 64 * 4;
    static constexpr int TOTAL = X_OFF + 4 * X_WAVE;
    // (m, l) of the exchanged units: in the odd set's third Vt slot, which no copy
    // of a block's prologue goes to
    static constexpr int ML_OFF = SET_BYTES + V_IN_SET + 2 * VTILE;
    static_assert(KTILE == VTILE && NLW >= 1, "one piece schedule serves K and Vt");
    static_assert(4 * 2 * 64 * 4 <= VTILE, "(m, l) of four waves fit a Vt slot");
    static_assert(TOTAL <= 160 * 1024, "LDS of one compute unit");
    __device__ static constexpr int fk(int row) { return (row / RPB) & (CPR - 1); }
    __device__ static constexpr int fv(int row) { return (row >> 2) & 3; }
};

template <int HD>
constexpr size_t pair_smem_bytes()
{
    return PairLds<HD>::TOTAL;
}

// One 32-row unit of a wave.
template <int HD>
struct PairUnit {
    PrefillRows<HD> R;
    f32x16 negm;                      // -m of the unit's rows, the block a score chain starts from
    float thr;                        // a row maximum above this moves the softmax reference
    uint32_t jt_lo, jt_hi;            // set-local tile indices the unit's rows take part in (empty: lo > hi)
    uint32_t pl_lo, pl_hi;            // ... of which these are plain: every (row, key) pair visible
    uint32_t head, row0;
};

template <int HD>
struct PairCtx {
    // wave-uniform
    const unsigned char* kbase;       // this KV head's K / Vt, bytes
    const unsigned char* vtbase;
    uint32_t m0k, m0v;                // LDS byte address of this wave's first K / Vt copy in ring slot 0
    uint32_t t0, nt, t_last;          // the set's first tile and tile count, the block's last tile
    uint32_t tail_tile;               // tiles from this one on reach past the appended rows
    uint32_t ring;                    // byte offset of the set's ring in the kernel's LDS
    uint32_t piece0;                  // first KiB piece of a tile this wave copies
    // per lane
    uint32_t gk_off[PairLds<HD>::NLW];   // offset inside a K tile of this lane's 16 bytes, per copy
    uint32_t gv_off;                     // ... inside a KiB piece of a Vt block
    uint32_t kop[HD / 16];               // LDS byte offset of the K operand read of contraction step i, slot 0
    uint32_t vop[2];                     // ... of the Vt operand read of half t, dimension block 0, slot 0
};

template <int HD>
__device__ __forceinline__ uint32_t pair_tile(const PairCtx<HD>& cx, uint32_t jt)
{
    return min(cx.t0 + 2 * jt, cx.t_last);
}

// Copy u of this wave's NLW copies of the set's K tile jt / Vt block jt into ring slot SLOT.
template <int HD, int SLOT>
__device__ __forceinline__ void pair_issue_k1(const PairCtx<HD>& cx, uint32_t jt, int u)
{
    using L = PairLds<HD>;
    const unsigned char* src = cx.kbase + (size_t)pair_tile(cx, jt) * L::KTILE;
    lds_direct_load(cx.m0k + SLOT * L::KTILE + u * 1024, src, cx.gk_off[u]);
}

template <int HD, int SLOT>
__device__ __forceinline__ void pair_issue_v1(const PairCtx<HD>& cx, uint32_t jt, int u)
{
    using L = PairLds<HD>;
    const unsigned char* src = cx.vtbase + (size_t)pair_tile(cx, jt) * L::VTILE + (cx.piece0 + u) * 1024;
    lds_direct_load(cx.m0v + SLOT * L::VTILE + u * 1024, src, cx.gv_off);
}

template <int HD, int SLOT>
__device__ __forceinline__ void pair_issue_k(const PairCtx<HD>& cx, uint32_t jt)
{
#pragma unroll
    for (int u = 0; u < PairLds<HD>::NLW; u++) pair_issue_k1<HD, SLOT>(cx, jt, u);
}

template <int HD, int SLOT>
__device__ __forceinline__ void pair_issue_v(const PairCtx<HD>& cx, uint32_t jt)
{
#pragma unroll
    for (int u = 0; u < PairLds<HD>::NLW; u++) pair_issue_v1<HD, SLOT>(cx, jt, u);
}

// Zeroes, in the staged Vt of the set's tile jt (ring slot SLOT), the positions
// that were never appended (0 * garbage must not reach the accumulator).  Every
// lane patches the chunks its own copies delivered.
template <int HD, int SLOT>
__device__ __forceinline__ void pair_patch_tail(unsigned char* smem, const PairCtx<HD>& cx, uint32_t jt,
                                                int lane, uint32_t kv_valid)
{
    using L = PairLds<HD>;
    const uint32_t tile = pair_tile(cx, jt);
    if (tile < cx.tail_tile) return;
#pragma unroll
    for (int u = 0; u < L::NLW; u++) {
        const int row = lane / 4;                         // Vt row (dimension) inside the piece: fv sees its low bits only
        const int c = (lane & 3) ^ L::fv(row);            // key chunk this slot holds
        const uint32_t key0 = tile * kTileKeys + c * 8;
        u32x4* at = reinterpret_cast<u32x4*>(smem + cx.ring + L::V_IN_SET + SLOT * L::VTILE +
                                             (cx.piece0 + u) * 1024 + lane * 16);
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

// Masks of a tile that is not plain for the unit (rare, wave-uniform branch);
// written in place, behind the row maximum `after` (see il_mask_special).
template <int HD>
__device__ __forceinline__ void pair_mask_special(const PairUnit<HD>& U, f32x16& c, uint32_t tile, uint32_t jt,
                                                  int g, float after)
{
    const float ninf = -INFINITY;
    asm volatile("" ::"v"(after));
    if (jt < U.jt_lo || jt > U.jt_hi) {
#pragma unroll
        for (int r = 0; r < 16; r++) asm volatile("v_mov_b32 %0, %1" : "+v"(c[r]) : "v"(ninf), "v"(after));
    } else {
        const uint32_t kb = tile * kTileKeys;
#pragma unroll
        for (int r = 0; r < 16; r++) {
            const uint32_t key = kb + 16 * (r >> 3) + 8 * g + (r & 7);
            const uint64_t hide = __builtin_amdgcn_ballot_w64(key > U.R.pos || key < U.R.row_lo);
            asm volatile("v_cndmask_b32 %0, %0, %1, %2" : "+v"(c[r]) : "v"(ninf), "s"(hide), "v"(after));
        }
    }
}

// The softmax reference of a row moves (rare, wave-uniform branch).
template <int HD>
__device__ __forceinline__ void pair_move_reference(PairUnit<HD>& U, f32x16& c, float tmax, bool jump)
{
    PrefillRows<HD>& R = U.R;
    const bool unset = (R.m_run == -INFINITY);
    const float delta = jump ? tmax : 0.f;
    const float alpha = jump ? (unset ? 0.f : fast_exp2(-delta)) : 1.0f;
    R.l_run *= alpha;
#pragma unroll
    for (int dt = 0; dt < HD / 32; dt++)
#pragma unroll
        for (int r = 0; r < 16; r++) R.o[dt][r] *= alpha;
#pragma unroll
    for (int r = 0; r < 16; r++) asm volatile("v_sub_f32 %0, %0, %1" : "+v"(c[r]) : "v"(delta));
    if (jump) R.m_run = (unset ? 0.f : R.m_run) + delta;
    const bool still = (R.m_run == -INFINITY);
    const float nm = still ? 0.f : -R.m_run;
#pragma unroll
    for (int r = 0; r < 16; r++) asm volatile("v_mov_b32 %0, %1" : "+v"(U.negm[r]) : "v"(nm));
    asm volatile("v_mov_b32 %0, %1" : "+v"(U.thr) : "v"(still ? -INFINITY : kLazyLog2));
}

// Row maximum of `c` (taken as if the tile were plain), masks where it is not,
// the maximum joined across the two lanes of a row and, rarely, a move of the
// row's reference.
template <int HD>
__device__ __forceinline__ void pair_settle(PairUnit<HD>& U, const PairCtx<HD>& cx, f32x16& c, uint32_t jt, int g)
{
    float tmax = il_max16(c);
    if (jt < U.pl_lo || jt > U.pl_hi) {
        pair_mask_special<HD>(U, c, cx.t0 + 2 * jt, jt, g, tmax);
        tmax = il_max16(c);
    }
    {
        const uint32_t u = __float_as_uint(tmax);
        const auto sw = __builtin_amdgcn_permlane32_swap(u, u, false, false);
        tmax = max3_raw(__uint_as_float(sw[0]), __uint_as_float(sw[1]), tmax);
    }
    const bool jump = tmax > U.thr;
    if (__builtin_amdgcn_ballot_w64(jump) != 0) pair_move_reference<HD>(U, c, tmax, jump);
}

// The matrix instructions, spelled out so that each operand sits in the register
// file it is meant for: scores in ordinary vector registers (the vector ALU works
// on them), output accumulators and the Q^T operand in accumulation registers
// (only matrix instructions touch them in the loop).  With the builtin the
// compiler of a one-wave-per-SIMD kernel gives every result an accumulation
// register and copies scores out and operands in around each instruction.
// No wait states are inserted for these: a result is first read by a vector
// instruction at least two matrix instructions later (see pair_step), and by the
// next link of its own chain one matrix instruction later.
__device__ __forceinline__ f32x16 pair_mfma_first(half8 a, half8 b, const f32x16& c)
{
    f32x16 d;
    asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %3" : "=&v"(d) : "a"(a), "a"(b), "v"(c));
    return d;
}

__device__ __forceinline__ void pair_mfma_link(f32x16& d, half8 a, half8 b)
{
    asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+v"(d) : "a"(a), "a"(b));
}

// A finished operand moved to accumulation registers once, as a value of that
// register file (an operand that is made in vector registers and only named as
// an accumulation-register input is copied over before every use).
__device__ __forceinline__ half8 pair_to_acc(half8 v)
{
    half8 a;
    asm volatile("" : "=a"(a) : "0"(v));
    return a;
}

__device__ __forceinline__ void pair_mfma_acc(f32x16& d, half8 a, half8 b)
{
    asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+a"(d) : "v"(a), "v"(b));
}

// Step j of a wave (P == j % kRing).  On entry cur[u] holds unit u's scores of the
// set's tile j (masked, reference settled), kf the K operands of tile j+1; on exit
// nxt[u] holds the scores of tile j+1 in the same state and kf the operands of
// tile j+2.
template <int HD, int P>
__device__ __forceinline__ void pair_step(PairUnit<HD> (&U)[2], const PairCtx<HD>& cx, const f32x16 (&cur)[2],
                                          f32x16 (&nxt)[2], u32x4 (&pop)[2][2], half8 (&kf)[HD / 16],
                                          half8 (&vf)[HD / 16], unsigned char* smem, uint32_t j, int lane, int g,
                                          uint32_t kv_valid)
{
    using L = PairLds<HD>;
    constexpr int NS = HD / 16, ND = HD / 32;
    constexpr int PAIRS = 8 / NS;         // pairs of probabilities formed behind each link of a chain
    static_assert(kRing == 3 && 8 % NS == 0 && NS >= 2 * L::NLW, "slot and interleave arithmetic below");
    constexpr int VS = P;                 // slot of Vt of tile j
    constexpr int KS = (P + 2) % 3;       // slot of K of tile j+2
    constexpr int KC = (P + 1) % 3;       // K of tile j+4 replaces K of tile j+1 (read in the previous step)
    constexpr int VC = (P + 2) % 3;       // Vt of tile j+2 replaces Vt of tile j-1 (read in the previous step)
    constexpr int TS = (P + 1) % 3;       // slot of Vt of tile j+1, whose tail is patched once it has landed

    float psum[2] = {0.f, 0.f};
    const half2v ones = {(_Float16)1.0f, (_Float16)1.0f};
#pragma unroll
    for (int i = 0; i < NS; i++) {
#pragma unroll
        for (int u = 0; u < 2; u++) {
            if (i == 0)
                nxt[u] = pair_mfma_first(kf[0], U[u].R.qop[0], U[u].negm);
            else
                pair_mfma_link(nxt[u], kf[i], U[u].R.qop[i]);
            if (u == 0 && !(WR_PAIR_PROBE & 8))
                vf[i] = *reinterpret_cast<const half8*>(smem + cx.vop[i / ND] + VS * L::VTILE + (i % ND) * 2048);
#pragma unroll
            for (int q = 0; q < ((WR_PAIR_PROBE & 1) ? 0 : PAIRS); q++) {
                const int r = 2 * (i * PAIRS + q);
                const half2v ph = {(_Float16)fast_exp2(cur[u][r]), (_Float16)fast_exp2(cur[u][r + 1])};
                psum[u] = __builtin_amdgcn_fdot2(ph, ones, psum[u], false);
                pop[u][r >> 3][(r & 7) >> 1] = __builtin_bit_cast(uint32_t, ph);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
    }
    U[0].R.l_run += psum[0];
    U[1].R.l_run += psum[1];
#pragma unroll
    for (int i = 0; i < NS; i++) {
        const int t = i / ND, dt = i % ND;
#pragma unroll
        for (int u = 0; u < 2; u++) pair_mfma_acc(U[u].R.o[dt], vf[i], __builtin_bit_cast(half8, pop[u][t]));
        if (!(WR_PAIR_PROBE & 8)) kf[i] = *reinterpret_cast<const half8*>(smem + cx.kop[i] + KS * L::KTILE);
        if (!(WR_PAIR_PROBE & 2)) {
            if (i < L::NLW) pair_issue_k1<HD, KC>(cx, j + 4, i);
            else if (i < 2 * L::NLW) pair_issue_v1<HD, VC>(cx, j + 2, i - L::NLW);
        }
        // The scores of tile j+1 are results of hand-written matrix instructions:
        // nothing may read them before two more matrix instructions have been
        // issued behind the last link (the compiler knows of no wait states here).
        if (i == 0) __builtin_amdgcn_sched_barrier(0);
    }
    if (!(WR_PAIR_PROBE & 16)) {
        pair_settle<HD>(U[0], cx, nxt[0], j + 1, g);
        pair_settle<HD>(U[1], cx, nxt[1], j + 1, g);
    }
    // all copies but this step's have landed: K of tile j+3 and Vt of tile j+1,
    // which the next step reads once the barrier has published them
    if (!(WR_PAIR_PROBE & 2)) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * L::NLW) : "memory");
    pair_patch_tail<HD, TS>(smem, cx, j + 1, lane, kv_valid);
    __builtin_amdgcn_sched_barrier(0);
    if (!(WR_PAIR_PROBE & 4)) asm volatile("s_barrier" ::: "memory");
    __builtin_amdgcn_sched_barrier(0);
}

// Q rows of one unit as read from global memory, already in operand order: the
// lane's own row, eight consecutive dimensions per contraction step.
template <int HD>
struct PairQ {
    float4 x[HD / 16][2];
};

template <int HD, bool Q16>
__device__ __forceinline__ void pair_load_q(PairQ<HD>& q, const PrefillArgs& a, uint32_t row0, uint32_t head,
                                            int n, int g)
{
    const uint32_t row = min(row0 + n, a.T - 1);          // idle rows re-read the last one
    const size_t at = ((size_t)row * a.nq + head) * HD + g * 8;
    if (WR_PAIR_PROBE & 32) {
#pragma unroll
        for (int i = 0; i < HD / 16; i++) q.x[i][0] = q.x[i][1] = make_float4(0.f, 0.f, 0.f, 0.f);
        return;
    }
    if constexpr (Q16) {                                  // eight finished halves: 16 bytes
        const uint16_t* src = a.q16 + at;
#pragma unroll
        for (int i = 0; i < HD / 16; i++) {
            const uint4 h = *reinterpret_cast<const uint4*>(src + i * 16);
            q.x[i][0] = make_float4(__uint_as_float(h.x), __uint_as_float(h.y), __uint_as_float(h.z),
                                    __uint_as_float(h.w));
        }
    } else {
        const float* src = a.q + at;
#pragma unroll
        for (int i = 0; i < HD / 16; i++) {
            q.x[i][0] = *reinterpret_cast<const float4*>(src + i * 16);
            q.x[i][1] = *reinterpret_cast<const float4*>(src + i * 16 + 4);
        }
    }
}

template <int HD, bool Q16>
__device__ __forceinline__ void pair_convert_q(PrefillRows<HD>& R, PairQ<HD>& q, const PrefillArgs& a)
{
    if constexpr (Q16) {
#pragma unroll
        for (int i = 0; i < HD / 16; i++) {
            const u32x4 h = {__float_as_uint(q.x[i][0].x), __float_as_uint(q.x[i][0].y),
                             __float_as_uint(q.x[i][0].z), __float_as_uint(q.x[i][0].w)};
            R.qop[i] = pair_to_acc(__builtin_bit_cast(half8, h));
            q.x[i][0] = make_float4(0.f, 0.f, 0.f, 0.f);  // consumed: nothing of it has to outlive the step loop
        }
    } else {
#pragma unroll
        for (int i = 0; i < HD / 16; i++) {
            const half4 lo = q_scaled_f16(q.x[i][0], a.qscale), hi = q_scaled_f16(q.x[i][1], a.qscale);
            R.qop[i] = pair_to_acc(half8{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]});
            q.x[i][0] = q.x[i][1] = make_float4(0.f, 0.f, 0.f, 0.f);
        }
    }
}

// The tile range of position block pb for key set kg, into the context.
template <int HD>
__device__ __forceinline__ void pair_ctx_tiles(PairCtx<HD>& cx, const PrefillArgs& a, uint32_t pb, uint32_t BP,
                                               int kg, uint32_t& t_first, uint32_t& t_last)
{
    prefill_block_tiles(a, pb, BP, t_first, t_last);
    cx.t0 = t_first + kg;                                 // this set's tiles: t0, t0 + 2, ...
    cx.nt = (cx.t0 <= t_last) ? (t_last - cx.t0) / 2 + 1 : 0;
    cx.t_last = t_last;
}

// Which of the set's tiles the unit's rows take part in, and which of those are plain.
template <int HD>
__device__ __forceinline__ void pair_unit_ranges(PairUnit<HD>& U, const PairCtx<HD>& cx)
{
    const PrefillRows<HD>& R = U.R;
    uint32_t jt_lo = 1, jt_hi = 0, pl_lo = 1, pl_hi = 0;
    const uint32_t lo_t = max(R.wt_first, cx.t0), hi_t = min(R.wt_last, cx.t_last);
    if (R.wave_ok && cx.nt > 0 && lo_t <= hi_t && (lo_t - cx.t0 + 1) / 2 <= (hi_t - cx.t0) / 2) {
        jt_lo = (lo_t - cx.t0 + 1) / 2;
        jt_hi = (hi_t - cx.t0) / 2;
    }
    // Tile kb holds an invisible (row, key) pair if kb + 31 > the first row's
    // position (diagonal), i.e. from tile edge_hi on, or kb < the last row's
    // window floor, i.e. below tile edge_lo.  The others are plain.
    const uint32_t edge_hi = (R.w_first_pos + 1) / kTileKeys;
    const uint32_t edge_lo = (R.w_hi_lo + kTileKeys - 1) / kTileKeys;
    if (jt_lo <= jt_hi && edge_hi >= 1 && edge_hi - 1 >= cx.t0) {
        const uint32_t lo = edge_lo > cx.t0 ? max(jt_lo, (edge_lo - cx.t0 + 1) / 2) : jt_lo;
        const uint32_t hi = min(jt_hi, (edge_hi - 1 - cx.t0) / 2);
        if (lo <= hi) {
            pl_lo = lo;
            pl_hi = hi;
        }
    }
    U.jt_lo = (uint32_t)__builtin_amdgcn_readfirstlane(jt_lo);
    U.jt_hi = (uint32_t)__builtin_amdgcn_readfirstlane(jt_hi);
    U.pl_lo = (uint32_t)__builtin_amdgcn_readfirstlane(pl_lo);
    U.pl_hi = (uint32_t)__builtin_amdgcn_readfirstlane(pl_hi);
}

// The copies and loads a block starts with: the first three K tiles and two Vt
// blocks of the set into their ring slots, in order of need, and the wave's Q rows.
template <int HD, bool Q16>
__device__ __forceinline__ void pair_first_loads(const PairCtx<HD>& cx, PairQ<HD> (&q)[2], const PrefillArgs& a,
                                                 const uint32_t (&row0)[2], const uint32_t (&head)[2], int n, int g)
{
    pair_load_q<HD, Q16>(q[0], a, row0[0], head[0], n, g);
    pair_issue_k<HD, 0>(cx, 0);
    pair_issue_v<HD, 0>(cx, 0);
    pair_load_q<HD, Q16>(q[1], a, row0[1], head[1], n, g);
    pair_issue_k<HD, 1>(cx, 1);
    pair_issue_k<HD, 2>(cx, 2);
    pair_issue_v<HD, 1>(cx, 1);
}

// Unit `mine` of the pair is finished by this wave: its partial is merged with
// the partner wave's (read from the partner's scratch), normalised and stored;
// unit `theirs` went into this wave's scratch before the barrier.
template <int HD>
__device__ __forceinline__ void pair_send(const PairUnit<HD>& U, unsigned char* smem, int wave, int lane)
{
    using L = PairLds<HD>;
    f32x4* x = reinterpret_cast<f32x4*>(smem + L::X_OFF + wave * L::X_WAVE);
#pragma unroll
    for (int dt = 0; dt < HD / 32; dt++)
#pragma unroll
        for (int q4 = 0; q4 < 4; q4++)
        {
            x[(dt * 4 + q4) * 64 + lane] = f32x4{U.R.o[dt][4 * q4 + 0], U.R.o[dt][4 * q4 + 1],
                                                 U.R.o[dt][4 * q4 + 2], U.R.o[dt][4 * q4 + 3]};
            // a few registers at a time: the next block's Q rows are in flight in the others
            __builtin_amdgcn_sched_barrier(0);
        }
    float* ml = reinterpret_cast<float*>(smem + L::ML_OFF) + wave * 128;
    ml[lane] = U.R.m_run;
    ml[64 + lane] = U.R.l_run;
}

template <int HD>
__device__ __forceinline__ void pair_finish(PairUnit<HD>& U, const PrefillArgs& a, unsigned char* smem,
                                            int partner, int lane, int n, int g)
{
    using L = PairLds<HD>;
    PrefillRows<HD>& R = U.R;
    const f32x4* x = reinterpret_cast<const f32x4*>(smem + L::X_OFF + partner * L::X_WAVE);
    const float* ml = reinterpret_cast<const float*>(smem + L::ML_OFF) + partner * 128;
    const float m1 = ml[lane], l1 = ml[64 + lane];
    const float m = fmaxf(R.m_run, m1);
    const float f0m = (R.m_run == -INFINITY) ? 0.f : fast_exp2(R.m_run - m);
    const float f1m = (m1 == -INFINITY) ? 0.f : fast_exp2(m1 - m);
    const float l_tot = wave_pair32_sum(R.l_run * f0m + l1 * f1m);
    const float inv = (l_tot > 0.f) ? 1.0f / l_tot : 0.f;
    const float w0 = f0m * inv, w1 = f1m * inv;
    const uint32_t my_row = U.row0 + n;
    float* orow = a.out + ((size_t)min(my_row, a.T - 1) * a.nq + U.head) * HD + 4 * g;
    const bool live = my_row < a.T;
#pragma unroll
    for (int dt = 0; dt < HD / 32; dt++)
#pragma unroll
        for (int q4 = 0; q4 < 4; q4++) {
            const f32x4 p = x[(dt * 4 + q4) * 64 + lane];
            float4 v;
            v.x = R.o[dt][4 * q4 + 0] * w0 + p[0] * w1;
            v.y = R.o[dt][4 * q4 + 1] * w0 + p[1] * w1;
            v.z = R.o[dt][4 * q4 + 2] * w0 + p[2] * w1;
            v.w = R.o[dt][4 * q4 + 3] * w0 + p[3] * w1;
            if (live) *reinterpret_cast<float4*>(orow + dt * 32 + 8 * q4) = v;
            if (q4 & 1) __builtin_amdgcn_sched_barrier(0);    // two lines of registers at a time
        }
}

// One position block.  started: the block's first loads are already on their way
// (q holds its Q rows).  next_pb >= 0: once this block's loop is over, the first
// loads of block next_pb are issued, before the exchange and the stores, and q
// returns its Q rows.
template <int HD, bool Q16>
__device__ __forceinline__ void pair_block(const PrefillArgs& a, unsigned char* smem, uint32_t pb, uint32_t kvh,
                                           uint32_t hc, const unsigned char* kbase, const unsigned char* vtbase,
                                           bool started, PairQ<HD> (&q)[2], int next_pb)
{
    using L = PairLds<HD>;
    const int tid = threadIdx.x;
    const int lane = il_fresh_lane();
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int n = lane & 31, g = lane >> 5;
    const int kg = wave >> 1, hp = wave & 1;              // key set (tile parity), pair of units served
    const uint32_t G = a.group;
    const uint32_t Gw = G < 4 ? G : 4;
    const uint32_t BP = 32 * (4 / Gw);                    // positions per block
    const uint32_t kv_valid = a.p0 + a.T;                 // rows of the cache that hold data
    uint32_t head[2], sub_rows[2], row0[2];
#pragma unroll
    for (int u = 0; u < 2; u++) {
        const uint32_t unit = 2 * hp + u;
        head[u] = (uint32_t)__builtin_amdgcn_readfirstlane(kvh * G + hc * Gw + (unit % Gw));
        sub_rows[u] = (uint32_t)__builtin_amdgcn_readfirstlane((unit / Gw) * 32);
        row0[u] = pb * BP + sub_rows[u];
    }
    uint32_t t_first, t_last;

    PairUnit<HD> U[2];
    PairCtx<HD> cx;
    pair_ctx_tiles<HD>(cx, a, pb, BP, kg, t_first, t_last);
    cx.tail_tile = kv_valid / kTileKeys;
    cx.kbase = kbase;
    cx.vtbase = vtbase;
    cx.ring = kg * L::SET_BYTES;
    cx.piece0 = hp * L::NLW;
    {
        const uint32_t lds0 = (uint32_t)__builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)smem);
        cx.m0k = lds0 + cx.ring + cx.piece0 * 1024;
        cx.m0v = lds0 + cx.ring + L::V_IN_SET + cx.piece0 * 1024;
    }
#pragma unroll
    for (int u = 0; u < 2; u++) {
        prefill_rows_init<HD, false>(U[u].R, a, row0[u], head[u], n, g);
        pair_unit_ranges<HD>(U[u], cx);
        U[u].thr = -INFINITY;
        U[u].head = head[u];
        U[u].row0 = row0[u];
#pragma unroll
        for (int r = 0; r < 16; r++) U[u].negm[r] = 0.f;
    }
    {
        // K: lane -> (row of the tile, slot); fetch the chunk that belongs in that slot
#pragma unroll
        for (int u = 0; u < L::NLW; u++) {
            const int row = (hp * L::NLW + u) * (1024 / L::RB) + lane / L::CPR;
            const int chunk = (lane % L::CPR) ^ L::fk(row);
            cx.gk_off[u] = ((k_tile_half(row) * L::CPR + chunk) * 16 + k_tile_slot(row)) * 16;
        }
        // Vt: rows of 64 bytes, four slots each; a KiB piece is 16 rows, and the
        // slot permutation sees the row's low four bits only
        const int vrow = lane / 4;
        cx.gv_off = vrow * 64 + ((lane & 3) ^ L::fv(vrow)) * 16;
        static_assert(L::fv(16) == L::fv(0), "the Vt slot permutation repeats every 16 rows");
        const int krow = prefill_key_perm(n);             // tile row this lane feeds to MFMA row n
        const uint32_t kread = krow * L::RB + ((g ^ L::fk(krow)) * 16);
        const uint32_t vread = n * 64 + ((g ^ L::fv(n)) * 16);
#pragma unroll
        for (int i = 0; i < HD / 16; i++) cx.kop[i] = (cx.ring + kread) ^ (i * 32);
#pragma unroll
        for (int t = 0; t < 2; t++) cx.vop[t] = cx.ring + L::V_IN_SET + (vread ^ (t * 32));
    }
    // steps of the loop: the even set's tile count (the odd set has as many or one
    // fewer and spends its last step on probabilities of zero); the same in every wave
    const uint32_t nsteps = (t_last - t_first) / 2 + 1;

    if (!started) pair_first_loads<HD, Q16>(cx, q, a, row0, head, n, g);

    f32x16 sa[2], sb[2];
    u32x4 pop[2][2];
    half8 kf[HD / 16], vf[HD / 16];
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    pair_convert_q<HD, Q16>(U[0].R, q[0], a);
    pair_convert_q<HD, Q16>(U[1].R, q[1], a);
    pair_patch_tail<HD, 0>(smem, cx, 0, lane, kv_valid);
    il_barrier();                                         // first tiles visible to all
    // scores of the set's first tile
#pragma unroll
    for (int i = 0; i < HD / 16; i++) kf[i] = *reinterpret_cast<const half8*>(smem + cx.kop[i]);
#pragma unroll
    for (int i = 0; i < HD / 16; i++)
#pragma unroll
        for (int u = 0; u < 2; u++) {
            if (i == 0)
                sa[u] = pair_mfma_first(kf[0], U[u].R.qop[0], U[u].negm);    // negm: zeros so far
            else
                pair_mfma_link(sa[u], kf[i], U[u].R.qop[i]);
        }
    il_barrier();                                         // slot 0 of K has been read by all: it is refilled
    pair_issue_k<HD, 0>(cx, 3);
#pragma unroll
    for (int i = 0; i < HD / 16; i++) kf[i] = *reinterpret_cast<const half8*>(smem + cx.kop[i] + L::KTILE);
    pair_settle<HD>(U[0], cx, sa[0], 0, g);
    pair_settle<HD>(U[1], cx, sa[1], 0, g);
    il_barrier();                                         // slot 1 of K has been read by all: step 0 refills it

#define WR_PAIR_STEP(PHASE, CUR, NXT)                                                  \
    pair_step<HD, PHASE>(U, cx, CUR, NXT, pop, kf, vf, smem, j, lane, g, kv_valid);    \
    if (++j >= nsteps) break;
#pragma unroll 1
    for (uint32_t j = 0;;) {
        WR_PAIR_STEP(0, sa, sb)
        WR_PAIR_STEP(1, sb, sa)
        WR_PAIR_STEP(2, sa, sb)
        WR_PAIR_STEP(0, sb, sa)
        WR_PAIR_STEP(1, sa, sb)
        WR_PAIR_STEP(2, sb, sa)
    }
#undef WR_PAIR_STEP

    // the ring must be quiet before anything else lands in it (the last steps'
    // copies still target it)
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    const int lane_e = il_fresh_lane();
    const int n_e = lane_e & 31, g_e = lane_e >> 5;
    if (next_pb >= 0) {
        PairCtx<HD> cn = cx;
        uint32_t nf, nl;
        pair_ctx_tiles<HD>(cn, a, (uint32_t)next_pb, BP, kg, nf, nl);
        const uint32_t nrow0[2] = {(uint32_t)next_pb * BP + sub_rows[0], (uint32_t)next_pb * BP + sub_rows[1]};
        pair_first_loads<HD, Q16>(cn, q, a, nrow0, head, n_e, g_e);
    }
    if (WR_PAIR_PROBE & 64) return;
    // the wave of key set s finishes unit s of its pair and hands the other one over
    if (kg == 0)
        pair_send<HD>(U[1], smem, wave, lane_e);
    else
        pair_send<HD>(U[0], smem, wave, lane_e);
    lds_barrier();                                        // LDS traffic only: the next block's loads stay in flight
    if (kg == 0)
        pair_finish<HD>(U[0], a, smem, wave ^ 2, lane_e, n_e, g_e);
    else
        pair_finish<HD>(U[1], a, smem, wave ^ 2, lane_e, n_e, g_e);
}

// grid = (KV heads x head chunks, ceil(blocks / 2)): consecutive workgroups (which
// the dispatcher deals round-robin to the XCDs) differ in KV head, so one XCD's
// L2 keeps seeing the same few heads' K / Vt.  Workgroup y takes position block
// (blocks-1-y) and then block y: a long block and a short one, so every
// workgroup streams the same number of tiles despite the causal triangle.
// a.single: grid.y = blocks, one block per workgroup, long blocks first.
template <int HD, bool Q16>
__global__ __launch_bounds__(kPairThreads, 1) void prefill_pair_kernel(const PrefillArgs a)
{
    extern __shared__ __attribute__((aligned(16))) unsigned char prefill_smem_raw[];
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
    PairQ<HD> q[2];
    if (a.single || hi == lo) {
        pair_block<HD, Q16>(a, prefill_smem_raw, hi, kvh, hc, kbase, vtbase, false, q, -1);
    } else {
        pair_block<HD, Q16>(a, prefill_smem_raw, hi, kvh, hc, kbase, vtbase, false, q, (int)lo);
        lds_barrier();                                    // LDS changes hands
        pair_block<HD, Q16>(a, prefill_smem_raw, lo, kvh, hc, kbase, vtbase, true, q, -1);
    }
}

}  // namespace wr
