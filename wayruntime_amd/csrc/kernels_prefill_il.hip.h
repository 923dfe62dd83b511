// Causal prefill attention on the matrix cores for head dims up to 128
// (v_mfma_f32_32x32x16_f16, F32 accumulate).  MFMA-bound: 4 * nq * hd flops per
// (query row, visible key).
//
// Semantics: kernels_prefill.hip.h (reference: the prefill loop
// src/core/session.c:615-625 over src/core/kernels.c:1475-1523).
//
// Workgroup = 8 waves = one KV head x 4 (head, 32-row block) pairs x 2 key sets:
// waves 0-3 take the even 32-key tiles of the block's key range, waves 4-7 the
// odd ones (split-K inside the workgroup, the two partial (m, l, O) triples merged
// through LDS at the end), two waves per SIMD at <= 256 registers each.  Per wave
// and tile, with the query row as the MFMA COLUMN (lane % 32):
//   S^T[key][row]  = K[key][:] . Q^T[:][row]          HD/16 MFMAs, a dependent chain
//   online softmax on the 16 scores a lane holds (+ one exchange with lane^32)
//   O^T[dim][row] += Vt[dim][key] . P^T[key][row]     HD/16 MFMAs
// K rows enter the first MFMA permuted so that the scores a lane ends up with are
// 8 consecutive keys per contraction step: P^T is then already the second MFMA's
// operand, and the matching Vt operand is one 16-byte read of the block-transposed
// V.  Q is rounded to F16 once, P per tile.  The softmax reference is lazy: it
// moves only when a row's maximum exceeds it by more than 2^kLazyLog2 (with 32
// independent rows per wave an eager maximum moves in most tiles and costs a
// 64-register rescale each time), and the score chain starts from a block of -m,
// so the scores come out with the reference already subtracted.
//
// Data movement: tiles travel from global memory straight into LDS
// (global_load_lds_dwordx4: no staging registers, no LDS store instructions), each
// set into its own ring of three tile slots, issued one step before the barrier
// that publishes them.  Such a copy writes a wave's 64 x 16 bytes to consecutive
// LDS addresses, so rows cannot be padded; the 16-byte chunks of a row are permuted
// instead (chunk c of row r sits at slot c ^ f(r)), on the global side where any
// permutation inside a row keeps the access coalesced; f is chosen so that the
// sixteen rows a 128-bit LDS read touches per cycle fall into sixteen different
// slots of the 256-byte bank row.  Copies are issued unconditionally (tile indices
// clamped to the block's last tile; duplicates land in slots nobody reads) so the
// number in flight is the same at every wait.
//
// Shape of a step.  A wave issues in order; what it issues right behind a matrix
// instruction runs in that instruction's shadow (about six instructions per
// 32x32x16 MFMA), and two waves of a SIMD that both keep a matrix instruction
// ready share the matrix pipe without leaving it idle.  So both key sets run in
// phase and every step is one stream in which each MFMA is followed by its share
// of the step's other work:
//
//   first half:   the score chain S(j+1) = K(j+1).Q^T, and behind each link one
//                 Vt operand read of tile j and a share of the exponentials and
//                 packs of S(j) (two score buffers alternate);
//   second half:  O^T += Vt(j).P(j)^T, and between the products the K operand
//                 reads of tile j+2 (the chain has consumed its own), the step's
//                 copies from global memory into LDS and the row maximum of
//                 S(j+1);
//   one hardware barrier per step publishes the copies that have landed and
//   frees the ring slots the next step overwrites.
//
// The loop is unrolled over the ring and the two score buffers (six step
// variants): slot offsets are immediates, operand addresses loop-invariant
// registers, and nothing is copied between steps.  Rare paths (masks at the
// diagonal and the window edge, a moving reference, the tail of the appended
// rows) are wave-uniform branches that update registers in place.
//
// A result of a matrix instruction must not be read by a vector instruction too
// early, and the hardware does not hold the reader back: the wait states are the
// compiler's job, and it does not look inside inline assembly.  Every
// hand-written instruction that touches scores is therefore ordered behind a
// compiler-visible read of them (il_max16).
#pragma once

#include "kernels_prefill.hip.h"

namespace wr {

constexpr int kSplitThreads = 512;
constexpr int kRing = 3;

template <int HD>
struct SplitLds {
    static constexpr int RB = 2 * HD;                     // bytes per K row
    static constexpr int CPR = HD / 8;                    // 16-byte chunks per K row
    static constexpr int RPB = 256 / RB > 0 ? 256 / RB : 1;   // K rows per 256-byte bank row
    static constexpr int KTILE = kTileKeys * RB;          // bytes of one tile's K
    static constexpr int VTILE = HD * kVBlock * 2;        // bytes of one tile's Vt block
    static constexpr int NL = KTILE / 1024 / 4;           // loads per wave and tile, each of K and Vt
    static constexpr int SET_BYTES = kRing * (KTILE + VTILE);   // one wave set's ring
    static constexpr int V_IN_SET = kRing * KTILE;        // Vt slots follow the K slots
    static constexpr int Q_OFF = 2 * SET_BYTES;           // Q staging, [4][32][HD + 8] halves
    static constexpr int Q_BYTES = 4 * 32 * (HD + 8) * 2;
    // Merge scratch (end of a block): at the end of the kernel's LDS, over the Q
    // staging (Q is in registers by then) and, where 160 KiB are not enough for
    // everything, over the tail of the odd set's last Vt slot.  It stays clear of
    // every slot the first copies of a block go to, so the next block's first
    // tiles can be on their way while this block is merged and stored.
    static constexpr int MERGE_BYTES = 4 * (HD / 2 + 2) * 64 * 4;
    static constexpr int LDS_MAX = 160 * 1024;
    static constexpr int MERGE_OFF = (Q_OFF + Q_BYTES + MERGE_BYTES <= LDS_MAX) ? Q_OFF + Q_BYTES
                                                                                : LDS_MAX - MERGE_BYTES;
    static constexpr int TOTAL = MERGE_OFF + MERGE_BYTES;
    static_assert(MERGE_OFF >= SET_BYTES + V_IN_SET + 2 * VTILE,
                  "merge scratch may overlap the odd set's third Vt slot only (no copy of a block's prologue lands there)");
    static_assert(KTILE == VTILE && NL >= 1, "one chunk schedule serves K and Vt");
    // slot permutation of K rows / Vt rows
    __device__ static constexpr int fk(int row) { return (row / RPB) & (CPR - 1); }
    __device__ static constexpr int fv(int row) { return (row >> 2) & 3; }
};

template <int HD>
constexpr size_t split_smem_bytes()
{
    return SplitLds<HD>::TOTAL;
}

// max of three without the canonicalising self-maximum the compiler puts in
// front of every fmaxf operand (the operands here are never signalling NaNs
// that anyone would want quieted)
__device__ __forceinline__ float max3_raw(float a, float b, float c)
{
    float r;
    asm("v_max3_f32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
    return r;
}

template <int HD>
struct IlCtx {
    // wave-uniform
    const unsigned char* kbase;       // this KV head's K / Vt, bytes
    const unsigned char* vtbase;
    uint32_t m0k, m0v;                // LDS byte address of this wave's first K / Vt copy in ring slot 0
    uint32_t t0, nt, t_last;          // the set's first tile and tile count, the block's last tile
    uint32_t tail_tile;               // tiles from this one on reach past the appended rows
    uint32_t jt_lo, jt_hi;            // set-local tile indices this wave's rows take part in (empty: lo > hi)
    uint32_t pl_lo, pl_hi;            // ... of which these are plain: every (row, key) pair visible
    uint32_t ring;                    // byte offset of the set's ring in the kernel's LDS
    // per lane
    uint32_t gk_off, gv_off;          // offset inside a K tile / Vt block of this lane's 16 bytes
    const unsigned char* kop[HD / 16];   // K operand read of contraction step i, ring slot 0
    const unsigned char* vop[2];         // Vt operand read of half t, dimension block 0, ring slot 0
    float thr;                        // a row maximum above this moves the softmax reference
};

// The set's tile with index jt, clamped to the block's last tile (copies past a
// set's range land in ring slots nobody reads, so the number in flight is fixed).
template <int HD>
__device__ __forceinline__ uint32_t il_tile(const IlCtx<HD>& cx, uint32_t jt)
{
    return min(cx.t0 + 2 * jt, cx.t_last);
}

// One of this wave's NL copies of the set's K tile jt / Vt block jt into ring slot SLOT.
template <int HD, int SLOT>
__device__ __forceinline__ void il_issue_k1(const IlCtx<HD>& cx, uint32_t jt, int u)
{
    using L = SplitLds<HD>;
    const unsigned char* src = cx.kbase + (size_t)il_tile(cx, jt) * L::KTILE;
    lds_direct_load(cx.m0k + SLOT * L::KTILE + u * 4096, src + u * 128, cx.gk_off);
}

template <int HD, int SLOT>
__device__ __forceinline__ void il_issue_v1(const IlCtx<HD>& cx, uint32_t jt, int u)
{
    using L = SplitLds<HD>;
    const unsigned char* src = cx.vtbase + (size_t)il_tile(cx, jt) * L::VTILE;
    lds_direct_load(cx.m0v + SLOT * L::VTILE + u * 4096, src + u * 4096, cx.gv_off);
}

template <int HD, int SLOT>
__device__ __forceinline__ void il_issue_k(const IlCtx<HD>& cx, uint32_t jt)
{
#pragma unroll
    for (int u = 0; u < SplitLds<HD>::NL; u++) il_issue_k1<HD, SLOT>(cx, jt, u);
}

template <int HD, int SLOT>
__device__ __forceinline__ void il_issue_v(const IlCtx<HD>& cx, uint32_t jt)
{
#pragma unroll
    for (int u = 0; u < SplitLds<HD>::NL; u++) il_issue_v1<HD, SLOT>(cx, jt, u);
}

// Zeroes, in the staged Vt of the set's tile jt (ring slot SLOT), the positions
// that were never appended: they may hold anything, and 0 * garbage must not
// reach the accumulator.  Every lane patches the chunks its own copies
// delivered, so only this wave's copies have to have landed.
template <int HD, int SLOT>
__device__ __forceinline__ void il_patch_tail(unsigned char* smem, const IlCtx<HD>& cx, uint32_t jt,
                                              int sub, int lane, uint32_t kv_valid)
{
    using L = SplitLds<HD>;
    const uint32_t tile = il_tile(cx, jt);
    if (tile < cx.tail_tile) return;
#pragma unroll
    for (int u = 0; u < L::NL; u++) {
        const int q = sub + 4 * u;
        const int row = q * 16 + lane / 4;                // Vt row (dimension)
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

__device__ __forceinline__ void il_barrier()
{
    __builtin_amdgcn_sched_barrier(0);
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
    __builtin_amdgcn_sched_barrier(0);
}

// Row maximum of the sixteen scores a lane holds, in one block of instructions
// (v_max3 without the canonicalising self-maximum a compiler-made maximum gets
// per operand, and without a hazard nop after every statement).
//
// The scores are the result of a matrix instruction, and the hardware does not
// hold back a vector instruction that reads such a result too early: the wait
// states are the compiler's job, and it does not look inside inline assembly.
// So the first instruction to touch the scores is one the compiler sees (an add
// of zero), and the block of maxima depends on its result; every other
// hand-written instruction on the scores is ordered behind this maximum.
__device__ __forceinline__ float il_max16(const f32x16& c)
{
    const float c0 = c[0] + 0.0f;
    float r;
    asm("v_max3_f32 %0, %1, %2, %3\n\t"
        "v_max3_f32 %0, %0, %4, %5\n\t"
        "v_max3_f32 %0, %0, %6, %7\n\t"
        "v_max3_f32 %0, %0, %8, %9\n\t"
        "v_max3_f32 %0, %0, %10, %11\n\t"
        "v_max3_f32 %0, %0, %12, %13\n\t"
        "v_max3_f32 %0, %0, %14, %15\n\t"
        "v_max_f32 %0, %0, %16"
        : "=&v"(r)
        : "v"(c0), "v"(c[1]), "v"(c[2]), "v"(c[3]), "v"(c[4]), "v"(c[5]), "v"(c[6]), "v"(c[7]), "v"(c[8]),
          "v"(c[9]), "v"(c[10]), "v"(c[11]), "v"(c[12]), "v"(c[13]), "v"(c[14]), "v"(c[15]));
    return r;
}

// Masks of a tile that is not plain for this wave (rare, wave-uniform branch).
// Both masks write the score registers in place, instruction by instruction:
// written as ordinary assignments they give the masked scores new registers,
// and the path that skips the masks (the one that matters) pays sixteen copies.
// `after`: the row maximum taken of `c` before (il_max16); naming it as an input
// keeps these hand-written instructions behind the first compiler-visible read
// of the matrix instruction's result.
template <int HD>
__device__ __forceinline__ void il_mask_special(const PrefillRows<HD>& R, const IlCtx<HD>& cx, f32x16& c,
                                                uint32_t tile, uint32_t jt, int g, float after)
{
    const float ninf = -INFINITY;
    asm volatile("" ::"v"(after));
    if (jt < cx.jt_lo || jt > cx.jt_hi) {
        // this wave's rows do not see the tile at all: probabilities of zero
#pragma unroll
        for (int r = 0; r < 16; r++) asm volatile("v_mov_b32 %0, %1" : "+v"(c[r]) : "v"(ninf), "v"(after));
    } else {
        // register r of this lane: key kb + 16*(r/8) + 8*g + r%8, row n; some
        // (row, key) pair of the tile is above the diagonal or below the window
        const uint32_t kb = tile * kTileKeys;
#pragma unroll
        for (int r = 0; r < 16; r++) {
            const uint32_t key = kb + 16 * (r >> 3) + 8 * g + (r & 7);
            const uint64_t hide = __builtin_amdgcn_ballot_w64(key > R.pos || key < R.row_lo);
            asm volatile("v_cndmask_b32 %0, %0, %1, %2" : "+v"(c[r]) : "v"(ninf), "s"(hide), "v"(after));
        }
    }
}

// The softmax reference of a row moves (rare, wave-uniform branch): this tile's
// scores are shifted, the accumulators rescaled and the block of -m rewritten.
template <int HD>
__device__ __forceinline__ void il_move_reference(PrefillRows<HD>& R, IlCtx<HD>& cx, f32x16& negm,
                                                  f32x16& c, float tmax, bool jump)
{
    const bool unset = (R.m_run == -INFINITY);
    const float delta = jump ? tmax : 0.f;
    const float alpha = jump ? (unset ? 0.f : fast_exp2(-delta)) : 1.0f;
    R.l_run *= alpha;
#pragma unroll
    for (int dt = 0; dt < HD / 32; dt++)
#pragma unroll
        for (int r = 0; r < 16; r++) R.o[dt][r] *= alpha;
    // updated in place with the instructions spelled out: left to itself the
    // compiler gives the updated values new registers and pays with 32 copies
    // on the path that skips this branch, which is the one that matters
#pragma unroll
    for (int r = 0; r < 16; r++) asm volatile("v_sub_f32 %0, %0, %1" : "+v"(c[r]) : "v"(delta));
    if (jump) R.m_run = (unset ? 0.f : R.m_run) + delta;
    const bool still = (R.m_run == -INFINITY);
    const float nm = still ? 0.f : -R.m_run;
#pragma unroll
    for (int r = 0; r < 16; r++) asm volatile("v_mov_b32 %0, %1" : "+v"(negm[r]) : "v"(nm));
    asm volatile("v_mov_b32 %0, %1" : "+v"(cx.thr) : "v"(still ? -INFINITY : kLazyLog2));
}

// The row maximum of the scores in `c` joined across the two lanes of a row and,
// rarely, a move of the row's reference.
template <int HD>
__device__ __forceinline__ void il_settle(PrefillRows<HD>& R, IlCtx<HD>& cx, f32x16& negm, f32x16& c, float tmax)
{
    {
        const uint32_t u = __float_as_uint(tmax);
        const auto sw = __builtin_amdgcn_permlane32_swap(u, u, false, false);
        tmax = max3_raw(__uint_as_float(sw[0]), __uint_as_float(sw[1]), tmax);   // same in both lanes of a row
    }
    const bool jump = tmax > cx.thr;                      // thr: -inf until the row has a reference, then kLazyLog2
    if (__builtin_amdgcn_ballot_w64(jump) != 0) il_move_reference<HD>(R, cx, negm, c, tmax, jump);
}

// Step j of a wave (P == j % kRing).  On entry `cur` holds the scores of the set's
// tile j (masked, reference settled), kf the K operands of tile j+1; on exit `nxt`
// holds the scores of tile j+1 in the same state and kf the operands of tile j+2.
template <int HD, int P>
__device__ __forceinline__ void il_step(PrefillRows<HD>& R, IlCtx<HD>& cx, f32x16& negm, const f32x16& cur,
                                        f32x16& nxt, u32x4 (&pop)[2], half8 (&kf)[HD / 16],
                                        half8 (&vf)[HD / 16], unsigned char* smem, uint32_t j, int sub,
                                        int lane, int g, uint32_t kv_valid)
{
    using L = SplitLds<HD>;
    constexpr int NS = HD / 16, ND = HD / 32;
    constexpr int PAIRS = 8 / NS;         // pairs of probabilities formed behind each link of the chain
    static_assert(kRing == 3 && 8 % NS == 0 && NS >= 2 * L::NL, "slot and interleave arithmetic below");
    constexpr int VS = P;                 // slot of Vt of tile j
    constexpr int KS = (P + 2) % 3;       // slot of K of tile j+2
    constexpr int KC = (P + 1) % 3;       // K of tile j+4 replaces K of tile j+1 (read in the previous step)
    constexpr int VC = (P + 2) % 3;       // Vt of tile j+2 replaces Vt of tile j-1 (read in the previous step)
    constexpr int TS = (P + 1) % 3;       // slot of Vt of tile j+1, whose tail is patched once it has landed

    float psum = 0.f;
    const half2v ones = {(_Float16)1.0f, (_Float16)1.0f};
#pragma unroll
    for (int i = 0; i < NS; i++) {
        if (i == 0)
            nxt = __builtin_amdgcn_mfma_f32_32x32x16_f16(kf[0], R.qop[0], negm, 0, 0, 0);
        else
            nxt = __builtin_amdgcn_mfma_f32_32x32x16_f16(kf[i], R.qop[i], nxt, 0, 0, 0);
        vf[i] = *reinterpret_cast<const half8*>(cx.vop[i / ND] + VS * L::VTILE + (i % ND) * 2048);
#pragma unroll
        for (int q = 0; q < PAIRS; q++) {
            // two exp2, one pack to F16, one dot product with (1, 1): the normaliser
            // is the sum of exactly the rounded values P.V multiplies
            const int r = 2 * (i * PAIRS + q);
            const half2v ph = {(_Float16)fast_exp2(cur[r]), (_Float16)fast_exp2(cur[r + 1])};
            psum = __builtin_amdgcn_fdot2(ph, ones, psum, false);
            pop[r >> 3][(r & 7) >> 1] = __builtin_bit_cast(uint32_t, ph);
        }
        // every link keeps its own share of the vector work behind it (left to
        // itself the scheduler bunches the exponentials behind the first links,
        // and both waves of a SIMD then leave the matrix pipe idle together)
        __builtin_amdgcn_sched_barrier(0);
    }
    R.l_run += psum;
#pragma unroll
    for (int i = 0; i < NS; i++) {
        const int t = i / ND, dt = i % ND;
        R.o[dt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(vf[i], __builtin_bit_cast(half8, pop[t]), R.o[dt], 0, 0,
                                                           0);
        kf[i] = *reinterpret_cast<const half8*>(cx.kop[i] + KS * L::KTILE);
        if (i < L::NL) il_issue_k1<HD, KC>(cx, j + 4, i);
        else if (i < 2 * L::NL) il_issue_v1<HD, VC>(cx, j + 2, i - L::NL);
    }
    // The row maximum runs in the products' shadow as if the tile were plain; a
    // tile with invisible (row, key) pairs is masked afterwards and its maximum
    // taken again (rare, wave-uniform).  Kept behind the products so that the
    // whole step up to here is one block the scheduler can interleave.
    float tmax = il_max16(nxt);
    const uint32_t jt = j + 1;
    if (jt < cx.pl_lo || jt > cx.pl_hi) {
        il_mask_special<HD>(R, cx, nxt, cx.t0 + 2 * jt, jt, g, tmax);
        tmax = il_max16(nxt);
    }
    il_settle<HD>(R, cx, negm, nxt, tmax);
    // all copies but this step's have landed: K of tile j+3 and Vt of tile j+1,
    // which the next step reads once the barrier has published them
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * L::NL) : "memory");
    il_patch_tail<HD, TS>(smem, cx, j + 1, sub, lane, kv_valid);
    // (no wait for this step's K operand reads here: their slot is not overwritten
    // before the step after next, long after the next chain has consumed them)
    __builtin_amdgcn_sched_barrier(0);
    asm volatile("s_barrier" ::: "memory");
    __builtin_amdgcn_sched_barrier(0);
}

// The lane's index, computed where it is asked for.  The step loop runs at the
// register limit; whatever the code after it derives from a lane index that
// was computed before it would have to live through the loop (or be spilled,
// and a reload waits for every load in flight, the next block's first tiles
// included).
__device__ __forceinline__ int il_fresh_lane()
{
    int l;
    asm volatile("v_mbcnt_lo_u32_b32 %0, -1, 0\n\tv_mbcnt_hi_u32_b32 %0, -1, %0" : "=v"(l));
    return l;
}

// Q rows of one wave (16 of the sub-block's 32), as read from global memory:
// every row is 4*HD contiguous bytes, read with whole-row coalesced loads.
template <int HD>
struct IlQRows {
    static constexpr int LPR = HD / 4;                    // lanes per row (one float4 each)
    static constexpr int RPI = 64 / LPR;                  // rows per load instruction
    float4 x[16 / RPI];
};

template <int HD>
__device__ __forceinline__ void il_load_q(IlQRows<HD>& q, const PrefillArgs& a, uint32_t row0, uint32_t head,
                                          int kg, int lane)
{
    using Q = IlQRows<HD>;
#pragma unroll
    for (int j = 0; j < 16 / Q::RPI; j++) {
        const int r = kg * 16 + j * Q::RPI + lane / Q::LPR;
        const uint32_t row = min(row0 + r, a.T - 1);      // idle rows re-read the last one
        const size_t at = ((size_t)row * a.nq + head) * HD + (lane % Q::LPR) * 4;
        if (a.q16 != nullptr) {                           // four finished halves: 8 bytes in .x and .y
            const uint2 h = *reinterpret_cast<const uint2*>(a.q16 + at);
            q.x[j] = make_float4(__uint_as_float(h.x), __uint_as_float(h.y), 0.f, 0.f);
        } else {
            q.x[j] = *reinterpret_cast<const float4*>(a.q + at);
        }
    }
}

// The tile range of position block pb for key set kg, into the context.
template <int HD>
__device__ __forceinline__ void il_ctx_tiles(IlCtx<HD>& cx, const PrefillArgs& a, uint32_t pb, uint32_t BP,
                                             int kg, uint32_t& t_first, uint32_t& t_last)
{
    prefill_block_tiles(a, pb, BP, t_first, t_last);
    cx.t0 = t_first + kg;                                 // this set's tiles: t0, t0 + 2, ...
    cx.nt = (cx.t0 <= t_last) ? (t_last - cx.t0) / 2 + 1 : 0;
    cx.t_last = t_last;
}

// The copies and loads a block starts with: the first three K tiles and two Vt
// blocks of the set into their ring slots, in order of need, and the wave's Q rows.
template <int HD>
__device__ __forceinline__ void il_first_loads(const IlCtx<HD>& cx, IlQRows<HD>& q, const PrefillArgs& a,
                                               uint32_t row0, uint32_t head, int kg, int lane)
{
    il_load_q<HD>(q, a, row0, head, kg, lane);
    il_issue_k<HD, 0>(cx, 0);
    il_issue_k<HD, 1>(cx, 1);
    il_issue_v<HD, 0>(cx, 0);
    il_issue_k<HD, 2>(cx, 2);
    il_issue_v<HD, 1>(cx, 1);
}

// One position block.  started: the block's first loads are already on their way
// (q holds its Q rows).  next_pb >= 0: once this block's loop is over, the first
// loads of block next_pb are issued, before the merge and the stores, and q
// returns its Q rows.
template <int HD>
__device__ __forceinline__ void il_block(const PrefillArgs& a, unsigned char* smem, uint32_t pb,
                                         uint32_t kvh, uint32_t hc, const unsigned char* kbase, const unsigned char* vtbase,
                                         bool started, IlQRows<HD>& q, int next_pb)
{
    using L = SplitLds<HD>;
    static_assert(L::NL == 1 || L::NL == 2, "one or two copies per wave, tile and operand");
    const int tid = threadIdx.x;
    const int lane = il_fresh_lane();                     // per call: nothing lane-derived is shared between the blocks of a workgroup
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);   // in a scalar register
    const int n = lane & 31, g = lane >> 5;
    const int kg = wave >> 2, sub = wave & 3;             // key set (tile parity), rows served
    const uint32_t G = a.group;
    const uint32_t Gw = G < 4 ? G : 4;
    const uint32_t BP = 32 * (4 / Gw);                    // positions per block
    // wave-uniform, and pinned to scalar registers: integer division runs on the
    // vector unit, and a quotient left there costs a vector register for the
    // whole block (or a spill)
    const uint32_t head = (uint32_t)__builtin_amdgcn_readfirstlane(kvh * G + hc * Gw + (sub % Gw));
    const uint32_t sub_rows = (uint32_t)__builtin_amdgcn_readfirstlane((sub / Gw) * 32);
    const uint32_t row0 = pb * BP + sub_rows;             // first chunk row of this wave
    const uint32_t kv_valid = a.p0 + a.T;                 // rows of the cache that hold data
    uint32_t t_first, t_last;

    PrefillRows<HD> R;
    prefill_rows_init<HD, false>(R, a, row0, head, n, g);

    IlCtx<HD> cx;
    il_ctx_tiles<HD>(cx, a, pb, BP, kg, t_first, t_last);
    cx.tail_tile = kv_valid / kTileKeys;
    cx.kbase = kbase;
    cx.vtbase = vtbase;
    cx.ring = kg * L::SET_BYTES;
    {
        // low half of a generic LDS pointer = LDS byte address
        const uint32_t lds0 = (uint32_t)__builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)smem);
        cx.m0k = lds0 + cx.ring + sub * 1024;
        cx.m0v = lds0 + cx.ring + L::V_IN_SET + sub * 1024;
        // set-local tile indices this wave's rows take part in
        const uint32_t lo_t = max(R.wt_first, cx.t0), hi_t = min(R.wt_last, t_last);
        if (R.wave_ok && cx.nt > 0 && lo_t <= hi_t && (lo_t - cx.t0 + 1) / 2 <= (hi_t - cx.t0) / 2) {
            cx.jt_lo = (lo_t - cx.t0 + 1) / 2;
            cx.jt_hi = (hi_t - cx.t0) / 2;
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
        if (cx.jt_lo <= cx.jt_hi && edge_hi >= 1 && edge_hi - 1 >= cx.t0) {
            const uint32_t lo = edge_lo > cx.t0 ? max(cx.jt_lo, (edge_lo - cx.t0 + 1) / 2) : cx.jt_lo;
            const uint32_t hi = min(cx.jt_hi, (edge_hi - 1 - cx.t0) / 2);
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
        // K: lane -> (row of the tile, slot); fetch the chunk that belongs in that slot
        const int row = sub * (1024 / L::RB) + lane / L::CPR;
        const int chunk = (lane % L::CPR) ^ L::fk(row);
        cx.gk_off = ((k_tile_half(row) * L::CPR + chunk) * 16 + k_tile_slot(row)) * 16;
        // Vt: rows of 64 bytes, four slots each
        const int vrow = sub * 16 + lane / 4;
        cx.gv_off = vrow * 64 + ((lane & 3) ^ L::fv(vrow)) * 16;
        static_assert(L::NL == 1 || (4 * (1024 / L::RB) == 16 && L::fk(16) == L::fk(0) && L::fv(64) == L::fv(0)),
                      "the second copy is 16 K rows (128 bytes in the cache) / 64 Vt rows (4 KiB) further");
        const int krow = prefill_key_perm(n);             // tile row this lane feeds to MFMA row n
        const uint32_t kread = krow * L::RB + ((g ^ L::fk(krow)) * 16);
        const uint32_t vread = n * 64 + ((g ^ L::fv(n)) * 16);
#pragma unroll
        for (int i = 0; i < HD / 16; i++) cx.kop[i] = smem + ((cx.ring + kread) ^ (i * 32));
#pragma unroll
        for (int t = 0; t < 2; t++) cx.vop[t] = smem + cx.ring + L::V_IN_SET + (vread ^ (t * 32));
    }
    cx.thr = -INFINITY;
    // steps of the loop: the even set's tile count (the odd set has as many or one
    // fewer and spends its last step on probabilities of zero); the same in every wave
    const uint32_t nsteps = (t_last - t_first) / 2 + 1;

    // everything the first two vector blocks read, in order of need, and Q
    if (!started) il_first_loads<HD>(cx, q, a, row0, head, kg, lane);

    // Q is converted to pre-scaled F16 and turned into the per-lane operand
    // layout through LDS (the two waves serving a sub-block take 16 rows each).
    _Float16 (*qs)[32][HD + 8] = reinterpret_cast<_Float16 (*)[32][HD + 8]>(smem + L::Q_OFF);
    {
        using Q = IlQRows<HD>;
#pragma unroll
        for (int j = 0; j < 16 / Q::RPI; j++) {
            const int r = kg * 16 + j * Q::RPI + lane / Q::LPR;
            const float4 x = q.x[j];
            if (a.q16 != nullptr) {
                *reinterpret_cast<uint2*>(&qs[sub][r][(lane % Q::LPR) * 4]) =
                    make_uint2(__float_as_uint(x.x), __float_as_uint(x.y));
            } else {
                *reinterpret_cast<half4*>(&qs[sub][r][(lane % Q::LPR) * 4]) = q_scaled_f16(x, a.qscale);
            }
            q.x[j] = make_float4(0.f, 0.f, 0.f, 0.f);      // consumed: nothing of it has to outlive the step loop
        }
    }
    f32x16 sa, sb, negm;
    u32x4 pop[2];
    half8 kf[HD / 16], vf[HD / 16];
#pragma unroll
    for (int r = 0; r < 16; r++) sa[r] = sb[r] = negm[r] = 0.f;
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    il_patch_tail<HD, 0>(smem, cx, 0, sub, lane, kv_valid);
    il_barrier();                                         // first tiles and Q visible to all
#pragma unroll
    for (int i = 0; i < HD / 16; i++)
        R.qop[i] = *reinterpret_cast<const half8*>(&qs[sub][n][i * 16 + g * 8]);
    // scores of the set's first tile
#pragma unroll
    for (int i = 0; i < HD / 16; i++) kf[i] = *reinterpret_cast<const half8*>(cx.kop[i]);
#pragma unroll
    for (int i = 0; i < HD / 16; i++)
        sa = __builtin_amdgcn_mfma_f32_32x32x16_f16(kf[i], R.qop[i], sa, 0, 0, 0);
    il_barrier();                                         // slot 0 of K has been read by all: it is refilled
    il_issue_k<HD, 0>(cx, 3);
#pragma unroll
    for (int i = 0; i < HD / 16; i++) kf[i] = *reinterpret_cast<const half8*>(cx.kop[i] + L::KTILE);
    {
        float tmax0 = il_max16(sa);
        if (0 < cx.pl_lo || 0 > cx.pl_hi) {
            il_mask_special<HD>(R, cx, sa, cx.t0, 0, g, tmax0);
            tmax0 = il_max16(sa);
        }
        il_settle<HD>(R, cx, negm, sa, tmax0);
    }
    il_barrier();                                         // slot 1 of K has been read by all: step 0 refills it

    // steps of the loop: the even set's tile count (the odd set has as many or one
    // fewer and spends its last step on probabilities of zero); the same in every
    // wave, and every step ends with the workgroup's barrier
#define WR_IL_STEP(PHASE, CUR, NXT)                                                          \
    il_step<HD, PHASE>(R, cx, negm, CUR, NXT, pop, kf, vf, smem, j, sub, lane, g, kv_valid); \
    if (++j >= nsteps) break;
#pragma unroll 1
    for (uint32_t j = 0;;) {
        WR_IL_STEP(0, sa, sb)
        WR_IL_STEP(1, sb, sa)
        WR_IL_STEP(2, sa, sb)
        WR_IL_STEP(0, sb, sa)
        WR_IL_STEP(1, sa, sb)
        WR_IL_STEP(2, sb, sa)
    }
#undef WR_IL_STEP

    // merge the odd-tile partials into the even-tile waves; the ring must be
    // quiet first (the last steps' copies still target it)
    constexpr int NREG = HD / 2;
    float* mg = reinterpret_cast<float*>(smem + L::MERGE_OFF) + (size_t)sub * (NREG + 2) * 64;
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    const int lane_e = il_fresh_lane();                   // lane, n, g again, for the code after the loop
    const int n_e = lane_e & 31, g_e = lane_e >> 5;
    if (next_pb >= 0) {
        // the rings are quiet and the merge below does not touch the slots these
        // go to: the next block's first tiles and Q rows travel while this block
        // is merged and stored
        IlCtx<HD> cn = cx;
        uint32_t nf, nl;
        il_ctx_tiles<HD>(cn, a, (uint32_t)next_pb, BP, kg, nf, nl);
        il_first_loads<HD>(cn, q, a, (uint32_t)next_pb * BP + sub_rows, head, kg, lane_e);
    }
    if (kg == 1) {
#pragma unroll
        for (int dt = 0; dt < HD / 32; dt++)
#pragma unroll
            for (int r = 0; r < 16; r++) mg[(dt * 16 + r) * 64 + lane_e] = R.o[dt][r];
        mg[NREG * 64 + lane_e] = R.m_run;
        mg[(NREG + 1) * 64 + lane_e] = R.l_run;
    }
    lds_barrier();                                        // LDS traffic only: the next block's loads stay in flight
    // rows leave through LDS as well: the merged tile is written row-major into
    // the sub-block's own scratch, then both of its waves store whole rows
    float (*os)[HD + 4] = reinterpret_cast<float (*)[HD + 4]>(mg);
    static_assert((size_t)32 * (HD + 4) <= (size_t)(NREG + 2) * 64, "row-major tile fits the merge scratch");
    if (kg == 0) {
        const float m1 = mg[NREG * 64 + lane_e], l1 = mg[(NREG + 1) * 64 + lane_e];
        const float m = fmaxf(R.m_run, m1);
        const float f0m = (R.m_run == -INFINITY) ? 0.f : fast_exp2(R.m_run - m);
        const float f1m = (m1 == -INFINITY) ? 0.f : fast_exp2(m1 - m);
        const float l_tot = wave_pair32_sum(R.l_run * f0m + l1 * f1m);
        const float inv = (l_tot > 0.f) ? 1.0f / l_tot : 0.f;
        const float w0 = f0m * inv, w1 = f1m * inv;
#pragma unroll
        for (int dt = 0; dt < HD / 32; dt++)
#pragma unroll
            for (int r = 0; r < 16; r++)
                R.o[dt][r] = R.o[dt][r] * w0 + mg[(dt * 16 + r) * 64 + lane_e] * w1;
        // the scratch has been read into registers; the same wave now reuses it
#pragma unroll
        for (int dt = 0; dt < HD / 32; dt++)
#pragma unroll
            for (int q4 = 0; q4 < 4; q4++) {
                float4 v;
                v.x = R.o[dt][4 * q4 + 0];
                v.y = R.o[dt][4 * q4 + 1];
                v.z = R.o[dt][4 * q4 + 2];
                v.w = R.o[dt][4 * q4 + 3];
                *reinterpret_cast<float4*>(&os[n_e][dt * 32 + 8 * q4 + 4 * g_e]) = v;
            }
    }
    lds_barrier();
    {
        constexpr int LPR = HD / 4;                       // lanes per row (one float4 each)
        constexpr int RPI = 64 / LPR;                     // rows per store instruction
#pragma unroll
        for (int j = 0; j < 16 / RPI; j++) {
            const int r = kg * 16 + j * RPI + lane_e / LPR;
            const float4 v = *reinterpret_cast<const float4*>(&os[r][(lane_e % LPR) * 4]);
            if (row0 + r < a.T)
                *reinterpret_cast<float4*>(a.out + ((size_t)(row0 + r) * a.nq + head) * HD +
                                           (lane_e % LPR) * 4) = v;
        }
    }
}

// grid = (KV heads x head chunks, ceil(blocks / 2)): consecutive workgroups (which
// the dispatcher deals round-robin to the XCDs) differ in KV head, so one XCD's
// L2 keeps seeing the same few heads' K / Vt.  Workgroup y takes position block
// (blocks-1-y) and then block y: a long block and a short one, so every
// workgroup streams the same number of tiles despite the causal triangle.
// a.single: grid.y = blocks, one block per workgroup, long blocks first.
template <int HD>
__global__ __launch_bounds__(kSplitThreads, 1) void prefill_il_kernel(const PrefillArgs a)
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
    // this KV head's K / Vt, in scalar registers for both blocks
    const unsigned char* kbase =
        uniform_ptr(reinterpret_cast<const unsigned char*>(a.k + (size_t)kvh * a.ctx_pad * HD));
    const unsigned char* vtbase = uniform_ptr(reinterpret_cast<const unsigned char*>(
        a.vt + (size_t)kvh * (a.ctx_pad / kVBlock) * HD * kVBlock));
    IlQRows<HD> q;
    if (a.single || hi == lo) {
        il_block<HD>(a, prefill_smem_raw, hi, kvh, hc, kbase, vtbase, false, q, -1);
    } else {
        il_block<HD>(a, prefill_smem_raw, hi, kvh, hc, kbase, vtbase, false, q, (int)lo);
        lds_barrier();                                    // LDS changes hands
        il_block<HD>(a, prefill_smem_raw, lo, kvh, hc, kbase, vtbase, true, q, -1);
    }
}

}  // namespace wr
