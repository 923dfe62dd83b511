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
    static constexpr int ML_WAVE = 256;                   // floats per wave: m[64], l[64], w0[32], w1[32], spare
    // Q staging (start of a block, before anything is exchanged): the block's
    // rows as pre-scaled F16, [4 units][32 rows][HD + 8], over the exchange scratch
    static constexpr int QS_OFF = X_OFF;
    static constexpr int QS_ROW = (HD + 8) * 2;
    static constexpr int QS_BYTES = 4 * 32 * QS_ROW;
    // per-wave scratch of the rare rescale (32 floats), clear of the Q staging
    static constexpr int RS_OFF = X_OFF + 3 * X_WAVE + X_WAVE / 2;
    static_assert(KTILE == VTILE && NLW >= 1, "one piece schedule serves K and Vt");
    static_assert(4 * ML_WAVE * 4 <= VTILE, "the exchange's scalars of four waves fit a Vt slot");
    static_assert(QS_BYTES <= 3 * X_WAVE + X_WAVE / 2, "Q staging ends below the rescale scratch");
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
    if (__builtin_expect(tile < cx.tail_tile, 1)) return;
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

// The softmax reference of a row moves (rare, wave-uniform branch).  The output
// accumulators hold O[query][dim] (a lane: one dimension of sixteen queries), the
// factors belong to queries (a lane of the score layout: one query): they cross
// over through 32 floats of LDS, and only when some row that already has a
// reference moves it (a row without one has an all-zero accumulator).
template <int HD>
__device__ __forceinline__ void pair_move_reference(PairUnit<HD>& U, f32x16& c, float tmax, bool jump,
                                                    unsigned char* smem)
{
    using L = PairLds<HD>;
    PrefillRows<HD>& R = U.R;
    const bool unset = (R.m_run == -INFINITY);
    const float delta = jump ? tmax : 0.f;
    const float alpha = jump ? (unset ? 0.f : fast_exp2(-delta)) : 1.0f;
    R.l_run *= alpha;
    if (__builtin_amdgcn_ballot_w64(jump && !unset) != 0) {
        // The accumulators are results of hand-written matrix instructions, the
        // last of them issued just before this branch, and the compiler puts no
        // wait states in front of the reads below: wait for the matrix pipe here.
        asm volatile("s_nop 15\n\ts_nop 15\n\ts_nop 15\n\ts_nop 15" ::: "memory");
        const int lane = il_fresh_lane();
        const int n = lane & 31, g = lane >> 5;
        const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
        float* sc = reinterpret_cast<float*>(smem + L::RS_OFF) + wave * 32;
        if (g == 0) sc[n] = alpha;
#pragma unroll
        for (int q4 = 0; q4 < 4; q4++) {
            const f32x4 av = *reinterpret_cast<const f32x4*>(sc + 8 * q4 + 4 * g);
#pragma unroll
            for (int dt = 0; dt < HD / 32; dt++)
#pragma unroll
                for (int e = 0; e < 4; e++) R.o[dt][4 * q4 + e] *= av[e];
        }
    }
#pragma unroll
    for (int r = 0; r < 16; r++) asm volatile("v_sub_f32 %0, %0, %1" : "+v"(c[r]) : "v"(delta));
    if (jump) R.m_run = (unset ? 0.f : R.m_run) + delta;
    const bool still = (R.m_run == -INFINITY);
    const float nm = still ? 0.f : -R.m_run;
#pragma unroll
    for (int r = 0; r < 16; r++) asm volatile("v_mov_b32 %0, %1" : "+v"(U.negm[r]) : "v"(nm));
    asm volatile("v_mov_b32 %0, %1" : "+v"(U.thr) : "v"(still ? -INFINITY : kLazyLog2));
}

// Settling the scores of a tile, first half: masks where the tile is not plain
// for the unit (rare, wave-uniform branch), then the row maximum of the sixteen
// scores a lane holds.
template <int HD>
__device__ __forceinline__ void pair_settle_a(PairUnit<HD>& U, const PairCtx<HD>& cx, f32x16& c, uint32_t jt, int g,
                                              float& tmax)
{
    if (jt < U.pl_lo || jt > U.pl_hi) pair_mask_special<HD>(U, c, cx.t0 + 2 * jt, jt, g, 0.f);
    tmax = il_max16(c);
}

// Second half: the maximum joined across the two lanes of a row and, rarely, a
// move of the row's reference.
template <int HD>
__device__ __forceinline__ void pair_settle_b(float& tmax)
{
    const uint32_t u = __float_as_uint(tmax);
    const auto sw = __builtin_amdgcn_permlane32_swap(u, u, false, false);
    tmax = max3_raw(__uint_as_float(sw[0]), __uint_as_float(sw[1]), tmax);
}

// Third part: which rows' maxima exceed the threshold, as a lane mask in scalar
// registers, made slots before the step's end looks at it (a scalar branch on a
// comparison made just before it waits for the vector pipe to drain).
__device__ __forceinline__ uint64_t pair_settle_jumps(float tmax, float thr)
{
    uint64_t m;
    asm volatile("v_cmp_gt_f32 %0, %1, %2" : "=s"(m) : "v"(tmax), "v"(thr));
    return m;
}

// Last part, behind the step's products: the rare move.
template <int HD>
__device__ __forceinline__ void pair_settle_c(PairUnit<HD>& U, f32x16& c, float tmax, unsigned char* smem)
{
    const bool jump = tmax > U.thr;
    if (__builtin_amdgcn_ballot_w64(jump) != 0) pair_move_reference<HD>(U, c, tmax, jump, smem);
}

template <int HD>
__device__ __forceinline__ void pair_settle(PairUnit<HD>& U, const PairCtx<HD>& cx, f32x16& c, uint32_t jt, int g,
                                            unsigned char* smem)
{
    float tmax;
    pair_settle_a<HD>(U, cx, c, jt, g, tmax);
    pair_settle_b<HD>(tmax);
    pair_settle_c<HD>(U, c, tmax, smem);
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

// A link of a score chain and, in its shadow, a pair of scores of the tile before
// turned into probabilities: two exponentials (in place), their sum into the row
// sum, the rounded pair.  An exponential's result may be read by another kind of
// vector instruction only one instruction later: the order below keeps that.
__device__ __forceinline__ void pair_slot_chain(f32x16& d, half8 a, half8 b, f32x16& sc, int r, float& ps,
                                                u32x4& pk4, int e)
{
    asm volatile("v_mfma_f32_32x32x16_f16 %0, %5, %6, %0\n\t"
                 "v_exp_f32 %1, %1\n\t"
                 "v_exp_f32 %2, %2\n\t"
                 "v_add_f32 %3, %3, %1\n\t"
                 "v_add_f32 %3, %3, %2\n\t"
                 "v_cvt_pk_f16_f32 %4, %1, %2"
                 : "+v"(d), "+v"(sc[r]), "+v"(sc[r + 1]), "+v"(ps), "=v"(pk4[e])
                 : "a"(a), "a"(b));
}

__device__ __forceinline__ void pair_slot_chain_first(f32x16& d, half8 a, half8 b, const f32x16& c, f32x16& sc,
                                                      int r, float& ps, u32x4& pk4, int e)
{
    asm volatile("v_mfma_f32_32x32x16_f16 %0, %5, %6, %7\n\t"
                 "v_exp_f32 %1, %1\n\t"
                 "v_exp_f32 %2, %2\n\t"
                 "v_add_f32 %3, %3, %1\n\t"
                 "v_add_f32 %3, %3, %2\n\t"
                 "v_cvt_pk_f16_f32 %4, %1, %2"
                 : "=&v"(d), "+v"(sc[r]), "+v"(sc[r + 1]), "+v"(ps), "=v"(pk4[e])
                 : "a"(a), "a"(b), "v"(c));
}

// A product and, in its shadow, the first / second half of the row maximum of
// sixteen scores.
__device__ __forceinline__ void pair_slot_pv_max_a(f32x16& o, half8 a, half8 b, float& t, const f32x16& c)
{
    asm volatile("v_mfma_f32_32x32x16_f16 %0, %2, %3, %0\n\t"
                 "v_max3_f32 %1, %4, %5, %6\n\t"
                 "v_max3_f32 %1, %1, %7, %8\n\t"
                 "v_max3_f32 %1, %1, %9, %10\n\t"
                 "v_max3_f32 %1, %1, %11, %12"
                 : "+a"(o), "=&v"(t)
                 : "v"(a), "v"(b), "v"(c[0]), "v"(c[1]), "v"(c[2]), "v"(c[3]), "v"(c[4]), "v"(c[5]), "v"(c[6]),
                   "v"(c[7]), "v"(c[8]));
}

__device__ __forceinline__ void pair_slot_pv_max_b(f32x16& o, half8 a, half8 b, float& t, const f32x16& c)
{
    asm volatile("v_mfma_f32_32x32x16_f16 %0, %2, %3, %0\n\t"
                 "v_max3_f32 %1, %1, %4, %5\n\t"
                 "v_max3_f32 %1, %1, %6, %7\n\t"
                 "v_max3_f32 %1, %1, %8, %9\n\t"
                 "v_max_f32 %1, %1, %10"
                 : "+a"(o), "+v"(t)
                 : "v"(a), "v"(b), "v"(c[9]), "v"(c[10]), "v"(c[11]), "v"(c[12]), "v"(c[13]), "v"(c[14]),
                   "v"(c[15]));
}

// A product that names a value made by the statements before it, so that those
// stay in front of it.
__device__ __forceinline__ void pair_mfma_acc_after(f32x16& d, half8 a, half8 b, float& after)
{
    asm volatile("v_mfma_f32_32x32x16_f16 %0, %2, %3, %0" : "+a"(d), "+v"(after) : "v"(a), "v"(b));
}

// Step j of a wave (P == j % kRing).  On entry cur[u] holds unit u's scores of the
// set's tile j (masked, reference settled), kf the K operands of tile j+1; on exit
// nxt[u] holds the scores of tile j+1 in the same state and kf the operands of
// tile j+2.
template <int HD, int P>
__device__ __forceinline__ void pair_step(PairUnit<HD> (&U)[2], const PairCtx<HD>& cx, f32x16 (&cur)[2],
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

    // One slot per matrix instruction, each slot one block of hand-ordered
    // instructions: what follows a matrix instruction in its block is issued in
    // that instruction's shadow.  (Left as ordinary statements between pinned
    // matrix instructions, the additions and part of the exponentials were sunk
    // to the end of the step by the compiler, where nothing overlaps them.)
    //
    // Row sums by plain additions of the unrounded exponentials: a dot-product
    // instruction (v_dot2c_f32_f16 on the rounded pair) runs on the matrix pipe
    // and waits for the matrix instruction in front of it, which a lone wave
    // cannot afford (measured: MFMA + 2 dot2c = 55 clocks, MFMA + 6 additions = 36).
    static_assert(PAIRS == 1, "slot blocks below are written for one pair of scores per link");
    float psum[2] = {0.f, 0.f};
#pragma unroll
    for (int i = 0; i < NS; i++) {
#pragma unroll
        for (int u = 0; u < 2; u++) {
            const int r = 2 * i;
            if (i == 0)
                pair_slot_chain_first(nxt[u], kf[0], U[u].R.qop[0], U[u].negm, cur[u], r, psum[u], pop[u][r >> 3],
                                      (r & 7) >> 1);
            else
                pair_slot_chain(nxt[u], kf[i], U[u].R.qop[i], cur[u], r, psum[u], pop[u][r >> 3], (r & 7) >> 1);
            if (u == 0)
                vf[i] = *reinterpret_cast<const half8*>(smem + cx.vop[i / ND] + VS * L::VTILE + (i % ND) * 2048);
            __builtin_amdgcn_sched_barrier(0);
        }
    }
    U[0].R.l_run += psum[0];
    U[1].R.l_run += psum[1];
    // The products, and in their shadows the K operand reads of tile j+2, the
    // step's copies and the settling of S(j+1).  The scores of tile j+1 are results
    // of hand-written matrix instructions: nothing may read them before two more
    // matrix instructions have been issued behind the last link (the compiler knows
    // of no wait states here).
    float tmax[2] = {0.f, 0.f};
    uint64_t jumps[2] = {0, 0};
    constexpr int S0 = 2, S1 = 6;         // slots behind which unit 0 / unit 1 settle (three slots each)
#pragma unroll
    for (int s = 0; s < 2 * NS; s++) {
        const int i = s / 2, u = s % 2;
        const int t = i / ND, dt = i % ND;
        const half8 pp = __builtin_bit_cast(half8, pop[u][t]);
        if (s == S0 || s == S1) {
            const int w = (s == S0) ? 0 : 1;
            const uint32_t jt = j + 1;
            if (__builtin_expect(jt < U[w].pl_lo || jt > U[w].pl_hi, 0))
                pair_mask_special<HD>(U[w], nxt[w], cx.t0 + 2 * jt, jt, g, 0.f);
            pair_slot_pv_max_a(U[u].R.o[dt], pp, vf[i], tmax[w], nxt[w]);
        } else if (s == S0 + 1 || s == S1 + 1) {
            const int w = (s == S0 + 1) ? 0 : 1;
            pair_slot_pv_max_b(U[u].R.o[dt], pp, vf[i], tmax[w], nxt[w]);
        } else if (s == S0 + 2 || s == S1 + 2) {
            const int w = (s == S0 + 2) ? 0 : 1;
            pair_mfma_acc(U[u].R.o[dt], pp, vf[i]);
            pair_settle_b<HD>(tmax[w]);
        } else if (s == S0 + 3 || s == S1 + 3) {
            // (the joined maximum is an operand, so that it is made in the slot before)
            const int w = (s == S0 + 3) ? 0 : 1;
            pair_mfma_acc_after(U[u].R.o[dt], pp, vf[i], tmax[w]);
            jumps[w] = pair_settle_jumps(tmax[w], U[w].thr);
        } else {
            pair_mfma_acc(U[u].R.o[dt], pp, vf[i]);
        }
        if (u == 0) {
            kf[i] = *reinterpret_cast<const half8*>(smem + cx.kop[i] + KS * L::KTILE);
        } else {
            if (i < L::NLW) pair_issue_k1<HD, KC>(cx, j + 4, i);
            else if (i < 2 * L::NLW) pair_issue_v1<HD, VC>(cx, j + 2, i - L::NLW);
        }
        __builtin_amdgcn_sched_barrier(0);
    }
    if (__builtin_expect((jumps[0] | jumps[1]) != 0, 0)) {
        pair_settle_c<HD>(U[0], nxt[0], tmax[0], smem);
        pair_settle_c<HD>(U[1], nxt[1], tmax[1], smem);
    }
    // all copies but this step's have landed: K of tile j+3 and Vt of tile j+1,
    // which the next step reads once the barrier has published them
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * L::NLW) : "memory");
    pair_patch_tail<HD, TS>(smem, cx, j + 1, lane, kv_valid);
    __builtin_amdgcn_sched_barrier(0);
    asm volatile("s_barrier" ::: "memory");
    __builtin_amdgcn_sched_barrier(0);
}

// Q rows as read from global memory: wave w brings in the 32 rows of unit w with
// whole-row coalesced loads (a lane per row reads 64 different cache lines per
// instruction and takes four times as long to get through the vector cache).
template <int HD, bool Q16>
struct PairQ {
    static constexpr int LPR = Q16 ? HD / 8 : HD / 4;     // lanes per row (16 bytes each)
    static constexpr int RPI = 64 / LPR;                  // rows per load instruction
    static constexpr int NI = 32 / RPI;
    float4 x[NI];
};

template <int HD, bool Q16>
__device__ __forceinline__ void pair_load_q(PairQ<HD, Q16>& q, const PrefillArgs& a, uint32_t row0, uint32_t head,
                                            int lane)
{
    using Q = PairQ<HD, Q16>;
#pragma unroll
    for (int j = 0; j < Q::NI; j++) {
        const int r = j * Q::RPI + lane / Q::LPR;
        const uint32_t row = min(row0 + r, a.T - 1);      // idle rows re-read the last one
        if constexpr (Q16) {
            const size_t at = ((size_t)row * a.nq + head) * HD + (lane % Q::LPR) * 8;
            const uint4 h = *reinterpret_cast<const uint4*>(a.q16 + at);
            q.x[j] = make_float4(__uint_as_float(h.x), __uint_as_float(h.y), __uint_as_float(h.z),
                                 __uint_as_float(h.w));
        } else {
            const size_t at = ((size_t)row * a.nq + head) * HD + (lane % Q::LPR) * 4;
            q.x[j] = *reinterpret_cast<const float4*>(a.q + at);
        }
    }
}

// The rows of unit `unit` (this wave's index) scaled, rounded and written into
// the staging image, [unit][row][HD + 8] halves.
template <int HD, bool Q16>
__device__ __forceinline__ void pair_stage_q(PairQ<HD, Q16>& q, const PrefillArgs& a, unsigned char* smem, int unit,
                                             int lane)
{
    using L = PairLds<HD>;
    using Q = PairQ<HD, Q16>;
#pragma unroll
    for (int j = 0; j < Q::NI; j++) {
        const int r = j * Q::RPI + lane / Q::LPR;
        unsigned char* at = smem + L::QS_OFF + (unit * 32 + r) * L::QS_ROW + (lane % Q::LPR) * (Q16 ? 16 : 8);
        if constexpr (Q16)
            *reinterpret_cast<float4*>(at) = q.x[j];
        else
            *reinterpret_cast<half4*>(at) = q_scaled_f16(q.x[j], a.qscale);
        q.x[j] = make_float4(0.f, 0.f, 0.f, 0.f);          // consumed: nothing of it has to outlive the step loop
    }
}

// The Q^T operand of a unit out of the staging image: the lane's row, eight
// consecutive dimensions per contraction step.
template <int HD>
__device__ __forceinline__ void pair_read_q(PrefillRows<HD>& R, const unsigned char* smem, int unit, int n, int g)
{
    using L = PairLds<HD>;
#pragma unroll
    for (int i = 0; i < HD / 16; i++)
        R.qop[i] = pair_to_acc(*reinterpret_cast<const half8*>(smem + L::QS_OFF + (unit * 32 + n) * L::QS_ROW +
                                                               (i * 16 + g * 8) * 2));
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
// blocks of the set into their ring slots, in order of need, and the wave's share
// of the Q rows.
template <int HD, bool Q16>
__device__ __forceinline__ void pair_first_loads(const PairCtx<HD>& cx, PairQ<HD, Q16>& q, const PrefillArgs& a,
                                                 uint32_t qrow0, uint32_t qhead, int lane)
{
    pair_issue_k<HD, 0>(cx, 0);
    pair_load_q<HD, Q16>(q, a, qrow0, qhead, lane);
    pair_issue_v<HD, 0>(cx, 0);
    pair_issue_k<HD, 1>(cx, 1);
    pair_issue_k<HD, 2>(cx, 2);
    pair_issue_v<HD, 1>(cx, 1);
}

// End of a block.  The wave of key set s finishes unit s of its pair: the other
// unit's partial goes into this wave's scratch for the partner (pair_send), and
// after the barrier the partner's partial of this wave's unit is merged in,
// normalised and stored (pair_finish).  The accumulators hold O[query][dim], so a
// store instruction writes 128 contiguous bytes of two rows; the per-query
// weights cross over from the score layout through 64 floats of LDS.
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
    float* ml = reinterpret_cast<float*>(smem + L::ML_OFF) + wave * L::ML_WAVE;
    ml[lane] = U.R.m_run;
    ml[64 + lane] = U.R.l_run;
}

template <int HD, bool GUARD>
__device__ __forceinline__ void pair_finish_rows(PairUnit<HD>& U, const PrefillArgs& a, const f32x4* x,
                                                 const float* wsc, int lane, int n, int g)
{
    PrefillRows<HD>& R = U.R;
    const size_t rowstride = (size_t)a.nq * HD;
    float* ob = a.out + ((size_t)min(U.row0 + 4 * g, a.T - 1) * a.nq + U.head) * HD + n;
#pragma unroll
    for (int q4 = 0; q4 < 4; q4++) {
        const f32x4 w0v = *reinterpret_cast<const f32x4*>(wsc + 8 * q4 + 4 * g);
        const f32x4 w1v = *reinterpret_cast<const f32x4*>(wsc + 32 + 8 * q4 + 4 * g);
#pragma unroll
        for (int dt = 0; dt < HD / 32; dt++) {
            const f32x4 p = x[(dt * 4 + q4) * 64 + lane];
#pragma unroll
            for (int e = 0; e < 4; e++) {
                const float v = R.o[dt][4 * q4 + e] * w0v[e] + p[e] * w1v[e];
                const uint32_t row = U.row0 + 8 * q4 + 4 * g + e;
                if (!GUARD || row < a.T) ob[(size_t)(8 * q4 + e) * rowstride + dt * 32] = v;
            }
        }
        __builtin_amdgcn_sched_barrier(0);                // a quarter of the registers at a time
    }
}

template <int HD>
__device__ __forceinline__ void pair_finish(PairUnit<HD>& U, const PrefillArgs& a, unsigned char* smem, int wave,
                                            int lane, int n, int g)
{
    using L = PairLds<HD>;
    PrefillRows<HD>& R = U.R;
    const int partner = wave ^ 2;
    const f32x4* x = reinterpret_cast<const f32x4*>(smem + L::X_OFF + partner * L::X_WAVE);
    const float* ml = reinterpret_cast<const float*>(smem + L::ML_OFF) + partner * L::ML_WAVE;
    const float m1 = ml[lane], l1 = ml[64 + lane];
    const float m = fmaxf(R.m_run, m1);
    const float f0m = (R.m_run == -INFINITY) ? 0.f : fast_exp2(R.m_run - m);
    const float f1m = (m1 == -INFINITY) ? 0.f : fast_exp2(m1 - m);
    const float l_tot = wave_pair32_sum(R.l_run * f0m + l1 * f1m);
    const float inv = (l_tot > 0.f) ? 1.0f / l_tot : 0.f;
    // the weights of query n, to where the lanes that hold its outputs read them
    float* wsc = reinterpret_cast<float*>(smem + L::ML_OFF) + wave * L::ML_WAVE + 128;
    if (g == 0) {
        wsc[n] = f0m * inv;
        wsc[32 + n] = f1m * inv;
    }
    if (U.row0 + 32 <= a.T)
        pair_finish_rows<HD, false>(U, a, x, wsc, lane, n, g);
    else
        pair_finish_rows<HD, true>(U, a, x, wsc, lane, n, g);
}

// One position block.  started: the block's first loads are already on their way
// (q holds its Q rows).  next_pb >= 0: once this block's loop is over, the first
// loads of block next_pb are issued, before the exchange and the stores, and q
// returns its Q rows.
template <int HD, bool Q16>
__device__ __forceinline__ void pair_block(const PrefillArgs& a, unsigned char* smem, uint32_t pb, uint32_t kvh,
                                           uint32_t hc, const unsigned char* kbase, const unsigned char* vtbase,
                                           bool started, PairQ<HD, Q16>& q, int next_pb)
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

    // Q rows: wave w brings in unit w
    const uint32_t qhead = (uint32_t)__builtin_amdgcn_readfirstlane(kvh * G + hc * Gw + ((uint32_t)wave % Gw));
    const uint32_t qsub = (uint32_t)__builtin_amdgcn_readfirstlane(((uint32_t)wave / Gw) * 32);
    if (!started) pair_first_loads<HD, Q16>(cx, q, a, pb * BP + qsub, qhead, lane);

    f32x16 sa[2], sb[2];
    u32x4 pop[2][2];
    half8 kf[HD / 16], vf[HD / 16];
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    pair_stage_q<HD, Q16>(q, a, smem, wave, lane);
    pair_patch_tail<HD, 0>(smem, cx, 0, lane, kv_valid);
    il_barrier();                                         // first tiles and Q rows visible to all
    pair_read_q<HD>(U[0].R, smem, 2 * hp, n, g);
    pair_read_q<HD>(U[1].R, smem, 2 * hp + 1, n, g);
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
    pair_settle<HD>(U[0], cx, sa[0], 0, g, smem);
    pair_settle<HD>(U[1], cx, sa[1], 0, g, smem);
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
        pair_first_loads<HD, Q16>(cn, q, a, (uint32_t)next_pb * BP + qsub, qhead, lane_e);
    }
    // the wave of key set s finishes unit s of its pair and hands the other one over
    if (kg == 0)
        pair_send<HD>(U[1], smem, wave, lane_e);
    else
        pair_send<HD>(U[0], smem, wave, lane_e);
    lds_barrier();                                        // LDS traffic only: the next block's loads stay in flight
    if (kg == 0)
        pair_finish<HD>(U[0], a, smem, wave, lane_e, n_e, g_e);
    else
        pair_finish<HD>(U[1], a, smem, wave, lane_e, n_e, g_e);
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
    PairQ<HD, Q16> q;
    const bool two = !(a.single || hi == lo);
    // one copy of the block's code for both blocks: the kernel's instructions
    // have to come through an instruction cache two compute units share
    uint32_t pb = hi;
    bool started = false;
#pragma unroll 1
    for (int b = 0;; b++) {
        const int next = (b == 0 && two) ? (int)lo : -1;
        pair_block<HD, Q16>(a, prefill_smem_raw, pb, kvh, hc, kbase, vtbase, started, q, next);
        if (next < 0) break;
        lds_barrier();                                    // LDS changes hands
        pb = lo;
        started = true;
    }
}

}  // namespace wr
