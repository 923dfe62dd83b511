// Causal prefill attention on the matrix cores: both key sets of a workgroup in
// phase, every wave's matrix instructions spread evenly through its step.
//
// Same semantics, workgroup shape, LDS image and arithmetic as
// kernels_prefill_pp.hip.h (8 waves = one KV head x 4 (head, 32-row block) pairs
// x 2 key sets, ring of three tile slots per set, lazy softmax reference, the
// sets' partials merged through LDS).  What differs is the shape of a step.  A
// wave issues in order; what it issues right behind a matrix instruction runs
// in that instruction's shadow (about six instructions per 32x32x16 MFMA), and
// two waves of a SIMD that both keep a matrix instruction ready share the
// matrix pipe without leaving it idle.  So every step is one stream in which
// each MFMA is followed by its share of the step's other work:
//
//   first half:   the score chain S(j+1) = K(j+1).Q^T, and between its links the
//                 Vt operand reads of tile j and the exponentials, packs and
//                 row sums of S(j) (two score buffers alternate);
//   second half:  O^T += Vt(j).P(j)^T, and between the products the K operand
//                 reads of tile j+2 (the chain has consumed its own), the step's
//                 copies from global memory into LDS and the row maximum of
//                 S(j+1);
//   one hardware barrier per step publishes the copies that have landed and
//   frees the ring slots the next step overwrites.
//
// The loop is unrolled over the ring and the two score buffers (six step
// variants), so slot offsets are immediates and nothing is copied between steps.
#pragma once

#include "kernels_prefill_pp.hip.h"

namespace wr {

// The row maximum of the scores in `c` joined across the two lanes of a row and,
// rarely, a move of the row's reference.
template <int HD>
__device__ __forceinline__ void il_settle(PrefillRows<HD>& R, PpCtx<HD>& cx, f32x16& negm, f32x16& c, float tmax)
{
    {
        const uint32_t u = __float_as_uint(tmax);
        const auto sw = __builtin_amdgcn_permlane32_swap(u, u, false, false);
        tmax = max3_raw(__uint_as_float(sw[0]), __uint_as_float(sw[1]), tmax);   // same in both lanes of a row
    }
    const bool jump = tmax > cx.thr;                      // thr: -inf until the row has a reference, then kLazyLog2
    if (__builtin_amdgcn_ballot_w64(jump) != 0) pp_move_reference<HD>(R, cx, negm, c, tmax, jump);
}

// Step j of a wave (P == j % kRing).  On entry `cur` holds the scores of the set's
// tile j (masked, reference settled), kf the K operands of tile j+1; on exit `nxt`
// holds the scores of tile j+1 in the same state and kf the operands of tile j+2.
template <int HD, int P>
__device__ __forceinline__ void il_step(PrefillRows<HD>& R, PpCtx<HD>& cx, f32x16& negm, const f32x16& cur,
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
    }
    R.l_run += psum;
    // requested order of the first half: each link of the chain, one operand read,
    // then its share of the exponentials, packs and sums (masks: 0x8 MFMA, 0x100
    // LDS read, 0x2 vector ALU)
#pragma unroll
    for (int i = 0; i < NS; i++) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x002, 4 * PAIRS, 0);
    }
#pragma unroll
    for (int i = 0; i < NS; i++) {
        const int t = i / ND, dt = i % ND;
        R.o[dt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(vf[i], __builtin_bit_cast(half8, pop[t]), R.o[dt], 0, 0,
                                                           0);
        kf[i] = *reinterpret_cast<const half8*>(cx.kop[i] + KS * L::KTILE);
        if (i < L::NL) pp_issue_k1<HD, KC>(cx, j + 4, i);
        else if (i < 2 * L::NL) pp_issue_v1<HD, VC>(cx, j + 2, i - L::NL);
    }
    // The row maximum runs in the products' shadow as if the tile were plain; a
    // tile with invisible (row, key) pairs is masked afterwards and its maximum
    // taken again (rare, wave-uniform).  Kept behind the products so that the
    // whole step up to here is one block the scheduler can interleave.
    float tmax = pp_max16(nxt);
    const uint32_t jt = j + 1;
    if (jt < cx.pl_lo || jt > cx.pl_hi) {
        pp_mask_special<HD>(R, cx, nxt, cx.t0 + 2 * jt, jt, g, tmax);
        tmax = pp_max16(nxt);
    }
    il_settle<HD>(R, cx, negm, nxt, tmax);
    // all copies but this step's have landed: K of tile j+3 and Vt of tile j+1,
    // which the next step reads once the barrier has published them
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * L::NL) : "memory");
    pp_patch_tail<HD, TS>(smem, cx, j + 1, sub, lane, kv_valid);
    // (no wait for this step's K operand reads here: their slot is not overwritten
    // before the step after next, long after the next chain has consumed them)
    __builtin_amdgcn_sched_barrier(0);
    asm volatile("s_barrier" ::: "memory");
    __builtin_amdgcn_sched_barrier(0);
}

template <int HD>
__device__ __forceinline__ void il_block(const PrefillArgs& a, unsigned char* smem, uint32_t pb,
                                         uint32_t kvh, uint32_t hc)
{
    using L = SplitLds<HD>;
    static_assert(L::NL == 1 || L::NL == 2, "one or two copies per wave, tile and operand");
#ifdef WR_PP_PROF
    __builtin_amdgcn_sched_barrier(0);
    const unsigned long long il_ta = clock64();
    __builtin_amdgcn_sched_barrier(0);
#endif
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);   // in a scalar register
    const int n = lane & 31, g = lane >> 5;
    const int kg = wave >> 2, sub = wave & 3;             // key set (tile parity), rows served
    const uint32_t G = a.group;
    const uint32_t Gw = G < 4 ? G : 4;
    const uint32_t BP = 32 * (4 / Gw);                    // positions per block
    const uint32_t head = kvh * G + hc * Gw + (sub % Gw);
    const uint32_t row0 = pb * BP + (sub / Gw) * 32;      // first chunk row of this wave
    const uint32_t kv_valid = a.p0 + a.T;                 // rows of the cache that hold data
    uint32_t t_first, t_last;
    prefill_block_tiles(a, pb, BP, t_first, t_last);

    PrefillRows<HD> R;
    prefill_rows_init<HD, false>(R, a, row0, head, n, g);

    PpCtx<HD> cx;
    cx.t0 = t_first + kg;                                 // this set's tiles: t0, t0 + 2, ...
    cx.nt = (cx.t0 <= t_last) ? (t_last - cx.t0) / 2 + 1 : 0;
    cx.t_last = t_last;
    cx.tail_tile = kv_valid / kTileKeys;
    cx.kbase = uniform_ptr(reinterpret_cast<const unsigned char*>(a.k + (size_t)kvh * a.ctx_pad * HD));
    cx.vtbase = uniform_ptr(reinterpret_cast<const unsigned char*>(
        a.vt + (size_t)kvh * (a.ctx_pad / kVBlock) * HD * kVBlock));
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

#ifdef WR_PP_PROF
    __builtin_amdgcn_sched_barrier(0);
    const unsigned long long il_tb = clock64();
    __builtin_amdgcn_sched_barrier(0);
#endif
    // everything the first two vector blocks read, in order of need
    pp_issue_k<HD, 0>(cx, 0);
    pp_issue_k<HD, 1>(cx, 1);
    pp_issue_v<HD, 0>(cx, 0);
    pp_issue_k<HD, 2>(cx, 2);
    pp_issue_v<HD, 1>(cx, 1);

    // Q: every row is 4*HD contiguous bytes in global memory, so it is read with
    // whole-row coalesced loads (the two waves serving a sub-block take 16 rows
    // each), converted to pre-scaled F16 and turned into the per-lane operand
    // layout through LDS.
    _Float16 (*qs)[32][HD + 8] = reinterpret_cast<_Float16 (*)[32][HD + 8]>(smem + L::Q_OFF);
    {
        constexpr int LPR = HD / 4;                       // lanes per row (one float4 each)
        constexpr int RPI = 64 / LPR;                     // rows per load instruction
#pragma unroll
        for (int j = 0; j < 16 / RPI; j++) {
            const int r = kg * 16 + j * RPI + lane / LPR;
            const uint32_t row = min(row0 + r, a.T - 1);  // idle rows re-read the last one
            const float4 x = *reinterpret_cast<const float4*>(
                a.q + ((size_t)row * a.nq + head) * HD + (lane % LPR) * 4);
            half4 h;
            h[0] = (_Float16)(x.x * a.qscale);
            h[1] = (_Float16)(x.y * a.qscale);
            h[2] = (_Float16)(x.z * a.qscale);
            h[3] = (_Float16)(x.w * a.qscale);
            *reinterpret_cast<half4*>(&qs[sub][r][(lane % LPR) * 4]) = h;
        }
    }
#ifdef WR_PP_PROF
    const unsigned long long il_t0 = clock64();
#endif
    f32x16 sa, sb, negm;
    u32x4 pop[2];
    half8 kf[HD / 16], vf[HD / 16];
#pragma unroll
    for (int r = 0; r < 16; r++) sa[r] = sb[r] = negm[r] = 0.f;
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    pp_patch_tail<HD, 0>(smem, cx, 0, sub, lane, kv_valid);
    pp_barrier();                                         // first tiles and Q visible to all
#pragma unroll
    for (int i = 0; i < HD / 16; i++)
        R.qop[i] = *reinterpret_cast<const half8*>(&qs[sub][n][i * 16 + g * 8]);
    // scores of the set's first tile
#pragma unroll
    for (int i = 0; i < HD / 16; i++) kf[i] = *reinterpret_cast<const half8*>(cx.kop[i]);
#pragma unroll
    for (int i = 0; i < HD / 16; i++)
        sa = __builtin_amdgcn_mfma_f32_32x32x16_f16(kf[i], R.qop[i], sa, 0, 0, 0);
    pp_barrier();                                         // slot 0 of K has been read by all: it is refilled
    pp_issue_k<HD, 0>(cx, 3);
#pragma unroll
    for (int i = 0; i < HD / 16; i++) kf[i] = *reinterpret_cast<const half8*>(cx.kop[i] + L::KTILE);
    {
        float tmax0 = pp_max16(sa);
        if (0 < cx.pl_lo || 0 > cx.pl_hi) {
            pp_mask_special<HD>(R, cx, sa, cx.t0, 0, g, tmax0);
            tmax0 = pp_max16(sa);
        }
        il_settle<HD>(R, cx, negm, sa, tmax0);
    }
    pp_barrier();                                         // slot 1 of K has been read by all: step 0 refills it

    // steps of the loop: the even set's tile count (the odd set has as many or one
    // fewer and spends its last step on probabilities of zero); the same in every
    // wave, and every step ends with the workgroup's barrier
#ifdef WR_PP_PROF
    const unsigned long long il_t1 = clock64();
#endif
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
#ifdef WR_PP_PROF
    const unsigned long long il_t2 = clock64();
#endif

    // merge the odd-tile partials into the even-tile waves; the ring must be
    // quiet first (the last steps' copies still target it)
    constexpr int NREG = HD / 2;
    float* mg = reinterpret_cast<float*>(smem) + (size_t)sub * (NREG + 2) * 64;
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (kg == 1) {
#pragma unroll
        for (int dt = 0; dt < HD / 32; dt++)
#pragma unroll
            for (int r = 0; r < 16; r++) mg[(dt * 16 + r) * 64 + lane] = R.o[dt][r];
        mg[NREG * 64 + lane] = R.m_run;
        mg[(NREG + 1) * 64 + lane] = R.l_run;
    }
    __syncthreads();
    // rows leave through LDS as well: the merged tile is written row-major into
    // the sub-block's own scratch, then both of its waves store whole rows
    float (*os)[HD + 4] = reinterpret_cast<float (*)[HD + 4]>(mg);
    static_assert((size_t)32 * (HD + 4) <= (size_t)(NREG + 2) * 64, "row-major tile fits the merge scratch");
    if (kg == 0) {
        const float m1 = mg[NREG * 64 + lane], l1 = mg[(NREG + 1) * 64 + lane];
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
                R.o[dt][r] = R.o[dt][r] * w0 + mg[(dt * 16 + r) * 64 + lane] * w1;
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
                *reinterpret_cast<float4*>(&os[n][dt * 32 + 8 * q4 + 4 * g]) = v;
            }
    }
    __syncthreads();
    {
        constexpr int LPR = HD / 4;                       // lanes per row (one float4 each)
        constexpr int RPI = 64 / LPR;                     // rows per store instruction
#pragma unroll
        for (int j = 0; j < 16 / RPI; j++) {
            const int r = kg * 16 + j * RPI + lane / LPR;
            const float4 v = *reinterpret_cast<const float4*>(&os[r][(lane % LPR) * 4]);
            if (row0 + r < a.T)
                *reinterpret_cast<float4*>(a.out + ((size_t)(row0 + r) * a.nq + head) * HD +
                                           (lane % LPR) * 4) = v;
        }
    }
#ifdef WR_PP_PROF
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    if (blockIdx.x == 0 && blockIdx.y == 0 && lane == 0 && sub == 0) {
        const unsigned long long il_t3 = clock64();
        wr_pp_prof[kg][0] += il_t1 - il_t0;      // prologue (from the first copies to the loop)
        wr_pp_prof[kg][4] += il_tb - il_ta;      // setup
        wr_pp_prof[kg][5] += il_t0 - il_tb;      // first copies issued, Q loaded and staged
        wr_pp_prof[kg][1] += il_t2 - il_t1;      // loop
        wr_pp_prof[kg][2] += il_t3 - il_t2;      // merge and store
        wr_pp_prof[kg][6] += nsteps;
    }
#endif
}

// grid and block pairing as prefill_pp_kernel
template <int HD>
__global__ __launch_bounds__(kSplitThreads, 1) void prefill_il_kernel(const PrefillArgs a)
{
    extern __shared__ __attribute__((aligned(16))) unsigned char prefill_smem_raw[];
#ifdef WR_PP_PROF
    const unsigned long long k_t0 = clock64();
#endif
    const uint32_t G = a.group;
    const uint32_t Gw = G < 4 ? G : 4;
    const uint32_t chunks = G / Gw;
    const uint32_t kvh = blockIdx.x / chunks, hc = blockIdx.x % chunks;
    const uint32_t BP = 32 * (4 / Gw);
    const uint32_t nblk = (a.T + BP - 1) / BP;
    const uint32_t lo = blockIdx.y, hi = nblk - 1 - blockIdx.y;
    const int passes = a.single ? 1 : 2;
#pragma unroll 1
    for (int pass = 0; pass < passes; pass++) {
        if (pass) {
            if (hi == lo) break;
            __syncthreads();                              // LDS changes hands
        }
        il_block<HD>(a, prefill_smem_raw, pass ? lo : hi, kvh, hc);
    }
#ifdef WR_PP_PROF
    if (threadIdx.x == 0) {
        const unsigned long long k_t1 = clock64();
        atomicMax(&wr_pp_prof[1][3], k_t1 - k_t0);               // longest workgroup
        atomicMin(&wr_pp_prof[1][4], k_t0);                       // first entry (array cleared to ~0 by the reader)
        atomicMax(&wr_pp_prof[1][5], k_t1);                       // last exit
        if (blockIdx.x == 0 && blockIdx.y == 0) wr_pp_prof[0][3] = k_t1 - k_t0;
    }
#endif
}

}  // namespace wr
