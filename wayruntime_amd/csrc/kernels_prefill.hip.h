// Causal prefill attention over rows already appended to the cache.
//
// Semantics (reference: the prefill loop src/core/session.c:615-625 running a
// seq_q = 1 attention per token): row i of the chunk sits at absolute position
// p0 + i and attends keys 0 .. p0 + i; with a sliding window, the last
// `window` of those.
#pragma once

#include "common.hip.h"
#include "kernels_decode.hip.h"

namespace wr {

struct PrefillArgs {
    const uint16_t* k;
    const uint16_t* vt;
    const float* q;          // [T][nq][hd]
    float* out;              // [T][nq][hd]
    uint32_t p0, T, nq, nkv, group, hd, ctx_pad, window;
    float qscale;            // softmax scale * log2(e)
    uint32_t single;         // MFMA kernels: one position block per workgroup (grid = blocks) instead of a pair
    uint32_t* err;           // error word (host memory the device can write); see set_barrier
    uint32_t err_code;       // what to store there: kDevErrWaitExpired | layer
};

// Layout of the error word a kernel leaves for the host when it gives up a
// bounded wait: bit 31 set, the layer in the low bits.
constexpr uint32_t kDevErrWaitExpired = 0x80000000u;
constexpr uint32_t kDevErrLayerMask = 0x0000FFFFu;

// Any head_dim / group: one workgroup per (row, head), vector ALU only.
__global__ __launch_bounds__(kDecodeThreads) void prefill_generic_kernel(const PrefillArgs a)
{
    const uint32_t row = blockIdx.x, head = blockIdx.y;
    const uint32_t hd = a.hd;
    const uint32_t seq_k = a.p0 + row + 1;
    const uint32_t key_lo = (a.window > 0 && seq_k > a.window) ? seq_k - a.window : 0;

    __shared__ GenericShared sh;
    generic_attend_wg(sh, a.k, a.vt, a.ctx_pad, head / a.group, hd, key_lo, seq_k,
                      a.q + ((size_t)row * a.nq + head) * hd, a.qscale);
    const GenericMerge g = merge_generic(sh);
    for (uint32_t d = threadIdx.x; d < hd; d += kDecodeThreads) {
        float acc = 0.f;
#pragma unroll
        for (int w = 0; w < kDecodeWaves; w++) acc += sh.o[w][d] * g.fct[w];
        a.out[((size_t)row * a.nq + head) * hd + d] = (g.L > 0.f) ? acc / g.L : 0.f;
    }
}


// ------------------------------------------------------------------ MFMA --
// Causal flash attention on the matrix cores (v_mfma_f32_32x32x16_f16, F32
// accumulate).  MFMA-bound: 4 * nq * hd flops per (query row, visible key).
//
// Workgroup = 4 waves = one KV head x a block of positions x up to 4 heads of
// its GQA group: wave w serves head (w % Gw) at the 32 positions of sub-block
// (w / Gw), Gw = min(group, 4).  All waves share each 32-key K / Vt tile, staged
// once per workgroup through LDS (double buffered, one barrier per tile), so a
// tile fetched from L2 feeds 128 query rows.  Position blocks are issued
// heaviest first (the causal triangle makes late blocks the longest).
//
// Per wave and tile, with the query row as the MFMA COLUMN (lane % 32):
//   S^T[key][row]  = K[key][:] . Q^T[:][row]          HD/16 MFMAs
//   online softmax on the 16 scores a lane holds (+ one exchange with lane^32)
//   O^T[dim][row] += Vt[dim][key] . P^T[key][row]     HD/16 MFMAs
// K rows enter the first MFMA in a permuted order chosen so that the scores a
// lane ends up with are 8 consecutive keys per contraction step: P^T is then
// already laid out as the second MFMA's operand, and the matching Vt operand is
// one 16-byte read of the block-transposed V.  Q is rounded to F16 once (it is
// the only operand that is not F16 already); P is rounded to F16 per tile.

constexpr int kPrefillThreads = 256;
constexpr float kLazyLog2 = 8.0f;    // softmax reference point moves only on jumps above 2^8

__device__ __forceinline__ int prefill_key_perm(int m)
{
    const int a = m >> 3, g = (m >> 2) & 1, b = m & 3;
    return 16 * (a >> 1) + 8 * g + 4 * (a & 1) + b;
}

template <int HD>
struct PrefillSmem {
    // 16-byte row pads make the 128-bit LDS reads of the MFMA operands conflict free
    _Float16 k[2][kTileKeys][HD + 8];
    _Float16 v[2][HD][kVBlock + 8];
};

// One 16-byte chunk per thread and slot: a tile is HD/64 chunks of K and of Vt per thread.
template <int HD>
struct PrefillStage {
    u32x4 k[HD / 64], v[HD / 64];
};

template <int HD>
__device__ __forceinline__ void prefill_fetch(PrefillStage<HD>& st, const uint16_t* kbase,
                                              const uint16_t* vtbase, uint32_t tile, int tid)
{
    const u32x4* ksrc = reinterpret_cast<const u32x4*>(kbase + (size_t)tile * kTileKeys * HD);
    const u32x4* vsrc = reinterpret_cast<const u32x4*>(vtbase + (size_t)tile * HD * kVBlock);
#pragma unroll
    for (int c = 0; c < HD / 64; c++) {
        st.k[c] = ksrc[tid + c * kPrefillThreads];
        st.v[c] = vsrc[tid + c * kPrefillThreads];
    }
}

template <int HD>
__device__ __forceinline__ void prefill_stash(PrefillSmem<HD>& sm, int buf,
                                              const PrefillStage<HD>& st, uint32_t tile,
                                              uint32_t kv_valid, int tid)
{
    constexpr int KCH = HD / 8;                           // 16-byte chunks per K row
    const bool tail = (tile + 1) * kTileKeys > kv_valid;  // tile reaches past the appended rows
#pragma unroll
    for (int c = 0; c < HD / 64; c++) {
        const int ch = tid + c * kPrefillThreads;
        // unit ch of the cache's K tile is (half, chunk, slot); LDS keeps rows by position
        const int krow = (int)k_tile_pos(ch / (KCH * 16), ch % 16);
        *reinterpret_cast<u32x4*>(&sm.k[buf][krow][((ch / 16) % KCH) * 8]) = st.k[c];
        u32x4 v = st.v[c];
        if (tail) {
            // rows that were never appended may hold anything: zero them so
            // 0 * garbage cannot reach the accumulator
            const uint32_t key0 = tile * kTileKeys + (ch & 3) * 8;
            uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
            for (int e = 0; e < 4; e++) {
                if (key0 + 2 * e >= kv_valid) w[e] &= 0xFFFF0000u;
                if (key0 + 2 * e + 1 >= kv_valid) w[e] &= 0x0000FFFFu;
            }
            v = u32x4{w[0], w[1], w[2], w[3]};
        }
        *reinterpret_cast<u32x4*>(&sm.v[buf][ch >> 2][(ch & 3) * 8]) = v;
    }
}

// Per-wave state of one block of 32 query rows.
template <int HD>
struct PrefillRows {
    half8 qop[HD / 16];      // Q^T operand: column = this lane's row
    f32x16 o[HD / 32];       // O^T accumulators: dim = dt*32 + 8*(r/4) + 4g + r%4
    float m_run, l_run;
    uint32_t pos, row_lo;            // this lane's absolute position and window floor
    uint32_t w_first_pos, w_hi_lo;   // wave-wide: first row's position, last row's window floor
    uint32_t wt_first, wt_last;      // tiles this wave takes part in
    bool wave_ok;
};

// ktile: the tile's 32 K rows, vtile: its Vt block, both with padded rows.
// DUAL splits the score contraction over two accumulator chains (for kernels
// that run one wave per SIMD and cannot hide the matrix pipe's latency behind
// another wave).
template <int HD, bool DUAL>
__device__ __forceinline__ void prefill_compute(PrefillRows<HD>& R,
                                                const _Float16 (*ktile)[HD + 8],
                                                const _Float16 (*vtile)[kVBlock + 8],
                                                uint32_t tile, int n, int g, int krow)
{
    if (!R.wave_ok || tile < R.wt_first || tile > R.wt_last) return;
    const uint32_t kb = tile * kTileKeys;
    f32x16 c;
#pragma unroll
    for (int r = 0; r < 16; r++) c[r] = 0.f;
    // all K fragments of the tile are requested before the first MFMA, so the
    // LDS latency is paid once, not once per contraction step
    half8 kf[HD / 16];
#pragma unroll
    for (int s = 0; s < HD / 16; s++)
        kf[s] = *reinterpret_cast<const half8*>(&ktile[krow][s * 16 + g * 8]);
    if constexpr (DUAL) {
        // two independent accumulator chains keep the matrix pipe from waiting
        // on its own previous result
        f32x16 c_odd;
#pragma unroll
        for (int r = 0; r < 16; r++) c_odd[r] = 0.f;
#pragma unroll
        for (int s = 0; s < HD / 16; s += 2) {
            c = __builtin_amdgcn_mfma_f32_32x32x16_f16(kf[s], R.qop[s], c, 0, 0, 0);
            c_odd = __builtin_amdgcn_mfma_f32_32x32x16_f16(kf[s + 1], R.qop[s + 1], c_odd, 0, 0, 0);
        }
#pragma unroll
        for (int r = 0; r < 16; r++) c[r] += c_odd[r];
    } else {
#pragma unroll
        for (int s = 0; s < HD / 16; s++)
            c = __builtin_amdgcn_mfma_f32_32x32x16_f16(kf[s], R.qop[s], c, 0, 0, 0);
    }
    // register r of this lane: key kb + 16*(r/8) + 8*g + r%8, row n.
    // Some (row, key) pair of the tile is invisible: above the diagonal of the
    // wave's first row, or below the window of its last row.
    const bool edge = (kb + kTileKeys - 1 > R.w_first_pos) || (kb < R.w_hi_lo);
    if (edge) {
#pragma unroll
        for (int r = 0; r < 16; r++) {
            const uint32_t key = kb + 16 * (r >> 3) + 8 * g + (r & 7);
            if (key > R.pos || key < R.row_lo) c[r] = -INFINITY;
        }
    }
    float tmax = c[0];
#pragma unroll
    for (int r = 1; r < 16; r++) tmax = fmaxf(tmax, c[r]);
    tmax = wave_pair32_max(tmax);
    // Lazy reference point: m_run only moves when a row's maximum exceeds it by
    // more than kLazyLog2 (log2 units).  Until then later tiles' probabilities
    // are taken relative to the stale reference (at most 2^kLazyLog2, far inside
    // F16 range) and the accumulators need no rescale; O / l is unchanged, only
    // the common factor differs.  With 32 independent rows per wave an eager
    // maximum moves in most tiles, so this takes the 64-register rescale out of
    // the steady state.
    const bool jump = tmax > R.m_run + kLazyLog2;          // false for tmax = -inf
    const float m_new = jump ? tmax : R.m_run;
    const float m_safe = (m_new == -INFINITY) ? 0.f : m_new;   // row with nothing visible yet

    half8 pop[2];
    float psum = 0.f;
#pragma unroll
    for (int r = 0; r < 16; r++) {
        const float p = fast_exp2(c[r] - m_safe);
        psum += p;
        pop[r >> 3][r & 7] = (_Float16)p;
    }
    if (__builtin_amdgcn_ballot_w64(jump) != 0) {
        const float alpha = jump ? fast_exp2(R.m_run - m_safe) : 1.0f;
        R.l_run *= alpha;
#pragma unroll
        for (int dt = 0; dt < HD / 32; dt++)
#pragma unroll
            for (int r = 0; r < 16; r++) R.o[dt][r] *= alpha;
    }
    R.m_run = m_new;
    R.l_run += psum;
    // contraction step outermost: consecutive MFMAs hit different accumulators
#pragma unroll
    for (int t = 0; t < 2; t++) {
#pragma unroll
        for (int dt = 0; dt < HD / 32; dt++) {
            const half8 vf =
                *reinterpret_cast<const half8*>(&vtile[dt * 32 + n][16 * t + 8 * g]);
            R.o[dt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(vf, pop[t], R.o[dt], 0, 0, 0);
        }
    }
}

// Sets up a wave's 32 rows starting at chunk row `row0` for `head`: positions,
// window floors, tile range, empty accumulators and (LOADQ) the Q^T operand,
// read straight from global memory, each lane its own row.
template <int HD, bool LOADQ = true>
__device__ __forceinline__ void prefill_rows_init(PrefillRows<HD>& R, const PrefillArgs& a,
                                                  uint32_t row0, uint32_t head, int n, int g)
{
    const uint32_t T = a.T, p0 = a.p0;
    const uint32_t my_row = row0 + n;
    const bool row_ok = my_row < T;
    R.pos = p0 + (row_ok ? my_row : T - 1);               // clamped for idle rows
    R.row_lo = (a.window > 0 && R.pos + 1 > a.window) ? R.pos + 1 - a.window : 0;
    // this wave's own tile range (a wave with no valid row computes nothing)
    R.wave_ok = row0 < T;
    const uint32_t w_last_pos = p0 + min(T - 1, row0 + 31);
    R.w_first_pos = p0 + row0;
    const uint32_t w_lo =
        (a.window > 0 && R.w_first_pos + 1 > a.window) ? R.w_first_pos + 1 - a.window : 0;
    R.w_hi_lo = (a.window > 0 && w_last_pos + 1 > a.window) ? w_last_pos + 1 - a.window : 0;
    R.wt_first = w_lo / kTileKeys;
    R.wt_last = w_last_pos / kTileKeys;

    // Q^T operand: contraction slots (g, j) = dims s*16 + g*8 + j, pre-scaled
    const float* qrow = a.q + ((size_t)(row_ok ? my_row : T - 1) * a.nq + head) * HD;
    if constexpr (LOADQ) {
#pragma unroll
        for (int s = 0; s < HD / 16; s++) {
            const float4 x0 = *reinterpret_cast<const float4*>(qrow + s * 16 + g * 8);
            const float4 x1 = *reinterpret_cast<const float4*>(qrow + s * 16 + g * 8 + 4);
            R.qop[s][0] = (_Float16)(x0.x * a.qscale);
            R.qop[s][1] = (_Float16)(x0.y * a.qscale);
            R.qop[s][2] = (_Float16)(x0.z * a.qscale);
            R.qop[s][3] = (_Float16)(x0.w * a.qscale);
            R.qop[s][4] = (_Float16)(x1.x * a.qscale);
            R.qop[s][5] = (_Float16)(x1.y * a.qscale);
            R.qop[s][6] = (_Float16)(x1.z * a.qscale);
            R.qop[s][7] = (_Float16)(x1.w * a.qscale);
        }
    }
#pragma unroll
    for (int dt = 0; dt < HD / 32; dt++)
#pragma unroll
        for (int r = 0; r < 16; r++) R.o[dt][r] = 0.f;
    R.m_run = -INFINITY;
    R.l_run = 0.f;
}

// Normalises and writes a wave's rows.
template <int HD>
__device__ __forceinline__ void prefill_rows_store(const PrefillRows<HD>& R, const PrefillArgs& a,
                                                   uint32_t row0, uint32_t head, int n, int g)
{
    const float l_tot = wave_pair32_sum(R.l_run);
    const float inv = (l_tot > 0.f) ? 1.0f / l_tot : 0.f;
    const uint32_t my_row = row0 + n;
    if (my_row < a.T) {
        float* orow = a.out + ((size_t)my_row * a.nq + head) * HD;
#pragma unroll
        for (int dt = 0; dt < HD / 32; dt++) {
#pragma unroll
            for (int q4 = 0; q4 < 4; q4++) {
                float4 v;
                v.x = R.o[dt][4 * q4 + 0] * inv;
                v.y = R.o[dt][4 * q4 + 1] * inv;
                v.z = R.o[dt][4 * q4 + 2] * inv;
                v.w = R.o[dt][4 * q4 + 3] * inv;
                *reinterpret_cast<float4*>(orow + dt * 32 + 8 * q4 + 4 * g) = v;
            }
        }
    }
}

// Tile range a block of positions [pb*BP, (pb+1)*BP) streams.
__device__ __forceinline__ void prefill_block_tiles(const PrefillArgs& a, uint32_t pb, uint32_t BP,
                                                    uint32_t& t_first, uint32_t& t_last)
{
    const uint32_t wg_last_row = min(a.T, (pb + 1) * BP) - 1;
    const uint32_t wg_first_pos = a.p0 + pb * BP;
    const uint32_t wg_lo =
        (a.window > 0 && wg_first_pos + 1 > a.window) ? wg_first_pos + 1 - a.window : 0;
    t_first = wg_lo / kTileKeys;
    t_last = (a.p0 + wg_last_row) / kTileKeys;            // inclusive
}

// One position block of one workgroup: loads Q, streams the visible K / Vt
// tiles (two tiles of global loads in flight ahead of the one being computed),
// writes the rows.
template <int HD>
__device__ __forceinline__ void prefill_block(const PrefillArgs& a, PrefillSmem<HD>& sm,
                                              uint32_t pb, uint32_t kvh, uint32_t hc)
{
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int n = lane & 31, g = lane >> 5;
    const uint32_t G = a.group;
    const uint32_t Gw = G < 4 ? G : 4;
    const uint32_t BP = 32 * (4 / Gw);                    // positions per block
    const uint32_t head = kvh * G + hc * Gw + (wave % Gw);
    const uint32_t row0 = pb * BP + (wave / Gw) * 32;     // first chunk row of this wave
    const uint32_t kv_valid = a.p0 + a.T;                 // rows of the cache that hold data
    uint32_t t_first, t_last;
    prefill_block_tiles(a, pb, BP, t_first, t_last);

    const uint16_t* kbase = a.k + (size_t)kvh * a.ctx_pad * HD;
    const uint16_t* vtbase = a.vt + (size_t)kvh * (a.ctx_pad / kVBlock) * HD * kVBlock;
    PrefillStage<HD> s0, s1;
    uint32_t tile = t_first;
    prefill_fetch<HD>(s0, kbase, vtbase, tile, tid);
    if (tile + 1 <= t_last) prefill_fetch<HD>(s1, kbase, vtbase, tile + 1, tid);

    PrefillRows<HD> R;
    prefill_rows_init<HD>(R, a, row0, head, n, g);
    const int krow = prefill_key_perm(n);                 // LDS row this lane feeds to MFMA row n

    for (;;) {
        prefill_stash<HD>(sm, 0, s0, tile, kv_valid, tid);
        lds_barrier();
        if (tile + 2 <= t_last) prefill_fetch<HD>(s0, kbase, vtbase, tile + 2, tid);
        prefill_compute<HD, true>(R, sm.k[0], sm.v[0], tile, n, g, krow);
        if (++tile > t_last) break;
        prefill_stash<HD>(sm, 1, s1, tile, kv_valid, tid);
        lds_barrier();
        if (tile + 2 <= t_last) prefill_fetch<HD>(s1, kbase, vtbase, tile + 2, tid);
        prefill_compute<HD, true>(R, sm.k[1], sm.v[1], tile, n, g, krow);
        if (++tile > t_last) break;
    }
    prefill_rows_store<HD>(R, a, row0, head, n, g);
}

// grid = (ceil(blocks / 2), KV heads x head chunks).  Workgroup x takes position
// block (blocks-1-x) and then block x: a long block and a short one, so every
// workgroup streams the same number of tiles despite the causal triangle.
// a.single: grid.x = blocks and workgroup x takes block (blocks-1-x) only (the
// long blocks start first); for launches whose pairs would leave CUs idle.
template <int HD>
__global__ __launch_bounds__(kPrefillThreads, 1) void prefill_mfma_kernel(const PrefillArgs a)
{
    __shared__ __attribute__((aligned(16))) PrefillSmem<HD> sm;
    const uint32_t G = a.group;
    const uint32_t Gw = G < 4 ? G : 4;
    const uint32_t chunks = G / Gw;                       // head chunks per KV head (1, or 2 for G = 8)
    const uint32_t kvh = blockIdx.y / chunks, hc = blockIdx.y % chunks;
    const uint32_t BP = 32 * (4 / Gw);
    const uint32_t nblk = (a.T + BP - 1) / BP;
    const uint32_t lo = blockIdx.x, hi = nblk - 1 - blockIdx.x;
    prefill_block<HD>(a, sm, hi, kvh, hc);
    if (!a.single && hi != lo) {
        __syncthreads();                                  // LDS buffers change hands
        prefill_block<HD>(a, sm, lo, kvh, hc);
    }
}


// ------------------------------------------------- MFMA, two waves per SIMD --
// Same arithmetic per wave and tile as above, restructured so that the matrix
// pipe, the vector ALU, LDS and the global-load path work at the same time:
//
//  * The keys of a block are split over two wave sets: waves 0-3 take the even
//    tiles of the block's range, waves 4-7 the odd ones; the two partial
//    (m, l, O) triples are merged through LDS at the end.  Eight waves put two
//    on every SIMD.
//  * Each wave is software-pipelined across its tiles: while the exponentials
//    of tile j run on the vector ALU, the score MFMAs of tile j+1 (a dependent
//    chain) and the first half of tile j's P.V MFMAs run on the matrix pipe.
//    To have tile j+1's K next to tile j's Vt, K is staged one step ahead of V.
//  * The two wave sets run independently of each other until the merge: each
//    stages its own tiles in its own ring of three tile buffers and synchronises
//    its four waves with a counter in LDS instead of the workgroup barrier.
//    The two waves that share a SIMD belong to different sets, so they drift
//    apart and one's barrier wait or LDS latency is covered by the other's
//    arithmetic; a workgroup-wide barrier per step would keep them in lock-step,
//    both waiting at the same time.
//  * Tiles travel from global memory straight into LDS
//    (global_load_lds_dwordx4: no staging registers, no LDS store instructions),
//    issued from inside the step's arithmetic three steps (K) / two steps (Vt)
//    before their first use.
//  * Such a load writes the wave's 64 x 16 bytes to consecutive LDS addresses, so
//    rows cannot be padded; the 16-byte chunks of a row are permuted instead
//    (chunk c of row r sits at slot c ^ f(r)), on the global side where any
//    permutation inside a row keeps the access coalesced.  f is chosen so that
//    the sixteen rows a 128-bit LDS read touches per cycle fall into sixteen
//    different slots of the 256-byte bank row.
//  * Loads are issued unconditionally (tile indices clamped to the set's last
//    tile; duplicates land in ring slots nobody reads) so the number in flight
//    is the same at every barrier and "all but the newest N" is a fixed wait.
//  * Instruction order inside a step is requested from the scheduler with
//    scheduling-group barriers: one MFMA, then the few vector / LDS
//    instructions its execution time covers.
//
// Head dims up to 128 only: beyond that a wave needs more than the 256 registers
// two waves per SIMD leave it.

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
    static constexpr int CNT_OFF = Q_OFF + Q_BYTES;       // the two sets' arrival counters
    static constexpr int MERGE_BYTES = 4 * (HD / 2 + 2) * 64 * 4;   // laid over the rings
    static constexpr int TOTAL = CNT_OFF + 16;
    static_assert(MERGE_BYTES <= Q_OFF, "merge scratch fits the rings");
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

// What one wave set streams (tiles t0, t0+2, ... : nt of them), from where, and
// this lane's invariant addresses.
template <int HD>
struct SplitCtx {
    const unsigned char* kbase;       // this KV head's K / Vt, bytes
    const unsigned char* vtbase;
    uint32_t lds0;                    // LDS byte address of the kernel's dynamic LDS
    uint32_t ring;                    // byte offset of this set's ring in it
    uint32_t cnt;                     // byte offset of this set's arrival counter
    uint32_t t0, nt, t_last, kv_valid;   // nt may be 0 (the odd set of a one-tile block)
    // Lane-invariant addresses, one register each; the others follow from them:
    // a wave's second load of a tile is the first one kKStep / 4 KiB further (same
    // slot permutation), and the operand read of contraction step s / half t is the
    // first one with address bits 5-7 / bit 5 flipped (the permutation is an
    // XOR of the chunk index, the step is the chunk index's upper bits).
    uint32_t gk_off;                  // lane's byte offset inside a K tile, first load
    uint32_t gv_off;                  // ... inside a Vt block
    uint32_t kread;                   // LDS offset of the K operand read of step 0 (ring slot 0)
    uint32_t vread;                   // ... of the Vt operand read of t = 0, dt = 0
};

// Loads of the set's j-th K tile into ring slot `slot`.  KiB q = sub + 4u of the
// LDS image (tile rows by position, 1024 / RB rows per KiB) is gathered from the
// cache's K tile, 16 bytes per lane: rows 16 apart share half and chunk and sit
// eight slots = 128 bytes apart there.
template <int HD>
__device__ __forceinline__ void split_issue_k(const SplitCtx<HD>& cx, uint32_t j, int slot, int sub)
{
    using L = SplitLds<HD>;
    const uint32_t tile = min(cx.t0 + 2 * j, cx.t_last);  // past the range: a duplicate nobody reads
    const unsigned char* src = cx.kbase + (size_t)tile * L::KTILE;
#pragma unroll
    for (int u = 0; u < L::NL; u++)
        lds_direct_load(cx.lds0 + cx.ring + slot * L::KTILE + (sub + 4 * u) * 1024, src + u * 128,
                        cx.gk_off);
}

template <int HD>
__device__ __forceinline__ void split_issue_v(const SplitCtx<HD>& cx, uint32_t j, int slot, int sub)
{
    using L = SplitLds<HD>;
    const uint32_t tile = min(cx.t0 + 2 * j, cx.t_last);
    const unsigned char* src = cx.vtbase + (size_t)tile * L::VTILE;
#pragma unroll
    for (int u = 0; u < L::NL; u++)
        lds_direct_load(cx.lds0 + cx.ring + L::V_IN_SET + slot * L::VTILE + (sub + 4 * u) * 1024,
                        src + u * 4096, cx.gv_off);
}

// Rows that were never appended may hold anything: zero them in the staged Vt
// of the set's j-th tile so 0 * garbage cannot reach the accumulator.  Only the
// tile holding the end of the appended rows is affected.  Every lane patches
// the chunks its own loads delivered, so the caller only has to have waited for
// this wave's loads.
template <int HD>
__device__ __forceinline__ void split_patch_tail(unsigned char* smem, const SplitCtx<HD>& cx,
                                                 uint32_t j, int sub, int lane)
{
    using L = SplitLds<HD>;
    const uint32_t tile = min(cx.t0 + 2 * j, cx.t_last);  // as loaded (an idle set holds a duplicate)
    if ((tile + 1) * kTileKeys <= cx.kv_valid) return;
    const int slot = j % kRing;
#pragma unroll
    for (int u = 0; u < L::NL; u++) {
        const int q = sub + 4 * u;
        const int row = q * 16 + lane / 4;                // Vt row (dimension)
        const int c = (lane & 3) ^ L::fv(row);            // key chunk this slot holds
        const uint32_t key0 = tile * kTileKeys + c * 8;
        u32x4* at = reinterpret_cast<u32x4*>(smem + cx.ring + L::V_IN_SET + slot * L::VTILE +
                                             q * 1024 + lane * 16);
        u32x4 v = *at;
        uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
        for (int e = 0; e < 4; e++) {
            if (key0 + 2 * e >= cx.kv_valid) w[e] &= 0xFFFF0000u;
            if (key0 + 2 * e + 1 >= cx.kv_valid) w[e] &= 0x0000FFFFu;
        }
        *at = u32x4{w[0], w[1], w[2], w[3]};
    }
}

// The data movement of step j: K of the set's tile j+3 and Vt of tile j+2
// replace K of tile j and Vt of tile j-1, both read for the last time in step j-1.
template <int HD>
__device__ __forceinline__ void split_move(const SplitCtx<HD>& cx, uint32_t j, int sub)
{
    split_issue_k<HD>(cx, j + 3, j % kRing, sub);
    split_issue_v<HD>(cx, j + 2, (j + 2) % kRing, sub);
}

// Barrier among the four waves of one set: every wave adds one to the set's
// counter in LDS and waits until it has reached `target` (4 x the number of
// barriers so far; the counter is never reset inside a block).  The wait is
// bounded: should a wave never arrive, the others go on instead of hanging the
// device, with wrong data, and say so: lane 0 stores `err_code` in the error
// word, which the host finds at its next wait for the stream and turns into an
// error status for the caller.
__device__ __forceinline__ void set_barrier(unsigned char* smem, uint32_t cnt_off, uint32_t target,
                                            int lane, uint32_t* err, uint32_t err_code)
{
    uint32_t* cnt = reinterpret_cast<uint32_t*>(smem + cnt_off);
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    if (lane == 0) __hip_atomic_fetch_add(cnt, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    bool arrived = false;
    for (uint32_t spins = 0; spins < (1u << 22); spins++) {
        const uint32_t seen = (uint32_t)__builtin_amdgcn_readfirstlane(
            __hip_atomic_load(cnt, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP));
        if ((int32_t)(seen - target) >= 0) {
            arrived = true;
            break;
        }
        __builtin_amdgcn_s_sleep(1);
    }
    if (!arrived && lane == 0) *err = err_code;
    asm volatile("" ::: "memory");
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

// First part of a tile's softmax: masks, row maximum, reference point.
//
// The scores arrive with the row's reference point already subtracted: the
// score chain starts from the accumulator block `negm` (-m_run in all sixteen
// registers; 0 while the row has no reference yet), so in the steady state the
// probabilities are exp2 of the scores as they are, with no subtraction.  The
// reference moves only when a row's maximum exceeds it by more than kLazyLog2
// (or is the row's first finite score): then the scores of this tile are
// shifted, the accumulators rescaled and `negm` rewritten.  With 32 independent
// rows per wave an eager maximum would move in most tiles.
template <int HD>
__device__ __forceinline__ void split_softmax_begin(PrefillRows<HD>& R, f32x16& negm, f32x16& c,
                                                    uint32_t tile, int g)
{
    const uint32_t kb = tile * kTileKeys;
    // register r of this lane: key kb + 16*(r/8) + 8*g + r%8, row n.
    // Some (row, key) pair of the tile is invisible: above the diagonal of the
    // wave's first row, or below the window of its last row.
    const bool edge = (kb + kTileKeys - 1 > R.w_first_pos) || (kb < R.w_hi_lo);
    if (edge) {
#pragma unroll
        for (int r = 0; r < 16; r++) {
            const uint32_t key = kb + 16 * (r >> 3) + 8 * g + (r & 7);
            if (key > R.pos || key < R.row_lo) c[r] = -INFINITY;
        }
    }
    float tmax = max3_raw(c[0], c[1], c[2]);
#pragma unroll
    for (int r = 3; r < 15; r += 2) tmax = max3_raw(tmax, c[r], c[r + 1]);
    tmax = max3_raw(tmax, c[15], c[15]);
    {
        const uint32_t u = __float_as_uint(tmax);
        const auto sw = __builtin_amdgcn_permlane32_swap(u, u, false, false);
        tmax = max3_raw(__uint_as_float(sw[0]), __uint_as_float(sw[1]), tmax);   // same in both lanes of a row
    }
    const bool unset = (R.m_run == -INFINITY);
    const bool jump = unset ? (tmax > -INFINITY) : (tmax > kLazyLog2);
    if (__builtin_amdgcn_ballot_w64(jump) != 0) {
        const float delta = jump ? tmax : 0.f;
        const float alpha = jump ? (unset ? 0.f : fast_exp2(-delta)) : 1.0f;
        R.l_run *= alpha;
#pragma unroll
        for (int dt = 0; dt < HD / 32; dt++)
#pragma unroll
            for (int r = 0; r < 16; r++) R.o[dt][r] *= alpha;
        // The two blocks are updated in place, with the instructions spelled
        // out: left to itself the compiler gives the updated values new
        // registers and pays for it with 32 copies on the path that skips this
        // branch, which is the one that matters.
#pragma unroll
        for (int r = 0; r < 16; r++)
            asm volatile("v_sub_f32 %0, %0, %1" : "+v"(c[r]) : "v"(delta));
        if (jump) R.m_run = (unset ? 0.f : R.m_run) + delta;
        const float nm = (R.m_run == -INFINITY) ? 0.f : -R.m_run;
#pragma unroll
        for (int r = 0; r < 16; r++)
            asm volatile("v_mov_b32 %0, %1" : "+v"(negm[r]) : "v"(nm));
    }
}

// Scores of one tile only (a wave's first tile).  kslot: byte offset of the ring
// slot holding the tile's K.
template <int HD>
__device__ __forceinline__ void split_scores(const PrefillRows<HD>& R, const f32x16& negm,
                                             f32x16& sn, const unsigned char* smem,
                                             const SplitCtx<HD>& cx, uint32_t kslot)
{
    half8 kf[HD / 16];
#pragma unroll
    for (int s = 0; s < HD / 16; s++)
        kf[s] = *reinterpret_cast<const half8*>(smem + ((kslot + cx.kread) ^ (s * 32)));
    sn = __builtin_amdgcn_mfma_f32_32x32x16_f16(kf[0], R.qop[0], negm, 0, 0, 0);
#pragma unroll
    for (int s = 1; s < HD / 16; s++)
        sn = __builtin_amdgcn_mfma_f32_32x32x16_f16(kf[s], R.qop[s], sn, 0, 0, 0);
}

// Instruction order of the steady-state step, as a request to the scheduler
// (the counts must be literals, hence the recursion).  Every score MFMA, joined
// in the second half by one P.V MFMA, is followed by VPS vector instructions;
// LDS reads go behind the MFMA that frees their registers.
// Masks: 0x8 MFMA, 0x2 vector ALU, 0x100 LDS read.
template <int S, int NS, int VPS>
__device__ __forceinline__ void split_step_order()
{
    if constexpr (S < NS) {
        if constexpr (S >= NS / 2)
            __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);
        else
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        if constexpr (S == 0 || S == NS / 2) __builtin_amdgcn_sched_group_barrier(0x100, NS / 2, 0);
        __builtin_amdgcn_sched_group_barrier(0x002, VPS, 0);
        split_step_order<S + 1, NS, VPS>();
    }
}

// Steady state: softmax and P.V of the tile whose scores are in `c`, interleaved
// with the score MFMAs of the wave's next tile (result in `sn`) and with the
// step's data movement.
template <int HD>
__device__ __forceinline__ void split_step(PrefillRows<HD>& R, f32x16& negm, f32x16& c, f32x16& sn,
                                           const unsigned char* smem, const SplitCtx<HD>& cx,
                                           uint32_t i, int wave, uint32_t kslot, uint32_t vslot,
                                           uint32_t tile, int g)
{
    constexpr int NS = HD / 16;           // score MFMAs per tile
    constexpr int EPS = 16 / NS;          // exponentials placed behind each of them
    constexpr int ND = HD / 32;           // accumulators of O^T (== NS / 2)
    half8 kf0[NS / 2], kf1[NS / 2], vf0[ND], vf1[ND];
#pragma unroll
    for (int s = 0; s < NS / 2; s++)
        kf0[s] = *reinterpret_cast<const half8*>(smem + ((kslot + cx.kread) ^ (s * 32)));
#pragma unroll
    for (int dt = 0; dt < ND; dt++)
        vf0[dt] = *reinterpret_cast<const half8*>(smem + (vslot + cx.vread) + dt * 2048);
    split_softmax_begin<HD>(R, negm, c, tile, g);
    __builtin_amdgcn_sched_barrier(0);

    half8 pop[2];
    float psum = 0.f;
    const half2v ones = {(_Float16)1.0f, (_Float16)1.0f};
#pragma unroll
    for (int s = 0; s < NS; s++) {
        // the chain starts from the reference block and writes the next scores
        // directly (no copy of either)
        if (s == 0)
            sn = __builtin_amdgcn_mfma_f32_32x32x16_f16(kf0[0], R.qop[0], negm, 0, 0, 0);
        else
            sn = __builtin_amdgcn_mfma_f32_32x32x16_f16(
                s < NS / 2 ? kf0[s % (NS / 2)] : kf1[s % (NS / 2)], R.qop[s], sn, 0, 0, 0);
        if (s == 0) {
#pragma unroll
            for (int s2 = 0; s2 < NS / 2; s2++)
                kf1[s2] = *reinterpret_cast<const half8*>(smem + ((kslot + cx.kread) ^ ((NS / 2 + s2) * 32)));
        }
        if (s == NS / 2) {
#pragma unroll
            for (int dt = 0; dt < ND; dt++)
                vf1[dt] = *reinterpret_cast<const half8*>(smem + ((vslot + cx.vread) ^ 32) + dt * 2048);
        }
        if (s >= NS / 2) {
            // the first eight probabilities are complete: their half of P.V fills
            // the idle slots of the score chain
            const int dt = s - NS / 2;
            R.o[dt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(vf0[dt], pop[0], R.o[dt], 0, 0, 0);
        }
        // probabilities in pairs: two exp2, one pack to F16, one dot product with
        // (1, 1) that adds the two ROUNDED values to the row sum, so the
        // normaliser is the sum of exactly what P.V multiplies
#pragma unroll
        for (int e = 0; e < EPS; e += 2) {
            const int r = s * EPS + e;
            const half2v ph = {(_Float16)fast_exp2(c[r]), (_Float16)fast_exp2(c[r + 1])};
            psum = __builtin_amdgcn_fdot2(ph, ones, psum, false);
            pop[r >> 3][r & 7] = ph[0];
            pop[r >> 3][(r & 7) + 1] = ph[1];
        }
    }
    R.l_run += psum;
#pragma unroll
    for (int dt = 0; dt < ND; dt++)
        R.o[dt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(vf1[dt], pop[1], R.o[dt], 0, 0, 0);
    // vector work of one probability: exp2, half a pack, half a dot product
    split_step_order<0, NS, 2 * EPS + 1>();
    __builtin_amdgcn_sched_group_barrier(0x008, ND, 0);
    // the loads for later steps leave once the operand reads are in the queue
    split_move<HD>(cx, i, wave & 3);
}

// Work of one wave in its set's step j: the set's j-th tile is finished (scores
// in `c`), the scores of tile j+1 go to `sn`, and the wave's share of the step's
// loads is issued.  Every wave runs the same code in every step: a wave whose
// range does not hold the step's tile works on scores of -inf (probabilities 0;
// the staged Vt it multiplies them with is real data of the block), and scores
// computed for a tile past its range are never used.  One path keeps the
// accumulators in the same registers throughout the loop.
template <int HD>
__device__ __forceinline__ void split_wave_step(PrefillRows<HD>& R, f32x16& negm, f32x16& c,
                                                f32x16& sn,
                                                const unsigned char* smem, const SplitCtx<HD>& cx,
                                                uint32_t j, int wave, int g)
{
    using L = SplitLds<HD>;
    const uint32_t tile = cx.t0 + 2 * j;
    const bool has_cur = R.wave_ok && tile >= R.wt_first && tile <= R.wt_last;
    if (!has_cur) {
        // rare and wave-uniform: keep it a branch (the empty statement stops the
        // compiler from turning it into sixteen selects executed in every step)
        asm volatile("" ::: "memory");
#pragma unroll
        for (int r = 0; r < 16; r++) c[r] = -INFINITY;
    }
    const uint32_t kslot = cx.ring + ((j + 1) % kRing) * L::KTILE;   // K is one step ahead of Vt
    const uint32_t vslot = cx.ring + L::V_IN_SET + (j % kRing) * L::VTILE;
    split_step<HD>(R, negm, c, sn, smem, cx, j, wave, kslot, vslot, tile, g);
}

template <int HD>
__device__ __forceinline__ void split_block(const PrefillArgs& a, unsigned char* smem,
                                            uint32_t pb, uint32_t kvh, uint32_t hc)
{
    using L = SplitLds<HD>;
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
    uint32_t t_first, t_last;
    prefill_block_tiles(a, pb, BP, t_first, t_last);
    SplitCtx<HD> cx;
    cx.t0 = t_first + kg;                                 // this set's tiles: t0, t0 + 2, ...
    cx.nt = (cx.t0 <= t_last) ? (t_last - cx.t0) / 2 + 1 : 0;
    cx.t_last = t_last;
    cx.kv_valid = a.p0 + a.T;                             // rows of the cache that hold data
    cx.kbase = uniform_ptr(reinterpret_cast<const unsigned char*>(a.k + (size_t)kvh * a.ctx_pad * HD));
    cx.vtbase = uniform_ptr(reinterpret_cast<const unsigned char*>(
        a.vt + (size_t)kvh * (a.ctx_pad / kVBlock) * HD * kVBlock));
    // low half of a generic LDS pointer = LDS byte address
    cx.lds0 = (uint32_t)__builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)smem);
    cx.ring = kg * L::SET_BYTES;
    cx.cnt = L::CNT_OFF + kg * 4;
    {
        // K: lane -> (row of the tile, slot); fetch the chunk that belongs in that slot
        const int row = sub * (1024 / L::RB) + lane / L::CPR;
        const int chunk = (lane % L::CPR) ^ L::fk(row);
        cx.gk_off = ((k_tile_half(row) * L::CPR + chunk) * 16 + k_tile_slot(row)) * 16;
        // Vt: rows of 64 bytes, four slots each
        const int vrow = sub * 16 + lane / 4;
        cx.gv_off = vrow * 64 + ((lane & 3) ^ L::fv(vrow)) * 16;
        static_assert(L::NL == 1 || (L::NL == 2 && 4 * (1024 / L::RB) == 16 && L::fk(16) == L::fk(0) &&
                                     L::fv(64) == L::fv(0)),
                      "the second load is 16 K rows (128 bytes in the cache) / 64 Vt rows (4 KiB) further");
        const int krow = prefill_key_perm(n);             // tile row this lane feeds to MFMA row n
        cx.kread = krow * L::RB + ((g ^ L::fk(krow)) * 16);
        cx.vread = n * 64 + ((g ^ L::fv(n)) * 16);
    }

    // Everything steps 0 and 1 of this set read, in order of need.  (A set
    // without a tile, the odd set of a one-tile block, goes through one step
    // all the same, on duplicates of the block's last tile and scores of -inf:
    // a path around the loop would cost the loop its register allocation.)
    split_issue_k<HD>(cx, 0, 0, sub);
    split_issue_k<HD>(cx, 1, 1, sub);
    split_issue_v<HD>(cx, 0, 0, sub);
    split_issue_k<HD>(cx, 2, 2, sub);
    split_issue_v<HD>(cx, 1, 1, sub);
    if (tid < 2) reinterpret_cast<uint32_t*>(smem + L::CNT_OFF)[tid] = 0;

    PrefillRows<HD> R;
    prefill_rows_init<HD, false>(R, a, row0, head, n, g);

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

    // prologue: the first tiles, Q and the zeroed counters become visible to
    // the whole workgroup, then every set computes its first scores
    f32x16 s0, s1, negm;
#pragma unroll
    for (int r = 0; r < 16; r++) s0[r] = s1[r] = negm[r] = 0.f;
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    lds_barrier();
#pragma unroll
    for (int s = 0; s < HD / 16; s++)
        R.qop[s] = *reinterpret_cast<const half8*>(&qs[sub][n][s * 16 + g * 8]);
    if (R.wave_ok && cx.t0 >= R.wt_first && cx.t0 <= R.wt_last)
        split_scores<HD>(R, negm, s0, smem, cx, cx.ring);

    // Before the barrier of step j every load of this wave but the ones step
    // j-1 issued has landed: K of tile j+1 and Vt of tile j, which step j
    // reads, left in step j-2.  The barrier is the set's own: it publishes the
    // four waves' loads to each other and tells them that the slots step j
    // overwrites are no longer being read.
    const uint32_t nsteps = max(cx.nt, 1u);
    for (uint32_t j = 0;; j += 2) {
        asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * L::NL) : "memory");
        split_patch_tail<HD>(smem, cx, j, sub, lane);
        set_barrier(smem, cx.cnt, 4 * (j + 1), lane, a.err, a.err_code);
        split_wave_step<HD>(R, negm, s0, s1, smem, cx, j, wave, g);
        if (j + 1 >= nsteps) break;
        asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * L::NL) : "memory");
        split_patch_tail<HD>(smem, cx, j + 1, sub, lane);
        set_barrier(smem, cx.cnt, 4 * (j + 2), lane, a.err, a.err_code);
        split_wave_step<HD>(R, negm, s1, s0, smem, cx, j + 1, wave, g);
        if (j + 2 >= nsteps) break;
    }

    // merge the odd-tile partials into the even-tile waves; the ring must be
    // quiet first (the last steps' loads still target it)
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
}

// grid = (KV heads x head chunks, ceil(blocks / 2)): consecutive workgroups (which
// the dispatcher deals round-robin to the XCDs) differ in KV head, so one XCD's
// L2 keeps seeing the same few heads' K / Vt.  Workgroup y takes position block
// (blocks-1-y) and then block y: a long block and a short one, so every
// workgroup streams the same number of tiles despite the causal triangle.
// a.single: grid.y = blocks, one block per workgroup, long blocks first.
template <int HD>
__global__ __launch_bounds__(kSplitThreads, 1) void prefill_split_kernel(const PrefillArgs a)
{
    extern __shared__ __attribute__((aligned(16))) unsigned char prefill_smem_raw[];
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
        split_block<HD>(a, prefill_smem_raw, pass ? lo : hi, kvh, hc);
    }
}

}  // namespace wr
