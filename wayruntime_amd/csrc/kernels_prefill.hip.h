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
    const uint16_t* q16;     // or: the same rows as binary16, already multiplied by qscale (prefill_il_kernel only)
    float* out;              // [T][nq][hd]
    uint32_t p0, T, nq, nkv, group, hd, ctx_pad, window;
    float qscale;            // softmax scale * log2(e)
    uint32_t single;         // MFMA kernels: one position block per workgroup (grid = blocks) instead of a pair
};

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

}  // namespace wr
