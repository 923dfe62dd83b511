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

__device__ __forceinline__ int prefill_key_perm(int m)
{
    const int a = m >> 3, g = (m >> 2) & 1, b = m & 3;
    return 16 * (a >> 1) + 8 * g + 4 * (a & 1) + b;
}

template <int HD>
__global__ __launch_bounds__(kPrefillThreads, 2) void prefill_mfma_kernel(const PrefillArgs a)
{
    constexpr int KSTR = HD + 8;              // halves per K row in LDS (16-byte pad: conflict-free b128 reads)
    constexpr int VSTR = kVBlock + 8;         // halves per Vt row in LDS
    constexpr int KCH = HD / 8;               // 16-byte chunks per K row
    __shared__ __attribute__((aligned(16))) _Float16 lds_k[2][kTileKeys][KSTR];
    __shared__ __attribute__((aligned(16))) _Float16 lds_v[2][HD][VSTR];

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int n = lane & 31, g = lane >> 5;
    const uint32_t G = a.group;
    const uint32_t Gw = G < 4 ? G : 4;
    const uint32_t chunks = G / Gw;                       // head chunks per KV head (1, or 2 for G = 8)
    const uint32_t kvh = blockIdx.y / chunks, hc = blockIdx.y % chunks;
    const uint32_t BP = 32 * (4 / Gw);                    // positions per workgroup
    const uint32_t pb = gridDim.x - 1 - blockIdx.x;       // heaviest block first
    const uint32_t head = kvh * G + hc * Gw + (wave % Gw);
    const uint32_t row0 = pb * BP + (wave / Gw) * 32;     // first chunk row of this wave
    const uint32_t T = a.T, p0 = a.p0;
    const uint32_t kv_valid = p0 + T;                     // rows of the cache that hold data

    const uint32_t my_row = row0 + n;
    const bool row_ok = my_row < T;
    const uint32_t pos = p0 + (row_ok ? my_row : T - 1);  // absolute position (clamped for idle rows)
    const uint32_t row_lo = (a.window > 0 && pos + 1 > a.window) ? pos + 1 - a.window : 0;

    // workgroup-wide tile range
    const uint32_t wg_last_row = min(T, (pb + 1) * BP) - 1;
    const uint32_t wg_first_pos = p0 + pb * BP;
    const uint32_t wg_lo = (a.window > 0 && wg_first_pos + 1 > a.window) ? wg_first_pos + 1 - a.window : 0;
    const uint32_t t_first = wg_lo / kTileKeys;
    const uint32_t t_last = (p0 + wg_last_row) / kTileKeys;          // inclusive
    // this wave's own range (a wave with no valid row computes nothing)
    const bool wave_ok = row0 < T;
    const uint32_t w_last_pos = p0 + min(T - 1, row0 + 31);
    const uint32_t w_first_pos = p0 + row0;
    const uint32_t w_lo = (a.window > 0 && w_first_pos + 1 > a.window) ? w_first_pos + 1 - a.window : 0;
    const uint32_t wt_first = w_lo / kTileKeys;
    const uint32_t wt_last = w_last_pos / kTileKeys;

    // Q^T operand: column n = this lane's row, contraction slots (g, j) = dims s*16 + g*8 + j
    half8 qop[HD / 16];
    {
        const float* qrow = a.q + ((size_t)(row_ok ? my_row : T - 1) * a.nq + head) * HD;
#pragma unroll
        for (int s = 0; s < HD / 16; s++) {
            const float4 x0 = *reinterpret_cast<const float4*>(qrow + s * 16 + g * 8);
            const float4 x1 = *reinterpret_cast<const float4*>(qrow + s * 16 + g * 8 + 4);
            qop[s][0] = (_Float16)(x0.x * a.qscale);
            qop[s][1] = (_Float16)(x0.y * a.qscale);
            qop[s][2] = (_Float16)(x0.z * a.qscale);
            qop[s][3] = (_Float16)(x0.w * a.qscale);
            qop[s][4] = (_Float16)(x1.x * a.qscale);
            qop[s][5] = (_Float16)(x1.y * a.qscale);
            qop[s][6] = (_Float16)(x1.z * a.qscale);
            qop[s][7] = (_Float16)(x1.w * a.qscale);
        }
    }

    f32x16 o[HD / 32];
#pragma unroll
    for (int dt = 0; dt < HD / 32; dt++)
#pragma unroll
        for (int r = 0; r < 16; r++) o[dt][r] = 0.f;
    float m_run = -INFINITY, l_run = 0.f;

    const uint16_t* kbase = a.k + (size_t)kvh * a.ctx_pad * HD;
    const uint16_t* vtbase = a.vt + (size_t)kvh * (a.ctx_pad / kVBlock) * HD * kVBlock;
    const int krow = prefill_key_perm(n);                 // LDS row this lane feeds to MFMA row n

    // staging registers: each thread moves HD/64 16-byte chunks of K and of Vt per tile
    constexpr int NCH = HD / 64;
    u32x4 stage_k[NCH], stage_v[NCH];
    auto fetch = [&](uint32_t tile) {
        const u32x4* ksrc = reinterpret_cast<const u32x4*>(kbase + (size_t)tile * kTileKeys * HD);
        const u32x4* vsrc = reinterpret_cast<const u32x4*>(vtbase + (size_t)tile * HD * kVBlock);
#pragma unroll
        for (int c = 0; c < NCH; c++) {
            stage_k[c] = ksrc[tid + c * kPrefillThreads];
            stage_v[c] = vsrc[tid + c * kPrefillThreads];
        }
    };
    auto stash = [&](int buf, uint32_t tile) {
        const bool tail = (tile + 1) * kTileKeys > kv_valid;    // tile reaches past the appended rows
#pragma unroll
        for (int c = 0; c < NCH; c++) {
            const int ch = tid + c * kPrefillThreads;
            *reinterpret_cast<u32x4*>(&lds_k[buf][ch / KCH][(ch % KCH) * 8]) = stage_k[c];
            u32x4 v = stage_v[c];
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
            *reinterpret_cast<u32x4*>(&lds_v[buf][ch >> 2][(ch & 3) * 8]) = v;
        }
    };

    fetch(t_first);
    int buf = 0;
    for (uint32_t tile = t_first; tile <= t_last; tile++, buf ^= 1) {
        stash(buf, tile);
        __syncthreads();
        if (tile < t_last) fetch(tile + 1);
        if (!wave_ok || tile < wt_first || tile > wt_last) continue;

        const uint32_t kb = tile * kTileKeys;
        f32x16 c;
#pragma unroll
        for (int r = 0; r < 16; r++) c[r] = 0.f;
#pragma unroll
        for (int s = 0; s < HD / 16; s++) {
            const half8 kf = *reinterpret_cast<const half8*>(&lds_k[buf][krow][s * 16 + g * 8]);
            c = __builtin_amdgcn_mfma_f32_32x32x16_f16(kf, qop[s], c, 0, 0, 0);
        }
        // register r of this lane: key kb + 16*(r/8) + 8*g + r%8, row n
        // some (row, key) pair of this tile is invisible: above the diagonal of
        // the wave's first row, or below the window of its last row
        const uint32_t w_hi_lo =
            (a.window > 0 && w_last_pos + 1 > a.window) ? w_last_pos + 1 - a.window : 0;
        const bool edge = (kb + kTileKeys - 1 > w_first_pos) || (kb < w_hi_lo);
        if (edge) {
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const uint32_t key = kb + 16 * (r >> 3) + 8 * g + (r & 7);
                if (key > pos || key < row_lo) c[r] = -INFINITY;
            }
        }
        float tmax = c[0];
#pragma unroll
        for (int r = 1; r < 16; r++) tmax = fmaxf(tmax, c[r]);
        tmax = fmaxf(tmax, wave_xor_f32(tmax, 32));
        const float m_new = fmaxf(m_run, tmax);
        const float m_safe = (m_new == -INFINITY) ? 0.f : m_new;   // row with nothing visible yet
        const float alpha = fast_exp2(m_run - m_safe);
        m_run = m_new;

        half8 pop[2];
        float psum = 0.f;
#pragma unroll
        for (int r = 0; r < 16; r++) {
            const float p = fast_exp2(c[r] - m_safe);
            psum += p;
            pop[r >> 3][r & 7] = (_Float16)p;
        }
        l_run = l_run * alpha + psum;

        // rescale only when some row's maximum moved (wave-uniform test)
        if (__builtin_amdgcn_ballot_w64(alpha != 1.0f) != 0) {
#pragma unroll
            for (int dt = 0; dt < HD / 32; dt++)
#pragma unroll
                for (int r = 0; r < 16; r++) o[dt][r] *= alpha;
        }
#pragma unroll
        for (int dt = 0; dt < HD / 32; dt++) {
#pragma unroll
            for (int t = 0; t < 2; t++) {
                const half8 vf =
                    *reinterpret_cast<const half8*>(&lds_v[buf][dt * 32 + n][16 * t + 8 * g]);
                o[dt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(vf, pop[t], o[dt], 0, 0, 0);
            }
        }
    }

    const float l_tot = l_run + wave_xor_f32(l_run, 32);
    const float inv = (l_tot > 0.f) ? 1.0f / l_tot : 0.f;
    if (row_ok) {
        float* orow = a.out + ((size_t)my_row * a.nq + head) * HD;
#pragma unroll
        for (int dt = 0; dt < HD / 32; dt++) {
#pragma unroll
            for (int q4 = 0; q4 < 4; q4++) {
                float4 v;
                v.x = o[dt][4 * q4 + 0] * inv;
                v.y = o[dt][4 * q4 + 1] * inv;
                v.z = o[dt][4 * q4 + 2] * inv;
                v.w = o[dt][4 * q4 + 3] * inv;
                *reinterpret_cast<float4*>(orow + dt * 32 + 8 * q4 + 4 * g) = v;
            }
        }
    }
}

}  // namespace wr
