// Split-K decode attention (one query row per head) over the F16 cache.
//
// Computes what the reference computes with seq_q = 1
// (reference: src/core/kernels.c:1475-1523): for head qh with KV head
// kvh = qh / group, softmax over the visible keys of scale * q.k, times V.
// Summation order differs from the reference (keys are split over waves and
// workgroups and merged by log-sum-exp), so results agree to rounding, not
// bit for bit.
//
// Work decomposition: grid = (key splits, KV heads, sessions).  One workgroup
// owns ONE KV head of one session over a contiguous run of 32-key tiles and
// serves the whole GQA group from it, so every K and V byte is fetched from
// HBM exactly once.  Its four waves take tiles round-robin and keep private
// online-softmax state (m, l, O); they merge through LDS at the end and the
// workgroup writes either the final rows (single split) or one partial
// (m, l, unnormalised O) per head that decode_combine_kernel merges.
//
// HBM-bound: algorithmic bytes per launch = 4 * nkv * hd * sum(seq_k)
// (K and V, two bytes each); Q, O and partials are <1 %.
//
// Inside a wave the two contractions run on the matrix cores only to take the
// arithmetic off the vector ALUs (a 4-head group would otherwise need ~100
// VALU ops per 32 bytes loaded, which caps bandwidth).  Accuracy is kept at
// F32 level by splitting the F32 operands into two halves-precision terms:
// q = q_hi + q_lo and p = p_hi + p_lo, each term a separate MFMA into the same
// F32 accumulator.  K and V are already F16, so nothing is lost there.
//
//   S^T[key][head] = K[key][:] . Q^T[:][head]      v_mfma_f32_16x16x32_f16
//   O^T[dim][head] += Vt[dim][key] . P^T[key][head]
//
// Orientation is chosen so a head is a COLUMN: lane l owns column l%16 in
// both accumulators, so max / sum / rescale of one head never leave the lane
// except for one exchange across the four 16-lane groups.
#pragma once

#include "common.hip.h"

namespace wr {

constexpr int kDecodeThreads = 256;
constexpr int kDecodeWaves = 4;
constexpr int kTileKeys = 32;
constexpr int kMaxGroupMfma = 8;      // heads per KV head the MFMA kernel serves
constexpr int kBatchMax = 16;

struct DecodeSession {
    const uint16_t* k;       // K of this layer
    const uint16_t* vt;      // Vt of this layer
    uint32_t seq_k;          // valid rows
    uint32_t key_lo;         // first visible key (sliding window), else 0
    uint32_t ctx_pad;        // rows allocated per KV head (multiple of 32)
    uint32_t n_splits;       // workgroups along the key axis
};

struct DecodeArgs {
    DecodeSession s[kBatchMax];
    const float* q;          // [n][nq][hd]
    float* out;              // [n][nq][hd]
    float* part_o;           // [n][nq][max_splits][hd], unnormalised
    float* part_ml;          // [n][nq][max_splits][2] = (m in log2 units, l)
    uint32_t nq, nkv, group, hd;
    uint32_t tiles_per_wg;   // 32-key tiles per workgroup
    uint32_t max_splits;
    uint32_t direct;         // 1: every session has one split, write final rows
    float qscale;            // softmax scale * log2(e)
};

struct TileRange {
    uint32_t t_begin, t_end;      // tiles [t_begin, t_end)
};

__device__ __forceinline__ TileRange split_tiles(const DecodeSession& S, uint32_t split,
                                                 uint32_t tiles_per_wg)
{
    const uint32_t first = S.key_lo / kTileKeys;
    const uint32_t last = (S.seq_k + kTileKeys - 1) / kTileKeys;
    TileRange r;
    r.t_begin = first + split * tiles_per_wg;
    r.t_end = min(r.t_begin + tiles_per_wg, last);
    return r;
}

// ------------------------------------------------------------------ MFMA --

template <int HD>
struct DecodeFrag {
    half8 k[2][HD / 32];     // two 16-key sub-tiles x (HD/32) contraction steps
    half8 v[HD / 16];        // HD/16 dimension tiles x 32 keys
};

template <int HD>
__device__ __forceinline__ void load_frag(DecodeFrag<HD>& f, const uint16_t* __restrict__ kbase,
                                          const uint16_t* __restrict__ vtbase, uint32_t tile,
                                          int lane)
{
    const int m = lane & 15, g = lane >> 4;
    const uint32_t kb = tile * kTileKeys;
    // Sub-tile t feeds MFMA row m with key kb + 8*(m/4) + 4t + m%4, so that the
    // accumulator of lane group g ends up holding keys kb+8g .. kb+8g+7 in
    // order: exactly the eight consecutive positions that group reads from Vt.
#pragma unroll
    for (int t = 0; t < 2; t++) {
        const uint32_t key = kb + 8 * (m >> 2) + 4 * t + (m & 3);
        const half8* row = reinterpret_cast<const half8*>(kbase + (size_t)key * HD);
#pragma unroll
        for (int s = 0; s < HD / 32; s++) f.k[t][s] = row[s * 4 + g];
    }
    const half8* vb = reinterpret_cast<const half8*>(vtbase + (size_t)tile * HD * kVBlock);
#pragma unroll
    for (int dt = 0; dt < HD / 16; dt++) f.v[dt] = vb[(dt * 16 + m) * 4 + g];
}

template <int HD>
struct DecodeState {
    f32x4 o[HD / 16];        // O^T: dim = dt*16 + 4g + r, head = lane%16
    float m;                 // running max (log2 units), common to the 4 groups
    float l;                 // this lane group's share of the denominator
};

template <int HD>
__device__ __forceinline__ void process_tile(DecodeState<HD>& st, DecodeFrag<HD>& f,
                                             const half8 (&qhi)[HD / 32],
                                             const half8 (&qlo)[HD / 32], uint32_t tile,
                                             uint32_t key_lo, uint32_t seq_k, int lane)
{
    const int g = lane >> 4;
    const uint32_t kb = tile * kTileKeys;

    f32x4 c[2];
#pragma unroll
    for (int t = 0; t < 2; t++) {
        c[t] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int s = 0; s < HD / 32; s++) {
            c[t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(f.k[t][s], qhi[s], c[t], 0, 0, 0);
            c[t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(f.k[t][s], qlo[s], c[t], 0, 0, 0);
        }
    }
    float sc[8];
#pragma unroll
    for (int j = 0; j < 8; j++) sc[j] = c[j >> 2][j & 3];

    const bool boundary = (kb < key_lo) || (kb + kTileKeys > seq_k);
    if (boundary) {
        const uint32_t k0 = kb + 8 * g;
#pragma unroll
        for (int j = 0; j < 8; j++) {
            const uint32_t key = k0 + j;
            if (key < key_lo || key >= seq_k) sc[j] = -INFINITY;
        }
        // Rows above the cursor may hold anything; zero them so 0 * garbage
        // cannot poison the accumulator.
        if (kb + kTileKeys > seq_k) {
#pragma unroll
            for (int dt = 0; dt < HD / 16; dt++) {
#pragma unroll
                for (int j = 0; j < 8; j++)
                    if (k0 + j >= seq_k) f.v[dt][j] = (_Float16)0.0f;
            }
        }
    }

    float tmax = sc[0];
#pragma unroll
    for (int j = 1; j < 8; j++) tmax = fmaxf(tmax, sc[j]);
    tmax = fmaxf(tmax, wave_xor_f32(tmax, 16));
    tmax = fmaxf(tmax, wave_xor_f32(tmax, 32));

    const float m_new = fmaxf(st.m, tmax);
    const float alpha = fast_exp2(st.m - m_new);
    st.m = m_new;

    half8 phi, plo;
    float psum = 0.f;
#pragma unroll
    for (int j = 0; j < 8; j++) {
        const float p = fast_exp2(sc[j] - m_new);
        psum += p;
        const _Float16 h = (_Float16)p;
        phi[j] = h;
        plo[j] = (_Float16)(p - (float)h);
    }
    st.l = st.l * alpha + psum;

#pragma unroll
    for (int dt = 0; dt < HD / 16; dt++) {
        st.o[dt] *= alpha;
        st.o[dt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(f.v[dt], phi, st.o[dt], 0, 0, 0);
        st.o[dt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(f.v[dt], plo, st.o[dt], 0, 0, 0);
    }
}

// Waves per SIMD the register budget is sized for: two double-buffered tiles of
// a 256-wide head need more than 256 registers, so that shape runs one wave
// per SIMD with the full 512-register file (32 KB of loads in flight per wave).
template <int HD>
constexpr int decode_waves_per_simd() { return HD >= 256 ? 1 : 2; }

template <int HD>
__global__ __launch_bounds__(kDecodeThreads, decode_waves_per_simd<HD>())
void decode_mfma_kernel(const DecodeArgs a)
{
    const uint32_t split = blockIdx.x, kvh = blockIdx.y, sess = blockIdx.z;
    const DecodeSession S = a.s[sess];
    if (split >= S.n_splits) return;

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int n = lane & 15, g = lane >> 4;
    const uint32_t G = a.group;
    const TileRange tr = split_tiles(S, split, a.tiles_per_wg);

    // Q^T operand: column n is head kvh*G + n (zero beyond the group), scaled
    // into log2 units and split into two half-precision terms.
    half8 qhi[HD / 32], qlo[HD / 32];
    {
        const float* qrow = a.q + ((size_t)sess * a.nq + kvh * G + (n < (int)G ? n : 0)) * HD;
#pragma unroll
        for (int s = 0; s < HD / 32; s++) {
#pragma unroll
            for (int j = 0; j < 8; j++) {
                float x = (n < (int)G) ? qrow[s * 32 + g * 8 + j] * a.qscale : 0.f;
                const _Float16 h = (_Float16)x;
                qhi[s][j] = h;
                qlo[s][j] = (_Float16)(x - (float)h);
            }
        }
    }

    DecodeState<HD> st;
#pragma unroll
    for (int dt = 0; dt < HD / 16; dt++) st.o[dt] = f32x4{0.f, 0.f, 0.f, 0.f};
    st.m = -INFINITY;
    st.l = 0.f;

    const uint16_t* kbase = S.k + (size_t)kvh * S.ctx_pad * HD;
    const uint16_t* vtbase = S.vt + (size_t)kvh * (S.ctx_pad / kVBlock) * HD * kVBlock;

    uint32_t t = tr.t_begin + wave;
    if (t < tr.t_end) {
        DecodeFrag<HD> fa, fb;
        load_frag<HD>(fa, kbase, vtbase, t, lane);
        for (;;) {
            const uint32_t t1 = t + kDecodeWaves;
            if (t1 < tr.t_end) load_frag<HD>(fb, kbase, vtbase, t1, lane);
            process_tile<HD>(st, fa, qhi, qlo, t, S.key_lo, S.seq_k, lane);
            if (t1 >= tr.t_end) break;
            const uint32_t t2 = t1 + kDecodeWaves;
            if (t2 < tr.t_end) load_frag<HD>(fa, kbase, vtbase, t2, lane);
            process_tile<HD>(st, fb, qhi, qlo, t1, S.key_lo, S.seq_k, lane);
            if (t2 >= tr.t_end) break;
            t = t2;
        }
    }
    // denominator: add the four lane groups' shares
    st.l += wave_xor_f32(st.l, 16);
    st.l += wave_xor_f32(st.l, 32);

    __shared__ float lds_o[kDecodeWaves][kMaxGroupMfma][HD];
    __shared__ float lds_m[kDecodeWaves][kMaxGroupMfma];
    __shared__ float lds_l[kDecodeWaves][kMaxGroupMfma];
    if (n < (int)G) {
#pragma unroll
        for (int dt = 0; dt < HD / 16; dt++)
#pragma unroll
            for (int r = 0; r < 4; r++) lds_o[wave][n][dt * 16 + 4 * g + r] = st.o[dt][r];
        if (g == 0) {
            lds_m[wave][n] = st.m;
            lds_l[wave][n] = st.l;
        }
    }
    __syncthreads();

    for (uint32_t idx = threadIdx.x; idx < G * HD; idx += kDecodeThreads) {
        const uint32_t h = idx / HD, d = idx % HD;
        float M = lds_m[0][h];
#pragma unroll
        for (int w = 1; w < kDecodeWaves; w++) M = fmaxf(M, lds_m[w][h]);
        float acc = 0.f, L = 0.f;
#pragma unroll
        for (int w = 0; w < kDecodeWaves; w++) {
            const float fct = fast_exp2(lds_m[w][h] - M);   // idle wave: exp2(-inf) = 0
            acc += lds_o[w][h][d] * fct;
            L += lds_l[w][h] * fct;
        }
        const uint32_t head = kvh * G + h;
        if (a.direct) {
            a.out[((size_t)sess * a.nq + head) * HD + d] = (L > 0.f) ? acc / L : 0.f;
        } else {
            const size_t pi = ((size_t)sess * a.nq + head) * a.max_splits + split;
            a.part_o[pi * HD + d] = acc;
            if (d == 0) {
                a.part_ml[pi * 2 + 0] = M;
                a.part_ml[pi * 2 + 1] = L;
            }
        }
    }
}

// --------------------------------------------------------------- generic --
// Any head_dim up to 1024 and any group size: one workgroup per (split, query
// head, session), vector ALU only.  Slow; exists so every shape the reference
// accepts has a device path, and as a second implementation to cross-check
// the MFMA kernel against.

constexpr int kGenericMaxPerLane = 16;      // 1024 / 64
constexpr int kFlashDMax = 1024;            // largest head_dim (reference: WR_FLASH_D_MAX)

struct GenericShared {
    float o[kDecodeWaves][kFlashDMax];
    float m[kDecodeWaves];
    float l[kDecodeWaves];
};

// One workgroup attends one query row of one head over keys
// [key_begin, key_end): waves take keys round-robin, lanes split head_dim.
// On return (after the barrier inside) sh holds each wave's (m, l, O) and the
// caller merges them with merge_generic().
__device__ __forceinline__ void generic_attend_wg(GenericShared& sh, const uint16_t* __restrict__ k,
                                                  const uint16_t* __restrict__ vt, uint32_t ctx_pad,
                                                  uint32_t kvh, uint32_t hd, uint32_t key_begin,
                                                  uint32_t key_end, const float* __restrict__ qrow,
                                                  float qscale)
{
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    float qv[kGenericMaxPerLane], o[kGenericMaxPerLane];
#pragma unroll
    for (int i = 0; i < kGenericMaxPerLane; i++) {
        const uint32_t d = lane + 64 * i;
        qv[i] = (d < hd) ? qrow[d] * qscale : 0.f;
        o[i] = 0.f;
    }
    float m = -INFINITY, l = 0.f;

    for (uint32_t key = key_begin + wave; key < key_end; key += kDecodeWaves) {
        const uint16_t* krow = k + k_row_offset(kvh, ctx_pad, key, hd);
        float dot = 0.f;
#pragma unroll
        for (int i = 0; i < kGenericMaxPerLane; i++) {
            const uint32_t d = lane + 64 * i;
            if (d < hd) dot += qv[i] * (float)(*reinterpret_cast<const _Float16*>(krow + d));
        }
#pragma unroll
        for (int off = 32; off >= 1; off >>= 1) dot += wave_xor_f32(dot, off);
        const float m_new = fmaxf(m, dot);
        const float alpha = fast_exp2(m - m_new);
        const float p = fast_exp2(dot - m_new);
        l = l * alpha + p;
        m = m_new;
#pragma unroll
        for (int i = 0; i < kGenericMaxPerLane; i++) {
            const uint32_t d = lane + 64 * i;
            if (d < hd) {
                const uint16_t vb = vt[vt_offset(kvh, ctx_pad, key, d, hd)];
                o[i] = o[i] * alpha + p * (float)(*reinterpret_cast<const _Float16*>(&vb));
            }
        }
    }
#pragma unroll
    for (int i = 0; i < kGenericMaxPerLane; i++) {
        const uint32_t d = lane + 64 * i;
        if (d < hd) sh.o[wave][d] = o[i];
    }
    if (lane == 0) {
        sh.m[wave] = m;
        sh.l[wave] = l;
    }
    __syncthreads();
}

struct GenericMerge {
    float M, L;
    float fct[kDecodeWaves];
};

__device__ __forceinline__ GenericMerge merge_generic(const GenericShared& sh)
{
    GenericMerge g;
    g.M = sh.m[0];
#pragma unroll
    for (int w = 1; w < kDecodeWaves; w++) g.M = fmaxf(g.M, sh.m[w]);
    g.L = 0.f;
#pragma unroll
    for (int w = 0; w < kDecodeWaves; w++) {
        g.fct[w] = fast_exp2(sh.m[w] - g.M);       // idle wave: exp2(-inf) = 0
        g.L += sh.l[w] * g.fct[w];
    }
    return g;
}

__global__ __launch_bounds__(kDecodeThreads) void decode_generic_kernel(const DecodeArgs a)
{
    const uint32_t split = blockIdx.x, head = blockIdx.y, sess = blockIdx.z;
    const DecodeSession S = a.s[sess];
    if (split >= S.n_splits) return;
    const uint32_t hd = a.hd;
    const uint32_t kvh = head / a.group;
    const TileRange tr = split_tiles(S, split, a.tiles_per_wg);
    const uint32_t key_begin = max(tr.t_begin * kTileKeys, S.key_lo);
    const uint32_t key_end = min(tr.t_end * kTileKeys, S.seq_k);

    __shared__ GenericShared sh;
    generic_attend_wg(sh, S.k, S.vt, S.ctx_pad, kvh, hd, key_begin, key_end,
                      a.q + ((size_t)sess * a.nq + head) * hd, a.qscale);
    const GenericMerge g = merge_generic(sh);

    for (uint32_t d = threadIdx.x; d < hd; d += kDecodeThreads) {
        float acc = 0.f;
#pragma unroll
        for (int w = 0; w < kDecodeWaves; w++) acc += sh.o[w][d] * g.fct[w];
        if (a.direct) {
            a.out[((size_t)sess * a.nq + head) * hd + d] = (g.L > 0.f) ? acc / g.L : 0.f;
        } else {
            const size_t pi = ((size_t)sess * a.nq + head) * a.max_splits + split;
            a.part_o[pi * hd + d] = acc;
            if (d == 0) {
                a.part_ml[pi * 2 + 0] = g.M;
                a.part_ml[pi * 2 + 1] = g.L;
            }
        }
    }
}

// --------------------------------------------------------------- combine --
// Merges the per-split partials of one (session, head): log-sum-exp over the
// split maxima, then one normalisation.  grid = (nq, sessions).

__global__ __launch_bounds__(128) void decode_combine_kernel(const DecodeArgs a)
{
    const uint32_t head = blockIdx.x, sess = blockIdx.y;
    const uint32_t ns = a.s[sess].n_splits;
    const uint32_t hd = a.hd;
    const size_t base = ((size_t)sess * a.nq + head) * a.max_splits;

    float M = -INFINITY;
    for (uint32_t i = 0; i < ns; i++) M = fmaxf(M, a.part_ml[(base + i) * 2]);
    float L = 0.f;
    for (uint32_t i = 0; i < ns; i++)
        L += a.part_ml[(base + i) * 2 + 1] * fast_exp2(a.part_ml[(base + i) * 2] - M);
    const float inv = (L > 0.f) ? 1.0f / L : 0.f;

    for (uint32_t d = threadIdx.x; d < hd; d += blockDim.x) {
        float acc = 0.f;
        for (uint32_t i = 0; i < ns; i++)
            acc += a.part_o[(base + i) * hd + d] * fast_exp2(a.part_ml[(base + i) * 2] - M);
        a.out[((size_t)sess * a.nq + head) * hd + d] = acc * inv;
    }
}

}  // namespace wr
