// Split-K decode attention (one query row per head) over the F16 cache.
//
// Computes what the reference computes with seq_q = 1
// (reference: src/core/kernels.c:1475-1523): for head qh with KV head
// kvh = qh / group, softmax over the visible keys of scale * q.k, times V.
// Summation order differs from the reference (keys are split over waves and
// workgroups and merged by log-sum-exp), so results agree to rounding, not
// bit for bit.
//
// Work decomposition: grid = (KV heads, work-list entries), one entry per
// (session, key split).  One workgroup
// owns ONE KV head of one session over a contiguous run of 32-key tiles and
// serves the whole GQA group from it, so every K and V byte is fetched from
// HBM exactly once.  Its four waves take tiles round-robin and keep private
// online-softmax state (m, l, O); they merge through LDS at the end.  A
// session with one split gets its final rows written directly; otherwise the
// workgroup publishes a partial (m, l, unnormalised O) per head, takes a
// ticket from a per-(session, KV head) counter, and the workgroup that draws
// the last ticket merges all partials and writes the rows.  One launch, no
// second pass.
//
// HBM-bound: algorithmic bytes per launch = 4 * nkv * hd * sum(seq_k)
// (K and V, two bytes each); Q, O and partials are <1 %.
//
// Inside a wave the two contractions run on the matrix cores only to take the
// arithmetic off the vector ALUs (a 4-head group would otherwise need ~100
// VALU ops per 32 bytes loaded, which caps bandwidth).  Accuracy is kept at
// F32 level by splitting each F32 operand into two half-precision terms,
// x = x_hi + x_lo, and giving the two terms their own COLUMNS of the same
// MFMA: column h carries the hi term of head h, column h + G the lo term.
// The two columns are added after the first contraction (scores) and at the
// very end of the second (outputs).  K and V are already F16, nothing is lost
// there.
//
//   S^T[key][col] = K[key][:] . Q^T[:][col]        v_mfma_f32_16x16x32_f16
//   O^T[dim][col] += Vt[dim][key] . P^T[key][col]
//
// A head is a COLUMN: lane l owns column l%16 in both accumulators, so max,
// sum and rescale of one head stay inside the lane except for one exchange
// across the four 16-lane groups and one with the partner column.
#pragma once

#include "common.hip.h"
#include "row8.hip.h"

namespace wr {

constexpr int kDecodeThreads = 256;
constexpr int kDecodeWaves = 4;
constexpr int kTileKeys = 32;
constexpr int kMaxGroupMfma = 8;      // heads per KV head the MFMA kernel serves (2G <= 16 columns)
constexpr int kBatchMax = 16;
constexpr int kFlashDMax = 1024;      // largest head_dim (reference: WR_FLASH_D_MAX)

struct DecodeSession {
    const uint16_t* k;       // K of this layer
    const uint16_t* vt;      // Vt of this layer
    uint32_t seq_k;          // valid rows
    uint32_t key_lo;         // first visible key (sliding window), else 0
    uint32_t ctx_pad;        // rows allocated per KV head (multiple of 32)
    uint32_t n_splits;       // workgroups along the key axis
    uint32_t tiles_per_wg;   // 32-key tiles per workgroup (a function of this session only)
    uint16_t tail_tiles;     // the session's last tiles that form the last split on their own (0: none)
    uint16_t parts_per_wg;   // consecutive splits one workgroup works through (1 or 2: in a launch that fills
                             // the device a short session's workgroups take two, and the last of them then
                             // runs a body split followed by the tail split)
};

struct DecodeArgs {
    DecodeSession s[kBatchMax];
    const float* q;          // [n][nq][hd]
    float* out;              // [n][nq][hd]
    float* part_o;           // [n][nq][max_splits][hd], unnormalised
    float* part_ml;          // [n][nq][max_splits][2] = (m in log2 units, l)
    uint32_t* counters;      // tickets, zero between launches: [n][nkv] (MFMA) or [n][nq] (generic)
    uint32_t nq, nkv, group, hd;
    uint32_t max_splits;
    float qscale;            // softmax scale * log2(e)
    // Work list: one entry per (session, key split) that exists, longest first;
    // entry = session << 8 | split.  The grid is (heads, entries) with the head
    // index fastest, so that with 8 KV heads each XCD (workgroups go to XCDs
    // round-robin by linear id) serves one KV head of every session and gets
    // the same share of a ragged batch.
    uint32_t n_items;
    alignas(4) uint16_t items[kBatchMax * 64];
};

// Work-list entry y.  Read as the 32-bit word that holds it: the index is the
// same for the whole workgroup, and a 32-bit read of a kernel argument is a
// scalar load, where a 16-bit one is a vector load the whole wave waits for
// before it can ask for anything else.
__device__ __forceinline__ uint32_t decode_item(const DecodeArgs& a, uint32_t y)
{
    const uint32_t w = reinterpret_cast<const uint32_t*>(a.items)[y >> 1];
    return (y & 1u) ? (w >> 16) : (w & 0xFFFFu);
}

// The decode step's new row made inside the attention launch (FUSED form of the
// MFMA kernel, head dim 128): row i of qkv is session i's stacked projection
// [nq Q heads | nkv K heads | nkv V heads]; the heads get their per-head RMSNorm
// (when the weights are given) and the rotation of the row's position, Q goes
// straight into the kernel's Q^T operand, and the workgroup whose key range
// holds the new position (seq_k - 1) truncates K and V to F16, writes them into
// the cache for later steps and puts them into its own copy of that tile, which
// was read before the row existed.  The arithmetic is qkv_append_kernel's
// (row8.hip.h), so Q, the cache and the output are the bits of the two launches
// this replaces (reference: src/core/session.c:459-496).
struct DecodeFusedArgs {
    const float* qkv;        // [n][ld]
    const float* q_norm;     // [hd] or null
    const float* k_norm;
    const float* cos_sin;    // [n][n_rot][2], or null when n_rot == 0
    uint32_t ld, n_rot;
    float eps;
    uint32_t pad_;
};

template <int HD>
struct DecodeNewRow {        // the new position's K and V as the cache holds them
    uint16_t k[HD];
    uint16_t v[HD];
};

struct TileRange {
    uint32_t t_begin, t_end;      // tiles [t_begin, t_end)
};

__device__ __forceinline__ TileRange split_tiles(const DecodeSession& S, uint32_t split)
{
    const uint32_t tiles_per_wg = S.tiles_per_wg;
    const uint32_t first = S.key_lo / kTileKeys;
    const uint32_t last = (S.seq_k + kTileKeys - 1) / kTileKeys;
    TileRange r;
    if (S.tail_tiles != 0 && split == S.n_splits - 1) {   // the tail: a split of its own
        r.t_begin = last - S.tail_tiles;
        r.t_end = last;
        return r;
    }
    r.t_begin = first + split * tiles_per_wg;
    r.t_end = min(r.t_begin + tiles_per_wg, last - S.tail_tiles);
    return r;
}

// Called by every thread of a workgroup after it has stored its partial rows
// for heads [head0, head0 + nh) of `sess` at its split index.  The workgroup
// that draws the last of the n_splits tickets merges the partials of those
// heads (log-sum-exp over the split maxima, one normalisation), writes the
// final rows and puts the counter back to zero for the next launch.
constexpr int kMaxSplits = 64;        // key splits per session (host picks tiles_per_wg to respect it)
constexpr int kMergeInRegs = 16;      // up to this many partials a merge holds in registers
static_assert(kTileKeys == kKTile, "decode tiles are the cache's K tiles");
static_assert(sizeof(DecodeArgs::items) == kBatchMax * kMaxSplits * sizeof(uint16_t), "work list size");

// Partial rows cross workgroups (and XCDs, each with its own L2) inside one
// launch.  They are written and read with agent-scope relaxed atomics: on
// gfx950 those are write-through stores / L2-coherent loads (sc1), so the data
// itself never sits dirty in one XCD's L2.  Ordering against the ticket comes
// from every thread waiting until its own stores have been acknowledged
// (s_waitcnt vmcnt(0), written out below: a workgroup-scope release fence
// compiles to no wait at all here, because the waves of a workgroup share one
// CU) and a workgroup barrier before one thread takes the ticket.  A
// device-wide release fence instead would write back the whole L2
// (buffer_wbl2) from every workgroup: measured at 5-10x the kernel's run time.
#if defined(__HIP_DEVICE_COMPILE__) && !defined(__gfx950__)
#error "the cross-workgroup exchange below relies on how gfx950 executes agent-scope relaxed atomics (sc1 write-through stores, L2-coherent loads); it has not been argued for any other target"
#endif
__device__ __forceinline__ float part_load(const float* p)
{
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void part_store(float* p, float v)
{
    __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Merge of up to N partials per head, everything a thread needs asked for at
// once: its output element's partial values and the head's (m, l) pairs; the
// thread works the weights out for itself.  One trip to memory instead of two
// dependent ones, at the end of the launch where nothing hides them.  (Slots
// past n_splits re-read partial 0 with weight zero; which N serves a session
// depends on its split count alone.)
template <int N>
__device__ __forceinline__ void merge_in_regs(const DecodeArgs& a, uint32_t sess, uint32_t head0,
                                              uint32_t nh, uint32_t n_splits)
{
    const uint32_t hd = a.hd;
    for (uint32_t idx = threadIdx.x; idx < nh * hd; idx += blockDim.x) {
        const uint32_t h = idx / hd, d = idx % hd;
        const size_t p0 = ((size_t)sess * a.nq + head0 + h) * a.max_splits;
        float v[N], m[N], l[N];
#pragma unroll
        for (uint32_t i = 0; i < (uint32_t)N; i++) {
            const uint32_t ii = i < n_splits ? i : 0;
            v[i] = part_load(a.part_o + (p0 + ii) * hd + d);
            m[i] = part_load(&a.part_ml[(p0 + ii) * 2]);
            l[i] = part_load(&a.part_ml[(p0 + ii) * 2 + 1]);
        }
        float M = -INFINITY;
#pragma unroll
        for (uint32_t i = 0; i < (uint32_t)N; i++)
            if (i < n_splits) M = fmaxf(M, m[i]);
        float L = 0.f;
#pragma unroll
        for (uint32_t i = 0; i < (uint32_t)N; i++) {
            m[i] = (i < n_splits) ? fast_exp2(m[i] - M) : 0.f;
            L += l[i] * m[i];
        }
        const float inv = (L > 0.f) ? 1.0f / L : 0.f;
        float acc[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (uint32_t i = 0; i < (uint32_t)N; i++) acc[i & 3] += v[i] * (m[i] * inv);
        a.out[((size_t)sess * a.nq + head0 + h) * hd + d] = (acc[0] + acc[1]) + (acc[2] + acc[3]);
    }
}

// Called by every thread of a workgroup after it has stored its partial rows
// for heads [head0, head0 + nh) of `sess` at its split indices.  The workgroup
// that draws the last of the n_wgs tickets (the workgroups that share the
// session's n_splits partials between them) merges the partials of those
// heads (log-sum-exp over the split maxima, one normalisation), writes the
// final rows and puts the counter back to zero for the next launch.
// `scratch` is LDS the caller no longer needs: 3 * nh * kMaxSplits floats.
__device__ __forceinline__ void publish_and_merge(const DecodeArgs& a, uint32_t sess,
                                                  uint32_t head0, uint32_t nh, uint32_t n_splits,
                                                  uint32_t n_wgs, uint32_t counter_idx, float* scratch)
{
    __shared__ uint32_t s_ticket;
    // own partial stores acknowledged: the ticket below must not be drawn while
    // one of them is still on its way (the workgroup that merges would read
    // what the address held before)
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (threadIdx.x == 0)
        s_ticket = __hip_atomic_fetch_add(&a.counters[counter_idx], 1u, __ATOMIC_RELAXED,
                                          __HIP_MEMORY_SCOPE_AGENT);
    __syncthreads();
    if (s_ticket != n_wgs - 1) return;
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");

    const uint32_t hd = a.hd;
    if (n_splits <= kMergeInRegs) {
        if (n_splits <= 4)
            merge_in_regs<4>(a, sess, head0, nh, n_splits);
        else if (n_splits <= 8)
            merge_in_regs<8>(a, sess, head0, nh, n_splits);
        else if (n_splits <= 12)
            merge_in_regs<12>(a, sess, head0, nh, n_splits);
        else
            merge_in_regs<kMergeInRegs>(a, sess, head0, nh, n_splits);
        if (threadIdx.x == 0) a.counters[counter_idx] = 0;
        return;
    }

    float* s_m = scratch;                       // [nh][kMaxSplits]
    float* s_l = scratch + nh * kMaxSplits;
    float* s_w = scratch + 2 * nh * kMaxSplits;
    for (uint32_t idx = threadIdx.x; idx < nh * n_splits; idx += blockDim.x) {
        const uint32_t h = idx / n_splits, i = idx % n_splits;
        const size_t pi = ((size_t)sess * a.nq + head0 + h) * a.max_splits + i;
        s_m[h * kMaxSplits + i] = part_load(&a.part_ml[pi * 2]);
        s_l[h * kMaxSplits + i] = part_load(&a.part_ml[pi * 2 + 1]);
    }
    __syncthreads();
    if (threadIdx.x < nh) {
        const uint32_t h = threadIdx.x;
        float M = -INFINITY;
        for (uint32_t i = 0; i < n_splits; i++) M = fmaxf(M, s_m[h * kMaxSplits + i]);
        float L = 0.f;
        for (uint32_t i = 0; i < n_splits; i++) {
            const float f = fast_exp2(s_m[h * kMaxSplits + i] - M);
            s_w[h * kMaxSplits + i] = f;
            L += s_l[h * kMaxSplits + i] * f;
        }
        const float inv = (L > 0.f) ? 1.0f / L : 0.f;
        for (uint32_t i = 0; i < n_splits; i++) s_w[h * kMaxSplits + i] *= inv;
    }
    __syncthreads();

    for (uint32_t idx = threadIdx.x; idx < nh * hd; idx += blockDim.x) {
        const uint32_t h = idx / hd, d = idx % hd;
        const float* po = a.part_o + (((size_t)sess * a.nq + head0 + h) * a.max_splits) * hd + d;
        const float* w = s_w + h * kMaxSplits;
        float acc0 = 0.f, acc1 = 0.f, acc2 = 0.f, acc3 = 0.f;
        uint32_t i = 0;
        for (; i + 4 <= n_splits; i += 4) {
            const float v0 = part_load(po + (size_t)(i + 0) * hd);
            const float v1 = part_load(po + (size_t)(i + 1) * hd);
            const float v2 = part_load(po + (size_t)(i + 2) * hd);
            const float v3 = part_load(po + (size_t)(i + 3) * hd);
            acc0 += v0 * w[i + 0];
            acc1 += v1 * w[i + 1];
            acc2 += v2 * w[i + 2];
            acc3 += v3 * w[i + 3];
        }
        for (; i < n_splits; i++) acc0 += part_load(po + (size_t)i * hd) * w[i];
        a.out[((size_t)sess * a.nq + head0 + h) * hd + d] = (acc0 + acc1) + (acc2 + acc3);
    }
    if (threadIdx.x == 0) a.counters[counter_idx] = 0;
}

// A query element scaled and split into the two half-precision terms the first
// contraction takes (x = hi + lo).  One place, with contraction of the product
// into the subtraction switched off: the kernel that makes the new row itself
// and the one that is handed finished Q rows must produce the same bits, and
// left to itself the compiler fuses "v * qscale - hi" in one and not the other.
__device__ __forceinline__ void q_hi_lo(float v, float qscale, _Float16& hi, _Float16& lo)
{
#pragma clang fp contract(off)
    const float x = v * qscale;
    hi = (_Float16)x;
    lo = (_Float16)(x - (float)hi);
}

// ------------------------------------------------------------------ MFMA --

template <int HD>
struct DecodeFrag {
    half8 k[2][HD / 32];     // two 16-key sub-tiles x (HD/32) contraction steps
    half8 v[HD / 16];        // HD/16 dimension tiles x 32 keys
};

// The cache is read exactly once per launch: non-temporal loads keep it from
// displacing anything useful in the caches.
__device__ __forceinline__ half8 stream_load(const half8* p) { return __builtin_nontemporal_load(p); }

template <int HD>
__device__ __forceinline__ void load_frag_k(DecodeFrag<HD>& f, const uint16_t* __restrict__ kbase,
                                            uint32_t tile, int lane)
{
    // Half t of the tile feeds sub-tile t: MFMA row m is slot m of the half, and
    // lane group g reads chunk 4s + g of it for contraction step s.  In the
    // cache's K layout that is one contiguous KiB per load.  Slot m of half t is
    // position 8*(m/4) + 4t + m%4 of the tile, so the accumulator of lane group
    // g ends up holding keys 8g .. 8g+7 in order: exactly the eight consecutive
    // positions that group reads from Vt.
    const half8* base = reinterpret_cast<const half8*>(kbase + (size_t)tile * kTileKeys * HD) + lane;
#pragma unroll
    for (int t = 0; t < 2; t++) {
#pragma unroll
        for (int s = 0; s < HD / 32; s++)
            f.k[t][s] = stream_load(&base[(t * (HD / 8) + s * 4) * 16]);
    }
}

template <int HD>
__device__ __forceinline__ void load_frag_v(DecodeFrag<HD>& f, const uint16_t* __restrict__ vtbase,
                                            uint32_t tile, int lane)
{
    const int m = lane & 15, g = lane >> 4;
    const half8* vb = reinterpret_cast<const half8*>(vtbase + (size_t)tile * HD * kVBlock);
#pragma unroll
    for (int dt = 0; dt < HD / 16; dt++) f.v[dt] = stream_load(&vb[(dt * 16 + m) * 4 + g]);
}

template <int HD>
__device__ __forceinline__ void load_frag(DecodeFrag<HD>& f, const uint16_t* __restrict__ kbase,
                                          const uint16_t* __restrict__ vtbase, uint32_t tile,
                                          int lane)
{
    load_frag_k<HD>(f, kbase, tile, lane);
    load_frag_v<HD>(f, vtbase, tile, lane);
}

template <int HD>
struct DecodeState {
    f32x4 o[HD / 16];        // O^T: dim = dt*16 + 4g + r, column = lane%16
    float m;                 // running max (log2 units), common to the 4 groups
    float l;                 // this lane group's share of the denominator
};

// Scores of one tile, S^T[key][column], before the hi and lo columns are added.
template <int HD>
__device__ __forceinline__ void tile_scores(f32x4 (&c)[2], const DecodeFrag<HD>& f,
                                            const half8 (&qop)[HD / 32])
{
#pragma unroll
    for (int t = 0; t < 2; t++) {
        c[t] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int s = 0; s < HD / 32; s++)
            c[t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(f.k[t][s], qop[s], c[t], 0, 0, 0);
    }
}

// Same, with the Q^T operand read from LDS row by row instead of being held in
// registers (the 256-wide head has no registers to spare for it).
template <int HD>
__device__ __forceinline__ void tile_scores_lds(f32x4 (&c)[2], const DecodeFrag<HD>& f,
                                                const _Float16* __restrict__ qrow)
{
    c[0] = f32x4{0.f, 0.f, 0.f, 0.f};
    c[1] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int s = 0; s < HD / 32; s++) {
        const half8 qs = *reinterpret_cast<const half8*>(qrow + s * 32);
        c[0] = __builtin_amdgcn_mfma_f32_16x16x32_f16(f.k[0][s], qs, c[0], 0, 0, 0);
        c[1] = __builtin_amdgcn_mfma_f32_16x16x32_f16(f.k[1][s], qs, c[1], 0, 0, 0);
    }
}

// Online-softmax update of one tile from its raw scores, and the P.V product.
// col_kind: 0 = hi column of a head, 1 = lo column, 2 = unused column.
template <int HD>
__device__ __forceinline__ void tile_update(DecodeState<HD>& st, DecodeFrag<HD>& f,
                                            const f32x4 (&c)[2], uint32_t tile, uint32_t key_lo,
                                            uint32_t seq_k, int lane, int partner_addr,
                                            int col_kind)
{
    const int g = lane >> 4;
    const uint32_t kb = tile * kTileKeys;

    // score = hi column + lo column; both columns of a head end up with the sum
    float sc[8];
#pragma unroll
    for (int j = 0; j < 8; j++) {
        const float own = c[j >> 2][j & 3];
        const float other = __int_as_float(
            __builtin_amdgcn_ds_bpermute(partner_addr, __float_as_int(own)));
        sc[j] = (col_kind == 2) ? own : own + other;
    }

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

    half8 pop;
    float psum = 0.f;
#pragma unroll
    for (int j = 0; j < 8; j++) {
        const float p = fast_exp2(sc[j] - m_new);
        psum += p;
        const _Float16 h = (_Float16)p;
        const _Float16 lo = (_Float16)(p - (float)h);
        pop[j] = (col_kind == 0) ? h : ((col_kind == 1) ? lo : (_Float16)0.0f);
    }
    st.l = st.l * alpha + psum;

#pragma unroll
    for (int dt = 0; dt < HD / 16; dt++) {
        st.o[dt] *= alpha;
        st.o[dt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(f.v[dt], pop, st.o[dt], 0, 0, 0);
    }
}

// Position p (0..31) of a tile held in registers replaced by the new row: its K
// row is slot k_tile_slot(p) of half k_tile_half(p) (the lanes 16 g + slot hold
// its chunks 4 s + g), its V values are element p % 8 of the lanes of group p / 8.
template <int HD>
__device__ __forceinline__ void patch_new_row(DecodeFrag<HD>& f, const DecodeNewRow<HD>& nr, uint32_t p,
                                              int lane)
{
    const uint32_t m = lane & 15, g = lane >> 4;
    if (m == k_tile_slot(p)) {
        const bool upper = k_tile_half(p) != 0;
#pragma unroll
        for (int s = 0; s < HD / 32; s++) {
            const half8 kv = *reinterpret_cast<const half8*>(&nr.k[(4 * s + g) * 8]);
            if (upper)
                f.k[1][s] = kv;
            else
                f.k[0][s] = kv;
        }
    }
    if (g == (p >> 3)) {
        // element p % 8 of eight halves = one half of 32-bit word (p % 8) / 2: a
        // bit-field insert per word and a select on the word index, not a chain
        // of selects per half (this runs once per launch, in one wave, with the
        // rest of the workgroup waiting for that wave's tile: its length in
        // instructions is what it costs)
        const uint32_t e = p & 7, w = e >> 1;
        const uint32_t keep = (e & 1) ? 0x0000FFFFu : 0xFFFF0000u;
#pragma unroll
        for (int dt = 0; dt < HD / 16; dt++) {
            const uint32_t both = (uint32_t)nr.v[dt * 16 + m] * 0x10001u;
            u32x4 words = __builtin_bit_cast(u32x4, f.v[dt]);
#pragma unroll
            for (int wi = 0; wi < 4; wi++) {
                const uint32_t nw = (words[wi] & keep) | (both & ~keep);
                words[wi] = ((uint32_t)wi == w) ? nw : words[wi];
            }
            f.v[dt] = __builtin_bit_cast(half8, words);
        }
    }
}

template <int HD>
__device__ __forceinline__ void process_tile(DecodeState<HD>& st, DecodeFrag<HD>& f,
                                             const half8 (&qop)[HD / 32], uint32_t tile,
                                             uint32_t key_lo, uint32_t seq_k, int lane,
                                             int partner_addr, int col_kind,
                                             const DecodeNewRow<HD>* nr = nullptr, uint32_t patch_tile = 0xFFFFFFFFu)
{
    if (nr != nullptr && tile == patch_tile) patch_new_row<HD>(f, *nr, (seq_k - 1) % kTileKeys, lane);
    f32x4 c[2];
    tile_scores<HD>(c, f, qop);
    tile_update<HD>(st, f, c, tile, key_lo, seq_k, lane, partner_addr, col_kind);
}

// Head dims 128 and 256 keep ONE tile per wave in registers and ask for the next
// tile's K as soon as the scores are out and for its V as soon as P.V is done;
// the other waves of the SIMD compute while those loads are in flight.  At 256
// a tile is 128 registers and two waves share a SIMD (double buffering it with
// one wave per SIMD and 512 registers spilled addresses, and a spill reload
// waits for every load in flight).  At 128 the single tile makes room for three
// workgroups per CU (142 registers) where two tiles per wave allowed two (218):
// measured against the double-buffered form, 16 x 4096 keys 44.7 -> 44.4 us, the
// ragged batch of 16 34.7 -> 33.7, one session of 2048 keys 8.5 -> 7.9 and of
// 8192 keys 15.3 -> 14.7, the fused decode launch at ~520 keys 10.4 -> 8.9 (four
// workgroups per CU spill: 46 us at 16 x 4096).  The arithmetic of a wave is the
// same in both forms (same tiles, same order, same chains).  Head dim 64 holds
// two tiles per wave at 126 registers.
template <int HD>
constexpr bool decode_single_buffered() { return HD >= 128; }
template <int HD>
constexpr int decode_wgs_per_cu() { return HD >= 256 ? 2 : 3; }

template <int HD, bool FUSED = false>
__global__ __launch_bounds__(kDecodeThreads, decode_wgs_per_cu<HD>())
void decode_mfma_kernel(const DecodeArgs a, const DecodeFusedArgs fz)
{
    static_assert(!FUSED || HD == 128, "the fused form is built for head dim 128");
    const uint32_t kvh = blockIdx.x;
    const uint32_t item = decode_item(a, blockIdx.y);
    // Kernel arguments are read through the scalar cache, which starts every
    // launch empty: each read of a line not yet seen is a trip to memory, and
    // left to the compiler there were four of them in a row before the first
    // tile could be asked for (the entry; the session's sizes; the launch's
    // scalars; the session's pointers: 2 us).  Two are needed: the entry together
    // with the line that holds the launch's scalars (and the one with the new
    // row's arguments), then the whole session record at once.  The empty asm
    // statements pin where the values must have arrived.
    const float* args_line = a.q;
    const float* fused_line = FUSED ? fz.qkv : nullptr;
    asm volatile("" ::"s"(item), "s"(args_line), "s"(fused_line));
    const uint32_t sess = item >> 8, split = item & 0xFFu;
    const DecodeSession S = a.s[sess];
    if constexpr (!FUSED)
        asm volatile("" ::"s"(S.k), "s"(S.vt), "s"(S.seq_k), "s"(S.key_lo), "s"(S.ctx_pad), "s"(S.n_splits),
                     "s"(S.tiles_per_wg), "s"((uint32_t)S.tail_tiles), "s"((uint32_t)S.parts_per_wg));

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int n = lane & 15, g = lane >> 4;
    const int G = (int)a.group;
    // The splits this workgroup works through, one after the other: [sp0, sp1).
    // A split is the unit of arithmetic (one partial) and a function of the
    // session alone; how many consecutive ones a workgroup takes is the host's
    // choice per launch and changes no bit.
    const uint32_t ppw = S.parts_per_wg;
    const uint32_t sp0 = split * ppw, sp1 = min(sp0 + ppw, S.n_splits);
    TileRange tr = split_tiles(S, sp0);
    const TileRange tr_last = split_tiles(S, sp1 - 1);

    const uint16_t* kbase = S.k + (size_t)kvh * S.ctx_pad * HD;
    const uint16_t* vtbase = S.vt + (size_t)kvh * (S.ctx_pad / kVBlock) * HD * kVBlock;

    // Loads go out in the order they are needed back: the group's Q rows (a few
    // KB), then this wave's first tile, then (where a wave holds two tiles) its
    // second.  Memory channels serve requests roughly in arrival order and every
    // workgroup of the launch starts at once, so a Q request issued after the
    // tiles waits behind the whole launch's first tiles (5 us at 16 x 4096), and
    // no workgroup can ask for a second tile until then: the queue runs dry once.
    constexpr bool kSingle = decode_single_buffered<HD>();
    constexpr int kQPerThread = kMaxGroupMfma * HD / kDecodeThreads;
    constexpr int kNJ = FUSED ? HD / 64 : 1;
    float qreg[kQPerThread];
    float xrow[kNJ][8];                                   // FUSED: this lane's share of one head of the new row
    // FUSED: the new position's tile, whether this workgroup's range holds it,
    // and the wave that has it (its last tile)
    const uint32_t new_pos = S.seq_k - 1, new_tile = new_pos / kTileKeys;
    const bool owner = FUSED && new_tile >= tr.t_begin && new_tile < tr_last.t_end;
    const uint32_t patch_tile =
        (owner && (new_tile - tr_last.t_begin) % kDecodeWaves == (uint32_t)wave) ? new_tile : 0xFFFFFFFFu;
    const uint32_t hslot = threadIdx.x >> 3, part = threadIdx.x & 7;   // FUSED: head slot (Q heads, K, V), lane of eight
    // FUSED: the new row's values are asked for here, before the tiles, and worked
    // out after the tiles have been asked for: a wave's loads return in the order
    // they were issued.  Lanes of eight without a head shadow head slot 0, so that
    // every load is unconditional and the waits below stay exact.
    Row8Loads<kNJ> rl;
    // Head slots: the group's Q heads in wave 0 (slots 0 .. G-1), the K head in wave
    // 1 (slot 8), the V head in wave 2 (slot 16): three waves work on them side by
    // side, where one wave would run the three branches one after the other (and
    // fetch their code one after the other) with the workgroup waiting at the
    // barrier behind it.
    constexpr uint32_t kSlotK = 8, kSlotV = 16;
    static_assert(kMaxGroupMfma <= (int)kSlotK, "Q heads fit before the K slot");
    const bool slot_q = hslot < (uint32_t)G, slot_k = owner && hslot == kSlotK, slot_v = owner && hslot == kSlotV;
    const uint32_t hs = (slot_q || slot_k || slot_v) ? hslot : 0u;
    if constexpr (FUSED) {
        const bool is_q = hs < (uint32_t)G, is_k = hs == kSlotK;
        const uint32_t head = is_q ? kvh * G + hs : (is_k ? a.nq + kvh : a.nq + a.nkv + kvh);
        const float* src = fz.qkv + (size_t)sess * fz.ld + (size_t)head * HD + part * 8;
        // (a V head reads the Q norm's weights and the table and uses neither)
        row8_head_request<kNJ>(rl, src, is_k ? fz.k_norm : fz.q_norm, part,
                               fz.cos_sin ? fz.cos_sin + (size_t)sess * fz.n_rot * 2 : nullptr, fz.n_rot);
    } else {
        const float* qg = a.q + ((size_t)sess * a.nq + kvh * G) * HD;     // G contiguous rows
#pragma unroll
        for (int i = 0; i < kQPerThread; i++) {
            const int idx = threadIdx.x + i * kDecodeThreads;
            qreg[i] = (idx < G * HD) ? qg[idx] : 0.f;
        }
    }
    // Both loads are unconditional (a wave with fewer tiles re-reads the
    // workgroup's last one and ignores it): the compiler places its waits by
    // counting the loads issued since the one it needs, and a load that is only
    // sometimes issued makes it assume the smaller count everywhere downstream,
    // which turns "wait for this tile" into "wait for the prefetched tile too".
    DecodeFrag<HD> fa, fb;
    uint32_t t = tr.t_begin + wave;
    load_frag<HD>(fa, kbase, vtbase, min(t, tr.t_end - 1), lane);
    if constexpr (!kSingle) load_frag<HD>(fb, kbase, vtbase, min(t + kDecodeWaves, tr.t_end - 1), lane);
    if constexpr (FUSED)
        row8_head_finish<kNJ>(xrow, rl, fz.q_norm != nullptr && hs != kSlotV, false, fz.eps, part,
                              fz.cos_sin != nullptr && hs != kSlotV, fz.n_rot);

    // Q^T operand through LDS: row c of lds_q is MFMA column c.  Columns
    // 0..G-1 hold the hi terms of the group's heads, G..2G-1 the lo terms,
    // the rest zero; values are pre-multiplied by scale*log2(e).
    __shared__ __attribute__((aligned(16))) _Float16 lds_q[16][HD + 8];
    __shared__ __attribute__((aligned(16))) DecodeNewRow<FUSED ? HD : 8> new_row;
    if constexpr (FUSED) {
        if (hslot < (uint32_t)G) {
            // a Q head: element 64 c + 8 part + e of MFMA columns hslot (hi) and hslot + G (lo)
            // (element by element: written as two 16-byte vectors the conversions
            // become packed ones, which round a lo term in the subnormal range of
            // binary16 differently from the scalar conversion of the kernel that is
            // handed finished Q rows -- and the two must agree bit for bit)
#pragma unroll
            for (int c = 0; c < kNJ; c++)
#pragma unroll
                for (int e = 0; e < 8; e++) {
                    const int d = c * 64 + (int)part * 8 + e;
                    _Float16 hi, lo;
                    q_hi_lo(xrow[c][e], a.qscale, hi, lo);
                    lds_q[hslot][d] = hi;
                    lds_q[hslot + G][d] = lo;
                }
        } else if (slot_k) {
            // the K head: truncated to F16, into the cache and into the workgroup's copy
            uint16_t* kw = const_cast<uint16_t*>(S.k);
#pragma unroll
            for (int c = 0; c < kNJ; c++) {
                uint32_t w[4];
#pragma unroll
                for (int e = 0; e < 4; e++)
                    w[e] = (uint32_t)f32_to_f16_trunc(xrow[c][2 * e]) |
                           ((uint32_t)f32_to_f16_trunc(xrow[c][2 * e + 1]) << 16);
                const u32x4 packed = u32x4{w[0], w[1], w[2], w[3]};
                *reinterpret_cast<u32x4*>(kw + k_offset(kvh, S.ctx_pad, new_pos, c * 64 + part * 8, HD)) = packed;
                *reinterpret_cast<u32x4*>(&new_row.k[c * 64 + part * 8]) = packed;
            }
        } else if (slot_v) {
            // the V head: truncated, into the block-transposed Vt and the workgroup's copy
            uint16_t* vw = const_cast<uint16_t*>(S.vt);
#pragma unroll
            for (int c = 0; c < kNJ; c++)
#pragma unroll
                for (int e = 0; e < 8; e++) {
                    const uint32_t d = c * 64 + part * 8 + e;
                    const uint16_t bits = f32_to_f16_trunc(xrow[c][e]);
                    vw[vt_offset(kvh, S.ctx_pad, new_pos, d, HD)] = bits;
                    new_row.v[d] = bits;
                }
        }
        for (int idx = threadIdx.x; idx < (16 - 2 * G) * HD; idx += kDecodeThreads)
            lds_q[2 * G + idx / HD][idx % HD] = (_Float16)0.0f;
    } else {
#pragma unroll
        for (int i = 0; i < kQPerThread; i++) {
            const int idx = threadIdx.x + i * kDecodeThreads;
            if (idx < G * HD) {
                const int h = idx / HD, d = idx % HD;
                _Float16 hi, lo;
                q_hi_lo(qreg[i], a.qscale, hi, lo);
                lds_q[h][d] = hi;
                lds_q[h + G][d] = lo;
            }
        }
        for (int idx = threadIdx.x; idx < (16 - 2 * G) * HD; idx += kDecodeThreads)
            lds_q[2 * G + idx / HD][idx % HD] = (_Float16)0.0f;
    }
    __syncthreads();
    const DecodeNewRow<HD>* nrp = nullptr;
    if constexpr (FUSED) nrp = reinterpret_cast<const DecodeNewRow<HD>*>(&new_row);
    half8 qop[kSingle ? 1 : HD / 32];
    if constexpr (!kSingle) {
#pragma unroll
        for (int s = 0; s < HD / 32; s++)
            qop[s] = *reinterpret_cast<const half8*>(&lds_q[n][s * 32 + g * 8]);
    }

    const int col_kind = (n < G) ? 0 : ((n < 2 * G) ? 1 : 2);
    const int partner = (n < G) ? lane + G : ((n < 2 * G) ? lane - G : lane);
    const int partner_addr = partner * 4;

    __shared__ float lds_o[kDecodeWaves][kMaxGroupMfma][HD];
    __shared__ float lds_m[kDecodeWaves][kMaxGroupMfma];
    __shared__ float lds_l[kDecodeWaves][kMaxGroupMfma];
    const bool direct = (S.n_splits == 1);
    for (uint32_t sp = sp0;;) {
        DecodeState<HD> st;
#pragma unroll
        for (int dt = 0; dt < HD / 16; dt++) st.o[dt] = f32x4{0.f, 0.f, 0.f, 0.f};
        st.m = -INFINITY;
        st.l = 0.f;

        // Loads inside the loops below are unconditional too, and the last tiles
        // are peeled off, for the same reason.
        if constexpr (kSingle) {
            const _Float16* qrow = &lds_q[n][g * 8];
            if (t < tr.t_end) {
                f32x4 c[2];
                while (t + kDecodeWaves < tr.t_end) {
                    // keeps the Q^T reads inside the loop: hoisted, they would cost
                    // the registers this path does not have
                    asm volatile("" ::: "memory");
                    tile_scores_lds<HD>(c, fa, qrow);
                    load_frag_k<HD>(fa, kbase, t + kDecodeWaves, lane);
                    tile_update<HD>(st, fa, c, t, S.key_lo, S.seq_k, lane, partner_addr, col_kind);
                    load_frag_v<HD>(fa, vtbase, t + kDecodeWaves, lane);
                    t += kDecodeWaves;
                }
                // (the new position's tile is the last of its wave)
                if (nrp != nullptr && t == patch_tile) patch_new_row<HD>(fa, *nrp, (S.seq_k - 1) % kTileKeys, lane);
                tile_scores_lds<HD>(c, fa, qrow);
                tile_update<HD>(st, fa, c, t, S.key_lo, S.seq_k, lane, partner_addr, col_kind);
            }
        } else if (t < tr.t_end) {
            // fa holds tile t, fb tile t + W (both asked for above); each tile's
            // buffer is refilled with the tile two rounds on as soon as it is used
            while (t + 3 * kDecodeWaves < tr.t_end) {
                process_tile<HD>(st, fa, qop, t, S.key_lo, S.seq_k, lane, partner_addr, col_kind, nrp, patch_tile);
                load_frag<HD>(fa, kbase, vtbase, t + 2 * kDecodeWaves, lane);
                process_tile<HD>(st, fb, qop, t + kDecodeWaves, S.key_lo, S.seq_k, lane, partner_addr,
                                 col_kind, nrp, patch_tile);
                load_frag<HD>(fb, kbase, vtbase, t + 3 * kDecodeWaves, lane);
                t += 2 * kDecodeWaves;
            }
            // one, two or three tiles left; the first two are in flight
            process_tile<HD>(st, fa, qop, t, S.key_lo, S.seq_k, lane, partner_addr, col_kind, nrp, patch_tile);
            if (t + 2 * kDecodeWaves < tr.t_end) {
                load_frag<HD>(fa, kbase, vtbase, t + 2 * kDecodeWaves, lane);
                process_tile<HD>(st, fb, qop, t + kDecodeWaves, S.key_lo, S.seq_k, lane, partner_addr,
                                 col_kind, nrp, patch_tile);
                process_tile<HD>(st, fa, qop, t + 2 * kDecodeWaves, S.key_lo, S.seq_k, lane, partner_addr,
                                 col_kind, nrp, patch_tile);
            } else if (t + kDecodeWaves < tr.t_end) {
                process_tile<HD>(st, fb, qop, t + kDecodeWaves, S.key_lo, S.seq_k, lane, partner_addr,
                                 col_kind, nrp, patch_tile);
            }
        }
        // the next split's first tiles travel while this one's waves are merged
        // (not at head_dim 256: that shape has no register to spare for a loop
        // around its tile loop, and the host never gives it two splits)
        const bool more = HD < 256 && sp + 1 < sp1;
        TileRange tr_next = tr;
        if (more) {
            tr_next = split_tiles(S, sp + 1);
            t = tr_next.t_begin + wave;
            load_frag<HD>(fa, kbase, vtbase, min(t, tr_next.t_end - 1), lane);
            if constexpr (!kSingle) load_frag<HD>(fb, kbase, vtbase, min(t + kDecodeWaves, tr_next.t_end - 1), lane);
        }
        // denominator: add the four lane groups' shares
        st.l += wave_xor_f32(st.l, 16);
        st.l += wave_xor_f32(st.l, 32);
        // outputs: hi column + lo column
#pragma unroll
        for (int dt = 0; dt < HD / 16; dt++)
#pragma unroll
            for (int r = 0; r < 4; r++)
                st.o[dt][r] += __int_as_float(
                    __builtin_amdgcn_ds_bpermute(partner_addr, __float_as_int(st.o[dt][r])));

        if (n < G) {
#pragma unroll
            for (int dt = 0; dt < HD / 16; dt++)
#pragma unroll
                for (int r = 0; r < 4; r++) lds_o[wave][n][dt * 16 + 4 * g + r] = st.o[dt][r];
            if (g == 0) {
                lds_m[wave][n] = st.m;
                lds_l[wave][n] = st.l;
            }
        }
        lds_barrier();            // LDS only: the next split's tiles stay in flight

        for (uint32_t idx = threadIdx.x; idx < (uint32_t)G * HD; idx += kDecodeThreads) {
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
            if (direct) {
                a.out[((size_t)sess * a.nq + head) * HD + d] = (L > 0.f) ? acc / L : 0.f;
            } else {
                const size_t pi = ((size_t)sess * a.nq + head) * a.max_splits + sp;
                part_store(&a.part_o[pi * HD + d], acc);
                if (d == 0) {
                    part_store(&a.part_ml[pi * 2 + 0], M);
                    part_store(&a.part_ml[pi * 2 + 1], L);
                }
            }
        }
        if (!more) break;
        // lds_o, lds_m, lds_l are written again by the next split.  (This barrier
        // also waits for the partial stores above and for the tile asked for:
        // with stores still pending the compiler could no longer count on loads
        // returning in order, and every wait of the tile loop would become a
        // wait for everything.)
        __syncthreads();
        tr = tr_next;
        sp++;
    }
    if (!direct) {
        __syncthreads();      // lds_o is reused as merge scratch
        publish_and_merge(a, sess, kvh * G, G, S.n_splits, (S.n_splits + ppw - 1) / ppw, sess * a.nkv + kvh,
                          &lds_o[0][0][0]);
    }
}

// --------------------------------------------------------------- generic --
// Any head_dim up to 1024 and any group size: one workgroup per (split, query
// head, session), vector ALU only.  Slow; exists so every shape the reference
// accepts has a device path, and as a second implementation to cross-check
// the MFMA kernel against.

constexpr int kGenericMaxPerLane = 16;      // 1024 / 64

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
        float dot = 0.f;
#pragma unroll
        for (int i = 0; i < kGenericMaxPerLane; i++) {
            const uint32_t d = lane + 64 * i;
            if (d < hd)
                dot += qv[i] * (float)(*reinterpret_cast<const _Float16*>(
                                   k + k_offset(kvh, ctx_pad, key, d, hd)));
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
    const uint32_t head = blockIdx.x;
    const uint32_t item = decode_item(a, blockIdx.y);
    const uint32_t sess = item >> 8, split = item & 0xFFu;
    const DecodeSession S = a.s[sess];
    const uint32_t hd = a.hd;
    const uint32_t kvh = head / a.group;
    const TileRange tr = split_tiles(S, split);
    const uint32_t key_begin = max(tr.t_begin * kTileKeys, S.key_lo);
    const uint32_t key_end = min(tr.t_end * kTileKeys, S.seq_k);

    __shared__ GenericShared sh;
    generic_attend_wg(sh, S.k, S.vt, S.ctx_pad, kvh, hd, key_begin, key_end,
                      a.q + ((size_t)sess * a.nq + head) * hd, a.qscale);
    const GenericMerge g = merge_generic(sh);

    const bool direct = (S.n_splits == 1);
    for (uint32_t d = threadIdx.x; d < hd; d += kDecodeThreads) {
        float acc = 0.f;
#pragma unroll
        for (int w = 0; w < kDecodeWaves; w++) acc += sh.o[w][d] * g.fct[w];
        if (direct) {
            a.out[((size_t)sess * a.nq + head) * hd + d] = (g.L > 0.f) ? acc / g.L : 0.f;
        } else {
            const size_t pi = ((size_t)sess * a.nq + head) * a.max_splits + split;
            part_store(&a.part_o[pi * hd + d], acc);
            if (d == 0) {
                part_store(&a.part_ml[pi * 2 + 0], g.M);
                part_store(&a.part_ml[pi * 2 + 1], g.L);
            }
        }
    }
    if (!direct) {
        __syncthreads();      // sh.o is reused as merge scratch
        publish_and_merge(a, sess, head, 1, S.n_splits, S.n_splits, sess * a.nq + head, &sh.o[0][0]);
    }
}

}  // namespace wr
