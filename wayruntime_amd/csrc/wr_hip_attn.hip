// C ABI of the MI355X attention path: device state, cache slabs, argument
// checking and kernel launches.  Declarations and the reference interfaces
// each entry point stands in for are in include/wr_hip_attn.h.
//
// There is no CPU path in this file: without a gfx950 device init fails and
// every other entry point returns WR_HIP_ERR_STATE.

#include <hip/hip_runtime.h>
#include <hip/hip_ext.h>

#include <algorithm>
#include <atomic>
#include <cmath>
#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <mutex>
#include <new>
#include <vector>

#include "../../include/wr_hip_attn.h"
#include "common.hip.h"
#include "kernels_append.hip.h"
#include "kernels_decode.hip.h"
#include "kernels_prefill.hip.h"
#include "kernels_prefill_il.hip.h"
#include "kernels_prefill_pair.hip.h"
#include "kernels_prefill_ild.hip.h"
#include "kernels_proj.hip.h"
#include "kernels_rows.hip.h"

using namespace wr;

// Scratch of wr_hip_attn_decode_batched_dev_noalloc, the one entry point that
// allocates nothing: the split-K tickets (first kNoAllocTicketBytes) and the
// partial rows (the rest).  Every device the library runs on holds its own copy
// until the process ends.  In host code the array's name is only a stand-in: the
// device address is asked for once per device at init (hipGetSymbolAddress) and
// kept in Lib::noalloc_ws; host code uses that pointer, never the name.
constexpr size_t kNoAllocTicketBytes = 64u * 1024u;            // 16 sessions x 1024 heads
constexpr size_t kNoAllocScratchBytes = 20u * 1024u * 1024u;   // tickets + partials
constexpr uint32_t kNoAllocMaxHeads = (uint32_t)(kNoAllocTicketBytes / sizeof(uint32_t) / WR_HIP_BATCH_MAX);
constexpr int kMaxDevices = 16;
static __device__ __align__(256) unsigned char scratch[kNoAllocScratchBytes];

// Clears n 32-bit words (tickets).  A kernel rather than a memset call so that a
// caller may record the launch into a graph.
__global__ void fill_u32_kernel(uint32_t* p, uint32_t n, uint32_t v)
{
    const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = v;
}

struct wr_hip_weight {
    uint32_t n_out, n_in;
    void* tiles;                 // F16, tile order (kernels_proj.hip.h)
    size_t bytes;
};

struct wr_hip_kv {
    uint32_t n_layers, nkv, max_ctx, ctx_pad;
    uint32_t hd[WR_HIP_MAX_LAYERS];
    size_t k_off[WR_HIP_MAX_LAYERS];     // byte offsets into slab
    size_t vt_off[WR_HIP_MAX_LAYERS];
    uint8_t* slab;
    size_t bytes;
};

namespace {

struct Buffer {
    void* p = nullptr;
    size_t cap = 0;
};

// What one calling thread submits through: its own stream, so that sessions
// driven from different threads overlap on the device (the reference lets
// independent sessions run concurrently, include/wayruntime.h:29-40), and the
// buffers whose contents belong to the launches on that stream.
struct Ctx {
    hipStream_t stream = nullptr;
    Buffer d_stage;              // device staging for host-pointer entry points
    Buffer d_part;               // split-K partials
    Buffer d_proj;               // projection operand fragments and row scales
    uint32_t* d_counters = nullptr;   // split-K tickets, zero whenever no launch is in flight
    // Error word: page-locked host memory that kernels can write.  A kernel that
    // gives up a bounded wait (and so goes on with data it cannot vouch for) stores
    // (bit 31 | layer) there; the host reads it after every wait for the
    // stream (no copy, no extra latency).  None of the present kernels waits on
    // anything but the hardware barrier, so nothing writes it today; a kernel that
    // spins on a flag must bound the spin and report here.
    volatile uint32_t* err_host = nullptr;
    uint32_t* err_dev = nullptr;
    Buffer h_pin;                // pinned host staging
    std::vector<hipEvent_t> ev;  // kernel timing (profile_begin / profile_end of this thread)
    uint32_t ev_used = 0;
    bool profiling = false;
};

struct Lib {
    std::mutex mu;               // init / shutdown, the set of thread contexts, the knobs
    std::atomic<bool> inited{false};   // read without the lock by every entry point
    int device = -1;
    uint32_t n_cus = 256;        // compute units of the device in use
    std::atomic<uint64_t> generation{0};   // bumped by every init: contexts of an earlier one are gone
    std::vector<Ctx*> ctxs;      // every context of this generation
    std::vector<Ctx*> idle;      // contexts whose thread has ended, for the next new thread
    char name[320] = "uninitialised";
    unsigned char* noalloc_ws[kMaxDevices] = {};   // device address of `scratch`, per device
    // The fixed scratch array is one per device: launches that use it are
    // chained across threads' streams through this event (recorded after each,
    // waited for before the next), under its own lock.
    std::mutex noalloc_mu;
    hipEvent_t noalloc_done = nullptr;
    bool noalloc_recorded = false;
    std::atomic<uint64_t> calls{0};
    wr_hip_log_fn log_fn = nullptr;
    void* log_user = nullptr;
    std::atomic<uint32_t> tune_keys_per_wg{0};
    std::atomic<int> force_generic{0};
    std::atomic<int> prefill_256_four_waves{0};   // WR_HIP_PREFILL_256_FOUR_WAVES=1: head dim 256 keeps the earlier four-wave prefill kernel
    std::atomic<int> prefill_two_waves{1};        // WR_HIP_PREFILL_TWO_WAVES=0: head dim 128 takes the one-wave-per-SIMD prefill kernel
} g;

// The calling thread's context (set by Entered, below).
thread_local Ctx* cx = nullptr;

constexpr uint32_t kDevErrLayerMask = 0x0000FFFFu;     // error word: bit 31 set (kDevErrWaitExpired), the layer in the low bits
constexpr float kLog2e = 1.4426950408889634f;
constexpr uint32_t kDefaultTilesPerWg = 32;  // split-K decode: 1024 keys per workgroup
constexpr uint32_t kMaxHeads = 4096;        // query heads per session the ticket array is sized for
constexpr size_t kPinSmall = 1u << 20;      // host copies up to this size go through pinned staging

void logmsg(int level, const char* fmt, ...)
{
    char buf[512];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof buf, fmt, ap);
    va_end(ap);
    if (g.log_fn)
        g.log_fn(level, buf, g.log_user);
    else
        fprintf(stderr, "[wr_hip_attn] %s\n", buf);
}

int hip_fail(hipError_t e, const char* what, uint32_t layer)
{
    logmsg(0, "hip: %s failed at layer %u: %s", what, layer, hipGetErrorString(e));
    return (e == hipErrorOutOfMemory) ? WR_HIP_ERR_NOMEM : WR_HIP_ERR_INTERNAL;
}

#define HIP_TRY(expr, what, layer)                                   \
    do {                                                             \
        hipError_t e_ = (expr);                                      \
        if (e_ != hipSuccess) return hip_fail(e_, what, layer);      \
    } while (0)

int ensure_device(Buffer& b, size_t need)
{
    if (need <= b.cap) return WR_HIP_OK;
    HIP_TRY(hipStreamSynchronize(cx->stream), "sync before workspace growth", 0);
    if (b.p) (void)hipFree(b.p);
    b.p = nullptr;
    b.cap = 0;
    const size_t want = need + need / 2 + 4096;
    HIP_TRY(hipMalloc(&b.p, want), "workspace alloc", 0);
    b.cap = want;
    return WR_HIP_OK;
}

int ensure_pinned(Buffer& b, size_t need)
{
    if (need <= b.cap) return WR_HIP_OK;
    HIP_TRY(hipStreamSynchronize(cx->stream), "sync before pinned growth", 0);
    if (b.p) (void)hipHostFree(b.p);
    b.p = nullptr;
    b.cap = 0;
    const size_t want = need + need / 2 + 4096;
    HIP_TRY(hipHostMalloc(&b.p, want, hipHostMallocDefault), "pinned alloc", 0);
    b.cap = want;
    return WR_HIP_OK;
}

// Puts the split-K tickets back to zero.  They return to zero by themselves at
// the end of every launch that completes; after a launch or a wait has failed
// nothing is known about them, and a non-zero ticket would make the next launch
// merge partial rows that were never written.
void reset_tickets()
{
    if (!cx->d_counters) return;
    const size_t cb = (size_t)WR_HIP_BATCH_MAX * kMaxHeads * sizeof(uint32_t);
    if (hipMemsetAsync(cx->d_counters, 0, cb, cx->stream) == hipSuccess) (void)hipStreamSynchronize(cx->stream);
    (void)hipGetLastError();
}

// Waits for the calling thread's stream, then looks at the error word.  Every entry point
// that promises results on return waits through here, so a kernel that gave up a
// bounded wait (and went on with wrong data) turns into WR_HIP_ERR_INTERNAL on the
// first call that could hand those results to the caller, logged with the layer
// (as the reference reports op failures, src/core/session.c:170-174).
int sync_checked(const char* what, uint32_t layer)
{
    const hipError_t e = hipStreamSynchronize(cx->stream);
    if (e != hipSuccess) {
        const int rc = hip_fail(e, what, layer);
        reset_tickets();
        return rc;
    }
    const uint32_t w = cx->err_host ? *cx->err_host : 0u;
    if (w != 0) {
        *cx->err_host = 0;
        logmsg(0, "device: a kernel's bounded wait expired at layer %u (error word 0x%08x, seen at: %s); "
                  "results produced since the previous wait are invalid", w & kDevErrLayerMask, w, what);
        reset_tickets();
        return WR_HIP_ERR_INTERNAL;
    }
    return WR_HIP_OK;
}

// Host -> device / device -> host on the stream.  Small transfers go
// through pinned staging (predictable latency); large ones are handed to the
// runtime directly.  Both leave the stream synchronised for the host buffer.
int copy_up(void* dst_dev, const void* src_host, size_t bytes, size_t pin_off)
{
    if (bytes == 0) return WR_HIP_OK;
    if (pin_off + bytes <= cx->h_pin.cap && bytes <= kPinSmall) {
        memcpy((uint8_t*)cx->h_pin.p + pin_off, src_host, bytes);
        HIP_TRY(hipMemcpyAsync(dst_dev, (uint8_t*)cx->h_pin.p + pin_off, bytes,
                               hipMemcpyHostToDevice, cx->stream), "h2d", 0);
    } else {
        HIP_TRY(hipMemcpyAsync(dst_dev, src_host, bytes, hipMemcpyHostToDevice, cx->stream),
                "h2d", 0);
        HIP_TRY(hipStreamSynchronize(cx->stream), "h2d sync", 0);
    }
    return WR_HIP_OK;
}

int copy_down_sync(void* dst_host, const void* src_dev, size_t bytes)
{
    if (bytes == 0) return sync_checked("sync", 0);
    if (bytes <= cx->h_pin.cap && bytes <= kPinSmall) {
        HIP_TRY(hipMemcpyAsync(cx->h_pin.p, src_dev, bytes, hipMemcpyDeviceToHost, cx->stream),
                "d2h", 0);
        int rc = sync_checked("d2h sync", 0);
        if (rc) return rc;
        memcpy(dst_host, cx->h_pin.p, bytes);
    } else {
        HIP_TRY(hipMemcpyAsync(dst_host, src_dev, bytes, hipMemcpyDeviceToHost, cx->stream),
                "d2h", 0);
        int rc = sync_checked("d2h sync", 0);
        if (rc) return rc;
    }
    return WR_HIP_OK;
}

template <typename Kern, typename A0, typename A1>
void launch_main(Kern kernel, dim3 grid, dim3 block, const A0& a0, const A1& a1, size_t lds_bytes)
{
    if (cx->profiling && cx->ev_used + 2 <= cx->ev.size()) {
        hipExtLaunchKernelGGL(kernel, grid, block, lds_bytes, cx->stream, cx->ev[cx->ev_used],
                              cx->ev[cx->ev_used + 1], 0, a0, a1);
        cx->ev_used += 2;
    } else {
        hipLaunchKernelGGL(kernel, grid, block, lds_bytes, cx->stream, a0, a1);
    }
}

template <typename Kern, typename Args>
void launch_main(Kern kernel, dim3 grid, dim3 block, const Args& args, size_t lds_bytes = 0)
{
    if (cx->profiling && cx->ev_used + 2 <= cx->ev.size()) {
        hipExtLaunchKernelGGL(kernel, grid, block, lds_bytes, cx->stream, cx->ev[cx->ev_used],
                              cx->ev[cx->ev_used + 1], 0, args);
        cx->ev_used += 2;
    } else {
        hipLaunchKernelGGL(kernel, grid, block, lds_bytes, cx->stream, args);
    }
}

bool mfma_shape(uint32_t hd, uint32_t group)
{
    return !g.force_generic && (hd == 64 || hd == 128 || hd == 256) && group <= kMaxGroupMfma;
}

int check_layer(const wr_hip_kv* kv, uint32_t layer)
{
    if (!kv) return WR_HIP_ERR_INVAL;
    if (layer >= kv->n_layers || kv->hd[layer] == 0) return WR_HIP_ERR_INVAL;
    return WR_HIP_OK;
}

uint32_t key_lo_for(uint32_t window, uint32_t seq_k)
{
    return (window > 0 && seq_k > window) ? seq_k - window : 0;
}

// ------------------------------------------------------------------------
// Bodies (the caller has entered: device current, cx set).

template <typename Src>
int append_rows_locked(wr_hip_kv* kv, uint32_t layer, uint32_t pos, uint32_t n_rows,
                       const Src* k_dev, const Src* v_dev)
{
    const uint32_t hd = kv->hd[layer], nkv = kv->nkv;
    uint16_t* kbase = reinterpret_cast<uint16_t*>(kv->slab + kv->k_off[layer]);
    uint16_t* vbase = reinterpret_cast<uint16_t*>(kv->slab + kv->vt_off[layer]);
    const size_t total = (size_t)n_rows * nkv * hd;
    const uint32_t blocks = (uint32_t)((total + 255) / 256);
    hipLaunchKernelGGL(HIP_KERNEL_NAME(append_k_kernel<Src>), dim3(blocks), dim3(256), 0, cx->stream,
                       k_dev, kbase, pos, n_rows, nkv, hd, kv->ctx_pad);
    const uint32_t nblk = (pos + n_rows - 1) / kVBlock - pos / kVBlock + 1;
    hipLaunchKernelGGL(HIP_KERNEL_NAME(append_v_kernel<Src>), dim3((hd + 63) / 64, nkv, nblk),
                       dim3(256), 0, cx->stream, v_dev, vbase, pos, n_rows, nkv, hd, kv->ctx_pad);
    HIP_TRY(hipGetLastError(), "append launch", layer);
    return WR_HIP_OK;
}

int check_append(const wr_hip_kv* kv, uint32_t layer, uint32_t pos, uint32_t n_rows,
                 const void* k, const void* v)
{
    if (!g.inited) return WR_HIP_ERR_STATE;
    int rc = check_layer(kv, layer);
    if (rc) return rc;
    if (n_rows == 0) return WR_HIP_OK;
    if (!k || !v) return WR_HIP_ERR_INVAL;
    if ((uint64_t)pos + n_rows > kv->max_ctx) return WR_HIP_ERR_CTX_FULL;
    return WR_HIP_OK;
}

// Where a launch keeps its split-K tickets and partial rows: the library's own
// growable buffers (ws == nullptr), or a fixed workspace that is never grown.
struct DecodeWorkspace {
    unsigned char* ws = nullptr;     // tickets at 0, partials from ticket_bytes on
    size_t ticket_bytes = 0;
    size_t bytes = 0;
};

int decode_locked(uint32_t n, wr_hip_kv* const* kv, uint32_t layer, const uint32_t* seq_k,
                  const float* q_dev, float* out_dev, uint32_t nq, float scale_override,
                  uint32_t window, const DecodeWorkspace& fixed = DecodeWorkspace(),
                  const DecodeFusedArgs* fused = nullptr)
{
    const uint32_t hd = kv[0]->hd[layer], nkv = kv[0]->nkv;
    const uint32_t group = nq / nkv;
    const bool use_mfma = mfma_shape(hd, group);

    DecodeArgs a;
    memset(&a, 0, sizeof a);
    uint64_t tiles_total = 0;
    uint32_t tiles[kBatchMax];
    for (uint32_t i = 0; i < n; i++) {
        DecodeSession& s = a.s[i];
        s.k = reinterpret_cast<const uint16_t*>(kv[i]->slab + kv[i]->k_off[layer]);
        s.vt = reinterpret_cast<const uint16_t*>(kv[i]->slab + kv[i]->vt_off[layer]);
        s.seq_k = seq_k[i];
        s.key_lo = key_lo_for(window, seq_k[i]);
        s.ctx_pad = kv[i]->ctx_pad;
        tiles[i] = (s.seq_k + kTileKeys - 1) / kTileKeys - s.key_lo / kTileKeys;
        tiles_total += tiles[i];
    }

    // Keys per workgroup.  The rule looks at ONE session only (its own visible
    // key range), never at the rest of the batch: a session's arithmetic is then
    // the same whether it is stepped alone or with others, which is what makes
    // the batched step bit-identical to serial steps (reference contract:
    // src/core/batch.c:15-19).  Half a MiB of K+V per workgroup (1024 keys at
    // head_dim 128, 512 at 256): 16 sessions of 4096 run as fast with it as
    // with twice that, and a single session's chain of tiles is half as long
    // (one session of 8192 keys: 27 -> 17 us); from
    // 8K keys up an eighth of the session per workgroup measured better
    // (fewer partials and workgroup turnovers: 82 % -> 86 % of HBM peak at
    // 16 x 32768).  A short session (up to 2048 keys at head_dim 128) takes a
    // quarter of that per workgroup: its launch is a chain of latencies, and a
    // workgroup that has all its tiles in flight at once ends sooner than one
    // that walks eight of them per wave (one session of 1024 keys: 12.0 -> 7.8 us,
    // of 2048: 13.8 -> 8.2 us; 16 sessions of ~520: the step of a 28-layer model
    // 2.03 -> 1.89 ms).  A medium session (more than 2048 and fewer than 4096 keys)
    // takes half: one session of 3000 keys 14 -> 10.6 us, the ragged batch of 16
    // 35.2 -> 34.6 us; at 4096 keys and beyond the full figure stands (16 x 4096
    // loses 4-8 % with halves).  The session's tiles are spread evenly over the workgroups,
    // and the floor keeps the in-kernel merge within kMaxSplits partials.
    // A long session (from 8K keys up at head_dim 128) is cut into twice as
    // many splits as it gets workgroups in a full launch, and a workgroup there
    // works through two consecutive splits, one after the other: the unit of
    // arithmetic (a split: one partial, the tiles dealt to the four waves in
    // turn) stays a function of the session alone, while a launch too small to
    // give every CU a workgroup sends each split to a workgroup of its own.
    // One session of 8192 keys: 64 -> 128 workgroups, 14.8 -> 11.2 us; of 16384:
    // 24.5 -> 16.2; of 32768: 43.9 -> 26.9.  The price in a full launch is one
    // extra merge of the four waves per workgroup: not measurable at 16 x 32768.
    // (The same from 4096 keys up costs 16 x 4096 4.5 %: those workgroups have
    // 32 tiles, and the waves meeting in the middle is 2 us of their 40.)
    // A caller that serves one session at a time can go further with
    // wr_hip_attn_set_tuning.
    (void)tiles_total;
    uint32_t max_splits = 1;
    const uint32_t tune = g.tune_keys_per_wg.load(std::memory_order_relaxed);
    bool pairs[kBatchMax];
    uint32_t wgs_paired = 0;
    for (uint32_t i = 0; i < n; i++) {
        uint32_t tpw, tail = 0;
        pairs[i] = false;
        bool short_pairs = false;
        if (tune) {
            tpw = tune / kTileKeys;
            if (tpw == 0) tpw = 1;
        } else {
            uint32_t cap = kDefaultTilesPerWg * 128u / (hd < 32 ? 32 : hd);
            if (cap == 0) cap = 1;
            if (tiles[i] <= 2 * cap) {                                  // a short session: see above
                cap = cap >= 4 ? cap / 4 : 1;
                // ... whose LAST four tiles are a split of their own: one tile per
                // wave.  In a decode step the last tile holds the new position: the
                // workgroup that has it also makes the new row's K and V and patches
                // them in, and with a full share of tiles on top it finishes last and
                // the merge waits for it (timestamps: its ticket 2 us after the
                // others').  With one tile per wave it finishes first, and a workgroup
                // that is done anyway merges: the decode step of a 28-layer model at
                // ~520 keys 1.02 -> 1.00 ms, sixteen sessions 1.90 -> 1.87 ms.  (A tail
                // of ONE tile does the same for one session and costs sixteen 2-3 %:
                // it adds a workgroup per session and KV head.)  A caller that has
                // appended the row itself pays for the extra split instead: one
                // session of 1024 keys 7.8 -> 8.2 us, of 2048 keys 8.1 -> 8.8 us.
                if (tiles[i] >= 6) tail = 4;
                // In a launch that fills the device two consecutive splits of a short
                // session share a workgroup as well (the splits keep their size):
                // the ragged batch of 16 has 816 workgroups for 768 places otherwise,
                // 33.5 -> 32.8 us; sixteen sessions of ~500 keys unchanged.
                short_pairs = use_mfma && hd <= 128;
            } else if (tiles[i] < 4 * cap) {
                cap = cap >= 2 ? cap / 2 : 1;                           // a medium one: see above
            } else if (cap <= tiles[i] / 8) {
                cap = tiles[i] / 8;
                pairs[i] = use_mfma && hd <= 128;                       // a long one: see above
            }
            const uint32_t body = tiles[i] - tail;
            const uint32_t want = (body + cap - 1) / cap;              // workgroups
            tpw = (body + want - 1) / want;                            // even share
            if (pairs[i]) tpw = (tpw + 1) / 2;                         // two splits per workgroup
            if (short_pairs) pairs[i] = true;
        }
        const uint32_t body = tiles[i] - tail;
        const uint32_t room = kMaxSplits - (tail ? 1u : 0u);
        const uint32_t floor_tiles = (body + room - 1) / room;
        if (tpw < floor_tiles) tpw = floor_tiles;
        a.s[i].tiles_per_wg = tpw;
        a.s[i].tail_tiles = (uint16_t)tail;
        a.s[i].parts_per_wg = 1;
        a.s[i].n_splits = (body + tpw - 1) / tpw + (tail ? 1u : 0u);
        if (a.s[i].n_splits > max_splits) max_splits = a.s[i].n_splits;
        wgs_paired += pairs[i] ? (a.s[i].n_splits + 1) / 2 : a.s[i].n_splits;
    }
    // (the launch as a whole decides this, not the session: it changes which
    // workgroup does a split, never the split)
    if ((uint64_t)wgs_paired * nkv >= g.n_cus)
        for (uint32_t i = 0; i < n; i++)
            if (pairs[i]) a.s[i].parts_per_wg = 2;
    // work list, longest entries first (ties keep session, split order)
    {
        uint32_t len[kBatchMax * kMaxSplits];
        uint32_t cnt = 0;
        for (uint32_t i = 0; i < n; i++) {
            const uint32_t body = tiles[i] - a.s[i].tail_tiles;
            const uint32_t ppw = a.s[i].parts_per_wg;
            for (uint32_t wg = 0; wg * ppw < a.s[i].n_splits; wg++) {
                uint32_t l = 0;
                for (uint32_t sp = wg * ppw; sp < (wg + 1) * ppw && sp < a.s[i].n_splits; sp++) {
                    if (a.s[i].tail_tiles && sp == a.s[i].n_splits - 1) {
                        l += a.s[i].tail_tiles;
                    } else {
                        const uint32_t begin = sp * a.s[i].tiles_per_wg;
                        const uint32_t left = body - begin;
                        l += left < a.s[i].tiles_per_wg ? left : a.s[i].tiles_per_wg;
                    }
                }
                len[cnt] = l;
                a.items[cnt++] = (uint16_t)((i << 8) | wg);
            }
        }
        for (uint32_t i = 1; i < cnt; i++) {           // insertion sort: at most 1024 entries
            const uint32_t l = len[i];
            const uint16_t it = a.items[i];
            uint32_t j = i;
            while (j > 0 && len[j - 1] < l) {
                len[j] = len[j - 1];
                a.items[j] = a.items[j - 1];
                j--;
            }
            len[j] = l;
            a.items[j] = it;
        }
        a.n_items = cnt;
    }
    a.q = q_dev;
    a.out = out_dev;
    a.nq = nq;
    a.nkv = nkv;
    a.group = group;
    a.hd = hd;
    a.max_splits = max_splits;
    a.counters = fixed.ws ? reinterpret_cast<uint32_t*>(fixed.ws) : cx->d_counters;
    const float scale = (scale_override > 0.0f) ? scale_override : 1.0f / sqrtf((float)hd);
    a.qscale = scale * kLog2e;

    if (max_splits > 1) {
        const size_t po = (size_t)n * nq * max_splits * hd * sizeof(float);
        const size_t pml = (size_t)n * nq * max_splits * 2 * sizeof(float);
        uint8_t* base;
        if (fixed.ws) {
            if (fixed.ticket_bytes + po + pml > fixed.bytes) {
                logmsg(0, "decode (no-alloc form): %zu bytes of split-K partials exceed the fixed "
                          "workspace of %zu bytes (layer %u)", po + pml, fixed.bytes - fixed.ticket_bytes,
                       layer);
                return WR_HIP_ERR_LIMIT;
            }
            base = fixed.ws + fixed.ticket_bytes;
        } else {
            int rc = ensure_device(cx->d_part, po + pml);
            if (rc) return rc;
            base = reinterpret_cast<uint8_t*>(cx->d_part.p);
        }
        a.part_o = reinterpret_cast<float*>(base);
        a.part_ml = reinterpret_cast<float*>(base + po);
        if (fixed.ws) {
            // the array keeps the last call's contents: the tickets this launch
            // uses must start at zero
            const uint32_t words = n * (use_mfma ? nkv : nq);
            hipLaunchKernelGGL(fill_u32_kernel, dim3((words + 255) / 256), dim3(256), 0, cx->stream,
                               a.counters, words, 0u);
        }
    }

    if (fused && !(use_mfma && hd == 128)) return WR_HIP_ERR_UNSUPPORTED;
    if (use_mfma) {
        const dim3 grid(nkv, a.n_items), block(kDecodeThreads);
        DecodeFusedArgs none;
        memset(&none, 0, sizeof none);
        if (fused)
            launch_main(decode_mfma_kernel<128, true>, grid, block, a, *fused, 0);
        else if (hd == 64)
            launch_main(decode_mfma_kernel<64>, grid, block, a, none, 0);
        else if (hd == 128)
            launch_main(decode_mfma_kernel<128>, grid, block, a, none, 0);
        else
            launch_main(decode_mfma_kernel<256>, grid, block, a, none, 0);
    } else {
        launch_main(decode_generic_kernel, dim3(nq, a.n_items), dim3(kDecodeThreads), a);
    }
    {
        const hipError_t e = hipGetLastError();
        if (e != hipSuccess) {
            const int rc = hip_fail(e, "decode launch", layer);
            reset_tickets();
            return rc;
        }
    }
    return WR_HIP_OK;
}

int check_decode(uint32_t n, wr_hip_kv* const* kv, uint32_t layer, const uint32_t* seq_k,
                 const void* q, const void* out, uint32_t nq)
{
    if (!g.inited) return WR_HIP_ERR_STATE;
    if (!kv || !seq_k || !q || !out) return WR_HIP_ERR_INVAL;
    if (n == 0 || n > WR_HIP_BATCH_MAX) return WR_HIP_ERR_LIMIT;
    for (uint32_t i = 0; i < n; i++)
        if (!kv[i]) return WR_HIP_ERR_INVAL;
    // The reference counts an attention call once its pointer checks have passed
    // and before it looks at any shape (src/core/kernels.c:1418-1423), so calls
    // refused for their shapes count too: one per session here.
    g.calls.fetch_add(n, std::memory_order_relaxed);
    for (uint32_t i = 0; i < n; i++) {
        int rc = check_layer(kv[i], layer);
        if (rc) return rc;
        if (kv[i]->nkv != kv[0]->nkv || kv[i]->hd[layer] != kv[0]->hd[layer])
            return WR_HIP_ERR_INVAL;
        for (uint32_t j = 0; j < i; j++)
            if (kv[i] == kv[j]) return WR_HIP_ERR_INVAL;
    }
    if (nq == 0 || nq % kv[0]->nkv != 0) return WR_HIP_ERR_INVAL;
    if (nq > kMaxHeads) return WR_HIP_ERR_LIMIT;
    for (uint32_t i = 0; i < n; i++) {
        if (seq_k[i] == 0) return WR_HIP_ERR_INVAL;
        if (seq_k[i] > WR_HIP_ATTN_MAX_SEQ) return WR_HIP_ERR_LIMIT;
        if (seq_k[i] > kv[i]->max_ctx) return WR_HIP_ERR_INVAL;
    }
    return WR_HIP_OK;
}

int prefill_locked(wr_hip_kv* kv, uint32_t layer, uint32_t p0, uint32_t T, const float* q_dev,
                   float* out_dev, uint32_t nq, float scale_override, uint32_t window,
                   const uint16_t* q16_dev = nullptr)
{
    const uint32_t hd = kv->hd[layer];
    PrefillArgs a;
    memset(&a, 0, sizeof a);
    a.k = reinterpret_cast<const uint16_t*>(kv->slab + kv->k_off[layer]);
    a.vt = reinterpret_cast<const uint16_t*>(kv->slab + kv->vt_off[layer]);
    a.q = q_dev;
    a.q16 = q16_dev;
    a.out = out_dev;
    a.p0 = p0;
    a.T = T;
    a.nq = nq;
    a.nkv = kv->nkv;
    a.group = nq / kv->nkv;
    a.hd = hd;
    a.ctx_pad = kv->ctx_pad;
    a.window = window;
    const float scale = (scale_override > 0.0f) ? scale_override : 1.0f / sqrtf((float)hd);
    a.qscale = scale * kLog2e;
    const uint32_t G = a.group;
    const bool mfma = !g.force_generic && (hd == 64 || hd == 128 || hd == 256) &&
                      (G == 1 || G == 2 || G == 4 || G == 8);
    if (q16_dev && !(mfma && (hd == 64 || hd == 128))) return WR_HIP_ERR_UNSUPPORTED;
    if (mfma) {
        const uint32_t Gw = G < 4 ? G : 4;
        const uint32_t BP = 32 * (4 / Gw);
        const uint32_t nblk = (T + BP - 1) / BP;
        const uint32_t ny = kv->nkv * (G / Gw);
        // A long and a short block per workgroup balance the causal triangle, but
        // every block pays its own prologue and epilogue: when the pairs would
        // not even give every CU a workgroup, one block per workgroup finishes
        // with the longest block instead of with a pair's sum plus a second
        // prologue and epilogue.
        a.single = ((nblk + 1) / 2) * ny < g.n_cus ? 1 : 0;
        const uint32_t nwg = a.single ? nblk : (nblk + 1) / 2;
        if (hd == 64)
            launch_main(prefill_il_kernel<64>, dim3(ny, nwg), dim3(kSplitThreads), a,
                        split_smem_bytes<64>());
        else if (hd == 128 && !g.prefill_two_waves) {
            if (q16_dev)
                launch_main(prefill_pair_kernel<128, true>, dim3(ny, nwg), dim3(kPairThreads), a,
                            pair_smem_bytes<128>());
            else
                launch_main(prefill_pair_kernel<128, false>, dim3(ny, nwg), dim3(kPairThreads), a,
                            pair_smem_bytes<128>());
        } else if (hd == 128)
            launch_main(prefill_il_kernel<128>, dim3(ny, nwg), dim3(kSplitThreads), a,
                        split_smem_bytes<128>());
        else if (!g.prefill_256_four_waves)   // 256: the wave sets divide the dimensions
            launch_main(prefill_ild_kernel, dim3(ny, nwg), dim3(kSplitThreads), a, ild_smem_bytes());
        else   // the earlier form: one wave per SIMD owns all 256 dimensions of its rows
            launch_main(prefill_mfma_kernel<256>, dim3(nwg, ny), dim3(kPrefillThreads), a);
    } else {
        launch_main(prefill_generic_kernel, dim3(T, nq), dim3(kDecodeThreads), a);
    }
    HIP_TRY(hipGetLastError(), "prefill launch", layer);
    return WR_HIP_OK;
}

int check_prefill(const wr_hip_kv* kv, uint32_t layer, uint32_t p0, uint32_t T, const void* q,
                  const void* out, uint32_t nq)
{
    if (!g.inited) return WR_HIP_ERR_STATE;
    if (!kv || !q || !out) return WR_HIP_ERR_INVAL;
    // one count per row: prefill stands for T attention calls of the reference,
    // each counted after its pointer checks and before its shape checks
    // (src/core/kernels.c:1418-1423)
    g.calls.fetch_add(T, std::memory_order_relaxed);
    int rc = check_layer(kv, layer);
    if (rc) return rc;
    if (T == 0) return WR_HIP_ERR_INVAL;
    if (nq == 0 || nq % kv->nkv != 0) return WR_HIP_ERR_INVAL;
    if ((uint64_t)p0 + T > WR_HIP_ATTN_MAX_SEQ) return WR_HIP_ERR_LIMIT;
    if ((uint64_t)p0 + T > kv->max_ctx) return WR_HIP_ERR_INVAL;
    return WR_HIP_OK;
}

// ---- thread contexts -------------------------------------------------------

void ctx_destroy(Ctx* c)
{
    if (!c) return;
    if (c->stream) (void)hipStreamSynchronize(c->stream);
    for (hipEvent_t e : c->ev) (void)hipEventDestroy(e);
    if (c->d_stage.p) (void)hipFree(c->d_stage.p);
    if (c->d_part.p) (void)hipFree(c->d_part.p);
    if (c->d_proj.p) (void)hipFree(c->d_proj.p);
    if (c->d_counters) (void)hipFree(c->d_counters);
    if (c->h_pin.p) (void)hipHostFree(c->h_pin.p);
    if (c->err_host) (void)hipHostFree((void*)c->err_host);
    if (c->stream) (void)hipStreamDestroy(c->stream);
    delete c;
}

// A new context: stream (default priority), staging, zeroed tickets, error word.
// Caller holds g.mu and has set the device.
Ctx* ctx_create()
{
    Ctx* c = new (std::nothrow) Ctx();
    if (!c) return nullptr;
    Ctx* const saved = cx;
    cx = c;                                  // the helpers below work on the current context
    int rc = WR_HIP_OK;
    hipError_t e = hipStreamCreateWithFlags(&c->stream, hipStreamNonBlocking);
    if (e != hipSuccess) rc = hip_fail(e, "stream create", 0);
    if (rc == WR_HIP_OK) rc = ensure_pinned(c->h_pin, 2 * kPinSmall);
    if (rc == WR_HIP_OK) rc = ensure_device(c->d_stage, 2 * kPinSmall);
    if (rc == WR_HIP_OK) {
        const size_t cb = (size_t)WR_HIP_BATCH_MAX * kMaxHeads * sizeof(uint32_t);
        e = hipMalloc((void**)&c->d_counters, cb);
        if (e == hipSuccess) e = hipMemsetAsync(c->d_counters, 0, cb, c->stream);
        if (e == hipSuccess) e = hipStreamSynchronize(c->stream);
        if (e != hipSuccess) rc = hip_fail(e, "ticket array", 0);
    }
    if (rc == WR_HIP_OK) {
        void* hp = nullptr;
        void* dp = nullptr;
        e = hipHostMalloc(&hp, 64, hipHostMallocMapped);
        if (e == hipSuccess) e = hipHostGetDevicePointer(&dp, hp, 0);
        if (e != hipSuccess) {
            rc = hip_fail(e, "error word", 0);
            if (hp) (void)hipHostFree(hp);
        } else {
            memset(hp, 0, 64);
            c->err_host = reinterpret_cast<volatile uint32_t*>(hp);
            c->err_dev = reinterpret_cast<uint32_t*>(dp);
        }
    }
    cx = saved;
    if (rc != WR_HIP_OK) {
        ctx_destroy(c);
        return nullptr;
    }
    return c;
}

// Hands a thread's context back when the thread ends, for the next new thread
// (threads of a pool come and go; their streams and staging need not).
struct ThreadSlot {
    Ctx* c = nullptr;
    uint64_t generation = 0;
    ~ThreadSlot()
    {
        if (!c) return;
        std::lock_guard<std::mutex> lk(g.mu);
        if (g.inited && generation == g.generation) g.idle.push_back(c);
    }
};
thread_local ThreadSlot t_slot;

// Every entry point that touches the device starts here: the device is made
// current for the calling thread and `cx` is the thread's context, created on
// the thread's first call.  ok() is false when that failed (out of memory) or
// the library is not initialised.  No lock is held afterwards: calls from
// different threads run side by side, each on its own stream.
struct Entered {
    bool good = false;
    Entered()
    {
        if (!g.inited) return;
        (void)hipSetDevice(g.device);
        if (!t_slot.c || t_slot.generation != g.generation) {
            std::lock_guard<std::mutex> lk(g.mu);
            if (!g.inited) return;
            Ctx* c = nullptr;
            if (!g.idle.empty()) {
                c = g.idle.back();
                g.idle.pop_back();
                c->profiling = false;            // the thread that had it before may have ended mid-measurement
                c->ev_used = 0;
            } else {
                c = ctx_create();
                if (c) g.ctxs.push_back(c);
            }
            t_slot.c = c;
            t_slot.generation = g.generation;
        }
        cx = t_slot.c;
        good = cx != nullptr;
    }
    bool ok() const { return good; }
};

#define ENTER()                                   \
    Entered entered_;                             \
    if (!entered_.ok()) return g.inited ? WR_HIP_ERR_NOMEM : WR_HIP_ERR_STATE

}  // namespace

// projections: launch helpers (the caller has entered)
namespace {

template <int GROUPS, int NT>
void launch_proj(const ProjArgs& a, uint32_t groups)
{
    const uint32_t runs = (a.N / 16 + NT - 1) / NT;              // runs of 16*NT outputs
    const uint32_t per_block = 4 / a.ksplit;
    launch_main(proj_rows_kernel<GROUPS, NT>,
                dim3((runs + per_block - 1) / per_block, (groups + GROUPS - 1) / GROUPS),
                dim3(kProjThreads), a);
}

// Prefill-sized row counts: the largest tile that still fills the chip.
//   LDS-staged, eight waves, 256 outputs x 128 rows per workgroup, from one workgroup per CU;
//   LDS-staged, 128 x 128, from two workgroups per CU;
//   LDS-staged, 128 x 64, from one per CU (software-pipelined: a SIMD may hold a single wave);
//   registers, 64 x 32, the four waves split the input range;
//   registers, 32 x 32, likewise.
constexpr int kProjGemmMinRows = 64;
constexpr size_t kProjRow1MaxLds = 60 * 1024;      // inputs up to 15 360 take the one-row kernel

template <int GROUPS, int NT>
void launch_proj_gemm_split(const ProjArgs& a, uint32_t groups)
{
    launch_main(proj_gemm_split_kernel<GROUPS, NT>,
                dim3((a.N / 16 + NT - 1) / NT, (groups + GROUPS - 1) / GROUPS), dim3(kProjThreads), a);
}

void launch_proj_gemm(const ProjArgs& a, uint32_t groups)
{
    const uint32_t nt = a.N / 16, panels = (nt + 7) / 8;
    // one-dimensional grids: eight equal shares of output panels, times the row panels
    const uint32_t share = (panels + 7) / 8 * 8;
    const uint32_t wide = (nt + 15) / 16, wshare = (wide + 7) / 8 * 8;
    // The eight-wave tile runs one workgroup per CU, in rounds of 256: when its
    // last round would leave more than 10 % of the CUs idle, the four-wave tile
    // (two per CU, half the work each) loses less (2047 rows x 6144 outputs:
    // 384 eight-wave tiles, 1.5 rounds, 83 us; 768 four-wave tiles 65 us.
    // 1024 rows x 28672 outputs: 896 eight-wave tiles, 3.5 rounds, 559 us;
    // 1792 four-wave tiles 530 us).
    const uint32_t n_wide = wide * ((groups + 15) / 16), n_big = panels * ((groups + 15) / 16);
    const uint32_t rounds = (n_wide + 255) / 256;
    const bool wide_fills = n_wide >= 256 && (n_wide * 100 >= rounds * 256 * 90 || n_big < 512);
    // The four-wave tiles run two per CU, in rounds of 512.  The 128 x 128 tile moves
    // fewer bytes per MFMA than the 128 x 64 one (2048 rows x 4096 -> 6144: 226 against
    // 243 us) but has half as many workgroups to fill its last round with: where that
    // round would be thin (under 70 % full) and the smaller tile's is fuller by a tenth
    // or more, the smaller tile wins (1536 rows x 1024 -> 6144: 576 tiles, 1.1 rounds,
    // 59.8 us; 1152 smaller ones 49 us.  At three quarters full the larger tile still
    // holds its own: 2047 rows x 1024 -> 6144 65.6 against 64.8 us, 2048 x 4096 -> 6144
    // 226 against 243).
    const uint32_t n_small = panels * ((groups + 7) / 8);
    const uint32_t rounds_b = (n_big + 511) / 512, rounds_s = (n_small + 511) / 512;
    const bool small_fills_better = n_small >= 512 && n_big * 100 < rounds_b * 512 * 70 &&
                                    (uint64_t)n_small * rounds_b * 100 >= (uint64_t)n_big * rounds_s * 100 + (uint64_t)rounds_b * rounds_s * 512 * 10;
    if (wide_fills)
        launch_main(proj_gemm_lds_kernel<8, 4, 4>, dim3(wshare * ((groups + 15) / 16)), dim3(512), a,
                    gemm_lds_bytes<8, 4, 4>());
    else if (n_big >= 512 && !small_fills_better)
        launch_main(proj_gemm_lds_kernel<8, 2, 3>, dim3(share * ((groups + 15) / 16)), dim3(kProjThreads), a,
                    gemm_lds_bytes<8, 2, 3>());
    else if (panels * ((groups + 7) / 8) >= 512)          // two and more per CU cover each other's latency
        launch_main(proj_gemm_lds_kernel<4, 2, 3>, dim3(share * ((groups + 7) / 8)), dim3(kProjThreads), a,
                    gemm_lds_bytes<4, 2, 3>());
    else if (panels * ((groups + 7) / 8) >= 256 && (a.K / 32) % 2 == 0 && a.K >= 2048)
        // one per CU and a long input range: two sets of waves halve it (two waves per SIMD, half the
        // chain of k-steps; 2047 rows x 2048 -> 1024: 40.3 -> 28.3 us, x 3072 -> 1024: 40 -> 36.6; at
        // 1024 inputs the sum through LDS costs more than the shorter chain gives)
        launch_main(proj_gemm_lds_kernel<4, 2, 4, true, 2>, dim3(share * ((groups + 7) / 8)), dim3(2 * kProjThreads), a,
                    gemm_lds_bytes<4, 2, 4, 2>());
    else if (panels * ((groups + 7) / 8) >= 256)          // one per CU, one wave per SIMD: pipelined reads
        launch_main(proj_gemm_lds_kernel<4, 2, 4, true>, dim3(share * ((groups + 7) / 8)), dim3(kProjThreads), a,
                    gemm_lds_bytes<4, 2, 4>());
    else if (((nt + 3) / 4) * ((groups + 3) / 4) >= 384)
        launch_proj_gemm_split<4, 4>(a, groups);
    else
        launch_proj_gemm_split<4, 2>(a, groups);
}

// What feeds a projection: the rows as they are, their RMS normalisation, or
// the gated activation of rows that hold gate and up values side by side.
struct ProjSource {
    int kind = kProjSrcPlain;
    const float* norm_w = nullptr;
    float eps = 0.f;
};

// y_dev[rows][ldy] = source(x_dev)[rows][n_in] . W^T (+ add_dev), rows <= kProjMaxRows.
// The caller has entered.
int proj_chunk_locked(const wr_hip_weight* w, uint32_t rows, const float* x_dev, uint32_t ldx,
                      const ProjSource& src, const float* add_dev, float* y_dev, uint32_t ldy)
{
    // row groups of eight, padded to what one wave takes (1, 2, or runs of 4)
    uint32_t groups = (rows + 7) / 8;
    const bool gemm = rows >= (uint32_t)kProjGemmMinRows;  // the GEMM kernel clamps instead of padding
    if (groups > 2 && !gemm) groups = (groups + 3) / 4 * 4;
    const uint32_t ktiles = w->n_in / 32;
    // one row: the fragment step runs inside the product's kernel (4 bytes of LDS per input)
    const bool row1 = rows == 1 && (size_t)w->n_in * 4 <= kProjRow1MaxLds;
    const size_t frag_bytes = (size_t)groups * ktiles * 1024;
    int rc = ensure_device(cx->d_proj, frag_bytes + kProjMaxRows * sizeof(float));
    if (rc) return rc;
    half8* frag = reinterpret_cast<half8*>(cx->d_proj.p);
    float* scales = reinterpret_cast<float*>((uint8_t*)cx->d_proj.p + frag_bytes);
    ProjPrepArgs pa;
    pa.x = x_dev;
    pa.norm_w = src.norm_w;
    pa.frag = frag;
    pa.scales = scales;
    pa.ldx = ldx;
    pa.R = rows;
    pa.K = w->n_in;
    pa.eps = src.eps;
    const dim3 pgrid(groups * 8), pblock(256);
    const bool in_regs = w->n_in <= 4096;           // two chunks of eight values per thread
    // many rows: a workgroup per row group (whole-line writes); it reads rows
    // with 16-byte loads
    const bool by_group = gemm && ldx % 4 == 0 && ((uintptr_t)x_dev & 15) == 0 &&
                          ((uintptr_t)src.norm_w & 15) == 0;
    const uint32_t kin = w->n_in;
#define WR_LAUNCH_PREP_GROUP(SRC, CH) \
    hipLaunchKernelGGL(HIP_KERNEL_NAME(proj_prep_group_kernel<SRC, CH>), dim3(groups), pblock, 0, cx->stream, pa)
#define WR_LAUNCH_PREP(SRC)                                                                          \
    do {                                                                                             \
        if (by_group && kin <= 1024)                                                                 \
            WR_LAUNCH_PREP_GROUP(SRC, 4);                                                            \
        else if (by_group && kin <= 2048)                                                            \
            WR_LAUNCH_PREP_GROUP(SRC, 8);                                                            \
        else if (by_group && kin <= 4096)                                                            \
            WR_LAUNCH_PREP_GROUP(SRC, 16);                                                           \
        else if (by_group)                                                                           \
            WR_LAUNCH_PREP_GROUP(SRC, 0);                                                            \
        else if (in_regs)                                                                            \
            hipLaunchKernelGGL(HIP_KERNEL_NAME(proj_prep_kernel<SRC, 2>), pgrid, pblock, 0, cx->stream, pa); \
        else                                                                                         \
            hipLaunchKernelGGL(HIP_KERNEL_NAME(proj_prep_kernel<SRC, 0>), pgrid, pblock, 0, cx->stream, pa); \
    } while (0)
    if (row1)
        ;                                           // no fragment launch
    else if (src.kind == kProjSrcRmsNorm)
        WR_LAUNCH_PREP(kProjSrcRmsNorm);
    else if (src.kind == kProjSrcSwiglu)
        WR_LAUNCH_PREP(kProjSrcSwiglu);
    else if (src.kind == kProjSrcGeglu)
        WR_LAUNCH_PREP(kProjSrcGeglu);
    else
        WR_LAUNCH_PREP(kProjSrcPlain);
#undef WR_LAUNCH_PREP
#undef WR_LAUNCH_PREP_GROUP
    ProjArgs a;
    a.w = reinterpret_cast<const half8*>(w->tiles);
    a.xfrag = frag;
    a.scales = scales;
    a.bias_rows = add_dev;
    a.y = y_dev;
    a.N = w->n_out;
    a.K = w->n_in;
    a.R = rows;
    a.ldy = ldy;
    // Waves that share a run of outputs (contiguous parts of the inputs, summed
    // through LDS in a fixed order): enough that a narrow weight still gives
    // one to two thousand waves.  A function of the weight's shape only: a row's
    // sums are then split the same way whether it travels alone or with up to
    // fifteen others, so a batched step's rows equal the serial steps' bit
    // for bit (reference contract: src/core/batch.c:15-19).  Larger row counts
    // (prefill chunks) use one wave per run.
    const uint32_t tiles = w->n_out / 16;
    uint32_t ksplit = 1;
    if (groups <= 2) {
        while (ksplit < 4 && tiles * ksplit < 2048 && ktiles % (ksplit * 2) == 0 &&
               ktiles / (ksplit * 2) >= 4)
            ksplit *= 2;
    }
    a.ksplit = ksplit;
    if (row1) {
        const dim3 grid((tiles + 4 / ksplit - 1) / (4 / ksplit)), block(kProjThreads);
        const size_t lds = (size_t)w->n_in * 4;
        if (src.kind == kProjSrcRmsNorm)
            launch_main(proj_row1_kernel<kProjSrcRmsNorm>, grid, block, a, pa, lds);
        else if (src.kind == kProjSrcSwiglu)
            launch_main(proj_row1_kernel<kProjSrcSwiglu>, grid, block, a, pa, lds);
        else if (src.kind == kProjSrcGeglu)
            launch_main(proj_row1_kernel<kProjSrcGeglu>, grid, block, a, pa, lds);
        else
            launch_main(proj_row1_kernel<kProjSrcPlain>, grid, block, a, pa, lds);
    } else if (gemm)
        launch_proj_gemm(a, groups);
    else if (groups == 1)
        launch_proj<1, 1>(a, groups);
    else if (groups == 2 && tiles * ksplit >= 2048)
        launch_proj<2, 2>(a, groups);       // wide weight: two output tiles per operand load
    else if (groups == 2)
        launch_proj<2, 1>(a, groups);       // narrow weight: every wave counts
    else
        launch_proj<4, 4>(a, groups);       // grid.y = groups / 4
    HIP_TRY(hipGetLastError(), "projection launch", 0);
    return WR_HIP_OK;
}

int proj_locked(const wr_hip_weight* w, uint32_t rows, const float* x_dev, uint32_t ldx,
                const ProjSource& src, const float* add_dev, float* y_dev, uint32_t ldy)
{
    for (uint32_t done = 0; done < rows; done += kProjMaxRows) {
        const uint32_t n = rows - done < (uint32_t)kProjMaxRows ? rows - done : (uint32_t)kProjMaxRows;
        int rc = proj_chunk_locked(w, n, x_dev + (size_t)done * ldx, ldx, src,
                                   add_dev ? add_dev + (size_t)done * ldy : nullptr,
                                   y_dev + (size_t)done * ldy, ldy);
        if (rc) return rc;
    }
    return WR_HIP_OK;
}

}  // namespace

// ======================================================================= ABI

extern "C" {

int wr_hip_attn_init(int device)
{
    std::lock_guard<std::mutex> lk(g.mu);
    if (g.inited) return WR_HIP_ERR_STATE;
    int count = 0;
    if (hipGetDeviceCount(&count) != hipSuccess || count <= 0) {
        logmsg(0, "init: no HIP device visible; this library has no CPU path");
        return WR_HIP_ERR_UNSUPPORTED;
    }
    if (device < 0 || device >= count) return WR_HIP_ERR_INVAL;
    hipDeviceProp_t prop;
    HIP_TRY(hipSetDevice(device), "set device", 0);
    HIP_TRY(hipGetDeviceProperties(&prop, device), "device properties", 0);
    if (strncmp(prop.gcnArchName, "gfx950", 6) != 0) {
        logmsg(0, "init: device %d is %s; the kernels are built for gfx950 only", device,
               prop.gcnArchName);
        return WR_HIP_ERR_UNSUPPORTED;
    }
    g.device = device;
    g.n_cus = prop.multiProcessorCount > 0 ? (uint32_t)prop.multiProcessorCount : 256u;
    snprintf(g.name, sizeof g.name, "%s %s, %d CUs, %.1f GiB", prop.gcnArchName, prop.name,
             prop.multiProcessorCount, (double)prop.totalGlobalMem / (1024.0 * 1024.0 * 1024.0));
    g.inited = true;
    g.calls.store(0);
    {
        const char* e = getenv("WR_HIP_PREFILL_TWO_WAVES");
        g.prefill_two_waves = (e && e[0] == '0') ? 0 : 1;
        e = getenv("WR_HIP_PREFILL_256_FOUR_WAVES");
        g.prefill_256_four_waves = (e && e[0] == '1') ? 1 : 0;
    }
    g.generation++;
    int rc = WR_HIP_OK;
    {
        const hipError_t e = hipEventCreateWithFlags(&g.noalloc_done, hipEventDisableTiming);
        if (e != hipSuccess) rc = hip_fail(e, "event create", 0);
        g.noalloc_recorded = false;
    }
    if (rc == WR_HIP_OK) {
        // device address of the no-alloc entry point's scratch array, once per
        // device, with that device current
        if (device >= kMaxDevices) {
            rc = WR_HIP_ERR_LIMIT;
        } else if (!g.noalloc_ws[device]) {
            void* p = nullptr;
            hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
            if (e != hipSuccess || !p)
                rc = hip_fail(e, "address of the no-alloc scratch array", 0);
            else
                g.noalloc_ws[device] = reinterpret_cast<unsigned char*>(p);
        }
    }
    if (rc == WR_HIP_OK) {
        // the two-waves-per-SIMD prefill kernels stage more than the 64 KiB a
        // kernel may use without asking
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(prefill_il_kernel<64>),
                                           hipFuncAttributeMaxDynamicSharedMemorySize,
                                           (int)split_smem_bytes<64>());
        if (e == hipSuccess)
            e = hipFuncSetAttribute(reinterpret_cast<const void*>(prefill_il_kernel<128>),
                                    hipFuncAttributeMaxDynamicSharedMemorySize,
                                    (int)split_smem_bytes<128>());
        if (e == hipSuccess)
            e = hipFuncSetAttribute(reinterpret_cast<const void*>(prefill_pair_kernel<128, false>),
                                    hipFuncAttributeMaxDynamicSharedMemorySize,
                                    (int)pair_smem_bytes<128>());
        if (e == hipSuccess)
            e = hipFuncSetAttribute(reinterpret_cast<const void*>(prefill_pair_kernel<128, true>),
                                    hipFuncAttributeMaxDynamicSharedMemorySize,
                                    (int)pair_smem_bytes<128>());
        if (e == hipSuccess)
            e = hipFuncSetAttribute(reinterpret_cast<const void*>(prefill_ild_kernel),
                                    hipFuncAttributeMaxDynamicSharedMemorySize, (int)ild_smem_bytes());
        if (e == hipSuccess)
            e = hipFuncSetAttribute(reinterpret_cast<const void*>(proj_gemm_lds_kernel<8, 2, 3>),
                                    hipFuncAttributeMaxDynamicSharedMemorySize, (int)gemm_lds_bytes<8, 2, 3>());
        if (e == hipSuccess)
            e = hipFuncSetAttribute(reinterpret_cast<const void*>(proj_gemm_lds_kernel<4, 2, 4, true>),
                                    hipFuncAttributeMaxDynamicSharedMemorySize, (int)gemm_lds_bytes<4, 2, 4>());
        if (e == hipSuccess)
            e = hipFuncSetAttribute(reinterpret_cast<const void*>(proj_gemm_lds_kernel<4, 2, 4, true, 2>),
                                    hipFuncAttributeMaxDynamicSharedMemorySize, (int)gemm_lds_bytes<4, 2, 4, 2>());
        if (e == hipSuccess)
            e = hipFuncSetAttribute(reinterpret_cast<const void*>(proj_gemm_lds_kernel<8, 4, 4>),
                                    hipFuncAttributeMaxDynamicSharedMemorySize, (int)gemm_lds_bytes<8, 4, 4>());
        if (e != hipSuccess) rc = hip_fail(e, "kernel LDS size", 0);
    }
    if (rc != WR_HIP_OK) {
        g.inited = false;
        if (g.noalloc_done) (void)hipEventDestroy(g.noalloc_done);
        g.noalloc_done = nullptr;
    }
    return rc;
}

void wr_hip_attn_shutdown(void)
{
    std::lock_guard<std::mutex> lk(g.mu);
    if (!g.inited) return;
    (void)hipSetDevice(g.device);
    for (Ctx* c : g.ctxs) ctx_destroy(c);      // waits for each stream first
    g.ctxs.clear();
    g.idle.clear();
    cx = nullptr;
    if (g.noalloc_done) (void)hipEventDestroy(g.noalloc_done);
    g.noalloc_done = nullptr;
    g.inited = false;
    g.device = -1;
    g.tune_keys_per_wg = 0;
    g.force_generic = 0;
}

void wr_hip_attn_set_log(wr_hip_log_fn fn, void* user)
{
    g.log_fn = fn;
    g.log_user = user;
}

uint64_t wr_hip_attn_calls(void) { return g.calls.load(std::memory_order_relaxed); }

const char* wr_hip_attn_device_name(void) { return g.name; }

uint32_t wr_hip_attn_caps(void) { return WR_HIP_CAP_PROJ; }

void wr_hip_attn_set_prefill_one_wave(int on)
{
    g.prefill_two_waves = on ? 0 : 1;
}

void wr_hip_attn_set_tuning(uint32_t decode_keys_per_wg, int force_generic)
{
    std::lock_guard<std::mutex> lk(g.mu);
    g.tune_keys_per_wg = decode_keys_per_wg;
    g.force_generic = force_generic;
}

// ---------------------------------------------------------------- storage --

int wr_hip_attn_kv_create(uint32_t n_layers, const uint32_t* hd_per_layer, uint32_t nkv,
                          uint32_t max_ctx, wr_hip_kv** out)
{
    if (!out) return WR_HIP_ERR_INVAL;
    *out = nullptr;
    if (!g.inited) return WR_HIP_ERR_STATE;
    if (!hd_per_layer || n_layers == 0 || nkv == 0 || max_ctx == 0) return WR_HIP_ERR_INVAL;
    if (n_layers > WR_HIP_MAX_LAYERS) return WR_HIP_ERR_LIMIT;
    if (max_ctx > WR_HIP_ATTN_MAX_SEQ) return WR_HIP_ERR_LIMIT;
    for (uint32_t L = 0; L < n_layers; L++)
        if (hd_per_layer[L] > WR_HIP_FLASH_D_MAX) return WR_HIP_ERR_LIMIT;

    wr_hip_kv* kv = new (std::nothrow) wr_hip_kv();
    if (!kv) return WR_HIP_ERR_NOMEM;
    kv->n_layers = n_layers;
    kv->nkv = nkv;
    kv->max_ctx = max_ctx;
    kv->ctx_pad = (max_ctx + kVBlock - 1) / kVBlock * kVBlock;
    size_t cur = 0;
    bool any = false;
    for (uint32_t L = 0; L < n_layers; L++) {
        kv->hd[L] = hd_per_layer[L];
        if (kv->hd[L] == 0) continue;
        any = true;
        // K rows are padded to whole 16-byte chunks (common.hip.h); Vt is not
        const size_t k_side = ((size_t)nkv * kv->ctx_pad * k_padded_hd(kv->hd[L]) * 2 + 255) & ~(size_t)255;
        const size_t v_side = ((size_t)nkv * kv->ctx_pad * kv->hd[L] * 2 + 255) & ~(size_t)255;
        kv->k_off[L] = cur;
        cur += k_side;
        kv->vt_off[L] = cur;
        cur += v_side;
    }
    if (!any) {
        delete kv;
        return WR_HIP_ERR_INVAL;
    }
    kv->bytes = cur;

    ENTER();
    hipError_t e = hipMalloc((void**)&kv->slab, cur);
    if (e != hipSuccess) {
        logmsg(0, "session: device slab alloc failed (%zu bytes): %s", cur, hipGetErrorString(e));
        delete kv;
        return WR_HIP_ERR_NOMEM;
    }
    e = hipMemsetAsync(kv->slab, 0, cur, cx->stream);
    if (e == hipSuccess) e = hipStreamSynchronize(cx->stream);
    if (e != hipSuccess) {
        (void)hipFree(kv->slab);
        delete kv;
        return hip_fail(e, "slab clear", 0);
    }
    *out = kv;
    return WR_HIP_OK;
}

void wr_hip_attn_kv_destroy(wr_hip_kv* kv)
{
    if (!kv) return;
    if (g.inited) {
        Entered entered_;
        if (entered_.ok()) (void)hipStreamSynchronize(cx->stream);
        if (kv->slab) (void)hipFree(kv->slab);     // (waits for the device's other streams by itself)
    }
    delete kv;
}

uint64_t wr_hip_attn_kv_bytes(const wr_hip_kv* kv) { return kv ? kv->bytes : 0; }

// ----------------------------------------------------------------- append --

int wr_hip_attn_append_dev(wr_hip_kv* kv, uint32_t layer, uint32_t pos, uint32_t n_rows,
                           const float* k_f32_dev, const float* v_f32_dev)
{
    int rc = check_append(kv, layer, pos, n_rows, k_f32_dev, v_f32_dev);
    if (rc || n_rows == 0) return rc;
    ENTER();
    return append_rows_locked<float>(kv, layer, pos, n_rows, k_f32_dev, v_f32_dev);
}

int wr_hip_attn_append_batched_dev(uint32_t n, wr_hip_kv* const* kv, uint32_t layer,
                                   const uint32_t* pos, const float* k_f32_dev,
                                   const float* v_f32_dev)
{
    if (!g.inited) return WR_HIP_ERR_STATE;
    if (!kv || !pos || !k_f32_dev || !v_f32_dev) return WR_HIP_ERR_INVAL;
    if (n == 0 || n > WR_HIP_BATCH_MAX) return WR_HIP_ERR_LIMIT;
    AppendBatchArgs a;
    memset(&a, 0, sizeof a);
    for (uint32_t i = 0; i < n; i++) {
        int rc = check_layer(kv[i], layer);
        if (rc) return rc;
        if (kv[i]->nkv != kv[0]->nkv || kv[i]->hd[layer] != kv[0]->hd[layer]) return WR_HIP_ERR_INVAL;
        for (uint32_t j = 0; j < i; j++)
            if (kv[i] == kv[j]) return WR_HIP_ERR_INVAL;
        if (pos[i] >= kv[i]->max_ctx) return WR_HIP_ERR_CTX_FULL;      // nothing is written
        a.k[i] = reinterpret_cast<uint16_t*>(kv[i]->slab + kv[i]->k_off[layer]);
        a.vt[i] = reinterpret_cast<uint16_t*>(kv[i]->slab + kv[i]->vt_off[layer]);
        a.pos[i] = pos[i];
        a.ctx_pad[i] = kv[i]->ctx_pad;
    }
    a.k_src = k_f32_dev;
    a.v_src = v_f32_dev;
    a.nkv = kv[0]->nkv;
    a.hd = kv[0]->hd[layer];
    ENTER();
    hipLaunchKernelGGL(append_batch_kernel, dim3(n), dim3(256), 0, cx->stream, a);
    HIP_TRY(hipGetLastError(), "batched append launch", layer);
    return WR_HIP_OK;
}

int wr_hip_attn_rope_dev(void* x_dev, const void* cos_sin_dev, uint32_t rows, uint32_t heads,
                         uint32_t hd, uint32_t n_rot)
{
    if (!g.inited) return WR_HIP_ERR_STATE;
    if (!x_dev || !cos_sin_dev) return WR_HIP_ERR_INVAL;
    if (hd < 2 || (hd & 1) || heads == 0 || n_rot > hd / 2) return WR_HIP_ERR_INVAL;
    if (rows == 0 || n_rot == 0) return WR_HIP_OK;
    ENTER();
    const size_t total = (size_t)rows * heads * n_rot;
    hipLaunchKernelGGL(rope_rows_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0,
                       cx->stream, reinterpret_cast<float*>(x_dev),
                       reinterpret_cast<const float*>(cos_sin_dev), rows, heads, hd, n_rot);
    HIP_TRY(hipGetLastError(), "rope launch", 0);
    return WR_HIP_OK;
}

int wr_hip_attn_rope_table_dev(float* cos_sin_dev, uint32_t rows, uint32_t pos0,
                               const uint32_t* pos, uint32_t hd, float theta_base,
                               uint32_t n_rot_pairs)
{
    if (!g.inited) return WR_HIP_ERR_STATE;
    if (!cos_sin_dev || rows == 0) return WR_HIP_ERR_INVAL;
    if (hd < 2 || (hd & 1)) return WR_HIP_ERR_INVAL;
    if (pos && rows > WR_HIP_BATCH_MAX) return WR_HIP_ERR_INVAL;
    // The kernel folds an angle into [-pi, pi] by subtracting 2 pi in a loop, as
    // the reference does (src/core/mathx.c:112-147); from an angle of 2^27 on a
    // float's spacing exceeds 2 pi, the subtraction rounds back to itself and the
    // loop never ends.  The reference's callers stay below WR_ATTN_MAX_SEQ: the
    // same bound here, before anything is launched.
    if (!pos && (uint64_t)pos0 + rows > WR_HIP_ATTN_MAX_SEQ) return WR_HIP_ERR_LIMIT;
    for (uint32_t i = 0; pos && i < rows; i++)
        if (pos[i] >= WR_HIP_ATTN_MAX_SEQ) return WR_HIP_ERR_LIMIT;
    RopeTableArgs a{};
    a.out = cos_sin_dev;
    a.rows = rows;
    a.hd = hd;
    a.n_rot = (n_rot_pairs >= 1 && n_rot_pairs < hd / 2) ? n_rot_pairs : hd / 2;
    a.theta = theta_base < 1.0f ? 10000.0f : theta_base;
    a.pos0 = pos0;
    a.listed = pos ? 1u : 0u;
    for (uint32_t i = 0; pos && i < rows; i++) a.pos[i] = pos[i];
    ENTER();
    hipLaunchKernelGGL(rope_table_kernel, dim3((rows + 63u) / 64u, a.n_rot), dim3(64), 0, cx->stream, a);
    HIP_TRY(hipGetLastError(), "rotary table launch", 0);
    return WR_HIP_OK;
}

int wr_hip_attn_append_rope(wr_hip_kv* kv, uint32_t layer, uint32_t pos, uint32_t n_rows,
                            const float* k_f32, const float* v_f32, const float* cos_sin,
                            uint32_t n_rot)
{
    int rc = check_append(kv, layer, pos, n_rows, k_f32, v_f32);
    if (rc) return rc;
    if (!cos_sin && n_rot > 0) return WR_HIP_ERR_INVAL;
    if (n_rot > kv->hd[layer] / 2) return WR_HIP_ERR_INVAL;
    if (n_rows == 0) return WR_HIP_OK;
    const uint32_t hd = kv->hd[layer], nkv = kv->nkv;
    const size_t bytes = (size_t)n_rows * nkv * hd * sizeof(float);
    const size_t tbytes = (size_t)n_rows * n_rot * 2 * sizeof(float);
    ENTER();
    rc = ensure_device(cx->d_stage, 2 * bytes + tbytes);
    if (rc) return rc;
    float* dk = reinterpret_cast<float*>(cx->d_stage.p);
    float* dv = reinterpret_cast<float*>((uint8_t*)cx->d_stage.p + bytes);
    float* dt = reinterpret_cast<float*>((uint8_t*)cx->d_stage.p + 2 * bytes);
    rc = copy_up(dk, k_f32, bytes, 0);
    if (rc == WR_HIP_OK) rc = copy_up(dv, v_f32, bytes, bytes);
    if (rc == WR_HIP_OK) rc = copy_up(dt, cos_sin, tbytes, 2 * bytes);
    if (rc == WR_HIP_OK && n_rot > 0) {
        const size_t total = (size_t)n_rows * nkv * n_rot;
        hipLaunchKernelGGL(rope_rows_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0,
                           cx->stream, dk, dt, n_rows, nkv, hd, n_rot);
        HIP_TRY(hipGetLastError(), "rope launch", layer);
    }
    if (rc == WR_HIP_OK) rc = append_rows_locked<float>(kv, layer, pos, n_rows, dk, dv);
    // the staging buffers are reused by the next call: wait for the kernels
    if (rc == WR_HIP_OK) HIP_TRY(hipStreamSynchronize(cx->stream), "append sync", layer);
    return rc;
}

int wr_hip_attn_append(wr_hip_kv* kv, uint32_t layer, uint32_t pos, uint32_t n_rows,
                       const float* k_f32, const float* v_f32)
{
    int rc = check_append(kv, layer, pos, n_rows, k_f32, v_f32);
    if (rc || n_rows == 0) return rc;
    const size_t bytes = (size_t)n_rows * kv->nkv * kv->hd[layer] * sizeof(float);
    ENTER();
    rc = ensure_device(cx->d_stage, 2 * bytes);
    if (rc) return rc;
    float* dk = reinterpret_cast<float*>(cx->d_stage.p);
    float* dv = reinterpret_cast<float*>((uint8_t*)cx->d_stage.p + bytes);
    rc = copy_up(dk, k_f32, bytes, 0);
    if (rc == WR_HIP_OK) rc = copy_up(dv, v_f32, bytes, bytes);
    if (rc == WR_HIP_OK) rc = append_rows_locked<float>(kv, layer, pos, n_rows, dk, dv);
    // the staging buffers are reused by the next call: wait for the kernels
    if (rc == WR_HIP_OK) HIP_TRY(hipStreamSynchronize(cx->stream), "append sync", layer);
    return rc;
}

int wr_hip_attn_kv_write(wr_hip_kv* kv, uint32_t layer, uint32_t pos, uint32_t n_rows,
                         const uint16_t* k_f16, const uint16_t* v_f16)
{
    int rc = check_append(kv, layer, pos, n_rows, k_f16, v_f16);
    if (rc || n_rows == 0) return rc;
    const size_t bytes = (size_t)n_rows * kv->nkv * kv->hd[layer] * sizeof(uint16_t);
    ENTER();
    rc = ensure_device(cx->d_stage, 2 * bytes);
    if (rc) return rc;
    uint16_t* dk = reinterpret_cast<uint16_t*>(cx->d_stage.p);
    uint16_t* dv = reinterpret_cast<uint16_t*>((uint8_t*)cx->d_stage.p + bytes);
    rc = copy_up(dk, k_f16, bytes, 0);
    if (rc == WR_HIP_OK) rc = copy_up(dv, v_f16, bytes, bytes);
    if (rc == WR_HIP_OK) rc = append_rows_locked<uint16_t>(kv, layer, pos, n_rows, dk, dv);
    if (rc == WR_HIP_OK) HIP_TRY(hipStreamSynchronize(cx->stream), "kv_write sync", layer);
    return rc;
}

int wr_hip_attn_kv_read(wr_hip_kv* kv, uint32_t layer, uint32_t pos, uint32_t n_rows,
                        uint16_t* k_f16, uint16_t* v_f16)
{
    if (!g.inited) return WR_HIP_ERR_STATE;
    int rc = check_layer(kv, layer);
    if (rc) return rc;
    if (n_rows == 0) return WR_HIP_OK;
    if (!k_f16 || !v_f16) return WR_HIP_ERR_INVAL;
    if ((uint64_t)pos + n_rows > kv->max_ctx) return WR_HIP_ERR_INVAL;
    const uint32_t hd = kv->hd[layer], nkv = kv->nkv;
    const size_t total = (size_t)n_rows * nkv * hd;
    const size_t bytes = total * sizeof(uint16_t);
    ENTER();
    rc = ensure_device(cx->d_stage, 2 * bytes);
    if (rc) return rc;
    uint16_t* dk = reinterpret_cast<uint16_t*>(cx->d_stage.p);
    uint16_t* dv = reinterpret_cast<uint16_t*>((uint8_t*)cx->d_stage.p + bytes);
    hipLaunchKernelGGL(export_kv_kernel, dim3((uint32_t)((total + 255) / 256)), dim3(256), 0,
                       cx->stream,
                       reinterpret_cast<const uint16_t*>(kv->slab + kv->k_off[layer]),
                       reinterpret_cast<const uint16_t*>(kv->slab + kv->vt_off[layer]), dk, dv, pos,
                       n_rows, nkv, hd, kv->ctx_pad);
    HIP_TRY(hipGetLastError(), "export launch", layer);
    rc = copy_down_sync(k_f16, dk, bytes);
    if (rc == WR_HIP_OK) rc = copy_down_sync(v_f16, dv, bytes);
    return rc;
}

// ----------------------------------------------------------------- decode --

int wr_hip_attn_decode_batched_dev(uint32_t n, wr_hip_kv* const* kv, uint32_t layer,
                                   const uint32_t* seq_k, const float* q_dev, float* out_dev,
                                   uint32_t nq, float scale_override, uint32_t window)
{
    int rc = check_decode(n, kv, layer, seq_k, q_dev, out_dev, nq);
    if (rc) return rc;
    ENTER();
    return decode_locked(n, kv, layer, seq_k, q_dev, out_dev, nq, scale_override, window);
}

int wr_hip_attn_decode_batched_dev_noalloc(uint32_t n, wr_hip_kv* const* kv, uint32_t layer,
                                           const uint32_t* seq_k, const float* q_dev,
                                           float* out_dev, uint32_t nq, float scale_override,
                                           uint32_t window)
{
    int rc = check_decode(n, kv, layer, seq_k, q_dev, out_dev, nq);
    if (rc) return rc;
    if (nq > kNoAllocMaxHeads) {
        logmsg(0, "decode (no-alloc form): %u query heads exceed the %u the fixed ticket array holds",
               nq, kNoAllocMaxHeads);
        return WR_HIP_ERR_LIMIT;
    }
    // A thread's first call into the library makes its stream and staging
    // buffers (hipStreamCreate, hipMalloc, hipHostMalloc): that call cannot be
    // this one.  Any other entry point (wr_hip_attn_sync is enough) does it.
    if (!t_slot.c || t_slot.generation != g.generation) {
        logmsg(0, "decode (no-alloc form): the calling thread has no stream context yet; "
                  "make one other library call from it first (wr_hip_attn_sync will do)");
        return WR_HIP_ERR_STATE;
    }
    ENTER();
    DecodeWorkspace fixed;
    fixed.ws = g.noalloc_ws[g.device];
    fixed.ticket_bytes = kNoAllocTicketBytes;
    fixed.bytes = kNoAllocScratchBytes;
    if (!fixed.ws) return WR_HIP_ERR_STATE;
    // One array per device, whatever thread calls: this launch waits for the
    // previous one that used it (on whichever stream that was), and leaves its
    // own mark for the next.  Event waits and records allocate nothing.
    std::lock_guard<std::mutex> chain(g.noalloc_mu);
    if (g.noalloc_recorded)
        HIP_TRY(hipStreamWaitEvent(cx->stream, g.noalloc_done, 0), "wait for the scratch array", layer);
    rc = decode_locked(n, kv, layer, seq_k, q_dev, out_dev, nq, scale_override, window, fixed);
    if (hipEventRecord(g.noalloc_done, cx->stream) == hipSuccess) g.noalloc_recorded = true;
    return rc;
}

int wr_hip_attn_append_decode_batched_dev(uint32_t n, wr_hip_kv* const* kv, uint32_t layer,
                                          const uint32_t* pos, const float* qkv_dev, uint32_t ld,
                                          uint32_t nq, const float* q_norm_dev, const float* k_norm_dev,
                                          float eps, const float* cos_sin_dev, uint32_t n_rot,
                                          float* out_dev, float scale_override, uint32_t window)
{
    if (!g.inited) return WR_HIP_ERR_STATE;
    if (!kv || !pos || !qkv_dev || !out_dev) return WR_HIP_ERR_INVAL;
    if (n == 0 || n > WR_HIP_BATCH_MAX) return WR_HIP_ERR_LIMIT;
    for (uint32_t i = 0; i < n; i++) {
        if (!kv[i]) return WR_HIP_ERR_INVAL;
        int rc = check_layer(kv[i], layer);
        if (rc) return rc;
    }
    const uint32_t hd = kv[0]->hd[layer], nkv = kv[0]->nkv;
    if (nq == 0 || nq % nkv != 0) return WR_HIP_ERR_INVAL;
    if ((q_norm_dev == nullptr) != (k_norm_dev == nullptr)) return WR_HIP_ERR_INVAL;
    if (n_rot > hd / 2 || (n_rot > 0 && !cos_sin_dev)) return WR_HIP_ERR_INVAL;
    if ((uint64_t)ld < (uint64_t)(nq + 2 * nkv) * hd) return WR_HIP_ERR_INVAL;
    // What the in-kernel form of the row step takes; for anything else the caller
    // keeps the two separate calls (nothing has been counted or written yet).
    const uintptr_t addrs = (uintptr_t)qkv_dev | (uintptr_t)cos_sin_dev | (uintptr_t)q_norm_dev |
                            (uintptr_t)k_norm_dev;
    if (hd != 128 || !mfma_shape(hd, nq / nkv) || n_rot % 8 != 0 || ld % 4 != 0 || addrs % 16 != 0)
        return WR_HIP_ERR_UNSUPPORTED;
    uint32_t seq_k[WR_HIP_BATCH_MAX];
    for (uint32_t i = 0; i < n; i++) {
        if (pos[i] >= kv[i]->max_ctx) return WR_HIP_ERR_CTX_FULL;          // as the append: nothing is written
        seq_k[i] = pos[i] + 1;
    }
    int rc = check_decode(n, kv, layer, seq_k, qkv_dev, out_dev, nq);      // the attention's own checks, the call counter
    if (rc) return rc;
    DecodeFusedArgs fz;
    memset(&fz, 0, sizeof fz);
    fz.qkv = qkv_dev;
    fz.q_norm = q_norm_dev;
    fz.k_norm = k_norm_dev;
    fz.cos_sin = n_rot ? cos_sin_dev : nullptr;
    fz.ld = ld;
    fz.n_rot = n_rot;
    fz.eps = eps;
    ENTER();
    return decode_locked(n, kv, layer, seq_k, nullptr, out_dev, nq, scale_override, window, DecodeWorkspace(), &fz);
}

int wr_hip_attn_decode_batched(uint32_t n, wr_hip_kv* const* kv, uint32_t layer,
                               const uint32_t* seq_k, const float* const* q, float* const* out,
                               uint32_t nq, float scale_override, uint32_t window)
{
    int rc = check_decode(n, kv, layer, seq_k, q, out, nq);
    if (rc) return rc;
    for (uint32_t i = 0; i < n; i++)
        if (!q[i] || !out[i]) return WR_HIP_ERR_INVAL;
    const size_t row = (size_t)nq * kv[0]->hd[layer] * sizeof(float);
    ENTER();
    rc = ensure_device(cx->d_stage, 2 * n * row);
    if (rc) return rc;
    rc = ensure_pinned(cx->h_pin, n * row);
    if (rc) return rc;
    float* dq = reinterpret_cast<float*>(cx->d_stage.p);
    float* dout = reinterpret_cast<float*>((uint8_t*)cx->d_stage.p + n * row);
    for (uint32_t i = 0; i < n; i++) memcpy((uint8_t*)cx->h_pin.p + i * row, q[i], row);
    HIP_TRY(hipMemcpyAsync(dq, cx->h_pin.p, n * row, hipMemcpyHostToDevice, cx->stream), "q h2d",
            layer);
    rc = decode_locked(n, kv, layer, seq_k, dq, dout, nq, scale_override, window);
    if (rc) return rc;
    HIP_TRY(hipMemcpyAsync(cx->h_pin.p, dout, n * row, hipMemcpyDeviceToHost, cx->stream), "out d2h",
            layer);
    rc = sync_checked("decode sync", layer);
    if (rc) return rc;
    for (uint32_t i = 0; i < n; i++) memcpy(out[i], (uint8_t*)cx->h_pin.p + i * row, row);
    return WR_HIP_OK;
}

int wr_hip_attn_decode(wr_hip_kv* kv, uint32_t layer, uint32_t seq_k, const float* q, float* out,
                       uint32_t nq, float scale_override, uint32_t window)
{
    wr_hip_kv* kvs[1] = {kv};
    const float* qs[1] = {q};
    float* outs[1] = {out};
    if (!kv || !q || !out) return g.inited ? WR_HIP_ERR_INVAL : WR_HIP_ERR_STATE;
    return wr_hip_attn_decode_batched(1, kvs, layer, &seq_k, qs, outs, nq, scale_override, window);
}

int wr_hip_attn_append_decode_batched(uint32_t n, wr_hip_kv* const* kv, uint32_t layer,
                                      const uint32_t* pos, const float* const* k_f32,
                                      const float* const* v_f32, const float* const* q,
                                      float* const* out, uint32_t nq, float scale_override,
                                      uint32_t window)
{
    if (!g.inited) return WR_HIP_ERR_STATE;
    if (!kv || !pos || !k_f32 || !v_f32 || !q || !out) return WR_HIP_ERR_INVAL;
    if (n == 0 || n > WR_HIP_BATCH_MAX) return WR_HIP_ERR_LIMIT;
    for (uint32_t i = 0; i < n; i++) {
        if (!k_f32[i] || !v_f32[i] || !q[i] || !out[i]) return WR_HIP_ERR_INVAL;
        int rc = check_layer(kv[i], layer);
        if (rc) return rc;
    }
    const uint32_t hd = kv[0]->hd[layer], nkv = kv[0]->nkv;
    if (nq == 0 || nq % nkv != 0) return WR_HIP_ERR_INVAL;
    uint32_t seq_k[WR_HIP_BATCH_MAX];
    for (uint32_t i = 0; i < n; i++) {
        if (pos[i] >= kv[i]->max_ctx) return WR_HIP_ERR_CTX_FULL;          // as the append: nothing is written
        seq_k[i] = pos[i] + 1;
    }
    int rc = check_decode(n, kv, layer, seq_k, q, out, nq);
    if (rc) return rc;
    // One staged image, one copy up, the output rows behind it.  For the one-launch
    // kernel session i's rows lie as [nq Q | nkv K | nkv V], the stacked-projection
    // form it reads; for the two-step form the Q rows are packed in front (what the
    // attention reads) and the [K | V] pairs follow.
    const size_t qrow = (size_t)nq * hd, krow = (size_t)nkv * hd;
    const uint32_t ld = (uint32_t)(qrow + 2 * krow);
    const bool one_launch = hd == 128 && mfma_shape(hd, nq / nkv);
    const size_t in_bytes = (size_t)n * ld * sizeof(float), out_bytes = n * qrow * sizeof(float);
    ENTER();
    rc = ensure_device(cx->d_stage, in_bytes + out_bytes);
    if (rc) return rc;
    rc = ensure_pinned(cx->h_pin, in_bytes);
    if (rc) return rc;
    float* din = reinterpret_cast<float*>(cx->d_stage.p);
    float* dout = reinterpret_cast<float*>((uint8_t*)cx->d_stage.p + in_bytes);
    float* pin = reinterpret_cast<float*>(cx->h_pin.p);
    for (uint32_t i = 0; i < n; i++) {
        float* qdst = one_launch ? pin + (size_t)i * ld : pin + (size_t)i * qrow;
        float* kdst = one_launch ? qdst + qrow : pin + (size_t)n * qrow + (size_t)i * 2 * krow;
        memcpy(qdst, q[i], qrow * sizeof(float));
        memcpy(kdst, k_f32[i], krow * sizeof(float));
        memcpy(kdst + krow, v_f32[i], krow * sizeof(float));
    }
    HIP_TRY(hipMemcpyAsync(din, pin, in_bytes, hipMemcpyHostToDevice, cx->stream), "rows h2d", layer);
    if (one_launch) {
        // rows taken as they stand: no norm weights, no rotation
        DecodeFusedArgs fz;
        memset(&fz, 0, sizeof fz);
        fz.qkv = din;
        fz.ld = ld;
        rc = decode_locked(n, kv, layer, seq_k, nullptr, dout, nq, scale_override, window,
                           DecodeWorkspace(), &fz);
    } else {
        // the same two steps as separate launches on the one stream, no wait between them
        const float* dkv = din + (size_t)n * qrow;
        for (uint32_t i = 0; i < n && rc == WR_HIP_OK; i++)
            rc = append_rows_locked<float>(kv[i], layer, pos[i], 1, dkv + (size_t)i * 2 * krow,
                                           dkv + (size_t)i * 2 * krow + krow);
        if (rc == WR_HIP_OK)
            rc = decode_locked(n, kv, layer, seq_k, din, dout, nq, scale_override, window);
    }
    if (rc) return rc;
    HIP_TRY(hipMemcpyAsync(cx->h_pin.p, dout, out_bytes, hipMemcpyDeviceToHost, cx->stream), "out d2h",
            layer);
    rc = sync_checked("append+decode sync", layer);
    if (rc) return rc;
    for (uint32_t i = 0; i < n; i++)
        memcpy(out[i], (uint8_t*)cx->h_pin.p + i * qrow * sizeof(float), qrow * sizeof(float));
    return WR_HIP_OK;
}

int wr_hip_attn_append_decode(wr_hip_kv* kv, uint32_t layer, uint32_t pos, const float* k_f32,
                              const float* v_f32, const float* q, float* out, uint32_t nq,
                              float scale_override, uint32_t window)
{
    wr_hip_kv* kvs[1] = {kv};
    const float* ks[1] = {k_f32};
    const float* vs[1] = {v_f32};
    const float* qs[1] = {q};
    float* outs[1] = {out};
    return wr_hip_attn_append_decode_batched(1, kvs, layer, &pos, ks, vs, qs, outs, nq, scale_override,
                                             window);
}

// ---------------------------------------------------------------- prefill --

int wr_hip_attn_prefill_dev(wr_hip_kv* kv, uint32_t layer, uint32_t p0, uint32_t T,
                            const float* q_dev, float* out_dev, uint32_t nq, float scale_override,
                            uint32_t window)
{
    int rc = check_prefill(kv, layer, p0, T, q_dev, out_dev, nq);
    if (rc) return rc;
    ENTER();
    return prefill_locked(kv, layer, p0, T, q_dev, out_dev, nq, scale_override, window);
}

int wr_hip_attn_prefill_q16_dev(wr_hip_kv* kv, uint32_t layer, uint32_t p0, uint32_t T,
                                const uint16_t* q16_dev, float* out_dev, uint32_t nq, float scale_override,
                                uint32_t window)
{
    int rc = check_prefill(kv, layer, p0, T, q16_dev, out_dev, nq);
    if (rc) return rc;
    if (((uintptr_t)q16_dev & 7) != 0) return WR_HIP_ERR_INVAL;
    ENTER();
    return prefill_locked(kv, layer, p0, T, nullptr, out_dev, nq, scale_override, window, q16_dev);
}

int wr_hip_attn_prefill(wr_hip_kv* kv, uint32_t layer, uint32_t p0, uint32_t T, const float* q,
                        float* out, uint32_t nq, float scale_override, uint32_t window)
{
    int rc = check_prefill(kv, layer, p0, T, q, out, nq);
    if (rc) return rc;
    const size_t bytes = (size_t)T * nq * kv->hd[layer] * sizeof(float);
    ENTER();
    rc = ensure_device(cx->d_stage, 2 * bytes);
    if (rc) return rc;
    float* dq = reinterpret_cast<float*>(cx->d_stage.p);
    float* dout = reinterpret_cast<float*>((uint8_t*)cx->d_stage.p + bytes);
    rc = copy_up(dq, q, bytes, 0);
    if (rc == WR_HIP_OK)
        rc = prefill_locked(kv, layer, p0, T, dq, dout, nq, scale_override, window);
    if (rc == WR_HIP_OK) rc = copy_down_sync(out, dout, bytes);
    return rc;
}

// ------------------------------------------------------- device utilities --

void* wr_hip_attn_dev_alloc(size_t bytes)
{
    if (!g.inited || bytes == 0) return nullptr;
    Entered entered_;
    if (!entered_.ok()) return nullptr;
    void* p = nullptr;
    if (hipMalloc(&p, bytes) != hipSuccess) return nullptr;
    return p;
}

void wr_hip_attn_dev_free(void* p)
{
    if (!g.inited || !p) return;
    Entered entered_;
    if (!entered_.ok()) return;
    (void)hipStreamSynchronize(cx->stream);
    (void)hipFree(p);
}

void* wr_hip_attn_host_alloc(size_t bytes)
{
    if (!g.inited || bytes == 0) return nullptr;
    Entered entered_;
    if (!entered_.ok()) return nullptr;
    void* p = nullptr;
    if (hipHostMalloc(&p, bytes, hipHostMallocDefault) != hipSuccess) return nullptr;
    return p;
}

void wr_hip_attn_host_free(void* p)
{
    if (!g.inited || !p) return;
    Entered entered_;
    if (!entered_.ok()) return;
    (void)hipStreamSynchronize(cx->stream);
    (void)hipHostFree(p);
}

int wr_hip_attn_h2d(void* dst_dev, const void* src_host, size_t bytes)
{
    if (!g.inited) return WR_HIP_ERR_STATE;
    if (!dst_dev || !src_host) return WR_HIP_ERR_INVAL;
    ENTER();
    HIP_TRY(hipMemcpyAsync(dst_dev, src_host, bytes, hipMemcpyHostToDevice, cx->stream), "h2d", 0);
    HIP_TRY(hipStreamSynchronize(cx->stream), "h2d sync", 0);
    return WR_HIP_OK;
}

int wr_hip_attn_d2h(void* dst_host, const void* src_dev, size_t bytes)
{
    if (!g.inited) return WR_HIP_ERR_STATE;
    if (!dst_host || !src_dev) return WR_HIP_ERR_INVAL;
    ENTER();
    HIP_TRY(hipMemcpyAsync(dst_host, src_dev, bytes, hipMemcpyDeviceToHost, cx->stream), "d2h", 0);
    return sync_checked("d2h sync", 0);
}

int wr_hip_attn_sync(void)
{
    if (!g.inited) return WR_HIP_ERR_STATE;
    ENTER();
    return sync_checked("sync", 0);
}

void* wr_hip_attn_stream(void)
{
    Entered entered_;
    return entered_.ok() ? (void*)cx->stream : nullptr;
}

// ------------------------------------------------------------ projections --

int wr_hip_proj_weight_create(uint32_t n_parts, const uint16_t* const* parts_f16,
                              const uint32_t* rows_per_part, uint32_t n_in, wr_hip_weight** out)
{
    if (!out) return WR_HIP_ERR_INVAL;
    *out = nullptr;
    if (!g.inited) return WR_HIP_ERR_STATE;
    if (n_parts == 0 || !parts_f16 || !rows_per_part || n_in == 0 || n_in % 32 != 0)
        return WR_HIP_ERR_INVAL;
    uint64_t n_out = 0;
    for (uint32_t i = 0; i < n_parts; i++) {
        if (!parts_f16[i] || rows_per_part[i] == 0) return WR_HIP_ERR_INVAL;
        n_out += rows_per_part[i];
    }
    if (n_out % 16 != 0 || n_out > 0x7FFFFFFFu) return WR_HIP_ERR_INVAL;
    wr_hip_weight* w = new (std::nothrow) wr_hip_weight();
    if (!w) return WR_HIP_ERR_NOMEM;
    w->n_out = (uint32_t)n_out;
    w->n_in = n_in;
    w->bytes = (size_t)n_out * n_in * 2;
    w->tiles = nullptr;

    ENTER();
    void* rowmajor = nullptr;
    hipError_t e = hipMalloc(&w->tiles, w->bytes);
    if (e == hipSuccess) e = hipMalloc(&rowmajor, w->bytes);
    if (e != hipSuccess) {
        logmsg(0, "projection: device weight alloc failed (%zu bytes): %s", w->bytes,
               hipGetErrorString(e));
        if (w->tiles) (void)hipFree(w->tiles);
        delete w;
        return WR_HIP_ERR_NOMEM;
    }
    size_t off = 0;
    for (uint32_t i = 0; i < n_parts && e == hipSuccess; i++) {
        const size_t nb = (size_t)rows_per_part[i] * n_in * 2;
        e = hipMemcpyAsync((uint8_t*)rowmajor + off, parts_f16[i], nb, hipMemcpyHostToDevice, cx->stream);
        if (e == hipSuccess) e = hipStreamSynchronize(cx->stream);     // pageable source
        off += nb;
    }
    if (e == hipSuccess) {
        const size_t units = w->bytes / 16;
        hipLaunchKernelGGL(proj_pack_weights_kernel, dim3((uint32_t)((units + 255) / 256)), dim3(256),
                           0, cx->stream, reinterpret_cast<const uint16_t*>(rowmajor),
                           reinterpret_cast<u32x4*>(w->tiles), w->n_out, w->n_in);
        e = hipGetLastError();
        if (e == hipSuccess) e = hipStreamSynchronize(cx->stream);
    }
    (void)hipFree(rowmajor);
    if (e != hipSuccess) {
        (void)hipFree(w->tiles);
        delete w;
        return hip_fail(e, "weight upload", 0);
    }
    *out = w;
    return WR_HIP_OK;
}

void wr_hip_proj_weight_destroy(wr_hip_weight* w)
{
    if (!w) return;
    if (g.inited) {
        Entered entered_;
        if (entered_.ok()) (void)hipStreamSynchronize(cx->stream);
        (void)hipFree(w->tiles);
    }
    delete w;
}

static int check_proj(const wr_hip_weight* w, uint32_t rows, const void* x, uint32_t ldx,
                      uint32_t min_ldx, const void* y, uint32_t ldy)
{
    if (!g.inited) return WR_HIP_ERR_STATE;
    if (!w || !x || !y) return WR_HIP_ERR_INVAL;
    if (rows == 0) return WR_HIP_OK;
    if (ldx < min_ldx || ldy < w->n_out || ldy % 4 != 0) return WR_HIP_ERR_INVAL;
    return WR_HIP_OK;
}

static int proj_dev_common(const wr_hip_weight* w, uint32_t rows, const float* x_dev, uint32_t ldx,
                           uint32_t min_ldx, const ProjSource& src, const float* add_dev,
                           float* y_dev, uint32_t ldy)
{
    int rc = check_proj(w, rows, x_dev, ldx, min_ldx, y_dev, ldy);
    if (rc || rows == 0) return rc;
    if (((uintptr_t)y_dev & 15) || (add_dev && ((uintptr_t)add_dev & 15))) return WR_HIP_ERR_INVAL;
    ENTER();
    return proj_locked(w, rows, x_dev, ldx, src, add_dev, y_dev, ldy);
}

int wr_hip_proj_rows_dev(const wr_hip_weight* w, uint32_t rows, const float* x_dev, uint32_t ldx,
                         const float* add_dev, float* y_dev, uint32_t ldy)
{
    return proj_dev_common(w, rows, x_dev, ldx, w ? w->n_in : 0, ProjSource(), add_dev, y_dev, ldy);
}

int wr_hip_proj_rows_norm_dev(const wr_hip_weight* w, uint32_t rows, const float* x_dev,
                              uint32_t ldx, const float* norm_w_dev, float eps,
                              const float* add_dev, float* y_dev, uint32_t ldy)
{
    if (g.inited && !norm_w_dev) return WR_HIP_ERR_INVAL;
    ProjSource src;
    src.kind = kProjSrcRmsNorm;
    src.norm_w = norm_w_dev;
    src.eps = eps;
    return proj_dev_common(w, rows, x_dev, ldx, w ? w->n_in : 0, src, add_dev, y_dev, ldy);
}

int wr_hip_proj_rows_swiglu_dev(const wr_hip_weight* w, uint32_t rows, const float* gate_up_dev,
                                uint32_t ld, const float* add_dev, float* y_dev, uint32_t ldy)
{
    ProjSource src;
    src.kind = kProjSrcSwiglu;
    return proj_dev_common(w, rows, gate_up_dev, ld, w ? 2 * w->n_in : 0, src, add_dev, y_dev, ldy);
}

int wr_hip_proj_rows_geglu_dev(const wr_hip_weight* w, uint32_t rows, const float* gate_up_dev,
                               uint32_t ld, const float* add_dev, float* y_dev, uint32_t ldy)
{
    ProjSource src;
    src.kind = kProjSrcGeglu;
    return proj_dev_common(w, rows, gate_up_dev, ld, w ? 2 * w->n_in : 0, src, add_dev, y_dev, ldy);
}

int wr_hip_proj_rows(const wr_hip_weight* w, uint32_t rows, const float* x, float* y)
{
    if (w && (w->n_out % 4 != 0)) return WR_HIP_ERR_INVAL;
    int rc = check_proj(w, rows, x, w ? w->n_in : 0, w ? w->n_in : 0, y, w ? w->n_out : 0);
    if (rc || rows == 0) return rc;
    const size_t xb = ((size_t)rows * w->n_in * sizeof(float) + 255) & ~(size_t)255;
    const size_t yb = (size_t)rows * w->n_out * sizeof(float);
    ENTER();
    rc = ensure_device(cx->d_stage, xb + yb);
    if (rc) return rc;
    float* dx = reinterpret_cast<float*>(cx->d_stage.p);
    float* dy = reinterpret_cast<float*>((uint8_t*)cx->d_stage.p + xb);
    rc = copy_up(dx, x, (size_t)rows * w->n_in * sizeof(float), 0);
    if (rc == WR_HIP_OK) rc = proj_locked(w, rows, dx, w->n_in, ProjSource(), nullptr, dy, w->n_out);
    if (rc == WR_HIP_OK) rc = copy_down_sync(y, dy, yb);
    return rc;
}

// ------------------------------------------------------------- row steps --

int wr_hip_rows_rmsnorm_dev(const float* x_dev, uint32_t ldx, const float* w_dev, uint32_t wn,
                            float* out_dev, uint32_t ldo, uint32_t rows, uint32_t dim, float eps)
{
    if (!g.inited) return WR_HIP_ERR_STATE;
    if (!x_dev || !out_dev || dim == 0 || ldx < dim || ldo < dim) return WR_HIP_ERR_INVAL;
    if (wn > 0 && !w_dev) return WR_HIP_ERR_INVAL;
    if (rows == 0) return WR_HIP_OK;
    ENTER();
    hipLaunchKernelGGL(rmsnorm_rows_kernel, dim3(rows), dim3(256), 0, cx->stream, x_dev, ldx, w_dev, wn,
                       out_dev, ldo, dim, eps, 0);
    HIP_TRY(hipGetLastError(), "rmsnorm launch", 0);
    return WR_HIP_OK;
}

int wr_hip_rows_rmsnorm_add_dev(const float* x_dev, uint32_t ldx, const float* w_dev, uint32_t wn,
                                float* acc_dev, uint32_t lda, uint32_t rows, uint32_t dim, float eps)
{
    if (!g.inited) return WR_HIP_ERR_STATE;
    if (!x_dev || !acc_dev || dim == 0 || ldx < dim || lda < dim) return WR_HIP_ERR_INVAL;
    if (wn > 0 && !w_dev) return WR_HIP_ERR_INVAL;
    if (rows == 0) return WR_HIP_OK;
    ENTER();
    hipLaunchKernelGGL(rmsnorm_rows_kernel, dim3(rows), dim3(256), 0, cx->stream, x_dev, ldx, w_dev, wn,
                       acc_dev, lda, dim, eps, 1);
    HIP_TRY(hipGetLastError(), "rmsnorm + add launch", 0);
    return WR_HIP_OK;
}

int wr_hip_rows_qkv_prep_dev(const float* qkv_dev, uint32_t ld, uint32_t rows, uint32_t nq,
                             uint32_t nkv, uint32_t hd, const float* q_norm_dev,
                             const float* k_norm_dev, float eps, const float* cos_sin_dev,
                             uint32_t n_rot, float* q_out_dev, float* k_out_dev, float* v_out_dev)
{
    if (!g.inited) return WR_HIP_ERR_STATE;
    if (!qkv_dev || !q_out_dev || !k_out_dev || !v_out_dev) return WR_HIP_ERR_INVAL;
    if (nq == 0 || nkv == 0 || hd < 2 || (hd & 1) || hd > (uint32_t)kRowsMaxHd) return WR_HIP_ERR_INVAL;
    if ((uint64_t)ld < (uint64_t)(nq + 2 * nkv) * hd) return WR_HIP_ERR_INVAL;
    if (n_rot > hd / 2 || (n_rot > 0 && !cos_sin_dev)) return WR_HIP_ERR_INVAL;
    if ((q_norm_dev == nullptr) != (k_norm_dev == nullptr)) return WR_HIP_ERR_INVAL;
    if (rows == 0) return WR_HIP_OK;
    QkvPrepArgs a;
    a.qkv = qkv_dev;
    a.q_norm = q_norm_dev;
    a.k_norm = k_norm_dev;
    a.cos_sin = cos_sin_dev;
    a.q_out = q_out_dev;
    a.k_out = k_out_dev;
    a.v_out = v_out_dev;
    a.ld = ld;
    a.nq = nq;
    a.nkv = nkv;
    a.hd = hd;
    a.n_rot = n_rot;
    a.eps = eps;
    ENTER();
    hipLaunchKernelGGL(qkv_prep_kernel, dim3(rows, nq + 2 * nkv), dim3(64), 0, cx->stream, a);
    HIP_TRY(hipGetLastError(), "qkv prep launch", 0);
    return WR_HIP_OK;
}

// q16_out_dev != nullptr: Q leaves as binary16 rows multiplied by the softmax
// scale times log2(e) (what wr_hip_attn_prefill_q16_dev takes) instead of F32.
static int qkv_append_common(const float* qkv_dev, uint32_t ld, uint32_t rows, uint32_t nq,
                             const float* q_norm_dev, const float* k_norm_dev, float eps,
                             const float* cos_sin_dev, uint32_t n_rot, uint32_t n_kv,
                             wr_hip_kv* const* kv, uint32_t layer, const uint32_t* pos,
                             float* q_out_dev, uint16_t* q16_out_dev, float scale_override, uint32_t flags)
{
    if (!g.inited) return WR_HIP_ERR_STATE;
    if (!qkv_dev || (!q_out_dev && !q16_out_dev) || !kv || !pos || nq == 0) return WR_HIP_ERR_INVAL;
    if (flags & ~(uint32_t)(WR_HIP_QKV_V_NORM | WR_HIP_QKV_Q_ONLY)) return WR_HIP_ERR_INVAL;
    const bool q_only = (flags & WR_HIP_QKV_Q_ONLY) != 0;
    if (n_kv == 0 || (n_kv != 1 && n_kv != rows)) return WR_HIP_ERR_INVAL;
    if (n_kv > WR_HIP_BATCH_MAX) return WR_HIP_ERR_LIMIT;
    QkvAppendArgs a;
    memset(&a, 0, sizeof a);
    for (uint32_t i = 0; i < n_kv; i++) {
        int rc = check_layer(kv[i], layer);
        if (rc) return rc;
        if (kv[i]->nkv != kv[0]->nkv || kv[i]->hd[layer] != kv[0]->hd[layer]) return WR_HIP_ERR_INVAL;
        for (uint32_t j = 0; j < i; j++)
            if (kv[i] == kv[j]) return WR_HIP_ERR_INVAL;
        const uint64_t end = (uint64_t)pos[i] + (n_kv == 1 ? rows : 1);
        if (!q_only && end > kv[i]->max_ctx) return WR_HIP_ERR_CTX_FULL;   // nothing is written
        a.k[i] = reinterpret_cast<uint16_t*>(kv[i]->slab + kv[i]->k_off[layer]);
        a.vt[i] = reinterpret_cast<uint16_t*>(kv[i]->slab + kv[i]->vt_off[layer]);
        a.pos[i] = pos[i];
        a.ctx_pad[i] = kv[i]->ctx_pad;
    }
    const uint32_t nkv = kv[0]->nkv, hd = kv[0]->hd[layer];
    if (hd < 2 || (hd & 1)) return WR_HIP_ERR_INVAL;
    if (hd > 512) return WR_HIP_ERR_LIMIT;                // the V block gathered in LDS: hd * 68 bytes
    if ((uint64_t)ld < (uint64_t)(nq + (q_only ? 0 : 2 * nkv)) * hd) return WR_HIP_ERR_INVAL;
    if (n_rot > hd / 2 || (n_rot > 0 && !cos_sin_dev)) return WR_HIP_ERR_INVAL;
    if (!q_only && (q_norm_dev == nullptr) != (k_norm_dev == nullptr)) return WR_HIP_ERR_INVAL;
    if (rows == 0) return WR_HIP_OK;
    a.v_norm = (flags & WR_HIP_QKV_V_NORM) ? 1 : 0;
    a.qkv = qkv_dev;
    a.q_norm = q_norm_dev;
    a.k_norm = k_norm_dev;
    a.cos_sin = n_rot ? cos_sin_dev : nullptr;           // a table of zero pairs per row holds nothing to read
    a.q_out = q_out_dev;
    a.ld = ld;
    a.nq = nq;
    a.nkv = nkv;
    a.hd = hd;
    a.n_rot = n_rot;
    a.rows = rows;
    a.per_session = (n_kv > 1 || rows == 1) ? 1 : 0;
    a.eps = eps;
    {
        // eight lanes per position with 16-byte accesses where the shapes and
        // the addresses allow it (every model on the device walk does)
        const uintptr_t addrs = (uintptr_t)qkv_dev | (uintptr_t)q_out_dev | (uintptr_t)q16_out_dev |
                                (uintptr_t)cos_sin_dev | (uintptr_t)q_norm_dev | (uintptr_t)k_norm_dev;
        if ((hd == 128 || hd == 256) && n_rot % 8 == 0 && ld % 4 == 0 && addrs % 16 == 0) a.row8 = hd / 64;
    }
    if (q16_out_dev) {
        // only the eight-lane form writes it, and only the 128-wide head has a
        // prefill kernel that reads it
        if (a.row8 != 2) return WR_HIP_ERR_UNSUPPORTED;
        const float scale = (scale_override > 0.0f) ? scale_override : 1.0f / sqrtf((float)hd);
        a.q16_out = q16_out_dev;
        a.q16_scale = scale * kLog2e;                     // prefill_locked's qscale, by the same expression
    }
    const uint32_t gx = a.per_session ? rows : (pos[0] + rows - 1) / kVBlock - pos[0] / kVBlock + 1;
    const size_t lds = std::max((size_t)4 * hd * sizeof(float), (size_t)hd * (kVBlock + 2) * sizeof(uint16_t));
    ENTER();
    hipLaunchKernelGGL(qkv_append_kernel, dim3(gx, nq + (q_only ? 0 : 2 * nkv)), dim3(256), lds, cx->stream, a);
    HIP_TRY(hipGetLastError(), "qkv append launch", layer);
    return WR_HIP_OK;
}

int wr_hip_rows_qkv_append_dev(const float* qkv_dev, uint32_t ld, uint32_t rows, uint32_t nq,
                               const float* q_norm_dev, const float* k_norm_dev, float eps,
                               const float* cos_sin_dev, uint32_t n_rot, uint32_t n_kv,
                               wr_hip_kv* const* kv, uint32_t layer, const uint32_t* pos,
                               float* q_out_dev, uint32_t flags)
{
    if (!q_out_dev) return g.inited ? WR_HIP_ERR_INVAL : WR_HIP_ERR_STATE;
    return qkv_append_common(qkv_dev, ld, rows, nq, q_norm_dev, k_norm_dev, eps, cos_sin_dev, n_rot, n_kv, kv,
                             layer, pos, q_out_dev, nullptr, 0.0f, flags);
}

int wr_hip_rows_qkv_append_q16_dev(const float* qkv_dev, uint32_t ld, uint32_t rows, uint32_t nq,
                                   const float* q_norm_dev, const float* k_norm_dev, float eps,
                                   const float* cos_sin_dev, uint32_t n_rot, uint32_t n_kv,
                                   wr_hip_kv* const* kv, uint32_t layer, const uint32_t* pos,
                                   uint16_t* q16_out_dev, float scale_override, uint32_t flags)
{
    if (!q16_out_dev) return g.inited ? WR_HIP_ERR_INVAL : WR_HIP_ERR_STATE;
    return qkv_append_common(qkv_dev, ld, rows, nq, q_norm_dev, k_norm_dev, eps, cos_sin_dev, n_rot, n_kv, kv,
                             layer, pos, nullptr, q16_out_dev, scale_override, flags);
}

int wr_hip_rows_swiglu_dev(const float* gate_up_dev, uint32_t ld, float* act_dev, uint32_t ldo,
                           uint32_t rows, uint32_t ffn)
{
    if (!g.inited) return WR_HIP_ERR_STATE;
    if (!gate_up_dev || !act_dev || ffn == 0 || (uint64_t)ld < 2ull * ffn || ldo < ffn)
        return WR_HIP_ERR_INVAL;
    if (rows == 0) return WR_HIP_OK;
    ENTER();
    const size_t total = (size_t)rows * ffn;
    hipLaunchKernelGGL(swiglu_rows_kernel, dim3((uint32_t)((total + 255) / 256)), dim3(256), 0,
                       cx->stream, gate_up_dev, ld, act_dev, ldo, rows, ffn);
    HIP_TRY(hipGetLastError(), "swiglu launch", 0);
    return WR_HIP_OK;
}

uint32_t wr_hip_proj_weight_rows(const wr_hip_weight* w) { return w ? w->n_out : 0; }
uint32_t wr_hip_proj_weight_cols(const wr_hip_weight* w) { return w ? w->n_in : 0; }

int wr_hip_attn_profile_begin(uint32_t max_launches)
{
    if (!g.inited) return WR_HIP_ERR_STATE;
    ENTER();
    HIP_TRY(hipStreamSynchronize(cx->stream), "sync", 0);
    while (cx->ev.size() < 2 * (size_t)max_launches) {
        hipEvent_t e;
        HIP_TRY(hipEventCreate(&e), "event create", 0);
        cx->ev.push_back(e);
    }
    cx->ev_used = 0;
    cx->profiling = true;
    return WR_HIP_OK;
}

int wr_hip_attn_profile_end(double* total_ms, uint32_t* n_launches)
{
    if (!g.inited) return WR_HIP_ERR_STATE;
    ENTER();
    HIP_TRY(hipStreamSynchronize(cx->stream), "sync", 0);
    double sum = 0.0;
    for (uint32_t i = 0; i + 1 < cx->ev_used; i += 2) {
        float ms = 0.f;
        HIP_TRY(hipEventElapsedTime(&ms, cx->ev[i], cx->ev[i + 1]), "event elapsed", 0);
        sum += ms;
    }
    if (total_ms) *total_ms = sum;
    if (n_launches) *n_launches = cx->ev_used / 2;
    cx->profiling = false;
    cx->ev_used = 0;
    return WR_HIP_OK;
}

}  // extern "C"
