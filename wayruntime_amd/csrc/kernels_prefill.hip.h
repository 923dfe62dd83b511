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

}  // namespace wr
