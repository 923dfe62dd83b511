/*
 * wr_oracle.h — CPU oracle for the GQA attention path.  TEST INFRASTRUCTURE.
 *
 * A plain-C restatement of the reference algorithm, written so that its
 * output is bit-identical to the compiled reference (same loop order, same
 * constants, same sentinels).  Nothing in the shipped library links, loads
 * or calls this; only the tests, the smoke check and the CPU-baseline leg of
 * the benchmark do, and only as the checker.
 *
 * Every function names the reference range it follows (paths relative to the
 * reference tree).  Build with -O3 -ffp-contract=off and WITHOUT -ffast-math
 * or -march flags that enable FMA contraction: bit parity depends on the
 * scalar F32 multiply-then-add sequence.
 *
 * Pinning status of each function (what fixes its behaviour besides this
 * text) is listed next to it; there is no "parity unpinned" function here.
 */
#ifndef WR_ORACLE_H
#define WR_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Status values, numerically equal to the reference's wr_status
 * (include/wayruntime/wayruntime.h:82-107). */
enum {
    WRO_OK           = 0,
    WRO_ERR_INVAL    = -4,
    WRO_ERR_NOMEM    = -5,
    WRO_ERR_CTX_FULL = -6,
    WRO_ERR_LIMIT    = -8,
    WRO_ERR_INTERNAL = -10
};

/* Limits (src/core/internal.h:186-197).  The sequence cap is a run-time
 * value here so one build serves both the default 4096 and the 32768
 * configuration. */
#define WRO_FLASH_BLOCK 64
#define WRO_FLASH_D_MAX 1024
void     wro_set_attn_max_seq(uint32_t cap);
uint32_t wro_get_attn_max_seq(void);

/* ---- scalar math: src/core/mathx.c:37-57, 72-86, 98-110, 124-147 --------
 * pinned by: bit-compare against the compiled reference on dense grids
 * (tests/golden/mathx_*.bin), closed forms to ~1e-5. */
float wro_exp(float x);
float wro_log(float x);
float wro_sqrt(float x);
float wro_sin(float x);
float wro_cos(float x);

/* ---- F16 codecs: src/core/quant.c:86-136 --------------------------------
 * pinned by: known answers test/unit_tests.c:100-107, exhaustive round trip
 * over all 65536 patterns, bit-compare against the compiled reference. */
float    wro_f16_to_f32(uint16_t h);
uint16_t wro_f32_to_f16(float f);          /* TRUNCATING */

/* ---- tensor descriptor subset: src/core/internal.h:105-132 -------------- */
#define WRO_DTYPE_F32 0
#define WRO_DTYPE_F16 1
#define WRO_TENSOR_GROWABLE (1u << 1)

typedef struct wro_tensor {
    void    *data;
    uint64_t size_bytes;
    uint32_t shape[8];
    uint8_t  ndim;
    uint8_t  dtype;          /* WRO_DTYPE_F32 or WRO_DTYPE_F16 */
    uint16_t flags;
    uint32_t valid_rows;
} wro_tensor;

/* Convenience initialiser: contiguous tensor over caller memory. */
void wro_tensor_wrap(wro_tensor *t, void *data, uint8_t dtype, uint8_t ndim,
                     const uint32_t *shape, uint16_t flags);

/* src/core/tensor.c:124-134 */
int wro_tensor_set_valid_rows(wro_tensor *t, uint32_t new_rows);

/* ---- attention: src/core/kernels.c:1414-1527 ----------------------------
 * Error contract kernels.c:1418-1454.  calls_counter, when non-NULL, is
 * bumped exactly where the reference bumps WR_CTR_ATTENTION_CALLS
 * (kernels.c:1423: after the NULL/ndim checks, before the shape checks).
 * pinned by: golden outputs of the compiled reference (tests/golden),
 * the reference's own self-test fixtures (kernels.c:1907-2062, 2185-2208),
 * materialised softmax in double precision, invariants. */
int wro_op_gqa_attention(const wro_tensor *Q, const wro_tensor *K,
                         const wro_tensor *V, wro_tensor *C,
                         float scale_override, uint32_t window,
                         uint64_t *calls_counter);

/* Raw-pointer form of the same loop nest for seq_q query rows over
 * seq_k cached positions; K/V are F16 [seq_k, nkv, hd] position-major.
 * No argument checking beyond what the loop needs. */
void wro_attention_f16kv(const float *q, const uint16_t *k, const uint16_t *v,
                         float *out, uint32_t seq_q, uint32_t nq, uint32_t nkv,
                         uint32_t hd, uint32_t seq_k, float scale_override,
                         uint32_t window);

/* ---- KV append: src/core/session.c:139-154 ------------------------------
 * kv must be an F16 GROWABLE tensor [max_ctx, nkv, hd]; row is nkv*hd F32.
 * pinned by: codec pins above + cursor behaviour of the llm_step fixture
 * (session.c:946-985). */
int wro_kv_append_row(wro_tensor *kv, const float *row, uint32_t nkv,
                      uint32_t hd);

/* ---- causal prefill: loop of seq_q = 1 calls, src/core/session.c:615-625 --
 * The cache already holds rows 0 .. p0+T-1 (truncated F16).  Row i of q
 * attends keys 0 .. p0+i.  window has the per-call meaning of the reference:
 * the last `window` keys visible to that row.
 * pinned by: definition (row i == decode call at seq_k = p0+i+1). */
void wro_causal_prefill(const float *q, const uint16_t *k, const uint16_t *v,
                        float *out, uint32_t p0, uint32_t T, uint32_t nq,
                        uint32_t nkv, uint32_t hd, float scale_override,
                        uint32_t window);
/* Same, rows [row_lo, row_hi) only (so a caller may spread rows over
 * threads or check a sample of rows). */
void wro_causal_prefill_rows(const float *q, const uint16_t *k,
                             const uint16_t *v, float *out, uint32_t p0,
                             uint32_t row_lo, uint32_t row_hi, uint32_t nq,
                             uint32_t nkv, uint32_t hd, float scale_override,
                             uint32_t window);

/* ---- batched decode: loop of independent calls, src/core/batch.c:156-164 -- */
void wro_batched_decode(uint32_t n, const float *const *q,
                        const uint16_t *const *k, const uint16_t *const *v,
                        float *const *out, const uint32_t *seq_k, uint32_t nq,
                        uint32_t nkv, uint32_t hd, float scale_override,
                        uint32_t window);

/* ---- RoPE: src/core/kernels.c:1356-1412 ---------------------------------
 * x is [seq, heads, hd] F32, rotated in place; first row is at `pos`.
 * pinned by: bit-compare against the compiled reference; ops_test_rope
 * known answers (kernels.c:2160-2183). */
int wro_rope_table(float *out, uint32_t seq, uint32_t hd, uint32_t pos,
                   float theta_base, uint32_t n_rot_pairs);
int wro_rope(float *x, uint32_t seq, uint32_t heads, uint32_t hd,
             uint32_t pos, float theta_base, uint32_t n_rot_pairs);

/* y[M][N] = a[M][K] . W[N][K]^T, W given as F16 bit patterns and widened to
 * F32 first; scalar summation order (src/core/kernels.c:124-137). */
int wro_matmul_w16(const float *a, const uint16_t *w_f16, float *c, uint32_t M,
                   uint32_t K, uint32_t N);

/* src/core/kernels.c:1276-1316 */
int wro_rmsnorm(const float *x, const float *w, uint32_t wn, float *out,
                uint32_t rows, uint32_t dim, float eps);

/* src/core/kernels.c:1243-1258, 963-967 */
int wro_silu_mul(const float *g, const float *u, float *out, uint64_t n);

#ifdef __cplusplus
}
#endif
#endif /* WR_ORACLE_H */
