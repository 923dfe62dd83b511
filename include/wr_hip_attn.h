/*
 * wr_hip_attn.h — C ABI of the MI355X (gfx950) attention path.
 *
 * A C11 host engine calls these in place of the reference's CPU attention
 * op, its KV append and its KV storage.  Plain C linkage, plain pointers and
 * sizes, int returns; no C++ or framework types cross this boundary.
 *
 * Each entry point names the reference interface it replaces (paths relative
 * to the reference tree).
 *
 * Conventions (reference: include/wayruntime/wayruntime.h:82-107):
 *   - return 0 (WR_OK) on success, a negative wr_status value on failure;
 *   - nothing is ever truncated or clamped: a sequence above the cap is
 *     WR_HIP_ERR_LIMIT, a full cache is WR_HIP_ERR_CTX_FULL;
 *   - a failed call leaves cache contents below the caller's cursor intact.
 *     The cursor itself (how many rows are valid) is owned by the caller, as
 *     the reference keeps it in the session (src/core/session.c:160-168):
 *     rollback is "reset the cursor"; rows above it are never read;
 *   - host-pointer entry points are synchronous: results are in the caller's
 *     buffer on return.  `_dev` entry points take device pointers, enqueue on
 *     the calling thread's stream and return without waiting;
 *   - thread safety: calls on DIFFERENT wr_hip_kv objects may run concurrently
 *     from different threads (reference threading contract,
 *     include/wayruntime/wayruntime.h:29-40); calls on one object must be
 *     serialised by the caller (the session lock does that);
 *   - streams: every calling thread has a stream of its own in the library
 *     (made on the thread's first call, handed on to a later thread when the
 *     thread ends), with its own staging, split-K tickets and partial rows, so
 *     work submitted from different threads overlaps on the device.  "The
 *     stream" below is always the calling thread's: `_dev` calls made by one
 *     thread run in the order made, wr_hip_attn_sync and the synchronous
 *     entry points wait for the calling thread's work only.  Device memory
 *     written by one thread's `_dev` calls may be used from another thread
 *     once the first has waited (wr_hip_attn_sync or any synchronous call).
 */
#ifndef WR_HIP_ATTN_H
#define WR_HIP_ATTN_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* wr_status values used on this path (wayruntime.h:82-107). */
#define WR_HIP_OK               0
#define WR_HIP_ERR_UNSUPPORTED (-3)
#define WR_HIP_ERR_INVAL       (-4)
#define WR_HIP_ERR_NOMEM       (-5)
#define WR_HIP_ERR_CTX_FULL    (-6)
#define WR_HIP_ERR_STATE       (-7)
#define WR_HIP_ERR_LIMIT       (-8)
#define WR_HIP_ERR_INTERNAL    (-10)

/* Limits.  WR_HIP_ATTN_MAX_SEQ plays the role of WR_ATTN_MAX_SEQ
 * (src/core/internal.h:186-193) raised for the long-context workloads;
 * WR_HIP_BATCH_MAX == WR_BATCH_MAX (wayruntime.h:423);
 * WR_HIP_FLASH_D_MAX == WR_FLASH_D_MAX (internal.h:197). */
#define WR_HIP_ATTN_MAX_SEQ   131072u
#define WR_HIP_BATCH_MAX      16u
#define WR_HIP_FLASH_D_MAX    1024u
#define WR_HIP_MAX_LAYERS     64u        /* WR_MAX_LAYERS, internal.h:184 */

/* Per-session device KV cache (opaque). */
typedef struct wr_hip_kv wr_hip_kv;

/* Log sink with the signature of wr_log_fn (wayruntime.h:126-130); device
 * errors are reported through it like session.c:170-174 reports op failures. */
typedef void (*wr_hip_log_fn)(int level, const char *msg, void *user);

/* ---- lifecycle ----------------------------------------------------------
 * Replaces: nothing on the CPU path; attaches where the engine is created and
 * destroyed (src/core/engine.c:119-178, 180).  One init per process; a second
 * init without shutdown returns WR_HIP_ERR_STATE (single engine per process,
 * engine.c:125-129).  Fails with WR_HIP_ERR_UNSUPPORTED when no gfx950 device
 * is present: there is no CPU fallback. */
int  wr_hip_attn_init(int device);
void wr_hip_attn_shutdown(void);
void wr_hip_attn_set_log(wr_hip_log_fn fn, void *user);
/* Number of attention calls issued, one per session-layer, the quantity the
 * reference counts in WR_CTR_ATTENTION_CALLS (src/core/kernels.c:1423). */
uint64_t wr_hip_attn_calls(void);
/* "gfx950 ..." description of the device in use (static storage). */
const char *wr_hip_attn_device_name(void);

/* ---- KV storage ---------------------------------------------------------
 * Replaces the KV half of session_build / wr_map_alloc / wr_map_free
 * (src/core/session.c:640-674, 775, 811): one device allocation per session,
 * made once, never grown.  Layers whose hd_per_layer entry is 0 get no
 * storage (KV-shared layers alias another layer, session.c:652-658; pass the
 * source layer's index to the other calls).  Allocation failure is
 * WR_HIP_ERR_NOMEM; max_ctx above the cap is WR_HIP_ERR_LIMIT
 * (session.c:755). */
int  wr_hip_attn_kv_create(uint32_t n_layers, const uint32_t *hd_per_layer,
                           uint32_t nkv, uint32_t max_ctx, wr_hip_kv **out);
void wr_hip_attn_kv_destroy(wr_hip_kv *kv);
uint64_t wr_hip_attn_kv_bytes(const wr_hip_kv *kv);

/* ---- append -------------------------------------------------------------
 * Replaces kv_append_row (src/core/session.c:139-154) for n_rows consecutive
 * positions: k_f32 / v_f32 are host F32 [n_rows, nkv, hd_layer]; the rows are
 * copied up and converted on the device with the reference's TRUNCATING
 * F32->F16 rule (src/core/quant.c:121-136) into rows pos .. pos+n_rows-1.
 * pos + n_rows > max_ctx is WR_HIP_ERR_CTX_FULL and writes nothing. */
int wr_hip_attn_append(wr_hip_kv *kv, uint32_t layer, uint32_t pos,
                       uint32_t n_rows, const float *k_f32,
                       const float *v_f32);

/* Append with the rotary embedding of the K rows done on the device (the step
 * the reference performs on the host right before kv_append_row:
 * wri_op_rope, src/core/kernels.c:1356-1412, called at session.c:477-478).
 * k_f32 holds the rows BEFORE rotation; cos_sin is host F32
 * [n_rows, n_rot, 2] = (cos, sin) of each row's angles, n_rot <= hd/2 pairs
 * rotated (element j with element j + hd/2).  The rotated rows are bit
 * identical to the reference's, so the cache is too.  v_f32 as in append. */
int wr_hip_attn_append_rope(wr_hip_kv *kv, uint32_t layer, uint32_t pos,
                            uint32_t n_rows, const float *k_f32,
                            const float *v_f32, const float *cos_sin,
                            uint32_t n_rot);

/* Test / tooling access to the cache in the reference's layout: F16 bit
 * patterns, position-major [n_rows, nkv, hd_layer] (the layout of the
 * reference's kv_k / kv_v tensors, src/core/internal.h:492-497).
 * kv_write stores already-converted rows verbatim. */
int wr_hip_attn_kv_read(wr_hip_kv *kv, uint32_t layer, uint32_t pos,
                        uint32_t n_rows, uint16_t *k_f16, uint16_t *v_f16);
int wr_hip_attn_kv_write(wr_hip_kv *kv, uint32_t layer, uint32_t pos,
                         uint32_t n_rows, const uint16_t *k_f16,
                         const uint16_t *v_f16);

/* ---- decode -------------------------------------------------------------
 * Replaces wri_op_gqa_attention with seq_q = 1 (src/core/kernels.c:1414-1527,
 * contract src/core/internal.h:325-338) at its two call sites
 * (src/core/session.c:341, 493).  q and out are host F32 [nq, hd_layer];
 * seq_k is the number of valid rows (the K tensor's valid_rows);
 * scale_override <= 0 means 1/sqrt(hd); window > 0 keeps only the last
 * `window` keys.  seq_k == 0 or nq % nkv != 0 is WR_HIP_ERR_INVAL; seq_k above
 * max_ctx is WR_HIP_ERR_INVAL (capacity), above the cap WR_HIP_ERR_LIMIT. */
int wr_hip_attn_decode(wr_hip_kv *kv, uint32_t layer, uint32_t seq_k,
                       const float *q, float *out, uint32_t nq,
                       float scale_override, uint32_t window);

/* One launch for n <= WR_HIP_BATCH_MAX sessions with ragged seq_k.
 * Replaces the per-session attention calls inside the batched step
 * (src/core/batch.c:156-164) when the host loop runs layer-major.  All caches
 * must have the same nkv and the same head_dim at `layer`.  n == 0 or
 * n > WR_HIP_BATCH_MAX is WR_HIP_ERR_LIMIT (batch.c:129). */
int wr_hip_attn_decode_batched(uint32_t n, wr_hip_kv *const *kv,
                               uint32_t layer, const uint32_t *seq_k,
                               const float *const *q, float *const *out,
                               uint32_t nq, float scale_override,
                               uint32_t window);

/* ---- a decode step's append and attention in one call ---------------------
 * Replaces the pair the reference makes per layer of a decode step,
 * kv_append_row then wri_op_gqa_attention (src/core/session.c:483-496): row
 * k_f32 / v_f32 [nkv, hd_layer] is truncated to F16 and stored at `pos`, then
 * the nq heads of q attend keys 0 .. pos (with `window` > 0, the last `window`
 * of them) into out.  All four are host F32 and taken as they stand (K and Q
 * already normed and rotated, as at that call site).  Cache bytes and output
 * are those of wr_hip_attn_append followed by wr_hip_attn_decode with
 * seq_k = pos + 1, bit for bit; what changes is the traffic: one copy up, one
 * launch where the shape allows it (head dim 128 with the matrix-core group
 * sizes; two launches back to back otherwise), one copy down, one wait --
 * half the synchronous round trips of the two calls.  pos >= max_ctx is
 * WR_HIP_ERR_CTX_FULL and nothing is written. */
int wr_hip_attn_append_decode(wr_hip_kv *kv, uint32_t layer, uint32_t pos,
                              const float *k_f32, const float *v_f32,
                              const float *q, float *out, uint32_t nq,
                              float scale_override, uint32_t window);

/* The same for n <= WR_HIP_BATCH_MAX sessions at once (the per-session appends
 * and the one batched attention of src/core/batch.c:152-196): row pointers per
 * session, pos[i] the position session i's row goes to.  Any pos[i] >= max_ctx
 * is WR_HIP_ERR_CTX_FULL with nothing written for any session. */
int wr_hip_attn_append_decode_batched(uint32_t n, wr_hip_kv *const *kv,
                                      uint32_t layer, const uint32_t *pos,
                                      const float *const *k_f32,
                                      const float *const *v_f32,
                                      const float *const *q, float *const *out,
                                      uint32_t nq, float scale_override,
                                      uint32_t window);

/* ---- causal prefill -----------------------------------------------------
 * Replaces the loop of seq_q = 1 attention calls that prefill runs
 * (src/core/session.c:615-625): rows p0 .. p0+T-1 have already been appended;
 * row i of q [T, nq, hd_layer] attends keys 0 .. p0+i (with `window` > 0, the
 * last `window` of those).  out is host F32 [T, nq, hd_layer]. */
int wr_hip_attn_prefill(wr_hip_kv *kv, uint32_t layer, uint32_t p0,
                        uint32_t T, const float *q, float *out, uint32_t nq,
                        float scale_override, uint32_t window);

/* ---- device-resident forms (measurement, device-side callers) ------------
 * Same semantics, but q / out / k_f32 / v_f32 are DEVICE pointers obtained
 * from wr_hip_attn_dev_alloc, the work is enqueued on the calling thread's stream and
 * the call returns without waiting; wr_hip_attn_sync waits.  For the batched
 * form q_dev and out_dev are [n, nq, hd] contiguous. */
void *wr_hip_attn_dev_alloc(size_t bytes);
void  wr_hip_attn_dev_free(void *p);
/* Page-locked host memory: copies to and from it run at the link's rate and
 * need no staging (a 10 MB block of logits comes down five times faster than
 * into pageable memory).  Freed with wr_hip_attn_host_free before shutdown. */
void *wr_hip_attn_host_alloc(size_t bytes);
void  wr_hip_attn_host_free(void *p);
int   wr_hip_attn_h2d(void *dst_dev, const void *src_host, size_t bytes);
int   wr_hip_attn_d2h(void *dst_host, const void *src_dev, size_t bytes);
int   wr_hip_attn_sync(void);
void *wr_hip_attn_stream(void);          /* hipStream_t of the calling thread */

int wr_hip_attn_append_dev(wr_hip_kv *kv, uint32_t layer, uint32_t pos,
                           uint32_t n_rows, const float *k_f32_dev,
                           const float *v_f32_dev);

/* One new row for each of n <= WR_HIP_BATCH_MAX sessions in one launch: row i
 * of k_f32_dev / v_f32_dev [n, nkv, hd] goes to position pos[i] of kv[i] (the n
 * kv_append_row calls of a batched step, src/core/batch.c:152-167 through
 * session.c:483-486).  Any pos[i] >= max_ctx is WR_HIP_ERR_CTX_FULL and
 * nothing is written; caches must differ and agree in nkv and head_dim. */
int wr_hip_attn_append_batched_dev(uint32_t n, wr_hip_kv *const *kv,
                                   uint32_t layer, const uint32_t *pos,
                                   const float *k_f32_dev,
                                   const float *v_f32_dev);

/* The same rotation alone, in place on device F32 rows [rows, heads, hd]
 * (wri_op_rope, src/core/kernels.c:1356-1412, for callers that keep Q or K on
 * the device); cos_sin_dev is device F32 [rows, n_rot, 2].  Asynchronous on
 * the stream like the other *_dev calls. */
int wr_hip_attn_rope_dev(void *x_dev, const void *cos_sin_dev, uint32_t rows,
                         uint32_t heads, uint32_t hd, uint32_t n_rot);
/* The table that rotation takes, made on the device: cos_sin_dev, device F32
 * [rows, n_rot, 2], receives (cos, sin) of position / base^(2j/hd) for row r's
 * position (pos[r] when pos, a host array of rows <= WR_HIP_BATCH_MAX entries,
 * is not NULL; pos0 + r otherwise) and pair j < n_rot, where n_rot is
 * n_rot_pairs when that is in [1, hd/2) and hd/2 otherwise, and a base below 1
 * stands for 10000 (the angle of wri_op_rope, src/core/kernels.c:1384-1404,
 * through the polynomials and the range reduction of src/core/mathx.c:37-57,
 * :72-86 and :112-147 operation for operation: the bytes equal what the
 * reference computes per element).  Every position must lie below
 * WR_HIP_ATTN_MAX_SEQ (the bound of the reference's callers; the range
 * reduction's loop does not end for angles beyond 2^27): WR_HIP_ERR_LIMIT
 * otherwise, before anything is launched.  Asynchronous on the stream. */
int wr_hip_attn_rope_table_dev(float *cos_sin_dev, uint32_t rows, uint32_t pos0,
                               const uint32_t *pos, uint32_t hd,
                               float theta_base, uint32_t n_rot_pairs);
int wr_hip_attn_decode_batched_dev(uint32_t n, wr_hip_kv *const *kv,
                                   uint32_t layer, const uint32_t *seq_k,
                                   const float *q_dev, float *out_dev,
                                   uint32_t nq, float scale_override,
                                   uint32_t window);
int wr_hip_attn_prefill_dev(wr_hip_kv *kv, uint32_t layer, uint32_t p0,
                            uint32_t T, const float *q_dev, float *out_dev,
                            uint32_t nq, float scale_override,
                            uint32_t window);
/* wr_hip_attn_prefill_dev for a caller whose Q rows never leave the device:
 * q16_dev [T][nq][hd] holds them as binary16, already multiplied by the
 * softmax scale times log2(e) -- exactly what the kernel makes of F32 rows
 * before its first contraction (it rounds Q to binary16 once), so the output equals wr_hip_attn_prefill_dev's bit for bit
 * at half the Q bytes.  wr_hip_rows_qkv_append_q16_dev writes that form.
 * Replaces the same reference call sites (src/core/session.c:599-630 with
 * src/core/kernels.c:1475-1523).  head_dim 64 and 128 with the matrix-core group
 * sizes; WR_HIP_ERR_UNSUPPORTED otherwise (the caller keeps the F32 form).
 * q16_dev must be 8-byte aligned. */
int wr_hip_attn_prefill_q16_dev(wr_hip_kv *kv, uint32_t layer, uint32_t p0,
                                uint32_t T, const uint16_t *q16_dev,
                                float *out_dev, uint32_t nq,
                                float scale_override, uint32_t window);

/* A decode step's row work and attention in one launch: row i of qkv_dev
 * [n][ld] is session i's stacked projection (nq Q heads, then nkv K heads, then
 * nkv V heads, hd wide each).  Every head gets its per-head RMSNorm when the two
 * weight vectors are given (src/core/session.c:459-474), Q and K the rotation of
 * cos_sin_dev's row i (:475-478); K and V are truncated to F16 and appended at
 * pos[i] (kv_append_row, :483-486), and the nq heads attend over keys
 * 0 .. pos[i] (wri_op_gqa_attention, :488-496) into out_dev [n][nq][hd].  Q, the
 * cache bytes and the output are those of wr_hip_rows_qkv_append_dev followed by
 * wr_hip_attn_decode_batched_dev with seq_k = pos + 1, bit for bit; the point is
 * one dependent launch less per layer of a decode step.  Takes head dim 128 with
 * 16-byte aligned operands, ld a multiple of 4 and n_rot of 8; anything else is
 * WR_HIP_ERR_UNSUPPORTED with nothing written or counted, and the caller makes
 * the two calls.  pos[i] >= max_ctx is WR_HIP_ERR_CTX_FULL, nothing written. */
int wr_hip_attn_append_decode_batched_dev(uint32_t n, wr_hip_kv *const *kv,
                                          uint32_t layer, const uint32_t *pos,
                                          const float *qkv_dev, uint32_t ld,
                                          uint32_t nq, const float *q_norm_dev,
                                          const float *k_norm_dev, float eps,
                                          const float *cos_sin_dev, uint32_t n_rot,
                                          float *out_dev, float scale_override,
                                          uint32_t window);

/* wr_hip_attn_decode_batched_dev for callers that cannot allocate device
 * memory while they run (tight serving loops with a fixed memory budget,
 * harnesses that forbid hipMalloc).  It has no counterpart in the reference.
 * Same arguments, same kernels and the same results bit for bit; the difference
 * is where the split-K tickets and partial rows live: in a fixed array of
 * WR_HIP_NOALLOC_SCRATCH_BYTES that is part of the library's device image
 * (every device the library runs on holds it until the process ends) instead
 * of a buffer the library grows on demand.  The call makes no hipMalloc,
 * hipFree or other allocating call.  A thread's FIRST call into the library
 * creates that thread's stream and staging buffers, which does allocate: this
 * entry point refuses to be that call (WR_HIP_ERR_STATE; any other entry point,
 * wr_hip_attn_sync for one, from the same thread beforehand is enough).  The
 * launch goes to the library's own stream of the calling thread, like every
 * other *_dev call, so it is not something a caller's stream capture records.
 * Limits: nq <= WR_HIP_NOALLOC_MAX_HEADS,
 * and n * nq * max_splits * (hd + 2) * 4 bytes of partials must fit the array
 * behind its first 64 KiB (with the automatic split rule a session has at most
 * 18 key splits: 16 sessions of 32 heads x 128 need 4.8 MB); beyond either,
 * WR_HIP_ERR_LIMIT and nothing is launched.  All calls on one device share the
 * array: the library runs them one after the other, also when they come from
 * different threads (each launch waits for an event the previous one
 * recorded), but a caller must not let two of them overlap on one device by
 * other means (two processes on one device, say): they would race. */
#define WR_HIP_NOALLOC_SCRATCH_BYTES (20u * 1024u * 1024u)
#define WR_HIP_NOALLOC_MAX_HEADS     1024u
int wr_hip_attn_decode_batched_dev_noalloc(uint32_t n, wr_hip_kv *const *kv,
                                           uint32_t layer, const uint32_t *seq_k,
                                           const float *q_dev, float *out_dev,
                                           uint32_t nq, float scale_override,
                                           uint32_t window);

/* What this build of the library offers beyond the attention path proper
 * (bit mask).  A caller that wants the projections and row steps below on the
 * device checks WR_HIP_CAP_PROJ first and otherwise keeps them on the host. */
#define WR_HIP_CAP_PROJ 1u
uint32_t wr_hip_attn_caps(void);

/* ---- projections ---------------------------------------------------------
 * The matrix products either side of the attention path, for callers that want
 * Q/K/V made and the output projected where the cache lives: replaces
 * wri_op_matmul at src/core/session.c:446-457 (wq, wk, wv) and :499-506 (wo)
 * for F16 weights (the reference widens them to F32 at load,
 * src/core/loader.c:164-190, and multiplies in F32, src/core/kernels.c:124-137;
 * here the F16 values are multiplied with F32 activations split into two
 * half-precision terms and summed in F32: results agree to F32 rounding, not
 * bit for bit, because the order of the sum differs).
 *
 * A weight is W[n_out][n_in], `n_in` contiguous (src/core/internal.h:113-118),
 * given as n_parts row blocks that are stacked in order (wq, wk, wv become one
 * product); n_in must be a multiple of 32 and the total n_out of 16, else
 * WR_HIP_ERR_INVAL.  The device copy is private to the library. */
typedef struct wr_hip_weight wr_hip_weight;
int  wr_hip_proj_weight_create(uint32_t n_parts, const uint16_t *const *parts_f16,
                               const uint32_t *rows_per_part, uint32_t n_in,
                               wr_hip_weight **out);
void wr_hip_proj_weight_destroy(wr_hip_weight *w);
uint32_t wr_hip_proj_weight_rows(const wr_hip_weight *w);
uint32_t wr_hip_proj_weight_cols(const wr_hip_weight *w);

/* y[rows][n_out] = x[rows][n_in] . W^T, host F32 in and out, synchronous. */
int wr_hip_proj_rows(const wr_hip_weight *w, uint32_t rows, const float *x,
                     float *y);
/* Device-resident form, asynchronous on the stream: row strides ldx >=
 * n_in and ldy >= n_out (ldy a multiple of 4, y_dev 16-byte aligned);
 * add_dev, if not NULL, is [rows][ldy] and is added to the product (the
 * residual add that follows wo, src/core/session.c:505-506). */
int wr_hip_proj_rows_dev(const wr_hip_weight *w, uint32_t rows,
                         const float *x_dev, uint32_t ldx,
                         const float *add_dev, float *y_dev, uint32_t ldy);

/* The same product fed by a row step that only exists to feed it, so the
 * intermediate rows are never written:
 *   _norm_dev:   y = rmsnorm(x; norm_w_dev [n_in], eps) . W^T (+ add)   (the
 *                attention / FFN / final norms, session.c:443, 509, 538, each
 *                followed by products only)
 *   _swiglu_dev: y = (silu(g) * u) . W^T (+ add), rows of gate_up_dev holding
 *                g = [0, n_in) and u = [n_in, 2 n_in), ld >= 2 n_in
 *                (session.c:521-534).
 * Values are those of wr_hip_rows_rmsnorm_dev / wr_hip_rows_swiglu_dev followed
 * by wr_hip_proj_rows_dev, bit for bit. */
int wr_hip_proj_rows_norm_dev(const wr_hip_weight *w, uint32_t rows,
                              const float *x_dev, uint32_t ldx,
                              const float *norm_w_dev, float eps,
                              const float *add_dev, float *y_dev, uint32_t ldy);
int wr_hip_proj_rows_swiglu_dev(const wr_hip_weight *w, uint32_t rows,
                                const float *gate_up_dev, uint32_t ld,
                                const float *add_dev, float *y_dev, uint32_t ldy);
/* the same with the tanh form of GELU in place of SiLU (wri_op_fused_gelu_mul,
 * src/core/kernels.c:969-976; Gemma's FFN, session.c:376-381) */
int wr_hip_proj_rows_geglu_dev(const wr_hip_weight *w, uint32_t rows,
                               const float *gate_up_dev, uint32_t ld,
                               const float *add_dev, float *y_dev, uint32_t ldy);

/* ---- row steps between the projections and the attention path --------------
 * For callers that keep a layer's activations on the device.  All arguments
 * are device pointers (wr_hip_attn_dev_alloc), all calls are asynchronous on
 * the stream.  Sums over a row are tree reductions here and
 * sequential loops in the reference, so results agree to F32 rounding.
 *
 * rmsnorm: out[r][j] = x[r][j] / sqrt(mean_j x[r][j]^2 + eps) * w[j % wn], or
 * without weight when wn == 0 (wri_op_rmsnorm, src/core/kernels.c:1276-1316;
 * called at src/core/session.c:443, 509, 538). */
int wr_hip_rows_rmsnorm_dev(const float *x_dev, uint32_t ldx, const float *w_dev,
                            uint32_t wn, float *out_dev, uint32_t ldo,
                            uint32_t rows, uint32_t dim, float eps);

/* rmsnorm_add: acc[r][j] += the same normalised value (Gemma's sandwich norms:
 * a sublayer's output is normalised before it joins the residual,
 * src/core/session.c:355-359, 391-395). */
int wr_hip_rows_rmsnorm_add_dev(const float *x_dev, uint32_t ldx, const float *w_dev,
                                uint32_t wn, float *acc_dev, uint32_t lda,
                                uint32_t rows, uint32_t dim, float eps);

/* qkv_prep: rows of a stacked projection [nq heads | nkv K heads | nkv V heads]
 * (row stride ld) are split into Q [rows, nq, hd], K and V [rows, nkv, hd].
 * Q and K heads get the per-head RMSNorm when q_norm_dev / k_norm_dev ([hd],
 * both or neither) are given (Qwen3, src/core/session.c:459-470), then the
 * rotary embedding with the caller's table cos_sin_dev [rows, n_rot, 2]
 * (split-half pairing, src/core/kernels.c:1356-1412, called at
 * session.c:473-480); V is copied.  hd must be even and <= 1024. */
int wr_hip_rows_qkv_prep_dev(const float *qkv_dev, uint32_t ld, uint32_t rows,
                             uint32_t nq, uint32_t nkv, uint32_t hd,
                             const float *q_norm_dev, const float *k_norm_dev,
                             float eps, const float *cos_sin_dev, uint32_t n_rot,
                             float *q_out_dev, float *k_out_dev, float *v_out_dev);

/* qkv_append: qkv_prep and the cache append in one launch, for callers whose
 * K and V rows exist only to be appended (src/core/session.c:459-486: the norm,
 * the rotation, then wri_kv_append for K and V).  Q leaves as in qkv_prep; the
 * rotated K heads and the V heads are truncated to binary16 as in
 * wr_hip_attn_append and written into the cache(s) directly.  Head counts and
 * head_dim of K and V are the cache's (layer `layer`).
 *   n_kv == 1: the rows are positions pos[0], pos[0]+1, ... of kv[0];
 *   n_kv == rows (<= WR_HIP_BATCH_MAX, distinct caches of one geometry): row i
 *   is position pos[i] of kv[i] (the batched step).
 * All or nothing: a position past a cache's max_ctx returns
 * WR_HIP_ERR_CTX_FULL before anything is written.  head_dim <= 512
 * (WR_HIP_ERR_LIMIT beyond; use qkv_prep + append).  Q and the cache bits
 * equal those of qkv_prep followed by the append, bit for bit. */
#define WR_HIP_QKV_V_NORM 1u   /* V heads get a weightless RMSNorm before they are stored (Gemma,
                                  src/core/session.c:318-323) */
#define WR_HIP_QKV_Q_ONLY 2u   /* the rows hold Q heads only and nothing is appended: a layer that
                                  reads another layer's cache (session.c:108-134); `layer` names
                                  the cache layer whose head_dim the Q heads have */
int wr_hip_rows_qkv_append_dev(const float *qkv_dev, uint32_t ld, uint32_t rows, uint32_t nq,
                               const float *q_norm_dev, const float *k_norm_dev, float eps,
                               const float *cos_sin_dev, uint32_t n_rot, uint32_t n_kv,
                               wr_hip_kv *const *kv, uint32_t layer, const uint32_t *pos,
                               float *q_out_dev, uint32_t flags);
/* The same (src/core/session.c:459-486), with Q written as binary16 rows
 * multiplied by the softmax scale (scale_override > 0, else 1/sqrt(hd)) times
 * log2(e): the operand wr_hip_attn_prefill_q16_dev takes.  K and V are appended
 * exactly as above.  head_dim 128 with the alignment of the eight-lane form
 * (16-byte aligned pointers, ld % 4 == 0, n_rot % 8 == 0);
 * WR_HIP_ERR_UNSUPPORTED otherwise, before anything is written. */
int wr_hip_rows_qkv_append_q16_dev(const float *qkv_dev, uint32_t ld, uint32_t rows, uint32_t nq,
                                   const float *q_norm_dev, const float *k_norm_dev, float eps,
                                   const float *cos_sin_dev, uint32_t n_rot, uint32_t n_kv,
                                   wr_hip_kv *const *kv, uint32_t layer, const uint32_t *pos,
                                   uint16_t *q16_out_dev, float scale_override, uint32_t flags);

/* swiglu: act[r][j] = silu(gu[r][j]) * gu[r][ffn + j] for rows of a stacked
 * gate/up projection (wri_op_fused_silu_mul, src/core/kernels.c:1243-1258 with
 * silu at :963-967; called at session.c:523-526). */
int wr_hip_rows_swiglu_dev(const float *gate_up_dev, uint32_t ld, float *act_dev,
                           uint32_t ldo, uint32_t rows, uint32_t ffn);

/* Tuning knobs for measurement (0 = automatic): keys handled per workgroup in
 * the split-K decode kernel, and a switch forcing the generic (non-MFMA)
 * kernels.  Not needed by a normal caller. */
void wr_hip_attn_set_tuning(uint32_t decode_keys_per_wg, int force_generic);

/* Measurement knob without a counterpart in the reference: which of the two
 * causal-prefill kernels head dim 128 takes.  0 (the default, also set by
 * WR_HIP_PREFILL_TWO_WAVES unset or "1" at init): eight waves per workgroup,
 * two per SIMD, one 32-row unit per wave.  1 (WR_HIP_PREFILL_TWO_WAVES=0): four
 * waves, one per SIMD, two units per wave.  Same results to rounding; the
 * second form is kept for comparison and is the slower one at present. */
void wr_hip_attn_set_prefill_one_wave(int on);

/* Kernel timing for the roofline figure.  Between profile_begin and
 * profile_end every launch of the MAIN kernel of a call (the split-K decode
 * kernel, or the prefill kernel; not the small combine / append kernels) is
 * bracketed by its own pair of events, so the sum is pure kernel time as a
 * profiler would report it.  profile_end waits for the stream, then returns
 * the summed milliseconds and the number of launches timed.  At most
 * max_launches launches are timed; further ones run untimed. */
int wr_hip_attn_profile_begin(uint32_t max_launches);
int wr_hip_attn_profile_end(double *total_ms, uint32_t *n_launches);

#ifdef __cplusplus
}
#endif
#endif /* WR_HIP_ATTN_H */
