/*
 * wr_host.h — internal contracts of the C11 host engine.
 *
 * The engine keeps the reference's decode structure (reference:
 * src/core/session.c, src/core/batch.c) but drives it layer-major over a set
 * of ROWS, so that one attention launch per layer serves a whole prefill chunk
 * or a whole batch of sessions.  A row is one token of one session at one
 * position; every CPU op here is row-wise, so the per-row arithmetic is the
 * same whether a row travels alone (wr_step), with its prompt neighbours
 * (wr_prefill) or with other sessions (wr_batch_step).
 */
#ifndef WR_HOST_H
#define WR_HOST_H

#include <pthread.h>
#include <stddef.h>
#include <stdint.h>

#include <wayruntime/wayruntime.h>

#include "../../include/wr_hip_attn.h"

#define WRH_MAX_LAYERS   64          /* reference: WR_MAX_LAYERS, src/core/internal.h:184 */
#define WRH_DEFAULT_CTX  4096        /* reference: WR_DEFAULT_MAX_CONTEXT, internal.h:194 */
#define WRH_PREFILL_CHUNK 256        /* rows per layer-major prefill pass, host walk */
#define WRH_DEVICE_PREFILL_CHUNK 4096 /* ... device walk: long passes give the attention kernel enough position blocks to fill the chip */

/* ---- scalar math with the reference's polynomials (wr_math.c) ------------- */
float wrh_exp(float x);
float wrh_log(float x);
float wrh_sqrt(float x);
float wrh_sin(float x);
float wrh_cos(float x);

/* ---- weights ------------------------------------------------------------- */
typedef struct wrh_weight {
    const void *data;        /* points into the mapped file */
    uint32_t    rows, cols;  /* [rows][cols], cols contiguous: W[out][in] or table[token][hidden] */
    uint8_t     is_f16;      /* 1 = binary16, 0 = float32 */
} wrh_weight;

typedef struct wrh_vec {
    const float *data;
    uint32_t     n;
} wrh_vec;

struct wr_engine {
    wr_engine_config cfg;
    int      n_threads;
    uint32_t models_live;
    uint64_t ctr[WR_COUNTER_COUNT];
};

struct wr_model {
    wr_engine *engine;
    char       arch[32];
    uint32_t   n_layers, n_q, n_kv, head_dim, hidden, ffn, vocab;
    uint32_t   train_context, max_context, n_rot_pairs;
    float      rms_eps, rope_base;
    uint8_t    has_qk_norm, tied_head, all_f16;

    /* Gemma family (reference: src/core/loader.c:576-628): sandwich norms,
     * GeGLU, embedding scale, attention scale 1.0, per-layer head_dim and
     * sliding window, KV-shared trailing layers, final-logit soft cap. */
    uint8_t    is_gemma, has_swa, swa_mode;
    uint8_t    swa[WRH_MAX_LAYERS];          /* 1 = sliding-window (local) layer */
    uint32_t   head_dim_swa, sliding_window, kv_shared_layers;
    uint32_t   hd_layer[WRH_MAX_LAYERS];     /* head_dim of each layer */
    uint32_t   kv_src[WRH_MAX_LAYERS];       /* layer whose cache layer L reads (L itself if it owns one) */
    float      rope_base_swa, embed_scale, attn_scale, logit_softcap;
    wrh_vec    post_attn_norm[WRH_MAX_LAYERS], post_ffw_norm[WRH_MAX_LAYERS];

    wrh_weight embed, lm_head;
    wrh_vec    final_norm;
    wrh_vec    attn_norm[WRH_MAX_LAYERS], ffn_norm[WRH_MAX_LAYERS];
    wrh_vec    q_norm[WRH_MAX_LAYERS], k_norm[WRH_MAX_LAYERS];
    wrh_weight wq[WRH_MAX_LAYERS], wk[WRH_MAX_LAYERS], wv[WRH_MAX_LAYERS], wo[WRH_MAX_LAYERS];
    wrh_weight w_gate[WRH_MAX_LAYERS], w_up[WRH_MAX_LAYERS], w_down[WRH_MAX_LAYERS];

    struct wrh_dev_model *dev;   /* device copies of the weights, NULL on the host walk */
    /* Scratch of the device walk's multi-row calls, kept between calls (a
     * 16-session step otherwise spends a third of its time allocating device
     * memory and faulting in ten megabytes of logits): one set for
     * wr_batch_step, one for wr_prefill.  A call that finds its set taken by a
     * concurrent call allocates its own as before. */
    struct wrh_scratch *batch_scratch, *prefill_scratch;

    void           *map;         /* mmap of the GGUF file */
    size_t          map_bytes;
    pthread_mutex_t lock;        /* guards session_refs */
    uint32_t        session_refs;
};

/* Scratch for R rows of the forward pass. */
typedef struct wrh_workspace {
    uint32_t rows_cap;
    float *residual, *normed;            /* [R][hidden] */
    float *q, *attn;                     /* [R][n_q*hd]  */
    float *k, *v;                        /* [R][n_kv*hd] */
    float *gate, *up;                    /* [R][ffn]     */
    float *proj;                         /* [R][hidden]  */
    float *rope;                         /* [R][hd/2][2] (cos, sin) of the rows' angles */
    float *rope_swa;                     /* the same for Gemma's sliding-window layers */
    void  *block;
    /* device walk: `residual` already holds the embedded rows of these tokens
     * (staged while the device worked on the rows before) */
    const uint32_t *staged_tokens;
    uint32_t staged_rows, staged_pos0;
} wrh_workspace;

struct wrh_scratch;
/* Takes the model's cached set (kind 0 = batch, 1 = prefill) when it is free,
 * growing it to rows / logit_rows; otherwise returns a fresh one.  NULL when
 * memory runs out.  Release returns it (a fresh one is freed). */
struct wrh_scratch *wrh_scratch_acquire(wr_model *m, int kind, uint32_t rows, uint32_t logit_rows);
void wrh_scratch_release(wr_model *m, struct wrh_scratch *sc);
void wrh_scratch_free_all(wr_model *m);

/* Device scratch for R rows of the device walk (wr_device.c). */
typedef struct wrh_devspace {
    uint32_t rows_cap, logit_rows;
    float *resid;                        /* [R][hidden] */
    float *qkv;                          /* [R][(n_q + 2 n_kv) * hd] */
    float *q, *attn;                     /* [R][n_q*hd] */
    float *k, *v;                        /* [R][n_kv*hd] */
    float *gu;                           /* [R][2 ffn]: gate | up */
    float *rope;                         /* [R][hd/2][2] */
    float *rope_swa;                     /* the same for Gemma's sliding-window layers */
    float *proj;                         /* [R][hidden]: a sublayer output on its way through a post-norm */
    float *logits;                       /* [logit_rows][vocab] */
    float *block;
} wrh_devspace;

/* Everything a multi-row call of the device walk needs besides the model. */
struct wrh_scratch {
    wrh_workspace ws;                    /* host rows (embedding) */
    wrh_devspace  ds;
    float        *logits_host;           /* page-locked, [logit_rows][vocab]; NULL when logit_rows == 0 */
    uint32_t      rows, logit_rows;
    int           cached;                /* belongs to the model (else freed on release) */
    int           busy;
};

struct wr_session {
    wr_model       *model;
    pthread_mutex_t lock;
    uint32_t        max_context;
    uint32_t        pos;                     /* tokens in the cache == next position */
    wr_status       last_status;
    wr_hip_kv      *kv;                      /* device cache */
    uint32_t        kv_rows[WRH_MAX_LAYERS]; /* per-layer cursor (the reference's valid_rows) */
    float          *logits;                  /* [vocab] */
    wrh_workspace   ws1;                     /* one-row scratch for wr_step */
    wrh_devspace    ds1;                     /* its device counterpart (device walk only) */
};

/* ---- ops (wr_ops.c) -------------------------------------------------------
 * All row-wise over R rows; `ld` is the row stride in floats. */
int  wrh_embed(const wrh_weight *table, uint32_t token, float *out_row);
void wrh_rmsnorm(const float *x, const float *w, uint32_t wn, float *out, uint32_t rows,
                 uint32_t dim, float eps);
/* C[r][j] = sum_k A[r][k] * W[j][k]; each output column is reduced whole in one
 * thread, so results do not depend on the thread count or on R. */
void wrh_matmul(wr_engine *e, const float *A, uint32_t R, uint32_t lda, const wrh_weight *W,
                float *C, uint32_t ldc);
void wrh_rope(float *x, uint32_t heads, uint32_t hd, uint32_t pos, float theta,
              uint32_t n_rot_pairs);
uint32_t wrh_rope_table(float *cos_sin, uint32_t hd, uint32_t pos, float theta,
                        uint32_t n_rot_pairs);
void wrh_rope_apply(float *x, uint32_t heads, uint32_t hd, const float *cos_sin, uint32_t n_rot);
void wrh_swiglu(wr_engine *e, float *gate, const float *up, uint64_t n);
void wrh_geglu(wr_engine *e, float *gate, const float *up, uint64_t n);
void wrh_softcap(float *x, uint64_t n, float cap);
void wrh_scale(float *x, uint64_t n, float s);
float wrh_tanh(float x);
void wrh_add(float *acc, const float *x, uint64_t n);

/* ---- model / gguf (wr_model.c) -------------------------------------------- */
void wrh_logf(wr_engine *e, int level, const char *fmt, ...) __attribute__((format(printf, 3, 4)));
extern wr_engine *wrh_engine;           /* the process engine, NULL when none */

/* ---- forward (wr_session.c) ------------------------------------------------ */
int  wrh_workspace_init(wrh_workspace *ws, const wr_model *m, uint32_t rows);
void wrh_workspace_free(wrh_workspace *ws);

/* ---- device walk (wr_device.c) --------------------------------------------- */
wr_status wrh_device_model_init(wr_model *m);
void      wrh_device_model_free(wr_model *m);
int       wrh_devspace_init(wrh_devspace *ws, const wr_model *m, uint32_t rows, uint32_t logit_rows);
void      wrh_devspace_free(wrh_devspace *ws);
wr_status wrh_forward_rows_device(wr_model *m, wrh_workspace *hs, wrh_devspace *ds, uint32_t R,
                                  wr_session *const *ss, const uint32_t *tokens, uint32_t pos0,
                                  int batch, int prefill, int fail_layer, float *logits_host,
                                  uint32_t logit_rows, uint32_t next_rows);

/* Test hook: make the attention call of `layer` fail with WR_ERR_INTERNAL once
 * (layer < 0 disarms).  The device is not involved: the failure is raised on
 * the host before the launch, so rollback paths can be exercised safely. */
void wrh_debug_fail_attention_at(int layer);

#endif /* WR_HOST_H */
