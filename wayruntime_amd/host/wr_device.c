/*
 * wr_device.c — the layer walk with every matrix product and row step on the
 * device (reference: src/core/session.c:440-538, the same block wr_session.c
 * walks on the host).  Used when the device library offers projections
 * (WR_HIP_CAP_PROJ) and every matrix of the model is F16 with dimensions the
 * projection kernel takes; WAYRT_HOST_LAYERS=1 in the environment keeps the
 * host walk, WAYRT_STEP_TWO_LAUNCHES=1 keeps a decode step's row step and its
 * attention as two launches.  Per call the host embeds the rows and sends them up once; the
 * rotary angles of their positions are made on the device (the reference's
 * polynomial sin / cos and range reduction restated there bit for bit:
 * wr_hip_attn_rope_table_dev); the layers run without coming back, and the
 * logits come down (wr_step, wr_batch_step) or nothing does (wr_prefill).  The Gemma
 * family's block (session.c:251-437) takes the same walk with its own steps:
 * per-layer head_dim, two rotary tables, layers that read another layer's
 * cache, the weightless V norm, sandwich norms, GeGLU, attention scale 1.
 *
 * Sums run in a different order than on the host (matrix-core tiles, tree
 * reductions), so activations agree with the host walk to F32 rounding, not
 * bit for bit; the greedy token stream is compared with the reference's in
 * the end-to-end test.
 */
#define _POSIX_C_SOURCE 200809L
#include "wr_host.h"

#include <stdlib.h>
#include <string.h>

typedef struct dev_layer {
    wr_hip_weight *wqkv, *wo, *wgu, *wdown;                   /* wqkv holds Q only on a layer without its own cache */
    const float *attn_norm, *ffn_norm, *q_norm, *k_norm;      /* device */
    const float *post_attn_norm, *post_ffw_norm;              /* Gemma */
} dev_layer;

struct wrh_dev_model {
    dev_layer     L[WRH_MAX_LAYERS];
    wr_hip_weight *lm_head;
    float         *vecs;                                       /* one device block for all norm vectors */
    const float   *final_norm;
    /* decode steps: does the library take the row step (split, norms, rotation,
     * append) inside the attention launch for this model?  0 = not asked yet,
     * 1 = yes, -1 = no (the two calls are made).  Read and written atomically:
     * sessions step from several threads. */
    int            step_in_one_launch;
    /* prompt passes: does the library take Q as binary16 rows for this model's
     * attention (same meaning of 0 / 1 / -1)? */
    int            prefill_q16;
};

static int proj_dims_ok(const wrh_weight *w)
{
    return w->is_f16 && w->cols % 32 == 0;
}

void wrh_device_model_free(wr_model *m)
{
    struct wrh_dev_model *d = m->dev;
    if (!d) return;
    for (uint32_t l = 0; l < m->n_layers; l++) {
        wr_hip_proj_weight_destroy(d->L[l].wqkv);
        wr_hip_proj_weight_destroy(d->L[l].wo);
        wr_hip_proj_weight_destroy(d->L[l].wgu);
        wr_hip_proj_weight_destroy(d->L[l].wdown);
    }
    wr_hip_proj_weight_destroy(d->lm_head);
    wr_hip_attn_dev_free(d->vecs);
    free(d);
    m->dev = NULL;
}

static int stack(wr_hip_weight **out, const wrh_weight *a, const wrh_weight *b, const wrh_weight *c)
{
    const uint16_t *parts[3] = {a->data, b ? b->data : NULL, c ? c->data : NULL};
    uint32_t rows[3] = {a->rows, b ? b->rows : 0, c ? c->rows : 0};
    return wr_hip_proj_weight_create(c ? 3 : (b ? 2 : 1), parts, rows, a->cols, out);
}

/* WR_OK with m->dev set, WR_OK with m->dev NULL when the model stays on the
 * host walk, or an error when uploading a model that qualifies fails. */
wr_status wrh_device_model_init(wr_model *m)
{
    m->dev = NULL;
    const char *env = getenv("WAYRT_HOST_LAYERS");
    if (env && env[0] == '1') return WR_OK;
    if (!(wr_hip_attn_caps() & WR_HIP_CAP_PROJ)) return WR_OK;
    int ok = proj_dims_ok(&m->lm_head) && m->vocab % 16 == 0 && m->hidden % 16 == 0 &&
             (2 * m->ffn) % 16 == 0;
    for (uint32_t l = 0; l < m->n_layers && ok; l++) {
        const uint32_t hd = m->hd_layer[l], qd = m->n_q * hd, kd = m->n_kv * hd;
        const int shared = m->kv_src[l] != l;
        ok = hd <= 512 &&                          /* the fused Q/K/V split + append */
             (qd + (shared ? 0 : 2 * kd)) % 16 == 0 && proj_dims_ok(&m->wq[l]) &&
             (shared || (proj_dims_ok(&m->wk[l]) && proj_dims_ok(&m->wv[l]))) &&
             proj_dims_ok(&m->wo[l]) && proj_dims_ok(&m->w_gate[l]) && proj_dims_ok(&m->w_up[l]) &&
             proj_dims_ok(&m->w_down[l]);
    }
    if (!ok) {
        wrh_logf(m->engine, 2, "device layers: model keeps the host walk (needs F16 matrices, "
                              "inputs a multiple of 32, outputs of 16)");
        return WR_OK;
    }

    struct wrh_dev_model *d = calloc(1, sizeof *d);
    if (!d) return WR_ERR_NOMEM;
    m->dev = d;
    /* WAYRT_STEP_TWO_LAUNCHES=1: a decode step's row step and attention stay two calls */
    env = getenv("WAYRT_STEP_TWO_LAUNCHES");
    if (env && env[0] == '1') d->step_in_one_launch = -1;
    /* WAYRT_PREFILL_Q_F32=1: prompt passes hand the attention kernel F32 Q rows */
    env = getenv("WAYRT_PREFILL_Q_F32");
    if (env && env[0] == '1') d->prefill_q16 = -1;
    int rc = WR_HIP_OK;
    /* norm vectors: [final | per layer: attn, ffn, (q, k), (post-attn, post-ffn)] */
    size_t n_vec = m->hidden;
    for (uint32_t l = 0; l < m->n_layers; l++)
        n_vec += m->attn_norm[l].n + m->ffn_norm[l].n + m->q_norm[l].n + m->k_norm[l].n +
                 m->post_attn_norm[l].n + m->post_ffw_norm[l].n;
    float *host = malloc(n_vec * sizeof(float));
    d->vecs = wr_hip_attn_dev_alloc(n_vec * sizeof(float));
    if (!host || !d->vecs) rc = WR_HIP_ERR_NOMEM;
    if (rc == WR_HIP_OK) {
        size_t at = 0;
#define PUT(vec, dst)                                                   \
        do {                                                            \
            if ((vec).n) {                                              \
                memcpy(host + at, (vec).data, (vec).n * sizeof(float)); \
                (dst) = d->vecs + at;                                   \
                at += (vec).n;                                          \
            }                                                           \
        } while (0)
        PUT(m->final_norm, d->final_norm);
        for (uint32_t l = 0; l < m->n_layers; l++) {
            PUT(m->attn_norm[l], d->L[l].attn_norm);
            PUT(m->ffn_norm[l], d->L[l].ffn_norm);
            PUT(m->q_norm[l], d->L[l].q_norm);
            PUT(m->k_norm[l], d->L[l].k_norm);
            PUT(m->post_attn_norm[l], d->L[l].post_attn_norm);
            PUT(m->post_ffw_norm[l], d->L[l].post_ffw_norm);
        }
#undef PUT
        rc = wr_hip_attn_h2d(d->vecs, host, n_vec * sizeof(float));
    }
    free(host);
    for (uint32_t l = 0; l < m->n_layers && rc == WR_HIP_OK; l++) {
        if (m->kv_src[l] != l)
            rc = stack(&d->L[l].wqkv, &m->wq[l], NULL, NULL);
        else
            rc = stack(&d->L[l].wqkv, &m->wq[l], &m->wk[l], &m->wv[l]);
        if (rc == WR_HIP_OK) rc = stack(&d->L[l].wo, &m->wo[l], NULL, NULL);
        if (rc == WR_HIP_OK) rc = stack(&d->L[l].wgu, &m->w_gate[l], &m->w_up[l], NULL);
        if (rc == WR_HIP_OK) rc = stack(&d->L[l].wdown, &m->w_down[l], NULL, NULL);
    }
    if (rc == WR_HIP_OK) rc = stack(&d->lm_head, &m->lm_head, NULL, NULL);
    /* the uploads ran on this thread's stream; sessions may step on others */
    if (rc == WR_HIP_OK) rc = wr_hip_attn_sync();
    if (rc != WR_HIP_OK) {
        wrh_logf(m->engine, 0, "device layers: weight upload failed (rc=%d)", rc);
        wrh_device_model_free(m);
        return (rc == WR_HIP_ERR_NOMEM) ? WR_ERR_NOMEM : WR_ERR_INTERNAL;
    }
    wrh_logf(m->engine, 2, "device layers: %u layers and the LM head are on the device", m->n_layers);
    return WR_OK;
}

/* ------------------------------------------------------------- workspace -- */

static size_t r64(size_t n) { return (n + 63) & ~(size_t)63; }       /* floats: 256-byte steps */

int wrh_devspace_init(wrh_devspace *ws, const wr_model *m, uint32_t rows, uint32_t logit_rows)
{
    memset(ws, 0, sizeof *ws);
    size_t hd = m->head_dim;
    for (uint32_t l = 0; l < m->n_layers; l++)
        if (m->hd_layer[l] > hd) hd = m->hd_layer[l];
    const size_t hidden = m->hidden, qd = (size_t)m->n_q * hd, kd = (size_t)m->n_kv * hd;
    const size_t ffn = m->ffn, R = rows;
    const size_t total = 2 * r64(R * hidden) + r64(R * (qd + 2 * kd)) + 2 * r64(R * qd) + 2 * r64(R * kd) +
                         r64(R * 2 * ffn) + 2 * r64(R * hd) + r64((size_t)logit_rows * m->vocab);
    float *b = wr_hip_attn_dev_alloc(total * sizeof(float));
    if (!b) return WR_ERR_NOMEM;
    ws->block = b;
    ws->rows_cap = rows;
    ws->logit_rows = logit_rows;
    ws->resid = b;   b += r64(R * hidden);
    ws->proj = b;    b += r64(R * hidden);
    ws->qkv = b;     b += r64(R * (qd + 2 * kd));
    ws->q = b;       b += r64(R * qd);
    ws->attn = b;    b += r64(R * qd);
    ws->k = b;       b += r64(R * kd);
    ws->v = b;       b += r64(R * kd);
    ws->gu = b;      b += r64(R * 2 * ffn);
    ws->rope = b;    b += r64(R * hd);
    ws->rope_swa = b; b += r64(R * hd);
    ws->logits = b;
    return WR_OK;
}

void wrh_devspace_free(wrh_devspace *ws)
{
    if (ws->block) wr_hip_attn_dev_free(ws->block);
    memset(ws, 0, sizeof *ws);
}

/* ---------------------------------------------------------- kept scratch -- */

static void scratch_destroy(struct wrh_scratch *sc)
{
    if (!sc) return;
    wrh_devspace_free(&sc->ds);
    wrh_workspace_free(&sc->ws);
    if (sc->logits_host) wr_hip_attn_host_free(sc->logits_host);
    free(sc);
}

static struct wrh_scratch *scratch_create(const wr_model *m, uint32_t rows, uint32_t logit_rows)
{
    struct wrh_scratch *sc = calloc(1, sizeof *sc);
    if (!sc) return NULL;
    sc->rows = rows;
    sc->logit_rows = logit_rows;
    int ok = wrh_workspace_init(&sc->ws, m, rows) == WR_OK;
    ok = ok && wrh_devspace_init(&sc->ds, m, rows, logit_rows) == WR_OK;
    if (ok && logit_rows) {
        sc->logits_host = wr_hip_attn_host_alloc((size_t)logit_rows * m->vocab * sizeof(float));
        ok = sc->logits_host != NULL;
    }
    if (!ok) {
        scratch_destroy(sc);
        return NULL;
    }
    return sc;
}

struct wrh_scratch *wrh_scratch_acquire(wr_model *m, int kind, uint32_t rows, uint32_t logit_rows)
{
    struct wrh_scratch **slot = kind ? &m->prefill_scratch : &m->batch_scratch;
    pthread_mutex_lock(&m->lock);
    struct wrh_scratch *sc = *slot;
    if (sc && sc->busy) {                              /* a concurrent call has it */
        pthread_mutex_unlock(&m->lock);
        return scratch_create(m, rows, logit_rows);
    }
    if (sc && (sc->rows < rows || sc->logit_rows < logit_rows)) {
        *slot = NULL;                                  /* too small: replace */
        scratch_destroy(sc);
        sc = NULL;
    }
    if (!sc) {
        /* a batch set is sized for the largest batch once; a prefill set for this call */
        const uint32_t r = kind ? rows : WR_BATCH_MAX;
        sc = scratch_create(m, r > rows ? r : rows, kind ? logit_rows : WR_BATCH_MAX);
        if (sc) {
            sc->cached = 1;
            *slot = sc;
        }
    }
    if (sc) sc->busy = 1;
    pthread_mutex_unlock(&m->lock);
    return sc;
}

void wrh_scratch_release(wr_model *m, struct wrh_scratch *sc)
{
    if (!sc) return;
    if (!sc->cached) {
        scratch_destroy(sc);
        return;
    }
    pthread_mutex_lock(&m->lock);
    sc->busy = 0;
    sc->ws.staged_rows = 0;
    pthread_mutex_unlock(&m->lock);
}

void wrh_scratch_free_all(wr_model *m)
{
    scratch_destroy(m->batch_scratch);
    scratch_destroy(m->prefill_scratch);
    m->batch_scratch = m->prefill_scratch = NULL;
}

/* --------------------------------------------------------------- forward -- */

static wr_status dev_fail(wr_engine *e, const char *what, uint32_t layer, int rc)
{
    wrh_logf(e, 0, "session: %s failed at layer %u (rc=%d)", what, layer, rc);
    if (rc == WR_HIP_ERR_CTX_FULL) return WR_ERR_CTX_FULL;
    return (rc < 0) ? (wr_status)rc : WR_ERR_INTERNAL;
}

#define TRY(call, what)                                        \
    do {                                                       \
        rc = (call);                                           \
        if (rc != WR_HIP_OK) return dev_fail(e, what, L, rc);  \
    } while (0)

/* Host part of a pass: the embedding rows of R tokens into the host workspace,
 * rows in parallel.  (The rotary angles are made on the device, where the
 * cache lives: wr_hip_attn_rope_table_dev.) */
static wr_status stage_rows(wr_model *m, wrh_workspace *hs, uint32_t R, const uint32_t *tokens)
{
    const uint32_t hidden = m->hidden;
    const wr_engine *e = m->engine;
    const int threads = (e && e->n_threads > 0) ? e->n_threads : 1;
    int bad = WR_OK;
#pragma omp parallel for num_threads(threads) schedule(static) if (R >= 4)
    for (uint32_t r = 0; r < R; r++) {
        float *row = hs->residual + (size_t)r * hidden;
        const int rc = wrh_embed(&m->embed, tokens[r], row);
        if (rc != WR_OK) __atomic_store_n(&bad, rc, __ATOMIC_RELAXED);
        /* Gemma: scaled embeddings (session.c:262-283) */
        if (m->is_gemma && m->embed_scale != 0.0f) wrh_scale(row, hidden, m->embed_scale);
    }
    return (wr_status)bad;
}

/* Stages the rows of the NEXT pass of a prefill; called between a pass's last
 * launch and its wait for the device, so the host's share of a pass costs no
 * wall time from the second pass on. */
void wrh_stage_next_rows(wr_model *m, wrh_workspace *hs, uint32_t R, const uint32_t *tokens,
                         uint32_t pos0)
{
    hs->staged_rows = 0;
    if (stage_rows(m, hs, R, tokens) != WR_OK) return;   /* the pass itself reports it */
    hs->staged_tokens = tokens;
    hs->staged_rows = R;
    hs->staged_pos0 = pos0;
}

/* Same contract as the host walk's forward_rows (wr_session.c), plus: when
 * logits_host is not NULL, the LM head runs for the first `logit_rows` rows
 * and their logits [logit_rows][vocab] are brought down; when next_rows is not
 * zero (prefill), the host stages that many further tokens (tokens + R, at
 * pos0 + R) while the device works. */
wr_status wrh_forward_rows_device(wr_model *m, wrh_workspace *hs, wrh_devspace *ds, uint32_t R,
                                  wr_session *const *ss, const uint32_t *tokens, uint32_t pos0,
                                  int batch, int prefill, int fail_layer, float *logits_host,
                                  uint32_t logit_rows, uint32_t next_rows)
{
    wr_engine *e = m->engine;
    const struct wrh_dev_model *d = m->dev;
    const uint32_t hidden = m->hidden, hd = m->head_dim, nq = m->n_q, nkv = m->n_kv;
    const uint32_t ffn = m->ffn;
    const uint32_t n_rot = (m->n_rot_pairs >= 1 && m->n_rot_pairs < hd / 2) ? m->n_rot_pairs : hd / 2;
    uint32_t L = 0;
    int rc;

    const int staged = !batch && hs->staged_rows == R && hs->staged_tokens == tokens && hs->staged_pos0 == pos0;
    hs->staged_rows = 0;
    if (!staged) {
        rc = stage_rows(m, hs, R, tokens);
        if (rc != WR_OK) return dev_fail(e, "embed", 0, rc);
    }
    TRY(wr_hip_attn_h2d(ds->resid, hs->residual, (size_t)R * hidden * sizeof(float)), "rows up");
    /* rotary tables of the rows' positions; Gemma's sliding-window layers have
     * their own head_dim and base and rotate fully (session.c:262-283) */
    uint32_t plist[WR_HIP_BATCH_MAX];
    if (batch) {
        if (R > WR_HIP_BATCH_MAX) return dev_fail(e, "angles", 0, WR_HIP_ERR_INVAL);
        for (uint32_t r = 0; r < R; r++) plist[r] = ss[r]->pos;
    }
    TRY(wr_hip_attn_rope_table_dev(ds->rope, R, pos0, batch ? plist : NULL, hd, m->rope_base,
                                   m->n_rot_pairs), "angles");
    const int gemma = m->is_gemma;
    const uint32_t hd_s = m->head_dim_swa ? m->head_dim_swa : hd;
    if (gemma && m->has_swa)
        TRY(wr_hip_attn_rope_table_dev(ds->rope_swa, R, pos0, batch ? plist : NULL, hd_s,
                                       m->rope_base_swa, 0), "angles");
    const float scale = gemma ? m->attn_scale : 0.0f;

    for (L = 0; L < m->n_layers; L++) {
        const dev_layer *dl = &d->L[L];
        /* per layer (Gemma; constant elsewhere): head_dim, rotary table, window, whose cache */
        const uint32_t hdl = m->hd_layer[L], qd = nq * hdl, kd = nkv * hdl;
        const uint32_t ksrc = m->kv_src[L];
        const int shared = ksrc != L;
        const int local = gemma && m->swa[L];
        const uint32_t window = (local && m->swa_mode != WR_SWA_DISABLED) ? m->sliding_window : 0u;
        const float *tab = local ? ds->rope_swa : ds->rope;
        const uint32_t nr = local ? hd_s / 2 : n_rot;
        const uint32_t width = qd + (shared ? 0 : 2 * kd);
        const uint32_t flags = shared ? WR_HIP_QKV_Q_ONLY : (gemma ? WR_HIP_QKV_V_NORM : 0u);

        TRY(wr_hip_proj_rows_norm_dev(dl->wqkv, R, ds->resid, hidden, dl->attn_norm, m->rms_eps, NULL,
                                      ds->qkv, width), "attn norm + qkv projection");
        /* Q/K/V split, per-head norms, rotation and the cache append in one launch */
        if (fail_layer == (int)L) return dev_fail(e, "gqa (injected)", L, WR_ERR_INTERNAL);
        /* A decode step of the plain block (one row per session): the row step and
         * the attention in ONE launch where the library takes the shape -- the
         * same bits as the two calls below, one dependent launch less per layer. */
        int fused_done = 0;
        if (!prefill && !gemma && !shared && (batch || R == 1) &&
            __atomic_load_n(&m->dev->step_in_one_launch, __ATOMIC_RELAXED) >= 0) {
            wr_hip_kv *kvs[WR_BATCH_MAX];
            uint32_t at[WR_BATCH_MAX];
            for (uint32_t r = 0; r < R; r++) {
                kvs[r] = batch ? ss[r]->kv : ss[0]->kv;
                at[r] = batch ? ss[r]->pos : pos0;
            }
            rc = wr_hip_attn_append_decode_batched_dev(R, kvs, ksrc, at, ds->qkv, width, nq, dl->q_norm, dl->k_norm,
                                                       m->rms_eps, tab, nr, ds->attn, scale, window);
            if (rc == WR_HIP_ERR_UNSUPPORTED) {
                /* remembered for the model (the refusal is about its shapes as a
                 * rule); said once, because the step is slower from here on */
                if (__atomic_exchange_n(&m->dev->step_in_one_launch, -1, __ATOMIC_RELAXED) != -1)
                    wrh_logf(e, 1, "device layers: the decode step's row is not made inside the attention launch "
                                   "(shape or alignment not taken, or generic kernels forced): two launches per "
                                   "layer from here on");
            } else {
                if (rc != WR_HIP_OK) return dev_fail(e, "kv append + gqa", L, rc);
                __atomic_store_n(&m->dev->step_in_one_launch, 1, __ATOMIC_RELAXED);
                for (uint32_t r = 0; r < R; r++) (batch ? ss[r] : ss[0])->kv_rows[L] = at[r] + 1;
                fused_done = 1;
            }
        }
        if (fused_done) {
            /* nothing left to do for the attention of this layer */
        } else if (batch) {
            wr_hip_kv *kvs[WR_BATCH_MAX];
            uint32_t seq_k[WR_BATCH_MAX];
            uint32_t at[WR_BATCH_MAX];
            for (uint32_t r = 0; r < R; r++) {
                kvs[r] = ss[r]->kv;
                at[r] = ss[r]->pos;
                seq_k[r] = ss[r]->pos + 1;
            }
            TRY(wr_hip_rows_qkv_append_dev(ds->qkv, width, R, nq, dl->q_norm, shared ? NULL : dl->k_norm,
                                           m->rms_eps, tab, nr, R, kvs, ksrc, at, ds->q, flags),
                "qkv split + kv append");
            if (!shared)
                for (uint32_t r = 0; r < R; r++) ss[r]->kv_rows[L] = ss[r]->pos + 1;
            TRY(wr_hip_attn_decode_batched_dev(R, kvs, ksrc, seq_k, ds->q, ds->attn, nq, scale, window), "gqa");
        } else {
            wr_session *s = ss[0];
            wr_hip_kv *one[1] = {s->kv};
            /* Prompt rows: Q goes to the attention kernel as the binary16 operand the
             * kernel would make of it anyway (same bits, half the bytes); shapes that
             * form does not take keep F32 rows. */
            int q16 = 0;
            if (prefill && __atomic_load_n(&m->dev->prefill_q16, __ATOMIC_RELAXED) >= 0) {
                const int r16 = wr_hip_rows_qkv_append_q16_dev(ds->qkv, width, R, nq, dl->q_norm,
                                                               shared ? NULL : dl->k_norm, m->rms_eps, tab, nr, 1,
                                                               one, ksrc, &pos0, (uint16_t *)ds->q, scale, flags);
                if (r16 == WR_HIP_ERR_UNSUPPORTED) {
                    if (__atomic_exchange_n(&m->dev->prefill_q16, -1, __ATOMIC_RELAXED) != -1)
                        wrh_logf(e, 1, "device layers: prompt rows keep F32 query rows (the binary16 form does not "
                                       "take this shape or alignment, or generic kernels are forced)");
                } else {
                    if (r16 != WR_HIP_OK) return dev_fail(e, "qkv split + kv append", L, r16);
                    q16 = 1;
                }
            }
            if (!q16)
                TRY(wr_hip_rows_qkv_append_dev(ds->qkv, width, R, nq, dl->q_norm, shared ? NULL : dl->k_norm,
                                               m->rms_eps, tab, nr, 1, one, ksrc, &pos0, ds->q, flags),
                    "qkv split + kv append");
            if (!shared) s->kv_rows[L] = pos0 + R;
            if (q16) {
                TRY(wr_hip_attn_prefill_q16_dev(s->kv, ksrc, pos0, R, (const uint16_t *)ds->q, ds->attn, nq, scale,
                                                window), "gqa");
            } else if (prefill) {
                TRY(wr_hip_attn_prefill_dev(s->kv, ksrc, pos0, R, ds->q, ds->attn, nq, scale, window), "gqa");
            } else {
                const uint32_t sk = pos0 + 1;
                TRY(wr_hip_attn_decode_batched_dev(1, one, ksrc, &sk, ds->q, ds->attn, nq, scale, window), "gqa");
            }
        }
        if (gemma) {
            /* sandwich norms: the sublayer output is normalised, then joins the residual */
            TRY(wr_hip_proj_rows_dev(dl->wo, R, ds->attn, qd, NULL, ds->proj, hidden), "output projection");
            TRY(wr_hip_rows_rmsnorm_add_dev(ds->proj, hidden, dl->post_attn_norm, hidden, ds->resid, hidden, R,
                                            hidden, m->rms_eps), "post-attention norm + residual");
            TRY(wr_hip_proj_rows_norm_dev(dl->wgu, R, ds->resid, hidden, dl->ffn_norm, m->rms_eps, NULL,
                                          ds->gu, 2 * ffn), "ffn norm + gate/up projection");
            TRY(wr_hip_proj_rows_geglu_dev(dl->wdown, R, ds->gu, 2 * ffn, NULL, ds->proj, hidden),
                "geglu + down projection");
            TRY(wr_hip_rows_rmsnorm_add_dev(ds->proj, hidden, dl->post_ffw_norm, hidden, ds->resid, hidden, R,
                                            hidden, m->rms_eps), "post-ffn norm + residual");
        } else {
            TRY(wr_hip_proj_rows_dev(dl->wo, R, ds->attn, qd, ds->resid, ds->resid, hidden),
                "output projection");
            TRY(wr_hip_proj_rows_norm_dev(dl->wgu, R, ds->resid, hidden, dl->ffn_norm, m->rms_eps, NULL,
                                          ds->gu, 2 * ffn), "ffn norm + gate/up projection");
            TRY(wr_hip_proj_rows_swiglu_dev(dl->wdown, R, ds->gu, 2 * ffn, ds->resid, ds->resid, hidden),
                "swiglu + down projection");
        }
    }
    L = m->n_layers;
    if (logits_host && logit_rows) {
        TRY(wr_hip_proj_rows_norm_dev(d->lm_head, logit_rows, ds->resid, hidden, d->final_norm,
                                      m->rms_eps, NULL, ds->logits, m->vocab), "final norm + lm head");
        TRY(wr_hip_attn_d2h(logits_host, ds->logits, (size_t)logit_rows * m->vocab * sizeof(float)),
            "logits down");
    } else {
        /* both uploads above were synchronous: the host buffers are free again */
        if (next_rows) wrh_stage_next_rows(m, hs, next_rows, tokens + R, pos0 + R);
        TRY(wr_hip_attn_sync(), "sync");
    }
    return WR_OK;
}
