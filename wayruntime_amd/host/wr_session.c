/*
 * wr_session.c — sessions and the three decode entry points of the host
 * engine: wr_step, wr_prefill, wr_batch_step.
 *
 * The layer walk is the reference's Llama / Qwen3 block (reference:
 * src/core/session.c:440-534): RMSNorm, Q/K/V projections, per-head Q/K
 * RMSNorm (Qwen3), RoPE, KV append, attention, output projection, residual,
 * RMSNorm, SwiGLU, down projection, residual; final RMSNorm; LM head.
 * Here it runs over R rows at once (layer-major).  When the model's weights
 * are on the device (wr_device.c) the whole walk runs there; otherwise the
 * walk below runs on the host and the two steps in the middle go to the
 * device:
 *
 *   reference kv_append_row (session.c:139-154, called :483-486)
 *                                  -> wr_hip_attn_append_rope     (wr_prefill)
 *   reference wri_op_gqa_attention (kernels.c:1414, called session.c:493)
 *                                  -> wr_hip_attn_prefill         (wr_prefill)
 *   the two back to back, a decode step's pair (session.c:483-496)
 *                                  -> wr_hip_attn_append_decode          (wr_step)
 *                                  -> wr_hip_attn_append_decode_batched  (wr_batch_step)
 *   (a layer that reads another layer's cache appends nothing and calls
 *    wr_hip_attn_decode / wr_hip_attn_decode_batched)
 *
 * Contracts kept from the reference: one mutex per session held for the whole
 * call (session.c:581-595); a call that cannot complete consumes nothing —
 * position and per-layer cursors return to their entry values
 * (session.c:160-168, 589-592, 608-626; batch.c:146-175); WR_ERR_CTX_FULL and
 * out-of-vocabulary tokens are refused, never clamped; batched sessions are
 * locked in ascending address order (batch.c:106-120, 139-142); position and
 * status are published with release stores (session.c:590, 594).
 */
#define _POSIX_C_SOURCE 200809L
#include "wr_host.h"

#include <stdlib.h>
#include <string.h>

static int g_fail_attention_layer = -1;

void wrh_debug_fail_attention_at(int layer) { g_fail_attention_layer = layer; }

/* ------------------------------------------------------------- workspace -- */

static size_t round64(size_t n) { return (n + 15) & ~(size_t)15; }   /* floats */

int wrh_workspace_init(wrh_workspace *ws, const wr_model *m, uint32_t rows)
{
    memset(ws, 0, sizeof *ws);
    uint32_t hd_max = m->head_dim;
    for (uint32_t l = 0; l < m->n_layers; l++)
        if (m->hd_layer[l] > hd_max) hd_max = m->hd_layer[l];
    const size_t h = round64((size_t)rows * m->hidden);
    const size_t qd = round64((size_t)rows * m->n_q * hd_max);
    const size_t kd = round64((size_t)rows * m->n_kv * hd_max);
    const size_t fd = round64((size_t)rows * m->ffn);
    const size_t rd = round64((size_t)rows * hd_max);
    const size_t total = 3 * h + 2 * qd + 2 * kd + 2 * fd + 2 * rd;
    float *b = NULL;
    if (posix_memalign((void **)&b, 64, total * sizeof(float)) != 0 || !b) return WR_ERR_NOMEM;
    ws->block = b;
    ws->rows_cap = rows;
    ws->residual = b;  b += h;
    ws->normed = b;    b += h;
    ws->proj = b;      b += h;
    ws->q = b;         b += qd;
    ws->attn = b;      b += qd;
    ws->k = b;         b += kd;
    ws->v = b;         b += kd;
    ws->gate = b;      b += fd;
    ws->up = b;        b += fd;
    ws->rope = b;      b += rd;
    ws->rope_swa = b;
    return WR_OK;
}

void wrh_workspace_free(wrh_workspace *ws)
{
    free(ws->block);
    memset(ws, 0, sizeof *ws);
}

/* --------------------------------------------------------------- forward -- */

typedef enum { FWD_STEP, FWD_PREFILL, FWD_BATCH } fwd_mode;

static wr_status op_fail(wr_engine *e, const char *what, uint32_t layer, int rc)
{
    wrh_logf(e, 0, "session: %s failed at layer %u (rc=%d)", what, layer, rc);
    return (rc < 0) ? (wr_status)rc : WR_ERR_INTERNAL;
}

/* The Gemma-family block over R already embedded rows (reference:
 * src/core/session.c:251-437 without the per-layer-input fold): sandwich norms
 * (the sublayer outputs are normalised before they join the residual), Q/K
 * RMSNorm per head, rotary embedding with the layer's own base (partial on
 * global layers, full on sliding-window layers), a weightless RMSNorm of V
 * before the append, attention with scale 1.0 and the layer's window over the
 * layer's own cache or, for a KV-shared layer, over its source layer's
 * (whose rows for these positions are already in place: sources precede
 * their readers), GeGLU. */
static wr_status forward_rows_gemma(wr_model *m, wrh_workspace *ws, uint32_t R,
                                    wr_session *const *ss, uint32_t pos0, fwd_mode mode)
{
    wr_engine *e = m->engine;
    const uint32_t hidden = m->hidden, nq = m->n_q, nkv = m->n_kv, ffn = m->ffn;
    int rc;

    if (m->embed_scale != 0.0f) wrh_scale(ws->residual, (uint64_t)R * hidden, m->embed_scale);

    /* the rows' angles, once per kind of layer: global (partial rotary, the
     * model's base) and sliding-window (full rotary, its own base and head_dim) */
    const uint32_t hd_g = m->head_dim, hd_s = m->head_dim_swa ? m->head_dim_swa : m->head_dim;
    const uint32_t nrot_g = (m->n_rot_pairs >= 1 && m->n_rot_pairs < hd_g / 2) ? m->n_rot_pairs : hd_g / 2;
    const uint32_t nrot_s = hd_s / 2;
    for (uint32_t r = 0; r < R; r++) {
        const uint32_t p = (mode == FWD_BATCH) ? ss[r]->pos : pos0 + r;
        (void)wrh_rope_table(ws->rope + (size_t)r * 2 * nrot_g, hd_g, p, m->rope_base, m->n_rot_pairs);
        if (m->has_swa)
            (void)wrh_rope_table(ws->rope_swa + (size_t)r * 2 * nrot_s, hd_s, p, m->rope_base_swa, 0);
    }

    for (uint32_t L = 0; L < m->n_layers; L++) {
        const int local = m->swa[L];
        const uint32_t hd = m->hd_layer[L], qd = nq * hd, kd = nkv * hd;
        const uint32_t ksrc = m->kv_src[L];
        const int shared = (ksrc != L);
        const uint32_t window = (local && m->swa_mode != WR_SWA_DISABLED) ? m->sliding_window : 0u;
        const float *tab = local ? ws->rope_swa : ws->rope;
        const uint32_t n_rot = local ? nrot_s : nrot_g;
        const size_t ts = (size_t)2 * n_rot;

        wrh_rmsnorm(ws->residual, m->attn_norm[L].data, m->attn_norm[L].n, ws->normed, R, hidden,
                    m->rms_eps);
        wrh_matmul(e, ws->normed, R, hidden, &m->wq[L], ws->q, qd);
        wrh_rmsnorm(ws->q, m->q_norm[L].data, m->q_norm[L].n, ws->q, R * nq, hd, m->rms_eps);
        for (uint32_t r = 0; r < R; r++)
            wrh_rope_apply(ws->q + (size_t)r * qd, nq, hd, tab + r * ts, n_rot);
        if (!shared) {
            wrh_matmul(e, ws->normed, R, hidden, &m->wk[L], ws->k, kd);
            wrh_matmul(e, ws->normed, R, hidden, &m->wv[L], ws->v, kd);
            wrh_rmsnorm(ws->k, m->k_norm[L].data, m->k_norm[L].n, ws->k, R * nkv, hd, m->rms_eps);
            wrh_rmsnorm(ws->v, NULL, 0, ws->v, R * nkv, hd, m->rms_eps);
        }

        if (g_fail_attention_layer == (int)L) {
            g_fail_attention_layer = -1;
            return op_fail(e, "gqa (injected)", L, WR_ERR_INTERNAL);
        }
        if (mode == FWD_BATCH) {
            wr_hip_kv *kvs[WR_BATCH_MAX];
            uint32_t seq_k[WR_BATCH_MAX];
            const float *qp[WR_BATCH_MAX];
            float *op[WR_BATCH_MAX];
            const float *kp[WR_BATCH_MAX], *vp[WR_BATCH_MAX];
            uint32_t at[WR_BATCH_MAX];
            for (uint32_t r = 0; r < R; r++) {
                kvs[r] = ss[r]->kv;
                at[r] = ss[r]->pos;
                seq_k[r] = ss[r]->pos + 1;
                qp[r] = ws->q + (size_t)r * qd;
                op[r] = ws->attn + (size_t)r * qd;
                kp[r] = ws->k + (size_t)r * kd;
                vp[r] = ws->v + (size_t)r * kd;
            }
            if (!shared) {
                /* the rows' K rotated here like Q, then every session's append and the
                 * batched attention in one call: one round trip to the device per layer */
                for (uint32_t r = 0; r < R; r++)
                    wrh_rope_apply(ws->k + (size_t)r * kd, nkv, hd, tab + r * ts, n_rot);
                rc = wr_hip_attn_append_decode_batched(R, kvs, L, at, kp, vp, qp, op, nq, m->attn_scale,
                                                       window);
                if (rc == WR_HIP_ERR_CTX_FULL) return WR_ERR_CTX_FULL;
                if (rc == WR_HIP_OK)
                    for (uint32_t r = 0; r < R; r++) ss[r]->kv_rows[L] = ss[r]->pos + 1;
            } else {
                rc = wr_hip_attn_decode_batched(R, kvs, ksrc, seq_k, qp, op, nq, m->attn_scale, window);
            }
        } else if (mode == FWD_STEP && !shared) {
            wr_session *s = ss[0];
            wrh_rope_apply(ws->k, nkv, hd, tab, n_rot);
            rc = wr_hip_attn_append_decode(s->kv, L, pos0, ws->k, ws->v, ws->q, ws->attn, nq, m->attn_scale,
                                           window);
            if (rc == WR_HIP_ERR_CTX_FULL) return WR_ERR_CTX_FULL;
            if (rc == WR_HIP_OK) s->kv_rows[L] = pos0 + 1;
        } else {
            wr_session *s = ss[0];
            if (!shared) {
                rc = wr_hip_attn_append_rope(s->kv, L, pos0, R, ws->k, ws->v, tab, n_rot);
                if (rc != WR_HIP_OK) return (rc == WR_HIP_ERR_CTX_FULL) ? WR_ERR_CTX_FULL
                                                                         : op_fail(e, "kv append", L, rc);
                s->kv_rows[L] = pos0 + R;
            }
            if (mode == FWD_STEP)
                rc = wr_hip_attn_decode(s->kv, ksrc, pos0 + 1, ws->q, ws->attn, nq, m->attn_scale, window);
            else
                rc = wr_hip_attn_prefill(s->kv, ksrc, pos0, R, ws->q, ws->attn, nq, m->attn_scale,
                                         window);
        }
        if (rc != WR_HIP_OK) return op_fail(e, "gqa", L, rc);

        wrh_matmul(e, ws->attn, R, qd, &m->wo[L], ws->proj, hidden);
        wrh_rmsnorm(ws->proj, m->post_attn_norm[L].data, m->post_attn_norm[L].n, ws->proj, R, hidden,
                    m->rms_eps);
        wrh_add(ws->residual, ws->proj, (uint64_t)R * hidden);

        wrh_rmsnorm(ws->residual, m->ffn_norm[L].data, m->ffn_norm[L].n, ws->normed, R, hidden,
                    m->rms_eps);
        wrh_matmul(e, ws->normed, R, hidden, &m->w_gate[L], ws->gate, ffn);
        wrh_matmul(e, ws->normed, R, hidden, &m->w_up[L], ws->up, ffn);
        wrh_geglu(e, ws->gate, ws->up, (uint64_t)R * ffn);
        wrh_matmul(e, ws->gate, R, ffn, &m->w_down[L], ws->proj, hidden);
        wrh_rmsnorm(ws->proj, m->post_ffw_norm[L].data, m->post_ffw_norm[L].n, ws->proj, R, hidden,
                    m->rms_eps);
        wrh_add(ws->residual, ws->proj, (uint64_t)R * hidden);
    }
    wrh_rmsnorm(ws->residual, m->final_norm.data, m->final_norm.n, ws->normed, R, hidden,
                m->rms_eps);
    return WR_OK;
}

/* Forward pass minus the LM head over R rows.
 *   FWD_STEP / FWD_PREFILL: all rows belong to ss[0], at positions pos0 .. pos0+R-1
 *   FWD_BATCH:              row r belongs to ss[r], at position ss[r]->pos
 * On success the post-final-norm hidden rows are in ws->normed and each
 * session's per-layer cursors have advanced; positions are NOT advanced.  On
 * failure the caller rolls the cursors back. */
static wr_status forward_rows(wr_model *m, wrh_workspace *ws, uint32_t R, wr_session *const *ss,
                              const uint32_t *tokens, uint32_t pos0, fwd_mode mode)
{
    wr_engine *e = m->engine;
    const uint32_t hidden = m->hidden, hd = m->head_dim, nq = m->n_q, nkv = m->n_kv;
    const uint32_t qd = nq * hd, kd = nkv * hd, ffn = m->ffn;
    int rc;

    for (uint32_t r = 0; r < R; r++) {
        rc = wrh_embed(&m->embed, tokens[r], ws->residual + (size_t)r * hidden);
        if (rc != WR_OK) return op_fail(e, "embed", 0, rc);
    }

    if (m->is_gemma) return forward_rows_gemma(m, ws, R, ss, pos0, mode);

    for (uint32_t L = 0; L < m->n_layers; L++) {
        wrh_rmsnorm(ws->residual, m->attn_norm[L].data, m->attn_norm[L].n, ws->normed, R, hidden,
                    m->rms_eps);
        wrh_matmul(e, ws->normed, R, hidden, &m->wq[L], ws->q, qd);
        wrh_matmul(e, ws->normed, R, hidden, &m->wk[L], ws->k, kd);
        wrh_matmul(e, ws->normed, R, hidden, &m->wv[L], ws->v, kd);

        if (m->has_qk_norm) {      /* per-head RMSNorm before RoPE (Qwen3) */
            wrh_rmsnorm(ws->q, m->q_norm[L].data, m->q_norm[L].n, ws->q, R * nq, hd, m->rms_eps);
            wrh_rmsnorm(ws->k, m->k_norm[L].data, m->k_norm[L].n, ws->k, R * nkv, hd, m->rms_eps);
        }
        /* RoPE (reference: session.c:475-478): the rows' angles are worked out
         * once here and Q is rotated on the host.  A decode step rotates K here
         * too and hands both rows to the one append-and-attend call; a prompt's K
         * goes up as projected and is rotated on the device inside the append
         * (same arithmetic, same bits). */
        const uint32_t n_rot =
            (m->n_rot_pairs >= 1 && m->n_rot_pairs < hd / 2) ? m->n_rot_pairs : hd / 2;
        const size_t ts = (size_t)2 * n_rot;              /* table row: n_rot (cos, sin) pairs */
        for (uint32_t r = 0; r < R; r++) {
            const uint32_t p = (mode == FWD_BATCH) ? ss[r]->pos : pos0 + r;
            (void)wrh_rope_table(ws->rope + r * ts, hd, p, m->rope_base, m->n_rot_pairs);
            wrh_rope_apply(ws->q + (size_t)r * qd, nq, hd, ws->rope + r * ts, n_rot);
        }

        /* Append after RoPE, then attend: the new token attends to itself. */
        if (g_fail_attention_layer == (int)L) {
            g_fail_attention_layer = -1;
            return op_fail(e, "gqa (injected)", L, WR_ERR_INTERNAL);
        }
        if (mode == FWD_BATCH) {
            wr_hip_kv *kvs[WR_BATCH_MAX];
            const float *qp[WR_BATCH_MAX];
            float *op[WR_BATCH_MAX];
            const float *kp[WR_BATCH_MAX], *vp[WR_BATCH_MAX];
            uint32_t at[WR_BATCH_MAX];
            for (uint32_t r = 0; r < R; r++) {
                wrh_rope_apply(ws->k + (size_t)r * kd, nkv, hd, ws->rope + r * ts, n_rot);
                kvs[r] = ss[r]->kv;
                at[r] = ss[r]->pos;
                qp[r] = ws->q + (size_t)r * qd;
                op[r] = ws->attn + (size_t)r * qd;
                kp[r] = ws->k + (size_t)r * kd;
                vp[r] = ws->v + (size_t)r * kd;
            }
            /* every session's append and the batched attention in one call */
            rc = wr_hip_attn_append_decode_batched(R, kvs, L, at, kp, vp, qp, op, nq, 0.0f, 0);
            if (rc == WR_HIP_ERR_CTX_FULL) return WR_ERR_CTX_FULL;
            if (rc == WR_HIP_OK)
                for (uint32_t r = 0; r < R; r++) ss[r]->kv_rows[L] = ss[r]->pos + 1;
        } else if (mode == FWD_STEP) {
            wr_session *s = ss[0];
            wrh_rope_apply(ws->k, nkv, hd, ws->rope, n_rot);
            rc = wr_hip_attn_append_decode(s->kv, L, pos0, ws->k, ws->v, ws->q, ws->attn, nq, 0.0f, 0);
            if (rc == WR_HIP_ERR_CTX_FULL) return WR_ERR_CTX_FULL;
            if (rc == WR_HIP_OK) s->kv_rows[L] = pos0 + 1;
        } else {
            wr_session *s = ss[0];
            rc = wr_hip_attn_append_rope(s->kv, L, pos0, R, ws->k, ws->v, ws->rope, n_rot);
            if (rc != WR_HIP_OK) return (rc == WR_HIP_ERR_CTX_FULL) ? WR_ERR_CTX_FULL
                                                                     : op_fail(e, "kv append", L, rc);
            s->kv_rows[L] = pos0 + R;
            rc = wr_hip_attn_prefill(s->kv, L, pos0, R, ws->q, ws->attn, nq, 0.0f, 0);
        }
        if (rc != WR_HIP_OK) return op_fail(e, "gqa", L, rc);

        wrh_matmul(e, ws->attn, R, qd, &m->wo[L], ws->proj, hidden);
        wrh_add(ws->residual, ws->proj, (uint64_t)R * hidden);

        wrh_rmsnorm(ws->residual, m->ffn_norm[L].data, m->ffn_norm[L].n, ws->normed, R, hidden,
                    m->rms_eps);
        wrh_matmul(e, ws->normed, R, hidden, &m->w_gate[L], ws->gate, ffn);
        wrh_matmul(e, ws->normed, R, hidden, &m->w_up[L], ws->up, ffn);
        wrh_swiglu(e, ws->gate, ws->up, (uint64_t)R * ffn);
        wrh_matmul(e, ws->gate, R, ffn, &m->w_down[L], ws->proj, hidden);
        wrh_add(ws->residual, ws->proj, (uint64_t)R * hidden);
    }
    wrh_rmsnorm(ws->residual, m->final_norm.data, m->final_norm.n, ws->normed, R, hidden,
                m->rms_eps);
    return WR_OK;
}

/* The injected failure, taken once: the layer to fail at, or -1. */
static int take_fail_layer(const wr_model *m)
{
    const int fl = g_fail_attention_layer;
    if (fl >= 0 && (uint32_t)fl < m->n_layers) g_fail_attention_layer = -1;
    return fl;
}

/* Cursors back to the committed position (reference: session.c:160-168).
 * Rows above the cursor stay in device memory and are never read. */
static void kv_rollback(wr_session *s)
{
    for (uint32_t L = 0; L < s->model->n_layers; L++) s->kv_rows[L] = s->pos;
}

/* ------------------------------------------------------------- lifecycle -- */

wr_status wr_session_create(wr_model *m, const wr_session_params *params, wr_session **out)
{
    if (!out) return WR_ERR_INVAL;
    *out = NULL;
    if (!m) return WR_ERR_INVAL;
    if (m->n_layers == 0 || m->n_kv == 0 || m->n_q == 0 || m->head_dim == 0 || m->hidden == 0 ||
        m->vocab == 0 || m->max_context == 0)
        return WR_ERR_INVAL;
    uint32_t max_ctx = m->max_context;
    if (params && params->max_context) {
        if (params->max_context > m->max_context) return WR_ERR_INVAL;
        max_ctx = params->max_context;
    }
    if (max_ctx > WR_HIP_ATTN_MAX_SEQ) return WR_ERR_LIMIT;

    wr_session *s = calloc(1, sizeof *s);
    if (!s) return WR_ERR_NOMEM;
    s->model = m;
    s->max_context = max_ctx;
    s->last_status = WR_OK;
    uint32_t hds[WRH_MAX_LAYERS];          /* 0 = no cache of its own (KV-shared layer) */
    for (uint32_t L = 0; L < m->n_layers; L++) hds[L] = (m->kv_src[L] == L) ? m->hd_layer[L] : 0;
    int rc = wr_hip_attn_kv_create(m->n_layers, hds, m->n_kv, max_ctx, &s->kv);
    if (rc != WR_HIP_OK) {
        wrh_logf(m->engine, 0, "session: device cache allocation failed (rc=%d)", rc);
        free(s);
        return (wr_status)rc;
    }
    s->logits = malloc((size_t)m->vocab * sizeof(float));
    if (!s->logits || wrh_workspace_init(&s->ws1, m, 1) != WR_OK ||
        (m->dev && wrh_devspace_init(&s->ds1, m, 1, 1) != WR_OK)) {
        free(s->logits);
        wrh_workspace_free(&s->ws1);
        wr_hip_attn_kv_destroy(s->kv);
        free(s);
        return WR_ERR_NOMEM;
    }
    pthread_mutex_init(&s->lock, NULL);
    pthread_mutex_lock(&m->lock);
    m->session_refs++;
    pthread_mutex_unlock(&m->lock);
    *out = s;
    return WR_OK;
}

void wr_session_destroy(wr_session *s)
{
    if (!s) return;
    wr_model *m = s->model;
    pthread_mutex_lock(&m->lock);
    if (m->session_refs) m->session_refs--;
    pthread_mutex_unlock(&m->lock);
    wr_hip_attn_kv_destroy(s->kv);
    wrh_workspace_free(&s->ws1);
    wrh_devspace_free(&s->ds1);
    free(s->logits);
    pthread_mutex_destroy(&s->lock);
    free(s);
}

uint32_t wr_session_pos(const wr_session *s)
{
    return s ? __atomic_load_n(&s->pos, __ATOMIC_ACQUIRE) : 0;
}

uint32_t wr_session_max_context(const wr_session *s) { return s ? s->max_context : 0; }

wr_status wr_session_status(const wr_session *s)
{
    return s ? __atomic_load_n(&s->last_status, __ATOMIC_ACQUIRE) : WR_ERR_INVAL;
}

/* ------------------------------------------------------------------ step -- */

const float *wr_step(wr_session *s, uint32_t token)
{
    if (!s) return NULL;
    wr_model *m = s->model;
    pthread_mutex_lock(&s->lock);
    wr_status st;
    if (s->pos >= s->max_context) {
        st = WR_ERR_CTX_FULL;                              /* consumed nothing */
    } else {
        wr_session *one[1] = {s};
        if (m->dev) {
            st = wrh_forward_rows_device(m, &s->ws1, &s->ds1, 1, one, &token, s->pos, 0, 0,
                                         take_fail_layer(m), s->logits, 1, 0);
            if (st == WR_OK && m->is_gemma) wrh_softcap(s->logits, m->vocab, m->logit_softcap);
        } else {
            st = forward_rows(m, &s->ws1, 1, one, &token, s->pos, FWD_STEP);
            if (st == WR_OK) {
                wrh_matmul(m->engine, s->ws1.normed, 1, m->hidden, &m->lm_head, s->logits, m->vocab);
                if (m->is_gemma) wrh_softcap(s->logits, m->vocab, m->logit_softcap);
            }
        }
        if (st == WR_OK)
            __atomic_store_n(&s->pos, s->pos + 1, __ATOMIC_RELEASE);
        else
            kv_rollback(s);
    }
    __atomic_store_n(&s->last_status, st, __ATOMIC_RELEASE);
    pthread_mutex_unlock(&s->lock);
    return (st == WR_OK) ? s->logits : NULL;
}

/* --------------------------------------------------------------- prefill -- */

int wr_prefill(wr_session *s, const uint32_t *ids, uint32_t n)
{
    if (!s) return WR_ERR_INVAL;
    if (n == 0) return 0;
    if (!ids) return WR_ERR_INVAL;
    wr_model *m = s->model;

    pthread_mutex_lock(&s->lock);
    wr_status st = WR_OK;
    const uint32_t pos_entry = s->pos;
    if ((uint64_t)s->pos + n > s->max_context) {
        st = WR_ERR_CTX_FULL;                              /* all or nothing */
    } else {
        /* a token outside the vocabulary anywhere in the prompt refuses the
         * whole call before anything is written */
        for (uint32_t i = 0; i < n && st == WR_OK; i++)
            if (ids[i] >= m->vocab) st = WR_ERR_INVAL;
        const uint32_t cap = m->dev ? WRH_DEVICE_PREFILL_CHUNK : WRH_PREFILL_CHUNK;
        const uint32_t chunk = n < cap ? n : cap;
        wr_session *one[1] = {s};
        if (st == WR_OK && m->dev) {
            /* device walk: scratch kept by the model between calls */
            struct wrh_scratch *sc = wrh_scratch_acquire(m, 1, chunk, 0);
            if (!sc) st = WR_ERR_NOMEM;
            for (uint32_t done = 0; done < n && st == WR_OK; done += chunk) {
                const uint32_t rows = (n - done < chunk) ? n - done : chunk;
                const uint32_t left = n - done - rows;                 /* staged while the device works */
                st = wrh_forward_rows_device(m, &sc->ws, &sc->ds, rows, one, ids + done, s->pos, 0, 1,
                                             take_fail_layer(m), NULL, 0, left < chunk ? left : chunk);
                if (st == WR_OK) __atomic_store_n(&s->pos, s->pos + rows, __ATOMIC_RELEASE);
            }
            wrh_scratch_release(m, sc);
        } else if (st == WR_OK) {
            wrh_workspace ws;
            if (wrh_workspace_init(&ws, m, chunk) != WR_OK) st = WR_ERR_NOMEM;
            if (st == WR_OK) {
                for (uint32_t done = 0; done < n && st == WR_OK; done += chunk) {
                    const uint32_t rows = (n - done < chunk) ? n - done : chunk;
                    st = forward_rows(m, &ws, rows, one, ids + done, s->pos, FWD_PREFILL);
                    if (st == WR_OK) __atomic_store_n(&s->pos, s->pos + rows, __ATOMIC_RELEASE);
                }
                wrh_workspace_free(&ws);
            }
        }
        if (st != WR_OK) {
            __atomic_store_n(&s->pos, pos_entry, __ATOMIC_RELEASE);
            kv_rollback(s);
        }
    }
    __atomic_store_n(&s->last_status, st, __ATOMIC_RELEASE);
    pthread_mutex_unlock(&s->lock);
    return (st == WR_OK) ? (int)n : (int)st;
}

/* ----------------------------------------------------------------- batch -- */

static void sort_by_address(wr_session **a, uint32_t n)
{
    for (uint32_t i = 1; i < n; i++) {
        wr_session *key = a[i];
        uint32_t j = i;
        for (; j > 0 && (uintptr_t)a[j - 1] > (uintptr_t)key; j--) a[j] = a[j - 1];
        a[j] = key;
    }
}

int wr_batch_step(wr_session *const *sessions, const uint32_t *tokens, uint32_t n,
                  const float **logits_out)
{
    if (!sessions || !tokens) return WR_ERR_INVAL;
    if (n == 0 || n > WR_BATCH_MAX) return WR_ERR_LIMIT;
    wr_model *m = sessions[0] ? sessions[0]->model : NULL;
    if (!m) return WR_ERR_STATE;
    for (uint32_t i = 0; i < n; i++) {
        if (!sessions[i] || sessions[i]->model != m) return WR_ERR_INVAL;
        for (uint32_t j = 0; j < i; j++)
            if (sessions[i] == sessions[j]) return WR_ERR_INVAL;
    }
    wr_session *locked[WR_BATCH_MAX];
    for (uint32_t i = 0; i < n; i++) locked[i] = sessions[i];
    sort_by_address(locked, n);
    for (uint32_t i = 0; i < n; i++) pthread_mutex_lock(&locked[i]->lock);

    wr_status st = WR_OK;
    for (uint32_t i = 0; i < n && st == WR_OK; i++)
        if (sessions[i]->pos >= sessions[i]->max_context) st = WR_ERR_CTX_FULL;

    wrh_workspace ws;
    float *big = NULL;
    int have_ws = 0;
    struct wrh_scratch *sc = NULL;
    if (st == WR_OK && m->dev) {
        /* device walk: rows, device scratch and page-locked logits kept by the model */
        sc = wrh_scratch_acquire(m, 0, n, n);
        if (!sc) st = WR_ERR_NOMEM;
        if (st == WR_OK)
            st = wrh_forward_rows_device(m, &sc->ws, &sc->ds, n, sessions, tokens, 0, 1, 0,
                                         take_fail_layer(m), sc->logits_host, n, 0);
        big = sc ? sc->logits_host : NULL;
    } else if (st == WR_OK) {
        if (wrh_workspace_init(&ws, m, n) == WR_OK) have_ws = 1;
        else st = WR_ERR_NOMEM;
        if (st == WR_OK) {
            big = malloc((size_t)n * m->vocab * sizeof(float));
            if (!big) st = WR_ERR_NOMEM;
        }
        if (st == WR_OK) st = forward_rows(m, &ws, n, sessions, tokens, 0, FWD_BATCH);
    }
    if (st == WR_OK) {
        /* one LM-head product for all n rows (reference: batch.c:45-104), then demux */
        if (!m->dev) wrh_matmul(m->engine, ws.normed, n, m->hidden, &m->lm_head, big, m->vocab);
        if (m->is_gemma) wrh_softcap(big, (uint64_t)n * m->vocab, m->logit_softcap);
        {
            /* 600 KB a session at a vocabulary of 150 000: one thread per session */
            const int threads = (m->engine && m->engine->n_threads > 0) ? m->engine->n_threads : 1;
#pragma omp parallel for num_threads(threads) schedule(static) if (n >= 4)
            for (uint32_t i = 0; i < n; i++)
                memcpy(sessions[i]->logits, big + (size_t)i * m->vocab, (size_t)m->vocab * sizeof(float));
        }
        for (uint32_t i = 0; i < n; i++)
            __atomic_store_n(&sessions[i]->pos, sessions[i]->pos + 1, __ATOMIC_RELEASE);
    } else {
        for (uint32_t i = 0; i < n; i++) kv_rollback(sessions[i]);      /* nobody advanced */
    }
    if (sc) wrh_scratch_release(m, sc);
    else free(big);
    if (have_ws) wrh_workspace_free(&ws);

    for (uint32_t i = 0; i < n; i++)
        __atomic_store_n(&sessions[i]->last_status, st, __ATOMIC_RELEASE);
    for (uint32_t i = n; i > 0; i--) pthread_mutex_unlock(&locked[i - 1]->lock);
    if (st != WR_OK) return (int)st;
    if (logits_out)
        for (uint32_t i = 0; i < n; i++) logits_out[i] = sessions[i]->logits;
    return (int)n;
}
