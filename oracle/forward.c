/*
 * CPU oracle, test infrastructure only: f32 forward primitives, the few-row
 * dequant-GEMM, block-causal verify attention, the drafter attention, and the
 * synthetic target / drafter forwards built from them.
 *
 * Follows crates/qwen-llm/src/forward.rs: rms_norm :1256-1264, silu :1278-1281,
 * softmax_in_place :1298-1309, mat_vec :1321-1334, rope_in_place :1347-1371,
 * single_token_with_hidden :96-163, ffn / ffn_moe :725-824, attn_step :834-932
 * (without the q-gate and with full-width RoPE, as the synthetic shapes are plain
 * Qwen3-style blocks), dflash_draft :380-662.  K and V are rounded to f16 when
 * they enter the cache, which is what the GPU session stores
 * (kernels/elementwise.metal:674-685).
 *
 * Sums are sequential f32 folds in index order, exactly as the reference's loops;
 * compile with -ffp-contract=off.
 */
#include "dflash_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>

void orc_rms_norm(const float *x, const float *w, size_t n, float eps, float *out) {
    float sum = 0.0f;
    for (size_t i = 0; i < n; i++) sum += x[i] * x[i];
    float mean_sq = sum / (float)n;
    float scale = 1.0f / sqrtf(mean_sq + eps);
    for (size_t i = 0; i < n; i++) out[i] = x[i] * scale * w[i];
}

float orc_silu(float x) { return x / (1.0f + expf(-x)); }
static float sigmoidf_(float x) { return 1.0f / (1.0f + expf(-x)); }

void orc_softmax_in_place(float *x, size_t n) {
    float mx = -INFINITY;
    for (size_t i = 0; i < n; i++) mx = fmaxf(mx, x[i]);
    float sum = 0.0f;
    for (size_t i = 0; i < n; i++) {
        x[i] = expf(x[i] - mx);
        sum += x[i];
    }
    float inv = 1.0f / sum;
    for (size_t i = 0; i < n; i++) x[i] *= inv;
}

void orc_mat_vec(const float *w, size_t n_in, size_t n_out, const float *x, float *y) {
    for (size_t o = 0; o < n_out; o++) {
        const float *row = w + o * n_in;
        float s = 0.0f;
        for (size_t i = 0; i < n_in; i++) s += x[i] * row[i];
        y[o] = s;
    }
}

void orc_rope_in_place(float *buf, size_t n_heads, size_t head_dim, size_t n_rot, uint32_t position,
                       float theta_base) {
    float pos = (float)position;
    size_t half = n_rot / 2;
    for (size_t h = 0; h < n_heads; h++) {
        float *p = buf + h * head_dim;
        for (size_t i = 0; i < half; i++) {
            float exponent = (float)(2 * i) / (float)n_rot;
            float freq = pos / powf(theta_base, exponent);
            float s = sinf(freq), c = cosf(freq);
            float a = p[i], b = p[i + half];
            p[i] = a * c - b * s;
            p[i + half] = a * s + b * c;
        }
    }
}

/* y[c][r] = sum_k deq(W[r][k]) x[c][k]: the reference's CPU form is dequant_to_f32
 * followed by mat_vec per row of x (forward.rs:1321-1334); here a weight row is
 * dequantised once and dotted with every x row, which is the same arithmetic. */
int orc_gemm_fewrow(int type, const uint8_t *w, const float *x, float *y, size_t n_in, size_t n_out,
                    size_t n_rows) {
    size_t rb = orc_row_bytes(type, n_in);
    if (rb == 0) return -1;
    int bad = 0;
#pragma omp parallel
    {
        float *row = (float *)malloc(n_in * sizeof(float));
#pragma omp for schedule(static)
        for (long o = 0; o < (long)n_out; o++) {
            if (orc_dequant(type, w + (size_t)o * rb, n_in, row)) {
                bad = 1;
                continue;
            }
            for (size_t c = 0; c < n_rows; c++) {
                const float *xr = x + c * n_in;
                float s = 0.0f;
                for (size_t i = 0; i < n_in; i++) s += xr[i] * row[i];
                y[c * n_out + (size_t)o] = s;
            }
        }
        free(row);
    }
    return bad ? -1 : 0;
}

/* forward.rs:893-922 applied per block row: row i attends cache positions [0, ctx_len+i] */
void orc_attn_verify_block(const float *q, const uint16_t *k_cache, const uint16_t *v_cache, size_t ctx_len,
                           size_t n_rows, size_t n_q, size_t n_kv, size_t hd, float scale, float *out) {
    size_t group = n_q / n_kv;
    size_t kv_dim = n_kv * hd;
#pragma omp parallel for collapse(2) schedule(dynamic, 1)
    for (long r = 0; r < (long)n_rows; r++) {
        for (long qh = 0; qh < (long)n_q; qh++) {
            size_t n_pos = ctx_len + (size_t)r + 1;
            size_t kvh = (size_t)qh / group;
            const float *qs = q + ((size_t)r * n_q + (size_t)qh) * hd;
            float *scores = (float *)malloc(n_pos * sizeof(float));
            for (size_t p = 0; p < n_pos; p++) {
                const uint16_t *ks = k_cache + p * kv_dim + kvh * hd;
                float s = 0.0f;
                for (size_t i = 0; i < hd; i++) s += qs[i] * orc_f16_to_f32(ks[i]);
                scores[p] = s * scale;
            }
            orc_softmax_in_place(scores, n_pos);
            float *o = out + ((size_t)r * n_q + (size_t)qh) * hd;
            for (size_t i = 0; i < hd; i++) o[i] = 0.0f;
            for (size_t p = 0; p < n_pos; p++) {
                const uint16_t *vs = v_cache + p * kv_dim + kvh * hd;
                float w = scores[p];
                for (size_t i = 0; i < hd; i++) o[i] += w * orc_f16_to_f32(vs[i]);
            }
            free(scores);
        }
    }
}

/* forward.rs:559-606 */
void orc_attn_draft(const float *q, const float *k_ctx, const float *v_ctx, const float *k_noise,
                    const float *v_noise, const int32_t *pos_ctx, size_t ctx_len, size_t n, size_t n_q,
                    size_t n_kv, size_t hd, uint32_t noise_start_pos, int causal, uint32_t swa_window,
                    float *out) {
    size_t group = n_q / n_kv;
    size_t kv_dim = n_kv * hd, q_dim = n_q * hd;
    size_t total = ctx_len + n;
    float kq_scale = 1.0f / sqrtf((float)hd);
#pragma omp parallel for collapse(2) schedule(dynamic, 1)
    for (long qi = 0; qi < (long)n; qi++) {
        for (long qh = 0; qh < (long)n_q; qh++) {
            uint32_t q_pos = noise_start_pos + (uint32_t)qi;
            size_t kvh = (size_t)qh / group;
            const float *qs = q + (size_t)qi * q_dim + (size_t)qh * hd;
            float *scores = (float *)malloc(total * sizeof(float));
            for (size_t k = 0; k < total; k++) {
                scores[k] = -INFINITY;
                uint32_t k_pos = k < ctx_len ? (uint32_t)pos_ctx[k] : noise_start_pos + (uint32_t)(k - ctx_len);
                uint32_t dist = q_pos > k_pos ? q_pos - k_pos : k_pos - q_pos;
                int allowed = (!causal || k_pos <= q_pos) && (swa_window == 0 || dist < swa_window);
                if (!allowed) continue;
                const float *ks = (k < ctx_len ? k_ctx + k * kv_dim : k_noise + (k - ctx_len) * kv_dim) + kvh * hd;
                float s = 0.0f;
                for (size_t d = 0; d < hd; d++) s += qs[d] * ks[d];
                scores[k] = s * kq_scale;
            }
            orc_softmax_in_place(scores, total);
            float *o = out + (size_t)qi * q_dim + (size_t)qh * hd;
            for (size_t d = 0; d < hd; d++) o[d] = 0.0f;
            for (size_t k = 0; k < total; k++) {
                float w = scores[k];
                if (!isfinite(w) || w == 0.0f) continue;
                const float *vs = (k < ctx_len ? v_ctx + k * kv_dim : v_noise + (k - ctx_len) * kv_dim) + kvh * hd;
                for (size_t d = 0; d < hd; d++) o[d] += w * vs[d];
            }
            free(scores);
        }
    }
}

/* ---------- synthetic decoder ---------- */

/* y[n_rows][n_out] = x[n_rows][n_in] . W^T over quant blocks */
static int qmat(const orc_qtensor *t, const float *x, float *y, size_t n_in, size_t n_out, size_t n_rows) {
    return orc_gemm_fewrow(t->type, t->data, x, y, n_in, n_out, n_rows);
}

static int qmat_expert(const orc_qtensor *t, size_t expert, const float *x, float *y, size_t n_in, size_t n_out) {
    size_t per = orc_row_bytes(t->type, n_in) * n_out;
    return orc_gemm_fewrow(t->type, t->data + expert * per, x, y, n_in, n_out, 1);
}

/* forward.rs:725-748 */
static int ffn_dense(const orc_layer *L, const float *x, size_t h, size_t f, float *out) {
    float *g = (float *)malloc(f * sizeof(float)), *u = (float *)malloc(f * sizeof(float));
    int rc = qmat(&L->gate, x, g, h, f, 1) | qmat(&L->up, x, u, h, f, 1);
    for (size_t i = 0; i < f; i++) g[i] = orc_silu(g[i]) * u[i];
    rc |= qmat(&L->down, g, out, f, h, 1);
    free(g);
    free(u);
    return rc;
}

/* Smallest relative gap between the last expert picked and the best one left out, over every routing decision since
 * the last orc_router_margin_take(): lets a test tell a wrong pick from a near tie that an f16-operand router may
 * break the other way.  Test scaffolding; not part of the reference. */
static float g_router_margin = INFINITY;
float orc_router_margin_take(void) {
    float m = g_router_margin;
    g_router_margin = INFINITY;
    return m;
}

/* forward.rs:749-824 */
static int ffn_moe(const orc_model_cfg *c, const orc_layer *L, const float *x, float *out) {
    size_t h = (size_t)c->hidden, ne = (size_t)c->n_expert;
    size_t used = (size_t)(c->n_expert_used < c->n_expert ? c->n_expert_used : c->n_expert);
    size_t fe = (size_t)c->ffn_expert, fs = (size_t)c->ffn_shared;
    float *probs = (float *)malloc(ne * sizeof(float));
    int rc = qmat(&L->router, x, probs, h, ne, 1);
    orc_softmax_in_place(probs, ne);
    /* top-k by probability, ties to the lower expert id (stable selection) */
    size_t *pick = (size_t *)malloc(used * sizeof(size_t));
    char *taken = (char *)calloc(ne, 1);
    for (size_t k = 0; k < used; k++) {
        size_t best = SIZE_MAX;
        for (size_t e = 0; e < ne; e++) {
            if (taken[e]) continue;
            if (best == SIZE_MAX || probs[e] > probs[best]) best = e;
        }
        taken[best] = 1;
        pick[k] = best;
    }
    if (used < ne) {
        float runner_up = 0.0f;
        for (size_t e = 0; e < ne; e++)
            if (!taken[e] && probs[e] > runner_up) runner_up = probs[e];
        float last = probs[pick[used - 1]];
        float rel = last > 0.0f ? (last - runner_up) / last : 0.0f;
        if (rel < g_router_margin) g_router_margin = rel;
    }
    float weight_sum = 0.0f;
    for (size_t k = 0; k < used; k++) weight_sum += probs[pick[k]];
    float floor14;
    uint32_t fb = 0x38800000u;
    memcpy(&floor14, &fb, 4);
    weight_sum = fmaxf(weight_sum, floor14);
    for (size_t i = 0; i < h; i++) out[i] = 0.0f;
    float *g = (float *)malloc((fe > fs ? fe : fs) * sizeof(float));
    float *u = (float *)malloc((fe > fs ? fe : fs) * sizeof(float));
    float *eo = (float *)malloc(h * sizeof(float));
    for (size_t k = 0; k < used; k++) {
        size_t e = pick[k];
        float weight = probs[e] / weight_sum;
        rc |= qmat_expert(&L->gate_exps, e, x, g, h, fe) | qmat_expert(&L->up_exps, e, x, u, h, fe);
        for (size_t i = 0; i < fe; i++) g[i] = orc_silu(g[i]) * u[i];
        rc |= qmat_expert(&L->down_exps, e, g, eo, fe, h);
        for (size_t i = 0; i < h; i++) out[i] += weight * eo[i];
    }
    float dot = 0.0f;
    for (size_t i = 0; i < h; i++) dot += x[i] * L->shexp_gate[i];
    float sg = sigmoidf_(dot);
    rc |= qmat(&L->gate, x, g, h, fs, 1) | qmat(&L->up, x, u, h, fs, 1);
    for (size_t i = 0; i < fs; i++) g[i] = orc_silu(g[i]) * u[i];
    rc |= qmat(&L->down, g, eo, fs, h, 1);
    for (size_t i = 0; i < h; i++) out[i] += sg * eo[i];
    free(probs);
    free(pick);
    free(taken);
    free(g);
    free(u);
    free(eo);
    return rc;
}

static int embed(const orc_qtensor *t, int32_t token, size_t h, float *out) {
    return orc_dequant(t->type, t->data + (size_t)token * orc_row_bytes(t->type, h), h, out);
}

int orc_target_verify(const orc_model *m, const int32_t *tokens, size_t n, size_t start_pos, uint16_t *k_cache,
                      uint16_t *v_cache, size_t kv_capacity, float *logits, const int32_t *tap_layers,
                      size_t n_tap, float *hidden_capture) {
    const orc_model_cfg *c = &m->cfg;
    size_t h = (size_t)c->hidden, hd = (size_t)c->head_dim, nq = (size_t)c->n_q, nkv = (size_t)c->n_kv;
    size_t q_dim = nq * hd, kv_dim = nkv * hd, V = (size_t)c->vocab, group = nq / nkv;
    if (start_pos + n > kv_capacity) return -1;
    float *x = (float *)malloc(h * sizeof(float)), *cur = (float *)malloc(h * sizeof(float));
    float *qb = (float *)malloc(q_dim * sizeof(float)), *kb = (float *)malloc(kv_dim * sizeof(float));
    float *vb = (float *)malloc(kv_dim * sizeof(float)), *ao = (float *)malloc(q_dim * sizeof(float));
    float *mix = (float *)malloc(h * sizeof(float)), *tmp = (float *)malloc((hd > h ? hd : h) * sizeof(float));
    float scale = 1.0f / sqrtf((float)hd);
    int rc = 0;
    for (size_t r = 0; r < n; r++) {
        int32_t tok = tokens[r];
        if (tok < 0 || (size_t)tok >= V) {
            rc = -2;
            break;
        }
        uint32_t position = (uint32_t)(start_pos + r);
        rc |= embed(&m->token_embd, tok, h, x);
        for (size_t il = 0; il < (size_t)c->n_layers; il++) {
            const orc_layer *L = &m->layers[il];
            orc_rms_norm(x, L->attn_norm, h, c->eps, cur);
            rc |= qmat(&L->wq, cur, qb, h, q_dim, 1) | qmat(&L->wk, cur, kb, h, kv_dim, 1) |
                  qmat(&L->wv, cur, vb, h, kv_dim, 1);
            for (size_t hi = 0; hi < nq; hi++) {
                orc_rms_norm(qb + hi * hd, L->q_norm, hd, c->eps, tmp);
                memcpy(qb + hi * hd, tmp, hd * sizeof(float));
            }
            for (size_t hi = 0; hi < nkv; hi++) {
                orc_rms_norm(kb + hi * hd, L->k_norm, hd, c->eps, tmp);
                memcpy(kb + hi * hd, tmp, hd * sizeof(float));
            }
            orc_rope_in_place(qb, nq, hd, hd, position, c->rope_theta);
            orc_rope_in_place(kb, nkv, hd, hd, position, c->rope_theta);
            uint16_t *kc = k_cache + il * kv_capacity * kv_dim, *vc = v_cache + il * kv_capacity * kv_dim;
            for (size_t i = 0; i < kv_dim; i++) {
                kc[(size_t)position * kv_dim + i] = orc_f32_to_f16(kb[i]);
                vc[(size_t)position * kv_dim + i] = orc_f32_to_f16(vb[i]);
            }
            size_t n_pos = (size_t)position + 1;
            float *scores = (float *)malloc(n_pos * sizeof(float));
            for (size_t qh = 0; qh < nq; qh++) {
                size_t kvh = qh / group;
                const float *qs = qb + qh * hd;
                for (size_t p = 0; p < n_pos; p++) {
                    const uint16_t *ks = kc + p * kv_dim + kvh * hd;
                    float s = 0.0f;
                    for (size_t i = 0; i < hd; i++) s += qs[i] * orc_f16_to_f32(ks[i]);
                    scores[p] = s * scale;
                }
                orc_softmax_in_place(scores, n_pos);
                float *o = ao + qh * hd;
                for (size_t i = 0; i < hd; i++) o[i] = 0.0f;
                for (size_t p = 0; p < n_pos; p++) {
                    const uint16_t *vs = vc + p * kv_dim + kvh * hd;
                    float w = scores[p];
                    for (size_t i = 0; i < hd; i++) o[i] += w * orc_f16_to_f32(vs[i]);
                }
            }
            free(scores);
            rc |= qmat(&L->wo, ao, mix, q_dim, h, 1);
            for (size_t i = 0; i < h; i++) x[i] += mix[i];
            orc_rms_norm(x, L->post_norm, h, c->eps, cur);
            if (c->n_expert > 0)
                rc |= ffn_moe(c, L, cur, mix);
            else
                rc |= ffn_dense(L, cur, h, (size_t)c->ffn, mix);
            for (size_t i = 0; i < h; i++) x[i] += mix[i];
            for (size_t t = 0; t < n_tap; t++)
                if ((size_t)tap_layers[t] == il && hidden_capture)
                    memcpy(hidden_capture + (r * n_tap + t) * h, x, h * sizeof(float));
        }
        orc_rms_norm(x, m->output_norm, h, c->eps, cur);
        rc |= qmat(&m->output, cur, logits + r * V, h, V, 1);
    }
    free(x);
    free(cur);
    free(qb);
    free(kb);
    free(vb);
    free(ao);
    free(mix);
    free(tmp);
    return rc;
}

/* forward.rs:380-662 */
int orc_dflash_draft(const orc_model *target, const orc_draft_head *head, const int32_t *noise_ids,
                     const float *target_ctx_stacked, size_t ctx_len, const int32_t *pos_ctx,
                     uint32_t noise_start_pos, float *logits) {
    return orc_dflash_draft_ex(target, head, NULL, noise_ids, target_ctx_stacked, ctx_len, pos_ctx, noise_start_pos, logits,
                               NULL);
}

/* forward.rs:380-662, with the DFlash-2 convolutions and selector gate of draft_block_inner
 * (metal_dflash.rs:16195-16275, 16795-16900, 17003-17030, 17098-17130) when ext is given */
int orc_dflash_draft_ex(const orc_model *target, const orc_draft_head *head, const orc_dflash2_ext *ext,
                        const int32_t *noise_ids, const float *target_ctx_stacked, size_t ctx_len,
                        const int32_t *pos_ctx, uint32_t noise_start_pos, float *logits, float *sel_h) {
    const orc_draft_cfg *c = &head->cfg;
    const int conv = ext && ext->conv_kernel_size > 0;
    const size_t ck = conv ? (size_t)ext->conv_kernel_size : 0, cg = conv ? (size_t)ext->conv_group_size : 1;
    size_t n = (size_t)c->block_size, h = (size_t)c->hidden, f = (size_t)c->ffn, hd = (size_t)c->head_dim;
    size_t nq = (size_t)c->n_q, nkv = (size_t)c->n_kv, q_dim = nq * hd, kv_dim = nkv * hd;
    size_t feat = (size_t)c->n_taps * h, V = (size_t)target->cfg.vocab;
    int rc = 0;
    float *ctx_h = (float *)malloc((ctx_len ? ctx_len : 1) * h * sizeof(float));
    float *tmp = (float *)malloc((h > hd ? h : hd) * sizeof(float));
    if (ctx_len) rc |= qmat(&head->fc, target_ctx_stacked, ctx_h, feat, h, ctx_len);
    for (size_t cidx = 0; cidx < ctx_len; cidx++) {
        orc_rms_norm(ctx_h + cidx * h, head->hidden_norm, h, c->eps, tmp);
        memcpy(ctx_h + cidx * h, tmp, h * sizeof(float));
    }
    float *x = (float *)malloc(n * h * sizeof(float)), *nn = (float *)malloc(n * h * sizeof(float));
    for (size_t i = 0; i < n; i++) {
        if (noise_ids[i] < 0 || (size_t)noise_ids[i] >= V) {
            rc = -2;
            goto done_early;
        }
        rc |= embed(&target->token_embd, noise_ids[i], h, x + i * h);
    }
    {
        float *q = (float *)malloc(n * q_dim * sizeof(float));
        float *kn = (float *)malloc(n * kv_dim * sizeof(float)), *vn = (float *)malloc(n * kv_dim * sizeof(float));
        float *kc = (float *)malloc((ctx_len ? ctx_len : 1) * kv_dim * sizeof(float));
        float *vc = (float *)malloc((ctx_len ? ctx_len : 1) * kv_dim * sizeof(float));
        float *ao = (float *)malloc(n * q_dim * sizeof(float)), *proj = (float *)malloc(n * h * sizeof(float));
        float *g = (float *)malloc(n * f * sizeof(float)), *u = (float *)malloc(n * f * sizeof(float));
        const size_t dyn_dim = conv ? 2 * ck * (h / cg) : 1;
        float *dyn = (float *)malloc(n * dyn_dim * sizeof(float)), *cv = (float *)malloc(n * h * sizeof(float));
        for (size_t il = 0; il < (size_t)c->n_layers; il++) {
            const orc_draft_layer *L = &head->layers[il];
            for (size_t i = 0; i < n; i++) orc_rms_norm(x + i * h, L->attn_norm, h, c->eps, nn + i * h);
            const float *src = nn;  /* what q/k/v read */
            if (conv) {
                rc |= qmat(&ext->conv_attn_proj[il], nn, dyn, h, dyn_dim, n);
                orc_dflash2_conv(nn, dyn, ext->conv_attn_base[il], cv, n, h, ck, cg, 0);
                src = cv;
            }
            rc |= qmat(&L->wq, src, q, h, q_dim, n) | qmat(&L->wk, src, kn, h, kv_dim, n) |
                  qmat(&L->wv, src, vn, h, kv_dim, n);
            if (ctx_len)
                rc |= qmat(&L->wk, ctx_h, kc, h, kv_dim, ctx_len) | qmat(&L->wv, ctx_h, vc, h, kv_dim, ctx_len);
            for (size_t i = 0; i < n; i++)
                for (size_t hi = 0; hi < nq; hi++) {
                    orc_rms_norm(q + i * q_dim + hi * hd, L->q_norm, hd, c->eps, tmp);
                    memcpy(q + i * q_dim + hi * hd, tmp, hd * sizeof(float));
                }
            for (size_t i = 0; i < n; i++)
                for (size_t hi = 0; hi < nkv; hi++) {
                    orc_rms_norm(kn + i * kv_dim + hi * hd, L->k_norm, hd, c->eps, tmp);
                    memcpy(kn + i * kv_dim + hi * hd, tmp, hd * sizeof(float));
                }
            for (size_t i = 0; i < ctx_len; i++)
                for (size_t hi = 0; hi < nkv; hi++) {
                    orc_rms_norm(kc + i * kv_dim + hi * hd, L->k_norm, hd, c->eps, tmp);
                    memcpy(kc + i * kv_dim + hi * hd, tmp, hd * sizeof(float));
                }
            for (size_t i = 0; i < n; i++) {
                uint32_t pos = noise_start_pos + (uint32_t)i;
                orc_rope_in_place(q + i * q_dim, nq, hd, hd, pos, c->rope_theta);
                orc_rope_in_place(kn + i * kv_dim, nkv, hd, hd, pos, c->rope_theta);
            }
            for (size_t i = 0; i < ctx_len; i++)
                orc_rope_in_place(kc + i * kv_dim, nkv, hd, hd, (uint32_t)pos_ctx[i], c->rope_theta);
            orc_attn_draft(q, kc, vc, kn, vn, pos_ctx, ctx_len, n, nq, nkv, hd, noise_start_pos, c->causal,
                           L->is_swa ? c->swa_window : 0u, ao);
            rc |= qmat(&L->wo, ao, proj, q_dim, h, n);
            if (conv) {  /* side 1 between attn_output and the residual; same coefficients */
                orc_dflash2_conv(proj, dyn, ext->conv_attn_base[il], cv, n, h, ck, cg, 1);
                for (size_t i = 0; i < n * h; i++) x[i] += cv[i];
            } else {
                for (size_t i = 0; i < n * h; i++) x[i] += proj[i];
            }
            for (size_t i = 0; i < n; i++) orc_rms_norm(x + i * h, L->post_norm, h, c->eps, nn + i * h);
            src = nn;  /* what gate/up read */
            if (conv) {
                rc |= qmat(&ext->conv_ffn_proj[il], nn, dyn, h, dyn_dim, n);
                orc_dflash2_conv(nn, dyn, ext->conv_ffn_base[il], cv, n, h, ck, cg, 0);
                src = cv;
            }
            rc |= qmat(&L->gate, src, g, h, f, n) | qmat(&L->up, src, u, h, f, n);
            for (size_t i = 0; i < n * f; i++) g[i] = orc_silu(g[i]) * u[i];
            rc |= qmat(&L->down, g, proj, f, h, n);
            if (conv) {
                orc_dflash2_conv(proj, dyn, ext->conv_ffn_base[il], cv, n, h, ck, cg, 1);
                for (size_t i = 0; i < n * h; i++) x[i] += cv[i];
            } else {
                for (size_t i = 0; i < n * h; i++) x[i] += proj[i];
            }
        }
        for (size_t i = 0; i < n; i++) orc_rms_norm(x + i * h, head->output_norm, h, c->eps, nn + i * h);
        rc |= qmat(&target->output, nn, logits, h, V, n);
        if (ext && sel_h && ext->selector_rank > 0) rc |= qmat(&ext->selector_hidden, nn, sel_h, h, (size_t)ext->selector_rank, n);
        free(dyn);
        free(cv);
        free(q);
        free(kn);
        free(vn);
        free(kc);
        free(vc);
        free(ao);
        free(proj);
        free(g);
        free(u);
    }
done_early:
    free(ctx_h);
    free(tmp);
    free(x);
    free(nn);
    return rc;
}
