/*
 * CPU oracle, test infrastructure only: sampler-v1, its speculative couplings and
 * the accept-prefix decision.
 *
 * Follows crates/qwen-llm/src/sampling.rs (config validation :133-144, greedy
 * :1159-1181, ordering keys :1206-1235, sorted candidates :1183-1202, chain
 * :1541-1615, couplings :692-790, RNG use :1654-1657) and
 * crates/qwen-llm/src/metal_dflash/accept.rs:76-183.  The order of every f64
 * operation is the reference's: sums are sequential folds, the temperature is a
 * division applied to each logit before the maximum is subtracted, and config
 * values are f32 widened to f64.
 */
#include "dflash_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>

/* ---------- config / stream ---------- */

/* sampling.rs:133-144 */
static int validate_cfg(const orc_sampling_config *c) {
    if (!isfinite(c->temperature) || c->temperature < 0.0f) return ORC_ERR_INVALID_TEMPERATURE;
    if (!isfinite(c->top_p) || !(0.0f < c->top_p && c->top_p <= 1.0f)) return ORC_ERR_INVALID_TOP_P;
    if (!isfinite(c->min_p) || !(0.0f <= c->min_p && c->min_p <= 1.0f)) return ORC_ERR_INVALID_MIN_P;
    return ORC_OK;
}

/* sampling.rs:346-366 */
int orc_sampler_init(orc_sampler *s, const orc_sampling_config *cfg) {
    int rc = validate_cfg(cfg);
    if (rc) return rc;
    s->cfg = *cfg;
    s->draws = 0;
    if (cfg->rng_kind == ORC_RNG_PHILOX) {
        s->s[0] = 0; /* stream position */
        s->s[1] = s->s[2] = s->s[3] = 0;
    } else {
        orc_xoshiro_seed(cfg->seed, s->s);
    }
    return ORC_OK;
}

static uint64_t raw_next(orc_sampler *s) {
    if (s->cfg.rng_kind == ORC_RNG_PHILOX) {
        uint64_t pos = s->s[0]++;
        uint32_t ctr[4] = {(uint32_t)pos, (uint32_t)(pos >> 32), 0, 0};
        uint32_t key[2] = {(uint32_t)s->cfg.seed, (uint32_t)(s->cfg.seed >> 32)};
        uint32_t out[4];
        orc_philox4x32_10(ctr, key, out);
        return (uint64_t)out[0] | ((uint64_t)out[1] << 32);
    }
    return orc_xoshiro_next(s->s);
}

int orc_sampler_at_draw(orc_sampler *s, const orc_sampling_config *cfg, uint64_t draws) {
    int rc = orc_sampler_init(s, cfg);
    if (rc) return rc;
    for (uint64_t i = 0; i < draws; i++) raw_next(s);
    s->draws = draws;
    return ORC_OK;
}

double orc_sampler_next_unit(orc_sampler *s) { return orc_unit_f64(raw_next(s)); }

/* ---------- ordering ---------- */

static uint32_t f32_bits(float f) {
    uint32_t b;
    memcpy(&b, &f, 4);
    return b;
}
static float bits_f32(uint32_t b) {
    float f;
    memcpy(&f, &b, 4);
    return f;
}

/* sampling.rs:1206-1220 */
static uint32_t descending_logit_bits(float logit) {
    uint32_t bits = f32_bits(logit);
    uint32_t ascending = (bits & 0x80000000u) ? ~bits : (bits | 0x80000000u);
    return ~ascending;
}
static uint64_t candidate_key(size_t token, float logit) {
    return ((uint64_t)descending_logit_bits(logit) << 32) | (uint64_t)token;
}
/* sampling.rs:1223-1235 */
static double key_logit(uint64_t key) {
    uint32_t ascending = ~(uint32_t)(key >> 32);
    uint32_t bits = (ascending & 0x80000000u) ? (ascending & 0x7fffffffu) : ~ascending;
    return (double)bits_f32(bits);
}
static int32_t key_token(uint64_t key) { return (int32_t)(uint32_t)key; }

/* f32 total order: -1 / 0 / +1 (Rust's f32::total_cmp) */
static int total_cmp(float a, float b) {
    int32_t x = (int32_t)f32_bits(a), y = (int32_t)f32_bits(b);
    x ^= (int32_t)((uint32_t)(x >> 31) >> 1);
    y ^= (int32_t)((uint32_t)(y >> 31) >> 1);
    return (x > y) - (x < y);
}

static int validate_shape(size_t n) {
    if (n == 0) return ORC_ERR_EMPTY_LOGITS;
    if (n > (size_t)INT32_MAX) return ORC_ERR_VOCAB_TOO_LARGE;
    return ORC_OK;
}

/* sampling.rs:1159-1181 */
int orc_greedy_token(const float *logits, size_t n, int32_t *token, int64_t *err_index) {
    int rc = validate_shape(n);
    if (rc) return rc;
    size_t best = 0;
    float best_logit = logits[0];
    if (isnan(best_logit)) {
        if (err_index) *err_index = 0;
        return ORC_ERR_NAN_LOGIT;
    }
    for (size_t t = 1; t < n; t++) {
        if (isnan(logits[t])) {
            if (err_index) *err_index = (int64_t)t;
            return ORC_ERR_NAN_LOGIT;
        }
        if (total_cmp(logits[t], best_logit) > 0) {
            best = t;
            best_logit = logits[t];
        }
    }
    *token = (int32_t)best;
    return ORC_OK;
}

/* kernels/elementwise.metal:1231-1286 (verify tail), as one serial scan: IEEE
 * comparisons (so NaN never becomes a candidate and -0.0 ties +0.0), the lowest index
 * wins ties, gap = top1 - top2 with duplicates counted (0 when the maximum occurs
 * twice, +inf for a single element), and an all-NaN row yields index -1. */
void orc_argmax_top2(const float *logits, size_t n, int32_t *idx, float *gap) {
    float v1 = -INFINITY, v2 = -INFINITY;
    uint32_t i1 = UINT32_MAX;
    for (size_t t = 0; t < n; t++) {
        float v = logits[t];
        if (v > v1) {
            v2 = v1;
            v1 = v;
            i1 = (uint32_t)t;
        } else if (v == v1 && (uint32_t)t < i1) {
            v2 = v1;
            i1 = (uint32_t)t;
        } else if (v > v2) {
            v2 = v;
        }
    }
    *idx = (int32_t)i1;
    *gap = v1 - v2;
}

/* kernels/dflash2.metal:73-170: descending total-order value, ties to the lower index */
void orc_top16(const float *logits, size_t n, int32_t ids[16], float vals[16]) {
    uint64_t keys[16];
    size_t cnt = 0;
    for (size_t t = 0; t < n; t++) {
        uint64_t key = candidate_key(t, logits[t]);
        if (cnt == 16 && key >= keys[15]) continue;
        size_t pos = cnt < 16 ? cnt : 15;
        while (pos > 0 && keys[pos - 1] > key) {
            keys[pos] = keys[pos - 1];
            pos--;
        }
        keys[pos] = key;
        if (cnt < 16) cnt++;
    }
    for (size_t i = 0; i < 16; i++) {
        if (i < cnt) {
            ids[i] = key_token(keys[i]);
            vals[i] = logits[(size_t)ids[i]];
        } else {
            ids[i] = -1;
            vals[i] = -INFINITY;
        }
    }
}

static int cmp_u64(const void *a, const void *b) {
    uint64_t x = *(const uint64_t *)a, y = *(const uint64_t *)b;
    return (x > y) - (x < y);
}

/* sampling.rs:1183-1202 / 1273-1296: returns the ordered keys (malloc'd) */
static int ordered_keys(const float *logits, size_t n, size_t top_k, uint64_t **keys_out, size_t *len_out,
                        int64_t *err_index) {
    int rc = validate_shape(n);
    if (rc) return rc;
    for (size_t t = 0; t < n; t++) {
        if (isnan(logits[t])) {
            if (err_index) *err_index = (int64_t)t;
            return ORC_ERR_NAN_LOGIT;
        }
    }
    if (top_k == 0 || top_k >= n) {
        uint64_t *keys = (uint64_t *)malloc(n * sizeof(uint64_t));
        for (size_t t = 0; t < n; t++) keys[t] = candidate_key(t, logits[t]);
        qsort(keys, n, sizeof(uint64_t), cmp_u64);
        *keys_out = keys;
        *len_out = n;
        return ORC_OK;
    }
    uint64_t *keys = (uint64_t *)malloc(top_k * sizeof(uint64_t));
    size_t cnt = 0;
    for (size_t t = 0; t < n; t++) {
        uint64_t key = candidate_key(t, logits[t]);
        if (cnt == top_k && key >= keys[top_k - 1]) continue;
        size_t pos = cnt < top_k ? cnt : top_k - 1;
        while (pos > 0 && keys[pos - 1] > key) {
            keys[pos] = keys[pos - 1];
            pos--;
        }
        keys[pos] = key;
        if (cnt < top_k) cnt++;
    }
    *keys_out = keys;
    *len_out = cnt;
    return ORC_OK;
}

/* ---------- the chain ---------- */

typedef struct {
    int32_t *tokens;
    double *weights;
    size_t len;
    double total;
    size_t sampled_index;
} dist_t;

static void dist_free(dist_t *d) {
    free(d->tokens);
    free(d->weights);
    d->tokens = NULL;
    d->weights = NULL;
}

/* sampling.rs:386-405 + 1541-1615 (diagnose / diagnose_candidates) */
static int diagnose(const orc_sampling_config *cfg, const float *logits, size_t n, double uniform, dist_t *d,
                    int64_t *err_index) {
    memset(d, 0, sizeof(*d));
    if (cfg->temperature == 0.0f) {
        int32_t tok;
        int rc = orc_greedy_token(logits, n, &tok, err_index);
        if (rc) return rc;
        d->tokens = (int32_t *)malloc(sizeof(int32_t));
        d->weights = (double *)malloc(sizeof(double));
        d->tokens[0] = tok;
        d->weights[0] = 1.0;
        d->len = 1;
        d->total = 1.0;
        d->sampled_index = 0;
        return ORC_OK;
    }
    uint64_t *keys = NULL;
    size_t len = 0;
    int rc = ordered_keys(logits, n, (size_t)cfg->top_k, &keys, &len, err_index);
    if (rc) return rc;

    double *l = (double *)malloc(len * sizeof(double));
    for (size_t i = 0; i < len; i++) l[i] = key_logit(keys[i]);

    /* min-p on pre-temperature f64 logits */
    if (cfg->min_p > 0.0f) {
        double max_logit = l[0];
        if (isfinite(max_logit)) {
            double threshold = max_logit + log((double)cfg->min_p);
            size_t keep = 0;
            for (size_t i = 0; i < len; i++) {
                if (l[i] >= threshold) {
                    l[keep] = l[i];
                    keys[keep] = keys[i];
                    keep++;
                }
            }
            len = keep;
        }
    }
    if (len == 0) {
        free(keys);
        free(l);
        return ORC_ERR_NO_CANDIDATES;
    }
    if (l[0] == INFINITY) {
        size_t keep = 0;
        for (size_t i = 0; i < len; i++) {
            if (l[i] == INFINITY) {
                l[keep] = l[i];
                keys[keep] = keys[i];
                keep++;
            }
        }
        len = keep;
    }
    double temperature = (double)cfg->temperature;
    for (size_t i = 0; i < len; i++) l[i] /= temperature;

    /* probability_weights (sampling.rs:1515-1539) */
    double *w = (double *)malloc(len * sizeof(double));
    size_t n_inf = 0;
    for (size_t i = 0; i < len; i++) n_inf += (l[i] == INFINITY);
    if (n_inf > 0) {
        for (size_t i = 0; i < len; i++) w[i] = (l[i] == INFINITY) ? 1.0 : 0.0;
    } else {
        double max_logit = l[0];
        if (max_logit == -INFINITY) {
            free(keys);
            free(l);
            free(w);
            return ORC_ERR_NO_CANDIDATES;
        }
        int finite = 1;
        for (size_t i = 0; i < len; i++) {
            w[i] = exp(l[i] - max_logit);
            finite &= isfinite(w[i]) ? 1 : 0;
        }
        if (!finite) {
            free(keys);
            free(l);
            free(w);
            return ORC_ERR_NO_CANDIDATES;
        }
    }

    if (cfg->top_p < 1.0f) {
        double total = -0.0;
        for (size_t i = 0; i < len; i++) total += w[i];
        double target = total * (double)cfg->top_p;
        double cumulative = 0.0;
        size_t keep = 0;
        for (size_t i = 0; i < len; i++) {
            cumulative += w[i];
            keep++;
            if (cumulative >= target) break;
        }
        if (keep < 1) keep = 1;
        len = keep;
    }

    double total_weight = -0.0;
    for (size_t i = 0; i < len; i++) total_weight += w[i];
    if (!(isfinite(total_weight) && total_weight > 0.0)) {
        free(keys);
        free(l);
        free(w);
        return ORC_ERR_NO_CANDIDATES;
    }
    double target = uniform * total_weight;
    double cumulative = 0.0;
    size_t index = len - 1;
    for (size_t i = 0; i < len; i++) {
        cumulative += w[i];
        if (target < cumulative) {
            index = i;
            break;
        }
    }
    d->tokens = (int32_t *)malloc(len * sizeof(int32_t));
    for (size_t i = 0; i < len; i++) d->tokens[i] = key_token(keys[i]);
    d->weights = w;
    d->len = len;
    d->total = total_weight;
    d->sampled_index = index;
    free(keys);
    free(l);
    return ORC_OK;
}

int orc_sampler_diagnose(const orc_sampler *s, const float *logits, size_t n, double uniform,
                         orc_weighted_candidate *cands, size_t cap, size_t *n_out, double *total_weight,
                         int32_t *sampled_token, size_t *candidate_index, int64_t *err_index) {
    dist_t d;
    int rc = diagnose(&s->cfg, logits, n, uniform, &d, err_index);
    if (rc) return rc;
    if (cands) {
        for (size_t i = 0; i < d.len && i < cap; i++) {
            cands[i].token = d.tokens[i];
            cands[i].pad = 0;
            cands[i].weight = d.weights[i];
        }
    }
    if (n_out) *n_out = d.len;
    if (total_weight) *total_weight = d.total;
    if (sampled_token) *sampled_token = d.tokens[d.sampled_index];
    if (candidate_index) *candidate_index = d.sampled_index;
    dist_free(&d);
    return ORC_OK;
}

/* sampling.rs:530-603: one draw per successful positive-temperature call */
int orc_sampler_sample(orc_sampler *s, const float *logits, size_t n, int32_t *token, size_t *candidate_index,
                       int64_t *err_index) {
    if (s->cfg.temperature == 0.0f) {
        if (candidate_index) *candidate_index = 0;
        return orc_greedy_token(logits, n, token, err_index);
    }
    orc_sampler next = *s;
    double u = orc_sampler_next_unit(&next);
    dist_t d;
    int rc = diagnose(&s->cfg, logits, n, u, &d, err_index);
    if (rc) return rc;
    *token = d.tokens[d.sampled_index];
    if (candidate_index) *candidate_index = d.sampled_index;
    dist_free(&d);
    next.draws = s->draws + 1;
    *s = next;
    return ORC_OK;
}

/* sampling.rs:692-703 */
int orc_couple_deterministic_proposal(orc_sampler *s, const float *logits, size_t n, int32_t proposal,
                                      int *accepted, int32_t *correction, int64_t *err_index) {
    int32_t target;
    int rc = orc_sampler_sample(s, logits, n, &target, NULL, err_index);
    if (rc) return rc;
    *accepted = (target == proposal);
    *correction = target;
    return ORC_OK;
}

/* sampling.rs:708-790 */
int orc_couple_sparse_proposal(orc_sampler *s, const float *logits, size_t n, int32_t proposal_token,
                               const orc_weighted_candidate *prop, size_t n_prop, int *accepted,
                               int32_t *correction, int64_t *err_index) {
    if (proposal_token < 0 || (size_t)proposal_token >= n) {
        if (err_index) *err_index = proposal_token;
        return ORC_ERR_PROPOSAL_TOKEN_OUT_OF_RANGE;
    }
    if (n_prop == 0) return ORC_ERR_NO_CANDIDATES;
    double proposal_total = 0.0, proposal_token_weight = 0.0;
    for (size_t i = 0; i < n_prop; i++) {
        if (prop[i].token < 0 || (size_t)prop[i].token >= n) {
            if (err_index) *err_index = prop[i].token;
            return ORC_ERR_PROPOSAL_TOKEN_OUT_OF_RANGE;
        }
        if (!isfinite(prop[i].weight) || prop[i].weight < 0.0) {
            if (err_index) *err_index = prop[i].token;
            return ORC_ERR_INVALID_PROPOSAL_WEIGHT;
        }
        proposal_total += prop[i].weight;
        if (prop[i].token == proposal_token) proposal_token_weight += prop[i].weight;
    }
    if (!(isfinite(proposal_total) && proposal_total > 0.0)) return ORC_ERR_NO_CANDIDATES;
    if (!(isfinite(proposal_token_weight) && proposal_token_weight > 0.0)) {
        if (err_index) *err_index = proposal_token;
        return ORC_ERR_MISSING_PROPOSAL_TOKEN;
    }

    dist_t d;
    int rc = diagnose(&s->cfg, logits, n, 0.0, &d, err_index);
    if (rc) return rc;
    double tp = -0.0;
    for (size_t i = 0; i < d.len; i++)
        if (d.tokens[i] == proposal_token) tp += d.weights[i];
    double target_probability = tp / d.total;
    double proposal_probability = proposal_token_weight / proposal_total;
    double acceptance = fmin(target_probability / proposal_probability, 1.0);
    s->draws += 1;
    if (orc_sampler_next_unit(s) < acceptance) {
        *accepted = 1;
        *correction = proposal_token;
        dist_free(&d);
        return ORC_OK;
    }
    double *residual = (double *)malloc(d.len * sizeof(double));
    double residual_total = 0.0;
    for (size_t i = 0; i < d.len; i++) {
        double p = d.weights[i] / d.total;
        double qs = -0.0;
        for (size_t j = 0; j < n_prop; j++)
            if (prop[j].token == d.tokens[i]) qs += prop[j].weight;
        double q = qs / proposal_total;
        double wgt = fmax(p - q, 0.0);
        residual_total += wgt;
        residual[i] = wgt;
    }
    if (!(isfinite(residual_total) && residual_total > 0.0)) {
        free(residual);
        dist_free(&d);
        return ORC_ERR_NO_CANDIDATES;
    }
    s->draws += 1;
    double threshold = orc_sampler_next_unit(s) * residual_total;
    double cumulative = 0.0;
    int32_t pick = d.tokens[d.len - 1];
    for (size_t i = 0; i < d.len; i++) {
        cumulative += residual[i];
        if (threshold < cumulative) {
            pick = d.tokens[i];
            break;
        }
    }
    *accepted = 0;
    *correction = pick;
    free(residual);
    dist_free(&d);
    return ORC_OK;
}

/* ---------- dense proposal (vocabulary-wide draft distribution) ----------
 *
 * The reference's proposals hold at most 16 candidates (metal_dflash.rs:17389-17404);
 * a vocabulary-wide q = softmax(draft/T) needs a defined summation order that a GPU
 * can reproduce.  Contract shared with the HIP kernels:
 *   e_i  = exp(f64(d_i)/f64(T) - f64(d_max)/f64(T))      (sampler weight form, :1416-1438)
 *   tile = 1024 consecutive tokens, zero padded; slot t (0..255) holds
 *          ((e[4t] + e[4t+1]) + e[4t+2]) + e[4t+3]; then for stride 128,64,..,1:
 *          slot[t] += slot[t+stride] (t < stride); tile sum = slot[0]
 *   P    = sequential sum of the tile sums from 0.0 in tile order
 * Everything on the target side is the sparse coupling above.
 */
static int dense_weights_total(const float *draft, size_t n, float temperature, double *dmax_scaled,
                               double *total, int64_t *err_index) {
    int rc = validate_shape(n);
    if (rc) return rc;
    float best = draft[0];
    for (size_t t = 0; t < n; t++) {
        if (isnan(draft[t])) {
            if (err_index) *err_index = (int64_t)t;
            return ORC_ERR_NAN_LOGIT;
        }
        if (total_cmp(draft[t], best) > 0) best = draft[t];
    }
    double T = (double)temperature;
    double mx = (double)best / T;
    if (!isfinite(mx)) return ORC_ERR_NO_CANDIDATES;
    double P = 0.0;
    double slot[256];
    for (size_t base = 0; base < n; base += 1024) {
        for (size_t t = 0; t < 256; t++) {
            double acc = 0.0;
            for (size_t e = 0; e < 4; e++) {
                size_t i = base + 4 * t + e;
                double v = (i < n) ? exp((double)draft[i] / T - mx) : 0.0;
                acc = (e == 0) ? v : acc + v;
            }
            slot[t] = acc;
        }
        for (size_t stride = 128; stride >= 1; stride >>= 1)
            for (size_t t = 0; t < stride; t++) slot[t] += slot[t + stride];
        P += slot[0];
    }
    *dmax_scaled = mx;
    *total = P;
    return ORC_OK;
}

double orc_dense_proposal_total(const float *draft_logits, size_t n, float draft_temperature,
                                int64_t *err_index) {
    double mx, P;
    if (dense_weights_total(draft_logits, n, draft_temperature, &mx, &P, err_index)) return NAN;
    return P;
}

int orc_couple_dense_proposal(orc_sampler *s, const float *target_logits, const float *draft_logits, size_t n,
                              float draft_temperature, int32_t proposal_token, int *accepted,
                              int32_t *correction, int64_t *err_index) {
    if (proposal_token < 0 || (size_t)proposal_token >= n) {
        if (err_index) *err_index = proposal_token;
        return ORC_ERR_PROPOSAL_TOKEN_OUT_OF_RANGE;
    }
    if (!(isfinite(draft_temperature) && draft_temperature > 0.0f)) return ORC_ERR_INVALID_TEMPERATURE;
    double mx, P;
    int rc = dense_weights_total(draft_logits, n, draft_temperature, &mx, &P, err_index);
    if (rc) return rc;
    if (!(isfinite(P) && P > 0.0)) return ORC_ERR_NO_CANDIDATES;
    double T = (double)draft_temperature;
    double wtok = exp((double)draft_logits[proposal_token] / T - mx);
    if (!(isfinite(wtok) && wtok > 0.0)) {
        if (err_index) *err_index = proposal_token;
        return ORC_ERR_MISSING_PROPOSAL_TOKEN;
    }
    dist_t d;
    rc = diagnose(&s->cfg, target_logits, n, 0.0, &d, err_index);
    if (rc) return rc;
    double tp = -0.0;
    for (size_t i = 0; i < d.len; i++)
        if (d.tokens[i] == proposal_token) tp += d.weights[i];
    double target_probability = tp / d.total;
    double proposal_probability = wtok / P;
    double acceptance = fmin(target_probability / proposal_probability, 1.0);
    s->draws += 1;
    if (orc_sampler_next_unit(s) < acceptance) {
        *accepted = 1;
        *correction = proposal_token;
        dist_free(&d);
        return ORC_OK;
    }
    double *residual = (double *)malloc(d.len * sizeof(double));
    double residual_total = 0.0;
    for (size_t i = 0; i < d.len; i++) {
        double p = d.weights[i] / d.total;
        double q = exp((double)draft_logits[d.tokens[i]] / T - mx) / P;
        double wgt = fmax(p - q, 0.0);
        residual_total += wgt;
        residual[i] = wgt;
    }
    if (!(isfinite(residual_total) && residual_total > 0.0)) {
        free(residual);
        dist_free(&d);
        return ORC_ERR_NO_CANDIDATES;
    }
    s->draws += 1;
    double threshold = orc_sampler_next_unit(s) * residual_total;
    double cumulative = 0.0;
    int32_t pick = d.tokens[d.len - 1];
    for (size_t i = 0; i < d.len; i++) {
        cumulative += residual[i];
        if (threshold < cumulative) {
            pick = d.tokens[i];
            break;
        }
    }
    *accepted = 0;
    *correction = pick;
    free(residual);
    dist_free(&d);
    return ORC_OK;
}

/* ---------- accept-prefix (metal_dflash/accept.rs:76-183) ---------- */

static int contains(const int32_t *ids, size_t n, int32_t v) {
    for (size_t i = 0; i < n; i++)
        if (ids[i] == v) return 1;
    return 0;
}

static void decision_clear(orc_accept_decision *out) {
    memset(out, 0, sizeof(*out));
    out->err_row = -1;
    out->err_index = -1;
}

/* mode 0: deterministic, 1: sparse proposals, 2: dense draft logits */
static int decide(const int32_t *verified, size_t n_tokens, const float *target_logits, size_t n_logits,
                  size_t vocab, int mode, size_t n_proposals, const int32_t *prop_tokens,
                  const size_t *prop_offsets, const size_t *prop_counts, const orc_weighted_candidate *prop_cands,
                  const float *draft_logits, float draft_temperature, orc_sampler *sampler, size_t budget,
                  const int32_t *stop_ids, size_t n_stop, orc_accept_decision *out) {
    decision_clear(out);
    if (n_tokens == 0) return ORC_ERR_INVALID_INPUT;
    if (vocab == 0 || vocab > (size_t)INT32_MAX) return ORC_ERR_INVALID_INPUT;
    if (n_tokens > SIZE_MAX / vocab || n_tokens * vocab != n_logits) return ORC_ERR_INVALID_INPUT;
    if (n_tokens > 64) return ORC_ERR_INVALID_INPUT;
    for (size_t i = 0; i < n_tokens; i++) {
        if (verified[i] < 0 || (size_t)verified[i] >= vocab) {
            out->err_row = (int32_t)i;
            out->err_index = verified[i];
            return ORC_ERR_INVALID_TOKEN;
        }
    }
    size_t n_drafts = n_tokens - 1;
    if (mode == 1) {
        if (n_proposals != n_drafts) return ORC_ERR_INVALID_INPUT;
        for (size_t row = 0; row < n_drafts; row++) {
            if (prop_tokens[row] != verified[row + 1]) {
                out->err_row = (int32_t)row;
                out->err_index = prop_tokens[row];
                return ORC_ERR_PROPOSAL_MISMATCH;
            }
            for (size_t j = 0; j < prop_counts[row]; j++) {
                int32_t t = prop_cands[prop_offsets[row] + j].token;
                if (t < 0 || (size_t)t >= vocab) {
                    out->err_row = (int32_t)row;
                    out->err_code = ORC_ERR_PROPOSAL_TOKEN_OUT_OF_RANGE;
                    out->err_index = t;
                    return ORC_ERR_PROPOSAL_TOKEN_OUT_OF_RANGE;
                }
            }
        }
    }
    int anchor_stop = ORC_STOP_NONE;
    if (contains(stop_ids, n_stop, verified[0]))
        anchor_stop = ORC_STOP_EOS;
    else if (budget == 0)
        anchor_stop = ORC_STOP_TOKEN_LIMIT;
    if (anchor_stop) {
        out->stop_reason = anchor_stop;
        out->carry_kind = ORC_CARRY_NONE;
        out->retain_input_count = 0;
        return ORC_OK;
    }

    orc_sampler next = *sampler;
    size_t accepted = 0;
    int carry_kind = ORC_CARRY_NONE, stop = ORC_STOP_NONE;
    int32_t carry_token = 0;
    for (;;) {
        size_t row = accepted;
        const float *logits = target_logits + row * vocab;
        int64_t err_index = -1;
        int rc;
        if (row == n_drafts) {
            int32_t bonus;
            rc = orc_sampler_sample(&next, logits, vocab, &bonus, NULL, &err_index);
            if (rc) goto sampling_error;
            carry_kind = ORC_CARRY_BONUS;
            carry_token = bonus;
            break;
        }
        int32_t draft = verified[row + 1];
        int acc = 0;
        int32_t correction = 0;
        if (mode == 1) {
            rc = orc_couple_sparse_proposal(&next, logits, vocab, prop_tokens[row],
                                            prop_cands + prop_offsets[row], prop_counts[row], &acc, &correction,
                                            &err_index);
        } else if (mode == 2) {
            rc = orc_couple_dense_proposal(&next, logits, draft_logits + row * vocab, vocab, draft_temperature,
                                           draft, &acc, &correction, &err_index);
        } else {
            rc = orc_couple_deterministic_proposal(&next, logits, vocab, draft, &acc, &correction, &err_index);
        }
        if (rc) {
        sampling_error:
            decision_clear(out);
            out->err_row = (int32_t)row;
            out->err_code = rc;
            out->err_index = err_index;
            return rc;
        }
        if (!acc) {
            carry_kind = ORC_CARRY_CORRECTION;
            carry_token = correction;
            break;
        }
        out->accepted_drafts[accepted++] = draft;
        if (contains(stop_ids, n_stop, draft)) {
            stop = ORC_STOP_EOS;
            break;
        }
        if (accepted == budget) {
            stop = ORC_STOP_TOKEN_LIMIT;
            break;
        }
    }
    out->n_accepted = (int32_t)accepted;
    out->carry_kind = carry_kind;
    out->carry_token = carry_token;
    out->stop_reason = stop;
    out->retain_input_count = (int32_t)(1 + accepted - (stop != ORC_STOP_NONE ? 1 : 0));
    *sampler = next;
    return ORC_OK;
}

int orc_decide_accept_prefix(const int32_t *verified_tokens, size_t n_tokens, const float *target_logits,
                             size_t n_logits, size_t vocab, int have_proposals, size_t n_proposals,
                             const int32_t *prop_tokens, const size_t *prop_offsets, const size_t *prop_counts,
                             const orc_weighted_candidate *prop_cands, orc_sampler *sampler,
                             size_t remaining_output_budget, const int32_t *stop_ids, size_t n_stop,
                             orc_accept_decision *out) {
    return decide(verified_tokens, n_tokens, target_logits, n_logits, vocab, have_proposals ? 1 : 0, n_proposals,
                  prop_tokens, prop_offsets, prop_counts, prop_cands, NULL, 0.0f, sampler,
                  remaining_output_budget, stop_ids, n_stop, out);
}

int orc_decide_accept_prefix_dense(const int32_t *verified_tokens, size_t n_tokens, const float *target_logits,
                                   const float *draft_logits, size_t vocab, float draft_temperature,
                                   orc_sampler *sampler, size_t remaining_output_budget, const int32_t *stop_ids,
                                   size_t n_stop, orc_accept_decision *out) {
    return decide(verified_tokens, n_tokens, target_logits, n_tokens * vocab, vocab, 2, 0, NULL, NULL, NULL, NULL,
                  draft_logits, draft_temperature, sampler, remaining_output_budget, stop_ids, n_stop, out);
}

/* Many independent block decisions at once, one per sampler, OpenMP across trials: each trial is exactly
 * orc_decide_accept_prefix_dense (draft_logits != NULL) or orc_decide_accept_prefix without proposals
 * (draft_logits == NULL) on its own slice.  For checking long seeded runs in bounded wall time; no counterpart
 * in the reference (its accept decision is per block). */
void orc_decide_accept_prefix_batch(size_t n_trials, const int32_t *verified_tokens, size_t n_tokens,
                                    const float *target_logits, const float *draft_logits, size_t vocab,
                                    float draft_temperature, orc_sampler *samplers, size_t remaining_output_budget,
                                    orc_accept_decision *out, int32_t *status) {
#pragma omp parallel for schedule(dynamic, 1)
    for (long t = 0; t < (long)n_trials; t++) {
        const int32_t *tok = verified_tokens + (size_t)t * n_tokens;
        const float *tl = target_logits + (size_t)t * n_tokens * vocab;
        if (draft_logits)
            status[t] = orc_decide_accept_prefix_dense(tok, n_tokens, tl, draft_logits + (size_t)t * (n_tokens - 1) * vocab, vocab,
                                                       draft_temperature, &samplers[t], remaining_output_budget, NULL, 0, &out[t]);
        else
            status[t] = orc_decide_accept_prefix(tok, n_tokens, tl, n_tokens * vocab, vocab, 0, 0, NULL, NULL, NULL, NULL,
                                                 &samplers[t], remaining_output_budget, NULL, 0, &out[t]);
    }
}
