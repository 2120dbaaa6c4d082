/*
 * CPU oracle, DFlash-2 extras: the two-tap dynamic depthwise convolution and the greedy
 * selector walk over predecessor/successor codebooks.  TEST INFRASTRUCTURE ONLY (see
 * dflash_oracle.h).
 */
#include "dflash_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>

/* kernels/dflash2.metal:40-69: y[t][c] = sum_tap (base[side][tap][c] + dyn[t][side][tap][g(c)]) * x[t-tap][c],
 * rows before the block are zeros, taps accumulated in order with a fused multiply-add. */
void orc_dflash2_conv(const float *x, const float *dyn, const float *base, float *y, size_t n_tokens, size_t h,
                      size_t kernel_size, size_t group_size, size_t side) {
    const size_t n_groups = h / group_size;
    const size_t dyn_stride = 2 * kernel_size * n_groups;
    for (size_t t = 0; t < n_tokens; t++) {
        for (size_t c = 0; c < h; c++) {
            const size_t g = c / group_size;
            float acc = 0.0f;
            for (size_t tap = 0; tap < kernel_size && tap <= t; tap++) {
                const float b = base[side * kernel_size * h + tap * h + c];
                const float d = dyn[t * dyn_stride + side * kernel_size * n_groups + tap * n_groups + g];
                acc = fmaf(b + d, x[(t - tap) * h + c], acc);
            }
            y[t * h + c] = acc;
        }
    }
}

/* DFlash2Codebook::dequant_row (metal_dflash.rs:3275-3343): row `row` of a [n_rows][rank] table.
 * Returns 0, or -1 when the row is out of range or the type has no row form here. */
int orc_codebook_row(const orc_codebook *cb, size_t row, float *out) {
    if (row >= cb->n_rows) return -1;
    const uint8_t *data = (const uint8_t *)cb->data;
    switch (cb->type) {
    case ORC_F32:
        memcpy(out, data + row * cb->rank * 4, cb->rank * 4);
        return 0;
    case ORC_F16:
        for (size_t j = 0; j < cb->rank; j++) {
            uint16_t bits;
            memcpy(&bits, data + (row * cb->rank + j) * 2, 2);
            out[j] = orc_f16_to_f32(bits);
        }
        return 0;
    case ORC_Q8_0:
    case ORC_Q4_K:
        return orc_dequant(cb->type, data + row * orc_row_bytes(cb->type, cb->rank), cb->rank, out);
    default:
        return -1;
    }
}

/* select_draft_path (metal_dflash.rs:17176-17251) and its replay diagnose_dflash2_selector_walk
 * (:3473-3617): out[0] = ids[0]; for every later position the candidate b maximising
 * vals[pos][b] + sum_r (pred[r] * sel_h[pos][r]) * succ_b[r], sums in rank order with separate
 * products and additions, strict > (the first maximum wins, candidate 0 when nothing compares
 * greater), candidates that are negative or at/over the successor table's rows skipped; the
 * chosen token's predecessor row conditions the next position.  scores (optional, [n][top_k])
 * receives every evaluated score and valid (optional, [n][top_k]) marks which candidates were
 * evaluated rather than skipped.
 * Returns 0, or -1 when a predecessor row is out of range. */
int orc_select_draft_path(const orc_codebook *pred_cb, const orc_codebook *succ_cb, size_t top_k, size_t rank,
                          int32_t carry, size_t n, const int32_t *ids, const float *vals, const float *sel_h,
                          int32_t *out, float *scores, uint8_t *valid) {
    float *pred = (float *)malloc(sizeof(float) * rank * 3);
    if (!pred) return -1;
    float *succ = pred + rank, *gate = succ + rank;
    int rc = 0;
    if (n == 0) goto done;
    out[0] = ids[0];
    if (carry < 0 || orc_codebook_row(pred_cb, (size_t)carry, pred)) {
        rc = -1;
        goto done;
    }
    for (size_t pos = 1; pos < n; pos++) {
        const float *hrow = sel_h + pos * rank;
        for (size_t r = 0; r < rank; r++) gate[r] = pred[r] * hrow[r];
        size_t best_b = 0;
        float best = -INFINITY;
        for (size_t b = 0; b < top_k; b++) {
            const int32_t cand = ids[pos * top_k + b];
            if (valid) valid[pos * top_k + b] = 0;
            if (cand < 0 || (size_t)cand >= succ_cb->n_rows) continue;
            if (orc_codebook_row(succ_cb, (size_t)cand, succ)) {
                rc = -1;
                goto done;
            }
            float dot = 0.0f;
            for (size_t r = 0; r < rank; r++) dot += gate[r] * succ[r];
            const float score = vals[pos * top_k + b] + dot;
            if (valid) valid[pos * top_k + b] = 1;
            if (scores) scores[pos * top_k + b] = score;
            if (score > best) {
                best = score;
                best_b = b;
            }
        }
        const int32_t chosen = ids[pos * top_k + best_b];
        out[pos] = chosen;
        if (chosen < 0 || orc_codebook_row(pred_cb, (size_t)chosen, pred)) {
            rc = -1;
            goto done;
        }
    }
done:
    free(pred);
    return rc;
}

/* draft_block_sampled (metal_dflash.rs:17268-17415): the walk above, but each position's token is
 * drawn by sample_with_distribution (sampling.rs:439-453) over the top_k scores (skipped candidates
 * score -inf) with the proposal sampler, one committed draw per position.  out[] is pre-filled with
 * ids[0]; counts[pos-1] / cands[(pos-1)*top_k ..] receive the candidates with positive weight as
 * (token id, weight) in distribution order.  Returns 0, -1 for a codebook row out of range, or the
 * sampler's ORC_* code; *err_pos is the position of the error. */
int orc_select_draft_path_sampled(const orc_codebook *pred_cb, const orc_codebook *succ_cb, size_t top_k, size_t rank,
                                  int32_t carry, size_t n, const int32_t *ids, const float *vals, const float *sel_h,
                                  orc_sampler *proposal, int32_t *out, int32_t *counts, orc_weighted_candidate *cands,
                                  size_t *err_pos) {
    float *pred = (float *)malloc(sizeof(float) * (rank * 3 + top_k));
    orc_weighted_candidate *dc = (orc_weighted_candidate *)malloc(sizeof(orc_weighted_candidate) * top_k);
    int rc = 0;
    if (!pred || !dc) {
        rc = -1;
        goto done;
    }
    float *succ = pred + rank, *gate = succ + rank, *scores = gate + rank;
    for (size_t p = 0; p < n; p++) out[p] = ids[0];
    if (n == 0) goto done;
    if (carry < 0 || orc_codebook_row(pred_cb, (size_t)carry, pred)) {
        rc = -1;
        if (err_pos) *err_pos = 0;
        goto done;
    }
    for (size_t pos = 1; pos < n; pos++) {
        if (err_pos) *err_pos = pos;
        const float *hrow = sel_h + pos * rank;
        for (size_t r = 0; r < rank; r++) gate[r] = pred[r] * hrow[r];
        for (size_t b = 0; b < top_k; b++) {
            scores[b] = -INFINITY;
            const int32_t cand = ids[pos * top_k + b];
            if (cand < 0 || (size_t)cand >= succ_cb->n_rows) continue;
            if (orc_codebook_row(succ_cb, (size_t)cand, succ)) {
                rc = -1;
                goto done;
            }
            float dot = 0.0f;
            for (size_t r = 0; r < rank; r++) dot += gate[r] * succ[r];
            scores[b] = vals[pos * top_k + b] + dot;
        }
        orc_sampler next = *proposal;
        const double u = orc_sampler_next_unit(&next);
        size_t n_c = 0, idx = 0;
        double total = 0.0;
        int32_t tok = 0;
        int64_t err_index = -1;
        rc = orc_sampler_diagnose(proposal, scores, top_k, u, dc, top_k, &n_c, &total, &tok, &idx, &err_index);
        if (rc) goto done;
        next.draws = proposal->draws + 1;
        *proposal = next;
        const int32_t chosen = ids[pos * top_k + (size_t)tok];
        int32_t cnt = 0;
        for (size_t i = 0; i < n_c; i++) {
            if (!(dc[i].weight > 0.0)) continue;
            cands[(pos - 1) * top_k + cnt].token = ids[pos * top_k + (size_t)dc[i].token];
            cands[(pos - 1) * top_k + cnt].pad = 0;
            cands[(pos - 1) * top_k + cnt].weight = dc[i].weight;
            cnt++;
        }
        counts[pos - 1] = cnt;
        out[pos] = chosen;
        if (chosen < 0 || orc_codebook_row(pred_cb, (size_t)chosen, pred)) {
            rc = -1;
            goto done;
        }
    }
done:
    free(pred);
    free(dc);
    return rc;
}
