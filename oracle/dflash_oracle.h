/*
 * CPU oracle for the DFlash speculative-decoding step.
 *
 * TEST INFRASTRUCTURE ONLY.  This is a plain-C restatement of the reference
 * engine's CPU algorithms for the path (ggml block dequantisation, the
 * sampler-v1 chain and its speculative couplings, the accept-prefix decision,
 * the f32 forward primitives and the block-causal verify attention).  Nothing
 * in the shipped library links or calls it; only the test-suite, the smoke
 * check and the benchmark's CPU-baseline leg load it, and there only as the
 * checker.
 *
 * Every function names the reference file:line it follows (paths relative to
 * the reference repository root).
 *
 * Parity pins (what each part is checked against before it is trusted):
 *   - Q4_K / Q6_K / Q8_0 dequant ....... known blocks + closed forms held by the
 *       reference's tests (codec.rs:474-577, metal/tests/q6_k_f32_tile.rs:27-107)
 *   - SplitMix64 / xoshiro256++ / unit-f64 / sampled token stream .... golden
 *       vectors (sampling.rs:1817-1878)
 *   - greedy tie rule ................. sampling.rs:1904-1909
 *   - sampler chain ................... filter/tie cases (sampling.rs:1998-2049),
 *       brute-force comparator ordering, draw-count cases (sampling.rs:2940-2984)
 *   - couplings ....................... serial-stream invariance (sampling.rs:2837-2865),
 *       target-marginal preservation (sampling.rs:2889-2937)
 *   - accept-prefix ................... the value-specified cases of
 *       metal_dflash/accept.rs:236-616
 *   - Philox4x32-10 ................... Random123 known-answer vectors
 *   - attention / RMSNorm / RoPE / SiLU / softmax ... f64 brute force and
 *       closed forms (metal/dflash.rs:1306-1317, forward.rs:1384-1385)
 *   - dense-proposal coupling (orc_couple_dense_proposal): the reference never
 *       builds a dense proposal; this function is pinned only through its
 *       reduction to the sparse coupling on small vocabularies.
 *   - DFlash-2 conv ................... closed forms (one tap = a product, zero rows before the
 *       block, side/group indexing against an independent numpy gather)
 *   - DFlash-2 selector walk .......... the known-answer walks of metal_dflash/tests.rs:2978-3094
 *       (scores, first-tie rule, sentinel and non-finite candidates, invalid predecessor)
 *   - DFlash-2 drafter forward (orc_dflash_draft_ex): the reference has no CPU form of it and its
 *       model-witness tests need checkpoint files, so it is pinned by what the formula fixes.
 *       Static part, by reduction to the DFlash-1 forward bit for bit: identity convolutions (zero
 *       coefficient projections, identity base kernels) reproduce it; a per-channel power-of-two scaling
 *       on side 1 equals the DFlash-1 forward with the matching rows of attn_output / ffn_down scaled (so
 *       side 1 sits on the sublayer outputs, side 0 on their inputs).  Dynamic coefficients, always with
 *       non-zero projections (metal_dflash.rs:16210-16262, 16795-16885, 17003-17022): an independent
 *       float64 model of the whole layer; a projection that makes the coefficients a constant c equals
 *       the static forward with base + c on both sides, for the attention pair and for the FFN pair
 *       separately while the other pair keeps its own random projection (each pair reads ONE coefficient
 *       vector, of its own projection); a norm doubled with the projection halved leaves every bit
 *       unchanged (coefficients come from the normed, pre-convolution input).
 *   - f64 exp/ln are the host libm's, as the reference's are its platform's:
 *       last-ulp behaviour is parity unpinned (decisions compare against
 *       uniforms and are insensitive to it except with probability ~2^-50).
 */
#ifndef DFLASH_ORACLE_H
#define DFLASH_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- ggml block geometry (tensor.rs:164-208) ---- */
enum { ORC_Q8_0 = 8, ORC_Q4_K = 12, ORC_Q6_K = 14 };
enum { ORC_QK_K = 256, ORC_Q4_K_BYTES = 144, ORC_Q6_K_BYTES = 210, ORC_Q8_0_BYTES = 34, ORC_QK8_0 = 32 };

float orc_f16_to_f32(uint16_t h);
uint16_t orc_f32_to_f16(float f); /* round-to-nearest-even */

/* block dequantisation, n_elems a multiple of the block size; returns 0 or -1 */
int orc_dequant_q4_k(const uint8_t *blocks, size_t n_elems, float *out);
int orc_dequant_q6_k(const uint8_t *blocks, size_t n_elems, float *out);
int orc_dequant_q8_0(const uint8_t *blocks, size_t n_elems, float *out);
int orc_dequant(int type, const uint8_t *blocks, size_t n_elems, float *out);
size_t orc_row_bytes(int type, size_t n_in);

/* ---- RNG ---- */
uint64_t orc_splitmix64_next(uint64_t *state);
void orc_xoshiro_seed(uint64_t seed, uint64_t s[4]);
uint64_t orc_xoshiro_next(uint64_t s[4]);
double orc_unit_f64(uint64_t raw);
void orc_philox4x32_10(const uint32_t ctr[4], const uint32_t key[2], uint32_t out[4]);

/* ---- sampler-v1 ---- */
enum {
    ORC_OK = 0,
    ORC_ERR_EMPTY_LOGITS = 1,
    ORC_ERR_INVALID_TEMPERATURE = 2,
    ORC_ERR_INVALID_TOP_P = 3,
    ORC_ERR_INVALID_MIN_P = 4,
    ORC_ERR_NAN_LOGIT = 5,
    ORC_ERR_VOCAB_TOO_LARGE = 6,
    ORC_ERR_NO_CANDIDATES = 7,
    ORC_ERR_PROPOSAL_TOKEN_OUT_OF_RANGE = 8,
    ORC_ERR_INVALID_PROPOSAL_WEIGHT = 9,
    ORC_ERR_MISSING_PROPOSAL_TOKEN = 10,
    ORC_ERR_INVALID_INPUT = 11,
    ORC_ERR_INVALID_TOKEN = 12,
    ORC_ERR_PROPOSAL_MISMATCH = 13
};

enum { ORC_RNG_XOSHIRO = 0, ORC_RNG_PHILOX = 1 };

typedef struct {
    float temperature;
    float top_p;
    float min_p;
    int32_t rng_kind;
    uint64_t top_k;
    uint64_t seed;
} orc_sampling_config;

typedef struct {
    orc_sampling_config cfg;
    uint64_t s[4];  /* xoshiro state */
    uint64_t draws; /* draw count; also the Philox counter */
} orc_sampler;

typedef struct {
    int32_t token;
    int32_t pad;
    double weight;
} orc_weighted_candidate;

int orc_sampler_init(orc_sampler *s, const orc_sampling_config *cfg);
int orc_sampler_at_draw(orc_sampler *s, const orc_sampling_config *cfg, uint64_t draws);
double orc_sampler_next_unit(orc_sampler *s); /* advances the stream, does not count a draw */

int orc_greedy_token(const float *logits, size_t n, int32_t *token, int64_t *err_index);
/* argmax + (top1 - top2) gap with the verify-tail contract: lowest index on ties,
 * gap 0 on duplicate max, +inf for n == 1, all-NaN row -> -1 */
void orc_argmax_top2(const float *logits, size_t n, int32_t *idx, float *gap);
/* top-16 by (total-order value desc, index asc); missing slots idx=-1 */
void orc_top16(const float *logits, size_t n, int32_t ids[16], float vals[16]);

/* Filtered categorical distribution (candidates in sampler order + weights). `cap`
 * bounds the candidate array; returns ORC_* and the count in *n_out. */
int orc_sampler_diagnose(const orc_sampler *s, const float *logits, size_t n, double uniform,
                         orc_weighted_candidate *cands, size_t cap, size_t *n_out,
                         double *total_weight, int32_t *sampled_token, size_t *candidate_index,
                         int64_t *err_index);
int orc_sampler_sample(orc_sampler *s, const float *logits, size_t n, int32_t *token,
                       size_t *candidate_index, int64_t *err_index);
/* decision: 1 accepted, 0 rejected (correction set) */
int orc_couple_deterministic_proposal(orc_sampler *s, const float *logits, size_t n, int32_t proposal,
                                      int *accepted, int32_t *correction, int64_t *err_index);
int orc_couple_sparse_proposal(orc_sampler *s, const float *logits, size_t n, int32_t proposal_token,
                               const orc_weighted_candidate *prop, size_t n_prop, int *accepted,
                               int32_t *correction, int64_t *err_index);
/* dense proposal q = softmax(draft_logits / T_draft) over the whole vocabulary */
int orc_couple_dense_proposal(orc_sampler *s, const float *target_logits, const float *draft_logits,
                              size_t n, float draft_temperature, int32_t proposal_token, int *accepted,
                              int32_t *correction, int64_t *err_index);
double orc_dense_proposal_total(const float *draft_logits, size_t n, float draft_temperature,
                                int64_t *err_index);

/* ---- accept-prefix (metal_dflash/accept.rs:76-183) ---- */
enum { ORC_CARRY_NONE = 0, ORC_CARRY_CORRECTION = 1, ORC_CARRY_BONUS = 2 };
enum { ORC_STOP_NONE = 0, ORC_STOP_EOS = 1, ORC_STOP_TOKEN_LIMIT = 2 };

typedef struct {
    int32_t n_accepted;
    int32_t accepted_drafts[64];
    int32_t carry_kind;
    int32_t carry_token;
    int32_t stop_reason;
    int32_t retain_input_count;
    int32_t err_row;   /* row of a sampling error, -1 otherwise */
    int32_t err_code;  /* nested ORC_ERR_* for sampling errors */
    int64_t err_index; /* token index of a NaN / offending token */
} orc_accept_decision;

/* proposals: optional; row r has prop_counts[r] candidates starting at prop_offsets[r] */
int orc_decide_accept_prefix(const int32_t *verified_tokens, size_t n_tokens, const float *target_logits,
                             size_t n_logits, size_t vocab, int have_proposals, size_t n_proposals,
                             const int32_t *prop_tokens, const size_t *prop_offsets,
                             const size_t *prop_counts, const orc_weighted_candidate *prop_cands,
                             orc_sampler *sampler, size_t remaining_output_budget, const int32_t *stop_ids,
                             size_t n_stop, orc_accept_decision *out);
/* the same block decision with a dense draft distribution per row (config: vocab-wide q) */
int orc_decide_accept_prefix_dense(const int32_t *verified_tokens, size_t n_tokens,
                                   const float *target_logits, const float *draft_logits, size_t vocab,
                                   float draft_temperature, orc_sampler *sampler,
                                   size_t remaining_output_budget, const int32_t *stop_ids, size_t n_stop,
                                   orc_accept_decision *out);

/* n_trials independent block decisions (dense proposals when draft_logits != NULL, deterministic drafts otherwise),
 * OpenMP across trials; trial t uses samplers[t], verified_tokens[t][n_tokens], target_logits[t][n_tokens][vocab],
 * draft_logits[t][n_tokens-1][vocab] and writes out[t], status[t] */
void orc_decide_accept_prefix_batch(size_t n_trials, const int32_t *verified_tokens, size_t n_tokens,
                                    const float *target_logits, const float *draft_logits, size_t vocab,
                                    float draft_temperature, orc_sampler *samplers, size_t remaining_output_budget,
                                    orc_accept_decision *out, int32_t *status);

/* smallest relative router gap (last pick vs best expert left out) since the previous call; +inf if none */
float orc_router_margin_take(void);

/* ---- f32 forward primitives (forward.rs:1244-1371) ---- */
void orc_rms_norm(const float *x, const float *w, size_t n, float eps, float *out);
float orc_silu(float x);
void orc_softmax_in_place(float *x, size_t n);
void orc_mat_vec(const float *w, size_t n_in, size_t n_out, const float *x, float *y);
void orc_rope_in_place(float *buf, size_t n_heads, size_t head_dim, size_t n_rot, uint32_t position,
                       float theta_base);

/* few-row GEMM baseline: dequantise W then y[c][r] = sum_k W[r][k] x[c][k] (f32) */
int orc_gemm_fewrow(int type, const uint8_t *w, const float *x, float *y, size_t n_in, size_t n_out,
                    size_t n_rows);

/* block-causal verify attention: q [n_rows][n_q][hd] f32, K/V cache f16 [ctx_len+n_rows][n_kv][hd],
 * row i attends keys [0, ctx_len+i]; out [n_rows][n_q][hd] f32 (forward.rs:893-922 per row) */
void orc_attn_verify_block(const float *q, const uint16_t *k_cache, const uint16_t *v_cache,
                           size_t ctx_len, size_t n_rows, size_t n_q, size_t n_kv, size_t hd, float scale,
                           float *out);

/* drafter attention over ctx || noise with causal / sliding-window mask (forward.rs:559-606) */
void orc_attn_draft(const float *q, const float *k_ctx, const float *v_ctx, const float *k_noise,
                    const float *v_noise, const int32_t *pos_ctx, size_t ctx_len, size_t n, size_t n_q,
                    size_t n_kv, size_t hd, uint32_t noise_start_pos, int causal, uint32_t swa_window,
                    float *out);

/* ---- synthetic dense decoder / drafter (forward.rs:96-163, 380-662, 725-932) ---- */
typedef struct {
    int32_t n_layers, hidden, n_q, n_kv, head_dim, ffn, vocab;
    int32_t n_expert, n_expert_used, ffn_expert, ffn_shared; /* n_expert == 0 -> dense FFN */
    float eps, rope_theta;
} orc_model_cfg;

typedef struct {
    int32_t type;
    int32_t pad;
    const uint8_t *data;
} orc_qtensor; /* quant blocks, row-major [n_out][n_in/blk] */

typedef struct {
    const float *attn_norm, *q_norm, *k_norm, *post_norm; /* f32 norm weights */
    orc_qtensor wq, wk, wv, wo, gate, up, down;           /* dense FFN or shared expert */
    orc_qtensor router;                                   /* [H -> E] (MoE only) */
    const float *shexp_gate;                              /* [H] f32 (MoE only) */
    orc_qtensor gate_exps, up_exps, down_exps;            /* [E] stacked expert matrices */
} orc_layer;

typedef struct {
    orc_model_cfg cfg;
    const orc_layer *layers;
    orc_qtensor token_embd, output; /* [V] rows of H */
    const float *output_norm;
} orc_model;

/* verify n tokens at start_pos..: appends K,V (f16) to caches [layer][cap][n_kv*hd], returns logits
 * [n][V] and optionally the pre-output-norm hidden of `n_tap` tapped layers laid out [n][n_tap][H] */
int orc_target_verify(const orc_model *m, const int32_t *tokens, size_t n, size_t start_pos,
                      uint16_t *k_cache, uint16_t *v_cache, size_t kv_capacity, float *logits,
                      const int32_t *tap_layers, size_t n_tap, float *hidden_capture);

typedef struct {
    int32_t n_layers, hidden, n_q, n_kv, head_dim, ffn, block_size, n_taps;
    int32_t causal;
    uint32_t swa_window;
    float eps, rope_theta;
} orc_draft_cfg;

typedef struct {
    const float *attn_norm, *q_norm, *k_norm, *post_norm;
    orc_qtensor wq, wk, wv, wo, gate, up, down;
    int32_t is_swa;
    int32_t pad;
} orc_draft_layer;

typedef struct {
    orc_draft_cfg cfg;
    const orc_draft_layer *layers;
    orc_qtensor fc; /* [n_taps*H -> H] */
    const float *hidden_norm, *output_norm;
} orc_draft_head;

/* forward.rs:380-662; embeddings and lm_head come from the target model */
int orc_dflash_draft(const orc_model *target, const orc_draft_head *head, const int32_t *noise_ids,
                     const float *target_ctx_stacked, size_t ctx_len, const int32_t *pos_ctx,
                     uint32_t noise_start_pos, float *logits);

/* ---- DFlash-2 extras (dflash2.c) ---- */
enum { ORC_F32 = 0, ORC_F16 = 1 };

/* kernels/dflash2.metal:40-69; x, y [n_tokens][h]; dyn [n_tokens][2*kernel_size*h/group_size]
 * laid out (group, tap, side) fastest to slowest; base [2][kernel_size][h] */
void orc_dflash2_conv(const float *x, const float *dyn, const float *base, float *y, size_t n_tokens, size_t h,
                      size_t kernel_size, size_t group_size, size_t side);

/* selector codebook: [n_rows][rank] rows of F32, F16, Q8_0 or Q4_K (metal_dflash.rs:3200-3343) */
typedef struct {
    int32_t type;
    int32_t pad;
    size_t rank, n_rows;
    const void *data;
} orc_codebook;

int orc_codebook_row(const orc_codebook *cb, size_t row, float *out);

/* metal_dflash.rs:17176-17251, 3473-3617 */
int orc_select_draft_path(const orc_codebook *pred_cb, const orc_codebook *succ_cb, size_t top_k, size_t rank,
                          int32_t carry, size_t n, const int32_t *ids, const float *vals, const float *sel_h,
                          int32_t *out, float *scores, uint8_t *valid);

/* metal_dflash.rs:17268-17415 */
int orc_select_draft_path_sampled(const orc_codebook *pred_cb, const orc_codebook *succ_cb, size_t top_k, size_t rank,
                                  int32_t carry, size_t n, const int32_t *ids, const float *vals, const float *sel_h,
                                  orc_sampler *proposal, int32_t *out, int32_t *counts, orc_weighted_candidate *cands,
                                  size_t *err_pos);

/* DFlash-2 drafter forward (draft_block_inner with layer.conv and head.selector present,
 * metal_dflash.rs:16195-16275, 16795-16900, 17003-17030, 17098-17130): per layer, the dynamic
 * coefficients dyn = conv_proj . (normed sublayer input) serve both sides of a sublayer; side 0
 * convolves the normed input that q/k/v (gate/up) read, side 1 convolves the sublayer's output
 * (attn_output / ffn_down) before the residual add.  The tail also returns the selector gate
 * sel_h = selector_hidden . (output-normed hidden), [block][selector_rank].  ext == NULL is
 * orc_dflash_draft. */
typedef struct {
    int32_t conv_kernel_size, conv_group_size, selector_rank, pad;
    const orc_qtensor *conv_attn_proj, *conv_ffn_proj; /* [n_layers], each [H -> 2*kernel*H/group] */
    const float *const *conv_attn_base;                /* [n_layers] -> [2][kernel][H] */
    const float *const *conv_ffn_base;
    orc_qtensor selector_hidden;                       /* [H -> rank] */
} orc_dflash2_ext;

int orc_dflash_draft_ex(const orc_model *target, const orc_draft_head *head, const orc_dflash2_ext *ext,
                        const int32_t *noise_ids, const float *target_ctx_stacked, size_t ctx_len,
                        const int32_t *pos_ctx, uint32_t noise_start_pos, float *logits, float *sel_h);

#ifdef __cplusplus
}
#endif
#endif
