// DFlash-2 extras of the block drafter: the two-tap dynamic depthwise convolution
// (kernel_dflash2_conv_f32, kernels/dflash2.metal:40-69) and the greedy selector walk over the
// predecessor / successor codebooks (select_draft_path, metal_dflash.rs:17176-17251; codebook rows
// DFlash2Codebook::dequant_row, :3275-3343) with its sampled form (draft_block_sampled,
// :17268-17415).  The per-row top-16 that feeds the walk is dflash_top16.
#include "common.h"
#include "device_quant.h"
#include "sampler_chain.h"

// The walk's scores follow the reference's scalar loop: every product and every addition is
// rounded on its own: plain operators with contraction switched off (the __f*_rn intrinsics do not
// stop the compiler from fusing them).
#pragma clang fp contract(off)

namespace {

// y[t][c] = sum_tap (base[side][tap][c] + dyn[t][side][tap][c / group_size]) * x[t - tap][c]; rows
// before the block count as zeros; taps accumulate in order with a fused multiply-add, as the
// reference kernel does.  One thread per element.
__global__ void __launch_bounds__(256)
    dflash2_conv_kernel(const float *__restrict__ x, const float *__restrict__ dyn, const float *__restrict__ base,
                        float *__restrict__ y, int n_tokens, int h, int kernel_size, int group_size, int side,
                        void *__restrict__ y_xf, int y_xf_kind) {
    const int64_t gid = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (gid >= static_cast<int64_t>(n_tokens) * h) return;
    const int t = static_cast<int>(gid / h), c = static_cast<int>(gid % h);
    const int n_groups = h / group_size, g = c / group_size;
    const size_t dyn_row = static_cast<size_t>(t) * 2 * kernel_size * n_groups + static_cast<size_t>(side) * kernel_size * n_groups;
    const size_t base_side = static_cast<size_t>(side) * kernel_size * h;
    float acc = 0.0f;
    for (int tap = 0; tap < kernel_size && tap <= t; tap++) {
        const float b = base[base_side + static_cast<size_t>(tap) * h + c];
        const float d = dyn[dyn_row + static_cast<size_t>(tap) * n_groups + g];
        acc = __builtin_fmaf(b + d, x[static_cast<size_t>(t - tap) * h + c], acc);
    }
    y[gid] = acc;
    if (y_xf) {
        // (h a multiple of 256: the grid has no ragged end and eight consecutive lanes hold eight consecutive channels of a row)
        float v[8];
#pragma unroll
        for (int i = 0; i < 8; i++) v[i] = __shfl_down(acc, i, 64);
        if ((c & 7) == 0) dfl_xf_store(y_xf, y_xf_kind, t, c, v[0], v[1], v[2], v[3], v[4], v[5], v[6], v[7]);
    }
}

struct Codebook {
    int type;
    int rank;
    int64_t n_rows;
    const uint8_t *data;
    size_t row_bytes;
};

// element r of row `row`
__device__ __forceinline__ float codebook_elem(const Codebook &cb, int64_t row, int r) {
    const uint8_t *p = cb.data + static_cast<size_t>(row) * cb.row_bytes;
    if (cb.type == DFLASH_TYPE_F16) return __half2float(reinterpret_cast<const __half *>(p)[r]);
    return dfl_dequant_elem(cb.type, p, r);
}

constexpr int kSelThreads = 256;
constexpr int kSelMaxTopK = 16;
constexpr int kSelMaxRank = 1024;

// What the sampled walk reports besides the tokens.
struct SampledOut {
    int32_t status;      // 0, 1 = predecessor row out of range, else a DFLASH_ERR_* of the sampler
    int32_t err_pos;     // position of that error
    int32_t n_sampled;   // positions whose draw was made (the proposal sampler advances by this)
    int32_t pad;
    int32_t counts[16];                          // candidates with positive weight per position (index pos - 1)
    dflash_weighted_candidate cands[15 * 16];    // [pos - 1][top_k], distribution order
};

// where the raw rows sit in the scores kernel's LDS, behind the decoded ones (bytes)
__host__ __device__ inline size_t sel_raw_pred_bytes(size_t row_bytes) { return (row_bytes + 15) / 16 * 16; }
__host__ __device__ inline size_t sel_raw_succ_stride(size_t row_bytes) { return (row_bytes + 3) / 4 * 4; }
// floats of the decoded rows in front of them: gate[rank], succ[top_k][rank + 1], rounded up to a 16-byte boundary
__host__ __device__ inline size_t sel_decoded_floats(int top_k, int rank) {
    return (static_cast<size_t>(rank) + static_cast<size_t>(top_k) * (rank + 1) + 3) / 4 * 4;
}

// The walk's scores do not have to wait for the walk: the predecessor of position pos is one of the top_k candidates
// of position pos - 1 (the carry token for pos = 1), so score(pos, a, b) for every candidate a of the previous position
// and every candidate b of this one is known work up front: (n - 1) x top_k workgroups, all at once, each with the
// reference's arithmetic for its sixteen scores.  Workgroup (a, pos): all threads dequantise the predecessor row of
// candidate a and the successor rows of position pos's candidates and form gate = pred * sel_h[pos] in LDS; thread b
// then scores candidate b with the reference's scalar loop (products and additions rounded separately, rank order):
// table[pos - 1][a][b] = vals[pos][b] + sum_r gate[r] * succ_b[r], NaN for a candidate without a successor row.  A
// previous candidate without a predecessor row gets no scores: the walk stops when it picks one.
__global__ void __launch_bounds__(kSelThreads)
    dflash2_scores_kernel(Codebook pred_cb, Codebook succ_cb, int top_k, int rank, int carry, int n,
                          const int32_t *__restrict__ ids, const float *__restrict__ vals, const float *__restrict__ sel_h,
                          float *__restrict__ table) {
    extern __shared__ float lds[];  // gate[rank], succ[top_k][rank + 1], then the raw rows: predecessor, top_k successors
    // (a successor row every rank + 1 floats: the sixteen scoring threads read element r of sixteen rows at once, and rows
    // a power of two apart would all sit in one bank)
    float *gate = lds, *succ = lds + rank;
    const int srow = rank + 1;
    const int tid = threadIdx.x;
    const int a = blockIdx.x, pos = 1 + blockIdx.y;
    if (pos == 1 && a != 0) return;  // (one predecessor only: the carry token)
    const int32_t prev = pos == 1 ? carry : ids[(pos - 1) * top_k + a];
    if (prev < 0 || prev >= pred_cb.n_rows) return;
    // The rows' bytes come in with coalesced loads first (decoding element by element straight from memory cost a cold
    // trip per field of every element).  Rows of every codebook type are a whole number of 2-byte words and start on
    // one; in LDS the predecessor row sits first and the successor rows follow, each on a 4-byte boundary.
    uint8_t *raw = reinterpret_cast<uint8_t *>(lds + sel_decoded_floats(top_k, rank));
    const int pw = static_cast<int>(pred_cb.row_bytes / 2), sw = static_cast<int>(succ_cb.row_bytes / 2);
    const size_t succ_at = sel_raw_pred_bytes(pred_cb.row_bytes), succ_stride = sel_raw_succ_stride(succ_cb.row_bytes);
    {
        const uint16_t *src = reinterpret_cast<const uint16_t *>(pred_cb.data + static_cast<size_t>(prev) * pred_cb.row_bytes);
        for (int i = tid; i < pw; i += kSelThreads) reinterpret_cast<uint16_t *>(raw)[i] = src[i];
    }
    for (int e = tid; e < top_k * sw; e += kSelThreads) {
        const int b = e / sw, i = e - b * sw;
        const int32_t cand = ids[pos * top_k + b];
        if (cand >= 0 && cand < succ_cb.n_rows)
            reinterpret_cast<uint16_t *>(raw + succ_at + b * succ_stride)[i] =
                reinterpret_cast<const uint16_t *>(succ_cb.data + static_cast<size_t>(cand) * succ_cb.row_bytes)[i];
    }
    __syncthreads();
    Codebook pred_l = pred_cb, succ_l = succ_cb;  // the same rows, now rows of an LDS copy
    pred_l.data = raw;
    succ_l.data = raw + succ_at;
    succ_l.row_bytes = succ_stride;
    const float *hrow = sel_h + static_cast<size_t>(pos) * rank;
    for (int r = tid; r < rank; r += kSelThreads) gate[r] = codebook_elem(pred_l, 0, r) * hrow[r];
    for (int e = tid; e < top_k * rank; e += kSelThreads) {
        const int b = e / rank, r = e - b * rank;
        const int32_t cand = ids[pos * top_k + b];
        if (cand >= 0 && cand < succ_cb.n_rows) succ[b * srow + r] = codebook_elem(succ_l, b, r);
    }
    __syncthreads();
    if (tid < top_k) {
        const int32_t cand = ids[pos * top_k + tid];
        float sc = __builtin_nanf("");  // skipped candidates never compare greater
        if (cand >= 0 && cand < succ_cb.n_rows) {
            float dot = 0.0f;
            const float *sr = succ + tid * srow;
            for (int r = 0; r < rank; r++) dot += gate[r] * sr[r];  // two roundings each (contraction is off in this file)
            sc = vals[pos * top_k + tid] + dot;
        }
        table[(static_cast<size_t>(pos - 1) * top_k + a) * top_k + tid] = sc;
    }
}

// The walk over the table, one workgroup: the table and the candidates go to LDS, thread 0 then follows the picks.
// Per position it keeps the first strict maximum of the previous pick's row of scores (greedy) or samples from
// softmax(score / T) with the sampler chain and the position's pre-drawn uniform (SAMPLED).  status: 0, or 1 when a
// picked token has no predecessor row (the walk stops there).
template <bool SAMPLED>
__global__ void __launch_bounds__(kSelThreads)
    dflash2_select_kernel(int64_t n_pred_rows, int64_t n_succ_rows, int top_k, int carry, int n, const int32_t *__restrict__ ids,
                          const float *__restrict__ table, int32_t *__restrict__ out, int32_t *__restrict__ status,
                          float temperature, const double *__restrict__ uniforms, SampledOut *__restrict__ sampled) {
    __shared__ float table_s[15 * kSelMaxTopK * kSelMaxTopK];
    __shared__ int32_t ids_s[16 * kSelMaxTopK];
    __shared__ RowDist dist;
    const int tid = threadIdx.x;
    if (tid == 0) {
        out[0] = ids[0];
        *status = 0;
        if (SAMPLED) {
            sampled->status = 0;
            sampled->err_pos = 0;
            sampled->n_sampled = 0;
            for (int p = 1; p < n; p++) out[p] = ids[0];  // the reference pre-fills every slot with the anchor's top-1
        }
    }
    if (n < 2) return;
    if (carry < 0 || carry >= n_pred_rows) {
        if (tid == 0) *status = 1;
        return;
    }
    for (int e = tid; e < (n - 1) * top_k * top_k; e += kSelThreads) table_s[e] = table[e];
    for (int e = tid; e < n * top_k; e += kSelThreads) ids_s[e] = ids[e];
    __syncthreads();
    if (!SAMPLED) {
        // greedy: lane b holds candidate b of the position; the first strict maximum over the candidates with a successor
        // row, as the scalar loop `if (score[b] > best)` from best = -inf keeps it (a NaN or -inf score is never greater:
        // with none greater, candidate 0 stands)
        if (tid >= 64) return;
        int prev_a = 0;
        for (int pos = 1; pos < n; pos++) {
            float sc = -INFINITY;
            int32_t cand = -1;
            if (tid < top_k) {
                cand = ids_s[pos * top_k + tid];
                const float v = table_s[(static_cast<size_t>(pos - 1) * top_k + prev_a) * top_k + tid];
                if (cand >= 0 && cand < n_succ_rows && v > -INFINITY) sc = v;
            }
            float best = sc;
#pragma unroll
            for (int off = 1; off < 16; off <<= 1) best = fmaxf(best, __shfl_xor(best, off, 64));
            best = __shfl(best, 0, 64);  // (lanes 0..15 agree; the others hold -inf)
            const unsigned long long at = __ballot(tid < top_k && sc == best && best > -INFINITY);
            const int best_b = at ? __builtin_ctzll(at) : 0;
            const int32_t chosen = __shfl(cand, best_b, 64);
            if (tid == 0) out[pos] = chosen;
            if (chosen < 0 || chosen >= n_pred_rows) {
                if (tid == 0) *status = 1;
                return;
            }
            prev_a = best_b;
        }
        return;
    }
    if (tid != 0) return;
    int prev_a = 0;  // which candidate of the previous position was picked (the carry token's scores sit in row 0)
    for (int pos = 1; pos < n; pos++) {
        const float *score = table_s + (static_cast<size_t>(pos - 1) * top_k + prev_a) * top_k;
        const int32_t *cands = ids_s + pos * top_k;
        int best_b = 0;
        if (!SAMPLED) {
            float best = -INFINITY;
            for (int b = 0; b < top_k; b++) {
                const int32_t cand = cands[b];
                if (cand < 0 || cand >= n_succ_rows) continue;
                if (score[b] > best) {
                    best = score[b];
                    best_b = b;
                }
            }
        } else {
            // scores of skipped candidates are -inf; the "tokens" of the distribution are candidate indices
            uint64_t keys[kSelMaxTopK];
            int nan_at = -1;
            for (int b = 0; b < top_k; b++) {
                const int32_t cand = cands[b];
                const float sc = (cand < 0 || cand >= n_succ_rows) ? -INFINITY : score[b];
                if (sc != sc && nan_at < 0) nan_at = b;
                const uint64_t key = cand_key(static_cast<uint32_t>(b), sc);
                int j = b;  // insertion sort, ascending keys = best first
                while (j > 0 && keys[j - 1] > key) {
                    keys[j] = keys[j - 1];
                    j--;
                }
                keys[j] = key;
            }
            dist.err = 0;
            if (nan_at >= 0) {
                dist.err = DFLASH_ERR_NAN_LOGIT;
            } else {
                ChainCfg cc = {};
                cc.temperature = temperature;
                cc.top_p = 1.0f;
                cc.min_p = 0.0f;
                cc.k = top_k;
                run_chain(keys, top_k, cc, &dist);
            }
            if (dist.err) {
                sampled->status = dist.err;
                sampled->err_pos = pos;
                *status = dist.err;
                return;  // sampler error: the walk stops
            }
            const int idx = pick_index(dist.weights, dist.n_keep, uniforms[pos - 1] * dist.total);
            best_b = dist.tokens[idx];
            sampled->n_sampled = pos;
            int cnt = 0;
            for (int i = 0; i < dist.n_keep; i++) {
                if (!(dist.weights[i] > 0.0)) continue;
                dflash_weighted_candidate &wc = sampled->cands[(pos - 1) * top_k + cnt++];
                wc.token = cands[dist.tokens[i]];
                wc.weight = dist.weights[i];
            }
            sampled->counts[pos - 1] = cnt;
        }
        const int32_t chosen = cands[best_b];
        out[pos] = chosen;
        if (chosen < 0 || chosen >= n_pred_rows) {
            *status = 1;
            if (SAMPLED) {
                sampled->status = 1;
                sampled->err_pos = pos;
            }
            return;
        }
        prev_a = best_b;
    }
}

// Both launches of a walk: the score table ((n - 1) x top_k x top_k floats of context workspace behind *ws_off), then
// the walk itself.
template <bool SAMPLED>
int32_t launch_walk(dflash_ctx *ctx, size_t *ws_off, const Codebook &pc, const Codebook &sc, int top_k, int rank, int carry, int n,
                    const int32_t *ids, const float *vals, const float *sel_h, int32_t *out, int32_t *status, float temperature,
                    const double *uniforms, SampledOut *sampled, hipStream_t st) {
    float *table = dfl_ws_take<float>(ctx, ws_off, static_cast<size_t>(15) * kSelMaxTopK * kSelMaxTopK * sizeof(float));
    if (!table) return dfl_fail(ctx, DFLASH_ERR_WORKSPACE, "select_draft_path: workspace too small");
    if (n > 1) {
        // (decoded rows as floats + the same rows' bytes)
        const size_t lds = sel_decoded_floats(top_k, rank) * sizeof(float) + sel_raw_pred_bytes(pc.row_bytes) +
                           static_cast<size_t>(top_k) * sel_raw_succ_stride(sc.row_bytes);
        if (pc.row_bytes % 2 || sc.row_bytes % 2 || reinterpret_cast<uintptr_t>(pc.data) % 2 || reinterpret_cast<uintptr_t>(sc.data) % 2)
            return dfl_fail(ctx, DFLASH_ERR_ALIGNMENT, "select_draft_path: codebook rows must start on 2-byte boundaries");
        if (lds > 48 * 1024) {
            if (const int32_t rc_ = dfl_raise_lds_limit(ctx, reinterpret_cast<const void *>(dflash2_scores_kernel), lds)) return rc_;
        }
        dflash2_scores_kernel<<<dim3(top_k, n - 1), kSelThreads, lds, st>>>(pc, sc, top_k, rank, carry, n, ids, vals, sel_h, table);
    }
    dflash2_select_kernel<SAMPLED><<<1, kSelThreads, 0, st>>>(pc.n_rows, sc.n_rows, top_k, carry, n, ids, table, out, status, temperature,
                                                               uniforms, sampled);
    DFL_HIP_CHECK(ctx, hipGetLastError());
    return DFLASH_OK;
}

int32_t check_codebook(dflash_ctx *ctx, const dflash_codebook *cb, int rank, Codebook *out, const char *what) {
    if (!cb || !cb->data || cb->n_rows < 1) return dfl_fail(ctx, DFLASH_ERR_INVALID_INPUT, "select_draft_path: %s codebook", what);
    size_t rb = 0;
    switch (cb->type) {
    case DFLASH_TYPE_F32: rb = static_cast<size_t>(rank) * 4; break;
    case DFLASH_TYPE_F16: rb = static_cast<size_t>(rank) * 2; break;
    case DFLASH_TYPE_Q8_0:
    case DFLASH_TYPE_Q4_K: rb = dflash_row_bytes(cb->type, rank); break;
    default: break;
    }
    if (rb == 0)
        return dfl_fail(ctx, DFLASH_ERR_UNSUPPORTED, "select_draft_path: %s codebook type %d with rank %d", what, cb->type, rank);
    *out = Codebook{cb->type, rank, cb->n_rows, static_cast<const uint8_t *>(cb->data), rb};
    return DFLASH_OK;
}

}  // namespace

extern "C" int32_t dflash_dflash2_conv(dflash_ctx *ctx, const float *x, const float *dyn, const float *base, float *y,
                                       int32_t n_tokens, int32_t h, int32_t kernel_size, int32_t group_size, int32_t side,
                                       dflash_stream_t stream) {
    return dfl_dflash2_conv(ctx, x, dyn, base, y, n_tokens, h, kernel_size, group_size, side, stream, nullptr, DFL_XF_NONE);
}

int32_t dfl_dflash2_conv(dflash_ctx *ctx, const float *x, const float *dyn, const float *base, float *y, int32_t n_tokens, int32_t h,
                         int32_t kernel_size, int32_t group_size, int32_t side, dflash_stream_t stream, void *y_xf, int y_xf_kind) {
    if (!ctx) return DFLASH_ERR_INVALID_INPUT;
    if (y_xf && (h % DFL_QK_K || n_tokens > 16 || (y_xf_kind != DFL_XF_Q4K && y_xf_kind != DFL_XF_Q6K)))
        return dfl_fail(ctx, DFLASH_ERR_BAD_SHAPE, "dflash2_conv: fragment-order output needs h %% 256 == 0, at most 16 rows and a kind");
    if (!x || !dyn || !base || !y) return dfl_fail(ctx, DFLASH_ERR_INVALID_INPUT, "dflash2_conv: null pointer");
    if (n_tokens < 1 || h < 1 || kernel_size < 1 || group_size < 1 || h % group_size || (side != 0 && side != 1))
        return dfl_fail(ctx, DFLASH_ERR_BAD_SHAPE, "dflash2_conv: n_tokens %d h %d kernel %d group %d side %d", n_tokens, h,
                        kernel_size, group_size, side);
    const size_t bytes = static_cast<size_t>(n_tokens) * h * sizeof(float);
    if (dfl_ranges_overlap(y, bytes, x, bytes))
        return dfl_fail(ctx, DFLASH_ERR_ALIAS, "dflash2_conv: y aliases x (taps read neighbouring rows)");
    const int64_t total = static_cast<int64_t>(n_tokens) * h;
    dflash2_conv_kernel<<<static_cast<unsigned>((total + 255) / 256), 256, 0, static_cast<hipStream_t>(stream)>>>(
        x, dyn, base, y, n_tokens, h, kernel_size, group_size, side, y_xf, y_xf_kind);
    DFL_HIP_CHECK(ctx, hipGetLastError());
    return DFLASH_OK;
}

extern "C" int32_t dflash_select_draft_path(dflash_ctx *ctx, const dflash_codebook *predecessor,
                                            const dflash_codebook *successor, int32_t rank, int32_t top_k, int32_t carry_token,
                                            int32_t n, const int32_t *topk_ids, const float *topk_vals, const float *sel_h,
                                            int32_t *out_tokens, int32_t *out_tokens_host, dflash_stream_t stream) {
    if (!ctx) return DFLASH_ERR_INVALID_INPUT;
    if (!topk_ids || !topk_vals || !sel_h || !out_tokens)
        return dfl_fail(ctx, DFLASH_ERR_INVALID_INPUT, "select_draft_path: null pointer");
    if (n < 1 || n > 16 || top_k < 1 || top_k > kSelMaxTopK || rank < 1 || rank > kSelMaxRank)
        return dfl_fail(ctx, DFLASH_ERR_BAD_SHAPE, "select_draft_path: n %d top_k %d rank %d", n, top_k, rank);
    Codebook pc, sc;
    int32_t rc;
    if ((rc = check_codebook(ctx, predecessor, rank, &pc, "predecessor"))) return rc;
    if ((rc = check_codebook(ctx, successor, rank, &sc, "successor"))) return rc;
    size_t off = 0;
    int32_t *status = dfl_ws_take<int32_t>(ctx, &off, sizeof(int32_t));
    if (!status) return dfl_fail(ctx, DFLASH_ERR_WORKSPACE, "select_draft_path: workspace too small");
    hipStream_t st = static_cast<hipStream_t>(stream);
    if ((rc = launch_walk<false>(ctx, &off, pc, sc, top_k, rank, carry_token, n, topk_ids, topk_vals, sel_h, out_tokens, status, 0.0f,
                                 nullptr, nullptr, st)))
        return rc;
    if (out_tokens_host) {
        // the blocking form also reports an invalid predecessor row, as the reference's CPU walk does
        int32_t status_host = 0;
        DFL_HIP_CHECK(ctx, hipMemcpyAsync(out_tokens_host, out_tokens, n * sizeof(int32_t), hipMemcpyDeviceToHost, st));
        DFL_HIP_CHECK(ctx, hipMemcpyAsync(&status_host, status, sizeof(int32_t), hipMemcpyDeviceToHost, st));
        DFL_HIP_CHECK(ctx, hipStreamSynchronize(st));
        if (status_host) return dfl_fail(ctx, DFLASH_ERR_INVALID_TOKEN, "select_draft_path: selector codebook row out of range");
    }
    return DFLASH_OK;
}

extern "C" int32_t dflash_select_draft_path_sampled(dflash_ctx *ctx, const dflash_codebook *predecessor,
                                                    const dflash_codebook *successor, int32_t rank, int32_t top_k,
                                                    int32_t carry_token, int32_t n, const int32_t *topk_ids,
                                                    const float *topk_vals, const float *sel_h,
                                                    dflash_sampler *proposal_sampler, int32_t *out_tokens_host,
                                                    int32_t *prop_counts_host, dflash_weighted_candidate *prop_cands_host,
                                                    dflash_stream_t stream) {
    if (!ctx) return DFLASH_ERR_INVALID_INPUT;
    if (!topk_ids || !topk_vals || !sel_h || !proposal_sampler || !out_tokens_host || !prop_counts_host || !prop_cands_host)
        return dfl_fail(ctx, DFLASH_ERR_INVALID_INPUT, "select_draft_path_sampled: null pointer");
    if (n < 1 || n > 16 || top_k < 1 || top_k > kSelMaxTopK || rank < 1 || rank > kSelMaxRank)
        return dfl_fail(ctx, DFLASH_ERR_BAD_SHAPE, "select_draft_path_sampled: n %d top_k %d rank %d", n, top_k, rank);
    const dflash_sampling_config &pc_cfg = proposal_sampler->cfg;
    if (!(pc_cfg.temperature > 0.0f) || pc_cfg.top_k != 0 || pc_cfg.top_p != 1.0f || pc_cfg.min_p != 0.0f)
        return dfl_fail(ctx, DFLASH_ERR_INVALID_INPUT,
                        "select_draft_path_sampled: the proposal sampler must use temperature without target filters");
    Codebook pc, sc;
    int32_t rc;
    if ((rc = check_codebook(ctx, predecessor, rank, &pc, "predecessor"))) return rc;
    if ((rc = check_codebook(ctx, successor, rank, &sc, "successor"))) return rc;
    size_t off = 0;
    int32_t *status = dfl_ws_take<int32_t>(ctx, &off, sizeof(int32_t));
    int32_t *out_dev = dfl_ws_take<int32_t>(ctx, &off, 16 * sizeof(int32_t));
    double *uniforms = dfl_ws_take<double>(ctx, &off, 16 * sizeof(double));
    SampledOut *sampled = dfl_ws_take<SampledOut>(ctx, &off, sizeof(SampledOut));
    if (!status || !out_dev || !uniforms || !sampled)
        return dfl_fail(ctx, DFLASH_ERR_WORKSPACE, "select_draft_path_sampled: workspace too small");
    hipStream_t st = static_cast<hipStream_t>(stream);
    // one uniform per position, drawn ahead; the sampler is advanced afterwards by the draws actually made
    double u_host[16] = {0};
    if (n > 1) dflash_sampler_peek(proposal_sampler, n - 1, u_host);
    DFL_HIP_CHECK(ctx, hipMemcpyAsync(uniforms, u_host, sizeof(u_host), hipMemcpyHostToDevice, st));
    if ((rc = launch_walk<true>(ctx, &off, pc, sc, top_k, rank, carry_token, n, topk_ids, topk_vals, sel_h, out_dev, status,
                                pc_cfg.temperature, uniforms, sampled, st)))
        return rc;
    static_assert(sizeof(SampledOut) <= DFL_PINNED_BYTES, "the walk's result is read back through the context's pinned page");
    const SampledOut &host = *static_cast<const SampledOut *>(ctx->pinned);
    DFL_HIP_CHECK(ctx, hipMemcpyAsync(ctx->pinned, sampled, sizeof(SampledOut), hipMemcpyDeviceToHost, st));
    DFL_HIP_CHECK(ctx, hipMemcpyAsync(out_tokens_host, out_dev, n * sizeof(int32_t), hipMemcpyDeviceToHost, st));
    DFL_HIP_CHECK(ctx, hipStreamSynchronize(st));
    // every completed position consumed one draw, as each sample_with_distribution call commits its own
    dflash_sampler_advance(proposal_sampler, static_cast<uint64_t>(host.n_sampled));
    if (host.status == 1)
        return dfl_fail(ctx, DFLASH_ERR_INVALID_TOKEN, "select_draft_path_sampled: selector codebook row out of range at position %d",
                        host.err_pos);
    if (host.status) return dfl_fail(ctx, host.status, "select_draft_path_sampled: sampler error at position %d", host.err_pos);
    for (int p = 0; p + 1 < n; p++) {
        prop_counts_host[p] = host.counts[p];
        for (int i = 0; i < host.counts[p]; i++) prop_cands_host[p * top_k + i] = host.cands[p * top_k + i];
    }
    return DFLASH_OK;
}
