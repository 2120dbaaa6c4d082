// Block-causal verify attention: the 16 draft rows of a block attend the whole prefix and
// each other causally, over an f16 KV cache, GQA.
//
// Replaces the reference's per-row loop (metal_dflash.rs:9963-10062: scatter one K/V row,
// then one single-query decode attention, sixteen times; kernels attn_v4.metal /
// attn.metal:266-336) with one pass that streams the KV cache once for all 16 rows:
//     o[i][h] = softmax(q[i][h] . K[0..L+i, kv(h)] * scale) . V[0..L+i, kv(h)]
//
// Mapping onto CDNA4 (split-KV flash decoding on MFMA):
//  * grid = (KV splits) x (KV heads); a workgroup owns one KV head and one contiguous chunk of
//    key positions; each of its waves owns one query head of the GQA group, i.e. a 16-row tile
//    (the block's rows are exactly the 16-wide side of v_mfma_f32_16x16x32_f16).
//  * scores are computed transposed, S^T = K . Q^T: K rows are the A operand in their natural
//    layout (a lane reads 16 contiguous bytes of a key), Q^T stays in registers for the whole
//    kernel (pre-multiplied by scale*log2(e), rounded to f16 as the reference's decode kernel
//    does, attn_v4.metal:20-31).  The result leaves every lane holding one query row and
//    eight consecutive keys of a 32-key step, which is exactly the B operand of the second
//    product O^T = V^T . P^T, so probabilities never move between lanes.
//  * V is read through its transposed cache layout [kv head][dim][position]: the A operand of
//    O^T wants 8 consecutive positions of one dim, 16 contiguous bytes there.
//  * online softmax in base 2 on the lanes' own values; the running maximum is shared by the
//    four lanes of a row with two cross-lane exchanges per 32 keys, the accumulator rescale is
//    skipped while no row's maximum moves.
//  * each workgroup writes (m, l, O) partials; a second small kernel merges the splits.
#include "common.h"

#include <cmath>

namespace {

typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
typedef float float4_t __attribute__((ext_vector_type(4)));

constexpr float kLog2e = 1.4426950408889634f;

// exchange with the lane 16 / 32 positions away (the other lanes that hold the same query row)
__device__ __forceinline__ float xor_lane(float v, int mask) {
    return __shfl_xor(v, mask, 64);
}

// MAXW = most waves (query heads per KV head) a workgroup may have; it sets the register budget.
template <int HD, typename TQ, int MAXW>
__global__ void __launch_bounds__(64 * MAXW)
    attn_split_kernel(const TQ *__restrict__ q, const _Float16 *__restrict__ k_cache,
                      const _Float16 *__restrict__ vt_cache, float *__restrict__ part_o, float *__restrict__ part_ml,
                      int64_t ctx_len, int n_rows, int n_q, int n_kv, int64_t vt_stride, int64_t chunk, float scale,
                      int full_block, int64_t window) {
    constexpr int KS = HD / 32;  // k-steps of the score product
    constexpr int DT = HD / 16;  // 16-dim tiles of the output
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int n = lane & 15, g = lane >> 4;
    const int group = n_q / n_kv;
    const int kvh = blockIdx.y;
    const int split = blockIdx.x;
    const int head = kvh * group + wave;
    const int64_t n_pos = ctx_len + n_rows;
    const int64_t c0 = split * chunk;
    const int64_t c1 = min(n_pos, c0 + chunk);
    const int64_t kv_dim = static_cast<int64_t>(n_kv) * HD;

    // Q^T fragments: lane (row n, g) holds Q[n][head][32 s + 8 g ..+8] * scale * log2(e)
    half8_t qf[KS];
    {
        const float mult = scale * kLog2e;
#pragma unroll
        for (int s = 0; s < KS; s++) {
#pragma unroll
            for (int i = 0; i < 8; i++) {
                float v = 0.0f;
                if (n < n_rows) v = static_cast<float>(q[(static_cast<int64_t>(n) * n_q + head) * HD + 32 * s + 8 * g + i]);
                qf[s][i] = static_cast<_Float16>(v * mult);
            }
        }
    }

    float4_t acc[DT];
#pragma unroll
    for (int t = 0; t < DT; t++) acc[t] = float4_t{0, 0, 0, 0};
    float m_run = -INFINITY;  // running maximum of row n (base-2 logits), shared by its four lanes
    float l_run = 0.0f;       // this lane's share of the row sum
    // visible keys of row n: [lo, hi].  Block-causal: everything up to the row's own position;
    // full_block (drafter, non-causal): the whole block; a sliding window keeps |distance| < window.
    const int64_t row_pos = ctx_len + n;
    int64_t row_hi = full_block ? n_pos - 1 : row_pos;
    int64_t row_lo = 0;
    if (window > 0) {
        row_lo = row_pos - window + 1;
        row_hi = min(row_hi, row_pos + window - 1);
    }

    const _Float16 *kbase = k_cache + static_cast<int64_t>(kvh) * HD + 8 * g;
    const _Float16 *vbase = vt_cache + static_cast<int64_t>(kvh) * HD * vt_stride;

    for (int64_t key0 = c0; key0 < c1; key0 += 32) {
        // scores of 32 keys: tile T holds keys key0 + 8 (m / 4) + 4 T + (m % 4) in its row m, so
        // that lane (n, g) ends up with keys key0 + 8 g .. + 7 (T = 0: first four, T = 1: last four)
        float4_t st[2];
#pragma unroll
        for (int T = 0; T < 2; T++) {
            int64_t key = key0 + 8 * (n >> 2) + 4 * T + (n & 3);
            key = key < n_pos ? key : n_pos - 1;
            const _Float16 *kp = kbase + key * kv_dim;
            float4_t s_acc = {0, 0, 0, 0};
#pragma unroll
            for (int s = 0; s < KS; s++) {
                half8_t kf = *reinterpret_cast<const half8_t *>(kp + 32 * s);
                s_acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(kf, qf[s], s_acc, 0, 0, 0);
            }
            st[T] = s_acc;
        }
        // mask: key visible to row n iff row_lo <= key <= row_hi and key < c1
        float p[8];
        float mx = -INFINITY;
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const int64_t key = key0 + 8 * g + i;
            float v = (i < 4) ? st[0][i] : st[1][i - 4];
            v = (key >= row_lo && key <= row_hi && key < c1) ? v : -INFINITY;
            p[i] = v;
            mx = fmaxf(mx, v);
        }
        mx = fmaxf(mx, xor_lane(mx, 16));
        mx = fmaxf(mx, xor_lane(mx, 32));
        const float m_new = fmaxf(m_run, mx);
        // all keys of this step masked for this row and nothing seen before: keep the state
        const float m_safe = (m_new == -INFINITY) ? 0.0f : m_new;
        const float alpha = exp2f(m_run - m_safe);  // 0 when m_run = -inf
        float psum = 0.0f;
#pragma unroll
        for (int i = 0; i < 8; i++) {
            p[i] = exp2f(p[i] - m_safe);
            psum += p[i];
        }
        l_run = l_run * alpha + psum;
        if (__builtin_amdgcn_ballot_w64(alpha != 1.0f) != 0) {
#pragma unroll
            for (int t = 0; t < DT; t++) acc[t] *= alpha;
        }
        m_run = m_new;
        half8_t pf;
#pragma unroll
        for (int i = 0; i < 8; i++) pf[i] = static_cast<_Float16>(p[i]);
        // O^T tile t (dims 16 t ..): A = V^T[dim 16 t + n][keys key0 + 8 g ..+8]
        const int64_t vkey = key0 + 8 * g;  // < vt_stride: the stride is a multiple of 32 and >= n_pos
        // positions past the end of the cache hold whatever was there before (possibly NaN bit
        // patterns), and 0 * NaN would poison the accumulator: zero them in the last step
        const bool tail = key0 + 32 > n_pos;
#pragma unroll
        for (int t = 0; t < DT; t++) {
            half8_t vf = *reinterpret_cast<const half8_t *>(vbase + static_cast<int64_t>(16 * t + n) * vt_stride + vkey);
            if (tail) {
#pragma unroll
                for (int i = 0; i < 8; i++)
                    if (vkey + i >= n_pos) vf[i] = static_cast<_Float16>(0.0f);
            }
            acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(vf, pf, acc[t], 0, 0, 0);
        }
    }

    // row sum over the four lanes of the row
    l_run += xor_lane(l_run, 16);
    l_run += xor_lane(l_run, 32);

    // partials: O^T tile t, lane (row n, g) holds dims 16 t + 4 g + i
    if (n < n_rows) {
        const int64_t slot = (static_cast<int64_t>(split) * n_q + head) * 16 + n;
        float *po = part_o + slot * HD;
#pragma unroll
        for (int t = 0; t < DT; t++) *reinterpret_cast<float4_t *>(po + 16 * t + 4 * g) = acc[t];
        if (g == 0) {
            part_ml[slot * 2] = m_run;
            part_ml[slot * 2 + 1] = l_run;
        }
    }
}

// out[row][head][:] = sum_s 2^(m_s - m*) O_s / sum_s 2^(m_s - m*) l_s
__global__ void __launch_bounds__(256)
    attn_combine_kernel(const float *__restrict__ part_o, const float *__restrict__ part_ml, float *__restrict__ out,
                        int n_rows, int n_q, int hd, int n_splits) {
    const int head = blockIdx.x, row = blockIdx.y;
    float m_star = -INFINITY;
    for (int s = 0; s < n_splits; s++) {
        const int64_t slot = (static_cast<int64_t>(s) * n_q + head) * 16 + row;
        m_star = fmaxf(m_star, part_ml[slot * 2]);
    }
    for (int d = threadIdx.x; d < hd; d += blockDim.x) {
        float o = 0.0f, l = 0.0f;
        for (int s = 0; s < n_splits; s++) {
            const int64_t slot = (static_cast<int64_t>(s) * n_q + head) * 16 + row;
            const float m = part_ml[slot * 2];
            if (m == -INFINITY) continue;
            const float wgt = exp2f(m - m_star);
            o += wgt * part_o[slot * hd + d];
            l += wgt * part_ml[slot * 2 + 1];
        }
        out[(static_cast<int64_t>(row) * n_q + head) * hd + d] = o / l;
    }
}

// V [pos][n_kv][hd] -> V^T [n_kv][hd][stride]; one workgroup per (32 positions, kv head)
__global__ void __launch_bounds__(256) transpose_v_kernel(const _Float16 *__restrict__ v, _Float16 *__restrict__ vt,
                                                          int64_t n_pos, int n_kv, int hd, int64_t stride) {
    __shared__ _Float16 tile[32][256 + 2];
    const int64_t p0 = static_cast<int64_t>(blockIdx.x) * 32;
    const int kvh = blockIdx.y;
    for (int e = threadIdx.x; e < 32 * hd; e += blockDim.x) {
        int pl = e / hd, d = e - pl * hd;
        int64_t pos = p0 + pl;
        tile[pl][d] = pos < n_pos ? v[(pos * n_kv + kvh) * hd + d] : static_cast<_Float16>(0.0f);
    }
    __syncthreads();
    for (int e = threadIdx.x; e < 32 * hd; e += blockDim.x) {
        int d = e >> 5, pl = e & 31;
        int64_t pos = p0 + pl;
        if (pos < stride) vt[(static_cast<int64_t>(kvh) * hd + d) * stride + pos] = tile[pl][d];
    }
}

template <int HD, typename TQ>
void launch_split(dim3 grid, int threads, hipStream_t st, const void *q, const _Float16 *k, const _Float16 *vt,
                  float *po, float *pml, int64_t ctx_len, int n_rows, int n_q, int n_kv, int64_t vt_stride,
                  int64_t chunk, float scale, int full_block, int64_t window) {
    if (threads <= 512)
        attn_split_kernel<HD, TQ, 8><<<grid, threads, 0, st>>>(static_cast<const TQ *>(q), k, vt, po, pml, ctx_len,
                                                               n_rows, n_q, n_kv, vt_stride, chunk, scale, full_block,
                                                               window);
    else
        attn_split_kernel<HD, TQ, 16><<<grid, threads, 0, st>>>(static_cast<const TQ *>(q), k, vt, po, pml, ctx_len,
                                                                n_rows, n_q, n_kv, vt_stride, chunk, scale, full_block,
                                                                window);
}

}  // namespace

extern "C" int32_t dflash_attn_verify_block(dflash_ctx *ctx, const void *q, int32_t q_type, const void *k_cache,
                                            const void *v_cache, int32_t v_layout, int64_t ctx_len, int32_t n_rows,
                                            int32_t n_q, int32_t n_kv, int32_t head_dim, int64_t kv_capacity,
                                            float scale, float *out, dflash_stream_t stream) {
    return dfl_attn_block(ctx, q, q_type, k_cache, v_cache, v_layout, ctx_len, n_rows, n_q, n_kv, head_dim, kv_capacity,
                          scale, out, stream, 0, 0);
}

int32_t dfl_attn_block(dflash_ctx *ctx, const void *q, int32_t q_type, const void *k_cache, const void *v_cache,
                       int32_t v_layout, int64_t ctx_len, int32_t n_rows, int32_t n_q, int32_t n_kv, int32_t head_dim,
                       int64_t kv_capacity, float scale, float *out, dflash_stream_t stream, int32_t full_block,
                       int64_t window) {
    if (!ctx) return DFLASH_ERR_INVALID_INPUT;
    if (!q || !k_cache || !v_cache || !out) return dfl_fail(ctx, DFLASH_ERR_INVALID_INPUT, "attn_verify: null pointer");
    if (n_rows < 1 || n_rows > 16) return dfl_fail(ctx, DFLASH_ERR_BAD_SHAPE, "attn_verify: n_rows %d outside 1..16", n_rows);
    if (n_q < 1 || n_kv < 1 || n_q % n_kv || n_q / n_kv > 16)
        return dfl_fail(ctx, DFLASH_ERR_BAD_SHAPE, "attn_verify: %d query heads over %d KV heads (group must be 1..16)",
                        n_q, n_kv);
    if (head_dim != 64 && head_dim != 128 && head_dim != 256)
        return dfl_fail(ctx, DFLASH_ERR_UNSUPPORTED, "attn_verify: head_dim %d (64, 128, 256 supported)", head_dim);
    if (ctx_len < 0 || ctx_len + n_rows > kv_capacity)
        return dfl_fail(ctx, DFLASH_ERR_STATE, "attn_verify: context %lld + %d rows exceeds the cache capacity %lld",
                        static_cast<long long>(ctx_len), n_rows, static_cast<long long>(kv_capacity));
    if (q_type != DFLASH_TYPE_F32 && q_type != DFLASH_TYPE_F16)
        return dfl_fail(ctx, DFLASH_ERR_UNSUPPORTED, "attn_verify: queries must be f32 or f16");
    if (v_layout != 0 && v_layout != 1) return dfl_fail(ctx, DFLASH_ERR_INVALID_INPUT, "attn_verify: v_layout");
    if (v_layout == 1 && kv_capacity % 32)
        return dfl_fail(ctx, DFLASH_ERR_ALIGNMENT, "attn_verify: transposed V needs a capacity that is a multiple of 32");
    if (reinterpret_cast<uintptr_t>(k_cache) % 16 || reinterpret_cast<uintptr_t>(v_cache) % 16 ||
        reinterpret_cast<uintptr_t>(out) % 16)
        return dfl_fail(ctx, DFLASH_ERR_ALIGNMENT, "attn_verify: K, V and the output must be 16-byte aligned");

    hipStream_t st = static_cast<hipStream_t>(stream);
    const int group = n_q / n_kv;
    const int64_t n_pos = ctx_len + n_rows;

    // KV splits: enough workgroups to cover the chip about twice, chunks a multiple of 32 keys
    // and at least 128 keys long (a split costs a partial tile per head and row)
    int64_t want = (2 * ctx->n_cu + n_kv - 1) / n_kv;
    int64_t chunk = (n_pos + want - 1) / want;
    chunk = (chunk + 31) / 32 * 32;
    if (chunk < 128) chunk = 128;
    const int n_splits = static_cast<int>((n_pos + chunk - 1) / chunk);

    size_t off = 0;
    float *part_o = dfl_ws_take<float>(ctx, &off, static_cast<size_t>(n_splits) * n_q * 16 * head_dim * sizeof(float));
    float *part_ml = dfl_ws_take<float>(ctx, &off, static_cast<size_t>(n_splits) * n_q * 16 * 2 * sizeof(float));
    const _Float16 *vt = static_cast<const _Float16 *>(v_cache);
    int64_t vt_stride = kv_capacity;
    if (v_layout == 0) {
        vt_stride = (n_pos + 31) / 32 * 32;
        _Float16 *vt_ws = dfl_ws_take<_Float16>(ctx, &off, static_cast<size_t>(n_kv) * head_dim * vt_stride * 2);
        if (!vt_ws)
            return dfl_fail(ctx, DFLASH_ERR_WORKSPACE,
                            "attn_verify: transposing V needs %zu workspace bytes; pass the transposed cache instead",
                            static_cast<size_t>(n_kv) * head_dim * vt_stride * 2);
        transpose_v_kernel<<<dim3(static_cast<unsigned>(vt_stride / 32), n_kv), 256, 0, st>>>(
            static_cast<const _Float16 *>(v_cache), vt_ws, n_pos, n_kv, head_dim, vt_stride);
        vt = vt_ws;
    }
    if (!part_o || !part_ml) return dfl_fail(ctx, DFLASH_ERR_WORKSPACE, "attn_verify: workspace too small");

    const dim3 grid(n_splits, n_kv);
    const int threads = 64 * group;
    const _Float16 *k = static_cast<const _Float16 *>(k_cache);
    {
        dfl_timed timer(ctx, st, DFL_T_ATTN);
#define DFL_ATTN(HD)                                                                                              \
    if (q_type == DFLASH_TYPE_F32)                                                                                \
        launch_split<HD, float>(grid, threads, st, q, k, vt, part_o, part_ml, ctx_len, n_rows, n_q, n_kv, vt_stride, \
                                chunk, scale, full_block, window);                                                \
    else                                                                                                          \
        launch_split<HD, _Float16>(grid, threads, st, q, k, vt, part_o, part_ml, ctx_len, n_rows, n_q, n_kv,      \
                                   vt_stride, chunk, scale, full_block, window)
        if (head_dim == 64) {
            DFL_ATTN(64);
        } else if (head_dim == 128) {
            DFL_ATTN(128);
        } else {
            DFL_ATTN(256);
        }
#undef DFL_ATTN
    }
    attn_combine_kernel<<<dim3(n_q, n_rows), head_dim < 256 ? head_dim : 256, 0, st>>>(part_o, part_ml, out, n_rows, n_q,
                                                                                   head_dim, n_splits);
    DFL_HIP_CHECK(ctx, hipGetLastError());
    return DFLASH_OK;
}
