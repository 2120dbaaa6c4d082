// Target packed verify, KV rollback and the block drafter, built from the few-row GEMM, the
// block-causal attention and small glue kernels.
//
// Reference: encode_packed_verify_layer_major_inner_for (metal_dflash.rs:9045-10690),
// encode_restore_after_partial_accept_inner (:15649-15777), draft_block_inner (:15952-17164),
// append_target_ctx_columns_now (:5798-5860); CPU forms forward.rs:96-163, 380-662, 725-932,
// 1256-1371.  Glue: kernels/attn.metal:35-69 (RMSNorm), :137-196 (q/k norm + RoPE),
// kernels/rope.metal:96-121, kernels/elementwise.metal:89, 193, 674-685, 727-900.
#include "common.h"
#include "device_quant.h"

#include <algorithm>
#include <array>
#include <map>
#include <mutex>
#include <chrono>
#include <cmath>
#include <cstring>
#include <new>
#include <vector>

namespace {

// kernel_get_rows_{f32,q4_K,q6_K,q8_0} (elementwise.metal:727-900): out[r][:] = deq(table[ids[r]])
__global__ void get_rows_kernel(int type, const uint8_t *__restrict__ table, size_t row_bytes,
                                const int32_t *__restrict__ ids, int hidden, float *__restrict__ out) {
    const int r = blockIdx.y;
    const int e = blockIdx.x * blockDim.x + threadIdx.x;
    if (e >= hidden) return;
    out[static_cast<size_t>(r) * hidden + e] = dfl_dequant_elem(type, table + static_cast<size_t>(ids[r]) * row_bytes, e);
}

__device__ float block_sum(float v, float *sh) {
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
    __syncthreads();
    if ((threadIdx.x & 63) == 0) sh[threadIdx.x >> 6] = v;
    __syncthreads();
    float r = 0.0f;
    for (int w = 0; w < static_cast<int>(blockDim.x >> 6); w++) r += sh[w];
    return r;
}

// kernel_rms_norm_batched_f32 (attn.metal:35-69), optionally preceded by the residual add that
// feeds it (kernel_add, elementwise.metal): x += add (add may be null), then
// y = x * rsqrt(mean(x^2) + eps) * w.  One row per workgroup; a row of up to 8192 values (n a
// multiple of 4) is read once and stays in registers between the two passes.  With gate_w, the row's
// sigmoid(y . gate_w) also goes to gate_out[row] (the shared-expert gate of a mixture-of-experts
// layer, forward.rs:749-824: the normalised row is at hand here, in registers).  With y_xf (n a multiple of 256, at most
// 8192: every width the whole-K GEMMs take), y also goes there as f16 in the fragment order a whole-K GEMM reads (common.h, "XF").
// With conv.dyn (a DFlash-2 drafter's residual adds, metal_dflash.rs:16795-16820, 17003-17022; rows of one block
// only): what is added to row t is not add[t] but the side-1 dynamic convolution of the rows of add,
//   sum_tap (base[1][tap][c] + dyn[t][1][tap][c / group_size]) * add[t - tap][c]   (rows before the block read as zeros),
// taps accumulated in order with a fused multiply-add - the arithmetic of dflash2_conv_kernel, which a launch of its
// own ran before.
struct ConvResid {
    const float *dyn = nullptr;   // [rows][2][kernel][n / group_size]
    const float *base = nullptr;  // [2][kernel][n]
    int kernel_size = 0, group_size = 1;
};
__global__ void __launch_bounds__(256) rms_norm_kernel(float *__restrict__ x, const float *__restrict__ add,
                                                       const float *__restrict__ w, float *__restrict__ y, int n,
                                                       float eps, const float *__restrict__ gate_w,
                                                       float *__restrict__ gate_out, void *__restrict__ y_xf = nullptr,
                                                       int y_xf_kind = 0, size_t xf_stride = 0, ConvResid conv = ConvResid()) {
    typedef float f4 __attribute__((ext_vector_type(4)));
    __shared__ float sh[4];
    float *xr = x + static_cast<size_t>(blockIdx.x) * n;
    const float *ar = add ? add + static_cast<size_t>(blockIdx.x) * n : nullptr;
    float *yr = y + static_cast<size_t>(blockIdx.x) * n;
    const int tid = threadIdx.x;
    if (conv.dyn && ar && n <= 8192 && n % 4 == 0) {
        // (the same two passes as below; the residual term is the convolution)
        constexpr int kVec = 8;
        const int t = blockIdx.x, ks = conv.kernel_size, n_groups = n / conv.group_size;
        const float *dyn_t = conv.dyn + (static_cast<size_t>(t) * 2 + 1) * ks * n_groups;
        const float *base1 = conv.base + static_cast<size_t>(ks) * n;
        f4 v[kVec];
        float s = 0.0f;
#pragma unroll
        for (int j = 0; j < kVec; j++) {
            const int i = 4 * (tid + 256 * j);
            v[j] = f4{0, 0, 0, 0};
            if (i < n) {
                f4 acc = {0, 0, 0, 0};
                // (the four channels' groups, once per vector: one division when the group size is a multiple of four)
                int grp[4];
                grp[0] = i / conv.group_size;
                if (conv.group_size % 4 == 0) {
                    grp[1] = grp[2] = grp[3] = grp[0];
                } else {
#pragma unroll
                    for (int e = 1; e < 4; e++) grp[e] = (i + e) / conv.group_size;
                }
                for (int tap = 0; tap < ks && tap <= t; tap++) {
                    const f4 b = *reinterpret_cast<const f4 *>(base1 + static_cast<size_t>(tap) * n + i);
                    const f4 src = *reinterpret_cast<const f4 *>(add + static_cast<size_t>(t - tap) * n + i);
                    const float *dg = dyn_t + static_cast<size_t>(tap) * n_groups;
#pragma unroll
                    for (int e = 0; e < 4; e++) acc[e] = __builtin_fmaf(b[e] + dg[grp[e]], src[e], acc[e]);
                }
                v[j] = *reinterpret_cast<const f4 *>(xr + i) + acc;
                *reinterpret_cast<f4 *>(xr + i) = v[j];
            }
            s += (v[j][0] * v[j][0] + v[j][1] * v[j][1]) + (v[j][2] * v[j][2] + v[j][3] * v[j][3]);
        }
        s = block_sum(s, sh);
        const float scale = 1.0f / sqrtf(s / static_cast<float>(n) + eps);
#pragma unroll
        for (int j = 0; j < kVec; j++) {
            const int i = 4 * (tid + 256 * j);
            if (i < n) {
                const f4 o = v[j] * scale * *reinterpret_cast<const f4 *>(w + i);
                *reinterpret_cast<f4 *>(yr + i) = o;
                if (y_xf)
                    dfl_xf_store_pair(static_cast<uint8_t *>(y_xf) + (blockIdx.x >> 4) * xf_stride, y_xf_kind, blockIdx.x & 15, i & ~7, o[0],
                                      o[1], o[2], o[3]);
            }
        }
        return;
    }
    if (n <= 8192 && n % 4 == 0) {
        // (vectors past the row are zeros and add nothing: a row of up to 4096 values sums exactly as with four vectors)
        constexpr int kVec = 8;
        f4 v[kVec], wv[kVec];
        float s = 0.0f;
#pragma unroll
        for (int j = 0; j < kVec; j++) {
            const int i = 4 * (tid + 256 * j);
            v[j] = f4{0, 0, 0, 0};
            if (i < n) {
                v[j] = *reinterpret_cast<const f4 *>(xr + i);
                if (ar) v[j] += *reinterpret_cast<const f4 *>(ar + i);
            }
        }
        // (the weights are asked for ahead of the sum's barrier, but behind the row: vector loads return in the order of
        // their issue, and the row is what the sum waits for)
#pragma unroll
        for (int j = 0; j < kVec; j++) {
            const int i = 4 * (tid + 256 * j);
            wv[j] = i < n ? *reinterpret_cast<const f4 *>(w + i) : f4{0, 0, 0, 0};
        }
#pragma unroll
        for (int j = 0; j < kVec; j++) {
            const int i = 4 * (tid + 256 * j);
            if (i < n && ar) *reinterpret_cast<f4 *>(xr + i) = v[j];
            s += (v[j][0] * v[j][0] + v[j][1] * v[j][1]) + (v[j][2] * v[j][2] + v[j][3] * v[j][3]);
        }
        s = block_sum(s, sh);
        const float scale = 1.0f / sqrtf(s / static_cast<float>(n) + eps);
        float dot = 0.0f;
#pragma unroll
        for (int j = 0; j < kVec; j++) {
            const int i = 4 * (tid + 256 * j);
            if (i < n) {
                const f4 o = v[j] * scale * wv[j];
                *reinterpret_cast<f4 *>(yr + i) = o;
                // (the host passes y_xf only for n a multiple of 256: whole waves are inside or outside the row)
                // (more than sixteen rows: block b of sixteen at y_xf + b * xf_stride bytes)
                if (y_xf)
                    dfl_xf_store_pair(static_cast<uint8_t *>(y_xf) + (blockIdx.x >> 4) * xf_stride, y_xf_kind, blockIdx.x & 15, i & ~7, o[0],
                                      o[1], o[2], o[3]);
                if (gate_w) {
                    const f4 gw = *reinterpret_cast<const f4 *>(gate_w + i);
                    dot += (o[0] * gw[0] + o[1] * gw[1]) + (o[2] * gw[2] + o[3] * gw[3]);
                }
            }
        }
        if (gate_w) {
            dot = block_sum(dot, sh);
            if (tid == 0) gate_out[blockIdx.x] = 1.0f / (1.0f + expf(-dot));
        }
        return;
    }
    float s = 0.0f;
    for (int i = tid; i < n; i += 256) {
        float v = xr[i];
        if (ar) {
            v += ar[i];
            xr[i] = v;
        }
        s += v * v;
    }
    s = block_sum(s, sh);
    const float scale = 1.0f / sqrtf(s / static_cast<float>(n) + eps);
    float dot = 0.0f;
    for (int i = tid; i < n; i += 256) {
        const float o = xr[i] * scale * w[i];
        yr[i] = o;
        if (gate_w) dot += o * gate_w[i];
    }
    if (gate_w) {
        dot = block_sum(dot, sh);
        if (tid == 0) gate_out[blockIdx.x] = 1.0f / (1.0f + expf(-dot));
    }
}

// kernel_qk_rms_norm_rope_f32_packed_consecutive (attn.metal:137-196) + the f32 -> f16 KV scatter
// (elementwise.metal:674-685).  One wave per (row, head): per-head RMSNorm (weight may be null),
// NeoX RoPE over the full head (pairs (i, i + hd/2), angle = pos / theta^(2i/hd)).
// Heads [0, n_q) are queries (rewritten in place, f32); heads [n_q, n_q+n_kv) are keys, written
// as f16 into k_dst[pos][kv head][:] (k_dst == null: rewritten in place as f32 instead).
// With vt_dst, n_kv more workgroups per row scatter the row's V heads, as f16, into column
// pos[row] of the transposed cache [kv head][dim][capacity].
__global__ void __launch_bounds__(64)
    qk_norm_rope_kernel(const float *q_in, int64_t q_ld, const float *k_in, int64_t k_ld, float *q_out, float *k_out,
                        const float *__restrict__ q_w, const float *__restrict__ k_w, _Float16 *__restrict__ k_dst,
                        const int32_t *__restrict__ pos, int n_q, int n_kv, int hd, float eps, float theta,
                        const float *__restrict__ v_src, int64_t v_ld, _Float16 *__restrict__ vt_dst, int64_t capacity) {
    const int row = blockIdx.y, head = blockIdx.x, lane = threadIdx.x;
    if (head >= n_q + n_kv) {
        const int vh = head - n_q - n_kv;
        const float *src = v_src + static_cast<size_t>(row) * v_ld + static_cast<size_t>(vh) * hd;
        _Float16 *dst = vt_dst + static_cast<size_t>(vh) * hd * capacity + pos[row];
        for (int i = lane; i < hd; i += 64) dst[static_cast<size_t>(i) * capacity] = static_cast<_Float16>(src[i]);
        return;
    }
    const bool is_q = head < n_q;
    // input rows may be slices of a wider matrix (row strides q_ld, k_ld); outputs are dense.  In
    // place (q_out == q_in with a dense q_ld) is fine: a lane reads its two elements before it
    // writes them.
    const float *v = is_q ? q_in + static_cast<size_t>(row) * q_ld + static_cast<size_t>(head) * hd
                          : k_in + static_cast<size_t>(row) * k_ld + static_cast<size_t>(head - n_q) * hd;
    float *o = is_q ? q_out + (static_cast<size_t>(row) * n_q + head) * hd
                    : (k_dst ? nullptr : k_out + (static_cast<size_t>(row) * n_kv + (head - n_q)) * hd);
    const float *w = is_q ? q_w : k_w;
    const int half = hd / 2;
    // heads of 128 or 256: a lane's two or four elements stay in registers between the two passes (element lane + 64 k
    // in r[k]; the partner of element i is i + half = r[k + half / 64]); same sums in the same order as the loops.
    // The norm's weights and the position are asked for right behind them (vector loads return in the order of their
    // issue: the elements, which the sum waits for, first), not after the sum: one trip to memory instead of two.
    const bool in_regs = hd == 256 || hd == 128;
    float r[4] = {0.0f, 0.0f, 0.0f, 0.0f}, wr[4] = {1.0f, 1.0f, 1.0f, 1.0f};
    float s = 0.0f;
    if (in_regs) {
#pragma unroll
        for (int k = 0; k < 4; k++)
            if (lane + 64 * k < hd) r[k] = v[lane + 64 * k];
        if (w) {
#pragma unroll
            for (int k = 0; k < 4; k++)
                if (lane + 64 * k < hd) wr[k] = w[lane + 64 * k];
        }
    }
    const int32_t pos_row = pos[row];
    if (in_regs) {
#pragma unroll
        for (int k = 0; k < 4; k++)
            if (lane + 64 * k < hd) s += r[k] * r[k];
    } else {
        for (int i = lane; i < hd; i += 64) s += v[i] * v[i];
    }
    for (int off = 32; off > 0; off >>= 1) s += __shfl_xor(s, off, 64);
    const float scale = 1.0f / sqrtf(s / static_cast<float>(hd) + eps);
    const float p = static_cast<float>(pos_row);
    for (int i = lane, k = 0; i < half; i += 64, k++) {
        float a, b;
        if (in_regs) {
            a = (k == 0 ? r[0] : r[1]) * scale;
            b = (hd == 256 ? (k == 0 ? r[2] : r[3]) : r[1]) * scale;
            if (w) {
                a *= k == 0 ? wr[0] : wr[1];
                b *= hd == 256 ? (k == 0 ? wr[2] : wr[3]) : wr[1];
            }
        } else {
            a = v[i] * scale;
            b = v[i + half] * scale;
            if (w) {
                a *= w[i];
                b *= w[i + half];
            }
        }
        const float freq = p / powf(theta, static_cast<float>(2 * i) / static_cast<float>(hd));
        float sn, cs;
        sincosf(freq, &sn, &cs);
        const float ra = a * cs - b * sn, rb = a * sn + b * cs;
        if (o) {
            o[i] = ra;
            o[i + half] = rb;
        } else {
            _Float16 *dst = k_dst + (static_cast<size_t>(pos_row) * n_kv + (head - n_q)) * hd;
            dst[i] = static_cast<_Float16>(ra);
            dst[i + half] = static_cast<_Float16>(rb);
        }
    }
}

// kernel_silu_mul_f32 (elementwise.metal:193): g = silu(g) * u
__global__ void silu_mul_kernel(float *__restrict__ g, const float *__restrict__ u, size_t n) {
    size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i < n) {
        float x = g[i];
        g[i] = x / (1.0f + expf(-x)) * u[i];
    }
}

// The same over two column slices of one wider matrix (gate and up projected in one GEMM):
// out[row][i] = silu(g[row * ld + i]) * u[row * ld + i], out dense [rows][n].
__global__ void silu_mul_ld_kernel(const float *__restrict__ g, const float *__restrict__ u, int64_t ld,
                                   float *__restrict__ out, int n) {
    const int row = blockIdx.y;
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) {
        const float x = g[static_cast<size_t>(row) * ld + i];
        out[static_cast<size_t>(row) * n + i] = x / (1.0f + expf(-x)) * u[static_cast<size_t>(row) * ld + i];
    }
}

// Up to sixteen host integers reach the device as a kernel argument (by value, in the dispatch
// packet) instead of through a pageable host-to-device copy, which costs tens of microseconds of
// idle GPU at every phase boundary of a speculative step.  ids may be null (positions only).
struct Int16Args {
    int32_t v[16];
};
// dev_ids (may be null): where ids.v[i] is negative, the id comes from dev_ids[i] instead, clamped
// into [0, vocab) (the host checks the copied-back values and reports an invalid token; the clamp only
// keeps the embedding gather inside its table meanwhile).
__global__ void set_ids_pos_kernel(Int16Args ids, Int16Args pos, int n, int32_t *__restrict__ ids_dst,
                                   int32_t *__restrict__ pos_dst, const int32_t *__restrict__ dev_ids, int vocab) {
    const int i = threadIdx.x;
    if (i < n) {
        if (ids_dst) {
            int32_t id = ids.v[i];
            if (dev_ids && id < 0) {
                id = dev_ids[i];
                if (id < 0 || id >= vocab) id = 0;
            }
            ids_dst[i] = id;
        }
        pos_dst[i] = pos.v[i];
    }
}

// The same for the rows of a prefill group: up to 512 token ids by value, positions start, start + 1, ...
constexpr int kMaxGroupRows = 512;
struct IntGroupArgs {
    int32_t v[kMaxGroupRows];
};
__global__ void set_group_ids_pos_kernel(IntGroupArgs ids, int start, int n, int32_t *__restrict__ ids_dst, int32_t *__restrict__ pos_dst) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) {
        ids_dst[i] = ids.v[i];
        pos_dst[i] = start + i;
    }
}

// kernel_add_inplace_f32 (elementwise.metal:89)
__global__ void add_kernel(float *__restrict__ x, const float *__restrict__ y, size_t n) {
    size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i < n) x[i] += y[i];
}

// hidden capture: dst[(row * n_taps + tap) * hidden + :] = x[row][:]
__global__ void capture_kernel(const float *__restrict__ x, float *__restrict__ dst, int hidden, int n_taps, int tap) {
    const int row = blockIdx.y;
    const int e = blockIdx.x * blockDim.x + threadIdx.x;
    if (e < hidden) dst[(static_cast<size_t>(row) * n_taps + tap) * hidden + e] = x[static_cast<size_t>(row) * hidden + e];
}

// Drafter attention (kernels/dflash_attn.metal:99-307; CPU forward.rs:559-606): query row i of the
// noise block over ctx || noise keys, f32, mask = (!causal || k_pos <= q_pos) &&
// (window == 0 || |q_pos - k_pos| < window).  One wave per (q head, row), online softmax.
__global__ void __launch_bounds__(64)
    draft_attn_kernel(const float *__restrict__ q, const float *__restrict__ k_ctx, const float *__restrict__ v_ctx,
                      const float *__restrict__ k_noise, const float *__restrict__ v_noise,
                      const int32_t *__restrict__ pos_ctx, int ctx_len, int n, int n_q, int n_kv, int hd,
                      int noise_start, int causal, int window, float *__restrict__ out) {
    const int head = blockIdx.x, row = blockIdx.y, lane = threadIdx.x;
    const int kvh = head / (n_q / n_kv);
    const int kv_dim = n_kv * hd;
    const int per = hd / 64;  // dims per lane (hd in {64,128,256})
    float qv[4], acc[4] = {0, 0, 0, 0};
    const float scale = 1.0f / sqrtf(static_cast<float>(hd));
    for (int i = 0; i < per; i++) qv[i] = q[(static_cast<size_t>(row) * n_q + head) * hd + lane * per + i];
    const int q_pos = noise_start + row;
    float m = -INFINITY, l = 0.0f;
    for (int kk = 0; kk < ctx_len + n; kk++) {
        const int k_pos = kk < ctx_len ? pos_ctx[kk] : noise_start + (kk - ctx_len);
        const int dist = q_pos > k_pos ? q_pos - k_pos : k_pos - q_pos;
        if ((causal && k_pos > q_pos) || (window != 0 && dist >= window)) continue;
        const float *kr = (kk < ctx_len ? k_ctx + static_cast<size_t>(kk) * kv_dim
                                        : k_noise + static_cast<size_t>(kk - ctx_len) * kv_dim) + kvh * hd + lane * per;
        const float *vr = (kk < ctx_len ? v_ctx + static_cast<size_t>(kk) * kv_dim
                                        : v_noise + static_cast<size_t>(kk - ctx_len) * kv_dim) + kvh * hd + lane * per;
        float s = 0.0f;
        for (int i = 0; i < per; i++) s += qv[i] * kr[i];
        for (int off = 32; off > 0; off >>= 1) s += __shfl_xor(s, off, 64);
        s *= scale;
        const float m_new = fmaxf(m, s);
        const float alpha = expf(m - m_new), p = expf(s - m_new);
        l = l * alpha + p;
        for (int i = 0; i < per; i++) acc[i] = acc[i] * alpha + p * vr[i];
        m = m_new;
    }
    for (int i = 0; i < per; i++) out[(static_cast<size_t>(row) * n_q + head) * hd + lane * per + i] = acc[i] / l;
}

// K/V rows f32 [m][kv_dim] -> f16 caches: K natural at row base + r, V transposed at column base + r
__global__ void kv_to_f16_kernel(const float *__restrict__ k, const float *__restrict__ v, int64_t v_ld,
                                 _Float16 *__restrict__ k16, _Float16 *__restrict__ vt16, int kv_dim, int64_t cap16,
                                 int64_t base, float *__restrict__ v_copy) {
    const int row = blockIdx.y;
    const int e = blockIdx.x * blockDim.x + threadIdx.x;
    if (e >= kv_dim) return;
    const float vv = v[static_cast<size_t>(row) * v_ld + e];
    k16[(base + row) * kv_dim + e] = static_cast<_Float16>(k[static_cast<size_t>(row) * kv_dim + e]);
    vt16[static_cast<size_t>(e) * cap16 + base + row] = static_cast<_Float16>(vv);
    if (v_copy) v_copy[static_cast<size_t>(row) * kv_dim + e] = vv;  // dense f32 copy of a V slice
}

// The drafter's context K/V of up to 16 new columns, every layer in one launch, out of the batched projection
// pk[layer][col][k heads | v heads]: what qk_norm_rope_kernel (key heads, same arithmetic) and kv_to_f16_kernel do
// per layer.  blockIdx = (head: keys then values, column, layer); one wave per head.
struct CtxKvNorms {
    const float *k_norm[16];  // per layer (may be null)
};
__global__ void __launch_bounds__(64)
    ctx_kv_finish_kernel(const float *__restrict__ pk, int kv_dim, CtxKvNorms norms, float *__restrict__ k_ctx,
                         float *__restrict__ v_ctx, size_t ctx_layer_stride, _Float16 *__restrict__ k16, _Float16 *__restrict__ vt16,
                         size_t f16_layer_stride, int64_t cap16, const int32_t *__restrict__ pos, int64_t c0, int n_kv, int hd,
                         float eps, float theta) {
    const int head = blockIdx.x, col = blockIdx.y, il = blockIdx.z, lane = threadIdx.x;
    const float *row = pk + (static_cast<size_t>(il) * 16 + col) * 2 * kv_dim;
    float *kc = k_ctx + il * ctx_layer_stride + (c0 + col) * kv_dim;
    float *vc = v_ctx + il * ctx_layer_stride + (c0 + col) * kv_dim;
    _Float16 *k16l = k16 + il * f16_layer_stride, *vt16l = vt16 + il * f16_layer_stride;
    if (head >= n_kv) {  // a value head: f32 copy, and the f16 mirror's transposed column
        const int vh = head - n_kv;
        for (int i = lane; i < hd; i += 64) {
            const int e = vh * hd + i;
            const float vv = row[kv_dim + e];
            vc[e] = vv;
            vt16l[static_cast<size_t>(e) * cap16 + c0 + col] = static_cast<_Float16>(vv);
        }
        return;
    }
    const float *v = row + static_cast<size_t>(head) * hd;
    const float *w = norms.k_norm[il];
    const int half = hd / 2;
    float s = 0.0f;
    for (int i = lane; i < hd; i += 64) s += v[i] * v[i];
    for (int off = 32; off > 0; off >>= 1) s += __shfl_xor(s, off, 64);
    const float scale = 1.0f / sqrtf(s / static_cast<float>(hd) + eps);
    const float p = static_cast<float>(pos[col]);
    for (int i = lane; i < half; i += 64) {
        float a = v[i] * scale, b = v[i + half] * scale;
        if (w) {
            a *= w[i];
            b *= w[i + half];
        }
        const float freq = p / powf(theta, static_cast<float>(2 * i) / static_cast<float>(hd));
        float sn, cs;
        sincosf(freq, &sn, &cs);
        const float ra = a * cs - b * sn, rb = a * sn + b * cs;
        const int e = head * hd + i;
        kc[e] = ra;
        kc[e + half] = rb;
        k16l[(c0 + col) * kv_dim + e] = static_cast<_Float16>(ra);
        k16l[(c0 + col) * kv_dim + e + half] = static_cast<_Float16>(rb);
    }
}

// The few words a speculative step hands back to the host (the verify's argmax and top-2 gaps, the drafter's
// tokens), written by one small kernel straight into the context's pinned page: [16] argmax, [16] drafts, [16] gaps.
__global__ void step_readback_kernel(const int32_t *__restrict__ argmax, const float *__restrict__ gap,
                                     const int32_t *__restrict__ draft, int n, int32_t *__restrict__ out) {
    const int i = threadIdx.x;
    if (i < n) {
        out[i] = argmax[i];
        out[16 + i] = draft[i];
        out[32 + i] = __float_as_int(gap[i]);
    }
}

template <typename T>
bool dev_alloc(T **p, size_t count) {
    return hipMalloc(reinterpret_cast<void **>(p), count * sizeof(T) + 256) == hipSuccess;
}

inline unsigned blocks_for(size_t n, int threads = 256) { return static_cast<unsigned>((n + threads - 1) / threads); }

int32_t gemm(dflash_ctx *ctx, const dflash_qtensor &w, const float *x, float *y, int64_t n_in, int64_t n_out, int n,
             hipStream_t st) {
    return dfl_gemm_fewrow_checked(ctx, w.type, w.data, x, DFLASH_TYPE_F32, y, n_in, n_out, n, st);
}

// True if b's rows follow a's rows_a rows directly in memory and both have the same type: the two
// are then one matrix of more rows, and one GEMM serves both (its output rows hold a's columns, then
// b's).  Loaders that place a layer's wq, wk, wv (and gate, up) back to back get this for free.
bool adjacent(const dflash_qtensor &a, int64_t rows_a, const dflash_qtensor &b, int64_t n_in) {
    const size_t rb = dflash_row_bytes(a.type, n_in);
    return a.type == b.type && rb != 0 &&
           static_cast<const uint8_t *>(b.data) == static_cast<const uint8_t *>(a.data) + static_cast<size_t>(rows_a) * rb;
}

// The fast kernels take a Q4_K / Q6_K tensor only if it was range-checked (dflash_check_scale_range); the model-level
// calls use nothing else, so they decline a model that holds an untagged one.  (The tiled order is checked when it is made.)
bool tensor_checked(const dflash_qtensor &t) {
    return !t.data || (t.type != DFLASH_TYPE_Q4_K && t.type != DFLASH_TYPE_Q6_K) || (t.flags & DFLASH_QT_RANGE_CHECKED);
}
int32_t unchecked(dflash_ctx *ctx, const char *what, int layer) {
    return dfl_fail(ctx, DFLASH_ERR_UNSUPPORTED,
                    "%s (layer %d) is a Q4_K / Q6_K tensor without DFLASH_QT_RANGE_CHECKED: run dflash_check_scale_range on it when it is uploaded",
                    what, layer);
}
int32_t model_tensors_checked(dflash_ctx *ctx, const dflash_model *m) {
    if (!tensor_checked(m->token_embd)) return unchecked(ctx, "token_embd", -1);
    if (!tensor_checked(m->output)) return unchecked(ctx, "output", -1);
    for (int il = 0; il < m->cfg.n_layers; il++) {
        const dflash_layer &L = m->layers[il];
        const dflash_qtensor *ts[] = {&L.wq, &L.wk, &L.wv, &L.wo, &L.gate, &L.up, &L.down, &L.router, &L.gate_exps, &L.up_exps, &L.down_exps};
        const char *names[] = {"wq", "wk", "wv", "wo", "gate", "up", "down", "router", "gate_exps", "up_exps", "down_exps"};
        for (int i = 0; i < 11; i++)
            if (!tensor_checked(*ts[i])) return unchecked(ctx, names[i], il);
    }
    return DFLASH_OK;
}
int32_t head_tensors_checked(dflash_ctx *ctx, const dflash_draft_head *h) {
    if (!tensor_checked(h->fc)) return unchecked(ctx, "fc", -1);
    if (!tensor_checked(h->selector_hidden)) return unchecked(ctx, "selector_hidden", -1);
    for (int il = 0; il < h->cfg.n_layers; il++) {
        const dflash_draft_layer &L = h->layers[il];
        const dflash_qtensor *ts[] = {&L.wq, &L.wk, &L.wv, &L.wo, &L.gate, &L.up, &L.down, &L.conv_attn_proj, &L.conv_ffn_proj};
        const char *names[] = {"wq", "wk", "wv", "wo", "gate", "up", "down", "conv_attn_proj", "conv_ffn_proj"};
        for (int i = 0; i < 9; i++)
            if (!tensor_checked(*ts[i])) return unchecked(ctx, names[i], il);
    }
    return DFLASH_OK;
}

// Which of a layer's projections take the whole-K kernel over activations in fragment order (gemm_whole.hip), and the
// XF kind each of them reads; DFL_XF_NONE: the projection stays with the streaming kernels and row-major activations.
// The kernel that PRODUCES a projection's input rows is told to write them in that order as well.
struct LayerXf {
    int qkv = DFL_XF_NONE, wo = DFL_XF_NONE, gate_up = DFL_XF_NONE, down = DFL_XF_NONE;
};
template <typename LayerT>
LayerXf layer_xf(const dflash_ctx *ctx, const LayerT &L, bool packed_qkv_allowed, int64_t H, int64_t q_dim, int64_t kv_dim,
                 int64_t ffn, bool dense_ffn) {
    LayerXf k;
    if (packed_qkv_allowed && adjacent(L.wq, q_dim, L.wk, H) && adjacent(L.wk, kv_dim, L.wv, H))
        k.qkv = dfl_whole_kind(ctx, L.wq.type, H, q_dim + 2 * kv_dim, 0);
    k.wo = dfl_whole_kind(ctx, L.wo.type, q_dim, H, 0);
    if (dense_ffn && ffn > 0) {
        if (adjacent(L.gate, ffn, L.up, H)) k.gate_up = dfl_whole_kind(ctx, L.gate.type, H, 2 * ffn, ffn);
        k.down = dfl_whole_kind(ctx, L.down.type, ffn, H, 0);
    }
    return k;
}

// The q, k and v projections of a layer.  Returns in *packed whether they went out as one GEMM into
// pk[n][q_dim + 2 kv_dim] (adjacent weights) or as separate ones into q, k, v.  xf_kind != DFL_XF_NONE (from
// layer_xf: implies adjacent weights): the rows are in x_xf in fragment order and the whole-K kernel takes them.
int32_t gemm_qkv(dflash_ctx *ctx, const dflash_qtensor &wq, const dflash_qtensor &wk, const dflash_qtensor &wv, const float *x,
                 float *q, float *k, float *v, float *pk, bool allow_packed, bool *packed, int64_t n_in, int64_t q_dim,
                 int64_t kv_dim, int n, hipStream_t st, const void *x_xf = nullptr, int xf_kind = DFL_XF_NONE) {
    *packed = allow_packed && pk && adjacent(wq, q_dim, wk, n_in) && adjacent(wk, kv_dim, wv, n_in);
    if (*packed && xf_kind != DFL_XF_NONE && x_xf)
        return dfl_gemm_whole(ctx, wq.type, wq.data, x_xf, pk, n_in, q_dim + 2 * kv_dim, n, 0, nullptr, DFL_XF_NONE, st);
    if (*packed) return gemm(ctx, wq, x, pk, n_in, q_dim + 2 * kv_dim, n, st);
    if (wq.type == DFLASH_TYPE_Q6_K && wk.type == DFLASH_TYPE_Q6_K && wv.type == DFLASH_TYPE_Q6_K && n_in % DFL_QK_K == 0) {
        const void *w[3] = {wq.data, wk.data, wv.data};
        float *y[3] = {q, k, v};
        const int64_t n_out[3] = {q_dim, kv_dim, kv_dim};
        return dfl_gemm_q6k_set(ctx, 3, w, y, n_out, x, DFLASH_TYPE_F32, n_in, n, st);
    }
    int32_t rc;
    if ((rc = gemm(ctx, wq, x, q, n_in, q_dim, n, st))) return rc;
    if ((rc = gemm(ctx, wk, x, k, n_in, kv_dim, n, st))) return rc;
    return gemm(ctx, wv, x, v, n_in, kv_dim, n, st);
}

// Dense SwiGLU input: g = silu(x Wg^T) * (x Wu^T), one GEMM when gate and up are adjacent.  xf_kind != DFL_XF_NONE
// (from layer_xf): the rows are in x_xf in fragment order and the whole-K kernel computes the pair with the
// activation in its epilogue; g_xf / g_xf_kind: the result also goes there in the order the down projection reads.
int32_t gemm_gate_up(dflash_ctx *ctx, const dflash_qtensor &gate, const dflash_qtensor &up, const float *x, float *g, float *u,
                     float *pk, int64_t n_in, int64_t ffn, int n, hipStream_t st, const void *x_xf = nullptr,
                     int xf_kind = DFL_XF_NONE, void *g_xf = nullptr, int g_xf_kind = DFL_XF_NONE) {
    int32_t rc;
    if (xf_kind != DFL_XF_NONE && x_xf)
        return dfl_gemm_whole(ctx, gate.type, gate.data, x_xf, g, n_in, 2 * ffn, n, ffn, g_xf_kind != DFL_XF_NONE ? g_xf : nullptr,
                              g_xf_kind, st);
    if (pk && adjacent(gate, ffn, up, n_in)) {
        // (a product split over K applies the activation in its reduction: one launch less)
        ctx->swiglu_out = ffn % 16 == 0 ? g : nullptr;
        ctx->swiglu_done = false;
        rc = gemm(ctx, gate, x, pk, n_in, 2 * ffn, n, st);
        const bool done = ctx->swiglu_done;
        ctx->swiglu_out = nullptr;
        ctx->swiglu_done = false;
        if (rc) return rc;
        if (!done)
            silu_mul_ld_kernel<<<dim3(blocks_for(static_cast<size_t>(ffn)), n), 256, 0, st>>>(pk, pk + ffn, 2 * ffn, g, static_cast<int>(ffn));
        return DFLASH_OK;
    }
    if ((rc = gemm(ctx, gate, x, g, n_in, ffn, n, st))) return rc;
    if ((rc = gemm(ctx, up, x, u, n_in, ffn, n, st))) return rc;
    silu_mul_kernel<<<blocks_for(static_cast<size_t>(n) * ffn), 256, 0, st>>>(g, u, static_cast<size_t>(n) * ffn);
    return DFLASH_OK;
}

int32_t embed_rows(dflash_ctx *ctx, const dflash_qtensor &t, const int32_t *ids_dev, int n, int hidden, float *out,
                   hipStream_t st) {
    size_t rb = dflash_row_bytes(t.type, hidden);
    if (rb == 0) return dfl_fail(ctx, DFLASH_ERR_UNSUPPORTED, "embedding type %d", t.type);
    get_rows_kernel<<<dim3(blocks_for(hidden), n), 256, 0, st>>>(t.type, static_cast<const uint8_t *>(t.data), rb, ids_dev,
                                                               hidden, out);
    return DFLASH_OK;
}

}  // namespace

struct dflash_session {
    dflash_model_cfg cfg;
    int64_t capacity = 0, kv_n_pos = 0;
    int n_taps = 0;
    _Float16 *k_cache = nullptr, *vt_cache = nullptr;
    float *x = nullptr, *cur = nullptr, *q = nullptr, *k = nullptr, *v = nullptr, *attn = nullptr, *mix = nullptr;
    float *g = nullptr, *u = nullptr, *logits = nullptr, *gap = nullptr;
    float *pk = nullptr;  // [16][max(q_dim + 2 kv_dim, 2 ffn)]: output of a fused q/k/v or gate/up GEMM
    // cur and attn once more, as f16 in MFMA fragment order, for the projections that take the whole-K kernel
    uint8_t *xf_cur = nullptr, *xf_attn = nullptr, *xf_g = nullptr;
    float *hidden = nullptr;  // [16][n_taps][hidden] capture slots of the speculative step
    int32_t *ids = nullptr, *pos = nullptr, *argmax = nullptr;
    dfl_moe_scratch moe;
    // Captured graphs of the packed verify, one per distinct call shape (a hash over the model's
    // tensors, the row count, the taps and the output pointers).  A shape is run eagerly the first
    // time, captured the second time and replayed from then on: everything position-dependent is
    // read from device memory (pos[], written before each launch), nothing else changes.
    std::map<uint64_t, hipGraphExec_t> graphs;
    std::map<uint64_t, int> graph_seen;
    int64_t graph_replays = 0;
    struct PrefillPipe *pipe = nullptr;  // extra lanes of dflash_prefill_blocks (dflash_prefill_prepare, else made on first use)
};

// Extra lanes of a pipelined prefill.  A 16-row block's layers are a chain of small dependent launches that leave most
// of the GPU idle; consecutive blocks, a layer or so apart, fill each other's gaps.  An extra lane has its own context
// (split-K partial tiles, attention workspace: what two concurrent launches of one kind must not share), its own
// scratch (a session of capacity 16 whose K/V pointers are redirected to the owner's cache) and its own stream.
// Block b needs the earlier blocks' K/V rows of a layer before its attention in that layer: one event per (lane,
// layer), recorded behind the launch that writes the rows and behind the wait for the previous block's event.
constexpr int kMaxPrefillLanes = 8;
// Scratch of the grouped prefill of a mixture-of-experts target: the rows of up to `rows / 16` consecutive blocks pass
// through a layer together (one launch per operator, the weights of a projection read once for all of them, the
// experts regrouped by dfl_moe_ffn_group), attention alone block by block.  Null pointers: not set up (a dense
// target, or no device memory for it), and the lanes below serve instead.
struct PrefillGroup {
    int rows = 0;
    float *x = nullptr, *cur = nullptr, *mix = nullptr, *pk = nullptr, *q = nullptr, *attn = nullptr;
    uint8_t *xf_cur = nullptr, *xf_attn = nullptr;
    int32_t *ids = nullptr, *pos = nullptr;
    dfl_moe_group_scratch moe;
};
struct PrefillPipe {
    PrefillGroup group;
    int n_lanes = 4;  // blocks in flight: lane 0 is the owner itself (its context, its scratch, the caller's stream)
    struct Extra {
        dflash_ctx *ctx = nullptr;
        dflash_session *shadow = nullptr;
        _Float16 *own_k = nullptr, *own_vt = nullptr;  // the shadow session's own (unused) cache, put back before it is destroyed
        int64_t own_capacity = 0;
        hipStream_t stream = nullptr;
        hipEvent_t join = nullptr;
    } extra[kMaxPrefillLanes - 1];
    std::vector<hipEvent_t> kv_done[kMaxPrefillLanes];
    hipEvent_t fork = nullptr;
    bool ready = false;
};
// what verify_enqueue is told when it runs as one lane of the pipeline
struct PrefillLane {
    const hipEvent_t *mine, *other;
    bool wait_other;  // there is a previous block on the other lane
};

struct dflash_draft_session {
    dflash_draft_cfg cfg;
    int64_t capacity = 0, ctx_len = 0, vocab = 0;
    int64_t ctx_h_ready = 0;  // columns whose fc + hidden_norm are done
    int64_t kv_ready = 0;     // columns whose per-layer K/V are done
    float *ctx_raw = nullptr;  // [cap][n_taps*H] captured target hiddens
    float *ctx_h = nullptr;    // [cap][H]
    float *k_ctx = nullptr, *v_ctx = nullptr;  // [layer][cap][kv_dim]
    // f16 mirror for the MFMA attention (used while the context positions are 0, 1, 2, ... and the
    // block starts right behind them): K [layer][cap16][kv_dim], V transposed [layer][kv_dim][cap16]
    _Float16 *k16 = nullptr, *vt16 = nullptr;
    int64_t cap16 = 0;
    bool contiguous = true;
    int32_t *pos_ctx = nullptr;                // [cap]
    float *x = nullptr, *cur = nullptr, *q = nullptr, *k = nullptr, *v = nullptr, *attn = nullptr, *mix = nullptr;
    float *g = nullptr, *u = nullptr, *logits = nullptr, *tmp = nullptr;
    float *pk = nullptr;  // [16][max(q_dim + 2 kv_dim, 2 ffn)]: output of a fused q/k/v or gate/up GEMM
    // cur, attn and g once more, as f16 in MFMA fragment order, for the projections that take the whole-K kernel
    uint8_t *xf_cur = nullptr, *xf_attn = nullptr, *xf_g = nullptr;
    int32_t *ids = nullptr, *pos = nullptr, *argmax = nullptr;
    // every layer's context K/V projection as ONE batched GEMM (draft_prepare): its output [layer][16][2 kv_dim],
    // the list 0 .. n_layers - 1 and its length for the batched kernel
    float *pk_layers = nullptr;
    int32_t *layer_ids = nullptr, *n_layers_dev = nullptr;
    // DFlash-2 (MetalDFlashSession conv_buf / conv_dyn_* / topk_* / sel_h, metal_dflash.rs:5144-5155)
    float *conv_buf = nullptr;   // [16][H]
    float *conv_dyn = nullptr;   // [16][2 * kernel * H / group]: one sublayer's coefficients at a time
    int32_t *topk_ids = nullptr; // [16][16]
    float *topk_vals = nullptr;  // [16][16]
    float *sel_h = nullptr;      // [16][selector_rank]
    // captured graphs of the block forward (everything after the context preparation), one per distinct
    // (head, target, outputs) key; see draft_block_impl
    std::map<uint64_t, hipGraphExec_t> graphs;
    std::map<uint64_t, int> graph_seen;
    int64_t graph_replays = 0;
};

extern "C" {

int32_t dflash_session_create(dflash_ctx *ctx, const dflash_model_cfg *cfg, int64_t kv_capacity, int32_t n_taps,
                              dflash_session **out) {
    if (!ctx || !cfg || !out) return DFLASH_ERR_INVALID_INPUT;
    *out = nullptr;
    if (cfg->n_layers < 1 || cfg->hidden < 1 || cfg->n_q < 1 || cfg->n_kv < 1 || cfg->n_q % cfg->n_kv ||
        (cfg->head_dim != 64 && cfg->head_dim != 128 && cfg->head_dim != 256) || cfg->vocab < 1 || kv_capacity < 1)
        return dfl_fail(ctx, DFLASH_ERR_BAD_SHAPE, "session_create: unsupported model shape");
    dflash_session *s = new (std::nothrow) dflash_session();
    if (!s) return DFLASH_ERR_HIP;
    s->cfg = *cfg;
    s->capacity = (kv_capacity + 31) / 32 * 32;
    s->n_taps = n_taps;
    const size_t kv_dim = static_cast<size_t>(cfg->n_kv) * cfg->head_dim, q_dim = static_cast<size_t>(cfg->n_q) * cfg->head_dim;
    const size_t f = std::max(std::max(cfg->ffn, cfg->ffn_shared), cfg->ffn_expert);
    const size_t per_layer = static_cast<size_t>(s->capacity) * kv_dim;
    bool ok = dev_alloc(&s->k_cache, per_layer * cfg->n_layers) && dev_alloc(&s->vt_cache, per_layer * cfg->n_layers) &&
              dev_alloc(&s->x, 16 * cfg->hidden) && dev_alloc(&s->cur, 16 * cfg->hidden) && dev_alloc(&s->q, 16 * q_dim) &&
              dev_alloc(&s->k, 16 * kv_dim) && dev_alloc(&s->v, 16 * kv_dim) && dev_alloc(&s->attn, 16 * q_dim) &&
              dev_alloc(&s->mix, 16 * cfg->hidden) && dev_alloc(&s->g, 16 * f) && dev_alloc(&s->u, 16 * f) &&
              dev_alloc(&s->pk, 16 * std::max(q_dim + 2 * kv_dim, 2 * f)) &&
              dev_alloc(&s->xf_cur, dfl_xf_bytes((cfg->hidden + 255) / 256 * 256)) &&
              dev_alloc(&s->xf_attn, dfl_xf_bytes((static_cast<int64_t>(q_dim) + 255) / 256 * 256)) &&
              dev_alloc(&s->xf_g, dfl_xf_bytes((static_cast<int64_t>(f) + 255) / 256 * 256)) &&
              dev_alloc(&s->logits, 16 * static_cast<size_t>(cfg->vocab)) && dev_alloc(&s->gap, 16) &&
              dev_alloc(&s->ids, 16) && dev_alloc(&s->pos, 16) && dev_alloc(&s->argmax, 16) &&
              dev_alloc(&s->hidden, 16 * static_cast<size_t>(std::max(n_taps, 1)) * cfg->hidden);
    if (ok && cfg->n_expert > 0) {
        const size_t used = std::min(cfg->n_expert_used, cfg->n_expert);
        ok = dev_alloc(&s->moe.probs, 16 * static_cast<size_t>(cfg->n_expert)) && dev_alloc(&s->moe.sel_e, 16 * used) &&
             dev_alloc(&s->moe.sel_w, 16 * used) && dev_alloc(&s->moe.sg, 16) &&
             dev_alloc(&s->moe.act, 16 * used * cfg->ffn_expert) &&
             dev_alloc(&s->moe.eo, 16 * (std::min<size_t>(16 * used, cfg->n_expert) + 1) * cfg->hidden) &&
             dev_alloc(&s->moe.gate_out, 16 * (std::min<size_t>(16 * used, cfg->n_expert) + 1) * cfg->ffn_expert) &&
             dev_alloc(&s->moe.ids, cfg->n_expert + 1) && dev_alloc(&s->moe.n_distinct, 1) && dev_alloc(&s->moe.slot_of, 16 * used) &&
             dev_alloc(&s->moe.shared, 16 * cfg->hidden);
        s->moe.g = s->g;
        s->moe.u = s->u;
    }
    if (ok) ok = hipMemset(s->vt_cache, 0, per_layer * cfg->n_layers * 2) == hipSuccess;
    if (!ok) {
        dflash_session_destroy(s);
        return dfl_fail(ctx, DFLASH_ERR_HIP, "session_create: out of device memory");
    }
    *out = s;
    return DFLASH_OK;
}

namespace {
void prefill_group_free(PrefillGroup *g) {
    void *ptrs[] = {g->x, g->cur, g->mix, g->pk, g->q, g->attn, g->xf_cur, g->xf_attn, g->ids, g->pos, g->moe.logits, g->moe.sg,
                    g->moe.sel_e, g->moe.sel_w, g->moe.pick_pos, g->moe.ids, g->moe.n_slots, g->moe.slot_rows, g->moe.xg, g->moe.act,
                    g->moe.eo};
    for (void *p : ptrs)
        if (p) (void)hipFree(p);
    *g = PrefillGroup();
}

// Blocks per pass of the grouped prefill (DFLASH_PREFILL_GROUP; 0 or 1 switches it off).  Measured on the 35B-A3B
// shape, 2032-token prompt: 21.2 / 23.3 / 26.1 thousand prompt tokens/s with 16 / 24 / 32 blocks a pass, 7.3 with the
// lanes (a pass reads every expert about once, so its cost grows slowly with its rows).
int prefill_group_blocks() {
    static const int v = [] {
        const char *e = getenv("DFLASH_PREFILL_GROUP");
        return e && *e ? atoi(e) : 32;
    }();
    return std::max(0, std::min(kMaxGroupRows / 16, v));
}

// Sets the group scratch up for a mixture-of-experts shape; leaves it empty (no error) where the shape is not one the
// grouped path takes or the memory is not there.
void prefill_group_alloc(dflash_session *s, PrefillGroup *g) {
    const dflash_model_cfg &c = s->cfg;
    const int blocks = prefill_group_blocks();
    const int used = c.n_expert_used < c.n_expert ? c.n_expert_used : c.n_expert;
    if (blocks < 2 || c.n_expert < 1 || c.n_expert > 256 || used < 1 || c.hidden % DFL_QK_K || c.ffn_expert % DFL_QK_K) return;
    int rows = 16 * blocks;
    while (rows > 16 && rows * used > 4096) rows -= 16;
    if (static_cast<int64_t>(rows) > s->capacity) rows = static_cast<int>((s->capacity + 15) / 16 * 16);
    if (rows < 32) return;
    const size_t H = c.hidden, q_dim = static_cast<size_t>(c.n_q) * c.head_dim, kv_dim = static_cast<size_t>(c.n_kv) * c.head_dim;
    const size_t R = rows, nb = rows / 16;
    const int max_slots = dfl_moe_group_max_slots(c, rows);
    const size_t S = max_slots;
    const bool ok = dev_alloc(&g->x, R * H) && dev_alloc(&g->cur, R * H) && dev_alloc(&g->mix, R * H) &&
                    dev_alloc(&g->pk, R * (q_dim + 2 * kv_dim)) && dev_alloc(&g->q, R * q_dim) && dev_alloc(&g->attn, R * q_dim) &&
                    dev_alloc(&g->xf_cur, nb * dfl_xf_bytes(H)) && dev_alloc(&g->xf_attn, nb * dfl_xf_bytes(q_dim)) &&
                    dev_alloc(&g->ids, R) && dev_alloc(&g->pos, R) && dev_alloc(&g->moe.logits, R * c.n_expert) &&
                    dev_alloc(&g->moe.sg, R) && dev_alloc(&g->moe.sel_e, R * used) && dev_alloc(&g->moe.sel_w, R * used) &&
                    dev_alloc(&g->moe.pick_pos, R * used) && dev_alloc(&g->moe.ids, S) && dev_alloc(&g->moe.n_slots, 1) &&
                    dev_alloc(&g->moe.slot_rows, S * 16) && dev_alloc(&g->moe.xg, S * 16 * H) &&
                    dev_alloc(&g->moe.act, S * 16 * c.ffn_expert) && dev_alloc(&g->moe.eo, S * 16 * H);
    if (!ok) {
        (void)hipGetLastError();  // (an allocation that failed leaves its error behind)
        prefill_group_free(g);
        return;
    }
    g->moe.max_slots = max_slots;
    g->rows = rows;
}
}  // namespace

void dflash_session_destroy(dflash_session *s) {
    if (!s) return;
    if (PrefillPipe *p = s->pipe) {
        for (auto &x : p->extra)
            if (x.stream) (void)hipStreamSynchronize(x.stream);
        for (auto &v : p->kv_done)
            for (hipEvent_t e : v)
                if (e) (void)hipEventDestroy(e);
        if (p->fork) (void)hipEventDestroy(p->fork);
        for (auto &x : p->extra) {
            if (x.join) (void)hipEventDestroy(x.join);
            if (x.shadow) {  // give it back its own cache before it frees what it owns
                x.shadow->k_cache = x.own_k;
                x.shadow->vt_cache = x.own_vt;
                x.shadow->capacity = x.own_capacity;
                dflash_session_destroy(x.shadow);
            }
            if (x.ctx) dflash_ctx_destroy(x.ctx);  // (the stream belongs to the process-wide pool)
        }
        prefill_group_free(&p->group);
        delete p;
        s->pipe = nullptr;
    }
    for (auto &g : s->graphs)
        if (g.second) (void)hipGraphExecDestroy(g.second);
    void *ptrs[] = {s->k_cache, s->vt_cache, s->x, s->cur, s->q, s->k, s->v, s->attn, s->mix,
                    s->g, s->u, s->logits, s->gap, s->ids, s->pos, s->argmax, s->hidden,
                    s->moe.probs, s->moe.sel_e, s->moe.sel_w, s->moe.sg, s->moe.act, s->moe.eo, s->moe.shared,
                    s->moe.gate_out, s->moe.ids, s->moe.n_distinct, s->moe.slot_of, s->pk, s->xf_cur, s->xf_attn, s->xf_g};
    for (void *p : ptrs)
        if (p) (void)hipFree(p);
    delete s;
}

int64_t dflash_session_kv_n_pos(const dflash_session *s) { return s ? s->kv_n_pos : -1; }

int64_t dflash_session_graph_replays(const dflash_session *s) { return s ? s->graph_replays : -1; }

namespace {

// 64-bit mix over a byte range (FNV-1a on 8-byte words, tail bytes one by one)
uint64_t hash_bytes(const void *p, size_t n, uint64_t h) {
    const uint8_t *b = static_cast<const uint8_t *>(p);
    size_t i = 0;
    for (; i + 8 <= n; i += 8) {
        uint64_t w;
        memcpy(&w, b + i, 8);
        h = (h ^ w) * 0x100000001b3ull;
        h ^= h >> 29;
    }
    for (; i < n; i++) h = (h ^ b[i]) * 0x100000001b3ull;
    return h;
}

// Key of a model for the captured-graph cache: the fields a launch depends on (shape, tensor types and device
// pointers), one by one, so that padding bytes a caller left uninitialised never split the cache.
uint64_t hash_model(const dflash_model *m) {
    uint64_t h = 0x9e3779b97f4a7c15ull;
    auto word = [&](uint64_t w) {
        h = (h ^ w) * 0x100000001b3ull;
        h ^= h >> 29;
    };
    auto ptr = [&](const void *p) { word(reinterpret_cast<uintptr_t>(p)); };
    auto qt = [&](const dflash_qtensor &t) {
        word(static_cast<uint32_t>(t.type));
        ptr(t.data);
    };
    const dflash_model_cfg &c = m->cfg;
    const int32_t ints[11] = {c.n_layers, c.hidden, c.n_q, c.n_kv, c.head_dim, c.ffn, c.vocab, c.n_expert, c.n_expert_used,
                              c.ffn_expert, c.ffn_shared};
    for (int32_t v : ints) word(static_cast<uint32_t>(v));
    uint32_t fb[2];
    memcpy(fb, &c.eps, 4);
    memcpy(fb + 1, &c.rope_theta, 4);
    word(fb[0]);
    word(fb[1]);
    qt(m->token_embd);
    qt(m->output);
    ptr(m->output_norm);
    for (int il = 0; il < c.n_layers; il++) {
        const dflash_layer &L = m->layers[il];
        ptr(L.attn_norm);
        ptr(L.q_norm);
        ptr(L.k_norm);
        ptr(L.post_norm);
        for (const dflash_qtensor *t : {&L.wq, &L.wk, &L.wv, &L.wo, &L.gate, &L.up, &L.down, &L.router, &L.gate_exps, &L.up_exps,
                                        &L.down_exps})
            qt(*t);
        ptr(L.shexp_gate);
    }
    return h;
}

// Every launch of one packed verify, from the embedding rows to the argmax, on `st`: no host
// reads, no synchronisation, nothing that depends on the position except through pos[] on the
// device, so the sequence can be captured once and replayed.
int32_t verify_enqueue(dflash_ctx *ctx, const dflash_model *model, dflash_session *s, int32_t n, int64_t start,
                       const int32_t *tap_layers, int32_t n_taps, float *hidden_capture, float *lg, int32_t *am, float *gp,
                       hipStream_t st, bool want_head = true, const PrefillLane *lane = nullptr) {
    const dflash_model_cfg &c = model->cfg;
    const int H = c.hidden, hd = c.head_dim;
    const size_t q_dim = static_cast<size_t>(c.n_q) * hd, kv_dim = static_cast<size_t>(c.n_kv) * hd;
    int32_t rc = embed_rows(ctx, model->token_embd, s->ids, n, H, s->x, st);
    if (rc) return rc;
    const float scale = 1.0f / sqrtf(static_cast<float>(hd));
    const size_t per_layer = static_cast<size_t>(s->capacity) * kv_dim;
    bool cur_ready = false;  // s->cur already holds this layer's normalised input
    const float *pending_resid = nullptr;  // a dense layer's FFN output still to be added to s->x
    // which projections of a layer read their rows in fragment order (past the last layer: `qkv` stands for the output head)
    const int head_kind = want_head ? dfl_whole_kind(ctx, model->output.type, H, c.vocab, 0) : DFL_XF_NONE;
    auto layer_kinds = [&](int il) {
        if (il < c.n_layers)
            return layer_xf(ctx, model->layers[il], s->pk != nullptr, H, static_cast<int64_t>(q_dim), static_cast<int64_t>(kv_dim), c.ffn,
                            c.n_expert == 0);
        LayerXf head;
        head.qkv = head_kind;
        return head;
    };
    for (int il = 0; il < c.n_layers; il++) {
        const dflash_layer &L = model->layers[il];
        _Float16 *kc = s->k_cache + il * per_layer, *vtc = s->vt_cache + il * per_layer;
        // (a mixture-of-experts layer leaves the next layer's normalised input behind)
        // (a dense layer leaves its FFN output in s->mix: the residual add is folded into this norm)
        const bool moe = c.n_expert > 0;
        const LayerXf xk = layer_kinds(il);
        if (!cur_ready)
            rms_norm_kernel<<<n, 256, 0, st>>>(s->x, pending_resid, L.attn_norm, s->cur, H, c.eps, nullptr, nullptr,
                                               xk.qkv ? s->xf_cur : nullptr, xk.qkv);
        pending_resid = nullptr;
        cur_ready = false;
        bool packed;
        if ((rc = gemm_qkv(ctx, L.wq, L.wk, L.wv, s->cur, s->q, s->k, s->v, s->pk, true, &packed, H, q_dim, kv_dim, n, st, s->xf_cur, xk.qkv)))
            return rc;
        const int64_t tot = q_dim + 2 * kv_dim;
        qk_norm_rope_kernel<<<dim3(c.n_q + 2 * c.n_kv, n), 64, 0, st>>>(
            packed ? s->pk : s->q, packed ? tot : q_dim, packed ? s->pk + q_dim : s->k, packed ? tot : kv_dim, s->q, s->k, L.q_norm,
            L.k_norm, kc, s->pos, c.n_q, c.n_kv, hd, c.eps, c.rope_theta, packed ? s->pk + q_dim + kv_dim : s->v,
            packed ? tot : kv_dim, vtc, s->capacity);
        if (lane) {
            // This block's K/V rows of the layer are written; the earlier blocks' must be before the attention reads
            // them.  The wait for the previous block comes first and the record behind it: the event then stands for
            // "rows of this block AND of every block before it", whichever lanes those ran on.
            if (lane->wait_other) DFL_HIP_CHECK(ctx, hipStreamWaitEvent(st, lane->other[il], 0));
            DFL_HIP_CHECK(ctx, hipEventRecord(lane->mine[il], st));
        }
        // A block nobody asked head outputs of needs nothing of the last layer beyond its K/V rows, unless that layer's
        // residual is tapped: its attention, output projection and FFN would only feed the head.
        if (!want_head && il == c.n_layers - 1) {
            bool tapped_last = false;
            for (int t = 0; t < n_taps; t++) tapped_last = tapped_last || tap_layers[t] == il;
            if (!tapped_last) break;
        }
        // under capture the context length is read from pos[0] on the device: the same launches then serve every
        // position of the bucket
        if ((rc = dfl_attn_block(ctx, s->q, DFLASH_TYPE_F32, kc, vtc, 1, start, n, c.n_q, c.n_kv, hd, s->capacity, scale,
                                 s->attn, st, 0, 0, ctx->capturing ? s->pos : nullptr, xk.wo ? s->xf_attn : nullptr, xk.wo)))
            return rc;
        if (xk.wo)
            rc = dfl_gemm_whole(ctx, L.wo.type, L.wo.data, s->xf_attn, s->mix, static_cast<int64_t>(q_dim), H, n, 0, nullptr, DFL_XF_NONE, st);
        else
            rc = gemm(ctx, L.wo, s->attn, s->mix, q_dim, H, n, st);
        if (rc) return rc;
        // x += mix first; a mixture-of-experts layer also gets its shared-expert gate from here
        // (where the router's launch can take the add and the norm along, they are left to it; s->x then gets its
        // s->mix together with the experts' sum)
        const bool norm_in_router = moe && dfl_moe_norm_fusable(ctx, c, L, n);
        if (!norm_in_router)
            rms_norm_kernel<<<n, 256, 0, st>>>(s->x, s->mix, L.post_norm, s->cur, H, c.eps, moe ? L.shexp_gate : nullptr,
                                               moe ? s->moe.sg : nullptr, xk.gate_up ? s->xf_cur : nullptr, xk.gate_up);
        if (moe) {
            const float *next_w = il + 1 < c.n_layers ? model->layers[il + 1].attn_norm : model->output_norm;
            const int next_kind = layer_kinds(il + 1).qkv;  // (the next layer's q/k/v read what this layer's last kernel normalises)
            if ((rc = dfl_moe_ffn(ctx, c, L, s->cur, n, s->moe, s->x, L.shexp_gate != nullptr, next_w, s->cur, &cur_ready, st,
                                  norm_in_router ? s->mix : nullptr, norm_in_router ? L.post_norm : nullptr,
                                  next_kind ? s->xf_cur : nullptr, next_kind)))
                return rc;
        } else {
            // the down projection reads fragment-order rows only where the gate/up launch can write them
            const int down_kind = xk.gate_up ? xk.down : DFL_XF_NONE;
            if ((rc = gemm_gate_up(ctx, L.gate, L.up, s->cur, s->g, s->u, s->pk, H, c.ffn, n, st, s->xf_cur, xk.gate_up, s->xf_g, down_kind)))
                return rc;
            if (down_kind)
                rc = dfl_gemm_whole(ctx, L.down.type, L.down.data, s->xf_g, s->mix, c.ffn, H, n, 0, nullptr, DFL_XF_NONE, st);
            else
                rc = gemm(ctx, L.down, s->g, s->mix, c.ffn, H, n, st);
            if (rc) return rc;
            // x += mix: by the next norm, unless this layer's residual is captured first
            bool tapped = false;
            for (int t = 0; t < n_taps; t++) tapped = tapped || tap_layers[t] == il;
            if (tapped)
                add_kernel<<<blocks_for(static_cast<size_t>(n) * H), 256, 0, st>>>(s->x, s->mix, static_cast<size_t>(n) * H);
            else
                pending_resid = s->mix;
        }
        for (int t = 0; t < n_taps; t++)
            if (tap_layers[t] == il)
                capture_kernel<<<dim3(blocks_for(H), n), 256, 0, st>>>(s->x, hidden_capture, H, n_taps, t);
    }
    if (want_head) {  // (not for a caller that asked for no output of it: a prefill block wants K/V and the taps only)
        if (!cur_ready)
            rms_norm_kernel<<<n, 256, 0, st>>>(s->x, pending_resid, model->output_norm, s->cur, H, c.eps, nullptr, nullptr,
                                               head_kind ? s->xf_cur : nullptr, head_kind);
        if (head_kind)
            rc = dfl_gemm_whole(ctx, model->output.type, model->output.data, s->xf_cur, lg, H, c.vocab, n, 0, nullptr, DFL_XF_NONE, st);
        else
            rc = gemm(ctx, model->output, s->cur, lg, H, c.vocab, n, st);
        if (rc) return rc;
        if ((rc = dflash_argmax_top2(ctx, lg, n, c.vocab, c.vocab, am, gp, st))) return rc;
    }
    DFL_HIP_CHECK(ctx, hipGetLastError());
    return DFLASH_OK;
}

}  // namespace

namespace {
int32_t verify_block_impl(dflash_ctx *ctx, const dflash_model *model, dflash_session *s, const int32_t *tokens,
                          const int32_t *dev_tokens, int32_t n, int64_t start, const int32_t *tap_layers, int32_t n_taps,
                          int32_t *argmax, float *gap, float *hidden_capture, float *logits, int32_t *argmax_host,
                          dflash_stream_t stream, bool want_head = true);
}

int32_t dflash_verify_block(dflash_ctx *ctx, const dflash_model *model, dflash_session *s, const int32_t *tokens,
                            int32_t n, int64_t start, const int32_t *tap_layers, int32_t n_taps, int32_t *argmax,
                            float *gap, float *hidden_capture, float *logits, int32_t *argmax_host,
                            dflash_stream_t stream) {
    // no output of the head asked for: it is not run (inside the library a null output means the session's own buffer)
    const bool want_head = argmax || gap || logits || argmax_host;
    return verify_block_impl(ctx, model, s, tokens, nullptr, n, start, tap_layers, n_taps, argmax, gap, hidden_capture, logits,
                             argmax_host, stream, want_head);
}

namespace {

// dev_tokens (may be null): device ids that stand in wherever tokens[i] is negative (the drafter's
// output, still on the device: a speculative step then needs no host round trip between drafting and
// verifying).
int32_t verify_block_impl(dflash_ctx *ctx, const dflash_model *model, dflash_session *s, const int32_t *tokens,
                          const int32_t *dev_tokens, int32_t n, int64_t start, const int32_t *tap_layers, int32_t n_taps,
                          int32_t *argmax, float *gap, float *hidden_capture, float *logits, int32_t *argmax_host,
                          dflash_stream_t stream, bool want_head) {
    if (!ctx) return DFLASH_ERR_INVALID_INPUT;
    if (!model || !s || !tokens) return dfl_fail(ctx, DFLASH_ERR_INVALID_INPUT, "verify_block: null argument");
    if (const int32_t rc_ = model_tensors_checked(ctx, model)) return rc_;
    const dflash_model_cfg &c = model->cfg;
    // guard walls (metal_dflash.rs:9080-9186)
    if (n < 1 || n > 16) return dfl_fail(ctx, DFLASH_ERR_BAD_SHAPE, "verify_block: n %d outside 1..16", n);
    if (s->kv_n_pos != start)
        return dfl_fail(ctx, DFLASH_ERR_STATE, "verify_block: kv_n_pos %lld != start_position %lld",
                        static_cast<long long>(s->kv_n_pos), static_cast<long long>(start));
    if (start < 0 || start + n > s->capacity)
        return dfl_fail(ctx, DFLASH_ERR_STATE, "verify_block: positions %lld..%lld exceed the KV capacity %lld",
                        static_cast<long long>(start), static_cast<long long>(start + n), static_cast<long long>(s->capacity));
    for (int i = 0; i < n; i++)
        if ((tokens[i] < 0 && !dev_tokens) || tokens[i] >= c.vocab)
            return dfl_fail(ctx, DFLASH_ERR_INVALID_TOKEN, "verify_block: token %d at index %d outside vocabulary %d",
                            tokens[i], i, c.vocab);
    if (n_taps < 0 || n_taps > s->n_taps || (n_taps > 0 && (!tap_layers || !hidden_capture)))
        return dfl_fail(ctx, DFLASH_ERR_INVALID_INPUT, "verify_block: hidden capture arguments");
    if (memcmp(&c, &s->cfg, sizeof(c)) != 0) return dfl_fail(ctx, DFLASH_ERR_STATE, "verify_block: session/model shape mismatch");

    hipStream_t st = static_cast<hipStream_t>(stream);
    Int16Args ids_arg = {}, pos_arg = {};
    for (int i = 0; i < n; i++) {
        ids_arg.v[i] = tokens[i];
        pos_arg.v[i] = static_cast<int32_t>(start + i);
    }
    set_ids_pos_kernel<<<1, 64, 0, st>>>(ids_arg, pos_arg, n, s->ids, s->pos, dev_tokens, c.vocab);
    float *lg = logits ? logits : s->logits;
    int32_t *am = argmax ? argmax : s->argmax;
    float *gp = gap ? gap : s->gap;
    int32_t rc = DFLASH_OK;
    const bool use_graph = ctx->graphs && !ctx->timing && ctx->gstream;
    uint64_t key = 0;
    if (use_graph) {
        key = hash_model(model);
        const uintptr_t outs[4] = {reinterpret_cast<uintptr_t>(hidden_capture), reinterpret_cast<uintptr_t>(lg),
                                   reinterpret_cast<uintptr_t>(am), reinterpret_cast<uintptr_t>(gp)};
        key = hash_bytes(outs, sizeof(outs), key);
        // (the attention launches are cut by the bucket of the context length: see dfl_attn_block)
        const int64_t shape[4] = {n, n_taps, dfl_attn_bucket(start + n), want_head ? 1 : 0};
        key = hash_bytes(shape, sizeof(shape), key);
        if (n_taps > 0) key = hash_bytes(tap_layers, sizeof(int32_t) * n_taps, key);
    }
    auto exec_it = use_graph ? s->graphs.find(key) : s->graphs.end();
    if (use_graph && exec_it == s->graphs.end() && s->graph_seen.size() > 256) s->graph_seen.clear();
    if (use_graph && exec_it == s->graphs.end() && s->graphs.size() < 16 && s->graph_seen[key]++ >= 1) {
        // second call of this shape: capture it
        hipGraph_t graph = nullptr;
        DFL_HIP_CHECK(ctx, hipStreamBeginCapture(ctx->gstream, hipStreamCaptureModeThreadLocal));
        ctx->capturing = true;
        rc = verify_enqueue(ctx, model, s, n, start, tap_layers, n_taps, hidden_capture, lg, am, gp, ctx->gstream, want_head);
        ctx->capturing = false;
        const hipError_t end = hipStreamEndCapture(ctx->gstream, &graph);
        if (rc) {
            if (graph) (void)hipGraphDestroy(graph);
            return rc;
        }
        DFL_HIP_CHECK(ctx, end);
        hipGraphExec_t exec = nullptr;
        const hipError_t inst = hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0);
        (void)hipGraphDestroy(graph);
        DFL_HIP_CHECK(ctx, inst);
        exec_it = s->graphs.emplace(key, exec).first;
    }
    if (exec_it != s->graphs.end()) {
        DFL_HIP_CHECK(ctx, hipEventRecord(ctx->g_in, st));
        DFL_HIP_CHECK(ctx, hipStreamWaitEvent(ctx->gstream, ctx->g_in, 0));
        DFL_HIP_CHECK(ctx, hipGraphLaunch(exec_it->second, ctx->gstream));
        s->graph_replays++;
        DFL_HIP_CHECK(ctx, hipEventRecord(ctx->g_out, ctx->gstream));
        DFL_HIP_CHECK(ctx, hipStreamWaitEvent(st, ctx->g_out, 0));
    } else if ((rc = verify_enqueue(ctx, model, s, n, start, tap_layers, n_taps, hidden_capture, lg, am, gp, st, want_head))) {
        return rc;
    }
    s->kv_n_pos = start + n;
    if (argmax_host) {
        DFL_HIP_CHECK(ctx, hipMemcpyAsync(ctx->pinned, am, n * sizeof(int32_t), hipMemcpyDeviceToHost, st));
        DFL_HIP_CHECK(ctx, hipStreamSynchronize(st));
        memcpy(argmax_host, ctx->pinned, n * sizeof(int32_t));
    }
    return DFLASH_OK;
}

}  // namespace

int32_t dflash_restore(dflash_ctx *ctx, dflash_session *s, int64_t start, int32_t n, int32_t n_keep) {
    if (!ctx || !s) return DFLASH_ERR_INVALID_INPUT;
    if (n < 1 || n_keep < 0 || n_keep > n)
        return dfl_fail(ctx, DFLASH_ERR_BAD_SHAPE, "restore: n_keep %d outside 0..%d", n_keep, n);
    if (s->kv_n_pos != start + n)
        return dfl_fail(ctx, DFLASH_ERR_STATE, "restore: kv_n_pos %lld != start %lld + n %d (must follow the matching verify)",
                        static_cast<long long>(s->kv_n_pos), static_cast<long long>(start), n);
    s->kv_n_pos = start + n_keep;  // stale rows stay in place; the next verify overwrites them
    return DFLASH_OK;
}

namespace {
void prefill_pipe_destroy_extras(PrefillPipe *p) {
    for (auto &x : p->extra) {
        if (x.join) (void)hipEventDestroy(x.join);
        if (x.shadow) {  // give it back its own cache before it frees what it owns
            x.shadow->k_cache = x.own_k;
            x.shadow->vt_cache = x.own_vt;
            x.shadow->capacity = x.own_capacity;
            dflash_session_destroy(x.shadow);
        }
        if (x.ctx) dflash_ctx_destroy(x.ctx);  // (the stream belongs to the process-wide pool)
        x = PrefillPipe::Extra();
    }
}

int32_t prefill_pipe_create_lanes(dflash_ctx *ctx, dflash_session *s, PrefillPipe *p);

// The extra lanes of the pipelined prefill.  If one of them cannot be made (device memory), what was made is taken down
// again and the prefill runs with the owner's lane alone: slower, never failing for that reason.
int32_t prefill_pipe_create(dflash_ctx *ctx, dflash_session *s) {
    PrefillPipe *p = new (std::nothrow) PrefillPipe();
    if (!p) return dfl_fail(ctx, DFLASH_ERR_HIP, "prefill_blocks: out of host memory");
    s->pipe = p;  // (whatever has been made so far is taken down with the session)
    prefill_group_alloc(s, &p->group);
    if (prefill_pipe_create_lanes(ctx, s, p) != DFLASH_OK) {
        for (auto &v : p->kv_done) {
            for (hipEvent_t e : v)
                if (e) (void)hipEventDestroy(e);
            v.clear();
        }
        if (p->fork) (void)hipEventDestroy(p->fork);
        p->fork = nullptr;
        prefill_pipe_destroy_extras(p);
        p->n_lanes = 1;
        p->kv_done[0].assign(s->cfg.n_layers, nullptr);
        for (hipEvent_t &e : p->kv_done[0]) DFL_HIP_CHECK(ctx, hipEventCreateWithFlags(&e, hipEventDisableTiming));
        DFL_HIP_CHECK(ctx, hipEventCreateWithFlags(&p->fork, hipEventDisableTiming));
        p->ready = true;
    }
    return DFLASH_OK;
}

int32_t prefill_pipe_create_lanes(dflash_ctx *ctx, dflash_session *s, PrefillPipe *p) {
    static const int lanes_env = [] {
        const char *v = getenv("DFLASH_PREFILL_LANES");
        return v && *v ? atoi(v) : 4;  // measured on the 35B-A3B shape: 3290 / 4530 / 5160 / 5650 / 5150 / 4870 prompt tokens/s with
    }();                               // 1 / 2 / 3 / 4 / 6 / 8 blocks in flight (a process has four hardware queues)
    p->n_lanes = std::max(1, std::min(kMaxPrefillLanes, lanes_env));
    for (int i = 0; i + 1 < p->n_lanes; i++) {
        PrefillPipe::Extra &x = p->extra[i];
        // A lane's context serves verify blocks only (attention partials, split-K tiles): the default workspace, not the
        // owner's, which may have been sized for the wide sampler.
        int32_t rc = dflash_ctx_create(ctx->device, std::min<size_t>(ctx->workspace_bytes, size_t(128) << 20), &x.ctx);
        if (rc) return dfl_fail(ctx, rc, "prefill_blocks: context of lane %d", i + 1);
        if ((rc = dflash_session_create(x.ctx, &s->cfg, 16, s->n_taps, &x.shadow)))
            return dfl_fail(ctx, rc, "prefill_blocks: scratch set of lane %d", i + 1);
        x.own_k = x.shadow->k_cache;
        x.own_vt = x.shadow->vt_cache;
        x.own_capacity = x.shadow->capacity;
        x.shadow->k_cache = s->k_cache;
        x.shadow->vt_cache = s->vt_cache;
        x.shadow->capacity = s->capacity;
        // The lane streams are made once per process and device and shared by every session.  Streams made afresh
        // for a second session (after the first one's were destroyed) landed on fewer hardware queues: its prefill
        // ran at the pace of two lanes (448 against 348 ms for 2048 tokens).
        {
            static std::mutex pool_mutex;
            static std::map<int, std::array<hipStream_t, kMaxPrefillLanes - 1>> pool;  // by device ordinal
            std::lock_guard<std::mutex> lock(pool_mutex);
            hipStream_t &slot = pool[ctx->device][i];  // (a new entry starts as null pointers)
            if (!slot) DFL_HIP_CHECK(ctx, hipStreamCreateWithFlags(&slot, hipStreamNonBlocking));
            x.stream = slot;
        }
        DFL_HIP_CHECK(ctx, hipEventCreateWithFlags(&x.join, hipEventDisableTiming));
    }
    for (int i = 0; i < p->n_lanes; i++) {
        p->kv_done[i].assign(s->cfg.n_layers, nullptr);
        for (hipEvent_t &e : p->kv_done[i]) DFL_HIP_CHECK(ctx, hipEventCreateWithFlags(&e, hipEventDisableTiming));
    }
    DFL_HIP_CHECK(ctx, hipEventCreateWithFlags(&p->fork, hipEventDisableTiming));
    p->ready = true;
    return DFLASH_OK;
}
}  // namespace

int32_t dflash_prefill_prepare(dflash_ctx *ctx, dflash_session *s) {
    if (!ctx) return DFLASH_ERR_INVALID_INPUT;
    if (!s) return dfl_fail(ctx, DFLASH_ERR_INVALID_INPUT, "prefill_prepare: null session");
    if (s->pipe) return s->pipe->ready ? DFLASH_OK : dfl_fail(ctx, DFLASH_ERR_STATE, "prefill_prepare: the extra lanes could not be set up earlier");
    return prefill_pipe_create(ctx, s);
}

namespace {

// Whether every layer of the model is one the grouped prefill takes: q/k/v adjacent and, like the output projection,
// a whole-K product over fragment-order rows; the experts as dfl_moe_ffn_group wants them.
bool prefill_group_takes(const dflash_ctx *ctx, const dflash_model *model, const PrefillGroup &g) {
    const dflash_model_cfg &c = model->cfg;
    if (!g.rows || c.n_expert < 1) return false;
    const int64_t H = c.hidden, q_dim = static_cast<int64_t>(c.n_q) * c.head_dim, kv_dim = static_cast<int64_t>(c.n_kv) * c.head_dim;
    for (int il = 0; il < c.n_layers; il++) {
        const dflash_layer &L = model->layers[il];
        const LayerXf k = layer_xf(ctx, L, true, H, q_dim, kv_dim, c.ffn, false);
        if (k.qkv == DFL_XF_NONE || k.wo == DFL_XF_NONE || !dfl_moe_group_fits(ctx, c, L, g.rows)) return false;
    }
    return true;
}

// One group of n rows (positions start .. start + n - 1) through every layer, on `st`: K/V rows into the session's
// cache, tapped residuals into hidden_capture.  A row gets the bits verify_enqueue gives it in its own 16-row block:
// every operator here is that block's operator over more rows (or the block's own launch: attention).
int32_t prefill_group_enqueue(dflash_ctx *ctx, const dflash_model *model, dflash_session *s, PrefillGroup &g, const int32_t *tokens,
                              int32_t n, int64_t start, const int32_t *tap_layers, int32_t n_taps, float *hidden_capture,
                              hipStream_t st) {
    const dflash_model_cfg &c = model->cfg;
    const int H = c.hidden, hd = c.head_dim;
    const size_t q_dim = static_cast<size_t>(c.n_q) * hd, kv_dim = static_cast<size_t>(c.n_kv) * hd;
    const int64_t tot = static_cast<int64_t>(q_dim + 2 * kv_dim);
    const size_t xf_h = dfl_xf_bytes(H), xf_q = dfl_xf_bytes(static_cast<int64_t>(q_dim));
    IntGroupArgs ids_arg = {};
    for (int i = 0; i < n; i++) ids_arg.v[i] = tokens[i];
    set_group_ids_pos_kernel<<<(n + 255) / 256, 256, 0, st>>>(ids_arg, static_cast<int>(start), n, g.ids, g.pos);
    int32_t rc = embed_rows(ctx, model->token_embd, g.ids, n, H, g.x, st);
    if (rc) return rc;
    const float scale = 1.0f / sqrtf(static_cast<float>(hd));
    const size_t per_layer = static_cast<size_t>(s->capacity) * kv_dim;
    auto qkv_kind = [&](int il) {
        return il < c.n_layers ? layer_xf(ctx, model->layers[il], true, H, static_cast<int64_t>(q_dim), static_cast<int64_t>(kv_dim), c.ffn, false).qkv
                               : DFL_XF_NONE;
    };
    for (int il = 0; il < c.n_layers; il++) {
        const dflash_layer &L = model->layers[il];
        _Float16 *kc = s->k_cache + il * per_layer, *vtc = s->vt_cache + il * per_layer;
        const LayerXf xk = layer_xf(ctx, L, true, H, static_cast<int64_t>(q_dim), static_cast<int64_t>(kv_dim), c.ffn, false);
        if (il == 0)  // (later layers: the experts' last kernel has normalised their input)
            rms_norm_kernel<<<n, 256, 0, st>>>(g.x, nullptr, L.attn_norm, g.cur, H, c.eps, nullptr, nullptr, g.xf_cur, xk.qkv, xf_h);
        if ((rc = dfl_gemm_whole_blocks(ctx, L.wq.type, L.wq.data, g.xf_cur, g.pk, H, tot, n, 0, nullptr, DFL_XF_NONE, st))) return rc;
        qk_norm_rope_kernel<<<dim3(c.n_q + 2 * c.n_kv, n), 64, 0, st>>>(g.pk, tot, g.pk + q_dim, tot, g.q, nullptr, L.q_norm, L.k_norm, kc,
                                                                      g.pos, c.n_q, c.n_kv, hd, c.eps, c.rope_theta,
                                                                      g.pk + q_dim + kv_dim, tot, vtc, s->capacity);
        // nothing of the last layer beyond its K/V rows is needed unless its residual is tapped (as in verify_enqueue)
        if (il == c.n_layers - 1) {
            bool tapped_last = false;
            for (int t = 0; t < n_taps; t++) tapped_last = tapped_last || tap_layers[t] == il;
            if (!tapped_last) break;
        }
        if ((rc = dfl_attn_blocks(ctx, g.q, DFLASH_TYPE_F32, kc, vtc, start, n, c.n_q, c.n_kv, hd, s->capacity, scale, g.attn, st, g.xf_attn,
                                  xk.wo)))
            return rc;
        if ((rc = dfl_gemm_whole_blocks(ctx, L.wo.type, L.wo.data, g.xf_attn, g.mix, static_cast<int64_t>(q_dim), H, n, 0, nullptr,
                                        DFL_XF_NONE, st)))
            return rc;
        const float *next_w = il + 1 < c.n_layers ? model->layers[il + 1].attn_norm : model->output_norm;
        const int next_kind = qkv_kind(il + 1);
        // x += mix, the experts' norm and the shared-expert gates: the block path's norm kernel over all the rows
        rms_norm_kernel<<<n, 256, 0, st>>>(g.x, g.mix, L.post_norm, g.cur, H, c.eps, L.shexp_gate, g.moe.sg);
        if ((rc = dfl_moe_ffn_group(ctx, c, L, g.x, g.cur, n, g.moe, next_w, next_kind ? g.xf_cur : nullptr, next_kind, xf_h, st)))
            return rc;
        for (int t = 0; t < n_taps; t++)
            if (tap_layers[t] == il)
                capture_kernel<<<dim3(blocks_for(H), n), 256, 0, st>>>(g.x, hidden_capture, H, n_taps, t);
    }
    DFL_HIP_CHECK(ctx, hipGetLastError());
    return DFLASH_OK;
}

}  // namespace

int32_t dflash_prefill_blocks(dflash_ctx *ctx, const dflash_model *model, dflash_session *s, const int32_t *tokens,
                              int32_t n_tokens, int64_t start, const int32_t *tap_layers, int32_t n_taps,
                              float *hidden_capture, dflash_stream_t stream) {
    if (!ctx) return DFLASH_ERR_INVALID_INPUT;
    if (!model || !s || !tokens) return dfl_fail(ctx, DFLASH_ERR_INVALID_INPUT, "prefill_blocks: null argument");
    if (const int32_t rc_ = model_tensors_checked(ctx, model)) return rc_;
    const dflash_model_cfg &c = model->cfg;
    if (n_tokens < 1) return dfl_fail(ctx, DFLASH_ERR_BAD_SHAPE, "prefill_blocks: n_tokens %d", n_tokens);
    if (s->kv_n_pos != start)
        return dfl_fail(ctx, DFLASH_ERR_STATE, "prefill_blocks: kv_n_pos %lld != start_position %lld",
                        static_cast<long long>(s->kv_n_pos), static_cast<long long>(start));
    if (start < 0 || start + n_tokens > s->capacity)
        return dfl_fail(ctx, DFLASH_ERR_STATE, "prefill_blocks: positions %lld..%lld exceed the KV capacity %lld",
                        static_cast<long long>(start), static_cast<long long>(start + n_tokens), static_cast<long long>(s->capacity));
    for (int i = 0; i < n_tokens; i++)
        if (tokens[i] < 0 || tokens[i] >= c.vocab)
            return dfl_fail(ctx, DFLASH_ERR_INVALID_TOKEN, "prefill_blocks: token %d at index %d outside vocabulary %d", tokens[i], i, c.vocab);
    if (n_taps < 0 || n_taps > s->n_taps || (n_taps > 0 && (!tap_layers || !hidden_capture)))
        return dfl_fail(ctx, DFLASH_ERR_INVALID_INPUT, "prefill_blocks: hidden capture arguments");
    if (memcmp(&c, &s->cfg, sizeof(c)) != 0) return dfl_fail(ctx, DFLASH_ERR_STATE, "prefill_blocks: session/model shape mismatch");
    int32_t rc = DFLASH_OK;
    if (!s->pipe && (rc = prefill_pipe_create(ctx, s))) return rc;
    PrefillPipe *p = s->pipe;
    if (!p->ready) return dfl_fail(ctx, DFLASH_ERR_STATE, "prefill_blocks: the extra lanes could not be set up earlier");
    if (n_tokens > 16 && start + n_tokens <= 0x7fffffffll && prefill_group_takes(ctx, model, p->group)) {
        // rows of many blocks per pass (see PrefillGroup); the caller's stream alone
        const size_t cap_row = static_cast<size_t>(std::max(n_taps, 0)) * c.hidden;
        for (int32_t t0 = 0; t0 < n_tokens; t0 += p->group.rows) {
            const int32_t n = std::min<int32_t>(p->group.rows, n_tokens - t0);
            if ((rc = prefill_group_enqueue(ctx, model, s, p->group, tokens + t0, n, start + t0, tap_layers, n_taps,
                                            hidden_capture ? hidden_capture + static_cast<size_t>(t0) * cap_row : nullptr,
                                            static_cast<hipStream_t>(stream)))) {
                (void)hipStreamSynchronize(static_cast<hipStream_t>(stream));
                return rc;  // (kv_n_pos unchanged: rows written past it are overwritten by the next block)
            }
        }
        s->kv_n_pos = start + n_tokens;
        return DFLASH_OK;
    }
    const int n_lanes = p->n_lanes;
    hipStream_t lanes_st[kMaxPrefillLanes] = {static_cast<hipStream_t>(stream)};
    dflash_ctx *lanes_ctx[kMaxPrefillLanes] = {ctx};
    dflash_session *lanes_s[kMaxPrefillLanes] = {s};
    // the extra lanes start behind whatever the caller's stream holds (earlier blocks' K/V rows among it)
    DFL_HIP_CHECK(ctx, hipEventRecord(p->fork, lanes_st[0]));
    for (int i = 1; i < n_lanes; i++) {
        lanes_st[i] = p->extra[i - 1].stream;
        lanes_ctx[i] = p->extra[i - 1].ctx;
        lanes_s[i] = p->extra[i - 1].shadow;
        DFL_HIP_CHECK(ctx, hipStreamWaitEvent(lanes_st[i], p->fork, 0));
    }
    const size_t cap_row = static_cast<size_t>(std::max(n_taps, 0)) * c.hidden;
    // Expert launches of different lanes cannot share a CU (a workgroup fills its LDS); with half the CUs each, two
    // run side by side.  Measured on the 35B-A3B shape, four lanes: 5840 / 6010 / 6280 / 6200 prompt tokens/s with
    // 256 / 192 / 128 / 96 workgroups per expert launch (a single block in flight loses with fewer: 4.4 -> 5.1 ms).
    static const int lane_wgs_env = [] {
        const char *v = getenv("DFLASH_PREFILL_MOE_WGS");
        return v && *v ? atoi(v) : 0;
    }();
    const int owner_wgs = ctx->batch_wgs;
    if (n_lanes > 1 && n_tokens > 16)  // (a lone block keeps the whole chip)
        for (int i = 0; i < n_lanes; i++) lanes_ctx[i]->batch_wgs = lane_wgs_env > 0 ? lane_wgs_env : std::max(1, ctx->n_cu / 2);
    int block = 0;
    for (int32_t t0 = 0; t0 < n_tokens && !rc; t0 += 16, block++) {
        const int lane_i = block % n_lanes, prev_i = (block + n_lanes - 1) % n_lanes;
        const int32_t n = std::min<int32_t>(16, n_tokens - t0);
        dflash_session *ls = lanes_s[lane_i];
        Int16Args ids_arg = {}, pos_arg = {};
        for (int i = 0; i < n; i++) {
            ids_arg.v[i] = tokens[t0 + i];
            pos_arg.v[i] = static_cast<int32_t>(start + t0 + i);
        }
        set_ids_pos_kernel<<<1, 64, 0, lanes_st[lane_i]>>>(ids_arg, pos_arg, n, ls->ids, ls->pos, nullptr, c.vocab);
        const PrefillLane lane = {p->kv_done[lane_i].data(), p->kv_done[prev_i].data(), block > 0 && n_lanes > 1};
        rc = verify_enqueue(lanes_ctx[lane_i], model, ls, n, start + t0, tap_layers, n_taps,
                            hidden_capture ? hidden_capture + static_cast<size_t>(t0) * cap_row : nullptr, ls->logits, ls->argmax, ls->gap,
                            lanes_st[lane_i], false, &lane);
        if (rc && lane_i > 0) rc = dfl_fail(ctx, rc, "prefill_blocks: %s", dflash_last_error(lanes_ctx[lane_i]));
    }
    ctx->batch_wgs = owner_wgs;
    for (int i = 1; i < n_lanes; i++) lanes_ctx[i]->batch_wgs = 0;
    // the caller's stream continues behind every lane
    hipError_t err = hipSuccess;
    for (int i = 1; i < n_lanes && err == hipSuccess; i++) {
        err = hipEventRecord(p->extra[i - 1].join, lanes_st[i]);
        if (err == hipSuccess) err = hipStreamWaitEvent(lanes_st[0], p->extra[i - 1].join, 0);
    }
    if (rc) {
        for (int i = n_lanes - 1; i >= 0; i--) (void)hipStreamSynchronize(lanes_st[i]);
        return rc;  // (kv_n_pos unchanged: rows written past it are overwritten by the next block)
    }
    DFL_HIP_CHECK(ctx, err);
    s->kv_n_pos = start + n_tokens;
    return DFLASH_OK;
}

int32_t dflash_draft_session_create(dflash_ctx *ctx, const dflash_draft_cfg *cfg, int64_t ctx_capacity, int64_t vocab,
                                    dflash_draft_session **out) {
    if (!ctx || !cfg || !out) return DFLASH_ERR_INVALID_INPUT;
    *out = nullptr;
    if (cfg->n_layers < 1 || cfg->block_size < 1 || cfg->block_size > 16 || cfg->n_q % cfg->n_kv ||
        (cfg->head_dim != 64 && cfg->head_dim != 128 && cfg->head_dim != 256) || cfg->n_taps < 1 || ctx_capacity < 1)
        return dfl_fail(ctx, DFLASH_ERR_BAD_SHAPE, "draft_session_create: unsupported drafter shape");
    // DFlash-2 walls (loader.rs:1047-1057; the selector reads the top-16 kernel's output, so top_k = 16)
    if (cfg->conv_kernel_size < 0 || cfg->conv_kernel_size > 8 || cfg->selector_rank < 0 || cfg->selector_rank > 1024 ||
        (cfg->conv_kernel_size > 0 && (cfg->conv_group_size < 1 || cfg->hidden % cfg->conv_group_size)) ||
        (cfg->selector_rank > 0 && cfg->selector_top_k != 16))
        return dfl_fail(ctx, DFLASH_ERR_BAD_SHAPE, "draft_session_create: unsupported DFlash-2 shape (kernel %d group %d rank %d top_k %d)",
                        cfg->conv_kernel_size, cfg->conv_group_size, cfg->selector_rank, cfg->selector_top_k);
    dflash_draft_session *s = new (std::nothrow) dflash_draft_session();
    if (!s) return DFLASH_ERR_HIP;
    s->cfg = *cfg;
    s->capacity = ctx_capacity;
    s->cap16 = (ctx_capacity + 16 + 31) / 32 * 32;
    s->vocab = vocab;
    const size_t H = cfg->hidden, kv_dim = static_cast<size_t>(cfg->n_kv) * cfg->head_dim,
                 q_dim = static_cast<size_t>(cfg->n_q) * cfg->head_dim, cap = ctx_capacity;
    bool ok = dev_alloc(&s->ctx_raw, cap * cfg->n_taps * H) && dev_alloc(&s->ctx_h, cap * H) &&
              dev_alloc(&s->k_ctx, cap * kv_dim * cfg->n_layers) && dev_alloc(&s->v_ctx, cap * kv_dim * cfg->n_layers) &&
              dev_alloc(&s->k16, ((cap + 16 + 31) / 32 * 32) * kv_dim * cfg->n_layers) &&
              dev_alloc(&s->vt16, ((cap + 16 + 31) / 32 * 32) * kv_dim * cfg->n_layers) &&
              dev_alloc(&s->pos_ctx, cap) && dev_alloc(&s->x, 16 * H) && dev_alloc(&s->cur, 16 * H) &&
              dev_alloc(&s->q, 16 * q_dim) && dev_alloc(&s->k, 16 * kv_dim) && dev_alloc(&s->v, 16 * kv_dim) &&
              dev_alloc(&s->attn, 16 * q_dim) && dev_alloc(&s->mix, 16 * H) && dev_alloc(&s->g, 16 * static_cast<size_t>(cfg->ffn)) &&
              dev_alloc(&s->u, 16 * static_cast<size_t>(cfg->ffn)) && dev_alloc(&s->logits, 16 * static_cast<size_t>(vocab)) &&
              dev_alloc(&s->pk, 16 * std::max(q_dim + 2 * kv_dim, 2 * static_cast<size_t>(cfg->ffn))) &&
              dev_alloc(&s->tmp, 16 * std::max(H, kv_dim)) && dev_alloc(&s->ids, 16) && dev_alloc(&s->pos, 16) &&
              dev_alloc(&s->argmax, 16) && dev_alloc(&s->pk_layers, static_cast<size_t>(cfg->n_layers) * 16 * 2 * kv_dim) &&
              dev_alloc(&s->layer_ids, static_cast<size_t>(cfg->n_layers)) && dev_alloc(&s->n_layers_dev, 1) &&
              dev_alloc(&s->xf_cur, dfl_xf_bytes((static_cast<int64_t>(H) + 255) / 256 * 256)) &&
              dev_alloc(&s->xf_attn, dfl_xf_bytes((static_cast<int64_t>(q_dim) + 255) / 256 * 256)) &&
              dev_alloc(&s->xf_g, dfl_xf_bytes((static_cast<int64_t>(cfg->ffn) + 255) / 256 * 256));
    if (ok) {
        std::vector<int32_t> ids(static_cast<size_t>(cfg->n_layers));
        for (int i = 0; i < cfg->n_layers; i++) ids[i] = i;
        const int32_t n = cfg->n_layers;
        ok = hipMemcpy(s->layer_ids, ids.data(), ids.size() * sizeof(int32_t), hipMemcpyHostToDevice) == hipSuccess &&
             hipMemcpy(s->n_layers_dev, &n, sizeof(n), hipMemcpyHostToDevice) == hipSuccess;
    }
    if (ok && cfg->conv_kernel_size > 0)
        ok = dev_alloc(&s->conv_buf, 16 * H) &&
             dev_alloc(&s->conv_dyn, 16 * static_cast<size_t>(2) * cfg->conv_kernel_size * (H / cfg->conv_group_size));
    if (ok && cfg->selector_rank > 0)
        ok = dev_alloc(&s->topk_ids, 16 * 16) && dev_alloc(&s->topk_vals, 16 * 16) &&
             dev_alloc(&s->sel_h, 16 * static_cast<size_t>(cfg->selector_rank));
    if (!ok) {
        dflash_draft_session_destroy(s);
        return dfl_fail(ctx, DFLASH_ERR_HIP, "draft_session_create: out of device memory");
    }
    *out = s;
    return DFLASH_OK;
}

void dflash_draft_session_destroy(dflash_draft_session *s) {
    if (!s) return;
    void *ptrs[] = {s->ctx_raw, s->ctx_h, s->k_ctx, s->v_ctx, s->k16, s->vt16, s->pos_ctx, s->x, s->cur, s->q, s->k, s->v,
                    s->attn, s->mix, s->g, s->u, s->logits, s->tmp, s->ids, s->pos, s->argmax, s->pk, s->pk_layers,
                    s->layer_ids, s->n_layers_dev, s->xf_cur, s->xf_attn, s->xf_g,
                    s->conv_buf, s->conv_dyn, s->topk_ids, s->topk_vals, s->sel_h};
    for (void *p : ptrs)
        if (p) (void)hipFree(p);
    for (auto &g : s->graphs)
        if (g.second) (void)hipGraphExecDestroy(g.second);
    delete s;
}

int64_t dflash_draft_session_graph_replays(const dflash_draft_session *s) { return s ? s->graph_replays : -1; }

int64_t dflash_draft_session_ctx_len(const dflash_draft_session *s) { return s ? s->ctx_len : -1; }

int32_t dflash_draft_append_ctx(dflash_ctx *ctx, dflash_draft_session *s, const float *hidden_capture, int32_t n_cols,
                                const int32_t *positions, dflash_stream_t stream) {
    if (!ctx || !s) return DFLASH_ERR_INVALID_INPUT;
    if (n_cols < 0 || (n_cols > 0 && (!hidden_capture || !positions)))
        return dfl_fail(ctx, DFLASH_ERR_INVALID_INPUT, "append_ctx: null argument");
    if (s->ctx_len + n_cols > s->capacity)
        return dfl_fail(ctx, DFLASH_ERR_STATE, "append_ctx: %lld + %d columns exceed the context capacity %lld",
                        static_cast<long long>(s->ctx_len), n_cols, static_cast<long long>(s->capacity));
    if (n_cols == 0) return DFLASH_OK;
    for (int i = 0; i < n_cols; i++)
        if (positions[i] != s->ctx_len + i) s->contiguous = false;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const size_t feat = static_cast<size_t>(s->cfg.n_taps) * s->cfg.hidden;
    DFL_HIP_CHECK(ctx, hipMemcpyAsync(s->ctx_raw + s->ctx_len * feat, hidden_capture, n_cols * feat * sizeof(float),
                                      hipMemcpyDeviceToDevice, st));
    if (n_cols <= 16) {
        Int16Args none = {}, pos_arg = {};
        for (int i = 0; i < n_cols; i++) pos_arg.v[i] = positions[i];
        set_ids_pos_kernel<<<1, 64, 0, st>>>(none, pos_arg, n_cols, nullptr, s->pos_ctx + s->ctx_len, nullptr, 0);
    } else {
        DFL_HIP_CHECK(ctx, hipMemcpyAsync(s->pos_ctx + s->ctx_len, positions, n_cols * sizeof(int32_t), hipMemcpyHostToDevice, st));
    }
    s->ctx_len += n_cols;
    return DFLASH_OK;
}

namespace {

// Phase 1 of the drafter (metal_dflash.rs:16045-16143) and the per-layer context K/V, for the
// context columns appended since the last call: fc + hidden_norm, then each layer's K (normed and
// rotated at the column's own position) and V, and the f16 mirror while it is kept (mirror).
// The watermarks advance once everything was enqueued without error.
int32_t draft_prepare(dflash_ctx *ctx, const dflash_draft_head *head, dflash_draft_session *s, bool mirror, hipStream_t st) {
    const dflash_draft_cfg &c = head->cfg;
    const int H = c.hidden, hd = c.head_dim;
    const size_t kv_dim = static_cast<size_t>(c.n_kv) * hd;
    const size_t feat = static_cast<size_t>(c.n_taps) * H;
    const bool fast = mirror;
    int32_t rc;
    if (s->ctx_h_ready >= s->ctx_len && s->kv_ready >= s->ctx_len) return DFLASH_OK;
    for (int64_t c0 = s->ctx_h_ready; c0 < s->ctx_len; c0 += 16) {
        const int m = static_cast<int>(std::min<int64_t>(16, s->ctx_len - c0));
        if ((rc = gemm(ctx, head->fc, s->ctx_raw + c0 * feat, s->tmp, feat, H, m, st))) return rc;
        rms_norm_kernel<<<m, 256, 0, st>>>(s->tmp, nullptr, head->hidden_norm, s->ctx_h + c0 * H, H, c.eps, nullptr, nullptr);
    }
    // Every layer's K/V projection reads the same rows (ctx_h): when the layers' [wk; wv] pairs are Q4_K matrices
    // an equal distance apart (the loader put all layers' q/k/v in one allocation), they run as ONE batched GEMM,
    // whole K per workgroup, and one kernel norms, rotates and scatters all layers' results: 2 launches per 16
    // columns instead of 4 per layer.
    bool layers_batched = fast && c.n_layers >= 2 && c.n_layers <= 16 && H % DFL_QK_K == 0 && s->pk_layers;
    size_t w_stride = 0;
    if (layers_batched) {
        const dflash_draft_layer &L0 = head->layers[0];
        const bool tiled0 = L0.wk.type == DFLASH_TYPE_Q4_K_TILED;
        layers_batched = (L0.wk.type == DFLASH_TYPE_Q4_K || tiled0) && (!tiled0 || (2 * kv_dim) % 256 == 0);
        w_stride = static_cast<size_t>(static_cast<const uint8_t *>(head->layers[1].wk.data) - static_cast<const uint8_t *>(L0.wk.data));
        for (int il = 0; il < c.n_layers && layers_batched; il++) {
            const dflash_draft_layer &L = head->layers[il];
            layers_batched = L.wk.type == L0.wk.type && adjacent(L.wk, kv_dim, L.wv, H) && head->layers[1].wk.data > L0.wk.data &&
                             static_cast<const uint8_t *>(L.wk.data) == static_cast<const uint8_t *>(L0.wk.data) + il * w_stride;
        }
        layers_batched = layers_batched && w_stride % 16 == 0;
    }
    if (layers_batched) {
        CtxKvNorms norms = {};
        for (int il = 0; il < c.n_layers; il++) norms.k_norm[il] = head->layers[il].k_norm;
        const bool tiled = head->layers[0].wk.type == DFLASH_TYPE_Q4_K_TILED;
        for (int64_t c0 = s->kv_ready; c0 < s->ctx_len; c0 += 16) {
            const int m = static_cast<int>(std::min<int64_t>(16, s->ctx_len - c0));
            if ((rc = dfl_gemm_q4k_batched(ctx, head->layers[0].wk.data, w_stride, nullptr, s->layer_ids, s->n_layers_dev, c.n_layers,
                                           s->ctx_h + c0 * H, DFLASH_TYPE_F32, 0, s->pk_layers, DFLASH_TYPE_F32, static_cast<size_t>(16) * 2 * kv_dim, H,
                                           2 * static_cast<int64_t>(kv_dim), m, 1, nullptr, nullptr, tiled ? 1 : 0, st)))
                return rc;
            ctx_kv_finish_kernel<<<dim3(2 * c.n_kv, m, c.n_layers), 64, 0, st>>>(
                s->pk_layers, static_cast<int>(kv_dim), norms, s->k_ctx, s->v_ctx, static_cast<size_t>(s->capacity) * kv_dim, s->k16,
                s->vt16, static_cast<size_t>(s->cap16) * kv_dim, s->cap16, s->pos_ctx + c0, c0, c.n_kv, hd, c.eps, c.rope_theta);
        }
    }
    for (int il = 0; il < c.n_layers && !layers_batched; il++) {
        const dflash_draft_layer &L = head->layers[il];
        float *kc = s->k_ctx + il * static_cast<size_t>(s->capacity) * kv_dim;
        float *vc = s->v_ctx + il * static_cast<size_t>(s->capacity) * kv_dim;
        _Float16 *k16 = s->k16 + il * static_cast<size_t>(s->cap16) * kv_dim;
        _Float16 *vt16 = s->vt16 + il * static_cast<size_t>(s->cap16) * kv_dim;
        // context K/V for the delta only, normed and rotated at the columns' own positions
        for (int64_t c0 = s->kv_ready; c0 < s->ctx_len; c0 += 16) {
            const int m = static_cast<int>(std::min<int64_t>(16, s->ctx_len - c0));
            // wk and wv adjacent: one GEMM into pk[m][2 kv_dim]; K is rotated out of it into the context
            // cache, V is copied out of it by the mirror kernel
            const bool kv_packed = fast && adjacent(L.wk, kv_dim, L.wv, H);
            if (kv_packed) {
                if ((rc = gemm(ctx, L.wk, s->ctx_h + c0 * H, s->pk, H, 2 * kv_dim, m, st))) return rc;
            } else {
                if ((rc = gemm(ctx, L.wk, s->ctx_h + c0 * H, kc + c0 * kv_dim, H, kv_dim, m, st))) return rc;
                if ((rc = gemm(ctx, L.wv, s->ctx_h + c0 * H, vc + c0 * kv_dim, H, kv_dim, m, st))) return rc;
            }
            qk_norm_rope_kernel<<<dim3(c.n_kv, m), 64, 0, st>>>(nullptr, 0, kv_packed ? s->pk : kc + c0 * kv_dim,
                                                               kv_packed ? 2 * kv_dim : kv_dim, nullptr, kc + c0 * kv_dim, nullptr,
                                                               L.k_norm, nullptr, s->pos_ctx + c0, 0, c.n_kv, hd, c.eps,
                                                               c.rope_theta, nullptr, 0, nullptr, 0);
            if (fast)
                kv_to_f16_kernel<<<dim3(blocks_for(kv_dim), m), 256, 0, st>>>(
                    kc + c0 * kv_dim, kv_packed ? s->pk + kv_dim : vc + c0 * kv_dim, kv_packed ? 2 * kv_dim : kv_dim, k16, vt16,
                    static_cast<int>(kv_dim), s->cap16, c0, kv_packed ? vc + c0 * kv_dim : nullptr);
        }
    }
    DFL_HIP_CHECK(ctx, hipGetLastError());
    s->ctx_h_ready = s->ctx_len;
    s->kv_ready = s->ctx_len;
    return DFLASH_OK;
}

}  // namespace

int32_t dflash_draft_session_selector_inputs(dflash_ctx *ctx, const dflash_draft_session *s, int32_t *topk_ids,
                                             float *topk_vals, float *sel_h, dflash_stream_t stream) {
    if (!ctx) return DFLASH_ERR_INVALID_INPUT;
    if (!s) return dfl_fail(ctx, DFLASH_ERR_INVALID_INPUT, "selector_inputs: null session");
    if (!s->sel_h) return dfl_fail(ctx, DFLASH_ERR_STATE, "selector_inputs: the session's drafter has no selector");
    hipStream_t st = static_cast<hipStream_t>(stream);
    const size_t n = s->cfg.block_size;
    if (topk_ids) DFL_HIP_CHECK(ctx, hipMemcpyAsync(topk_ids, s->topk_ids, n * 16 * sizeof(int32_t), hipMemcpyDeviceToDevice, st));
    if (topk_vals) DFL_HIP_CHECK(ctx, hipMemcpyAsync(topk_vals, s->topk_vals, n * 16 * sizeof(float), hipMemcpyDeviceToDevice, st));
    if (sel_h)
        DFL_HIP_CHECK(ctx, hipMemcpyAsync(sel_h, s->sel_h, n * s->cfg.selector_rank * sizeof(float), hipMemcpyDeviceToDevice, st));
    return DFLASH_OK;
}

int32_t dflash_draft_prepare_ctx(dflash_ctx *ctx, const dflash_draft_head *head, dflash_draft_session *s, dflash_stream_t stream) {
    if (!ctx) return DFLASH_ERR_INVALID_INPUT;
    if (!head || !s) return dfl_fail(ctx, DFLASH_ERR_INVALID_INPUT, "draft_prepare_ctx: null argument");
    if (const int32_t rc_ = head_tensors_checked(ctx, head)) return rc_;
    if (memcmp(&head->cfg, &s->cfg, sizeof(head->cfg)) != 0)
        return dfl_fail(ctx, DFLASH_ERR_STATE, "draft_prepare_ctx: session/head shape mismatch");
    return draft_prepare(ctx, head, s, s->contiguous && head->cfg.n_q / head->cfg.n_kv <= 16, static_cast<hipStream_t>(stream));
}

namespace {
int32_t draft_block_impl(dflash_ctx *ctx, const dflash_model *target, const dflash_draft_head *head, dflash_draft_session *s,
                         int32_t carry, int32_t mask_token, int64_t noise_start, int32_t *draft_argmax, float *draft_logits,
                         int32_t *argmax_host, dflash_stream_t stream, bool skip_selector_walk);
}

int32_t dflash_draft_block(dflash_ctx *ctx, const dflash_model *target, const dflash_draft_head *head,
                           dflash_draft_session *s, int32_t carry, int32_t mask_token, int64_t noise_start,
                           int32_t *draft_argmax, float *draft_logits, int32_t *argmax_host, dflash_stream_t stream) {
    return draft_block_impl(ctx, target, head, s, carry, mask_token, noise_start, draft_argmax, draft_logits, argmax_host, stream,
                            false);
}

namespace {

// skip_selector_walk (DFlash-2 heads): stop after the top-16 candidates and the selector gate are in
// the session's buffers; the caller walks the lattice itself (the sampled walk of a speculative step).
int32_t draft_block_impl(dflash_ctx *ctx, const dflash_model *target, const dflash_draft_head *head, dflash_draft_session *s,
                         int32_t carry, int32_t mask_token, int64_t noise_start, int32_t *draft_argmax, float *draft_logits,
                         int32_t *argmax_host, dflash_stream_t stream, bool skip_selector_walk) {
    if (!ctx) return DFLASH_ERR_INVALID_INPUT;
    if (!target || !head || !s) return dfl_fail(ctx, DFLASH_ERR_INVALID_INPUT, "draft_block: null argument");
    if (const int32_t rc_ = model_tensors_checked(ctx, target)) return rc_;
    if (const int32_t rc_ = head_tensors_checked(ctx, head)) return rc_;
    const dflash_draft_cfg &c = head->cfg;
    if (memcmp(&c, &s->cfg, sizeof(c)) != 0) return dfl_fail(ctx, DFLASH_ERR_STATE, "draft_block: session/head shape mismatch");
    if (c.hidden != target->cfg.hidden) return dfl_fail(ctx, DFLASH_ERR_BAD_SHAPE, "draft_block: drafter and target hidden sizes differ");
    const int V = target->cfg.vocab;
    if (V != s->vocab) return dfl_fail(ctx, DFLASH_ERR_STATE, "draft_block: vocabulary mismatch");
    if (carry < 0 || carry >= V || mask_token < 0 || mask_token >= V)
        return dfl_fail(ctx, DFLASH_ERR_INVALID_TOKEN, "draft_block: carry %d / mask %d outside vocabulary %d", carry, mask_token, V);
    hipStream_t st = static_cast<hipStream_t>(stream);
    const int N = c.block_size, H = c.hidden, hd = c.head_dim;
    const size_t q_dim = static_cast<size_t>(c.n_q) * hd, kv_dim = static_cast<size_t>(c.n_kv) * hd;
    const size_t feat = static_cast<size_t>(c.n_taps) * H;
    int32_t rc;
    // MFMA attention over the f16 mirror when context column i sits at position i and the block
    // starts at position ctx_len (the generation loop's case); else the general f32 kernel.  The
    // mirror is only kept current while that holds, so leaving the fast path is final.
    const bool fast = s->contiguous && noise_start == s->ctx_len && c.n_q / c.n_kv <= 16;
    if (!fast) s->contiguous = false;
    const bool conv = c.conv_kernel_size > 0;
    const int64_t conv_dyn_dim = conv ? static_cast<int64_t>(2) * c.conv_kernel_size * (H / c.conv_group_size) : 0;
    if (conv)
        for (int il = 0; il < c.n_layers; il++)
            if (!head->layers[il].conv_attn_proj.data || !head->layers[il].conv_ffn_proj.data || !head->layers[il].conv_attn_base ||
                !head->layers[il].conv_ffn_base)
                return dfl_fail(ctx, DFLASH_ERR_INVALID_INPUT, "draft_block: layer %d lacks its convolution tensors", il);
    if (c.selector_rank > 0 && (!head->selector_hidden.data || !head->selector_predecessor.data || !head->selector_successor.data))
        return dfl_fail(ctx, DFLASH_ERR_INVALID_INPUT, "draft_block: the head lacks its selector tensors");

    // phase 1 and the context K/V of the new columns (a no-op if dflash_draft_prepare_ctx ran)
    if ((rc = draft_prepare(ctx, head, s, fast, st))) return rc;
    // phase 2: noise embedding
    Int16Args ids_arg = {}, pos_arg = {};
    for (int i = 0; i < N; i++) {
        ids_arg.v[i] = i == 0 ? carry : mask_token;
        pos_arg.v[i] = static_cast<int32_t>(noise_start + i);
    }
    set_ids_pos_kernel<<<1, 64, 0, st>>>(ids_arg, pos_arg, N, s->ids, s->pos, nullptr, 0);
    float *lg = draft_logits ? draft_logits : s->logits;
    int32_t *am = draft_argmax ? draft_argmax : s->argmax;
    // Everything from the noise embedding to the argmax, on stream `st`: the launches depend on the call only through
    // device memory (ids, pos; the attention reads the context length from pos[0]) - except the DFlash-2 selector
    // walk, which takes the carry by value - so they can be captured once and replayed.
    auto enqueue = [&](hipStream_t st) -> int32_t {
    int32_t rc;
    if ((rc = embed_rows(ctx, target->token_embd, s->ids, N, H, s->x, st))) return rc;

    const float *pending_resid = nullptr;
    // DFlash-2: the side-1 convolution of a sublayer's output is what gets added to the residual; the norm kernel that
    // adds it computes it on the way (rms_norm_kernel's ConvResid), unless the width is one that kernel keeps no row in
    // registers for (then a launch of dflash2_conv_kernel comes first, as for the side-0 convolutions)
    const bool conv_in_norm = conv && H <= 8192 && H % 4 == 0;
    ConvResid pending_conv;
    for (int il = 0; il < c.n_layers; il++) {
        const dflash_draft_layer &L = head->layers[il];
        float *kc = s->k_ctx + il * static_cast<size_t>(s->capacity) * kv_dim;
        float *vc = s->v_ctx + il * static_cast<size_t>(s->capacity) * kv_dim;
        _Float16 *k16 = s->k16 + il * static_cast<size_t>(s->cap16) * kv_dim;
        _Float16 *vt16 = s->vt16 + il * static_cast<size_t>(s->cap16) * kv_dim;
        // the previous layer's second residual (x += ffn output) is folded into this norm
        // (in a DFlash-2 layer the side-0 convolution sits between the norm and the projection: it writes the fragment-order rows)
        const LayerXf xk = layer_xf(ctx, L, fast && s->pk != nullptr, H, static_cast<int64_t>(q_dim), static_cast<int64_t>(kv_dim), c.ffn, true);
        // (DFlash-2: the norm's fragment-order rows are for the coefficient projection when that is a one-launch product;
        // the convolution then writes q/k/v's over them, later in the stream)
        const int cp_attn = conv && fast ? dfl_whole_kind(ctx, L.conv_attn_proj.type, H, conv_dyn_dim, 0) : DFL_XF_NONE;
        const int cp_ffn = conv && fast ? dfl_whole_kind(ctx, L.conv_ffn_proj.type, H, conv_dyn_dim, 0) : DFL_XF_NONE;
        const int norm1_kind = conv ? cp_attn : xk.qkv;
        rms_norm_kernel<<<N, 256, 0, st>>>(s->x, pending_resid, L.attn_norm, s->cur, H, c.eps, nullptr, nullptr,
                                           norm1_kind ? s->xf_cur : nullptr, norm1_kind, 0, pending_conv);
        // DFlash-2 attention convolution (metal_dflash.rs:16210-16262): the dynamic coefficients come
        // from the normed input and serve both sides; q/k/v read the side-0 result
        const float *attn_src = s->cur;
        if (conv) {
            rc = cp_attn ? dfl_gemm_whole(ctx, L.conv_attn_proj.type, L.conv_attn_proj.data, s->xf_cur, s->conv_dyn, H, conv_dyn_dim, N, 0,
                                          nullptr, DFL_XF_NONE, st)
                         : gemm(ctx, L.conv_attn_proj, s->cur, s->conv_dyn, H, conv_dyn_dim, N, st);
            if (rc) return rc;
            if ((rc = dfl_dflash2_conv(ctx, s->cur, s->conv_dyn, L.conv_attn_base, s->conv_buf, N, H, c.conv_kernel_size,
                                       c.conv_group_size, 0, st, xk.qkv ? s->xf_cur : nullptr, xk.qkv)))
                return rc;
            attn_src = s->conv_buf;
        }
        bool packed;  // only on the fast path: the general attention kernel reads V dense
        if ((rc = gemm_qkv(ctx, L.wq, L.wk, L.wv, attn_src, s->q, s->k, s->v, s->pk, fast, &packed, H, q_dim, kv_dim, N, st, s->xf_cur, xk.qkv)))
            return rc;
        const int64_t tot = q_dim + 2 * kv_dim;
        if (fast) {
            // the block's own K (normed, rotated) and V go behind the context in the f16 mirror, written by the
            // same kernel (positions pos[i] = ctx_len + i on this path); one MFMA pass over context and block
            qk_norm_rope_kernel<<<dim3(c.n_q + 2 * c.n_kv, N), 64, 0, st>>>(
                packed ? s->pk : s->q, packed ? tot : q_dim, packed ? s->pk + q_dim : s->k, packed ? tot : kv_dim, s->q, s->k,
                L.q_norm, L.k_norm, k16, s->pos, c.n_q, c.n_kv, hd, c.eps, c.rope_theta, packed ? s->pk + q_dim + kv_dim : s->v,
                packed ? tot : kv_dim, vt16, s->cap16);
            // (under capture the context length is pos[0], read on the device: the launches then serve every context
            // of the bucket; chunking, and so the result, is the same either way)
            if ((rc = dfl_attn_block(ctx, s->q, DFLASH_TYPE_F32, k16, vt16, 1, s->ctx_len, N, c.n_q, c.n_kv, hd, s->cap16,
                                     1.0f / sqrtf(static_cast<float>(hd)), s->attn, st, c.causal ? 0 : 1,
                                     L.is_swa ? static_cast<int64_t>(c.swa_window) : 0, ctx->capturing ? s->pos : nullptr,
                                     xk.wo ? s->xf_attn : nullptr, xk.wo)))
                return rc;
        } else {
            qk_norm_rope_kernel<<<dim3(c.n_q + c.n_kv, N), 64, 0, st>>>(s->q, q_dim, s->k, kv_dim, s->q, s->k, L.q_norm, L.k_norm,
                                                                     nullptr, s->pos, c.n_q, c.n_kv, hd, c.eps, c.rope_theta,
                                                                     nullptr, 0, nullptr, 0);
            draft_attn_kernel<<<dim3(c.n_q, N), 64, 0, st>>>(s->q, kc, vc, s->k, s->v, s->pos_ctx, static_cast<int>(s->ctx_len),
                                                            N, c.n_q, c.n_kv, hd, static_cast<int>(noise_start), c.causal,
                                                            L.is_swa ? static_cast<int>(c.swa_window) : 0, s->attn);
        }
        if (fast && xk.wo)  // (only the MFMA attention writes its rows in fragment order)
            rc = dfl_gemm_whole(ctx, L.wo.type, L.wo.data, s->xf_attn, s->mix, static_cast<int64_t>(q_dim), H, N, 0, nullptr, DFL_XF_NONE, st);
        else
            rc = gemm(ctx, L.wo, s->attn, s->mix, q_dim, H, N, st);
        if (rc) return rc;
        // residual 1 (x += attn_output; DFlash-2: its side-1 convolution, same coefficients, :16795-16820),
        // folded into the norm that follows
        const float *resid = s->mix;
        ConvResid resid_conv;
        if (conv_in_norm) {
            resid_conv = ConvResid{s->conv_dyn, L.conv_attn_base, c.conv_kernel_size, c.conv_group_size};
        } else if (conv) {
            if ((rc = dflash_dflash2_conv(ctx, s->mix, s->conv_dyn, L.conv_attn_base, s->conv_buf, N, H, c.conv_kernel_size,
                                          c.conv_group_size, 1, st)))
                return rc;
            resid = s->conv_buf;
        }
        const int norm2_kind = conv ? cp_ffn : xk.gate_up;
        rms_norm_kernel<<<N, 256, 0, st>>>(s->x, resid, L.post_norm, s->cur, H, c.eps, nullptr, nullptr,
                                           norm2_kind ? s->xf_cur : nullptr, norm2_kind, 0, resid_conv);
        const float *ffn_src = s->cur;
        if (conv) {  // the FFN pair (:16836-16885, 17003-17022)
            rc = cp_ffn ? dfl_gemm_whole(ctx, L.conv_ffn_proj.type, L.conv_ffn_proj.data, s->xf_cur, s->conv_dyn, H, conv_dyn_dim, N, 0,
                                         nullptr, DFL_XF_NONE, st)
                        : gemm(ctx, L.conv_ffn_proj, s->cur, s->conv_dyn, H, conv_dyn_dim, N, st);
            if (rc) return rc;
            if ((rc = dfl_dflash2_conv(ctx, s->cur, s->conv_dyn, L.conv_ffn_base, s->conv_buf, N, H, c.conv_kernel_size,
                                       c.conv_group_size, 0, st, xk.gate_up ? s->xf_cur : nullptr, xk.gate_up)))
                return rc;
            ffn_src = s->conv_buf;
        }
        const int down_kind = xk.gate_up ? xk.down : DFL_XF_NONE;  // fragment-order rows only from the gate/up launch's epilogue
        if ((rc = gemm_gate_up(ctx, L.gate, L.up, ffn_src, s->g, s->u, s->pk, H, c.ffn, N, st, s->xf_cur, xk.gate_up, s->xf_g, down_kind)))
            return rc;
        if (down_kind)
            rc = dfl_gemm_whole(ctx, L.down.type, L.down.data, s->xf_g, s->mix, c.ffn, H, N, 0, nullptr, DFL_XF_NONE, st);
        else
            rc = gemm(ctx, L.down, s->g, s->mix, c.ffn, H, N, st);
        if (rc) return rc;
        resid = s->mix;
        pending_conv = ConvResid();
        if (conv_in_norm) {
            pending_conv = ConvResid{s->conv_dyn, L.conv_ffn_base, c.conv_kernel_size, c.conv_group_size};
        } else if (conv) {
            if ((rc = dflash_dflash2_conv(ctx, s->mix, s->conv_dyn, L.conv_ffn_base, s->conv_buf, N, H, c.conv_kernel_size,
                                          c.conv_group_size, 1, st)))
                return rc;
            resid = s->conv_buf;
        }
        pending_resid = resid;  // residual 2: added by the norm that reads x next (same x + r, one launch fewer)
    }
    const int head_kind = dfl_whole_kind(ctx, target->output.type, H, V, 0);
    rms_norm_kernel<<<N, 256, 0, st>>>(s->x, pending_resid, head->output_norm, s->cur, H, c.eps, nullptr, nullptr,
                                       head_kind ? s->xf_cur : nullptr, head_kind, 0, pending_conv);
    if (head_kind)
        rc = dfl_gemm_whole(ctx, target->output.type, target->output.data, s->xf_cur, lg, H, V, N, 0, nullptr, DFL_XF_NONE, st);
    else
        rc = gemm(ctx, target->output, s->cur, lg, H, V, N, st);
    if (rc) return rc;
    if (c.selector_rank > 0) {
        // DFlash-2 tail (:17098-17130, select_draft_path :17176-17251): the 16 best candidates of every
        // row, the selector gate W_h . h of the output-normed hidden, and the predecessor-conditioned
        // walk, all on the device
        if ((rc = dflash_top16(ctx, lg, N, V, V, s->topk_ids, s->topk_vals, st))) return rc;
        if ((rc = gemm(ctx, head->selector_hidden, s->cur, s->sel_h, H, c.selector_rank, N, st))) return rc;
        if (!skip_selector_walk &&
            (rc = dflash_select_draft_path(ctx, &head->selector_predecessor, &head->selector_successor, c.selector_rank,
                                           c.selector_top_k, carry, N, s->topk_ids, s->topk_vals, s->sel_h, am, nullptr, st)))
            return rc;
    } else if ((rc = dflash_argmax_greedy(ctx, lg, N, V, V, am, st))) {
        return rc;
    }
    return DFLASH_OK;
    };  // enqueue

    // Graph replay (off by default; DFLASH_DRAFT_GRAPH=1 or dflash_ctx_set_draft_graphs(ctx, 1) turn it on): a block is
    // about 80 launches of 4..8 us kernels.  Second call with the same key captures, later ones replay.  Measured on
    // the 5-layer drafter of the end-to-end configuration: 0.79 ms per block replayed against 0.77 ms launched one by
    // one - the block is bound by the kernels' own dependent-launch latency on the GPU, not by the host's enqueueing -
    // so it stays off, like the verify's.  Not for a walk that takes the carry by value, not on the
    // general-attention path (its launches depend on the context length), not under kernel timers.
    const bool walk_by_value = c.selector_rank > 0 && !skip_selector_walk;
    const bool use_graph = ctx->draft_graphs && fast && !walk_by_value && !ctx->timing && ctx->gstream;
    uint64_t key = 0;
    if (use_graph) {
        key = hash_model(target);
        const uintptr_t ptrs[6] = {reinterpret_cast<uintptr_t>(head->layers), reinterpret_cast<uintptr_t>(head->fc.data),
                                   reinterpret_cast<uintptr_t>(head->output_norm), reinterpret_cast<uintptr_t>(lg),
                                   reinterpret_cast<uintptr_t>(am), static_cast<uintptr_t>(skip_selector_walk)};
        key = hash_bytes(ptrs, sizeof(ptrs), key);
        const int64_t bucket = dfl_attn_bucket(s->ctx_len + c.block_size);  // (see dfl_attn_block)
        key = hash_bytes(&bucket, sizeof(bucket), key);
        for (int il = 0; il < c.n_layers; il++) {
            const dflash_draft_layer &L = head->layers[il];
            const uintptr_t lp[9] = {reinterpret_cast<uintptr_t>(L.wq.data), reinterpret_cast<uintptr_t>(L.wk.data),
                                     reinterpret_cast<uintptr_t>(L.wv.data), reinterpret_cast<uintptr_t>(L.wo.data),
                                     reinterpret_cast<uintptr_t>(L.gate.data), reinterpret_cast<uintptr_t>(L.up.data),
                                     reinterpret_cast<uintptr_t>(L.down.data), static_cast<uintptr_t>(L.wq.type),
                                     static_cast<uintptr_t>(L.is_swa)};
            key = hash_bytes(lp, sizeof(lp), key);
        }
    }
    auto exec_it = use_graph ? s->graphs.find(key) : s->graphs.end();
    if (use_graph && exec_it == s->graphs.end() && s->graph_seen.size() > 64) s->graph_seen.clear();
    if (use_graph && exec_it == s->graphs.end() && s->graphs.size() < 8 && s->graph_seen[key]++ >= 1) {
        hipGraph_t graph = nullptr;
        DFL_HIP_CHECK(ctx, hipStreamBeginCapture(ctx->gstream, hipStreamCaptureModeThreadLocal));
        ctx->capturing = true;
        rc = enqueue(ctx->gstream);
        ctx->capturing = false;
        const hipError_t end = hipStreamEndCapture(ctx->gstream, &graph);
        if (rc) {
            if (graph) (void)hipGraphDestroy(graph);
            return rc;
        }
        DFL_HIP_CHECK(ctx, end);
        hipGraphExec_t exec = nullptr;
        const hipError_t inst = hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0);
        (void)hipGraphDestroy(graph);
        DFL_HIP_CHECK(ctx, inst);
        exec_it = s->graphs.emplace(key, exec).first;
    }
    if (exec_it != s->graphs.end()) {
        DFL_HIP_CHECK(ctx, hipEventRecord(ctx->g_in, st));
        DFL_HIP_CHECK(ctx, hipStreamWaitEvent(ctx->gstream, ctx->g_in, 0));
        DFL_HIP_CHECK(ctx, hipGraphLaunch(exec_it->second, ctx->gstream));
        s->graph_replays++;
        DFL_HIP_CHECK(ctx, hipEventRecord(ctx->g_out, ctx->gstream));
        DFL_HIP_CHECK(ctx, hipStreamWaitEvent(st, ctx->g_out, 0));
    } else if ((rc = enqueue(st))) {
        return rc;
    }
    DFL_HIP_CHECK(ctx, hipGetLastError());
    // watermarks advance only once everything was enqueued without error (metal_dflash.rs:17143-17150)
    s->ctx_h_ready = s->ctx_len;
    s->kv_ready = s->ctx_len;
    if (argmax_host) {
        DFL_HIP_CHECK(ctx, hipMemcpyAsync(ctx->pinned, am, N * sizeof(int32_t), hipMemcpyDeviceToHost, st));
        DFL_HIP_CHECK(ctx, hipStreamSynchronize(st));
        memcpy(argmax_host, ctx->pinned, N * sizeof(int32_t));
    }
    return DFLASH_OK;
}

}  // namespace

int32_t dflash_accept_greedy(const int32_t *verify_input, const int32_t *verify_argmax, int32_t n, int64_t budget,
                             const int32_t *stop_ids, int32_t n_stop, dflash_accept_decision *out) {
    if (!verify_input || !verify_argmax || !out || n < 1 || n > 16 || budget < 0 || (n_stop > 0 && !stop_ids))
        return DFLASH_ERR_INVALID_INPUT;
    auto is_stop = [&](int32_t t) {
        for (int i = 0; i < n_stop; i++)
            if (stop_ids[i] == t) return true;
        return false;
    };
    memset(out, 0, sizeof(*out));
    out->err_row = -1;
    out->err_index = -1;
    if (is_stop(verify_input[0]) || budget == 0) {  // terminal anchor (accept.rs:131-145)
        out->stop_reason = is_stop(verify_input[0]) ? DFLASH_STOP_EOS : DFLASH_STOP_TOKEN_LIMIT;
        return DFLASH_OK;
    }
    int a = 0;
    for (;;) {
        if (a == n - 1) {
            out->carry_kind = DFLASH_CARRY_BONUS;
            out->carry_token = verify_argmax[a];
            break;
        }
        const int32_t draft = verify_input[a + 1];
        if (draft != verify_argmax[a]) {
            out->carry_kind = DFLASH_CARRY_CORRECTION;
            out->carry_token = verify_argmax[a];
            break;
        }
        out->accepted_drafts[a++] = draft;
        if (is_stop(draft)) {
            out->stop_reason = DFLASH_STOP_EOS;
            break;
        }
        if (a == budget) {
            out->stop_reason = DFLASH_STOP_TOKEN_LIMIT;
            break;
        }
    }
    out->n_accepted = a;
    out->retain_input_count = 1 + a - (out->stop_reason != DFLASH_STOP_NONE ? 1 : 0);
    return DFLASH_OK;
}

namespace {

double ms_since(std::chrono::steady_clock::time_point t0) {
    return std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - t0).count();
}

// Margin-guarded exact fallback of the greedy accept (qwen/dflash.rs:859-1057): when a committed
// row's packed top-2 gap is under the margin, roll the KV back and replay token by token.
int32_t margin_fallback(dflash_ctx *ctx, const dflash_model *target, dflash_session *sess, const int32_t *taps, int n_taps,
                        const int32_t *verify_input, int n_eff, int64_t pos, const dflash_step_cfg *cfg, int64_t budget,
                        const int32_t *stop_ids, int n_stop, dflash_step_result *res, hipStream_t st) {
    dflash_accept_decision &d = res->decision;
    if (d.retain_input_count == 0 && d.n_accepted == 0 && d.carry_kind == DFLASH_CARRY_NONE) return DFLASH_OK;  // anchor stop
    int n_accepted = d.n_accepted;
    int first_flagged = -1;
    for (int i = 0; i <= n_accepted && i < n_eff; i++) {
        const float g = res->verify_gap[i];
        if (!(std::isfinite(g) && g >= cfg->fallback_margin)) {
            first_flagged = i;
            break;
        }
    }
    if (first_flagged < 0) return DFLASH_OK;
    auto is_stop = [&](int32_t t) {
        for (int i = 0; i < n_stop; i++)
            if (stop_ids[i] == t) return true;
        return false;
    };
    res->fallback_ran = 1;
    int replay_start = cfg->fallback_partial ? first_flagged : 0;
    int32_t rc = dflash_restore(ctx, sess, pos, n_eff, replay_start);
    if (rc) return rc;
    const int packed_terminal = d.stop_reason;
    const size_t slot = static_cast<size_t>(std::max(n_taps, 1)) * target->cfg.hidden;
    int32_t targets[17];
    int accepted = 0, terminal = DFLASH_STOP_NONE, n_targets = 0;
    for (;;) {
        const bool partial = replay_start > 0;
        accepted = replay_start;
        terminal = replay_start == n_accepted ? packed_terminal : DFLASH_STOP_NONE;
        n_targets = replay_start;
        for (int i = 0; i < replay_start; i++) targets[i] = res->verify_argmax[i];
        int escalate = 0, rows = 0;
        auto replay_row = [&](int row, int32_t token, int32_t *arg, float *gap) -> int32_t {
            int32_t r = dflash_verify_block(ctx, target, sess, &token, 1, pos + row, taps, n_taps, nullptr, nullptr,
                                            n_taps ? sess->hidden + row * slot : nullptr, nullptr, arg, st);
            if (r) return r;
            if (hipMemcpy(gap, sess->gap, sizeof(float), hipMemcpyDeviceToHost) != hipSuccess)
                return dfl_fail(ctx, DFLASH_ERR_HIP, "fallback: gap read-back failed");
            rows++;
            return DFLASH_OK;
        };
        auto near_tie = [&](float g) { return !(std::isfinite(g) && g >= cfg->fallback_partial_min_gap); };
        if (terminal == DFLASH_STOP_NONE) {
            int32_t t;
            float g;
            if ((rc = replay_row(replay_start, verify_input[replay_start], &t, &g))) return rc;
            if (partial && near_tie(g)) {
                escalate = 1;
            } else {
                targets[n_targets++] = t;
                for (int i = replay_start; i + 1 < n_eff; i++) {
                    const int32_t draft = verify_input[i + 1];
                    if (draft != targets[i]) break;
                    accepted++;
                    if (is_stop(draft)) {
                        terminal = DFLASH_STOP_EOS;
                        break;
                    }
                    if (accepted == budget) {
                        terminal = DFLASH_STOP_TOKEN_LIMIT;
                        break;
                    }
                    if ((rc = replay_row(i + 1, draft, &t, &g))) return rc;
                    if (partial && near_tie(g)) {
                        escalate = 1;
                        break;
                    }
                    targets[n_targets++] = t;
                }
            }
        }
        res->fallback_rows_replayed += rows;
        if (!escalate) break;
        res->fallback_escalations++;
        const int64_t done = dflash_session_kv_n_pos(sess) - pos;
        if (done > 0 && (rc = dflash_restore(ctx, sess, pos, static_cast<int32_t>(done), 0))) return rc;
        replay_start = 0;
    }
    res->fallback_rows_kept = replay_start;
    for (int i = 0; i < n_targets; i++) res->verify_argmax[i] = targets[i];
    memset(&d, 0, sizeof(d));
    d.err_row = -1;
    d.err_index = -1;
    d.n_accepted = accepted;
    for (int i = 0; i < accepted; i++) d.accepted_drafts[i] = verify_input[i + 1];
    d.stop_reason = terminal;
    d.retain_input_count = terminal != DFLASH_STOP_NONE ? accepted : accepted + 1;
    if (terminal == DFLASH_STOP_NONE) {
        d.carry_kind = accepted == n_eff - 1 ? DFLASH_CARRY_BONUS : DFLASH_CARRY_CORRECTION;
        d.carry_token = targets[accepted];
    }
    return DFLASH_OK;
}

}  // namespace

int32_t dflash_spec_step(dflash_ctx *ctx, const dflash_model *target, const dflash_draft_head *head, dflash_session *sess,
                         dflash_draft_session *dsess, const int32_t *taps, int32_t n_taps, int32_t carry, int64_t position,
                         const dflash_step_cfg *cfg, dflash_sampler *sampler, dflash_sampler *proposal_sampler, int64_t budget,
                         const int32_t *stop_ids, int32_t n_stop, const int32_t *draft_override, dflash_step_result *res,
                         dflash_stream_t stream) {
    if (!ctx) return DFLASH_ERR_INVALID_INPUT;
    if (!target || !head || !sess || !dsess || !cfg || !res || (n_stop > 0 && !stop_ids) || budget < 0)
        return dfl_fail(ctx, DFLASH_ERR_INVALID_INPUT, "spec_step: null or invalid argument");
    if (cfg->sampled_mode != 0 && !sampler) return dfl_fail(ctx, DFLASH_ERR_INVALID_INPUT, "spec_step: sampled mode needs a sampler");
    const bool sampled_drafts = cfg->sampled_mode == 2;
    if (sampled_drafts && (!proposal_sampler || head->cfg.selector_rank <= 0 || draft_override))
        return dfl_fail(ctx, DFLASH_ERR_INVALID_INPUT,
                        "spec_step: sampled drafting needs a selector head and a proposal sampler, and takes no draft override");
    if (n_taps != head->cfg.n_taps || n_taps > sess->n_taps || !taps)
        return dfl_fail(ctx, DFLASH_ERR_BAD_SHAPE, "spec_step: %d tapped layers, the drafter expects %d", n_taps, head->cfg.n_taps);
    hipStream_t st = static_cast<hipStream_t>(stream);
    memset(res, 0, sizeof(*res));
    const int N = head->cfg.block_size;
    res->n_block = N;
    int32_t rc;
    // A failed step commits nothing: whatever phase fails, the target's KV position goes back to where the block
    // started and both samplers to their state on entry, so that the caller can retry (or fall back to a serial
    // step) on the same random stream.  The message of the failing call is kept.
    const dflash_sampler sampler_in = sampler ? *sampler : dflash_sampler{};
    const dflash_sampler proposal_in = proposal_sampler ? *proposal_sampler : dflash_sampler{};
    const int64_t kv_in = sess->kv_n_pos;
#define STEP_HIP(expr)                                                                                        \
    do {                                                                                                      \
        const hipError_t e_ = (expr);                                                                         \
        if (e_ != hipSuccess) return undo(dfl_fail(ctx, DFLASH_ERR_HIP, "spec_step: %s", hipGetErrorString(e_))); \
    } while (0)
    auto undo = [&](int32_t status) {
        if (sampler) *sampler = sampler_in;
        if (proposal_sampler) *proposal_sampler = proposal_in;
        sess->kv_n_pos = kv_in;  // stale rows stay in place; the next verify overwrites them
        return status;
    };

    auto t0 = std::chrono::steady_clock::now();
    int32_t prop_counts[16] = {0};
    dflash_weighted_candidate prop_cands[16 * 16];
    if (sampled_drafts) {
        // draft_block_sampled (metal_dflash.rs:17268-17415): the drafter up to its top-16 and selector gate,
        // then the walk that draws every position from softmax(score / T) with the proposal sampler
        if ((rc = draft_block_impl(ctx, target, head, dsess, carry, cfg->mask_token, position, nullptr, nullptr, nullptr, st, true)))
            return undo(rc);
        if ((rc = dflash_select_draft_path_sampled(ctx, &head->selector_predecessor, &head->selector_successor,
                                                   head->cfg.selector_rank, head->cfg.selector_top_k, carry, N, dsess->topk_ids,
                                                   dsess->topk_vals, dsess->sel_h, proposal_sampler, res->draft_tokens, prop_counts,
                                                   prop_cands, st)))
            return undo(rc);
    } else {
        // The drafter's tokens stay on the device and the verify is enqueued right behind the drafter:
        // no host round trip between the two phases, and the GPU does not wait for the host to start
        // launching the verify.  The phases are timed by events on the stream.
        // A prefix-replay step (qwen/dflash.rs:700-712) supplies every draft and skips the drafter, as the
        // reference does; the context columns it leaves pending are taken up by the next draft.
        if (cfg->replay_only) {
            for (int i = 0; i < N - 1; i++)
                if (!draft_override || draft_override[i] < 0)
                    return dfl_fail(ctx, DFLASH_ERR_INVALID_INPUT, "spec_step: a replay-only step needs all %d drafts", N - 1);
        }
        if (!cfg->replay_only &&
            (rc = dflash_draft_block(ctx, target, head, dsess, carry, cfg->mask_token, position, dsess->argmax, nullptr, nullptr, st)))
            return undo(rc);
    }
    const int32_t *verify_input = res->draft_tokens;
    if (sampled_drafts) {
        res->draft_ms = ms_since(t0);
        res->draft_tokens[0] = carry;
        t0 = std::chrono::steady_clock::now();
        if ((rc = dflash_verify_block(ctx, target, sess, verify_input, N, position, taps, n_taps, nullptr, nullptr, sess->hidden,
                                      nullptr, res->verify_argmax, st)))
            return undo(rc);
        STEP_HIP(hipMemcpy(res->verify_gap, sess->gap, N * sizeof(float), hipMemcpyDeviceToHost));
        res->verify_ms = ms_since(t0);
    } else {
        const bool timed = !ctx->timing;  // the per-kernel timers use the same events
        if (timed) STEP_HIP(hipEventRecord(ctx->ev0, st));
        int32_t tokens_in[16];
        tokens_in[0] = carry;
        for (int i = 1; i < N; i++) tokens_in[i] = (draft_override && draft_override[i - 1] >= 0) ? draft_override[i - 1] : -1;
        const double enqueue_draft_ms = ms_since(t0);
        t0 = std::chrono::steady_clock::now();
        if ((rc = verify_block_impl(ctx, target, sess, tokens_in, dsess->argmax, N, position, taps, n_taps, nullptr, nullptr,
                                    sess->hidden, nullptr, nullptr, st)))
            return undo(rc);
        if (timed) STEP_HIP(hipEventRecord(ctx->ev1, st));
        // read back through the context's pinned page, one wait
        int32_t *pin_argmax = static_cast<int32_t *>(ctx->pinned), *pin_draft = pin_argmax + 16;
        float *pin_gap = reinterpret_cast<float *>(pin_argmax + 32);
        void *pinned_dev = nullptr;
        if (hipHostGetDevicePointer(&pinned_dev, ctx->pinned, 0) == hipSuccess && pinned_dev) {
            // (one launch that writes the pinned page directly instead of three copy commands)
            step_readback_kernel<<<1, 64, 0, st>>>(sess->argmax, sess->gap, dsess->argmax, N, static_cast<int32_t *>(pinned_dev));
            STEP_HIP(hipGetLastError());
        } else {
            (void)hipGetLastError();
            STEP_HIP(hipMemcpyAsync(pin_argmax, sess->argmax, N * sizeof(int32_t), hipMemcpyDeviceToHost, st));
            STEP_HIP(hipMemcpyAsync(pin_gap, sess->gap, N * sizeof(float), hipMemcpyDeviceToHost, st));
            STEP_HIP(hipMemcpyAsync(pin_draft, dsess->argmax, N * sizeof(int32_t), hipMemcpyDeviceToHost, st));
        }
        STEP_HIP(hipStreamSynchronize(st));
        memcpy(res->verify_argmax, pin_argmax, N * sizeof(int32_t));
        memcpy(res->verify_gap, pin_gap, N * sizeof(float));
        memcpy(res->draft_tokens, pin_draft, N * sizeof(int32_t));
        const double wall_ms = enqueue_draft_ms + ms_since(t0);
        // the wall time of the two phases, split by the GPU time of the verify
        float verify_gpu_ms = 0.0f;
        if (timed && hipEventElapsedTime(&verify_gpu_ms, ctx->ev0, ctx->ev1) == hipSuccess && verify_gpu_ms < wall_ms) {
            res->verify_ms = verify_gpu_ms;
            res->draft_ms = wall_ms - verify_gpu_ms;
        } else {
            res->draft_ms = enqueue_draft_ms;
            res->verify_ms = wall_ms - enqueue_draft_ms;
        }
        for (int i = 1; i < N; i++) {
            if (tokens_in[i] >= 0) res->draft_tokens[i] = tokens_in[i];
            if (res->draft_tokens[i] < 0 || res->draft_tokens[i] >= target->cfg.vocab) {
                return undo(dfl_fail(ctx, DFLASH_ERR_INVALID_TOKEN, "spec_step: the drafter produced token %d at slot %d (vocabulary %d)",
                                res->draft_tokens[i], i, target->cfg.vocab));
            }
        }
        res->draft_tokens[0] = carry;
    }

    t0 = std::chrono::steady_clock::now();
    if (sampled_drafts) {  // couple_sparse_proposal with the walk's candidate distributions
        // the walk leaves row r's candidates at r * top_k; the decision takes the rows back to back
        const int top_k = head->cfg.selector_top_k;
        int n_packed = 0;
        for (int r = 0; r < N - 1; r++)
            for (int i = 0; i < prop_counts[r]; i++) prop_cands[n_packed++] = prop_cands[r * top_k + i];
        rc = dflash_accept_prefix(ctx, verify_input, N, sess->logits, target->cfg.vocab, 1, N - 1, verify_input + 1, prop_counts,
                                  prop_cands, nullptr, 0.0f, sampler, budget, stop_ids, n_stop, &res->decision, st);
    } else if (cfg->sampled_mode != 0) {
        rc = dflash_accept_prefix(ctx, verify_input, N, sess->logits, target->cfg.vocab, 0, 0, nullptr, nullptr, nullptr,
                                  nullptr, 0.0f, sampler, budget, stop_ids, n_stop, &res->decision, st);
    } else {
        rc = dflash_accept_greedy(verify_input, res->verify_argmax, N, budget, stop_ids, n_stop, &res->decision);
        if (rc) dfl_fail(ctx, rc, "spec_step: greedy accept rejected its input");
    }
    if (rc) return undo(rc);
    res->accept_ms = ms_since(t0);

    if (cfg->sampled_mode == 0 && cfg->fallback_margin > 0.0f) {
        t0 = std::chrono::steady_clock::now();
        if ((rc = margin_fallback(ctx, target, sess, taps, n_taps, verify_input, N, position, cfg, budget, stop_ids, n_stop, res, st)))
            return undo(rc);
        if (res->fallback_ran) res->fallback_ms = ms_since(t0);
    }

    const int n_keep = res->decision.retain_input_count;
    if (n_keep > 0) {  // columns 0..n_keep-1 are the carry and the accepted drafts (qwen/dflash.rs:1066-1084)
        t0 = std::chrono::steady_clock::now();
        int32_t positions[16];
        for (int i = 0; i < n_keep; i++) positions[i] = static_cast<int32_t>(position + i);
        if ((rc = dflash_draft_append_ctx(ctx, dsess, sess->hidden, n_keep, positions, st))) return undo(rc);
        STEP_HIP(hipStreamSynchronize(st));
        res->append_ms = ms_since(t0);
    }
    if (!res->fallback_ran && n_keep < N) {
        t0 = std::chrono::steady_clock::now();
        if ((rc = dflash_restore(ctx, sess, position, N, n_keep))) return undo(rc);
        res->restore_ms = ms_since(t0);
    }
    return DFLASH_OK;
}

#undef STEP_HIP

}  // extern "C"
