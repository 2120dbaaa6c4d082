// Internal declarations shared by the HIP translation units of libdflash_hip.
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <vector>

#include "../../include/dflash_hip.h"

struct dflash_ctx {
    int device = 0;
    char *workspace = nullptr;  // device scratch, owned
    size_t workspace_bytes = 0;
    int n_cu = 256;
    // split-K partial tiles of the Q4_K GEMM (written by the streaming kernel, added up by its reduce kernel)
    void *partials = nullptr;
    int n_partial_wgs = 0;
    // workgroups of a batched (expert) launch; 0 = one per CU.  The pipelined prefill sets it on its lanes' contexts for
    // the duration of a call: an expert workgroup fills a CU's LDS, so launches of different lanes cannot share a CU,
    // and with half the CUs each two of them run side by side, one's start-up and tail under the other's streaming.
    int batch_wgs = 0;
    size_t lds_bytes = 65536;  // LDS available to one workgroup
    char err[512] = {0};
    // per-kernel timers (off by default; when on, timed launches synchronise)
    bool timing = false;
    // Set by a caller inside the library for the duration of one few-row GEMM call on a fused gate | up matrix
    // (2 ffn output rows, ffn a multiple of 16): if the call is split over K, its reduction writes
    // silu(gate) * up to swiglu_out[n_rows][ffn] instead of the sums to Y and sets swiglu_done; if it is not (Y is
    // complete), swiglu_done stays false and the caller applies the activation itself.
    float *swiglu_out = nullptr;
    bool swiglu_done = false;
    hipEvent_t ev0 = nullptr, ev1 = nullptr;
    // start / stop stamps of single dispatches (hipExtLaunchKernelGGL), see DFL_T_KERNEL_*: while `stamping` is on, a stamped
    // launch takes the next event pair of the pool and does not wait; the pairs are read when the timers are queried
    bool stamping = false;
    std::vector<hipEvent_t> stamp_events;  // pairs
    std::vector<int> stamp_slot;           // slot of pair i
    size_t stamps_used = 0;
    double timed_ms[8] = {0};
    int64_t timed_launches[8] = {0};
    // captured-graph replay of the packed verify: a stream of the library's own to capture on and
    // launch into (the caller's may be the legacy default stream, which cannot be captured) and
    // the two events that order it against the caller's stream
    bool graphs = false;
    bool capturing = false;     // the launches being enqueued go into a graph: position-dependent values come from device memory
    bool draft_graphs = false;  // graph replay of the drafter's block forward (measured: no faster than direct launches)
    hipStream_t gstream = nullptr;
    hipEvent_t g_in = nullptr, g_out = nullptr;
    // pinned host staging for the few words a blocking call reads back (a device-to-host copy into pageable
    // memory is staged by the runtime and costs several microseconds each); one page, owned
    void *pinned = nullptr;
    // kernels whose dynamic-LDS limit has already been raised for this context (the attribute is kept per
    // device by the runtime, so the record lives with the context, not in process-wide flags)
    const void *lds_attr_fn[96] = {nullptr};
    size_t lds_attr_bytes[96] = {0};
    int n_lds_attr = 0;
};
enum { DFL_PINNED_BYTES = 8192 };

// Slots of the per-kernel timers.
enum { DFL_T_GEMM = 0, DFL_T_ATTN = 1, DFL_T_ACCEPT = 2, DFL_T_ARGMAX = 3, DFL_T_REDUCE = 4,
       // the tiled Q4_K streaming kernel and its reduction by the device's own start / stop stamps of that one dispatch (what a
       // kernel trace reports as its duration), not by events recorded around the launch (which add the dispatch latency)
       DFL_T_KERNEL_Q4K_TILED = 5, DFL_T_KERNEL_Q4K_REDUCE = 6 };

// Brackets the dominant kernel of a call with events on its stream when timing is on.
// The event pair a stamped launch passes to hipExtLaunchKernelGGL: null pointers while stamping is off.
struct dfl_stamp {
    hipEvent_t start = nullptr, stop = nullptr;
    dfl_stamp(dflash_ctx *ctx, int slot) {
        if (!ctx->stamping) return;
        if (ctx->stamps_used * 2 + 2 > ctx->stamp_events.size()) {
            hipEvent_t a = nullptr, b = nullptr;
            if (hipEventCreate(&a) != hipSuccess || hipEventCreate(&b) != hipSuccess) return;
            ctx->stamp_events.push_back(a);
            ctx->stamp_events.push_back(b);
            ctx->stamp_slot.push_back(slot);
        }
        start = ctx->stamp_events[2 * ctx->stamps_used];
        stop = ctx->stamp_events[2 * ctx->stamps_used + 1];
        ctx->stamp_slot[ctx->stamps_used] = slot;
        ctx->stamps_used++;
    }
};

struct dfl_timed {
    dflash_ctx *ctx;
    hipStream_t st;
    int slot;
    dfl_timed(dflash_ctx *c, hipStream_t s, int k) : ctx(c), st(s), slot(k) {
        if (ctx->timing) (void)hipEventRecord(ctx->ev0, st);
    }
    ~dfl_timed() {
        if (!ctx->timing) return;
        (void)hipEventRecord(ctx->ev1, st);
        (void)hipEventSynchronize(ctx->ev1);
        float ms = 0.0f;
        if (hipEventElapsedTime(&ms, ctx->ev0, ctx->ev1) == hipSuccess) {
            ctx->timed_ms[slot] += ms;
            ctx->timed_launches[slot] += 1;
        }
    }
};

// Records a message on the context and returns `status`.
int32_t dfl_fail(dflash_ctx *ctx, int32_t status, const char *fmt, ...);

#define DFL_HIP_CHECK(ctx, expr)                                                          \
    do {                                                                                  \
        hipError_t e_ = (expr);                                                           \
        if (e_ != hipSuccess)                                                             \
            return dfl_fail((ctx), DFLASH_ERR_HIP, "%s: %s", #expr, hipGetErrorString(e_)); \
    } while (0)

// Makes sure kernel `fn` may be launched with `bytes` of dynamic LDS on the context's device
// (hipFuncAttributeMaxDynamicSharedMemorySize), calling the runtime only the first time.
int32_t dfl_raise_lds_limit(dflash_ctx *ctx, const void *fn, size_t bytes);

// Carves `bytes` (256-aligned) out of the context workspace starting at *offset.
template <typename T>
static inline T *dfl_ws_take(dflash_ctx *ctx, size_t *offset, size_t bytes) {
    size_t start = (*offset + 255) & ~size_t(255);
    if (start + bytes > ctx->workspace_bytes) return nullptr;
    *offset = start + bytes;
    return reinterpret_cast<T *>(ctx->workspace + start);
}

static inline bool dfl_ranges_overlap(const void *a, size_t na, const void *b, size_t nb) {
    const char *pa = static_cast<const char *>(a), *pb = static_cast<const char *>(b);
    return pa < pb + nb && pb < pa + na;
}

enum { DFL_QK_K = 256, DFL_Q4_K_BYTES = 144, DFL_Q6_K_BYTES = 210, DFL_Q8_0_BYTES = 34, DFL_QK8_0 = 32 };

// ---- activations in MFMA fragment order ("XF") -----------------------------------------------------------------
// The hand-off format between a kernel that produces the 16 activation rows of a few-row GEMM and the whole-K GEMM
// kernels (gemm_whole.hip) that consume them: f16, already in the order the consumer's MFMA A operands are read in,
// so that a wave loads a stage's eight fragments with eight coalesced 16-byte loads and no trip through LDS.
// Per super-block b (256 values of K) 512 slots of 16 bytes: slot (t, lane) at byte ((b * 8 + t) * 64 + lane) * 16,
// lane = 16 g + m (m = row), holds row m's eight consecutive values k = 256 b + 8 o + {0,2,1,3,4,6,5,7}[i] (the order
// in which the nibble unpack emits a lane's weights), with octet o = 8 g + t for a Q4_K consumer and
// o = 16 (g >> 1) + 8 (t >> 2) + 4 (g & 1) + (t & 3) for a Q6_K consumer (its quarters interleave).  Rows a producer
// does not write keep whatever the buffer held: a row of the product depends on its own activation row only.
enum { DFL_XF_NONE = 0, DFL_XF_Q4K = 1, DFL_XF_Q6K = 2 };
static inline size_t dfl_xf_bytes(int64_t n_in) { return static_cast<size_t>(n_in / 256) * 8192; }
#ifdef __HIPCC__
// byte offset of the slot of row m's values k0 .. k0 + 7 (k0 a multiple of 8)
__host__ __device__ static inline uint32_t dfl_xf_slot(int kind, int m, int k0) {
    const int b = k0 >> 8, o = (k0 >> 3) & 31;
    int g, t;
    if (kind == DFL_XF_Q6K) {
        const int h = o >> 4, quarter = (o >> 2) & 3;
        g = 2 * h + (quarter & 1);
        t = 4 * (quarter >> 1) + (o & 3);
    } else {
        g = o >> 3;
        t = o & 7;
    }
    return static_cast<uint32_t>(((b * 8 + t) * 64 + 16 * g + m) * 16);
}
__device__ static inline void dfl_xf_store(void *xf, int kind, int m, int k0, float v0, float v1, float v2, float v3, float v4,
                                           float v5, float v6, float v7) {
    typedef _Float16 h8 __attribute__((ext_vector_type(8)));
    const h8 frag = {static_cast<_Float16>(v0), static_cast<_Float16>(v2), static_cast<_Float16>(v1), static_cast<_Float16>(v3),
                     static_cast<_Float16>(v4), static_cast<_Float16>(v6), static_cast<_Float16>(v5), static_cast<_Float16>(v7)};
    *reinterpret_cast<h8 *>(static_cast<uint8_t *>(xf) + dfl_xf_slot(kind, m, k0)) = frag;
}
// Lanes (2 p, 2 p + 1) of a wave hold values i .. i + 3 and i + 4 .. i + 7 of row m (i a multiple of 8 on the even lane):
// the even lane stores the octet.  Every lane of the wave must call it.
__device__ static inline void dfl_xf_store_pair(void *xf, int kind, int m, int i, float a, float b, float c, float d) {
    const float e = __shfl_down(a, 1, 64), f = __shfl_down(b, 1, 64), g = __shfl_down(c, 1, 64), h = __shfl_down(d, 1, 64);
    if ((threadIdx.x & 1) == 0) dfl_xf_store(xf, kind, m, i, a, b, c, d, e, f, g, h);
}
#endif

// Whole-K few-row GEMM over activations in XF order (gemm_whole.hip): y[n_rows][n_out] = x . w^T with every output tile's
// whole K inside one workgroup (its waves split K and add up in LDS in a fixed order): no partial tiles, no second launch.
// dfl_whole_kind: the XF kind a producer must write for this matrix (DFL_XF_NONE: the shape or type does not take
// this path: more than two stages per wave, or more tiles than one round of the chip).  pair_ffn > 0: w is a fused
// gate | up matrix of 2 * pair_ffn rows and the output is silu(gate) * up, [n_rows][pair_ffn]: as f32 in y (may be null)
// and / or as XF of kind y_xf_kind in y_xf (may be null), the activations of the down projection that follows.
int dfl_whole_kind(const dflash_ctx *ctx, int32_t w_type, int64_t n_in, int64_t n_out, int64_t pair_ffn);
int32_t dfl_gemm_whole(dflash_ctx *ctx, int32_t w_type, const void *w, const void *xf, float *y, int64_t n_in, int64_t n_out,
                       int32_t n_rows, int64_t pair_ffn, void *y_xf, int y_xf_kind, hipStream_t stream);
// The same for n_rows_total rows, sixteen to a block (the last one may be shorter): block i's rows are in XF order at
// xf + i * dfl_xf_bytes(n_in), its result at y + i * 16 * n_out (pair mode: 16 * pair_ffn; y_xf + i * dfl_xf_bytes(pair_ffn)).
// The weights are read once and stay in registers while the blocks pass; a row's bits are those of dfl_gemm_whole.
int32_t dfl_gemm_whole_blocks(dflash_ctx *ctx, int32_t w_type, const void *w, const void *xf, float *y, int64_t n_in, int64_t n_out,
                              int32_t n_rows_total, int64_t pair_ffn, void *y_xf, int y_xf_kind, hipStream_t stream);

// dflash_dflash2_conv whose result also goes to y_xf in fragment order (XF; h a multiple of 256), for the whole-K
// projection that reads it.
int32_t dfl_dflash2_conv(dflash_ctx *ctx, const float *x, const float *dyn, const float *base, float *y, int32_t n_tokens, int32_t h,
                         int32_t kernel_size, int32_t group_size, int32_t side, dflash_stream_t stream, void *y_xf, int y_xf_kind);

// Device scratch of the mixture-of-experts FFN (owned by the target session).
struct dfl_moe_scratch {
    float *probs = nullptr;   // [16][n_expert] router logits
    int32_t *sel_e = nullptr; // [16][n_used]
    float *sel_w = nullptr;   // [16][n_used]
    float *sg = nullptr;      // [16] shared-expert gate
    float *act = nullptr;     // [16*n_used][ffn_expert]           (per-slot path)
    float *eo = nullptr;      // [slots][16][hidden]; per-slot path: [16*n_used][hidden]
    float *gate_out = nullptr;  // [slots][16][ffn_expert]: silu(gate) * up of every slot (batched path)
    int32_t *ids = nullptr, *n_distinct = nullptr, *slot_of = nullptr;  // distinct experts, their count, pick -> slot
    float *shared = nullptr;  // [16][hidden]
    float *g = nullptr, *u = nullptr;  // [16][ffn_shared]
};

// x_resid[n][hidden] += moe_ffn(cur[n][hidden]) for one layer; enqueue only.  gate_done: scratch.sg
// already holds sigmoid(cur . shexp_gate) per row (the norm kernel that wrote cur computed it).
// next_norm_w / next_cur / next_done (all or none): the RMSNorm that reads x_resid next may be done
// in the same pass, next_cur = rms_norm(x_resid) * next_norm_w; *next_done says whether it was.
// next_xf / next_xf_kind: where that norm is done here, its rows also go to next_xf in fragment order (XF).
// pre_add / pre_norm_w (both or neither; only where dfl_moe_norm_fusable() holds): the layer's input has not been
// normalised yet, x_resid still lacks pre_add (the attention's output projection), and `cur` is where the normalised rows
// go: cur = rms_norm(x_resid + pre_add) * pre_norm_w, computed inside the router's launch with the shared-expert gate
// (gate_done is then implied); x_resid += pre_add happens where the experts' sum is added.
int32_t dfl_moe_ffn(dflash_ctx *ctx, const dflash_model_cfg &cfg, const dflash_layer &layer, float *cur, int n,
                    const dfl_moe_scratch &scratch, float *x_resid, bool gate_done, const float *next_norm_w,
                    float *next_cur, bool *next_done, hipStream_t stream, const float *pre_add = nullptr,
                    const float *pre_norm_w = nullptr, void *next_xf = nullptr, int next_xf_kind = 0);
bool dfl_moe_norm_fusable(const dflash_ctx *ctx, const dflash_model_cfg &cfg, const dflash_layer &layer, int n);

// The same FFN for the rows of several consecutive 16-row blocks at once (a prompt's prefill): the rows are regrouped
// by expert, so a pass reads every touched expert about once however many blocks there are.  cur holds the layer's
// normalised input and scratch.sg the rows' shared-expert gates (the norm kernel's work); x_resid += experts(cur),
// then cur = rms_norm(x_resid) * next_norm_w, also to next_xf (block b of sixteen rows at
// next_xf + b * next_xf_stride bytes) where next_xf_kind says so.  Every row gets the bits dfl_moe_ffn gives it inside
// its own block.  Takes layers with tiled Q4_K expert stacks and a shared expert of the experts' shape
// (dfl_moe_group_fits); scratch of dfl_moe_group_max_slots(cfg, n_rows) slots.  Enqueue only.
struct dfl_moe_group_scratch {
    float *logits = nullptr;      // [rows][n_expert]
    float *sg = nullptr;          // [rows]
    int32_t *sel_e = nullptr;     // [rows][n_used]
    float *sel_w = nullptr;       // [rows][n_used]
    int32_t *pick_pos = nullptr;  // [rows][n_used]: row of eo that holds the pick's output
    int32_t *ids = nullptr;       // [max_slots]
    int32_t *n_slots = nullptr;
    int32_t *slot_rows = nullptr; // [max_slots][16]
    _Float16 *xg = nullptr;       // [max_slots][16][hidden]
    _Float16 *act = nullptr;      // [max_slots][16][ffn_expert]
    float *eo = nullptr;          // [max_slots][16][hidden]
    int max_slots = 0;
};
int dfl_moe_group_max_slots(const dflash_model_cfg &cfg, int n_rows);
bool dfl_moe_group_fits(const dflash_ctx *ctx, const dflash_model_cfg &cfg, const dflash_layer &layer, int n_rows);
int32_t dfl_moe_ffn_group(dflash_ctx *ctx, const dflash_model_cfg &cfg, const dflash_layer &layer, float *x_resid,
                          float *cur, int n_rows, const dfl_moe_group_scratch &scratch, const float *next_norm_w, void *next_xf,
                          int next_xf_kind, size_t next_xf_stride, hipStream_t stream);

// Residual add + RMSNorm + shared-expert gate + Q8_0 router product of a mixture-of-experts layer as one launch:
// cur[n_rows][hidden] = rms_norm(x + add) * norm_w, gate_out[r] = sigmoid(cur[r] . gate_w),
// logits[n_rows][n_expert] = cur . router_w^T, bit-identical to the norm kernel followed by the few-row GEMM.
// x is left as it is.  dfl_router_norm_fits: whether the shape is one the kernel takes (hidden a multiple of 256, at
// most 2048; every row is a workgroup column of its own, 1..4096 of them); switched off by DFLASH_MOE_FUSED_NORM=0.  Enqueue only.
bool dfl_router_norm_fits(const dflash_ctx *ctx, int32_t router_type, const void *router_w, int64_t hidden, int32_t n_expert,
                          int32_t n_rows);
// The router product alone for any number of rows, sixteen to a workgroup row: logits[n_rows][n_expert] = cur . router_w^T
// with the bits dfl_router_norm (and the few-row GEMM of a Q8_0 router) gives each row.  Same shapes as dfl_router_norm_fits.
int32_t dfl_router_rows(dflash_ctx *ctx, const void *router_w, const float *cur, float *logits, int64_t hidden, int32_t n_expert,
                        int32_t n_rows, hipStream_t stream);
int32_t dfl_router_norm(dflash_ctx *ctx, const void *router_w, const float *x, const float *add, const float *norm_w,
                        const float *gate_w, float eps, float *cur, float *gate_out, float *logits, int64_t hidden,
                        int32_t n_expert, int32_t n_rows, hipStream_t stream);

// dflash_attn_verify_block with the drafter's masks: full_block != 0 lets every row see the whole
// block (non-causal), window > 0 keeps only keys with |distance| < window.  ctx_len_dev != null:
// the context length is read from that device word when the kernels run, so that the call can sit
// in a captured graph that is replayed at other positions.  How the keys are cut into chunks and
// the heads into workgroups depends on dfl_attn_bucket(ctx_len + n_rows) only, and with ctx_len_dev
// the launches are sized for the largest context of that bucket: a captured call stays valid, and
// bit-identical to a direct one, at every context of the bucket it was captured in (a graph key
// must therefore include the bucket).  out_xf / out_xf_kind: the rows [n_rows][n_q * head_dim] also go to out_xf in
// fragment order (XF), for the output projection that reads them.
// Lower bound of the power-of-two range [b, 2 b) that holds n_pos visible positions (at least 256).
inline int64_t dfl_attn_bucket(int64_t n_pos) {
    int64_t b = 256;
    while (2 * b <= n_pos) b *= 2;
    return b;
}
int32_t dfl_attn_block(dflash_ctx *ctx, const void *q, int32_t q_type, const void *k_cache, const void *v_cache,
                       int32_t v_layout, int64_t ctx_len, int32_t n_rows, int32_t n_q, int32_t n_kv, int32_t head_dim,
                       int64_t kv_capacity, float scale, float *out, dflash_stream_t stream, int32_t full_block,
                       int64_t window, const int32_t *ctx_len_dev, void *out_xf = nullptr, int out_xf_kind = 0);

// Block-causal attention of n_rows_total consecutive query rows, sixteen to a block, each block exactly as
// dfl_attn_block would run it alone at its own context length (ctx_len + 16 b): the same split of the keys, so the same
// bits.  Blocks whose context lengths fall in the same bucket go out as one launch pair (as many of them as the
// workspace has room for partial tiles of).  Transposed V cache; block b's rows at q + 16 b rows, out likewise,
// out_xf + b * dfl_xf_bytes(n_q * head_dim).  The K/V rows of all the blocks are in the cache already.
int32_t dfl_attn_blocks(dflash_ctx *ctx, const void *q, int32_t q_type, const void *k_cache, const void *vt_cache, int64_t ctx_len,
                        int32_t n_rows_total, int32_t n_q, int32_t n_kv, int32_t head_dim, int64_t kv_capacity, float scale,
                        float *out, dflash_stream_t stream, void *out_xf, int out_xf_kind);

// dflash_gemm_fewrow for a tensor of a model that passed dfl_model_tensors_checked (the fast kernels).
int32_t dfl_gemm_fewrow_checked(dflash_ctx *ctx, int32_t w_type, const void *w, const void *x, int32_t x_type, float *y,
                                int64_t n_in, int64_t n_out, int32_t n_rows, dflash_stream_t stream);

// Few-row Q6_K GEMMs of up to three matrices over the same activations (a layer's q, k and v
// projections) as one launch: y[m] = x . w[m]^T, [n_rows][n_out[m]] each.
int32_t dfl_gemm_q6k_set(dflash_ctx *ctx, int n_mats, const void *const *w, float *const *y, const int64_t *n_out, const void *x,
                         int32_t x_type, int64_t n_in, int32_t n_rows, dflash_stream_t stream);

// Few-row Q4_K GEMM over the matrices that the device-side list ids[0 .. *n_slots) picks out of a stack
// (w_stack + id * w_stride_bytes; id -1 = extra_w): slot j reads activations x + j * x_stride (elements; 0 = shared) and
// writes y + j * y_stride (floats) as [n_rows][n_out].  max_slots bounds *n_slots.  whole_groups != 0:
// no split K (results independent of the other matrices in the batch).  w_stack_up != null (needs
// whole_groups): SwiGLU pair, y = silu(x . gate^T) * (x . up^T) with the gate matrices from w_stack /
// extra_w and the up matrices, same ids, from w_stack_up / extra_w_up.  tiled != 0: every matrix (the stacks'
// members, the extras) is in the tiled order of dflash_repack_q4k_tiled and w_stride_bytes is the tiled size.
// y_type: DFLASH_TYPE_F32, or DFLASH_TYPE_F16 (y then points to f16 and y_stride counts f16 elements) where
// dfl_q4k_batched_f16_out() says the path that will run can write it.  Enqueue only.
bool dfl_q4k_batched_f16_out(const dflash_ctx *ctx, int32_t tiled, int32_t whole_groups, int64_t n_out);
// Routing folded into the launch (route != null; where dfl_q4k_batched_can_route() allows it): ids and n_slots are
// then OUTPUTS.  Every workgroup derives the block's expert list from the router logits itself (the arithmetic of
// the stand-alone routing kernel, n_expert <= 256), workgroup 0 writes ids, *n_slots, sel_e, sel_w and slot_of for
// the launches that follow; the shared-expert gate is not computed here.
struct dfl_route_args {
    const float *logits;  // [n_rows][n_expert]
    int32_t n_expert, n_used, with_shared;
    int32_t *sel_e;   // [n_rows][n_used]
    float *sel_w;     // [n_rows][n_used]
    int32_t *slot_of; // [n_rows][n_used]
};
bool dfl_q4k_batched_can_route(const dflash_ctx *ctx, int32_t tiled, int64_t n_out, int32_t n_expert, int32_t n_used);
int32_t dfl_gemm_q4k_batched(dflash_ctx *ctx, const void *w_stack, size_t w_stride_bytes, const void *extra_w,
                             const int32_t *ids, const int32_t *n_slots, int max_slots, const void *x, int32_t x_type,
                             size_t x_stride,
                             void *y, int32_t y_type, size_t y_stride, int64_t n_in, int64_t n_out, int32_t n_rows,
                             int32_t whole_groups, const void *w_stack_up, const void *extra_w_up, int32_t tiled,
                             dflash_stream_t stream, const dfl_route_args *route = nullptr);
