// Block dequantisation kernels: ggml Q4_K / Q6_K / Q8_0 -> f32, bit-exact with
// ggml's dequantize_row_* (closed forms pinned by the reference's tests,
// codec.rs:474-577 and metal/tests/q6_k_f32_tile.rs:46-107).  Every value is built
// from round-to-nearest f32 products and one subtraction, never a fused
// multiply-add, so __fmul_rn / __fsub_rn are used throughout.
#include "common.h"

#include <cstring>

namespace {

__device__ __forceinline__ float h2f(const uint8_t *p) {
    return __half2float(__ushort_as_half(static_cast<unsigned short>(p[0] | (p[1] << 8))));
}

// One thread per element; one 256-thread workgroup per super-block.
__global__ void __launch_bounds__(256) dequant_q4_k_kernel(const uint8_t *__restrict__ blocks, float *__restrict__ out,
                                                           size_t n_blocks) {
    size_t b = blockIdx.x;
    if (b >= n_blocks) return;
    const uint8_t *blk = blocks + b * DFL_Q4_K_BYTES;
    int e = threadIdx.x;
    int j = e >> 5;  // sub-block
    int l = e & 31;
    const uint8_t *s = blk + 4;
    int sc, m;
    if (j < 4) {
        sc = s[j] & 63;
        m = s[j + 4] & 63;
    } else {
        sc = (s[j + 4] & 0x0f) | ((s[j - 4] >> 6) << 4);
        m = (s[j + 4] >> 4) | ((s[j] >> 6) << 4);
    }
    uint8_t byte = blk[16 + 32 * (j >> 1) + l];
    int q = (j & 1) ? (byte >> 4) : (byte & 0x0f);
    float d1 = __fmul_rn(h2f(blk), static_cast<float>(sc));
    float m1 = __fmul_rn(h2f(blk + 2), static_cast<float>(m));
    out[b * DFL_QK_K + e] = __fsub_rn(__fmul_rn(d1, static_cast<float>(q)), m1);
}

__global__ void __launch_bounds__(256) dequant_q6_k_kernel(const uint8_t *__restrict__ blocks, float *__restrict__ out,
                                                           size_t n_blocks) {
    size_t b = blockIdx.x;
    if (b >= n_blocks) return;
    const uint8_t *blk = blocks + b * DFL_Q6_K_BYTES;
    int e = threadIdx.x;
    int n = e >> 7;         // 128-element half
    int r = e & 127;
    int k = r >> 5;         // which of q1..q4
    int l = r & 31;
    const uint8_t *ql = blk + 64 * n;
    const uint8_t *qh = blk + 128 + 32 * n;
    const int8_t *sc = reinterpret_cast<const int8_t *>(blk + 192 + 8 * n);
    int lo = (k & 1) ? ql[l + 32] : ql[l];
    lo = (k & 2) ? (lo >> 4) : (lo & 0x0f);
    int hi = (qh[l] >> (2 * k)) & 3;
    int q = (lo | (hi << 4)) - 32;
    float ds = __fmul_rn(h2f(blk + 208), static_cast<float>(sc[(l >> 4) + 2 * k]));
    out[b * DFL_QK_K + e] = __fmul_rn(ds, static_cast<float>(q));
}

// Q8_0 blocks hold 32 elements; eight blocks per 256-thread workgroup.
__global__ void __launch_bounds__(256) dequant_q8_0_kernel(const uint8_t *__restrict__ blocks, float *__restrict__ out,
                                                           size_t n_blocks) {
    size_t b = static_cast<size_t>(blockIdx.x) * 8 + (threadIdx.x >> 5);
    if (b >= n_blocks) return;
    const uint8_t *blk = blocks + b * DFL_Q8_0_BYTES;
    int i = threadIdx.x & 31;
    float q = static_cast<float>(reinterpret_cast<const int8_t *>(blk + 2)[i]);
    out[b * DFL_QK8_0 + i] = __fmul_rn(h2f(blk), q);
}

}  // namespace

extern "C" int32_t dflash_dequant(dflash_ctx *ctx, int32_t type, const void *blocks, size_t n_elems, float *out_f32,
                                  dflash_stream_t stream) {
    if (!ctx) return DFLASH_ERR_INVALID_INPUT;
    if (!blocks || !out_f32) return dfl_fail(ctx, DFLASH_ERR_INVALID_INPUT, "dequant: null pointer");
    hipStream_t st = static_cast<hipStream_t>(stream);
    const uint8_t *src = static_cast<const uint8_t *>(blocks);
    size_t blk = (type == DFLASH_TYPE_Q8_0) ? DFL_QK8_0 : DFL_QK_K;
    if (type != DFLASH_TYPE_Q4_K && type != DFLASH_TYPE_Q6_K && type != DFLASH_TYPE_Q8_0)
        return dfl_fail(ctx, DFLASH_ERR_UNSUPPORTED, "dequant: unsupported type %d", type);
    if (n_elems % blk)
        return dfl_fail(ctx, DFLASH_ERR_BAD_SHAPE, "dequant: %zu elements is not a multiple of the block size %zu",
                        n_elems, blk);
    size_t n_blocks = n_elems / blk;
    if (n_blocks == 0) return DFLASH_OK;
    if (n_blocks > 0x7fffffffull) return dfl_fail(ctx, DFLASH_ERR_BAD_SHAPE, "dequant: too many blocks");
    if (dfl_ranges_overlap(out_f32, n_elems * 4, blocks, dflash_row_bytes(type, n_elems)))
        return dfl_fail(ctx, DFLASH_ERR_ALIAS, "dequant: output aliases the blocks");
    if (type == DFLASH_TYPE_Q4_K)
        dequant_q4_k_kernel<<<dim3(static_cast<unsigned>(n_blocks)), 256, 0, st>>>(src, out_f32, n_blocks);
    else if (type == DFLASH_TYPE_Q6_K)
        dequant_q6_k_kernel<<<dim3(static_cast<unsigned>(n_blocks)), 256, 0, st>>>(src, out_f32, n_blocks);
    else
        dequant_q8_0_kernel<<<dim3(static_cast<unsigned>((n_blocks + 7) / 8)), 256, 0, st>>>(src, out_f32, n_blocks);
    DFL_HIP_CHECK(ctx, hipGetLastError());
    return DFLASH_OK;
}

// ---- streaming-read probe ----------------------------------------------------------------------
// Reads `bytes` of device memory once (a grid-stride loop of 16-byte loads, 8 workgroups of 256 threads per CU) and
// stores one word per workgroup: the rate a plain read-only stream reaches on this device, to set beside the rates
// of the kernels that stream weights.
namespace {
constexpr int kProbeThreads = 256;
__global__ void __launch_bounds__(kProbeThreads) read_probe_kernel(const uint4 *__restrict__ p, size_t n_pieces, uint32_t *__restrict__ out,
                                                                    int n_out_words) {
    uint4 a = {0, 0, 0, 0};
    for (size_t i = blockIdx.x * static_cast<size_t>(kProbeThreads) + threadIdx.x; i < n_pieces; i += static_cast<size_t>(gridDim.x) * kProbeThreads) {
        const uint4 v = p[i];
        a.x ^= v.x;
        a.y ^= v.y;
        a.z ^= v.z;
        a.w ^= v.w;
    }
    uint32_t acc = a.x ^ a.y ^ a.z ^ a.w;
    for (int off = 32; off > 0; off >>= 1) acc ^= __shfl_xor(acc, off, 64);
    if (threadIdx.x == 0) out[blockIdx.x % n_out_words] = acc;  // (a plain store: the words are a sink, not a checksum anyone reads)
}
}  // namespace

extern "C" int32_t dflash_hbm_read_probe(dflash_ctx *ctx, const void *const *bufs, int32_t n_bufs, size_t bytes, int32_t n_launches,
                                         void *out_words, dflash_stream_t stream) {
    if (!ctx) return DFLASH_ERR_INVALID_INPUT;
    if (!bufs || n_bufs < 1 || n_launches < 1 || !out_words || bytes % 16)
        return dfl_fail(ctx, DFLASH_ERR_INVALID_INPUT, "hbm_read_probe: buffers of a multiple of 16 bytes and %d output words", ctx->n_cu);
    for (int i = 0; i < n_bufs; i++)
        if (!bufs[i] || reinterpret_cast<uintptr_t>(bufs[i]) % 16)
            return dfl_fail(ctx, DFLASH_ERR_ALIGNMENT, "hbm_read_probe: buffer %d is null or not 16-byte aligned", i);
    for (int k = 0; k < n_launches; k++)
        read_probe_kernel<<<ctx->n_cu * 8, kProbeThreads, 0, static_cast<hipStream_t>(stream)>>>(
            static_cast<const uint4 *>(bufs[k % n_bufs]), bytes / 16, static_cast<uint32_t *>(out_words), ctx->n_cu);
    DFL_HIP_CHECK(ctx, hipGetLastError());
    return DFLASH_OK;
}

// ---- super-block scale range of a quantised tensor ------------------------------------------------
// The few-row Q4_K / Q6_K kernels form (1024 + code) * (d * scale) in f16 on the way to the MFMA: exact and fast,
// and finite only while |d| (and |dmin|) stay in the range below.  Real checkpoints are orders of magnitude inside
// it (d is a weight scale, about 1e-4 .. 1e-1); a tensor outside it is declined at load time instead of silently
// producing infinities.
namespace {
__global__ void __launch_bounds__(256) scale_range_kernel(const uint8_t *__restrict__ blocks, size_t n_blocks, int block_bytes, int d_off,
                                                          int dmin_off, uint32_t *__restrict__ out) {
    // out[0] = max |d| as f32 bits, out[1] = max |dmin|, out[2] = 1 if any is NaN or infinite
    uint32_t md = 0, mm = 0, bad = 0;
    for (size_t b = blockIdx.x * static_cast<size_t>(256) + threadIdx.x; b < n_blocks; b += static_cast<size_t>(gridDim.x) * 256) {
        const uint8_t *p = blocks + b * block_bytes;
        const __half d = *reinterpret_cast<const __half *>(p + d_off);
        const float fd = fabsf(__half2float(d));
        if (!(fd <= 65504.0f)) bad = 1;
        md = max(md, __float_as_uint(fd));
        if (dmin_off >= 0) {
            const float fm = fabsf(__half2float(*reinterpret_cast<const __half *>(p + dmin_off)));
            if (!(fm <= 65504.0f)) bad = 1;
            mm = max(mm, __float_as_uint(fm));
        }
    }
    for (int off = 32; off > 0; off >>= 1) {
        md = max(md, static_cast<uint32_t>(__shfl_xor(static_cast<int>(md), off, 64)));
        mm = max(mm, static_cast<uint32_t>(__shfl_xor(static_cast<int>(mm), off, 64)));
        bad |= static_cast<uint32_t>(__shfl_xor(static_cast<int>(bad), off, 64));
    }
    if ((threadIdx.x & 63) == 0) {
        atomicMax(out, md);  // non-negative floats order like their bit patterns
        atomicMax(out + 1, mm);
        if (bad) atomicOr(out + 2, 1u);
    }
}
}  // namespace

extern "C" int32_t dflash_check_scale_range(dflash_ctx *ctx, int32_t type, const void *blocks, size_t n_blocks, float *max_abs_host,
                                            dflash_stream_t stream) {
    if (!ctx) return DFLASH_ERR_INVALID_INPUT;
    if (!blocks || n_blocks == 0) return dfl_fail(ctx, DFLASH_ERR_INVALID_INPUT, "check_scale_range: no blocks");
    int block_bytes, d_off, dmin_off;
    float lim_d, lim_dmin;
    if (type == DFLASH_TYPE_Q4_K || type == DFLASH_TYPE_Q4_K_TILED) {
        block_bytes = DFL_Q4_K_BYTES, d_off = 0, dmin_off = 2, lim_d = DFLASH_Q4_K_MAX_D, lim_dmin = DFLASH_Q4_K_MAX_DMIN;
    } else if (type == DFLASH_TYPE_Q6_K) {
        block_bytes = DFL_Q6_K_BYTES, d_off = 208, dmin_off = -1, lim_d = DFLASH_Q6_K_MAX_D, lim_dmin = 0.0f;
    } else {
        if (max_abs_host) max_abs_host[0] = max_abs_host[1] = 0.0f;
        return DFLASH_OK;  // the other types' kernels scale in f32
    }
    hipStream_t st = static_cast<hipStream_t>(stream);
    size_t ws_off = 0;
    uint32_t *out = dfl_ws_take<uint32_t>(ctx, &ws_off, 4 * sizeof(uint32_t));
    if (!out) return dfl_fail(ctx, DFLASH_ERR_WORKSPACE, "check_scale_range: no workspace");
    DFL_HIP_CHECK(ctx, hipMemsetAsync(out, 0, 4 * sizeof(uint32_t), st));
    const size_t want = (n_blocks + 255) / 256;
    const unsigned grid = static_cast<unsigned>(want < static_cast<size_t>(ctx->n_cu) * 8 ? want : static_cast<size_t>(ctx->n_cu) * 8);
    scale_range_kernel<<<grid, 256, 0, st>>>(static_cast<const uint8_t *>(blocks), n_blocks, block_bytes, d_off, dmin_off, out);
    DFL_HIP_CHECK(ctx, hipGetLastError());
    uint32_t *host = static_cast<uint32_t *>(ctx->pinned);
    DFL_HIP_CHECK(ctx, hipMemcpyAsync(host, out, 4 * sizeof(uint32_t), hipMemcpyDeviceToHost, st));
    DFL_HIP_CHECK(ctx, hipStreamSynchronize(st));
    float md, mm;
    memcpy(&md, host, 4);
    memcpy(&mm, host + 1, 4);
    if (max_abs_host) max_abs_host[0] = md, max_abs_host[1] = mm;
    if (host[2] || md > lim_d || (dmin_off >= 0 && mm > lim_dmin))
        return dfl_fail(ctx, DFLASH_ERR_UNSUPPORTED,
                        "tensor declined: super-block scales out of the few-row kernels' f16 range (max |d| %g, limit %g; max |dmin| %g, limit %g%s)",
                        md, lim_d, mm, lim_dmin, host[2] ? "; NaN or infinite scale" : "");
    return DFLASH_OK;
}
