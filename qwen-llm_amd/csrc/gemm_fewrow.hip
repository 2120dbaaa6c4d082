// Few-row quantised GEMM for the 16-row verify block:
//   Y[n_rows][n_out] = X[n_rows][n_in] . W^T,   W = ggml quant blocks, row-major.
// Replaces encode_mat_mat_dispatch_dflash_verify (metal_forward/dispatch.rs:365-378)
// and its kernel (kernels/mat_mat_fewrow_gen.metal:374-474).
//
// Mapping onto CDNA4.  The 16 block rows are exactly the M side of
// v_mfma_f32_16x16x32_f16, so a wave owns 16 weight rows (one output tile) and
// streams them along K; lane l serves weight row l%16 and the k-octet l/16.
//
//  * Q4_K: a lane reads the 32 quant bytes of "its" chunk of a super-block (two
//    sub-blocks: low and high nibbles) straight from HBM.  Nibbles are turned into
//    exact f16 integers by OR-ing them into the mantissa of 1024.0 (low nibble) or
//    64.0 (high nibble, which sits four bits up), and one packed f16 fma per value
//    pair, fma(1024+q, s, -1024*s), yields round(q*s) with a single rounding
//    (s = d*sc_j in f16).  The per-sub-block minimum never touches the nibbles:
//    sum_k dmin*m_j*x[k] = dmin*m_j * (sum of x over the sub-block), so the eight
//    minima of a super-block meet eight pre-summed activations in one extra MFMA
//    per four super-blocks.  That keeps the vector ALU at ~10 instructions per
//    MFMA, below what the HBM stream needs.
//  * X is re-laid out once per call by a small kernel into the exact per-lane
//    fragment order the MFMA wants (and its sub-block sums are taken there), so the
//    hot loop loads every A fragment with one 16-byte load.
//  * K is split over the waves of a workgroup; their partial tiles are added in a
//    fixed order through LDS, so results are run-to-run deterministic.
//  * Q6_K / Q8_0 share a generic kernel: eight consecutive weights per lane are
//    dequantised to f16 and fed to the same MFMA.
#include "common.h"

#include <cstdlib>

namespace {

typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float float4_t __attribute__((ext_vector_type(4)));

constexpr int kMaxSplit = 16;

// ----------------------------------------------------------------------------
// X preparation
// ----------------------------------------------------------------------------

// Order in which a lane's eight values of one MFMA come out of the nibble unpack:
// value i is byte kPerm[i] of the eight bytes it covers.
__device__ __constant__ int kPerm[8] = {0, 2, 1, 3, 4, 6, 5, 7};

template <typename T>
__device__ __forceinline__ _Float16 load_x(const T *x, int m, int n_rows, int64_t n_in, int64_t k) {
    if (m >= n_rows) return static_cast<_Float16>(0.0f);
    return static_cast<_Float16>(x[static_cast<int64_t>(m) * n_in + k]);
}

// Q4_K layout: for super-block b, MFMA t (0..7), lane (m = lane%16, g = lane/16),
// value i:  k = 256 b + 64 g + (t < 4 ? 8 t : 32 + 8 (t-4)) + kPerm[i].
// Also writes, per super-block and row, the eight sub-block sums of the f16-rounded
// activations, split into a high and a low f16 part.
template <typename T>
__global__ void __launch_bounds__(256) prep_x_q4k_kernel(const T *__restrict__ x, half8_t *__restrict__ xp,
                                                         half8_t *__restrict__ xs_hi, half8_t *__restrict__ xs_lo,
                                                         int n_rows, int64_t n_in) {
    int b = blockIdx.x;
    for (int item = threadIdx.x; item < 512; item += 256) {
        int t = item >> 6, lane = item & 63;
        int m = lane & 15, g = lane >> 4;
        int64_t k0 = 256ll * b + 64 * g + (t < 4 ? 8 * t : 32 + 8 * (t - 4));
        half8_t v;
#pragma unroll
        for (int i = 0; i < 8; i++) v[i] = load_x(x, m, n_rows, n_in, k0 + kPerm[i]);
        xp[(static_cast<int64_t>(b) * 8 + t) * 64 + lane] = v;
    }
    if (threadIdx.x < 16) {
        int m = threadIdx.x;
        half8_t hi, lo;
#pragma unroll
        for (int j = 0; j < 8; j++) {
            float s = 0.0f;
            for (int e = 0; e < 32; e++) s += static_cast<float>(load_x(x, m, n_rows, n_in, 256ll * b + 32 * j + e));
            _Float16 h = static_cast<_Float16>(s);
            hi[j] = h;
            lo[j] = static_cast<_Float16>(s - static_cast<float>(h));
        }
        xs_hi[b * 16 + m] = hi;
        xs_lo[b * 16 + m] = lo;
    }
}

// Natural layout for the generic kernel: step s (32 k), lane (m, g), value i: k = 32 s + 8 g + i.
template <typename T>
__global__ void __launch_bounds__(256) prep_x_natural_kernel(const T *__restrict__ x, half8_t *__restrict__ xp,
                                                             int n_rows, int64_t n_in, int64_t n_steps) {
    int64_t item = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
    if (item >= n_steps * 64) return;
    int64_t s = item >> 6;
    int lane = item & 63;
    int m = lane & 15, g = lane >> 4;
    half8_t v;
#pragma unroll
    for (int i = 0; i < 8; i++) v[i] = load_x(x, m, n_rows, n_in, 32 * s + 8 * g + i);
    xp[item] = v;
}

// ----------------------------------------------------------------------------
// Q4_K kernel
// ----------------------------------------------------------------------------

__device__ __forceinline__ half2_t as_half2(uint32_t bits) { return __builtin_bit_cast(half2_t, bits); }

__device__ __forceinline__ half2_t splat(_Float16 v) {
    half2_t r = {v, v};
    return r;
}

// Eight f16 weights of one MFMA from two dwords of quant bytes.
//   HIGH = false: low nibbles,  1024 + q  via magic 0x6400, mask 0x000F
//   HIGH = true : high nibbles,   64 + q  via magic 0x5400, mask 0x00F0
// s2 = (s, s), c2 = (-1024 s, -1024 s) or (-64 s, -64 s).
// (a & mask) | magic in one VALU instruction.  The compiler splits this into two
// because both constants are literals; with the mask in an SGPR and the magic in a
// VGPR it is a single v_and_or_b32.
__device__ __forceinline__ uint32_t and_or(uint32_t a, uint32_t mask, uint32_t magic) {
    uint32_t r;
    asm("v_and_or_b32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "s"(mask), "v"(magic));
    return r;
}

template <bool HIGH>
__device__ __forceinline__ half8_t unpack_scale(uint32_t w0, uint32_t w1, half2_t s2, half2_t c2) {
    constexpr uint32_t mask = HIGH ? 0x00F000F0u : 0x000F000Fu;
    constexpr uint32_t magic = HIGH ? 0x54005400u : 0x64006400u;
    half2_t p0 = __builtin_elementwise_fma(as_half2(and_or(w0, mask, magic)), s2, c2);
    half2_t p1 = __builtin_elementwise_fma(as_half2(and_or(w0 >> 8, mask, magic)), s2, c2);
    half2_t p2 = __builtin_elementwise_fma(as_half2(and_or(w1, mask, magic)), s2, c2);
    half2_t p3 = __builtin_elementwise_fma(as_half2(and_or(w1 >> 8, mask, magic)), s2, c2);
    half8_t r = {p0[0], p0[1], p1[0], p1[1], p2[0], p2[1], p3[0], p3[1]};
    return r;
}

// Byte j of `v` (0..255) as an exact f16.
__device__ __forceinline__ _Float16 byte_to_half(uint32_t v, int j) {
    return static_cast<_Float16>(static_cast<float>((v >> (8 * j)) & 0xffu));
}

// R row tiles of 16 weight rows per wave; blockDim.x = 64 * n_split.
template <int R>
__global__ void __launch_bounds__(64 * kMaxSplit)
    gemm_q4k_kernel(const uint8_t *__restrict__ w, const half8_t *__restrict__ xp, const half8_t *__restrict__ xs_hi,
                    const half8_t *__restrict__ xs_lo, float *__restrict__ y, int n_out, int nb, int n_rows,
                    int n_split) {
    extern __shared__ float red[];  // [n_split][R][256]
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int n = lane & 15, g = lane >> 4;
    const int n0 = blockIdx.x * (16 * R);
    const int b0 = static_cast<int>(static_cast<int64_t>(nb) * wave / n_split);
    const int b1 = static_cast<int>(static_cast<int64_t>(nb) * (wave + 1) / n_split);
    const size_t row_bytes = static_cast<size_t>(nb) * DFL_Q4_K_BYTES;

    const uint8_t *rowp[R];
#pragma unroll
    for (int r = 0; r < R; r++) {
        int row = n0 + 16 * r + n;
        row = row < n_out ? row : n_out - 1;
        rowp[r] = w + static_cast<size_t>(row) * row_bytes;
    }

    float4_t acc[R], acc_min[R];
    uint4 min_hdr[R];
#pragma unroll
    for (int r = 0; r < R; r++) {
        acc[r] = float4_t{0, 0, 0, 0};
        acc_min[r] = float4_t{0, 0, 0, 0};
        min_hdr[r] = uint4{0, 0, 0, 0};
    }

    auto flush_min = [&](int quad_base) {
        // lane (n, g) holds the header of block quad_base + g (or zeros past the slice)
        int blk = quad_base + g;
        bool valid = blk < b1;
        half8_t a_hi = valid ? xs_hi[blk * 16 + n] : half8_t{0, 0, 0, 0, 0, 0, 0, 0};
        half8_t a_lo = valid ? xs_lo[blk * 16 + n] : half8_t{0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
        for (int r = 0; r < R; r++) {
            uint4 h = min_hdr[r];
            _Float16 dmin = __builtin_bit_cast(half2_t, h.x)[1];
            uint32_t lo_m = h.z & 0x3F3F3F3Fu;
            uint32_t hi_m = ((h.w >> 4) & 0x0F0F0F0Fu) | ((h.z >> 2) & 0x30303030u);
            half8_t bm;
#pragma unroll
            for (int j = 0; j < 4; j++) {
                bm[j] = byte_to_half(lo_m, j) * dmin;
                bm[4 + j] = byte_to_half(hi_m, j) * dmin;
            }
            acc_min[r] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a_hi, bm, acc_min[r], 0, 0, 0);
            acc_min[r] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a_lo, bm, acc_min[r], 0, 0, 0);
            min_hdr[r] = uint4{0, 0, 0, 0};
        }
    };

    for (int b = b0; b < b1; b++) {
        half8_t a[8];
#pragma unroll
        for (int t = 0; t < 8; t++) a[t] = xp[(static_cast<int64_t>(b) * 8 + t) * 64 + lane];
#pragma unroll
        for (int r = 0; r < R; r++) {
            const uint8_t *blk = rowp[r] + static_cast<size_t>(b) * DFL_Q4_K_BYTES;
            uint4 hdr = *reinterpret_cast<const uint4 *>(blk);
            uint4 q0 = *reinterpret_cast<const uint4 *>(blk + 16 + 32 * g);
            uint4 q1 = *reinterpret_cast<const uint4 *>(blk + 32 + 32 * g);
            if (((b - b0) & 3) == g) min_hdr[r] = hdr;

            // scales of sub-blocks 2g (low nibbles) and 2g+1 (high nibbles)
            uint32_t lo_sc = hdr.y & 0x3F3F3F3Fu;
            uint32_t hi_sc = (hdr.w & 0x0F0F0F0Fu) | ((hdr.y >> 2) & 0x30303030u);
            uint32_t sel = (g < 2 ? lo_sc : hi_sc) >> (16 * (g & 1));
            _Float16 d = __builtin_bit_cast(half2_t, hdr.x)[0];
            _Float16 s_lo = byte_to_half(sel, 0) * d;
            _Float16 s_hi = byte_to_half(sel, 1) * d;
            half2_t s2l = splat(s_lo), c2l = splat(s_lo * static_cast<_Float16>(-1024.0f));
            half2_t s2h = splat(s_hi), c2h = splat(s_hi * static_cast<_Float16>(-64.0f));

            uint32_t qw[8] = {q0.x, q0.y, q0.z, q0.w, q1.x, q1.y, q1.z, q1.w};
#pragma unroll
            for (int t = 0; t < 4; t++) {
                half8_t bl = unpack_scale<false>(qw[2 * t], qw[2 * t + 1], s2l, c2l);
                acc[r] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[t], bl, acc[r], 0, 0, 0);
            }
#pragma unroll
            for (int t = 0; t < 4; t++) {
                half8_t bh = unpack_scale<true>(qw[2 * t], qw[2 * t + 1], s2h, c2h);
                acc[r] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[4 + t], bh, acc[r], 0, 0, 0);
            }
        }
        if (((b - b0) & 3) == 3) flush_min(b - 3);
    }
    if ((b1 - b0) & 3) flush_min(b0 + ((b1 - b0) & ~3));

    // fixed-order reduction over the K-slices of this workgroup
#pragma unroll
    for (int r = 0; r < R; r++)
#pragma unroll
        for (int i = 0; i < 4; i++)
            red[(wave * R + r) * 256 + (4 * g + i) * 16 + n] = acc[r][i] - acc_min[r][i];
    __syncthreads();
    for (int e = threadIdx.x; e < R * 256; e += blockDim.x) {
        int r = e >> 8, m = (e >> 4) & 15, nn = e & 15;
        int row = n0 + 16 * r + nn;
        if (m < n_rows && row < n_out) {
            float s = 0.0f;
            for (int ws = 0; ws < n_split; ws++) s += red[(ws * R + r) * 256 + (e & 255)];
            y[static_cast<size_t>(m) * n_out + row] = s;
        }
    }
}

// ----------------------------------------------------------------------------
// Generic kernel (Q6_K, Q8_0): eight consecutive weights -> f16 -> MFMA
// ----------------------------------------------------------------------------

__device__ __forceinline__ float half_at(const uint8_t *p) {
    return __half2float(__ushort_as_half(static_cast<unsigned short>(p[0] | (p[1] << 8))));
}

template <int TYPE>
__device__ __forceinline__ half8_t dequant8(const uint8_t *row, int64_t k0);

// Q6_K: y = d * scale[i/16] * (q - 32); ql/qh interleave as in ggml's dequantize_row_q6_K
// (metal/tests/q6_k_f32_tile.rs:46-71).
template <>
__device__ __forceinline__ half8_t dequant8<DFLASH_TYPE_Q6_K>(const uint8_t *row, int64_t k0) {
    const uint8_t *blk = row + (k0 >> 8) * DFL_Q6_K_BYTES;
    int e = static_cast<int>(k0 & 255);
    int half_idx = e >> 7, r = e & 127, kq = r >> 5, l0 = r & 31;
    const uint8_t *ql = blk + 64 * half_idx + ((kq & 1) ? 32 : 0) + l0;
    const uint8_t *qh = blk + 128 + 32 * half_idx + l0;
    float ds = half_at(blk + 208) *
               static_cast<float>(reinterpret_cast<const int8_t *>(blk + 192 + 8 * half_idx)[(l0 >> 4) + 2 * kq]);
    half8_t v;
#pragma unroll
    for (int i = 0; i < 8; i++) {
        int lo = (kq & 2) ? (ql[i] >> 4) : (ql[i] & 0x0f);
        int hi = (qh[i] >> (2 * kq)) & 3;
        v[i] = static_cast<_Float16>(ds * static_cast<float>((lo | (hi << 4)) - 32));
    }
    return v;
}

template <>
__device__ __forceinline__ half8_t dequant8<DFLASH_TYPE_Q8_0>(const uint8_t *row, int64_t k0) {
    const uint8_t *blk = row + (k0 >> 5) * DFL_Q8_0_BYTES;
    float d = half_at(blk);
    const int8_t *q = reinterpret_cast<const int8_t *>(blk + 2 + (k0 & 31));
    half8_t v;
#pragma unroll
    for (int i = 0; i < 8; i++) v[i] = static_cast<_Float16>(d * static_cast<float>(q[i]));
    return v;
}

template <int TYPE>
__global__ void __launch_bounds__(64 * kMaxSplit)
    gemm_generic_kernel(const uint8_t *__restrict__ w, const half8_t *__restrict__ xp, float *__restrict__ y,
                        int n_out, int64_t n_steps, size_t row_bytes, int n_rows, int n_split) {
    extern __shared__ float red[];  // [n_split][256]
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int n = lane & 15, g = lane >> 4;
    const int n0 = blockIdx.x * 16;
    int row = n0 + n;
    row = row < n_out ? row : n_out - 1;
    const uint8_t *rowp = w + static_cast<size_t>(row) * row_bytes;
    const int64_t s0 = n_steps * wave / n_split, s1 = n_steps * (wave + 1) / n_split;
    float4_t acc = {0, 0, 0, 0};
    for (int64_t s = s0; s < s1; s++) {
        half8_t a = xp[s * 64 + lane];
        half8_t b = dequant8<TYPE>(rowp, 32 * s + 8 * g);
        acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, acc, 0, 0, 0);
    }
#pragma unroll
    for (int i = 0; i < 4; i++) red[wave * 256 + (4 * g + i) * 16 + n] = acc[i];
    __syncthreads();
    for (int e = threadIdx.x; e < 256; e += blockDim.x) {
        int m = e >> 4, nn = e & 15;
        if (m < n_rows && n0 + nn < n_out) {
            float sum = 0.0f;
            for (int ws = 0; ws < n_split; ws++) sum += red[ws * 256 + e];
            y[static_cast<size_t>(m) * n_out + n0 + nn] = sum;
        }
    }
}

int env_int(const char *name, int fallback) {
    const char *v = getenv(name);
    return (v && *v) ? atoi(v) : fallback;
}

}  // namespace

extern "C" int32_t dflash_gemm_fewrow(dflash_ctx *ctx, int32_t w_type, const void *w, const void *x, int32_t x_type,
                                      float *y, int64_t n_in, int64_t n_out, int32_t n_rows, dflash_stream_t stream) {
    if (!ctx) return DFLASH_ERR_INVALID_INPUT;
    if (!w || !x || !y) return dfl_fail(ctx, DFLASH_ERR_INVALID_INPUT, "gemm_fewrow: null pointer");
    if (n_rows < 1 || n_rows > 16)
        return dfl_fail(ctx, DFLASH_ERR_BAD_SHAPE, "gemm_fewrow: n_rows %d outside 1..16", n_rows);
    if (n_in <= 0 || n_out <= 0 || n_in > 0x7fffffffll || n_out > 0x7fffffffll)
        return dfl_fail(ctx, DFLASH_ERR_BAD_SHAPE, "gemm_fewrow: n_in %lld / n_out %lld out of range",
                        static_cast<long long>(n_in), static_cast<long long>(n_out));
    if (x_type != DFLASH_TYPE_F32 && x_type != DFLASH_TYPE_F16)
        return dfl_fail(ctx, DFLASH_ERR_UNSUPPORTED, "gemm_fewrow: activations must be f32 or f16");
    if (w_type != DFLASH_TYPE_Q4_K && w_type != DFLASH_TYPE_Q6_K && w_type != DFLASH_TYPE_Q8_0)
        return dfl_fail(ctx, DFLASH_ERR_UNSUPPORTED, "gemm_fewrow: weight type %d has no few-row kernel", w_type);
    const int64_t blk = (w_type == DFLASH_TYPE_Q8_0) ? DFL_QK8_0 : DFL_QK_K;
    if (n_in % blk)
        return dfl_fail(ctx, DFLASH_ERR_BAD_SHAPE, "gemm_fewrow: n_in %lld is not a multiple of %lld",
                        static_cast<long long>(n_in), static_cast<long long>(blk));
    const size_t row_bytes = dflash_row_bytes(w_type, static_cast<size_t>(n_in));
    const size_t w_bytes = row_bytes * static_cast<size_t>(n_out);
    const size_t x_bytes = static_cast<size_t>(n_rows) * n_in * (x_type == DFLASH_TYPE_F32 ? 4 : 2);
    const size_t y_bytes = static_cast<size_t>(n_rows) * n_out * 4;
    if (reinterpret_cast<uintptr_t>(w) % (w_type == DFLASH_TYPE_Q4_K ? 16 : 2) ||
        reinterpret_cast<uintptr_t>(x) % 4 || reinterpret_cast<uintptr_t>(y) % 4)
        return dfl_fail(ctx, DFLASH_ERR_ALIGNMENT, "gemm_fewrow: operand alignment");
    if (dfl_ranges_overlap(y, y_bytes, x, x_bytes) || dfl_ranges_overlap(y, y_bytes, w, w_bytes))
        return dfl_fail(ctx, DFLASH_ERR_ALIAS, "gemm_fewrow: y aliases an input");

    hipStream_t st = static_cast<hipStream_t>(stream);
    const int64_t n_steps = n_in / 32;
    size_t off = 0;
    half8_t *xp = dfl_ws_take<half8_t>(ctx, &off, static_cast<size_t>(n_steps) * 64 * sizeof(half8_t));
    const int tiles = static_cast<int>((n_out + 15) / 16);
    const int target_waves = 8 * ctx->n_cu;

    if (w_type == DFLASH_TYPE_Q4_K) {
        const int nb = static_cast<int>(n_in / DFL_QK_K);
        half8_t *xs_hi = dfl_ws_take<half8_t>(ctx, &off, static_cast<size_t>(nb) * 16 * sizeof(half8_t));
        half8_t *xs_lo = dfl_ws_take<half8_t>(ctx, &off, static_cast<size_t>(nb) * 16 * sizeof(half8_t));
        if (!xp || !xs_hi || !xs_lo) return dfl_fail(ctx, DFLASH_ERR_WORKSPACE, "gemm_fewrow: workspace too small");
        if (x_type == DFLASH_TYPE_F32)
            prep_x_q4k_kernel<float><<<nb, 256, 0, st>>>(static_cast<const float *>(x), xp, xs_hi, xs_lo, n_rows, n_in);
        else
            prep_x_q4k_kernel<_Float16>
                <<<nb, 256, 0, st>>>(static_cast<const _Float16 *>(x), xp, xs_hi, xs_lo, n_rows, n_in);
        int r_tiles = env_int("DFLASH_GEMM_R", tiles >= 4 * ctx->n_cu ? 2 : 1);
        if (r_tiles != 2) r_tiles = 1;
        int groups = (tiles + r_tiles - 1) / r_tiles;
        int split = (target_waves + groups - 1) / groups;
        split = env_int("DFLASH_GEMM_NSPLIT", split);
        if (split > nb) split = nb;
        if (split > kMaxSplit) split = kMaxSplit;
        if (split < 1) split = 1;
        size_t lds = static_cast<size_t>(split) * r_tiles * 256 * sizeof(float);
        const uint8_t *wb = static_cast<const uint8_t *>(w);
        dfl_timed timer(ctx, st, DFL_T_GEMM);
        if (r_tiles == 2)
            gemm_q4k_kernel<2><<<groups, 64 * split, lds, st>>>(wb, xp, xs_hi, xs_lo, y, static_cast<int>(n_out), nb,
                                                               n_rows, split);
        else
            gemm_q4k_kernel<1><<<groups, 64 * split, lds, st>>>(wb, xp, xs_hi, xs_lo, y, static_cast<int>(n_out), nb,
                                                               n_rows, split);
    } else {
        if (!xp) return dfl_fail(ctx, DFLASH_ERR_WORKSPACE, "gemm_fewrow: workspace too small");
        unsigned prep_grid = static_cast<unsigned>((n_steps * 64 + 255) / 256);
        if (x_type == DFLASH_TYPE_F32)
            prep_x_natural_kernel<float><<<prep_grid, 256, 0, st>>>(static_cast<const float *>(x), xp, n_rows, n_in,
                                                                    n_steps);
        else
            prep_x_natural_kernel<_Float16>
                <<<prep_grid, 256, 0, st>>>(static_cast<const _Float16 *>(x), xp, n_rows, n_in, n_steps);
        int split = (target_waves + tiles - 1) / tiles;
        split = env_int("DFLASH_GEMM_NSPLIT", split);
        if (split > n_steps) split = static_cast<int>(n_steps);
        if (split > kMaxSplit) split = kMaxSplit;
        if (split < 1) split = 1;
        size_t lds = static_cast<size_t>(split) * 256 * sizeof(float);
        const uint8_t *wb = static_cast<const uint8_t *>(w);
        dfl_timed timer(ctx, st, DFL_T_GEMM);
        if (w_type == DFLASH_TYPE_Q6_K)
            gemm_generic_kernel<DFLASH_TYPE_Q6_K>
                <<<tiles, 64 * split, lds, st>>>(wb, xp, y, static_cast<int>(n_out), n_steps, row_bytes, n_rows, split);
        else
            gemm_generic_kernel<DFLASH_TYPE_Q8_0>
                <<<tiles, 64 * split, lds, st>>>(wb, xp, y, static_cast<int>(n_out), n_steps, row_bytes, n_rows, split);
    }
    DFL_HIP_CHECK(ctx, hipGetLastError());
    return DFLASH_OK;
}
