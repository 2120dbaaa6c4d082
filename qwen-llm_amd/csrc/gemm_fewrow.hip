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
//    per four super-blocks.  That keeps the vector ALU near 10 instructions per
//    MFMA, below what the HBM stream needs.
//  * X is re-laid out once per call by a small kernel into the exact per-lane
//    fragment order the MFMA wants (and its sub-block sums are taken there).  A
//    workgroup of eight waves (eight output tiles) copies the fragments of its
//    K-slice into LDS once and every wave reads its A operands from there, so the
//    activation traffic out of L2 stays well below the weight stream.
//  * A wave issues the loads of every super-block of its K-slice before it computes
//    anything: the whole weight matrix is in flight at once and the kernel runs as a
//    single pass at the memory system's pace.
//  * K is split over workgroups; each writes its partial tiles and the last one to
//    arrive (a counter per tile group) adds them in slice order, so results are
//    run-to-run deterministic.
//  * Q6_K / Q8_0 share a generic kernel: eight consecutive weights per lane are
//    dequantised to f16 and fed to the same MFMA.
#include "common.h"

#include <cstdlib>

namespace {

typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float float4_t __attribute__((ext_vector_type(4)));

constexpr int kMaxSplit = 16;
constexpr int kWavesQ4K = 8;  // output tiles (waves) per workgroup of the Q4_K kernel

// ----------------------------------------------------------------------------
// X preparation
// ----------------------------------------------------------------------------

template <typename T>
__device__ __forceinline__ _Float16 load_x(const T *x, int m, int n_rows, int64_t n_in, int64_t k) {
    if (m >= n_rows) return static_cast<_Float16>(0.0f);
    return static_cast<_Float16>(x[static_cast<int64_t>(m) * n_in + k]);
}

// Q4_K layout: kQ4KBlockFrags (= 544) half8 entries per super-block b:
//   [t*64 + lane], t = 0..7 : A fragment of MFMA t for lane (m = lane%16, g = lane/16),
//        value i:  k = 256 b + 64 g + (t < 4 ? 8 t : 32 + 8 (t-4)) + perm[i],
//        perm = {0,2,1,3,4,6,5,7}: the order in which the nibble unpack emits a lane's values;
//   [512 + m], [528 + m]    : the eight sub-block sums of row m's f16-rounded activations,
//        split into a high and a low f16 part.
// One workgroup per super-block.
constexpr int kQ4KBlockFrags = 544;

template <typename T>
__global__ void __launch_bounds__(256) prep_x_q4k_kernel(const T *__restrict__ x, half8_t *__restrict__ xp,
                                                         int n_rows, int64_t n_in) {
    __shared__ _Float16 tile[16][256 + 8];
    const int b = blockIdx.x;
    const int tid = threadIdx.x;
    half8_t *out = xp + static_cast<int64_t>(b) * kQ4KBlockFrags;
#pragma unroll
    for (int m = 0; m < 16; m++) tile[m][tid] = load_x(x, m, n_rows, n_in, 256ll * b + tid);
    __syncthreads();
#pragma unroll
    for (int it = 0; it < 2; it++) {
        int item = tid + 256 * it;
        int t = item >> 6, lane = item & 63;
        int m = lane & 15, g = lane >> 4;
        int k0 = 64 * g + (t < 4 ? 8 * t : 32 + 8 * (t - 4));
        const _Float16 *src = &tile[m][k0];
        half8_t v = {src[0], src[2], src[1], src[3], src[4], src[6], src[5], src[7]};
        out[item] = v;
    }
    if (tid < 128) {
        int m = tid >> 3, j = tid & 7;
        float s = 0.0f;
#pragma unroll
        for (int e = 0; e < 32; e++) s += static_cast<float>(tile[m][32 * j + e]);
        _Float16 h = static_cast<_Float16>(s);
        _Float16 *sums = reinterpret_cast<_Float16 *>(out + 512);
        sums[m * 8 + j] = h;
        sums[128 + m * 8 + j] = static_cast<_Float16>(s - static_cast<float>(h));
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

// (a & mask) | magic in one VALU instruction.  The compiler splits this into two
// because both constants are literals; with the mask in an SGPR and the magic in a
// VGPR it is a single v_and_or_b32.
__device__ __forceinline__ uint32_t and_or(uint32_t a, uint32_t mask, uint32_t magic) {
    uint32_t r;
    asm("v_and_or_b32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "s"(mask), "v"(magic));
    return r;
}

// Eight f16 weights of one MFMA from two dwords of quant bytes.
//   HIGH = false: low nibbles,  1024 + q  via magic 0x6400, mask 0x000F
//   HIGH = true : high nibbles,   64 + q  via magic 0x5400, mask 0x00F0
// s2 = (s, s), c2 = (-1024 s, -1024 s) or (-64 s, -64 s).
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

// Grid: (tile groups) x (K slices); a workgroup is kWavesQ4K waves = kWavesQ4K output
// tiles over one K-slice of at most KB super-blocks.
// LDS: the slice's prepared activations, kQ4KBlockFrags half8 per super-block.
template <int KB>
__global__ void __launch_bounds__(64 * kWavesQ4K)
    gemm_q4k_kernel(const uint8_t *__restrict__ w, const half8_t *__restrict__ xp, float *__restrict__ y,
                    float *__restrict__ partials, int *__restrict__ counters, int n_out, int nb, int n_rows, int kb,
                    int n_slices) {
    extern __shared__ half8_t lds[];
    __shared__ int s_last;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int n = lane & 15, g = lane >> 4;
    const int group = blockIdx.x / n_slices;
    const int slice = blockIdx.x - group * n_slices;
    const int b0 = slice * kb;
    const int nblk = min(kb, nb - b0);
    const int tile = group * kWavesQ4K + wave;
    const int n_tiles = (n_out + 15) >> 4;
    const bool active = tile < n_tiles;
    const size_t row_bytes = static_cast<size_t>(nb) * DFL_Q4_K_BYTES;

    // Loads are unconditional (indices clamped into the slice) so that no control flow sits
    // between them: all of them are issued back to back and only then waited for.
    // 1. the K-slice's prepared activations: global -> registers (flat copy, tail clamped)
    constexpr int kCopies = (KB * kQ4KBlockFrags + 64 * kWavesQ4K - 1) / (64 * kWavesQ4K);
    const int n_frags = nblk * kQ4KBlockFrags;
    const half8_t *xsrc = xp + static_cast<int64_t>(b0) * kQ4KBlockFrags;
    half8_t xr[kCopies];
#pragma unroll
    for (int i = 0; i < kCopies; i++) xr[i] = xsrc[min(i * 64 * kWavesQ4K + tid, n_frags - 1)];

    // 2. every weight byte of this wave's tile and slice
    int row = tile * 16 + n;
    row = row < n_out ? row : n_out - 1;
    const uint8_t *rowp = w + static_cast<size_t>(row) * row_bytes + static_cast<size_t>(b0) * DFL_Q4_K_BYTES;
    uint4 hdr[KB], q0[KB], q1[KB];
#pragma unroll
    for (int i = 0; i < KB; i++) {
        const uint8_t *blk = rowp + min(i, nblk - 1) * DFL_Q4_K_BYTES;
        hdr[i] = *reinterpret_cast<const uint4 *>(blk);
        q0[i] = *reinterpret_cast<const uint4 *>(blk + 16 + 32 * g);
        q1[i] = *reinterpret_cast<const uint4 *>(blk + 32 + 32 * g);
    }
    __builtin_amdgcn_sched_barrier(0);  // everything above is in flight before anything below waits

    // 3. activations -> LDS (clamped duplicates rewrite the last entry with the same value)
#pragma unroll
    for (int i = 0; i < kCopies; i++) lds[min(i * 64 * kWavesQ4K + tid, n_frags - 1)] = xr[i];
    __syncthreads();

    // 4. main MFMAs.  Straight-line on purpose (a branch here lets the compiler sink the loads
    //    above into it): a slot past the end of a short slice re-reads the last super-block with
    //    its scales forced to zero, so it adds nothing.
    float4_t acc = {0, 0, 0, 0}, acc_min = {0, 0, 0, 0};
    const _Float16 zero = static_cast<_Float16>(0.0f);
#pragma unroll
    for (int i = 0; i < KB; i++) {
        // scales of sub-blocks 2g (low nibbles) and 2g+1 (high nibbles)
        uint32_t lo_sc = hdr[i].y & 0x3F3F3F3Fu;
        uint32_t hi_sc = (hdr[i].w & 0x0F0F0F0Fu) | ((hdr[i].y >> 2) & 0x30303030u);
        uint32_t sel = (g < 2 ? lo_sc : hi_sc) >> (16 * (g & 1));
        _Float16 d = (i < nblk) ? __builtin_bit_cast(half2_t, hdr[i].x)[0] : zero;
        _Float16 s_lo = byte_to_half(sel, 0) * d;
        _Float16 s_hi = byte_to_half(sel, 1) * d;
        half2_t s2l = splat(s_lo), c2l = splat(s_lo * static_cast<_Float16>(-1024.0f));
        half2_t s2h = splat(s_hi), c2h = splat(s_hi * static_cast<_Float16>(-64.0f));
        uint32_t qw[8] = {q0[i].x, q0[i].y, q0[i].z, q0[i].w, q1[i].x, q1[i].y, q1[i].z, q1[i].w};
        const half8_t *a = lds + min(i, nblk - 1) * kQ4KBlockFrags + lane;
#pragma unroll
        for (int t = 0; t < 4; t++) {
            half8_t bl = unpack_scale<false>(qw[2 * t], qw[2 * t + 1], s2l, c2l);
            acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[t * 64], bl, acc, 0, 0, 0);
        }
#pragma unroll
        for (int t = 0; t < 4; t++) {
            half8_t bh = unpack_scale<true>(qw[2 * t], qw[2 * t + 1], s2h, c2h);
            acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[(4 + t) * 64], bh, acc, 0, 0, 0);
        }
    }

    // 5. minima: lane (n, g) supplies the eight dmin*m_j of super-block 4q+g, against the
    //    sub-block sums of the same super-block
#pragma unroll
    for (int q = 0; q < (KB + 3) / 4; q++) {
        uint4 h = hdr[4 * q];
#pragma unroll
        for (int u = 1; u < 4; u++)
            if (4 * q + u < KB && g == u) h = hdr[4 * q + u];
        int blk = 4 * q + g;
        bool valid = blk < nblk;
        blk = valid ? blk : 0;
        _Float16 dmin = valid ? __builtin_bit_cast(half2_t, h.x)[1] : zero;
        uint32_t lo_m = h.z & 0x3F3F3F3Fu;
        uint32_t hi_m = ((h.w >> 4) & 0x0F0F0F0Fu) | ((h.z >> 2) & 0x30303030u);
        half8_t bm;
#pragma unroll
        for (int j = 0; j < 4; j++) {
            bm[j] = byte_to_half(lo_m, j) * dmin;
            bm[4 + j] = byte_to_half(hi_m, j) * dmin;
        }
        const half8_t *sums = lds + blk * kQ4KBlockFrags + 512 + n;
        acc_min = __builtin_amdgcn_mfma_f32_16x16x32_f16(sums[0], bm, acc_min, 0, 0, 0);
        acc_min = __builtin_amdgcn_mfma_f32_16x16x32_f16(sums[16], bm, acc_min, 0, 0, 0);
    }

    // 6. output: direct when K is not split, else partial tiles + last-arriver sum in slice order
    float4_t res = acc - acc_min;
    if (n_slices == 1) {
        if (active) {
            int orow = tile * 16 + n;
#pragma unroll
            for (int i = 0; i < 4; i++) {
                int m = 4 * g + i;
                if (m < n_rows && orow < n_out) y[static_cast<size_t>(m) * n_out + orow] = res[i];
            }
        }
        return;
    }
    // Partial tiles cross workgroups (and XCDs, whose L2s are not coherent with each other)
    // through agent-scope atomic stores and loads, which are performed at the coherent level
    // instruction by instruction.  A release fence here would write back the whole L2 once per
    // wave; waiting for this wave's own stores to complete before the arrival counter is
    // bumped gives the same ordering for the only data that matters.
    if (active) {
        float *p = partials + (static_cast<size_t>(slice) * n_tiles + tile) * 256;
#pragma unroll
        for (int i = 0; i < 4; i++)
            __hip_atomic_store(&p[(4 * g + i) * 16 + n], res[i], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (tid == 0)
        s_last = (__hip_atomic_fetch_add(&counters[group], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) ==
                  n_slices - 1);
    __syncthreads();
    if (!s_last) return;
    if (active) {
        float4_t sum = {0, 0, 0, 0};
        for (int s = 0; s < n_slices; s++) {
            const float *p = partials + (static_cast<size_t>(s) * n_tiles + tile) * 256;
#pragma unroll
            for (int i = 0; i < 4; i++)
                sum[i] += __hip_atomic_load(&p[(4 * g + i) * 16 + n], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        int orow = tile * 16 + n;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            int m = 4 * g + i;
            if (m < n_rows && orow < n_out) y[static_cast<size_t>(m) * n_out + orow] = sum[i];
        }
    }
    if (tid == 0) __hip_atomic_store(&counters[group], 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
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
        off = 0;
        xp = dfl_ws_take<half8_t>(ctx, &off, static_cast<size_t>(nb) * kQ4KBlockFrags * sizeof(half8_t));
        // K-slice length: 5 super-blocks when that divides K evenly, else 4
        int kb = env_int("DFLASH_GEMM_KB", (nb % 5 == 0) ? 5 : 4);
        if (kb < 1) kb = 1;
        if (kb > 8) kb = 8;
        if (kb > nb) kb = nb;
        const int n_slices = (nb + kb - 1) / kb;
        const int groups = (tiles + kWavesQ4K - 1) / kWavesQ4K;
        float *partials = nullptr;
        if (n_slices > 1)
            partials = dfl_ws_take<float>(ctx, &off, static_cast<size_t>(n_slices) * tiles * 256 * sizeof(float));
        if (!xp || (n_slices > 1 && !partials))
            return dfl_fail(ctx, DFLASH_ERR_WORKSPACE, "gemm_fewrow: workspace too small");
        if (groups > ctx->n_counters)
            return dfl_fail(ctx, DFLASH_ERR_BAD_SHAPE, "gemm_fewrow: n_out %lld needs more than %d tile groups",
                            static_cast<long long>(n_out), ctx->n_counters);
        {
            dfl_timed timer(ctx, st, DFL_T_PREP);
            if (x_type == DFLASH_TYPE_F32)
                prep_x_q4k_kernel<float><<<nb, 256, 0, st>>>(static_cast<const float *>(x), xp, n_rows, n_in);
            else
                prep_x_q4k_kernel<_Float16><<<nb, 256, 0, st>>>(static_cast<const _Float16 *>(x), xp, n_rows, n_in);
        }
        const uint8_t *wb = static_cast<const uint8_t *>(w);
        const int kbt = kb <= 4 ? 4 : (kb == 5 ? 5 : 8);
        const size_t lds = static_cast<size_t>(kbt) * kQ4KBlockFrags * sizeof(half8_t);
        const dim3 grid(static_cast<unsigned>(groups * n_slices));
        dfl_timed timer(ctx, st, DFL_T_GEMM);
#define DFL_LAUNCH_Q4K(KBT)                                                                                      \
    gemm_q4k_kernel<KBT><<<grid, 64 * kWavesQ4K, lds, st>>>(wb, xp, y, partials, ctx->counters,                  \
                                                           static_cast<int>(n_out), nb, n_rows, kb, n_slices)
        if (kbt == 4)
            DFL_LAUNCH_Q4K(4);
        else if (kbt == 5)
            DFL_LAUNCH_Q4K(5);
        else
            DFL_LAUNCH_Q4K(8);
#undef DFL_LAUNCH_Q4K
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
