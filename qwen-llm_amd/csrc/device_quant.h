// Element-wise device dequantisers, bit-exact with ggml's dequantize_row_{q4_K,q6_K,q8_0}
// (y = (d*sc)*q - (dmin*m), y = (d*sc)*(q-32), y = d*q; every product rounded separately).
// The compiler may fuse the last multiply into the subtraction; that changes nothing: d (f16, 11
// bits) x a 6-8 bit code x a 4-6 bit quant is at most 24 bits and exact in f32, so the fused and
// the separately rounded forms agree on every input.
#pragma once

#include "common.h"

__device__ __forceinline__ float dfl_h2f(const uint8_t *p) {
    return __half2float(__ushort_as_half(static_cast<unsigned short>(p[0] | (p[1] << 8))));
}

// 6-bit scale / min of sub-block j from the 12 packed bytes of a Q4_K super-block
__device__ __forceinline__ void dfl_q4k_scale_min(const uint8_t *s, int j, int *sc, int *m) {
    if (j < 4) {
        *sc = s[j] & 63;
        *m = s[j + 4] & 63;
    } else {
        *sc = (s[j + 4] & 0x0f) | ((s[j - 4] >> 6) << 4);
        *m = (s[j + 4] >> 4) | ((s[j] >> 6) << 4);
    }
}

// One element of a quantised row.
__device__ inline float dfl_dequant_elem(int type, const uint8_t *row, int e) {
    if (type == DFLASH_TYPE_F32) return reinterpret_cast<const float *>(row)[e];
    if (type == DFLASH_TYPE_Q8_0) {
        const uint8_t *blk = row + (e >> 5) * DFL_Q8_0_BYTES;
        return __fmul_rn(dfl_h2f(blk), static_cast<float>(reinterpret_cast<const int8_t *>(blk + 2)[e & 31]));
    }
    if (type == DFLASH_TYPE_Q4_K) {
        const uint8_t *blk = row + (e >> 8) * DFL_Q4_K_BYTES;
        const int i = e & 255, j = i >> 5, l = i & 31;
        int sc, m;
        dfl_q4k_scale_min(blk + 4, j, &sc, &m);
        const uint8_t byte = blk[16 + 32 * (j >> 1) + l];
        const int q = (j & 1) ? (byte >> 4) : (byte & 0x0f);
        const float d1 = __fmul_rn(dfl_h2f(blk), static_cast<float>(sc));
        const float m1 = __fmul_rn(dfl_h2f(blk + 2), static_cast<float>(m));
        return __fsub_rn(__fmul_rn(d1, static_cast<float>(q)), m1);
    }
    // Q6_K
    const uint8_t *blk = row + (e >> 8) * DFL_Q6_K_BYTES;
    const int i = e & 255, n = i >> 7, r = i & 127, k = r >> 5, l = r & 31;
    const uint8_t *ql = blk + 64 * n;
    const uint8_t *qh = blk + 128 + 32 * n;
    const int8_t *sc = reinterpret_cast<const int8_t *>(blk + 192 + 8 * n);
    int lo = (k & 1) ? ql[l + 32] : ql[l];
    lo = (k & 2) ? (lo >> 4) : (lo & 0x0f);
    const int hi = (qh[l] >> (2 * k)) & 3;
    const float ds = __fmul_rn(dfl_h2f(blk + 208), static_cast<float>(sc[(l >> 4) + 2 * k]));
    return __fmul_rn(ds, static_cast<float>((lo | (hi << 4)) - 32));
}

// The 32 consecutive elements [32*sb, 32*sb+32) of a quantised row.
__device__ inline void dfl_dequant_sub32(int type, const uint8_t *row, int sb, float *w) {
    if (type == DFLASH_TYPE_Q4_K) {
        const uint8_t *blk = row + (sb >> 3) * DFL_Q4_K_BYTES;
        const int j = sb & 7;
        int sc, m;
        dfl_q4k_scale_min(blk + 4, j, &sc, &m);
        const float d1 = __fmul_rn(dfl_h2f(blk), static_cast<float>(sc));
        const float m1 = __fmul_rn(dfl_h2f(blk + 2), static_cast<float>(m));
        const uint32_t *qs = reinterpret_cast<const uint32_t *>(blk + 16 + 32 * (j >> 1));  // 4-byte aligned
        const int shift = (j & 1) * 4;
#pragma unroll
        for (int v = 0; v < 8; v++) {
            const uint32_t word = qs[v] >> shift;
#pragma unroll
            for (int b = 0; b < 4; b++)
                w[4 * v + b] = __fsub_rn(__fmul_rn(d1, static_cast<float>((word >> (8 * b)) & 0x0f)), m1);
        }
        return;
    }
#pragma unroll 4
    for (int i = 0; i < 32; i++) w[i] = dfl_dequant_elem(type, row, 32 * sb + i);
}
