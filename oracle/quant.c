/*
 * CPU oracle, test infrastructure only: ggml block dequantisation.
 *
 * The reference dequantises through llama.cpp's `ggml_get_type_traits(t)->to_float`
 * (codec.rs:148-249; llama-cpp-sys-2 0.1.139, not vendored).  These loops restate
 * ggml's published `dequantize_row_*` and are pinned by the closed forms the
 * reference's own tests hold (codec.rs:474-577, metal/tests/q6_k_f32_tile.rs:46-107).
 * Compile with -ffp-contract=off: every value is two f32 products and (Q4_K) one
 * f32 subtraction, never a fused multiply-add.
 */
#include "dflash_oracle.h"

#include <string.h>

float orc_f16_to_f32(uint16_t h) {
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1fu;
    uint32_t man = h & 0x3ffu;
    uint32_t bits;
    if (exp == 0) {
        if (man == 0) {
            bits = sign;
        } else { /* subnormal: normalise */
            int shift = 0;
            while ((man & 0x400u) == 0) {
                man <<= 1;
                shift++;
            }
            man &= 0x3ffu;
            bits = sign | ((uint32_t)(127 - 15 - shift + 1) << 23) | (man << 13);
        }
    } else if (exp == 31) {
        bits = sign | 0x7f800000u | (man << 13);
    } else {
        bits = sign | ((exp + 127 - 15) << 23) | (man << 13);
    }
    float f;
    memcpy(&f, &bits, 4);
    return f;
}

uint16_t orc_f32_to_f16(float f) {
    uint32_t x;
    memcpy(&x, &f, 4);
    uint32_t sign = (x >> 16) & 0x8000u;
    uint32_t exp = (x >> 23) & 0xffu;
    uint32_t man = x & 0x7fffffu;
    if (exp == 255) { /* inf / nan */
        return (uint16_t)(sign | 0x7c00u | (man ? (0x200u | (man >> 13)) : 0));
    }
    int32_t e = (int32_t)exp - 127 + 15;
    if (e >= 31) return (uint16_t)(sign | 0x7c00u);
    if (e <= 0) {
        if (e < -10) return (uint16_t)sign;
        man |= 0x800000u;
        uint32_t shift = (uint32_t)(14 - e);
        uint32_t half = man >> shift;
        uint32_t rem = man & ((1u << shift) - 1);
        uint32_t mid = 1u << (shift - 1);
        if (rem > mid || (rem == mid && (half & 1))) half++;
        return (uint16_t)(sign | half);
    }
    uint32_t half = ((uint32_t)e << 10) | (man >> 13);
    uint32_t rem = man & 0x1fffu;
    if (rem > 0x1000u || (rem == 0x1000u && (half & 1))) half++;
    return (uint16_t)(sign | half);
}

static uint16_t rd16(const uint8_t *p) { return (uint16_t)(p[0] | (p[1] << 8)); }

/* 6-bit scale/min unpack: codec.rs:541-553 builds the inverse; GPU form
 * kernels/mat_mat_fewrow_gen.metal:45-69. */
static void q4k_scale_min(int j, const uint8_t *s, uint8_t *sc, uint8_t *m) {
    if (j < 4) {
        *sc = s[j] & 63;
        *m = s[j + 4] & 63;
    } else {
        *sc = (uint8_t)((s[j + 4] & 0x0f) | ((s[j - 4] >> 6) << 4));
        *m = (uint8_t)((s[j + 4] >> 4) | ((s[j] >> 6) << 4));
    }
}

/* Q4_K: 144 B / 256 elems: half d; half dmin; u8 scales[12]; u8 qs[128].
 * codec.rs:541-577 (expected = d*sc*q - dmin*m, f32). */
int orc_dequant_q4_k(const uint8_t *blocks, size_t n_elems, float *out) {
    if (n_elems % ORC_QK_K) return -1;
    size_t nb = n_elems / ORC_QK_K;
    for (size_t b = 0; b < nb; b++) {
        const uint8_t *blk = blocks + b * ORC_Q4_K_BYTES;
        float d = orc_f16_to_f32(rd16(blk));
        float dmin = orc_f16_to_f32(rd16(blk + 2));
        const uint8_t *scales = blk + 4;
        const uint8_t *qs = blk + 16;
        float *y = out + b * ORC_QK_K;
        for (int chunk = 0; chunk < 4; chunk++) {
            uint8_t sc, m;
            q4k_scale_min(2 * chunk, scales, &sc, &m);
            float d1 = d * (float)sc;
            float m1 = dmin * (float)m;
            q4k_scale_min(2 * chunk + 1, scales, &sc, &m);
            float d2 = d * (float)sc;
            float m2 = dmin * (float)m;
            for (int l = 0; l < 32; l++) y[chunk * 64 + l] = d1 * (float)(qs[chunk * 32 + l] & 0xf) - m1;
            for (int l = 0; l < 32; l++) y[chunk * 64 + 32 + l] = d2 * (float)(qs[chunk * 32 + l] >> 4) - m2;
        }
    }
    return 0;
}

/* Q6_K: 210 B / 256 elems: u8 ql[128]; u8 qh[64]; i8 scales[16]; half d.
 * metal/tests/q6_k_f32_tile.rs:46-71 (y = d * scale * q, left to right). */
int orc_dequant_q6_k(const uint8_t *blocks, size_t n_elems, float *out) {
    if (n_elems % ORC_QK_K) return -1;
    size_t nb = n_elems / ORC_QK_K;
    for (size_t b = 0; b < nb; b++) {
        const uint8_t *blk = blocks + b * ORC_Q6_K_BYTES;
        float d = orc_f16_to_f32(rd16(blk + 208));
        float *y = out + b * ORC_QK_K;
        for (int n = 0; n < 2; n++) {
            const uint8_t *ql = blk + 64 * n;
            const uint8_t *qh = blk + 128 + 32 * n;
            const int8_t *sc = (const int8_t *)(blk + 192 + 8 * n);
            for (int l = 0; l < 32; l++) {
                int is = l / 16;
                int q1 = (int)((ql[l] & 0xf) | ((qh[l] & 3) << 4)) - 32;
                int q2 = (int)((ql[l + 32] & 0xf) | (((qh[l] >> 2) & 3) << 4)) - 32;
                int q3 = (int)((ql[l] >> 4) | (((qh[l] >> 4) & 3) << 4)) - 32;
                int q4 = (int)((ql[l + 32] >> 4) | (((qh[l] >> 6) & 3) << 4)) - 32;
                y[128 * n + l] = d * (float)sc[is] * (float)q1;
                y[128 * n + l + 32] = d * (float)sc[is + 2] * (float)q2;
                y[128 * n + l + 64] = d * (float)sc[is + 4] * (float)q3;
                y[128 * n + l + 96] = d * (float)sc[is + 6] * (float)q4;
            }
        }
    }
    return 0;
}

/* Q8_0: 34 B / 32 elems: half d; i8 qs[32].  codec.rs:474-487. */
int orc_dequant_q8_0(const uint8_t *blocks, size_t n_elems, float *out) {
    if (n_elems % ORC_QK8_0) return -1;
    size_t nb = n_elems / ORC_QK8_0;
    for (size_t b = 0; b < nb; b++) {
        const uint8_t *blk = blocks + b * ORC_Q8_0_BYTES;
        float d = orc_f16_to_f32(rd16(blk));
        const int8_t *qs = (const int8_t *)(blk + 2);
        for (int i = 0; i < 32; i++) out[b * 32 + i] = d * (float)qs[i];
    }
    return 0;
}

int orc_dequant(int type, const uint8_t *blocks, size_t n_elems, float *out) {
    switch (type) {
    case ORC_Q4_K: return orc_dequant_q4_k(blocks, n_elems, out);
    case ORC_Q6_K: return orc_dequant_q6_k(blocks, n_elems, out);
    case ORC_Q8_0: return orc_dequant_q8_0(blocks, n_elems, out);
    /* unquantised tensors (tensor.rs:164-208): F32 as stored, F16 widened exactly */
    case ORC_F32: memcpy(out, blocks, n_elems * 4); return 0;
    case ORC_F16:
        for (size_t i = 0; i < n_elems; i++) {
            uint16_t bits;
            memcpy(&bits, blocks + 2 * i, 2);
            out[i] = orc_f16_to_f32(bits);
        }
        return 0;
    default: return -1;
    }
}

/* tensor.rs:164-208 */
size_t orc_row_bytes(int type, size_t n_in) {
    switch (type) {
    case ORC_Q4_K: return n_in / ORC_QK_K * ORC_Q4_K_BYTES;
    case ORC_Q6_K: return n_in / ORC_QK_K * ORC_Q6_K_BYTES;
    case ORC_Q8_0: return n_in / ORC_QK8_0 * ORC_Q8_0_BYTES;
    case ORC_F32: return n_in * 4;
    case ORC_F16: return n_in * 2;
    default: return 0;
    }
}
