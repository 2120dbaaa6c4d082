// Vector types and the quant-block -> f16 MFMA operand unpackers shared by the few-row GEMM kernels.
#pragma once

#include "common.h"

namespace {

typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float float4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));

__device__ __forceinline__ half2_t as_half2(uint32_t bits) { return __builtin_bit_cast(half2_t, bits); }

__device__ __forceinline__ half2_t splat(_Float16 v) {
    half2_t r = {v, v};
    return r;
}

// The f16 constants 1024.0 and 64.0 (as pairs) whose mantissas receive the nibbles.  They are
// passed through an empty asm once per kernel so the compiler sees VGPR values, not literals:
// (w & mask) | magic then selects as one v_and_or_b32 (mask in an SGPR) instead of two
// instructions with a literal each.
struct Q4KMagic {
    uint32_t lo, hi;
};
__device__ __forceinline__ Q4KMagic q4k_magic() {
    Q4KMagic m = {0x64006400u, 0x54005400u};
    asm volatile("" : "+v"(m.lo), "+v"(m.hi));
    return m;
}

// Eight f16 weights of one MFMA from two dwords of quant bytes.
//   HIGH = false: low nibbles,  1024 + q  via magic 0x6400, mask 0x000F
//   HIGH = true : high nibbles,   64 + q  via magic 0x5400, mask 0x00F0
// s2 = (s, s), c2 = (-1024 s, -1024 s) or (-64 s, -64 s).
template <bool HIGH>
__device__ __forceinline__ half8_t unpack_scale(uint32_t w0, uint32_t w1, half2_t s2, half2_t c2, uint32_t magic) {
    constexpr uint32_t mask = HIGH ? 0x00F000F0u : 0x000F000Fu;
    half2_t p0 = __builtin_elementwise_fma(as_half2((w0 & mask) | magic), s2, c2);
    half2_t p1 = __builtin_elementwise_fma(as_half2(((w0 >> 8) & mask) | magic), s2, c2);
    half2_t p2 = __builtin_elementwise_fma(as_half2((w1 & mask) | magic), s2, c2);
    half2_t p3 = __builtin_elementwise_fma(as_half2(((w1 >> 8) & mask) | magic), s2, c2);
    half8_t r = {p0[0], p0[1], p1[0], p1[1], p2[0], p2[1], p3[0], p3[1]};
    return r;
}

// Eight f16 weights of one MFMA: q = nibble | (two qh bits << 4), value round(q s).
//   HIGH = false: low nibbles, bits pre-shifted to 0..1:   1024 + q via magic 0x6400, c = -1024 s
//   HIGH = true : high nibbles (four bits up), qh bits go eight bits up: 64 + q via 0x5400, c = -64 s
template <bool HIGH>
__device__ __forceinline__ half8_t unpack6(uint32_t w0, uint32_t w1, uint32_t h0, uint32_t h1, half2_t s2, half2_t c2,
                                           uint32_t magic) {
    constexpr uint32_t mask = HIGH ? 0x00F000F0u : 0x000F000Fu;
    constexpr int up = HIGH ? 8 : 4;
    auto one = [&](uint32_t w, uint32_t h) {
        const uint32_t bits = ((w & mask) | magic) | ((h & 0x00030003u) << up);
        return __builtin_elementwise_fma(as_half2(bits), s2, c2);
    };
    const half2_t p0 = one(w0, h0), p1 = one(w0 >> 8, h0 >> 8), p2 = one(w1, h1), p3 = one(w1 >> 8, h1 >> 8);
    half8_t r = {p0[0], p0[1], p1[0], p1[1], p2[0], p2[1], p3[0], p3[1]};
    return r;
}

}  // namespace
