// Routing of one block row by one wave, for n_expert <= 256 and n_used <= 64: softmax over the router logits, top-k
// (higher probability first, equal probabilities to the lower expert id), renormalised weights in pick order (the
// reference's packed route, metal_dflash.rs:10184-10403; CPU form ffn_moe, forward.rs:749-824), and the row's picked
// experts as a 256-bit mask.  Shared by the stand-alone routing kernel (moe.hip) and the expert GEMM kernel that
// derives the block's expert list itself (gemm_fewrow.hip): same instructions, same order, same bits.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>

namespace dfl_route {

// Maximum of a float over the wave, in every lane: data-parallel-primitive moves within rows of 16 lanes (shift right
// by 1, 2, 4, 8: lane 15 of a row then holds the row's maximum), then lane 15 of rows 0 and 2 broadcast into rows 1
// and 3, then lane 31 into rows 2 and 3; lane 63 has the result.  NaN operands are ignored, as v_max_f32 does; lanes
// without a source keep their own value.  No LDS round trips, unlike a shuffle.
__device__ __forceinline__ float wave_max_f32(float v) {
    // One v_max_f32 with a DPP source per step.  (Written through update_dpp + fmaxf the compiler emits a copy, the
    // move, a canonicalising maximum and the maximum: five instructions a step, thirty a call, and every workgroup of an
    // expert launch makes eight calls per row with four waves on a SIMD before it can ask for its first weight byte.)
    // A lane without a source keeps its value (bound_ctrl off); two wait states between a write of v and its DPP read.
    asm volatile(
        "s_nop 1\n\tv_max_f32_dpp %0, %0, %0 row_shr:1 row_mask:0xf bank_mask:0xf\n\t"
        "s_nop 1\n\tv_max_f32_dpp %0, %0, %0 row_shr:2 row_mask:0xf bank_mask:0xf\n\t"
        "s_nop 1\n\tv_max_f32_dpp %0, %0, %0 row_shr:4 row_mask:0xf bank_mask:0xf\n\t"
        "s_nop 1\n\tv_max_f32_dpp %0, %0, %0 row_shr:8 row_mask:0xf bank_mask:0xf\n\t"
        "s_nop 1\n\tv_max_f32_dpp %0, %0, %0 row_bcast:15 row_mask:0xa bank_mask:0xf\n\t"
        "s_nop 1\n\tv_max_f32_dpp %0, %0, %0 row_bcast:31 row_mask:0xc bank_mask:0xf\n\t"
        "s_nop 1"
        : "+v"(v));
    return __uint_as_float(__builtin_amdgcn_readlane(__float_as_uint(v), 63));
}

// The sum over the wave by the same moves (lanes without a source add 0): lane 63 ends with
// ((row 0 + row 1) + (row 2 + row 3)), each row summed lane 0 upwards in a tree of shifts; every lane gets that value.
__device__ __forceinline__ float wave_sum_f32(float v) {
#define DFL_FADD_STEP(ctrl, row_mask) \
    v += __uint_as_float(__builtin_amdgcn_update_dpp(0u, __float_as_uint(v), ctrl, row_mask, 0xf, false))
    DFL_FADD_STEP(0x111, 0xf);
    DFL_FADD_STEP(0x112, 0xf);
    DFL_FADD_STEP(0x114, 0xf);
    DFL_FADD_STEP(0x118, 0xf);
    DFL_FADD_STEP(0x142, 0xa);
    DFL_FADD_STEP(0x143, 0xc);
#undef DFL_FADD_STEP
    return __uint_as_float(__builtin_amdgcn_readlane(__float_as_uint(v), 63));
}

struct RowPicks {
    int my_e;                  // lane k < n_used: the expert of pick k
    float my_w;                // lane k < n_used: its renormalised weight
    unsigned long long m[4];   // the row's picked experts (every lane)
};

// lg: the row's n_expert router logits (n_expert <= 64 kRegs: kRegs probabilities per lane).  Called by all 64 lanes of a wave.
// lgv[j]: logit of expert lane + 64 j, -infinity past n_expert.
template <int kRegs>
__device__ __forceinline__ RowPicks route_row_loaded(const float (&lgv)[kRegs], int n_expert, int n_used, int lane) {
    RowPicks r;
    r.my_e = 0;
    r.m[0] = r.m[1] = r.m[2] = r.m[3] = 0;
    float mx = -INFINITY;
#pragma unroll
    for (int j = 0; j < kRegs; j++) mx = fmaxf(mx, lgv[j]);
    mx = wave_max_f32(mx);
    float pv[kRegs];
    float sum = 0.0f;
#pragma unroll
    for (int j = 0; j < kRegs; j++) {
        pv[j] = 0.0f;
        if (lane + 64 * j < n_expert) {
            pv[j] = expf(lgv[j] - mx);
            sum += pv[j];
        }
    }
    sum = wave_sum_f32(sum);
    const float inv = 1.0f / sum;
#pragma unroll
    for (int j = 0; j < kRegs; j++) pv[j] = lane + 64 * j < n_expert ? pv[j] * inv : -1.0f;  // no such expert: never picked

    // pick k = the highest remaining probability, equal probabilities to the lower id: a wave-wide float maximum
    // (one DPP instruction per step), then the first lane / register that holds it, found with compares into scalar
    // masks.  Taken and missing experts are -1, NaN never compares equal: if nothing is left (NaN logits) the pick
    // falls back to an index in range.
    float my_p = 0.0f;
    for (int k = 0; k < n_used; k++) {
        float lmax = pv[0];
#pragma unroll
        for (int j = 1; j < kRegs; j++) lmax = fmaxf(lmax, pv[j]);
        const float pmax = wave_max_f32(lmax);
        int e_win = -1;
#pragma unroll
        for (int j = kRegs - 1; j >= 0; j--) {
            const unsigned long long hit = __builtin_amdgcn_ballot_w64(pv[j] == pmax);
            if (hit) e_win = 64 * j + __builtin_ctzll(hit);
        }
        const bool none = !(pmax >= 0.0f) || e_win < 0;
        if (none) e_win = k < n_expert ? k : n_expert - 1;
        if (lane == k) {
            r.my_e = e_win;
            my_p = none ? 0.0f : pmax;
        }
#pragma unroll
        for (int j = 0; j < 4; j++) {
            if (j < kRegs && lane + 64 * j == e_win) pv[j < kRegs ? j : 0] = -1.0f;  // taken
            if ((e_win >> 6) == j) r.m[j] |= 1ull << (e_win & 63);
        }
    }
    float wsum = 0.0f;
    for (int k = 0; k < n_used; k++) wsum += __uint_as_float(__builtin_amdgcn_readlane(__float_as_uint(my_p), k));  // in pick order
    wsum = fmaxf(wsum, 6.103515625e-05f);  // 2^-14
    r.my_w = my_p / wsum;
    return r;
}

// n_expert <= 256.  The common 128-expert router keeps two probabilities per lane instead of four: the same
// arithmetic on the same values in the same order (the registers it drops hold "no such expert"), half the
// per-pick work, which every workgroup of the expert launch spends before its first weight byte.
template <int kRegs>
__device__ __forceinline__ RowPicks route_row_regs(const float *__restrict__ lg, int n_expert, int n_used, int lane) {
    float lgv[kRegs];
#pragma unroll
    for (int j = 0; j < kRegs; j++) lgv[j] = lane + 64 * j < n_expert ? lg[lane + 64 * j] : -INFINITY;
    return route_row_loaded<kRegs>(lgv, n_expert, n_used, lane);
}
__device__ __forceinline__ RowPicks route_row(const float *__restrict__ lg, int n_expert, int n_used, int lane) {
    if (n_expert <= 128) return route_row_regs<2>(lg, n_expert, n_used, lane);
    return route_row_regs<4>(lg, n_expert, n_used, lane);
}
// The same from four logits per lane already in registers (a caller that loads them itself, ahead of other traffic).
__device__ __forceinline__ RowPicks route_row_from(const float (&lgv)[4], int n_expert, int n_used, int lane) {
    if (n_expert <= 128) {
        const float two[2] = {lgv[0], lgv[1]};
        return route_row_loaded<2>(two, n_expert, n_used, lane);
    }
    return route_row_loaded<4>(lgv, n_expert, n_used, lane);
}

// v[i & 3] without indexing the array by a run-time value (which would move it from registers to scratch memory)
__device__ __forceinline__ unsigned long long pick4(const unsigned long long v[4], int i) {
    i &= 3;
    return i == 0 ? v[0] : i == 1 ? v[1] : i == 2 ? v[2] : v[3];
}

// The union of the sixteen rows' masks (row_mask[row * 4 + j] in LDS, complete): lane l reads word l, four xor-shuffle
// steps OR the rows together, and words 0..3 are read back out of lanes 0..3.  Called by a whole wave.
__device__ __forceinline__ void union_of_rows(const unsigned long long *row_mask, int lane, unsigned long long un[4]) {
    unsigned long long v = row_mask[lane];
    for (int off = 4; off < 64; off <<= 1) {
        const unsigned lo = __shfl_xor(static_cast<unsigned>(v), off, 64), hi = __shfl_xor(static_cast<unsigned>(v >> 32), off, 64);
        v |= (static_cast<unsigned long long>(hi) << 32) | lo;
    }
#pragma unroll
    for (int j = 0; j < 4; j++) {
        // (readlane returns int: through unsigned, or a low word with bit 31 set would smear over the high word)
        const unsigned lo = static_cast<unsigned>(__builtin_amdgcn_readlane(static_cast<unsigned>(v), j));
        const unsigned hi = static_cast<unsigned>(__builtin_amdgcn_readlane(static_cast<unsigned>(v >> 32), j));
        un[j] = (static_cast<unsigned long long>(hi) << 32) | lo;
    }
}

// experts below e in the union of the rows' masks = e's slot in the block's ascending expert list
__device__ __forceinline__ int slot_below(const unsigned long long un[4], int e) {
    int below = 0;
#pragma unroll
    for (int j = 0; j < 4; j++) {
        if (j < (e >> 6)) below += __popcll(un[j]);
        if (j == (e >> 6)) below += __popcll(un[j] & ((1ull << (e & 63)) - 1));
    }
    return below;
}

}  // namespace dfl_route
