// Few-row quantised GEMM for the 16-row verify block:
//   Y[n_rows][n_out] = X[n_rows][n_in] . W^T,   W = ggml quant blocks, row-major.
// Replaces encode_mat_mat_dispatch_dflash_verify (metal_forward/dispatch.rs:365-378)
// and its kernel (kernels/mat_mat_fewrow_gen.metal:374-474).
//
// Mapping onto CDNA4.  The 16 block rows are exactly the M side of
// v_mfma_f32_16x16x32_f16, so a wave owns 16 weight rows (one output tile) and
// streams them along K; lane l serves weight row l%16 and the k-octet l/16.
//
//  * Q4_K: nibbles are turned into exact f16 integers by OR-ing them into the mantissa
//    of 1024.0 (low nibble) or 64.0 (high nibble, which sits four bits up), and one
//    packed f16 fma per value pair, fma(1024+q, s, -1024*s), yields round(q*s) with a
//    single rounding (s = d*sc_j in f16).  The per-sub-block minimum never touches the
//    nibbles: each weight MFMA has a twin that multiplies the same activation fragment
//    with dmin*m_j repeated eight times and accumulates into a second tile, subtracted
//    at the end.  The matrix cores are nearly idle in this kernel and the vector ALU is
//    not, so this is cheaper than pre-summing activations.
//  * The kernel is a persistent stream: one workgroup per CU walks a contiguous range of
//    (tile group x super-block) work, weights go HBM -> LDS with direct-to-LDS loads
//    through a ring of buffers, activations are converted to f16 MFMA fragments on the
//    way into the same ring.  See the comment on the kernel for the pipeline.
//  * K is split where the ranges cut a tile group; partial tiles are added by a second
//    small kernel in a fixed order, so results are run-to-run deterministic.
//  * Q6_K has its own kernel (half a super-block per step, see there); Q8_0 uses a simple one:
//    eight consecutive weights per lane are dequantised to f16 and fed to the same MFMA.
#include "common.h"
#include "device_quant.h"
#include "mfma_unpack.h"
#include "moe_route.h"

#include <hip/hip_ext.h>

#include <algorithm>
#include <cstdlib>
#include <cstring>
#include <mutex>

namespace {

constexpr int kMaxSplit = 16;

// ----------------------------------------------------------------------------
// Q4_K kernel
// ----------------------------------------------------------------------------

// Activation fragments of one super-block b in LDS: kQ4KBlockFrags (= 512) half8 entries:
//   [t*64 + lane], t = 0..7 : A fragment of MFMA t for lane (m = lane%16, g = lane/16),
//        value i:  k = 256 b + 64 g + 8 t + perm[i],
//        perm = {0,2,1,3,4,6,5,7}: the order in which the nibble unpack emits a lane's values.
constexpr int kQ4KBlockFrags = 512;

// Byte j of `v` (0..255) as an exact f16.
__device__ __forceinline__ _Float16 byte_to_half(uint32_t v, int j) {
    return static_cast<_Float16>(static_cast<float>((v >> (8 * j)) & 0xffu));
}

// Streaming Q4_K kernel.
//
// Work split.  The iteration space is (tile group) x (super-block), flattened group-major; a
// tile group is kWaves consecutive output tiles (16 weight rows each), one per wave of a
// workgroup.  The grid is one workgroup per CU and workgroup i owns the contiguous range
// [T i / G, T (i+1) / G) of that space, so every CU streams the same number of weight bytes
// whatever the shape.
//
// Data path.  A stage is one super-block of one tile group.  Its 16*kWaves weight rows (144
// contiguous bytes each) are copied global -> LDS by global_load_lds_dwordx4: consecutive lanes
// take consecutive 16-byte pieces, so HBM sees row-contiguous requests and no VGPR is held
// while a load is in flight; the piece -> address map of a lane is the same in every stage
// (only a uniform base moves), so a load costs no vector ALU work.  The stage's activations
// (16 rows x 256 values, straight from the caller's f32 or f16 matrix, L2-resident) are loaded
// into registers three stages ahead, rounded to f16, and written to LDS in MFMA fragment order
// together with their sub-block sums one stage ahead.  Three weight buffers rotate (while stage d
// is computed out of one, the weights of d+1 and d+2 are landing in the other two) and two
// activation buffers alternate.  The loads are issued between the MFMAs of
// the stage being computed (one weight load after every second MFMA, then the activations), in
// the same order in every wave, which makes "everything but the youngest group of loads has
// landed" a constant s_waitcnt at the top of a stage.  Waves then read their tile's quant bytes
// and A fragments with ds_read_b128 (row stride 9 pieces: conflict-free).  All per-stage
// bookkeeping is a handful of scalar additions: the scalar unit is shared by the CU's waves.
//
// Split K.  When a range leaves a tile group, the accumulators are flushed: straight to Y if
// this workgroup covered the group's whole K, else as a partial tile, which a second, chip-wide
// kernel adds up in workgroup order (deterministic sums, no spinning, no atomics).
template <int kWaves>
struct Q4KGeom {
    static constexpr int kThreads = 64 * kWaves;
    static constexpr int kRows = 16 * kWaves;
    static constexpr int kWPieces = kRows * 9;              // 16-byte pieces of weights per stage
    static constexpr int kWaveLoads = kWPieces / 64;        // weight wave-loads per stage
    static constexpr int kFull = kWaveLoads / kWaves;       // ... every wave issues this many,
    static constexpr int kExtra = kWaveLoads % kWaves;      // ... and waves below kExtra one more
    static constexpr int kXLoads = 16 / kWaves;             // activation loads per thread and stage
    // Weight stages in flight ahead of the one being computed.  A workgroup streams only as fast as
    // (bytes in flight) / (memory latency): with two 18 KB stages in flight an 8-wave group gets
    // ~14 KB/us whatever the rest of the chip does, so it keeps more of them in flight; a 16-wave
    // group's stages are twice the size and LDS holds no more than three of them.
#ifndef DFLASH_Q4K_AHEAD8
#define DFLASH_Q4K_AHEAD8 4
#endif
    static constexpr int kAhead = kWaves == 8 ? DFLASH_Q4K_AHEAD8 : 2;
    static constexpr int kRing = kAhead + 1;
    // LDS: a ring of kRing weight buffers, then two activation buffers (stage parity)
    static constexpr int kLdsPieces = kRing * kWPieces + 2 * kQ4KBlockFrags;
    static_assert(kLdsPieces * 16 <= 160 * 1024, "fits one CU's LDS");
    static_assert(kWPieces % 64 == 0, "whole wave-loads");
    static_assert(kFull + (kExtra ? 1 : 0) <= 4, "one weight load is issued after every second of a stage's 8 MFMAs");
    static_assert(kXLoads == 1 || kXLoads == 2, "8 or 16 waves");
};

// A workgroup-uniform pointer the compiler cannot prove uniform (it depends on a loaded matrix
// index): moved to scalar registers so that stepping it and adding it to loads is scalar work.
__device__ __forceinline__ const uint8_t *q4k_uniform(const uint8_t *p) {
    const uint64_t v = reinterpret_cast<uint64_t>(p);
    const uint32_t lo = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(v));
    const uint32_t hi = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(v >> 32));
    return reinterpret_cast<const uint8_t *>((static_cast<uint64_t>(hi) << 32) | lo);
}

typedef const __attribute__((address_space(1))) void *gptr_t;
typedef __attribute__((address_space(3))) void *lptr_t;

// Division of a 31-bit value by a divisor the host knows: n / d = (n * mul) >> (32 + shift), with
// mul = floor(2^(31 + L) / d) + 1, shift = L - 1, L = ceil(log2 d) (mul == 0 stands for d == 1).
// The kernel's work split is all uniform integer arithmetic, done by sixteen waves on one
// scalar unit: a generic division there costs tens of instructions, this one two.
struct Q4KDiv {
    uint32_t mul, shift;
};
__host__ __device__ __forceinline__ uint32_t q4k_div(uint32_t n, Q4KDiv f) {
#ifdef __HIP_DEVICE_COMPILE__
    return f.mul ? (__umulhi(n, f.mul) >> f.shift) : n;
#else
    return f.mul ? static_cast<uint32_t>((static_cast<uint64_t>(n) * f.mul) >> (32 + f.shift)) : n;
#endif
}
inline Q4KDiv q4k_make_div(uint32_t d) {
    if (d <= 1) return {0, 0};
    uint32_t L = 0;
    while ((1ull << L) < d) L++;
    return {static_cast<uint32_t>((1ull << (31 + L)) / d + 1), L - 1};
}

// index of the workgroup whose range contains flattened iteration `it`
// (all of this index arithmetic fits 32 bits: the host checks total * n_wg < 2^31)
__device__ __forceinline__ int q4k_wg_of(int it, int total, int n_wg) {
    return static_cast<int>((static_cast<uint32_t>(it + 1) * n_wg + total - 1) / static_cast<uint32_t>(total)) - 1;
}

struct Q4KRange {
    int total, it_begin, it_end;
    int nb, n_wg, first_group;
    int wg;  // this workgroup's position in the range order (not its dispatch index)
};

// Range order.  Workgroups are dispatched round-robin over the 8 XCDs, each with its own L2.
// Consecutive ranges share weight rows (their boundary cache lines), activation blocks and
// split-K partial tiles, so they are given to workgroups of the same XCD: dispatch index i
// serves range (i mod 8) * (n / 8) + i / 8 when the count is a multiple of 8.
__device__ __forceinline__ int q4k_range_index(int dispatch, int n_wg) {
    if (n_wg % 8) return dispatch;
    return (dispatch & 7) * (n_wg >> 3) + (dispatch >> 3);
}

// Batched mode (mixture-of-experts): the tile groups of several same-shaped matrices, picked out of
// a stack by a device-side list, form one iteration space.  Global group index = slot *
// groups_per_mat + local group; slot j uses matrix ids[j], activations x + j * x_stride and
// output y + j * y_stride.  ids == nullptr: one matrix, one slot.
struct Q4KBatch {
    const int32_t *ids;      // [*n_slots] matrix index per slot; -1 = the extra matrix
    const uint8_t *extra_w;  // a same-shaped matrix outside the stack (may be null if no id is -1)
    const int32_t *n_slots;  // device scalar
    size_t w_stride;         // bytes between matrices of the stack
    size_t x_stride;         // activation elements between slots (0: all slots share x)
    size_t y_stride;         // output floats between slots
    int groups_per_mat;
    Q4KDiv by_gpm, by_nb, by_wg;  // dividers by groups_per_mat, super-blocks per row, workgroup count
    // Ranges are cut at tile-group boundaries only: no split K, so a (row, matrix) result does not
    // depend on which other matrices take part (a verify block and a single-token pass then agree
    // bit for bit), at the price of coarser load balance.
    int whole_groups;
    // SwiGLU pair mode (needs whole_groups): slot j stands for TWO matrices, ids[j] of this stack
    // (gate) and ids[j] of a second stack w2 / extra_w2 (up), and y gets silu(x . gate^T) * (x . up^T).
    // In the kernel's iteration space every tile group appears twice in a row (virtual group 2 g is
    // the gate half, 2 g + 1 the up half of real group g); ranges are cut between pairs, the gate
    // tile waits in registers while the up tile is computed.
    int pair;
    const uint8_t *w2, *extra_w2;
    int y_f16;  // the output is f16 (gemm_q4k_experts_kernel only)
    // routing folded into gemm_q4k_experts_kernel (route_logits != null): ids / n_slots are written, not read
    const float *route_logits;
    int route_experts, route_used, route_shared;
    int32_t *route_sel_e, *route_slot_of;
    float *route_sel_w;
};

// Tiled order (see gemm_q4k_tiled_kernel): one wave's 16 rows of a stage, and a whole 256-row stage, in bytes.
constexpr int kTiledTileBytes = 16 * DFL_Q4_K_BYTES;    // 2304
constexpr int kTiledStageBytes = 16 * kTiledTileBytes;  // 36864

// Per-lane constants of the loads and of the activation write, set up once per kernel.
template <int kWaves>
struct Q4KLane {
    uint32_t w_off[Q4KGeom<kWaves>::kFull + 1];  // weight piece: byte offset from (group's first row, super-block)
    uint32_t x_off[Q4KGeom<kWaves>::kXLoads];    // activation vector: byte offset from x[0][256 b]
    uint32_t xw_off[Q4KGeom<kWaves>::kXLoads];   // its fragment half in LDS: byte offset from the activation buffer
    uint32_t sc_sel;                             // byte selector of this lane's two scale codes (see q4k_compute)
};

// Rows past n_out (ragged last group) re-read the last row; their results are never stored.
template <int kWaves>
__device__ __forceinline__ void q4k_lane_w_offsets(Q4KLane<kWaves> &L, int tid, int row0, int n_out,
                                                   uint32_t row_bytes, bool tiled = false) {
    using G = Q4KGeom<kWaves>;
    const int lane = tid & 63, wave = tid >> 6;
    const int last = n_out - 1 - row0;
#pragma unroll
    for (int j = 0; j <= G::kFull; j++) {
        const int p = min((j * kWaves + wave) * 64 + lane, G::kWPieces - 1);
        const int r = min(p / 9, last);
        // tiled order: a stage is its LDS image, 256 rows x 144 bytes in one piece (padding rows exist)
        L.w_off[j] = tiled ? static_cast<uint32_t>(p) * 16u : static_cast<uint32_t>(r) * row_bytes + static_cast<uint32_t>(p % 9) * 16u;
    }
}

// Activation item of (virtual wave vw = wave + kWaves r, lane l): row m = 8 (vw & 1) + (l & 7),
// four values k = 4c .. 4c+3 with c = 8 (vw >> 1) + (l >> 3): a virtual wave is one sub-block of
// eight rows, its global loads are eight 128-byte runs and its LDS writes are conflict-free.
template <int kWaves, typename XT>
__device__ __forceinline__ void q4k_lane_x_offsets(Q4KLane<kWaves> &L, int tid, int n_rows, uint32_t n_in) {
    using G = Q4KGeom<kWaves>;
    const int lane = tid & 63, wave = tid >> 6;
    L.sc_sel = (lane & 16) ? 0x04030402u : 0x04010400u;
#pragma unroll
    for (int r = 0; r < G::kXLoads; r++) {
        const int vw = wave + kWaves * r;
        const int m = 8 * (vw & 1) + (lane & 7), c = 8 * (vw >> 1) + (lane >> 3);
        const int g = c >> 4, c15 = c & 15;
        L.x_off[r] = (static_cast<uint32_t>(min(m, n_rows - 1)) * n_in + 4u * c) * static_cast<uint32_t>(sizeof(XT));
        L.xw_off[r] = static_cast<uint32_t>(((c15 >> 1) * 64 + m + 16 * g) * 16 + 8 * (c15 & 1));
    }
}

template <typename XT>
struct Q4KXVec;
template <>
struct Q4KXVec<float> {
    typedef float4_t type;
};
template <>
struct Q4KXVec<_Float16> {
    typedef half4_t type;
};

// Raw activations of one stage held by a thread.
template <int kWaves, typename XT>
struct Q4KXRaw {
    typename Q4KXVec<XT>::type v[Q4KGeom<kWaves>::kXLoads];
};

// The activation loads are written as asm so that the compiler's own wait-count insertion does not
// see them: it cannot know how many younger loads a stage has issued (that depends on how much of
// the range is left) and would drain the whole load queue, weights in flight included, before the
// first use of these registers.  The s_waitcnt at the top of each stage covers them instead: a
// stage's activations are always older than the youngest group of loads.
__device__ __forceinline__ void q4k_load_x_vec(const uint8_t *base, uint32_t off, float4_t &v) {
    asm volatile("global_load_dwordx4 %0, %1, %2" : "=v"(v) : "v"(off), "s"(base) : "memory");
}
__device__ __forceinline__ void q4k_load_x_vec(const uint8_t *base, uint32_t off, half4_t &v) {
    asm volatile("global_load_dwordx2 %0, %1, %2" : "=v"(v) : "v"(off), "s"(base) : "memory");
}

// Placed after the s_waitcnt that covers a set of activation registers: their uses cannot be
// scheduled above this point.
template <int kWaves, typename XT>
__device__ __forceinline__ void q4k_pin_x(Q4KXRaw<kWaves, XT> &raw) {
#pragma unroll
    for (int r = 0; r < Q4KGeom<kWaves>::kXLoads; r++) asm volatile("" : "+v"(raw.v[r]));
}

template <int kWaves, typename XT>
__device__ __forceinline__ void q4k_load_x(const uint8_t *xblock, const Q4KLane<kWaves> &L, Q4KXRaw<kWaves, XT> &raw) {
#pragma unroll
    for (int r = 0; r < Q4KGeom<kWaves>::kXLoads; r++) q4k_load_x_vec(xblock, L.x_off[r], raw.v[r]);
}

// Rounds a stage's raw activations to f16 and writes this thread's share of the fragments into
// the activation buffer at `buf`.  Rows past n_rows repeat the last row: output rows depend on
// their own activation row only, and those rows are never stored.
template <int kWaves, typename XT>
__device__ __forceinline__ void q4k_write_x(half8_t *buf, const Q4KLane<kWaves> &L, const Q4KXRaw<kWaves, XT> &raw) {
    uint8_t *base = reinterpret_cast<uint8_t *>(buf);
#pragma unroll
    for (int r = 0; r < Q4KGeom<kWaves>::kXLoads; r++) {
        _Float16 h[4];
#pragma unroll
        for (int i = 0; i < 4; i++) h[i] = static_cast<_Float16>(raw.v[r][i]);
        half4_t frag = {h[0], h[2], h[1], h[3]};
        *reinterpret_cast<half4_t *>(base + L.xw_off[r]) = frag;
    }
}

// One weight wave-load of the stage at `wstage` (uniform) into the buffer at `buf`.
template <int kWaves>
__device__ __forceinline__ void q4k_issue_w(const uint8_t *wstage, half8_t *buf, const Q4KLane<kWaves> &L, int j, int wave) {
    __builtin_amdgcn_global_load_lds((gptr_t)(wstage + L.w_off[j]), (lptr_t)(buf + (j * kWaves + wave) * 64), 16, 0, 0);
}

// One stage (one super-block) of this wave's tile out of the weight buffer `buf` and the activation
// buffer `xcur`: 8 MFMAs for the scaled nibbles, 8 for the minima.  hdr = {d|dmin, scales[0..3], [4..7], [8..11]}, q0/q1 = the lane's 32 quant bytes
// (chunk g: sub-blocks 2g in the low and 2g+1 in the high nibbles).  The loads of later stages
// are issued in between: one weight load after every second MFMA (spread over the MFMAs, the
// loads never queue up behind each other in the address unit), then the activations; the
// activations of the next stage are converted and written to LDS half way through.
template <int kWaves, typename XT>
__device__ __forceinline__ void q4k_compute(const half8_t *buf, const half8_t *xcur, int lane, int wave, Q4KMagic magic, float4_t &acc,
                                            float4_t &acc_min, bool issue_w, const uint8_t *wstage, half8_t *wbuf,
                                            bool issue_x, const uint8_t *xblock, const Q4KLane<kWaves> &L,
                                            Q4KXRaw<kWaves, XT> &raw, bool write_x, half8_t *xbuf) {
    using G = Q4KGeom<kWaves>;
    const int n = lane & 15, g = lane >> 4;
    const u32x4_t *blk = reinterpret_cast<const u32x4_t *>(buf) + (wave * 16 + n) * 9;
    const half8_t *a = xcur + lane;
    const u32x4_t hdr = blk[0], q0 = blk[1 + 2 * g], q1 = blk[2 + 2 * g];
    // all eight activation fragments are fetched up front: their LDS latencies overlap each other
    // and the scale decode instead of stalling every MFMA pair
    half8_t af[8];
#pragma unroll
    for (int t = 0; t < 8; t++) af[t] = a[t * 64];
    // scales and minima of sub-blocks 2g (low nibbles) and 2g+1 (high nibbles); the 6-bit codes of
    // sub-blocks 0..3 sit in one dword, those of 4..7 are split over two: select by bit mask,
    // not by branch
    const uint32_t upper = 0u - static_cast<uint32_t>(g >> 1);  // all ones for g = 2, 3
    const uint32_t sc_lo = hdr.y & 0x3F3F3F3Fu, sc_hi = (hdr.w & 0x0F0F0F0Fu) | ((hdr.y >> 2) & 0x30303030u);
    const uint32_t mn_lo = hdr.z & 0x3F3F3F3Fu, mn_hi = ((hdr.w >> 4) & 0x0F0F0F0Fu) | ((hdr.z >> 2) & 0x30303030u);
    const uint32_t sc_word = (sc_hi & upper) | (sc_lo & ~upper), mn_word = (mn_hi & upper) | (mn_lo & ~upper);
    // The two 6-bit codes of this lane sit in bytes (0,1) or (2,3) of those words.  A byte
    // permute drops each into the mantissa of an f16 1024.0 (the lane's selector picks the byte
    // pair), and one packed fma per pair, (1024 + code) * d - 1024 d, gives code * d rounded once:
    // S = (s of sub-block 2g, s of 2g+1), M = (dmin*m of 2g, of 2g+1).
    const half2_t dm = __builtin_bit_cast(half2_t, hdr.x);
    const half2_t p_sc = as_half2(__builtin_amdgcn_perm(0x64646464u, sc_word, L.sc_sel));
    const half2_t p_mn = as_half2(__builtin_amdgcn_perm(0x64646464u, mn_word, L.sc_sel));
    const half2_t neg = dm * splat(static_cast<_Float16>(-1024.0f));
    const half2_t S = __builtin_elementwise_fma(p_sc, splat(dm[0]), splat(neg[0]));
    const half2_t M = __builtin_elementwise_fma(p_mn, splat(dm[1]), splat(neg[1]));
    const half2_t unbias = {static_cast<_Float16>(-1024.0f), static_cast<_Float16>(-64.0f)};
    const half2_t Cs = S * unbias;
    const half2_t s2l = splat(S[0]), c2l = splat(Cs[0]);
    const half2_t s2h = splat(S[1]), c2h = splat(Cs[1]);
    // dmin*m of sub-blocks 2g and 2g+1, eight times each: the B operands of the minima MFMAs
    const _Float16 m_lo = M[0], m_hi = M[1];
    const half8_t bml = {m_lo, m_lo, m_lo, m_lo, m_lo, m_lo, m_lo, m_lo};
    const half8_t bmh = {m_hi, m_hi, m_hi, m_hi, m_hi, m_hi, m_hi, m_hi};
    const uint32_t qw[8] = {q0.x, q0.y, q0.z, q0.w, q1.x, q1.y, q1.z, q1.w};
#pragma unroll
    for (int t = 0; t < 4; t++) {
        half8_t bl = unpack_scale<false>(qw[2 * t], qw[2 * t + 1], s2l, c2l, magic.lo);
        acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(af[t], bl, acc, 0, 0, 0);
        acc_min = __builtin_amdgcn_mfma_f32_16x16x32_f16(af[t], bml, acc_min, 0, 0, 0);
        if (t & 1) {
            const int j = t >> 1;
            if (issue_w && (j < G::kFull || (j == G::kFull && wave < G::kExtra))) q4k_issue_w<kWaves>(wstage, wbuf, L, j, wave);
            __builtin_amdgcn_sched_barrier(0);
        }
    }
    // the next stage's activations (in registers since the wait at the top of this stage) go to
    // LDS here, off the critical path between that wait and the barrier
    if (write_x) q4k_write_x<kWaves, XT>(xbuf, L, raw);
#pragma unroll
    for (int t = 0; t < 4; t++) {
        half8_t bh = unpack_scale<true>(qw[2 * t], qw[2 * t + 1], s2h, c2h, magic.hi);
        acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(af[4 + t], bh, acc, 0, 0, 0);
        acc_min = __builtin_amdgcn_mfma_f32_16x16x32_f16(af[4 + t], bmh, acc_min, 0, 0, 0);
        if (t & 1) {
            const int j = 2 + (t >> 1);
            if (issue_w && (j < G::kFull || (j == G::kFull && wave < G::kExtra))) q4k_issue_w<kWaves>(wstage, wbuf, L, j, wave);
            __builtin_amdgcn_sched_barrier(0);
        }
    }
    if (issue_x) q4k_load_x<kWaves, XT>(xblock, L, raw);
}

// s_waitcnt vmcnt(n) with the other counters left alone (gfx9 encoding: vmcnt low bits [3:0],
// high bits [15:14]; expcnt [6:4] and lgkmcnt [11:8] at their maxima)
constexpr int q4k_vmcnt(int n) { return ((n & 0xF) | ((n & 0x30) << 10)) | 0x0F70; }
// s_waitcnt lgkmcnt(0) alone
constexpr int kWaitLds = 0xC07F;
// s_waitcnt vmcnt(v) for a wave-uniform run-time v (the instruction takes an immediate); anything
// past the table waits for every load, which is always sufficient
__device__ __forceinline__ void q4k_wait_vm(int v) {
    switch (v) {
#define DFL_VM(n)                                      \
    case n:                                            \
        __builtin_amdgcn_s_waitcnt(q4k_vmcnt(n));      \
        break;
        DFL_VM(1) DFL_VM(2) DFL_VM(3) DFL_VM(4) DFL_VM(5) DFL_VM(6) DFL_VM(7) DFL_VM(8) DFL_VM(9) DFL_VM(10) DFL_VM(11) DFL_VM(12)
        DFL_VM(13) DFL_VM(14) DFL_VM(15) DFL_VM(16) DFL_VM(17) DFL_VM(18) DFL_VM(19) DFL_VM(20) DFL_VM(21) DFL_VM(22) DFL_VM(23) DFL_VM(24)
        DFL_VM(25) DFL_VM(26) DFL_VM(27) DFL_VM(28) DFL_VM(29) DFL_VM(30) DFL_VM(31) DFL_VM(32) DFL_VM(33) DFL_VM(34) DFL_VM(35) DFL_VM(36)
        DFL_VM(37) DFL_VM(38) DFL_VM(39) DFL_VM(40) DFL_VM(41) DFL_VM(42) DFL_VM(43) DFL_VM(44) DFL_VM(45) DFL_VM(46) DFL_VM(47) DFL_VM(48)
        DFL_VM(49) DFL_VM(50) DFL_VM(51) DFL_VM(52) DFL_VM(53) DFL_VM(54) DFL_VM(55) DFL_VM(56) DFL_VM(57) DFL_VM(58) DFL_VM(59) DFL_VM(60)
        DFL_VM(61) DFL_VM(62)
#undef DFL_VM
    default:
        __builtin_amdgcn_s_waitcnt(q4k_vmcnt(0));
    }
}

// Ends a tile group's segment: Y directly if this workgroup covered the group's whole K, else a
// partial tile for the reduce kernel (slot 0: the range's first group, slot 1: its last).
template <int kWaves>
__device__ __forceinline__ void q4k_flush(const Q4KRange &rg, const Q4KBatch &bt, int group, float4_t &acc,
                                          float4_t &acc_min, float4_t &stash, float *__restrict__ y,
                                          float *__restrict__ partials, int n_out, int n_rows, int tid) {
    // rare path: an opaque copy of the thread index keeps its index arithmetic out of the stage loop
    asm volatile("" : "+v"(tid));
    const int lane = tid & 63, wave = tid >> 6, n = lane & 15, g = lane >> 4;
    float4_t res = acc - acc_min;
    acc = float4_t{0, 0, 0, 0};
    acc_min = float4_t{0, 0, 0, 0};
    // the group's whole K lies inside this workgroup's range: no other workgroup contributes
    const bool whole = group * rg.nb >= rg.it_begin && (group + 1) * rg.nb <= rg.it_end;
    if (bt.pair) {
        if ((group & 1) == 0) {  // gate half: keep the tile for the up half that follows
            stash = res;
            return;
        }
#pragma unroll
        for (int i = 0; i < 4; i++) res[i] = stash[i] / (1.0f + expf(-stash[i])) * res[i];  // silu(gate) * up
        group >>= 1;
    }
    const int slot_j = bt.ids ? static_cast<int>(q4k_div(group, bt.by_gpm)) : 0, lg = group - slot_j * bt.groups_per_mat;
    y += static_cast<size_t>(slot_j) * bt.y_stride;
    const int orow = (lg * kWaves + wave) * 16 + n;
    if (whole) {
        if (orow < n_out) {
#pragma unroll
            for (int i = 0; i < 4; i++)
                if (4 * g + i < n_rows) y[static_cast<size_t>(4 * g + i) * n_out + orow] = res[i];
        }
        return;
    }
    const int slot = (group == rg.first_group) ? 0 : 1;
    float *p = partials + ((static_cast<size_t>(rg.wg) * 2 + slot) * kWaves + wave) * 256;
#pragma unroll
    for (int i = 0; i < 4; i++) p[(4 * g + i) * 16 + n] = res[i];
}

// Second kernel of a split-K call: one workgroup per output tile of every tile group that was
// split over several workgroups of the streaming kernel; adds the partial tiles in workgroup
// order (so sums are run-to-run deterministic) and writes Y.  Spreading this over the chip
// instead of leaving it to the group's last contributor matters when K is long: a group then
// has a dozen partial tiles.  (Measured on MI355X: a last-arriver reduction inside the streaming
// kernel, with device-scope stores, one atomic arrival count per tile and device-scope loads, is slower
// than this second launch, 22.7 / 27.9 / 16.3 us per call against 21.8 / 20.7 / 12.8 us on the three
// M = 16 projection shapes: the contributors sit on different XCDs, so the chain store -> count -> load
// crosses to memory three times at the tail of the kernel; with device-scope fences instead, each of which
// writes back and invalidates an XCD's whole L2, it is nine times slower.  Leaving the sum to the kernel that
// reads Y inside the model (the q/k norm + RoPE kernel adding seven or eight partial tiles per element as it
// loads, the residual + RMSNorm kernel sixteen) is slower as well: 7.8 us instead of 5.0 + 4.0 for the former
// with its 320 waves, 11.7 instead of 5.4 + 3.9 for the latter with its 16 workgroups (a CU takes in only
// 20-30 KB per microsecond, so a narrow kernel that reads 8-16 times the data loses more than the launch it
// saves); a 40-layer verify took 4.77 ms instead of 4.70 ms with the first alone.)
// Element e = 16 m + n of output tile (group, wave) of a split group: the sum of its partial tiles in workgroup order.
template <int kWaves>
__device__ __forceinline__ float q4k_partial_sum(const float *__restrict__ partials, int group, int wave, int e, int nb, int total,
                                                 int n_wg, int wg_first, int wg_last) {
    // a contributor's partial sits in slot 0 if its range starts inside this group (true for all
    // but possibly the first contributor), else in slot 1
    const int first_begin = static_cast<int>(static_cast<uint32_t>(total) * wg_first / n_wg);
    const int first_slot = first_begin >= group * nb ? 0 : 1;
    const size_t stride = static_cast<size_t>(2) * kWaves * 256;  // floats per workgroup
    const float *p = partials + static_cast<size_t>(wave) * 256 + e;
    float sum = p[wg_first * stride + static_cast<size_t>(first_slot) * kWaves * 256];
    int wg = wg_first + 1;
    for (; wg + 3 <= wg_last; wg += 4) {
        const float a0 = p[wg * stride], a1 = p[(wg + 1) * stride], a2 = p[(wg + 2) * stride], a3 = p[(wg + 3) * stride];
        sum = (((sum + a0) + a1) + a2) + a3;
    }
    for (; wg <= wg_last; wg++) sum += p[wg * stride];
    return sum;
}

// The reduction of a fused gate | up product (one matrix of 2 ffn rows: the gate's, then the up's) with the SwiGLU
// that follows it: out[m][c] = silu(gate[m][c]) * up[m][c], one workgroup per 16 gate columns, each value either the
// sum of its partial tiles (same order as q4k_reduce_kernel) or, for a group one workgroup covered alone, what the
// streaming kernel stored in y.  One launch instead of the reduction and the activation kernel; same bits.
template <int kWaves>
__global__ void __launch_bounds__(256)
    q4k_reduce_swiglu_kernel(const float *__restrict__ partials, const float *__restrict__ y, float *__restrict__ out, int ffn, int nb,
                             int n_rows, int n_groups, int n_wg) {
    const int e = threadIdx.x, m = e >> 4, n = e & 15;
    const int col = blockIdx.x * 16 + n;
    if (m >= n_rows || col >= ffn) return;
    const int total = n_groups * nb, n_out = 2 * ffn;
    auto value = [&](int c) {
        const int tile = c >> 4, group = tile / kWaves, wave = tile - group * kWaves;
        const int wg_first = q4k_wg_of(group * nb, total, n_wg), wg_last = q4k_wg_of((group + 1) * nb - 1, total, n_wg);
        if (wg_first == wg_last) return y[static_cast<size_t>(m) * n_out + c];
        return q4k_partial_sum<kWaves>(partials, group, wave, e, nb, total, n_wg, wg_first, wg_last);
    };
    const float g = value(col), u = value(col + ffn);  // (ffn is a multiple of 16: the same n in both tiles)
    out[static_cast<size_t>(m) * ffn + col] = g / (1.0f + expf(-g)) * u;
}

template <int kWaves>
__global__ void __launch_bounds__(256)
    q4k_reduce_kernel(const float *__restrict__ partials, float *__restrict__ y, int n_out, int nb, int n_rows,
                      int n_groups, int n_wg, Q4KBatch bt) {
    const int group = blockIdx.x / kWaves, wave = blockIdx.x % kWaves;
    if (bt.ids) n_groups = bt.groups_per_mat * *bt.n_slots;
    if (group >= n_groups) return;
    const int total = n_groups * nb;
    const int wg_first = q4k_wg_of(group * nb, total, n_wg);
    const int wg_last = q4k_wg_of((group + 1) * nb - 1, total, n_wg);
    if (wg_first == wg_last) return;
    const int e = threadIdx.x, m = e >> 4, n = e & 15;
    const int slot_j = group / bt.groups_per_mat, lg = group - slot_j * bt.groups_per_mat;
    y += static_cast<size_t>(slot_j) * bt.y_stride;
    const int orow = (lg * kWaves + wave) * 16 + n;
    if (m >= n_rows || orow >= n_out) return;
    y[static_cast<size_t>(m) * n_out + orow] = q4k_partial_sum<kWaves>(partials, group, wave, e, nb, total, n_wg, wg_first, wg_last);
}

// Cache-policy bits of the direct-to-LDS weight loads of the tiled and the expert kernel (0: the default policy).
// Measured on the three projection shapes (50 / 50 / 18 MB, copies rotating through more than the memory-side cache):
// non-temporal (2), sc0 (1), sc1 (16) and sc0 + sc1 (17) all within 1 % of the default.
#ifndef DFL_W_AUX
#define DFL_W_AUX 0
#endif

#ifdef DFLASH_TRACE
// Debug build only: per-workgroup time stamps (100 MHz constant clock) of the streaming kernel.
__device__ unsigned long long *g_trace = nullptr;  // [n_wg][16]
#define DFL_TR(i)                                                                          \
    do {                                                                                   \
        if (threadIdx.x == 0 && g_trace) g_trace[blockIdx.x * 16 + (i)] = wall_clock64();  \
    } while (0)
__device__ unsigned long long *g_trace2 = nullptr;  // [n_wg][16 waves][4]: cycles in load wait / barrier / compute, stages
#define DFL_CYC() __builtin_readcyclecounter()
#define DFL_TRW(i)                                                                                          \
    do {                                                                                                    \
        if ((threadIdx.x & 63) == 0 && g_trace2) g_trace2[(blockIdx.x * 16 + (threadIdx.x >> 6)) * 8 + (i)] = wall_clock64(); \
    } while (0)
// the streaming kernel's stamps: a gate/up pair launch writes 1024 workgroups further on than a plain one
#define DFL_TRS(i)                                                                                              \
    do {                                                                                                        \
        if (threadIdx.x == 0 && g_trace) g_trace[(blockIdx.x + (bt.pair ? 1024 : 0)) * 16 + (i)] = wall_clock64(); \
    } while (0)
// the expert kernel's stamps, per wave, kept in scalar registers and written at the end: a gate/up pair launch writes
// 256 workgroups further on than a down launch
#define DFL_TRE_DECL unsigned long long tre_[7] = {0, 0, 0, 0, 0, 0, 0}
#define DFL_TRE(i) tre_[i] = wall_clock64()
#define DFL_TRE_FLUSH                                                                                                \
    do {                                                                                                             \
        if ((threadIdx.x & 63) == 0 && g_trace2) {                                                                   \
            unsigned long long *o_ = g_trace2 + ((blockIdx.x + (bt.pair ? 256 : 0)) * 16 + (threadIdx.x >> 6)) * 8;   \
            for (int i_ = 0; i_ < 7; i_++) o_[i_] = tre_[i_];                                                        \
        }                                                                                                            \
    } while (0)
#else
#define DFL_TRE_DECL \
    do {             \
    } while (0)
#define DFL_TRE_FLUSH \
    do {              \
    } while (0)
#define DFL_TRE(i) \
    do {           \
    } while (0)
#define DFL_TRS(i) \
    do {           \
    } while (0)
#define DFL_TRW(i) \
    do {           \
    } while (0)
#define DFL_TR(i) \
    do {          \
    } while (0)
#endif
// the norm + router kernel's stamps (debug build), one set per workgroup of its two-dimensional grid
#ifdef DFLASH_TRACE
#define DFL_TRR(i)                                                                                                            \
    do {                                                                                                                      \
        if (threadIdx.x == 0 && g_trace) g_trace[(blockIdx.y * gridDim.x + blockIdx.x) * 16 + (i)] = wall_clock64();           \
    } while (0)
#else
#define DFL_TRR(i) \
    do {           \
    } while (0)
#endif

template <int kWaves, typename XT>
__global__ void __launch_bounds__(64 * kWaves)
    gemm_q4k_stream_kernel(const uint8_t *__restrict__ w, const XT *__restrict__ x, float *__restrict__ y,
                           float *__restrict__ partials, int n_out, int nb, int n_rows, int n_groups, Q4KBatch bt, int tiled) {
    using G = Q4KGeom<kWaves>;
    extern __shared__ half8_t lds[];  // kLdsPieces

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    DFL_TRS(0);
    Q4KRange rg;
    rg.nb = nb;
    rg.n_wg = gridDim.x;
    const int vshift = bt.pair ? 1 : 0;  // virtual groups per real group, as a shift
    const int n_slots = bt.ids ? *bt.n_slots : 1;
    if (bt.ids) n_groups = (bt.groups_per_mat * n_slots) << vshift;  // how many matrices take part is decided on the device
    rg.total = n_groups * nb;
    rg.wg = q4k_range_index(blockIdx.x, rg.n_wg);
    if (bt.whole_groups) {
        // cut between real groups (pair mode: between pairs of virtual groups)
        const uint32_t units = static_cast<uint32_t>(n_groups) >> vshift;
        rg.it_begin = (static_cast<int>(q4k_div(units * rg.wg, bt.by_wg)) << vshift) * nb;
        rg.it_end = (static_cast<int>(q4k_div(units * (rg.wg + 1), bt.by_wg)) << vshift) * nb;
    } else {
        rg.it_begin = static_cast<int>(q4k_div(static_cast<uint32_t>(rg.total) * rg.wg, bt.by_wg));
        rg.it_end = static_cast<int>(q4k_div(static_cast<uint32_t>(rg.total) * (rg.wg + 1), bt.by_wg));
    }
    if (rg.it_begin >= rg.it_end) return;  // more workgroups than work
    rg.first_group = static_cast<int>(q4k_div(rg.it_begin, bt.by_nb));
    const int b0 = rg.it_begin - rg.first_group * nb;
    const uint32_t row_bytes = static_cast<uint32_t>(nb) * DFL_Q4_K_BYTES;
    const uint32_t n_in = static_cast<uint32_t>(nb) * DFL_QK_K;
    const size_t group_bytes = static_cast<size_t>(G::kRows) * row_bytes;
    const uint8_t *xbytes = reinterpret_cast<const uint8_t *>(x);
    constexpr uint32_t kXBlockBytes = DFL_QK_K * sizeof(XT);

    // first weight byte of a group's first row, its activations, and the local group index.  Tiled order: a
    // matrix is cut in 256-row tile groups stored [group][super-block][256 rows x 144 bytes]; an 8-wave workgroup
    // owns the lower or the upper 128 rows of one, i.e. the first or second half of each of its stages.
    constexpr int kPerTiled = 16 / kWaves;  // this kernel's groups per tile group of the tiled order
    // The matrix index of a slot comes out of a register window over the list (lane l holds the id of slot
    // slot_base + l), read with one vector load per 64 slots.  A load of ids[j] at every change of matrix would be
    // a vector load too (the compiler cannot prove the list is not written), and the wait for it is a wait for
    // every weight stage in flight: the prefetch would start from nothing at every tile group.
    int slot_base = -64;  // no window yet: the first use (before any weight load is issued) reads it
    int32_t ids_window = 0;
    auto slot_id = [&](int j) {
        if (j < slot_base || j >= slot_base + 64) {
            slot_base = j;
            ids_window = bt.ids[min(j + lane, n_slots - 1)];
            __builtin_amdgcn_s_waitcnt(q4k_vmcnt(0));
            asm volatile("" : "+v"(ids_window));
        }
        return __builtin_amdgcn_readlane(ids_window, j - slot_base);
    };
    auto group_w = [&](int group) {
        const uint8_t *mat = w;
        int lg = group;
        if (bt.ids) {
            const bool up = bt.pair && (group & 1);
            const int g = group >> vshift;
            const int j = static_cast<int>(q4k_div(g, bt.by_gpm));
            lg = g - j * bt.groups_per_mat;
            const int32_t id = slot_id(j);
            mat = id < 0 ? (up ? bt.extra_w2 : bt.extra_w) : (up ? bt.w2 : w) + static_cast<size_t>(id) * bt.w_stride;
        }
        if (tiled)
            return q4k_uniform(mat + static_cast<size_t>(lg / kPerTiled) * nb * kTiledStageBytes +
                               static_cast<size_t>(lg % kPerTiled) * (G::kRows * DFL_Q4_K_BYTES));
        return q4k_uniform(mat + static_cast<size_t>(lg) * group_bytes);
    };
    auto group_x = [&](int group) {
        if (!bt.ids) return xbytes;
        return xbytes + static_cast<size_t>(q4k_div(group >> vshift, bt.by_gpm)) * bt.x_stride * sizeof(XT);
    };
    auto group_local = [&](int group) {
        group >>= vshift;
        return bt.ids ? group - static_cast<int>(q4k_div(group, bt.by_gpm)) * bt.groups_per_mat : group;
    };
    DFL_TRS(10);
    Q4KLane<kWaves> L;
    q4k_lane_w_offsets<kWaves>(L, tid, group_local(rg.first_group) * G::kRows, n_out, row_bytes, tiled);
    DFL_TRS(11);

    // Cursors.  Weights: wstage = first byte of the next stage to load in its group's first row,
    // bw its super-block, gw its group, w_left the stages not loaded yet.  Activations run one
    // stage further ahead: xblock / bx / x_left.
    const uint8_t *wstage = group_w(rg.first_group) + static_cast<size_t>(b0) * (tiled ? kTiledStageBytes : DFL_Q4_K_BYTES);
    int bw = b0, gw = rg.first_group, w_left = rg.it_end - rg.it_begin;
    const uint8_t *xblock = group_x(rg.first_group) + static_cast<size_t>(b0) * kXBlockBytes;
    int bx = b0, gx = rg.first_group, x_left = w_left;
    const bool ragged = bt.groups_per_mat * G::kRows > n_out;  // a matrix's last group has fewer rows
    auto advance_w = [&]() {
        wstage += tiled ? kTiledStageBytes : DFL_Q4_K_BYTES;
        w_left--;
        if (++bw == nb) {
            bw = 0;
            gw++;
            if (w_left > 0) {
                wstage = group_w(gw);
                if (ragged && !tiled) q4k_lane_w_offsets<kWaves>(L, tid, group_local(gw) * G::kRows, n_out, row_bytes);
            }
        }
    };
    auto advance_x = [&]() {
        xblock += kXBlockBytes;
        x_left--;
        if (++bx == nb) {
            bx = 0;
            gx++;
            if (x_left > 0) xblock = group_x(gx);
        }
    };
    auto issue_w_all = [&](half8_t *buf) {
#pragma unroll
        for (int j = 0; j < G::kFull; j++) q4k_issue_w<kWaves>(wstage, buf, L, j, wave);
        if (wave < G::kExtra) q4k_issue_w<kWaves>(wstage, buf, L, G::kFull, wave);
    };
    constexpr int kAhead = G::kAhead, kRing = G::kRing;
    // weight ring: slot_c holds the stage being computed, slot_i takes the next stage to be loaded
    int slot_c = 0, slot_i = 0;
    auto ring = [&](int slot) { return lds + slot * G::kWPieces; };
    half8_t *x_c = lds + kRing * G::kWPieces, *x_n = x_c + kQ4KBlockFrags;

    // Loads are issued, and return, in groups: group 0 = [weights of stage 0 (first of all: everything
    // else here hides behind their latency), activations of stages 0 and 1], group p = [weights of
    // stage p, activations of stage p + 1].  The prologue issues groups 0 .. kAhead-1, stage d issues
    // group d + kAhead, and the top of stage d waits until group d has landed, i.e. until no more
    // loads are outstanding than the (up to kAhead - 1) younger groups hold.
    issue_w_all(ring(0));
    advance_w();
    slot_i = 1;
    q4k_lane_x_offsets<kWaves, XT>(L, tid, n_rows, n_in);
    float4_t acc = {0, 0, 0, 0}, acc_min = {0, 0, 0, 0}, stash = {0, 0, 0, 0};
    const Q4KMagic magic = q4k_magic();
    Q4KXRaw<kWaves, XT> raw_first, raws[kAhead];  // activations of stage 0; raws[d % kAhead]: those of stage d + 1
    q4k_load_x<kWaves, XT>(xblock, L, raw_first);
    advance_x();
    if (x_left > 0) {
        q4k_load_x<kWaves, XT>(xblock, L, raws[0]);
        advance_x();
    }
#pragma unroll
    for (int p = 1; p < kAhead; p++) {
        if (w_left > 0) {
            issue_w_all(ring(p));
            advance_w();
            slot_i = p + 1;
            if (x_left > 0) {
                q4k_load_x<kWaves, XT>(xblock, L, raws[p]);
                advance_x();
            }
        }
    }
    DFL_TRS(12);
    DFL_TRS(1);
    int gc = rg.first_group, bc = b0, n_left = rg.it_end - rg.it_begin;
    bool first = true;
    int done = 0;
    // One stage; `raw` holds the activations of the next stage and is refilled with those three ahead.
#ifdef DFLASH_TRACE
    unsigned long long cyc_wait = 0, cyc_bar = 0, cyc_comp = 0, cyc_n = 0;
#endif
    auto stage = [&](Q4KXRaw<kWaves, XT> &raw) {
        constexpr int kW0 = G::kFull, kW1 = G::kFull + 1, kX = G::kXLoads;
#ifdef DFLASH_TRACE
        const unsigned long long c0 = DFL_CYC();
#endif
        if (n_left > kAhead) {  // every younger group exists and is whole
            if (wave < G::kExtra)
                __builtin_amdgcn_s_waitcnt(q4k_vmcnt((kAhead - 1) * (kW1 + kX)));
            else
                __builtin_amdgcn_s_waitcnt(q4k_vmcnt((kAhead - 1) * (kW0 + kX)));
        } else {
            // the range ends within reach: n_left - 1 younger weight stages, the last of them without activations
            const int ow = n_left - 1, ox = n_left >= 2 ? n_left - 2 : 0;
            q4k_wait_vm(ow * (wave < G::kExtra ? kW1 : kW0) + ox * kX);
        }
#ifdef DFLASH_TRACE
        const unsigned long long c1 = DFL_CYC();
#endif
        q4k_pin_x<kWaves, XT>(raw);
        if (first) {
            q4k_pin_x<kWaves, XT>(raw_first);
            q4k_write_x<kWaves, XT>(x_c, L, raw_first);
        }
        first = false;
        __builtin_amdgcn_s_waitcnt(kWaitLds);
        // A bare barrier, not __syncthreads(): that one carries a workgroup-scope fence, which waits
        // for every load in flight and would undo the prefetch.  The waits above are the only
        // ordering this needs: each wave's own pieces have landed before it arrives here.
        __builtin_amdgcn_s_barrier();  // stage d is complete in its ring slot; the slot of stage d-1 is free
#ifdef DFLASH_TRACE
        const unsigned long long c2 = DFL_CYC();
#endif
        const bool iw = w_left > 0, ix = x_left > 0;
        q4k_compute<kWaves, XT>(ring(slot_c), x_c, lane, wave, magic, acc, acc_min, iw, wstage, ring(slot_i), ix, xblock, L, raw,
                                n_left > 1, x_n);
#ifdef DFLASH_TRACE
        {
            const unsigned long long c3 = DFL_CYC();
            cyc_wait += c1 - c0;
            cyc_bar += c2 - c1;
            cyc_comp += c3 - c2;
            cyc_n++;
        }
#endif
        if (iw) advance_w();
        if (ix) advance_x();
        slot_c = slot_c + 1 == kRing ? 0 : slot_c + 1;
        if (iw) slot_i = slot_i + 1 == kRing ? 0 : slot_i + 1;
        half8_t *t = x_c;
        x_c = x_n;
        x_n = t;
        n_left--;
        done++;
        if (done <= 8) DFL_TRS(1 + done);
        if (++bc == nb || n_left == 0) {
            q4k_flush<kWaves>(rg, bt, gc, acc, acc_min, stash, y, partials, n_out, n_rows, tid);
            bc = 0;
            gc++;
        }
    };
    while (n_left > 0) {
#pragma unroll
        for (int u = 0; u < kAhead; u++)
            if (n_left > 0) stage(raws[u]);
    }
    DFL_TRS(13);
#ifdef DFLASH_TRACE
    if (lane == 0 && g_trace2) {
        unsigned long long *t = g_trace2 + (static_cast<size_t>(blockIdx.x + (bt.pair ? 1024 : 0)) * 16 + wave) * 4;
        t[0] = cyc_wait;
        t[1] = cyc_bar;
        t[2] = cyc_comp;
        t[3] = cyc_n;
    }
#endif
}

// ----------------------------------------------------------------------------
// Q4_K slab kernel: the streaming kernel for a single matrix whose ranges are short
// ----------------------------------------------------------------------------
//
// Same work split, output flush and split-K reduction as gemm_q4k_stream_kernel (16-wave tile groups,
// one contiguous range of (tile group x super-block) stages per workgroup), for the common case that a
// workgroup's range is at most kSlabStages stages long: every C2-shaped projection on a 256-CU chip.
// What differs is what the waves of a workgroup share:
//   * the activations of ALL the range's stages are converted to f16 MFMA fragments once, at the start,
//     into a resident slab in LDS (8 KB per stage), together with each stage's sub-block sums;
//   * every wave then streams its own 16 weight rows through a private ring of three LDS buffers
//     (direct-to-LDS loads of 144 row-contiguous 16-byte pieces per stage) and never meets the other
//     waves again: no barrier per stage, no per-stage activation work, and a wave starts computing as
//     soon as ITS first 2.3 KB have landed instead of when the whole 37 KB stage has.
// The sub-block minima cost one MFMA per stage instead of eight: sum_k x[m][k] * (dmin m_j)[n] over a
// sub-block j is (sum_k x[m][k]) * (dmin m_j)[n], so the stage's 16 x 8 sub-block sums of the (f16-rounded)
// activations, split into f16 high and low parts, form one A fragment (k-slots: high and low part of
// sub-blocks 2g and 2g+1 for lane group g, four slots zero) against B = the lane's two minima twice.
constexpr int kSlabStages = 6;
constexpr int kSlabWaves = 16;
constexpr int kSlabRing = 3;
constexpr int kSlabWavePieces = 144;                          // 16 rows x 9 pieces of 16 bytes
constexpr int kSlabStageBytes = kQ4KBlockFrags * 16 + 64 * 8; // 512 A fragments + 64 x (4 f16) sub-block sums
constexpr int kSlabWaveLoads = 3;                             // 64 + 64 + 16 lanes
constexpr size_t kSlabLdsBytes = static_cast<size_t>(kSlabStages) * kSlabStageBytes +
                                 static_cast<size_t>(kSlabWaves) * kSlabRing * kSlabWavePieces * 16;
static_assert(kSlabLdsBytes <= 160 * 1024, "one workgroup per CU, all of its LDS");

// One stage of a wave's tile: 8 MFMAs for the scaled nibbles, one for the minima.
__device__ __forceinline__ void q4k_slab_compute(const u32x4_t *blk, const half8_t *a, const half4_t *twin, int g, uint32_t sc_sel,
                                                 Q4KMagic magic, float4_t &acc, float4_t &acc_min) {
    const u32x4_t hdr = blk[0], q0 = blk[1 + 2 * g], q1 = blk[2 + 2 * g];
    half8_t af[8];
#pragma unroll
    for (int t = 0; t < 8; t++) af[t] = a[t * 64];
    const half4_t tw = *twin;
    // scales and minima of sub-blocks 2g and 2g+1 (see q4k_compute)
    const uint32_t upper = 0u - static_cast<uint32_t>(g >> 1);
    const uint32_t sc_lo = hdr.y & 0x3F3F3F3Fu, sc_hi = (hdr.w & 0x0F0F0F0Fu) | ((hdr.y >> 2) & 0x30303030u);
    const uint32_t mn_lo = hdr.z & 0x3F3F3F3Fu, mn_hi = ((hdr.w >> 4) & 0x0F0F0F0Fu) | ((hdr.z >> 2) & 0x30303030u);
    const uint32_t sc_word = (sc_hi & upper) | (sc_lo & ~upper), mn_word = (mn_hi & upper) | (mn_lo & ~upper);
    const half2_t dm = __builtin_bit_cast(half2_t, hdr.x);
    const half2_t p_sc = as_half2(__builtin_amdgcn_perm(0x64646464u, sc_word, sc_sel));
    const half2_t p_mn = as_half2(__builtin_amdgcn_perm(0x64646464u, mn_word, sc_sel));
    const half2_t neg = dm * splat(static_cast<_Float16>(-1024.0f));
    const half2_t S = __builtin_elementwise_fma(p_sc, splat(dm[0]), splat(neg[0]));
    const half2_t M = __builtin_elementwise_fma(p_mn, splat(dm[1]), splat(neg[1]));
    const half2_t unbias = {static_cast<_Float16>(-1024.0f), static_cast<_Float16>(-64.0f)};
    const half2_t Cs = S * unbias;
    const half2_t s2l = splat(S[0]), c2l = splat(Cs[0]);
    const half2_t s2h = splat(S[1]), c2h = splat(Cs[1]);
    const uint32_t qw[8] = {q0.x, q0.y, q0.z, q0.w, q1.x, q1.y, q1.z, q1.w};
    const _Float16 zero = static_cast<_Float16>(0.0f);
    const half8_t a_min = {tw[0], tw[1], tw[2], tw[3], zero, zero, zero, zero};
    const half8_t b_min = {M[0], M[1], M[0], M[1], zero, zero, zero, zero};
    acc_min = __builtin_amdgcn_mfma_f32_16x16x32_f16(a_min, b_min, acc_min, 0, 0, 0);
#pragma unroll
    for (int t = 0; t < 4; t++) {
        const half8_t bl = unpack_scale<false>(qw[2 * t], qw[2 * t + 1], s2l, c2l, magic.lo);
        acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(af[t], bl, acc, 0, 0, 0);
    }
#pragma unroll
    for (int t = 0; t < 4; t++) {
        const half8_t bh = unpack_scale<true>(qw[2 * t], qw[2 * t + 1], s2h, c2h, magic.hi);
        acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(af[4 + t], bh, acc, 0, 0, 0);
    }
}

// s_waitcnt vmcnt(3 n): at most n load groups (three instructions each) still in flight, n uniform
__device__ __forceinline__ void q4k_slab_wait_groups(int n) {
    if (n <= 0)
        __builtin_amdgcn_s_waitcnt(q4k_vmcnt(0));
    else if (n == 1)
        __builtin_amdgcn_s_waitcnt(q4k_vmcnt(3));
    else if (n == 2)
        __builtin_amdgcn_s_waitcnt(q4k_vmcnt(6));
    else if (n == 3)
        __builtin_amdgcn_s_waitcnt(q4k_vmcnt(9));
    else if (n == 4)
        __builtin_amdgcn_s_waitcnt(q4k_vmcnt(12));
    else if (n == 5)
        __builtin_amdgcn_s_waitcnt(q4k_vmcnt(15));
    else
        __builtin_amdgcn_s_waitcnt(q4k_vmcnt(18));
}

template <typename XT>
__global__ void __launch_bounds__(64 * kSlabWaves)
    gemm_q4k_slab_kernel(const uint8_t *__restrict__ w, const XT *__restrict__ x, float *__restrict__ y,
                         float *__restrict__ partials, int n_out, int nb, int n_rows, int n_groups, Q4KBatch bt) {
    constexpr int kW = kSlabWaves;
    extern __shared__ half8_t lds[];
    uint8_t *slab = reinterpret_cast<uint8_t *>(lds);                                   // [kSlabStages][kSlabStageBytes]
    half8_t *ring = reinterpret_cast<half8_t *>(slab + kSlabStages * kSlabStageBytes);  // [wave][kSlabRing][144]
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    Q4KRange rg;
    rg.nb = nb;
    rg.n_wg = gridDim.x;
    rg.total = n_groups * nb;
    rg.wg = q4k_range_index(blockIdx.x, rg.n_wg);
    rg.it_begin = static_cast<int>(q4k_div(static_cast<uint32_t>(rg.total) * rg.wg, bt.by_wg));
    rg.it_end = static_cast<int>(q4k_div(static_cast<uint32_t>(rg.total) * (rg.wg + 1), bt.by_wg));
    const int len = rg.it_end - rg.it_begin;  // <= kSlabStages (host)
    if (len <= 0) return;
    DFL_TR(0);
    rg.first_group = static_cast<int>(q4k_div(rg.it_begin, bt.by_nb));
    const int b0 = rg.it_begin - rg.first_group * nb;
    const uint32_t row_bytes = static_cast<uint32_t>(nb) * DFL_Q4_K_BYTES;
    const uint32_t n_in = static_cast<uint32_t>(nb) * DFL_QK_K;
    const size_t group_bytes = static_cast<size_t>(16 * kW) * row_bytes;

    // ---- this wave's weight loads: piece p = 64 j + lane of its 16 rows x 9 pieces (j = 2: 16 lanes) ----
    half8_t *my_ring = ring + wave * (kSlabRing * kSlabWavePieces);
    uint32_t w_off[kSlabWaveLoads];
    auto set_w_offsets = [&](int group) {  // rows past n_out (ragged last group) re-read the last row
        const int last = n_out - 1 - (group * kW + wave) * 16;
#pragma unroll
        for (int j = 0; j < kSlabWaveLoads; j++) {
            const int p = min(64 * j + lane, kSlabWavePieces - 1);
            const int r = max(min(p / 9, last), -(wave * 16));  // a wave wholly past n_out stays inside the group
            w_off[j] = static_cast<uint32_t>(wave * 16 + r) * row_bytes + static_cast<uint32_t>(p % 9) * 16u;
        }
    };
    const bool ragged = n_groups * 16 * kW > n_out;
    set_w_offsets(rg.first_group);
    const uint8_t *wstage = w + static_cast<size_t>(rg.first_group) * group_bytes + static_cast<size_t>(b0) * DFL_Q4_K_BYTES;
    int bw = b0, gw = rg.first_group, w_issued = 0;
    auto issue_w = [&]() {  // the next stage's 144 pieces into ring buffer (w_issued % 3)
        half8_t *buf = my_ring + (w_issued % kSlabRing) * kSlabWavePieces;
        __builtin_amdgcn_global_load_lds((gptr_t)(wstage + w_off[0]), (lptr_t)(buf), 16, 0, 0);
        __builtin_amdgcn_global_load_lds((gptr_t)(wstage + w_off[1]), (lptr_t)(buf + 64), 16, 0, 0);
        if (lane < 16) __builtin_amdgcn_global_load_lds((gptr_t)(wstage + w_off[2]), (lptr_t)(buf + 128), 16, 0, 0);
        w_issued++;
        wstage += DFL_Q4_K_BYTES;
        if (++bw == nb) {
            bw = 0;
            gw++;
            if (w_issued < len) {
                wstage = w + static_cast<size_t>(gw) * group_bytes;
                if (ragged) set_w_offsets(gw);
            }
        }
    };

    // ---- activations of every stage of the range: loads first (they come from L2 and are needed first) ----
    // thread -> (row m, four values k = 4c .. 4c+3): wave = sub-block pair half, see q4k_lane_x_offsets
    const int xm = 8 * (wave & 1) + (lane & 7), xc = 8 * (wave >> 1) + (lane >> 3);
    const uint32_t x_off = (static_cast<uint32_t>(min(xm, n_rows - 1)) * n_in + 4u * xc) * static_cast<uint32_t>(sizeof(XT));
    const uint32_t xw_off = static_cast<uint32_t>((((xc & 15) >> 1) * 64 + xm + 16 * (xc >> 4)) * 16 + 8 * (xc & 1));
    const uint8_t *xbytes = reinterpret_cast<const uint8_t *>(x);
    typename Q4KXVec<XT>::type raw[kSlabStages];
    {
        int b = b0;
#pragma unroll
        for (int t = 0; t < kSlabStages; t++) {
            if (t < len) q4k_load_x_vec(xbytes + static_cast<size_t>(b) * (DFL_QK_K * sizeof(XT)), x_off, raw[t]);
            if (++b == nb) b = 0;
        }
    }
    issue_w();
    if (len > 1) issue_w();
    q4k_slab_wait_groups(w_issued);  // the activations (older than every weight load) are in registers
    DFL_TR(1);
    DFL_TRW(0);
#pragma unroll
    for (int t = 0; t < kSlabStages; t++) {
        if (t < len) {
            asm volatile("" : "+v"(raw[t]));
            uint8_t *stage = slab + t * kSlabStageBytes;
            _Float16 h[4];
#pragma unroll
            for (int i = 0; i < 4; i++) h[i] = static_cast<_Float16>(raw[t][i]);
            const half4_t frag = {h[0], h[2], h[1], h[3]};
            *reinterpret_cast<half4_t *>(stage + xw_off) = frag;
            // sub-block sum of the rounded values over the eight lanes that share this row
            float sum = (static_cast<float>(h[0]) + static_cast<float>(h[1])) + (static_cast<float>(h[2]) + static_cast<float>(h[3]));
            sum += __shfl_xor(sum, 8, 64);
            sum += __shfl_xor(sum, 16, 64);
            sum += __shfl_xor(sum, 32, 64);
            if (lane < 8) {
                const int j = wave >> 1;  // this wave's sub-block
                const _Float16 hi = static_cast<_Float16>(sum), lo = static_cast<_Float16>(sum - static_cast<float>(hi));
                _Float16 *tw = reinterpret_cast<_Float16 *>(stage + kQ4KBlockFrags * 16) + (xm + 16 * (j >> 1)) * 4 + (j & 1);
                tw[0] = hi;
                tw[2] = lo;
            }
        }
    }
    __builtin_amdgcn_s_waitcnt(kWaitLds);
    DFL_TRW(1);
    __builtin_amdgcn_s_barrier();  // the slab is complete; from here on the waves run independently
    DFL_TR(2);
    DFL_TRW(2);

    const int n = lane & 15, g = lane >> 4;
    const uint32_t sc_sel = (lane & 16) ? 0x04030402u : 0x04010400u;
    const Q4KMagic magic = q4k_magic();
    float4_t acc = {0, 0, 0, 0}, acc_min = {0, 0, 0, 0}, stash = {0, 0, 0, 0};
    int gc = rg.first_group, bc = b0;
    for (int t = 0; t < len; t++) {
        q4k_slab_wait_groups(w_issued - 1 - t);  // loads land in order: stage t has when only later ones are in flight
        if (t == 0) DFL_TRW(4);
        if (t == 1) DFL_TRW(5);
        if (t == 2) DFL_TRW(6);
        if (t == 3) DFL_TRW(7);
        if (w_issued < len) issue_w();           // stage t+2 into the buffer stage t-1 has been read out of
        DFL_TR(3 + t);
        const u32x4_t *blk = reinterpret_cast<const u32x4_t *>(my_ring + (t % kSlabRing) * kSlabWavePieces) + n * 9;
        const uint8_t *stage = slab + t * kSlabStageBytes;
        q4k_slab_compute(blk, reinterpret_cast<const half8_t *>(stage) + lane,
                         reinterpret_cast<const half4_t *>(stage + kQ4KBlockFrags * 16) + lane, g, sc_sel, magic, acc, acc_min);
        if (++bc == nb || t + 1 == len) {
            q4k_flush<kW>(rg, bt, gc, acc, acc_min, stash, y, partials, n_out, n_rows, tid);
            bc = 0;
            gc++;
        }
    }
    DFL_TR(9);
    DFL_TRW(3);
}

// ----------------------------------------------------------------------------
// Q4_K in tiled order: the slab kernel on weights repacked once, at load time
// ----------------------------------------------------------------------------
//
// In ggml order a matrix is [row][super-block] of 144-byte blocks, so the 16 rows x 1 super-block a wave needs per
// stage are sixteen 144-byte runs a row stride apart.  Measured on MI355X (50 MB matrix, counters of the slab kernel
// against a plain copy of the same bytes): L2 misses 496 k lines instead of 392 k (blocks straddle 128-byte lines and
// the two halves of a line are asked for at different times), 1.8x the L2 requests, and HBM delivering 5 TB/s of
// traffic where the copy gets 7.3 TB/s: the kernel's time is its memory traffic, not its arithmetic.
// The tiled order removes all three: the matrix is cut into tile groups of 256 rows (the last one padded with zero
// blocks) and stored as
//     [tile group][super-block][tile 0..15][row 0..15][144-byte block],
// i.e. stage (group, super-block) of the streaming kernels is one contiguous 36 864-byte piece, a wave's share of it
// (one tile) one contiguous, 128-byte aligned 2304-byte piece, and a workgroup's range of stages one contiguous run.
// Blocks are unchanged (same 144 bytes, same values): dflash_repack_q4k_tiled is a permutation of whole blocks.

__global__ void __launch_bounds__(256)
    q4k_repack_tiled_kernel(const uint8_t *__restrict__ src, uint8_t *__restrict__ dst, int n_out, int nb, int64_t n_pieces) {
    const int64_t p = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;  // 16-byte piece of the tiled matrix
    if (p >= n_pieces) return;
    const int piece = static_cast<int>(p % 9);
    const int64_t blk = p / 9;                       // block index in tiled order
    const int row_in_group = static_cast<int>(blk % 256);
    const int64_t stage = blk / 256;                 // group * nb + sb
    const int sb = static_cast<int>(stage % nb);
    const int64_t row = (stage / nb) * 256 + row_in_group;
    u32x4_t v = {0, 0, 0, 0};
    if (row < n_out) v = *reinterpret_cast<const u32x4_t *>(src + (row * nb + sb) * DFL_Q4_K_BYTES + piece * 16);
    *reinterpret_cast<u32x4_t *>(dst + p * 16) = v;
}

__device__ __forceinline__ void q4k_load_x8(const uint8_t *base, uint32_t off, float4_t &a, float4_t &b) {
    asm volatile("global_load_dwordx4 %0, %2, %3\n\tglobal_load_dwordx4 %1, %2, %3 offset:16" : "=&v"(a), "=&v"(b) : "v"(off), "s"(base) : "memory");
}
__device__ __forceinline__ void q4k_load_x8(const uint8_t *base, uint32_t off, half8_t &a, half8_t &) {
    asm volatile("global_load_dwordx4 %0, %1, %2" : "=v"(a) : "v"(off), "s"(base) : "memory");
}
template <typename XT>
struct Q4KX8;
template <>
struct Q4KX8<float> {
    typedef float4_t type;
    static constexpr int kLoads = 2;
};
template <>
struct Q4KX8<_Float16> {
    typedef half8_t type;
    static constexpr int kLoads = 1;
};
__device__ __forceinline__ void q4k_x8_to_half(const float4_t &a, const float4_t &b, _Float16 *h) {
#pragma unroll
    for (int i = 0; i < 4; i++) {
        h[i] = static_cast<_Float16>(a[i]);
        h[4 + i] = static_cast<_Float16>(b[i]);
    }
}
__device__ __forceinline__ void q4k_x8_to_half(const half8_t &a, const half8_t &, _Float16 *h) {
#pragma unroll
    for (int i = 0; i < 8; i++) h[i] = a[i];
}

// sum over the four lanes of a quad (every lane gets it), without a trip through LDS
__device__ __forceinline__ float q4k_quad_sum(float v) {
    v += __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, v), 0xB1, 0xF, 0xF, true));  // quad_perm [1,0,3,2]
    v += __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, v), 0x4E, 0xF, 0xF, true));  // quad_perm [2,3,0,1]
    return v;
}

// A stage's activation fragments in the tiled kernel: the eight 1 KB fragment sets (one per MFMA) sit 1040 bytes
// apart, so that the eight lanes that convert one row's 64 values (same slot in eight different sets) write to
// different banks; then the sub-block sums.
constexpr int kTiledFragStride = 1024 + 16;
constexpr int kTiledStageX = 8 * kTiledFragStride + 64 * 8;
constexpr size_t kTiledLdsBytes = static_cast<size_t>(kSlabStages) * kTiledStageX +
                                  static_cast<size_t>(kSlabWaves) * kSlabRing * kSlabWavePieces * 16;
static_assert(kTiledLdsBytes <= 160 * 1024, "one workgroup per CU, all of its LDS");

// q4k_slab_compute with the fragment sets kTiledFragStride apart
__device__ __forceinline__ void q4k_tiled_compute(const u32x4_t *blk, const uint8_t *stage, int lane, int g, uint32_t sc_sel,
                                                  Q4KMagic magic, float4_t &acc, float4_t &acc_min) {
    const u32x4_t hdr = blk[0], q0 = blk[1 + 2 * g], q1 = blk[2 + 2 * g];
    half8_t af[8];
#pragma unroll
    for (int t = 0; t < 8; t++) af[t] = *reinterpret_cast<const half8_t *>(stage + t * kTiledFragStride + lane * 16);
    const half4_t tw = *reinterpret_cast<const half4_t *>(stage + 8 * kTiledFragStride + lane * 8);
    const uint32_t upper = 0u - static_cast<uint32_t>(g >> 1);
    const uint32_t sc_lo = hdr.y & 0x3F3F3F3Fu, sc_hi = (hdr.w & 0x0F0F0F0Fu) | ((hdr.y >> 2) & 0x30303030u);
    const uint32_t mn_lo = hdr.z & 0x3F3F3F3Fu, mn_hi = ((hdr.w >> 4) & 0x0F0F0F0Fu) | ((hdr.z >> 2) & 0x30303030u);
    const uint32_t sc_word = (sc_hi & upper) | (sc_lo & ~upper), mn_word = (mn_hi & upper) | (mn_lo & ~upper);
    const half2_t dm = __builtin_bit_cast(half2_t, hdr.x);
    const half2_t p_sc = as_half2(__builtin_amdgcn_perm(0x64646464u, sc_word, sc_sel));
    const half2_t p_mn = as_half2(__builtin_amdgcn_perm(0x64646464u, mn_word, sc_sel));
    const half2_t neg = dm * splat(static_cast<_Float16>(-1024.0f));
    const half2_t S = __builtin_elementwise_fma(p_sc, splat(dm[0]), splat(neg[0]));
    const half2_t M = __builtin_elementwise_fma(p_mn, splat(dm[1]), splat(neg[1]));
    const half2_t unbias = {static_cast<_Float16>(-1024.0f), static_cast<_Float16>(-64.0f)};
    const half2_t Cs = S * unbias;
    const half2_t s2l = splat(S[0]), c2l = splat(Cs[0]);
    const half2_t s2h = splat(S[1]), c2h = splat(Cs[1]);
    const uint32_t qw[8] = {q0.x, q0.y, q0.z, q0.w, q1.x, q1.y, q1.z, q1.w};
    const _Float16 zero = static_cast<_Float16>(0.0f);
    const half8_t a_min = {tw[0], tw[1], tw[2], tw[3], zero, zero, zero, zero};
    const half8_t b_min = {M[0], M[1], M[0], M[1], zero, zero, zero, zero};
    acc_min = __builtin_amdgcn_mfma_f32_16x16x32_f16(a_min, b_min, acc_min, 0, 0, 0);
#pragma unroll
    for (int t = 0; t < 4; t++) {
        const half8_t bl = unpack_scale<false>(qw[2 * t], qw[2 * t + 1], s2l, c2l, magic.lo);
        acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(af[t], bl, acc, 0, 0, 0);
    }
#pragma unroll
    for (int t = 0; t < 4; t++) {
        const half8_t bh = unpack_scale<true>(qw[2 * t], qw[2 * t + 1], s2h, c2h, magic.hi);
        acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(af[4 + t], bh, acc, 0, 0, 0);
    }
}

// The tiled kernel.  Same work split, flush and reduction as the slab kernel.  Order of the prologue: the
// activation loads alone, then (once they are back and converted) the first three weight stages into the wave's
// ring; see the measurements at the issue points.
template <typename XT>
__global__ void __launch_bounds__(64 * kSlabWaves)
    gemm_q4k_tiled_kernel(const uint8_t *__restrict__ w, const XT *__restrict__ x, float *__restrict__ y,
                          float *__restrict__ partials, int n_out, int nb, int n_rows, int n_groups, Q4KBatch bt, int kPre) {
    constexpr int kW = kSlabWaves;
    extern __shared__ half8_t lds[];
    uint8_t *slab = reinterpret_cast<uint8_t *>(lds);                                // [kSlabStages][kTiledStageX]
    half8_t *ring = reinterpret_cast<half8_t *>(slab + kSlabStages * kTiledStageX);  // [wave][kSlabRing][144]
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    Q4KRange rg;
    rg.nb = nb;
    rg.n_wg = gridDim.x;
    rg.total = n_groups * nb;
    rg.wg = q4k_range_index(blockIdx.x, rg.n_wg);
    rg.it_begin = static_cast<int>(q4k_div(static_cast<uint32_t>(rg.total) * rg.wg, bt.by_wg));
    rg.it_end = static_cast<int>(q4k_div(static_cast<uint32_t>(rg.total) * (rg.wg + 1), bt.by_wg));
    const int len = rg.it_end - rg.it_begin;  // <= kSlabStages (host)
    if (len <= 0) return;
    DFL_TR(0);
    rg.first_group = static_cast<int>(q4k_div(rg.it_begin, bt.by_nb));
    const int b0 = rg.it_begin - rg.first_group * nb;
    const uint32_t n_in = static_cast<uint32_t>(nb) * DFL_QK_K;

    // ---- activations of every stage of the range ----
    // item (stage s, row m, eight values k = 8c .. 8c+7): virtual wave v = wave + 16 r covers stage v / 8, rows
    // 8 ((v >> 2) & 1) + (lane >> 3), chunks 8 (v & 3) + (lane & 7): eight lanes read one row's 128 (f16) or 256 (f32)
    // contiguous bytes, and the four lanes of a quad hold one sub-block of one row
    constexpr int kItems = (kSlabStages * 8 + kW - 1) / kW;  // 3
    typename Q4KX8<XT>::type raw_a[kItems], raw_b[kItems];
    const uint8_t *xbytes = reinterpret_cast<const uint8_t *>(x);
#pragma unroll
    for (int r = 0; r < kItems; r++) {
        const int v = wave + kW * r, s = v >> 3;
        if (s < len) {
            const int m = 8 * ((v >> 2) & 1) + (lane >> 3), c = 8 * (v & 3) + (lane & 7);
            int b = b0 + s;
            while (b >= nb) b -= nb;
            const uint32_t off = (static_cast<uint32_t>(min(m, n_rows - 1)) * n_in + 8u * c) * static_cast<uint32_t>(sizeof(XT));
            q4k_load_x8(xbytes + static_cast<size_t>(b) * (DFL_QK_K * sizeof(XT)), off, raw_a[r], raw_b[r]);
        }
    }

    // ---- this wave's weight tiles: 144 contiguous 16-byte pieces per stage, piece 64 j + lane in load j ----
    half8_t *my_ring = ring + wave * (kSlabRing * kSlabWavePieces);
    const uint8_t *wlane = w + static_cast<size_t>(rg.it_begin) * kTiledStageBytes + static_cast<size_t>(wave) * kTiledTileBytes +
                           static_cast<size_t>(lane) * 16;
    int w_issued = 0;
    auto issue_w = [&]() {  // the next stage's 144 pieces into ring buffer (w_issued % 3)
        half8_t *buf = my_ring + (w_issued % kSlabRing) * kSlabWavePieces;
        __builtin_amdgcn_global_load_lds((gptr_t)(wlane), (lptr_t)(buf), 16, 0, DFL_W_AUX);
        __builtin_amdgcn_global_load_lds((gptr_t)(wlane + 1024), (lptr_t)(buf + 64), 16, 0, DFL_W_AUX);
        if (lane < 16) __builtin_amdgcn_global_load_lds((gptr_t)(wlane + 2048), (lptr_t)(buf + 128), 16, 0, DFL_W_AUX);
        w_issued++;
        wlane += kTiledStageBytes;
    };
    // kPre (host: two, or one for ranges of at most two stages) stages go out ahead of the wait for the activations,
    // the rest of the first three after the slab barrier.  Measured (50 MB matrix, kernel time): 15.6 / 15.2 / 14.6 /
    // 14.8 us with 0 / 1 / 2 / 3 stages ahead.  A CU's memory pipeline
    // takes new loads only as fast as data returns (27 KB/us, its share of HBM), so a wave that issues more stalls
    // at the issue and reaches the barrier late; with none ahead the activations are back after 1.2 us instead of
    // 3.5, but the weights start 2 us later.  (Landing the weights in registers with plain loads and writing them
    // to one LDS buffer per wave instead of the direct-to-LDS ring measured the same: 14.65 against 14.60 us.)
    for (int t = 0; t < kPre; t++)
        if (t < len) issue_w();
    q4k_slab_wait_groups(w_issued);  // the activations (older than every weight load) are in registers
    DFL_TR(1);
    DFL_TRW(0);
#pragma unroll
    for (int r = 0; r < kItems; r++) {
        const int v = wave + kW * r, s = v >> 3;
        if (s < len) {
            asm volatile("" : "+v"(raw_a[r]));
            if (Q4KX8<XT>::kLoads == 2) asm volatile("" : "+v"(raw_b[r]));
            const int m = 8 * ((v >> 2) & 1) + (lane >> 3), c = 8 * (v & 3) + (lane & 7);
            const int j = c >> 2, quarter = c & 3;  // sub-block, eight-value unit in it
            uint8_t *stage = slab + s * kTiledStageX;
            _Float16 h[8];
            q4k_x8_to_half(raw_a[r], raw_b[r], h);
            // fragment slot of MFMA t = 4 (j & 1) + quarter, lane (m, g = j >> 1); element order of the unpack
            const half8_t frag = {h[0], h[2], h[1], h[3], h[4], h[6], h[5], h[7]};
            *reinterpret_cast<half8_t *>(stage + (4 * (j & 1) + quarter) * kTiledFragStride + (16 * (j >> 1) + m) * 16) = frag;
            float sum = 0.0f;
#pragma unroll
            for (int i = 0; i < 8; i++) sum += static_cast<float>(h[i]);
            sum = q4k_quad_sum(sum);  // the sub-block's sum of the rounded values
            if (quarter == 0) {
                const _Float16 hi = static_cast<_Float16>(sum), lo = static_cast<_Float16>(sum - static_cast<float>(hi));
                _Float16 *tw = reinterpret_cast<_Float16 *>(stage + 8 * kTiledFragStride) + (m + 16 * (j >> 1)) * 4 + (j & 1);
                tw[0] = hi;
                tw[2] = lo;
            }
        }
    }
    __builtin_amdgcn_s_waitcnt(kWaitLds);
    DFL_TRW(1);
    __builtin_amdgcn_s_barrier();  // the slab is complete; from here on the waves run independently
    DFL_TR(2);
    DFL_TRW(2);
    for (int t = kPre; t < kSlabRing; t++)
        if (t < len) issue_w();

    const int n = lane & 15, g = lane >> 4;
    const uint32_t sc_sel = (lane & 16) ? 0x04030402u : 0x04010400u;
    const Q4KMagic magic = q4k_magic();
    float4_t acc = {0, 0, 0, 0}, acc_min = {0, 0, 0, 0}, stash = {0, 0, 0, 0};
    int gc = rg.first_group, bc = b0;
    for (int t = 0; t < len; t++) {
        q4k_slab_wait_groups(w_issued - 1 - t);  // loads land in order: stage t has when only later ones are in flight
        if (t == 0) DFL_TRW(4);
        if (t == 1) DFL_TRW(5);
        if (t == 2) DFL_TRW(6);
        if (t == 3) DFL_TRW(7);
        DFL_TR(3 + t);
        const u32x4_t *blk = reinterpret_cast<const u32x4_t *>(my_ring + (t % kSlabRing) * kSlabWavePieces) + n * 9;
        q4k_tiled_compute(blk, slab + t * kTiledStageX, lane, g, sc_sel, magic, acc, acc_min);
        // stage t+3 into the buffer this stage has just been read out of (its reads are complete: the MFMAs above used them)
        if (w_issued < len) issue_w();
        if (++bc == nb || t + 1 == len) {
            q4k_flush<kW>(rg, bt, gc, acc, acc_min, stash, y, partials, n_out, n_rows, tid);
            bc = 0;
            gc++;
        }
    }
    DFL_TR(9);
    DFL_TRW(3);
}

// ----------------------------------------------------------------------------
// Q4_K expert kernel: the matrices a device-side list picks out of a stack, tiled order
// ----------------------------------------------------------------------------
//
// The batched mode of gemm_q4k_stream_kernel is bound by its own instructions (sixteen MFMAs and a workgroup barrier
// per stage, two waves per SIMD to hide them: a CU streams 15 KB/us where the single-matrix tiled kernel takes in
// 20) and by its coarse work unit (a 128-row group over the whole K: 186 units for 31 experts' gate/up on 256 CUs).
// This kernel gives the tiled kernel's structure to a batch: a wave owns one 16-row tile over the matrix's whole K
// (gate and up of the same tile in pair mode) and streams it through its private ring of three LDS buffers with
// direct-to-LDS loads, meeting the other waves only where the shared activations change.  The activations of four
// stages at a time sit in LDS as MFMA fragments with their sub-block sums (so the minima cost one MFMA per stage):
//   * x shared by every slot (gate/up, a drafter's per-layer projections of the same columns): a workgroup takes a
//     contiguous run of (slot, tile) units, sixteen per round, one per wave; the slab is refilled only when K is
//     longer than four stages (twice per round for K = 2048);
//   * x per slot (down: every expert has its own SwiGLU rows): a unit is (slot, sixteen tiles) and the slab is
//     refilled when the slot changes.
// A (row, matrix) result never depends on which other matrices take part: whole K per wave, fixed order.
constexpr int kExpChunk = 4;  // stages of activations in LDS at a time
constexpr size_t kExpRingEnd = static_cast<size_t>(kExpChunk) * kTiledStageX +
                               static_cast<size_t>(kSlabWaves) * kSlabRing * kSlabWavePieces * 16;
constexpr size_t kExpXchgEnd = kExpRingEnd + (kSlabWaves / 2) * 64 * sizeof(float4_t);  // + the up tiles of split pairs
constexpr int kExpRouteIds = 264;  // expert list of a routed launch: at most 256 experts + the shared one
constexpr size_t kExpLdsBytes = kExpXchgEnd + 16 * 4 * sizeof(unsigned long long) + kExpRouteIds * sizeof(int32_t);
static_assert(kExpLdsBytes <= 160 * 1024, "one workgroup per CU, all of its LDS");

// q4k_tiled_compute for the expert kernel, which carries more state per lane (activations on their way for the next
// refill, a second accumulator in pair mode) inside the 128 registers sixteen waves leave each other: the minima
// product is subtracted in the same accumulator (B operand negated) and the activation fragments are fetched four at
// a time.
__device__ __forceinline__ void q4k_experts_compute(const u32x4_t *blk, const uint8_t *stage, int lane, int g, uint32_t sc_sel,
                                                    Q4KMagic magic, float4_t &acc) {
    const u32x4_t hdr = blk[0], q0 = blk[1 + 2 * g], q1 = blk[2 + 2 * g];
    half8_t af[4];
#pragma unroll
    for (int t = 0; t < 4; t++) af[t] = *reinterpret_cast<const half8_t *>(stage + t * kTiledFragStride + lane * 16);
    const half4_t tw = *reinterpret_cast<const half4_t *>(stage + 8 * kTiledFragStride + lane * 8);
    const uint32_t upper = 0u - static_cast<uint32_t>(g >> 1);
    const uint32_t sc_lo = hdr.y & 0x3F3F3F3Fu, sc_hi = (hdr.w & 0x0F0F0F0Fu) | ((hdr.y >> 2) & 0x30303030u);
    const uint32_t mn_lo = hdr.z & 0x3F3F3F3Fu, mn_hi = ((hdr.w >> 4) & 0x0F0F0F0Fu) | ((hdr.z >> 2) & 0x30303030u);
    const uint32_t sc_word = (sc_hi & upper) | (sc_lo & ~upper), mn_word = (mn_hi & upper) | (mn_lo & ~upper);
    const half2_t dm = __builtin_bit_cast(half2_t, hdr.x);
    const half2_t p_sc = as_half2(__builtin_amdgcn_perm(0x64646464u, sc_word, sc_sel));
    const half2_t p_mn = as_half2(__builtin_amdgcn_perm(0x64646464u, mn_word, sc_sel));
    const half2_t neg = dm * splat(static_cast<_Float16>(-1024.0f));
    const half2_t S = __builtin_elementwise_fma(p_sc, splat(dm[0]), splat(neg[0]));
    // -(dmin * m): (1024 + code) * (-dmin) + 1024 dmin, rounded once like its positive twin
    const half2_t M = __builtin_elementwise_fma(p_mn, splat(-dm[1]), splat(-neg[1]));
    const half2_t unbias = {static_cast<_Float16>(-1024.0f), static_cast<_Float16>(-64.0f)};
    const half2_t Cs = S * unbias;
    const half2_t s2l = splat(S[0]), c2l = splat(Cs[0]);
    const half2_t s2h = splat(S[1]), c2h = splat(Cs[1]);
    const uint32_t qw[8] = {q0.x, q0.y, q0.z, q0.w, q1.x, q1.y, q1.z, q1.w};
    const _Float16 zero = static_cast<_Float16>(0.0f);
    const half8_t a_min = {tw[0], tw[1], tw[2], tw[3], zero, zero, zero, zero};
    const half8_t b_min = {M[0], M[1], M[0], M[1], zero, zero, zero, zero};
    acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(a_min, b_min, acc, 0, 0, 0);
#pragma unroll
    for (int t = 0; t < 4; t++) {
        const half8_t bl = unpack_scale<false>(qw[2 * t], qw[2 * t + 1], s2l, c2l, magic.lo);
        acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(af[t], bl, acc, 0, 0, 0);
    }
#pragma unroll
    for (int t = 0; t < 4; t++) af[t] = *reinterpret_cast<const half8_t *>(stage + (4 + t) * kTiledFragStride + lane * 16);
#pragma unroll
    for (int t = 0; t < 4; t++) {
        const half8_t bh = unpack_scale<true>(qw[2 * t], qw[2 * t + 1], s2h, c2h, magic.hi);
        acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(af[t], bh, acc, 0, 0, 0);
    }
}

template <typename XT, typename YT, bool kRoute>
__global__ void __launch_bounds__(64 * kSlabWaves)
    gemm_q4k_experts_kernel(const uint8_t *__restrict__ w, const XT *__restrict__ x, YT *__restrict__ y, int n_out, int nb,
                            int n_rows, Q4KBatch bt, int upm, Q4KDiv by_upm, int max_slots, int early_ids) {
    constexpr int kW = kSlabWaves;
    constexpr int kItems = kExpChunk * 8 / kW;  // activation items (eight values of one row) per thread and refill: 2
    constexpr int kXInstr = kItems * Q4KX8<XT>::kLoads;
    extern __shared__ half8_t lds[];
    uint8_t *slab = reinterpret_cast<uint8_t *>(lds);                              // [kExpChunk][kTiledStageX]
    half8_t *ring = reinterpret_cast<half8_t *>(slab + kExpChunk * kTiledStageX);  // [wave][kSlabRing][144]
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const bool per_slot_x = bt.x_stride != 0;
    DFL_TRE_DECL;
    DFL_TRE(0);
    // ---- activations: items as in gemm_q4k_tiled_kernel (virtual wave v = wave + 16 r: stage v / 8 of the chunk) ----
    typename Q4KX8<XT>::type raw_a[kItems], raw_b[kItems];
    const uint32_t n_in = static_cast<uint32_t>(nb) * DFL_QK_K;
    const uint8_t *xbytes = reinterpret_cast<const uint8_t *>(x);
    uint32_t x_off[kItems];
#pragma unroll
    for (int r = 0; r < kItems; r++) {
        const int v = wave + kW * r;
        const int m = 8 * ((v >> 2) & 1) + (lane >> 3), c = 8 * (v & 3) + (lane & 7);
        x_off[r] = (static_cast<uint32_t>(min(m, n_rows - 1)) * n_in + 8u * c) * static_cast<uint32_t>(sizeof(XT));
    }
    auto chunk_len = [&](int c) { return min(kExpChunk, nb - c * kExpChunk); };
    auto load_x = [&](int xslot, int c) {  // stages past the chunk's end re-read its last stage (never converted)
        const uint8_t *xb = q4k_uniform(xbytes + static_cast<size_t>(xslot) * bt.x_stride * sizeof(XT));
        const int last = chunk_len(c) - 1;
#pragma unroll
        for (int r = 0; r < kItems; r++) {
            const int sb = c * kExpChunk + min((wave + kW * r) >> 3, last);
            q4k_load_x8(xb + static_cast<size_t>(sb) * (DFL_QK_K * sizeof(XT)), x_off[r], raw_a[r], raw_b[r]);
        }
    };
    int32_t *ids_lds = reinterpret_cast<int32_t *>(reinterpret_cast<uint8_t *>(lds) + kExpXchgEnd + 16 * 4 * sizeof(unsigned long long));
    int slot_base = -64;  // no window of the list yet: the first use (before any weight load is issued) reads it
    int32_t ids_window = 0;
    int n_slots;
    if constexpr (kRoute) {
        // The block's routing, by every workgroup for itself: wave w takes row w (dfl_route::route_row, the arithmetic
        // of the stand-alone kernel), the union of the rows' masks gives the ascending expert list, kept in LDS.
        // The row's logits are fetched FIRST and waited for before the shared activations are requested: a CU takes in
        // 20-30 KB per microsecond, and behind the 64 KB of a chunk's f32 activations the 8 KB of logits arrived 2 us
        // later than alone (loads return in order).  The activations then travel while the rows are routed.  The loads
        // are asm loads with their own wait, like the activations': a wait the compiler placed at the logits' first use
        // would stand behind the activation loads again.
        unsigned long long *row_mask = reinterpret_cast<unsigned long long *>(reinterpret_cast<uint8_t *>(lds) + kExpXchgEnd);
        const int E = bt.route_experts, used = bt.route_used;
        float lgv[4] = {-INFINITY, -INFINITY, -INFINITY, -INFINITY};
        if (wave < n_rows) {
            const float *lrow = bt.route_logits + static_cast<size_t>(wave) * E + lane;
#pragma unroll
            for (int j = 0; j < 4; j++)
                if (lane + 64 * j < E) asm volatile("global_load_dword %0, %1, off" : "+v"(lgv[j]) : "v"(lrow + 64 * j) : "memory");
        }
        __builtin_amdgcn_s_waitcnt(q4k_vmcnt(0));
#pragma unroll
        for (int j = 0; j < 4; j++) asm volatile("" : "+v"(lgv[j]));
        load_x(0, 0);
        dfl_route::RowPicks pk;
        pk.my_e = 0;
        pk.my_w = 0.0f;
        pk.m[0] = pk.m[1] = pk.m[2] = pk.m[3] = 0;
        if (wave < n_rows) pk = dfl_route::route_row_from(lgv, E, used, lane);
        if (lane < 4) row_mask[wave * 4 + lane] = dfl_route::pick4(pk.m, lane);
        __builtin_amdgcn_s_waitcnt(kWaitLds);
        __builtin_amdgcn_s_barrier();
        unsigned long long un[4];
        dfl_route::union_of_rows(row_mask, lane, un);
        const int total = __popcll(un[0]) + __popcll(un[1]) + __popcll(un[2]) + __popcll(un[3]);
        n_slots = min(total + (bt.route_shared ? 1 : 0), max_slots);
        const bool listed = tid < E && ((dfl_route::pick4(un, tid >> 6) >> (tid & 63)) & 1);
        const int my_slot = listed ? dfl_route::slot_below(un, tid) : 0;
        if (listed) ids_lds[my_slot] = tid;
        if (tid == 0 && bt.route_shared) ids_lds[total] = -1;
        if (blockIdx.x == 0) {  // one copy for the launches that follow
            int32_t *ids_out = const_cast<int32_t *>(bt.ids);
            if (listed) ids_out[my_slot] = tid;
            if (tid == 0) {
                if (bt.route_shared) ids_out[total] = -1;
                *const_cast<int32_t *>(bt.n_slots) = n_slots;
            }
            if (wave < n_rows && lane < used) {
                bt.route_sel_e[wave * used + lane] = pk.my_e;
                bt.route_sel_w[wave * used + lane] = pk.my_w;
                bt.route_slot_of[wave * used + lane] = dfl_route::slot_below(un, pk.my_e);
            }
        }
        __builtin_amdgcn_s_waitcnt(kWaitLds);
        __builtin_amdgcn_s_barrier();
    } else {
        if (early_ids) {  // the first window of the list travels with the slot count: one trip to memory instead of two
            ids_window = bt.ids[min(lane, max_slots - 1)];
            slot_base = 0;
        }
        n_slots = min(*bt.n_slots, max_slots);  // (the bound the host sized the buffers for)
        // one wait for both, stated here on every path so that none is implied at the window's later uses
        __builtin_amdgcn_s_waitcnt(q4k_vmcnt(0));
        asm volatile("" : "+v"(ids_window));
    }
    DFL_TRE(1);
    const int tiles = (n_out + 15) >> 4;
    const int halves = bt.pair ? 2 : 1;
    const int n_chunks = (nb + kExpChunk - 1) / kExpChunk;
    // units: (slot, tile) with shared x, (slot, group of sixteen tiles) with x per slot; upm = units per matrix
    const uint32_t units = static_cast<uint32_t>(n_slots) * static_cast<uint32_t>(upm);
    const int wg = q4k_range_index(blockIdx.x, gridDim.x);
    const int u0 = static_cast<int>(q4k_div(units * wg, bt.by_wg)), u1 = static_cast<int>(q4k_div(units * (wg + 1), bt.by_wg));
    if (u0 >= u1) return;  // more workgroups than work (the whole workgroup leaves: no barrier is missed)
    // Pair mode with at most eight units for this workgroup: gate and up of a unit go to two waves (w and w + 8)
    // instead of one after the other on the same wave.  A lightly loaded wave is bound by its own chain of dependent
    // instructions (~0.7 us per stage with nothing else on its SIMD), so halving the chain is what shortens the
    // kernel; every product is still one wave's whole-K sum in the same order, so the bits do not depend on the mode.
    const bool hsplit = bt.pair && !per_slot_x && u1 - u0 <= kW / 2;
    const int n_rounds = per_slot_x ? u1 - u0 : (hsplit ? 1 : (u1 - u0 + kW - 1) / kW);
    const int h_begin = hsplit ? wave >> 3 : 0, h_end = hsplit ? h_begin + 1 : halves;

    // matrix index of a slot: a register window over the list (see gemm_q4k_stream_kernel)
    // (Measured and not kept: shared activations loaded at the very top of the kernel as well, ahead of the slot
    // count - 1.2-1.5 us slower per launch than this order.)
    auto slot_id = [&](int j) {
        if constexpr (kRoute) {  // the list is in LDS; whatever it holds, the index stays inside the stack
            const int32_t id = __builtin_amdgcn_readfirstlane(ids_lds[min(max(j, 0), kExpRouteIds - 1)]);
            return min(max(id, -1), bt.route_experts - 1);
        }
        if (j < slot_base || j >= slot_base + 64) {
            slot_base = j;
            ids_window = bt.ids[min(j + lane, n_slots - 1)];
            __builtin_amdgcn_s_waitcnt(q4k_vmcnt(0));
            asm volatile("" : "+v"(ids_window));
        }
        return __builtin_amdgcn_readlane(ids_window, j - slot_base);
    };
    // this wave's unit in round r
    auto unit_of = [&](int r, int &slot, int &tile) {
        if (per_slot_x) {
            const int g = u0 + r;
            slot = static_cast<int>(q4k_div(g, by_upm));
            tile = (g - slot * upm) * kW + wave;
            return tile < tiles;
        }
        const int u = hsplit ? u0 + (wave & 7) : u0 + r * kW + wave;
        slot = static_cast<int>(q4k_div(min(u, u1 - 1), by_upm));
        tile = u - slot * upm;
        return u < u1;
    };
    // whose activations round r needs (uniform over the workgroup)
    auto xslot_of = [&](int r) { return per_slot_x ? static_cast<int>(q4k_div(u0 + r, by_upm)) : 0; };
    auto tile_base = [&](int slot, int tile, int half) {
        const int32_t id = slot_id(slot);
        const uint8_t *mat = id < 0 ? (half ? bt.extra_w2 : bt.extra_w) : (half ? bt.w2 : w) + static_cast<size_t>(id) * bt.w_stride;
        return q4k_uniform(mat + static_cast<size_t>(tile >> 4) * nb * kTiledStageBytes + static_cast<size_t>(tile & 15) * kTiledTileBytes);
    };

    auto convert = [&](int c) {
        const int clen = chunk_len(c);
        int cl = lane;  // (opaque copy: the slab addresses are not worth registers across the stage loop)
        asm volatile("" : "+v"(cl));
#pragma unroll
        for (int r = 0; r < kItems; r++) {
            asm volatile("" : "+v"(raw_a[r]));
            if (Q4KX8<XT>::kLoads == 2) asm volatile("" : "+v"(raw_b[r]));
            const int v = wave + kW * r, s = v >> 3;
            if (s < clen) {
                const int m = 8 * ((v >> 2) & 1) + (cl >> 3), c8 = 8 * (v & 3) + (cl & 7);
                const int j = c8 >> 2, quarter = c8 & 3;  // sub-block, eight-value unit in it
                uint8_t *stage = slab + s * kTiledStageX;
                _Float16 h[8];
                q4k_x8_to_half(raw_a[r], raw_b[r], h);
                const half8_t frag = {h[0], h[2], h[1], h[3], h[4], h[6], h[5], h[7]};
                *reinterpret_cast<half8_t *>(stage + (4 * (j & 1) + quarter) * kTiledFragStride + (16 * (j >> 1) + m) * 16) = frag;
                float sum = 0.0f;
#pragma unroll
                for (int i = 0; i < 8; i++) sum += static_cast<float>(h[i]);
                sum = q4k_quad_sum(sum);
                if (quarter == 0) {
                    const _Float16 hi = static_cast<_Float16>(sum), lo = static_cast<_Float16>(sum - static_cast<float>(hi));
                    _Float16 *tw = reinterpret_cast<_Float16 *>(stage + 8 * kTiledFragStride) + (m + 16 * (j >> 1)) * 4 + (j & 1);
                    tw[0] = hi;
                    tw[2] = lo;
                }
            }
        }
    };

    // ---- this wave's weight stream: for every round it takes part in, chunk by chunk, gate then up, stage by stage ----
    // (Measured and not kept: a workgroup with k < 16 units letting its k waves divide the ring area among them, rings
    // up to 48 / k stages deep, filled at once or one extra stage per stage computed: 21.6 -> 22.9 us for 31 experts'
    // gate/up.  A lightly loaded wave is not waiting for memory but for its own stage, ~0.7 us of dependent LDS reads,
    // unpacking and MFMAs with nothing else on its SIMD to overlap.)
    constexpr int depth = kSlabRing;
    half8_t *my_ring = ring + wave * (depth * kSlabWavePieces);
    int it_r = 0, it_c = 0, it_h = h_begin, it_s = 0;
    bool it_valid = false;
    const uint8_t *it_base0 = nullptr, *it_base1 = nullptr;
    auto it_seek = [&]() {  // the first round at or after it_r with a unit for this wave
        int slot = 0, tile = 0;
        // (not unrolled: the first round almost always has a unit, and the compiler's four-at-a-time version spent a
        // hundred scalar instructions, in all sixteen waves, before the first weight load of a launch)
#pragma nounroll
        while (it_r < n_rounds && !unit_of(it_r, slot, tile)) it_r++;
        it_valid = it_r < n_rounds;
        if (it_valid) {
            it_base0 = tile_base(slot, tile, 0);
            if (bt.pair) it_base1 = tile_base(slot, tile, 1);
        }
    };
    int w_issued = 0, w_done = 0, ring_i = 0, ring_c = 0;
    auto issue = [&]() {  // the stream's next stage (144 pieces) into the ring
        const uint8_t *src = (it_h ? it_base1 : it_base0) + static_cast<size_t>(it_c * kExpChunk + it_s) * kTiledStageBytes +
                             static_cast<size_t>(lane) * 16;
        half8_t *buf = my_ring + ring_i * kSlabWavePieces;
        __builtin_amdgcn_global_load_lds((gptr_t)(src), (lptr_t)(buf), 16, 0, DFL_W_AUX);
        __builtin_amdgcn_global_load_lds((gptr_t)(src + 1024), (lptr_t)(buf + 64), 16, 0, DFL_W_AUX);
        if (lane < 16) __builtin_amdgcn_global_load_lds((gptr_t)(src + 2048), (lptr_t)(buf + 128), 16, 0, DFL_W_AUX);
        w_issued++;
        ring_i = ring_i + 1 == depth ? 0 : ring_i + 1;
        if (++it_s < chunk_len(it_c)) return;
        it_s = 0;
        if (++it_h < h_end) return;
        it_h = h_begin;
        if (++it_c < n_chunks) return;
        it_c = 0;
        it_r++;
        it_seek();
    };

    // ---- prologue: the first activations (oldest loads), two weight stages, then the slab ----
    int slab_slot = xslot_of(0), slab_chunk = 0;
    if (!kRoute) load_x(slab_slot, 0);
    it_seek();
    for (int t = 0; t < 2; t++)
        if (it_valid) issue();
    DFL_TRE(2);
    q4k_wait_vm(3 * w_issued);  // the activations are older than every weight load
    convert(0);
    __builtin_amdgcn_s_waitcnt(kWaitLds);
    __builtin_amdgcn_s_barrier();
    DFL_TRE(3);
    bool x_pending = false;  // activations of the next refill are on their way (issued when w_issued was x_pos)
    int x_pos = 0;

    const int n = lane & 15, g = lane >> 4;
    const uint32_t sc_sel = (lane & 16) ? 0x04030402u : 0x04010400u;
    const Q4KMagic magic = q4k_magic();
    for (int r = 0; r < n_rounds; r++) {
        int slot = 0, tile = 0;
        const bool active = unit_of(r, slot, tile);
        const int xslot = xslot_of(r);
        float4_t acc0 = {0, 0, 0, 0}, acc1 = {0, 0, 0, 0};
        for (int c = 0; c < n_chunks; c++) {
            if (xslot != slab_slot || c != slab_chunk) {
                __builtin_amdgcn_s_barrier();  // every wave has read what it needed of the old slab
                if (x_pending) q4k_wait_vm(3 * min(w_issued - x_pos, w_issued - w_done));
                x_pending = false;
                convert(c);
                __builtin_amdgcn_s_waitcnt(kWaitLds);
                __builtin_amdgcn_s_barrier();
                slab_slot = xslot;
                slab_chunk = c;
            }
            // the activations of the step after this one, if they differ, start now
            {
                int nslot = -1, nc = 0;
                if (c + 1 < n_chunks) {
                    nslot = xslot;
                    nc = c + 1;
                } else if (r + 1 < n_rounds) {
                    nslot = xslot_of(r + 1);
                }
                if (nslot >= 0 && (nslot != slab_slot || nc != slab_chunk)) {
                    load_x(nslot, nc);
                    x_pending = true;
                    x_pos = w_issued;
                }
            }
            while (w_issued - w_done < depth && it_valid) issue();  // (fills the ring once, after the prologue)
            if (!active) continue;
            const int clen = chunk_len(c);
            for (int h = h_begin; h < h_end; h++) {
                for (int s = 0; s < clen; s++) {
                    // stage w_done has landed when only younger loads are in flight
                    const bool x_younger = x_pending && x_pos > w_done;
                    q4k_wait_vm(3 * (w_issued - 1 - w_done) + (x_younger ? kXInstr : 0));
                    if (!x_younger) x_pending = false;
                    if (w_done == 0) DFL_TRE(4);
                    const u32x4_t *blk = reinterpret_cast<const u32x4_t *>(my_ring + ring_c * kSlabWavePieces) + n * 9;
                    if (h == 0)
                        q4k_experts_compute(blk, slab + s * kTiledStageX, lane, g, sc_sel, magic, acc0);
                    else
                        q4k_experts_compute(blk, slab + s * kTiledStageX, lane, g, sc_sel, magic, acc1);
                    w_done++;
                    ring_c = ring_c + 1 == depth ? 0 : ring_c + 1;
                    if (it_valid) issue();  // the next stage into the buffer this one has just been read out of
                }
            }
        }
        if (r + 1 == n_rounds) DFL_TRE(5);
        if (hsplit) {  // the up tile crosses to the wave that holds the gate tile
            float4_t *xchg = reinterpret_cast<float4_t *>(reinterpret_cast<uint8_t *>(lds) + kExpRingEnd) + (wave & 7) * 64 + lane;
            if (active && wave >= kW / 2) *xchg = acc1;
            __builtin_amdgcn_s_waitcnt(kWaitLds);
            __builtin_amdgcn_s_barrier();
            if (active && wave < kW / 2) acc1 = *xchg;
        }
        if (active && !(hsplit && wave >= kW / 2)) {
            float4_t res = acc0;
            if (bt.pair) {
#pragma unroll
                for (int i = 0; i < 4; i++) res[i] = res[i] / (1.0f + expf(-res[i])) * acc1[i];  // silu(gate) * up
            }
            // (rare path: an opaque copy of the lane index keeps its address arithmetic out of the stage loop's registers)
            int ol = lane;
            asm volatile("" : "+v"(ol));
            const int on = ol & 15, og = ol >> 4;
            YT *yo = y + static_cast<size_t>(slot) * bt.y_stride;
            const int orow = tile * 16 + on;
            if (orow < n_out) {
#pragma unroll
                for (int i = 0; i < 4; i++)
                    if (4 * og + i < n_rows) yo[static_cast<size_t>(4 * og + i) * n_out + orow] = static_cast<YT>(res[i]);
            }
        }
    }
    DFL_TRE(6);
    DFL_TRE_FLUSH;
}

// ----------------------------------------------------------------------------
// Q6_K streaming kernel
// ----------------------------------------------------------------------------
//
// Same work split, activation path, flush and split-K reduction as the Q4_K stream above (one
// workgroup per CU walks a contiguous range of (tile group x super-block), activations of a stage
// are converted once per workgroup into MFMA fragments in LDS).  The weight path differs: a Q6_K
// block is 210 bytes, so rows are only 2-byte aligned and are not copied straight into LDS.
// Instead every wave stages its own 16 rows: the 13 16-byte pieces of each row's block (and its f16
// d) are loaded into registers one stage ahead with wide unaligned loads - consecutive lanes take
// consecutive pieces, so a row's 208 bytes are fetched as one run - and written to a private,
// double-buffered LDS area at the top of the next stage.  Private areas need no barrier; the one
// barrier per stage is for the shared activation fragments.
//
// Lane (n, g) of a wave serves weight row n, half h = g / 2 of the super-block and, in that half, the
// quarters (g & 1) and 2 + (g & 1): the low and the high nibbles of the SAME 32 ql bytes, with the
// bit pairs 2 (g & 1) and 4 + 2 (g & 1) of the half's 32 qh bytes.  MFMA t < 4 takes elements
// 8 t .. 8 t + 7 of the low quarter, t >= 4 those of the high quarter.  A 6-bit value is assembled
// in the mantissa of an f16 1024.0 (low nibble | qh bits << 4) or 64.0 (high nibble, sitting four
// bits up, | qh bits << 8), and one packed fma per pair gives round(q * s), s = d * scale, exactly as
// for Q4_K.  The format's offset, -32 s per weight, is not folded into that fma (-1056 s is not
// exact in f16 and the error would be a quarter of a quant step on every weight of a sub-block):
// like the Q4_K minima it goes through a twin MFMA, the same activation fragment times 32 s
// repeated eight times, into a second accumulator that is subtracted at the end.
constexpr int kQ6KRowStride = 240;  // bytes between a wave's staged rows in LDS (210 used)

template <int kWaves>
struct Q6KGeom {
    static constexpr int kThreads = 64 * kWaves;
    static constexpr int kRows = 16 * kWaves;
    static constexpr int kWaveBytes = 16 * kQ6KRowStride;  // one staged block of a wave's 16 rows
    static constexpr int kWBytes = 2 * kWaves * kWaveBytes;
    static constexpr int kLdsBytes = kWBytes + 2 * kQ4KBlockFrags * 16;
};

// Activation item of a thread for the Q6_K lane assignment (see q4k_lane_x_offsets for the thread
// -> (row, four values) map): values k = 4 c .. 4 c + 3 of the super-block belong to half c / 32,
// quarter (c / 8) % 4, elements 4 (c % 8) ..
template <int kWaves, typename XT>
__device__ __forceinline__ void q6k_lane_x_offsets(Q4KLane<kWaves> &L, int tid, int n_rows, uint32_t n_in) {
    using G = Q4KGeom<kWaves>;
    const int lane = tid & 63, wave = tid >> 6;
#pragma unroll
    for (int r = 0; r < G::kXLoads; r++) {
        const int vw = wave + kWaves * r;
        const int m = 8 * (vw & 1) + (lane & 7), c = 8 * (vw >> 1) + (lane >> 3);
        const int h = c >> 5, quarter = (c >> 3) & 3, l4 = c & 7;
        const int g = 2 * h + (quarter & 1), t = 4 * (quarter >> 1) + (l4 >> 1);
        L.x_off[r] = (static_cast<uint32_t>(min(m, n_rows - 1)) * n_in + 4u * c) * static_cast<uint32_t>(sizeof(XT));
        L.xw_off[r] = static_cast<uint32_t>((t * 64 + m + 16 * g) * 16 + 8 * (l4 & 1));
    }
}

// A wave's weight registers for one stage: 208 16-byte pieces (16 rows x 13) over 64 lanes, and d.
struct Q6KRegs {
    u32x4_t p[4];
    uint32_t d;
};

struct Q6KLane {
    uint32_t g_off[4];  // global byte offset of piece j from (group's first row, super-block)
    uint32_t l_off[4];  // its LDS byte offset in the wave's area
    uint32_t gd_off;    // d of row (lane % 16)
    bool live3;         // the fourth piece exists (lane + 192 < 208); other lanes re-load piece 207 and drop it
};

__device__ __forceinline__ void q6k_lane_w_offsets(Q6KLane &W, int lane, int wave, int row0, int n_out, uint32_t row_bytes) {
    const int last = n_out - 1 - row0;  // rows past n_out (ragged last group) re-read the last row
#pragma unroll
    for (int j = 0; j < 4; j++) {
        const int i = min(lane + 64 * j, 207);
        const int r = i / 13, piece = i % 13;
        W.g_off[j] = static_cast<uint32_t>(min(wave * 16 + r, last)) * row_bytes + 16u * piece;
        W.l_off[j] = static_cast<uint32_t>(r * kQ6KRowStride + 16 * piece);
    }
    W.live3 = lane + 192 < 208;
    W.gd_off = static_cast<uint32_t>(min(wave * 16 + (lane & 15), last)) * row_bytes + 208u;
}

// Five loads per wave and stage (four 16-byte pieces and d), written as asm like the activation
// loads and for the same reason: the kernel's own s_waitcnt at the top of a stage covers them, and
// the compiler must not drain younger loads on their account.  The addresses are only 2-byte
// aligned; gfx950 runs with unaligned vector memory access enabled.
constexpr int kQ6KLoads = 5;
__device__ __forceinline__ void q6k_load_w(const uint8_t *wstage, const Q6KLane &W, Q6KRegs &R) {
#pragma unroll
    for (int j = 0; j < 4; j++)
        asm volatile("global_load_dwordx4 %0, %1, %2" : "=v"(R.p[j]) : "v"(W.g_off[j]), "s"(wstage) : "memory");
    asm volatile("global_load_ushort %0, %1, %2" : "=v"(R.d) : "v"(W.gd_off), "s"(wstage) : "memory");
}

// after the s_waitcnt that covers R: its uses cannot be scheduled above this point
__device__ __forceinline__ void q6k_pin_w(Q6KRegs &R) {
#pragma unroll
    for (int j = 0; j < 4; j++) asm volatile("" : "+v"(R.p[j]));
    asm volatile("" : "+v"(R.d));
}

__device__ __forceinline__ void q6k_store_w(uint8_t *area, const Q6KLane &W, const Q6KRegs &R, int lane) {
#pragma unroll
    for (int j = 0; j < 4; j++)
        if (j < 3 || W.live3) *reinterpret_cast<u32x4_t *>(area + W.l_off[j]) = R.p[j];
    if (lane < 16) *reinterpret_cast<uint16_t *>(area + lane * kQ6KRowStride + 208) = static_cast<uint16_t>(R.d);
}

template <int kWaves, typename XT>
__global__ void __launch_bounds__(64 * kWaves)
    gemm_q6k_stream_kernel(const uint8_t *__restrict__ w, const XT *__restrict__ x, float *__restrict__ y,
                           float *__restrict__ partials, int n_out, int nb, int n_rows, int n_groups, Q4KBatch bt) {
    using G6 = Q6KGeom<kWaves>;
    using G = Q4KGeom<kWaves>;
    extern __shared__ half8_t lds[];
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    Q4KRange rg;
    rg.nb = nb;
    rg.n_wg = gridDim.x;
    rg.total = n_groups * nb;
    rg.wg = q4k_range_index(blockIdx.x, rg.n_wg);
    rg.it_begin = static_cast<int>(q4k_div(static_cast<uint32_t>(rg.total) * rg.wg, bt.by_wg));
    rg.it_end = static_cast<int>(q4k_div(static_cast<uint32_t>(rg.total) * (rg.wg + 1), bt.by_wg));
    if (rg.it_begin >= rg.it_end) return;
    rg.first_group = static_cast<int>(q4k_div(rg.it_begin, bt.by_nb));
    const int b0 = rg.it_begin - rg.first_group * nb;
    const uint32_t row_bytes = static_cast<uint32_t>(nb) * DFL_Q6_K_BYTES;
    const uint32_t n_in = static_cast<uint32_t>(nb) * DFL_QK_K;
    const size_t group_bytes = static_cast<size_t>(G6::kRows) * row_bytes;
    constexpr uint32_t kXBlockBytes = DFL_QK_K * sizeof(XT);
    const bool ragged = n_groups * G6::kRows > n_out;

    Q6KLane W;
    q6k_lane_w_offsets(W, lane, wave, rg.first_group * G6::kRows, n_out, row_bytes);
    // cursors: weights (next stage to load), activations (next to load), compute
    const uint8_t *wstage = q4k_uniform(w + static_cast<size_t>(rg.first_group) * group_bytes + static_cast<size_t>(b0) * DFL_Q6_K_BYTES);
    int bw = b0, gw = rg.first_group, w_left = rg.it_end - rg.it_begin;
    const uint8_t *xblock = q4k_uniform(reinterpret_cast<const uint8_t *>(x) + static_cast<size_t>(b0) * kXBlockBytes);
    int bx = b0, x_left = w_left;
    auto advance_w = [&]() {
        wstage += DFL_Q6_K_BYTES;
        w_left--;
        if (++bw == nb) {
            bw = 0;
            gw++;
            if (w_left > 0) {
                wstage = q4k_uniform(w + static_cast<size_t>(gw) * group_bytes);
                // only the matrix's last group has rows to clamp (every other group's offsets are the same); the
                // lane index goes in through an opaque copy so that nothing of this rare path is kept in registers
                // (or spilled) across the stage loop
                if (ragged && gw == n_groups - 1) {
                    int ol = lane;
                    asm volatile("" : "+v"(ol));
                    q6k_lane_w_offsets(W, ol, wave, gw * G6::kRows, n_out, row_bytes);
                }
            }
        }
    };
    auto advance_x = [&]() {
        xblock += kXBlockBytes;
        x_left--;
        if (++bx == nb) {
            bx = 0;
            if (x_left > 0) xblock = reinterpret_cast<const uint8_t *>(x);
        }
    };
    uint8_t *area = reinterpret_cast<uint8_t *>(lds) + wave * (2 * G6::kWaveBytes);  // this wave's two weight buffers
    half8_t *x_c = reinterpret_cast<half8_t *>(reinterpret_cast<uint8_t *>(lds) + G6::kWBytes), *x_n = x_c + kQ4KBlockFrags;

    // prologue: weights of stage 0 into LDS, those of stage 1 into registers; activations of stages 0..2.
    // Load order from here on: ... W(d+1) at the top of stage d-1 | X(d+2) at its end | W(d+2) at the top
    // of stage d ...; the wait at the top of stage d leaves only the youngest activation loads in flight.
    Q6KRegs R;
    q6k_load_w(wstage, W, R);
    advance_w();
    Q4KLane<kWaves> L;
    q6k_lane_x_offsets<kWaves, XT>(L, tid, n_rows, n_in);
    Q4KXRaw<kWaves, XT> raw_first, raw_a, raw_b;
    q4k_load_x<kWaves, XT>(xblock, L, raw_first);
    advance_x();
    if (x_left > 0) {
        q4k_load_x<kWaves, XT>(xblock, L, raw_a);
        advance_x();
    }
    __builtin_amdgcn_s_waitcnt(q4k_vmcnt(0));
    q6k_pin_w(R);
    q4k_pin_x<kWaves, XT>(raw_first);
    q4k_pin_x<kWaves, XT>(raw_a);
    q6k_store_w(area, W, R, lane);
    if (w_left > 0) {
        q6k_load_w(wstage, W, R);
        advance_w();
    }
    bool young_x = false;
    if (x_left > 0) {
        q4k_load_x<kWaves, XT>(xblock, L, raw_b);
        advance_x();
        young_x = true;
    }

    const int n = lane & 15, g = lane >> 4;
    const int h = g >> 1, odd = g & 1;
    const uint32_t magic_lo = 0x64006400u, magic_hi = 0x54005400u;
    float4_t acc = {0, 0, 0, 0}, acc_off = {0, 0, 0, 0}, stash = {0, 0, 0, 0};  // stash: unused here (no pair mode)
    int gc = rg.first_group, bc = b0, n_left = rg.it_end - rg.it_begin;
    int cur = 0;  // weight buffer of the stage being computed
    bool first = true;
    auto stage = [&](Q4KXRaw<kWaves, XT> &raw) {
        // everything but the activation loads issued at the end of the previous stage has landed:
        // the next stage's weights (in R) and the next stage's activations (in raw)
        if (young_x)
            __builtin_amdgcn_s_waitcnt(q4k_vmcnt(G::kXLoads));
        else
            __builtin_amdgcn_s_waitcnt(q4k_vmcnt(0));
        q6k_pin_w(R);
        q4k_pin_x<kWaves, XT>(raw);
        // the next stage's weights go into the other buffer, the ones after that into the registers
        if (n_left > 1) q6k_store_w(area + (cur ^ 1) * G6::kWaveBytes, W, R, lane);
        if (w_left > 0) {
            q6k_load_w(wstage, W, R);
            advance_w();
        }
        if (first) q4k_write_x<kWaves, XT>(x_c, L, raw_first);
        first = false;
        __builtin_amdgcn_s_waitcnt(kWaitLds);
        __builtin_amdgcn_s_barrier();  // the stage's activation fragments are complete; the other fragment buffer is free
        const uint8_t *rowp = area + cur * G6::kWaveBytes + n * kQ6KRowStride;
        const u32x4_t qa = *reinterpret_cast<const u32x4_t *>(rowp + 64 * h + 32 * odd);
        const u32x4_t qb = *reinterpret_cast<const u32x4_t *>(rowp + 64 * h + 32 * odd + 16);
        u32x4_t ha = *reinterpret_cast<const u32x4_t *>(rowp + 128 + 32 * h);
        u32x4_t hb = *reinterpret_cast<const u32x4_t *>(rowp + 128 + 32 * h + 16);
        // scales of the half: bytes 2 q + (0, 1) belong to quarter q
        const uint32_t sc4 = (*reinterpret_cast<const uint32_t *>(rowp + 192 + 8 * h) >> (16 * odd)) & 0xffffu;       // low quarter
        const uint32_t sc4h = (*reinterpret_cast<const uint32_t *>(rowp + 192 + 8 * h + 4) >> (16 * odd)) & 0xffffu;  // high quarter
        const float d = __half2float(__ushort_as_half(*reinterpret_cast<const uint16_t *>(rowp + 208)));
        const half8_t *a = x_c + lane;
        half8_t af[8];
#pragma unroll
        for (int t = 0; t < 8; t++) af[t] = a[t * 64];
        // this lane's qh bit pairs start at bit 2 odd (low quarter) and 4 + 2 odd (high quarter)
        const int hs = 2 * odd;
        const uint32_t hq[8] = {ha.x >> hs, ha.y >> hs, ha.z >> hs, ha.w >> hs, hb.x >> hs, hb.y >> hs, hb.z >> hs, hb.w >> hs};
        const uint32_t ql[8] = {qa.x, qa.y, qa.z, qa.w, qb.x, qb.y, qb.z, qb.w};
        auto scale = [&](uint32_t pair, int j) {
            return static_cast<_Float16>(d * static_cast<float>(static_cast<int8_t>(pair >> (8 * j))));
        };
        const _Float16 s_l0 = scale(sc4, 0), s_l1 = scale(sc4, 1), s_h0 = scale(sc4h, 0), s_h1 = scale(sc4h, 1);
#pragma unroll
        for (int t = 0; t < 4; t++) {
            const _Float16 sl = (t >> 1) ? s_l1 : s_l0;
            half8_t bl = unpack6<false>(ql[2 * t], ql[2 * t + 1], hq[2 * t], hq[2 * t + 1], splat(sl),
                                        splat(sl * static_cast<_Float16>(-1024.0f)), magic_lo);
            acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(af[t], bl, acc, 0, 0, 0);
            const _Float16 o = sl * static_cast<_Float16>(32.0f);
            const half8_t bo = {o, o, o, o, o, o, o, o};
            acc_off = __builtin_amdgcn_mfma_f32_16x16x32_f16(af[t], bo, acc_off, 0, 0, 0);
        }
        if (n_left > 1) q4k_write_x<kWaves, XT>(x_n, L, raw);
#pragma unroll
        for (int t = 0; t < 4; t++) {
            const _Float16 sh = (t >> 1) ? s_h1 : s_h0;
            half8_t bh = unpack6<true>(ql[2 * t], ql[2 * t + 1], hq[2 * t] >> 4, hq[2 * t + 1] >> 4, splat(sh),
                                       splat(sh * static_cast<_Float16>(-64.0f)), magic_hi);
            acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(af[4 + t], bh, acc, 0, 0, 0);
            const _Float16 o = sh * static_cast<_Float16>(32.0f);
            const half8_t bo = {o, o, o, o, o, o, o, o};
            acc_off = __builtin_amdgcn_mfma_f32_16x16x32_f16(af[4 + t], bo, acc_off, 0, 0, 0);
        }
        young_x = x_left > 0;
        if (young_x) {
            q4k_load_x<kWaves, XT>(xblock, L, raw);
            advance_x();
        }
        cur ^= 1;
        half8_t *tx = x_c;
        x_c = x_n;
        x_n = tx;
        n_left--;
        if (++bc == nb || n_left == 0) {
            q4k_flush<kWaves>(rg, bt, gc, acc, acc_off, stash, y, partials, n_out, n_rows, tid);
            bc = 0;
            gc++;
        }
    };
    while (n_left > 0) {
        stage(raw_a);
        if (n_left == 0) break;
        stage(raw_b);
    }
}

// ----------------------------------------------------------------------------
// Generic kernel (Q8_0): eight consecutive weights -> f16 -> MFMA
// ----------------------------------------------------------------------------

__device__ __forceinline__ float half_at(const uint8_t *p) {
    return __half2float(__ushort_as_half(static_cast<unsigned short>(p[0] | (p[1] << 8))));
}

// Eight weights of a row, in two halves so that the loads of several steps can be in flight before
// the first conversion: the raw bytes, then the f16 fragment.
template <int TYPE>
struct Raw8;

template <>
struct Raw8<DFLASH_TYPE_Q8_0> {
    uint64_t q;  // eight int8 quants
    float d;
};

__device__ __forceinline__ uint64_t load_u64_unaligned(const uint8_t *p) {
    uint64_t v;
    __builtin_memcpy(&v, p, 8);
    return v;
}

template <int TYPE>
__device__ __forceinline__ Raw8<TYPE> load_raw8(const uint8_t *row, int64_t k0);
template <int TYPE>
__device__ __forceinline__ half8_t convert_raw8(const Raw8<TYPE> &r);

// Blocks are 34 bytes, so the quants are only 2-byte aligned; gfx950 runs with unaligned vector
// memory access enabled and the copy below becomes one 8-byte load.
template <>
__device__ __forceinline__ Raw8<DFLASH_TYPE_Q8_0> load_raw8<DFLASH_TYPE_Q8_0>(const uint8_t *row, int64_t k0) {
    const uint8_t *blk = row + (k0 >> 5) * DFL_Q8_0_BYTES;
    Raw8<DFLASH_TYPE_Q8_0> r;
    r.d = half_at(blk);
    r.q = load_u64_unaligned(blk + 2 + (k0 & 31));
    return r;
}

// f16(d * q) for eight int8 quants.  d is an f16 value and q has eight bits, so d * q is exact in f32 and the one rounding
// to f16 is the rounding of the exact product: a packed f16 multiply of d by q gives the same bits.  q itself is made
// without conversions: byte q ^ 0x80 = q + 128 in the mantissa of f16 1024.0, minus 1152.0 (exact in f16), two at a time.
template <>
__device__ __forceinline__ half8_t convert_raw8<DFLASH_TYPE_Q8_0>(const Raw8<DFLASH_TYPE_Q8_0> &r) {
    const uint32_t w[2] = {static_cast<uint32_t>(r.q), static_cast<uint32_t>(r.q >> 32)};
    const half2_t d2 = splat(static_cast<_Float16>(r.d)), off = splat(static_cast<_Float16>(-1152.0f));
    half8_t v;
#pragma unroll
    for (int j = 0; j < 2; j++) {
        const half2_t lo = (as_half2(__builtin_amdgcn_perm(0x64646464u, w[j], 0x04010400u) ^ 0x00800080u) + off) * d2;
        const half2_t hi = (as_half2(__builtin_amdgcn_perm(0x64646464u, w[j], 0x04030402u) ^ 0x00800080u) + off) * d2;
        v[4 * j] = lo[0];
        v[4 * j + 1] = lo[1];
        v[4 * j + 2] = hi[0];
        v[4 * j + 3] = hi[1];
    }
    return v;
}

// Unquantised matrices (a router or a small projection stored as F32 / F16): rows are 16-byte multiples
// because n_in is a multiple of 32.
template <>
struct Raw8<DFLASH_TYPE_F32> {
    float4_t a, b;
};
template <>
struct Raw8<DFLASH_TYPE_F16> {
    half8_t v;
};
template <>
__device__ __forceinline__ Raw8<DFLASH_TYPE_F32> load_raw8<DFLASH_TYPE_F32>(const uint8_t *row, int64_t k0) {
    const float *p = reinterpret_cast<const float *>(row) + k0;
    return Raw8<DFLASH_TYPE_F32>{*reinterpret_cast<const float4_t *>(p), *reinterpret_cast<const float4_t *>(p + 4)};
}
template <>
__device__ __forceinline__ half8_t convert_raw8<DFLASH_TYPE_F32>(const Raw8<DFLASH_TYPE_F32> &r) {
    return half8_t{static_cast<_Float16>(r.a[0]), static_cast<_Float16>(r.a[1]), static_cast<_Float16>(r.a[2]),
                   static_cast<_Float16>(r.a[3]), static_cast<_Float16>(r.b[0]), static_cast<_Float16>(r.b[1]),
                   static_cast<_Float16>(r.b[2]), static_cast<_Float16>(r.b[3])};
}
template <>
__device__ __forceinline__ Raw8<DFLASH_TYPE_F16> load_raw8<DFLASH_TYPE_F16>(const uint8_t *row, int64_t k0) {
    return Raw8<DFLASH_TYPE_F16>{*reinterpret_cast<const half8_t *>(reinterpret_cast<const _Float16 *>(row) + k0)};
}
template <>
__device__ __forceinline__ half8_t convert_raw8<DFLASH_TYPE_F16>(const Raw8<DFLASH_TYPE_F16> &r) {
    return r.v;
}

// Eight consecutive activations (16-byte aligned) in two halves as well: the raw load, then the f16
// fragment.
template <typename XT>
struct RawX8;
template <>
struct RawX8<float> {
    float4_t a, b;
};
template <>
struct RawX8<_Float16> {
    half8_t v;
};
__device__ __forceinline__ RawX8<float> load_rawx8(const float *p) {
    return RawX8<float>{*reinterpret_cast<const float4_t *>(p), *reinterpret_cast<const float4_t *>(p + 4)};
}
__device__ __forceinline__ RawX8<_Float16> load_rawx8(const _Float16 *p) {
    return RawX8<_Float16>{*reinterpret_cast<const half8_t *>(p)};
}
__device__ __forceinline__ half8_t convert_rawx8(const RawX8<float> &r) {
    return half8_t{static_cast<_Float16>(r.a[0]), static_cast<_Float16>(r.a[1]), static_cast<_Float16>(r.a[2]),
                   static_cast<_Float16>(r.a[3]), static_cast<_Float16>(r.b[0]), static_cast<_Float16>(r.b[1]),
                   static_cast<_Float16>(r.b[2]), static_cast<_Float16>(r.b[3])};
}
__device__ __forceinline__ half8_t convert_rawx8(const RawX8<_Float16> &r) { return r.v; }

template <int TYPE, typename XT>
__global__ void __launch_bounds__(64 * kMaxSplit)
    gemm_generic_kernel(const uint8_t *__restrict__ w, const XT *__restrict__ x, float *__restrict__ y, int n_out,
                        int64_t n_steps, size_t row_bytes, int n_rows, int n_split) {
    extern __shared__ float red[];  // [n_split][256]
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int n = lane & 15, g = lane >> 4;
    const int n0 = blockIdx.x * 16;
    int row = n0 + n;
    row = row < n_out ? row : n_out - 1;
    const uint8_t *rowp = w + static_cast<size_t>(row) * row_bytes;
    const int64_t s0 = n_steps * wave / n_split, s1 = n_steps * (wave + 1) / n_split;
    // lane (m = n, g) of the A operand: activation row n, straight from the caller's matrix.  Lanes
    // past n_rows repeat the last row (a row of A only reaches the same row of the product, which is
    // never stored for them): no branch around the loads, so the loads of all steps can be in flight
    const XT *xrow = x + static_cast<size_t>(n < n_rows ? n : n_rows - 1) * (static_cast<size_t>(n_steps) * 32) + 8 * g;
    float4_t acc = {0, 0, 0, 0};
    for (int64_t s = s0; s < s1; s++) {
        const RawX8<XT> a = load_rawx8(xrow + 32 * s);
        const Raw8<TYPE> r = load_raw8<TYPE>(rowp, 32 * s + 8 * g);
        acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(convert_rawx8(a), convert_raw8<TYPE>(r), acc, 0, 0, 0);
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

// ----------------------------------------------------------------------------
// Q8_0, staged: the same product with both operands brought in through LDS
// ----------------------------------------------------------------------------
//
// The kernel above reads MFMA operands straight from memory: each 16-lane group of a load touches 16
// different rows, i.e. 16 cache lines for 256 bytes, and the texture path (one line per clock) bounds
// the kernel, not latency or bandwidth (measured: 10.5 us for a 128 x 2048 router, 6 us of it the
// address path; issuing all loads at once changed nothing).  Here a workgroup copies its 16 weight
// rows and the activations in row-contiguous 16-byte pieces (a wave-load = 8 full lines), converts
// the activations to f16 once, and every wave then takes its fragments from LDS:
//   X  [step][k-group][row] half8 pieces, a step's four groups 17 pieces apart (the writes, which
//      walk along a row, and the fragment reads, which walk along the rows, are both conflict-free);
//   W  the raw rows, 16 bytes of padding between rows (16 rows land in 16 different banks).
// K is walked in chunks of 2048; waves split a chunk's 64 steps and add up in LDS in wave order, so
// for n_in <= 2048 the result is bit-identical to the kernel above.  Needs n_in % 256 == 0 (rows of
// 34-byte blocks are then 16-byte multiples).
constexpr int kQ8ChunkSteps = 64;                                  // 2048 weights of a row
constexpr int kQ8XPieces = kQ8ChunkSteps * 68;                     // padded: 4 groups x 17 pieces per step
constexpr int kQ8WRowStride = kQ8ChunkSteps * DFL_Q8_0_BYTES + 16; // bytes
constexpr size_t kQ8StagedLds = static_cast<size_t>(kMaxSplit) * 256 * sizeof(float) + static_cast<size_t>(kQ8XPieces) * 16 +
                                16 * static_cast<size_t>(kQ8WRowStride);

template <typename XT>
__global__ void __launch_bounds__(64 * kMaxSplit)
    gemm_q8_0_staged_kernel(const uint8_t *__restrict__ w, const XT *__restrict__ x, float *__restrict__ y, int n_out,
                            int n_steps, size_t row_bytes, int n_rows_total, int n_split) {
    // blockIdx.y: which block of sixteen rows (a prefill group hands over many)
    const int n_rows = min(16, n_rows_total - 16 * static_cast<int>(blockIdx.y));
    x += static_cast<size_t>(blockIdx.y) * 16 * (static_cast<size_t>(n_steps) * 32);
    y += static_cast<size_t>(blockIdx.y) * 16 * n_out;
    extern __shared__ __attribute__((aligned(16))) float red[];  // [kMaxSplit][256], then X pieces, then W rows
    half8_t *xs = reinterpret_cast<half8_t *>(red + kMaxSplit * 256);
    uint8_t *ws = reinterpret_cast<uint8_t *>(xs + kQ8XPieces);
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int n = lane & 15, g = lane >> 4;
    const int n0 = blockIdx.x * 16;
    float4_t acc = {0, 0, 0, 0};
    for (int c0 = 0; c0 < n_steps; c0 += kQ8ChunkSteps) {
        const int cs = min(kQ8ChunkSteps, n_steps - c0);  // steps of this chunk (a multiple of 8)
        if (c0) __syncthreads();                          // the previous chunk's fragments have been read
        // weights: cs * 34 / 16 pieces per row
        const int wp_row = cs * DFL_Q8_0_BYTES / 16;
        for (int p = tid; p < 16 * wp_row; p += blockDim.x) {
            const int r = p / wp_row, c = p - r * wp_row;
            const int row = min(n0 + r, n_out - 1);
            *reinterpret_cast<u32x4_t *>(ws + r * kQ8WRowStride + 16 * c) = *reinterpret_cast<const u32x4_t *>(
                w + static_cast<size_t>(row) * row_bytes + static_cast<size_t>(c0) * DFL_Q8_0_BYTES + 16 * c);
        }
        // activations: 4 cs pieces of eight per row; rows past n_rows repeat the last one
        const int xp_row = 4 * cs;
        for (int p = tid; p < 16 * xp_row; p += blockDim.x) {
            const int r = p / xp_row, c = p - r * xp_row;
            const XT *src = x + static_cast<size_t>(min(r, n_rows - 1)) * (static_cast<size_t>(n_steps) * 32) +
                            static_cast<size_t>(c0) * 32 + 8 * c;
            xs[(c >> 2) * 68 + (c & 3) * 17 + r] = convert_rawx8(load_rawx8(src));
        }
        __syncthreads();
        const int s0 = cs * wave / n_split, s1 = cs * (wave + 1) / n_split;
        const uint8_t *rowp = ws + n * kQ8WRowStride;
        for (int s = s0; s < s1; s++) {
            const uint8_t *blk = rowp + s * DFL_Q8_0_BYTES;  // 2-byte aligned
            const uint16_t *q16 = reinterpret_cast<const uint16_t *>(blk + 2 + 8 * g);
            Raw8<DFLASH_TYPE_Q8_0> r;
            r.d = static_cast<float>(__builtin_bit_cast(_Float16, *reinterpret_cast<const uint16_t *>(blk)));
            r.q = static_cast<uint64_t>(q16[0]) | (static_cast<uint64_t>(q16[1]) << 16) | (static_cast<uint64_t>(q16[2]) << 32) |
                  (static_cast<uint64_t>(q16[3]) << 48);
            acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(xs[s * 68 + g * 17 + n], convert_raw8<DFLASH_TYPE_Q8_0>(r), acc, 0, 0, 0);
        }
    }
#pragma unroll
    for (int i = 0; i < 4; i++) red[wave * 256 + (4 * g + i) * 16 + n] = acc[i];
    __syncthreads();
    for (int e = tid; e < 256; e += blockDim.x) {
        const int m = e >> 4, nn = e & 15;
        if (m < n_rows && n0 + nn < n_out) {
            float sum = 0.0f;
            for (int wv = 0; wv < n_split; wv++) sum += red[wv * 256 + e];
            y[static_cast<size_t>(m) * n_out + n0 + nn] = sum;
        }
    }
}

// The router of a mixture-of-experts layer together with the residual add, the RMSNorm and the shared-expert gate
// that precede it (rms_norm_kernel of the model followed by the kernel above, as one launch).  One workgroup per
// (16 experts, block row): it normalises its row of x + add exactly as the norm kernel does (256 threads, the row in
// registers), keeps the f16 copy in LDS as the one live row of the MFMA's X operand (the other fifteen are zeros: a
// row's products do not depend on its neighbours) and multiplies it with its 16 staged weight rows.  The kernel
// above gives a workgroup all 16 rows, 162 KB to take in where this one takes 50 KB, and a CU takes in only 20-30 KB
// per microsecond: 16 x 8 small workgroups instead of 8 large ones, and no launch for the norm.  (Measured first
// with the norm of all 16 rows inside each of the 8 workgroups, 290 KB each: slower than the two launches.)  The
// workgroups of tile 0 write the row's f32 copy (cur, read by the expert products) and its gate.  x itself is NOT
// updated (other workgroups are still reading the row): the caller adds `add` again where it next updates the
// residual.  Sums are taken in rms_norm_kernel's order (the first four waves do the norm) and the product in the order
// of the kernel above with 16 waves, so cur, gate_out and y have the bits of the two separate launches.  One 64-step
// chunk: hidden <= 2048.
__global__ void __launch_bounds__(64 * kMaxSplit)
    q8_0_norm_router_kernel(const uint8_t *__restrict__ w, const float *__restrict__ x, const float *__restrict__ add,
                            const float *__restrict__ norm_w, const float *__restrict__ gate_w, float eps,
                            float *__restrict__ cur, float *__restrict__ gate_out, float *__restrict__ y, int n_out,
                            int n_steps, size_t row_bytes) {
    typedef float f4 __attribute__((ext_vector_type(4)));
    typedef _Float16 h4 __attribute__((ext_vector_type(4)));
    __shared__ __attribute__((aligned(16))) uint8_t ws[16 * kQ8WRowStride];  // the raw weight rows, padded as above
    __shared__ half8_t xrow[4 * kQ8ChunkSteps];                              // [step][k-group]: the normalised row
    __shared__ float red[kMaxSplit][16];
    __shared__ float sq_part[4], dot_part[4];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int n = lane & 15, g = lane >> 4;
    const int n0 = blockIdx.x * 16, r = blockIdx.y;
    const int hidden = 32 * n_steps;
    const bool first_tile = blockIdx.x == 0;
    const bool norm_wave = wave < 4;  // the norm is the work of 256 threads, as in rms_norm_kernel; the row's loads go out first
    DFL_TRR(0);
    f4 v[2] = {f4{0, 0, 0, 0}, f4{0, 0, 0, 0}}, nw[2] = {f4{0, 0, 0, 0}, f4{0, 0, 0, 0}};
    if (norm_wave) {
        const float *xr = x + static_cast<size_t>(r) * hidden, *ar = add + static_cast<size_t>(r) * hidden;
#pragma unroll
        for (int j = 0; j < 2; j++) {
            const int i = 4 * (tid + 256 * j);
            if (i < hidden) {
                v[j] = *reinterpret_cast<const f4 *>(xr + i) + *reinterpret_cast<const f4 *>(ar + i);
                nw[j] = *reinterpret_cast<const f4 *>(norm_w + i);
            }
        }
    }
    const int wp_row = n_steps * DFL_Q8_0_BYTES / 16;
    for (int p = tid; p < 16 * wp_row; p += 64 * kMaxSplit) {
        const int wr = p / wp_row, c = p - wr * wp_row;
        const int row = min(n0 + wr, n_out - 1);
        *reinterpret_cast<u32x4_t *>(ws + wr * kQ8WRowStride + 16 * c) =
            *reinterpret_cast<const u32x4_t *>(w + static_cast<size_t>(row) * row_bytes + 16 * c);
    }
    if (norm_wave) {
        float s = 0.0f;
#pragma unroll
        for (int j = 0; j < 2; j++)
            s += (v[j][0] * v[j][0] + v[j][1] * v[j][1]) + (v[j][2] * v[j][2] + v[j][3] * v[j][3]);
        for (int off = 32; off > 0; off >>= 1) s += __shfl_xor(s, off, 64);
        if (lane == 0) sq_part[wave] = s;
    }
    DFL_TRR(1);
    __syncthreads();
    DFL_TRR(2);
    if (norm_wave) {
        float tot = 0.0f;
#pragma unroll
        for (int k = 0; k < 4; k++) tot += sq_part[k];
        const float scale = 1.0f / sqrtf(tot / static_cast<float>(hidden) + eps);
        float dot = 0.0f;
#pragma unroll
        for (int j = 0; j < 2; j++) {
            const int i = 4 * (tid + 256 * j);
            if (i < hidden) {
                const f4 o = v[j] * scale * nw[j];
                if (first_tile) {
                    *reinterpret_cast<f4 *>(cur + static_cast<size_t>(r) * hidden + i) = o;
                    const f4 gw = *reinterpret_cast<const f4 *>(gate_w + i);
                    dot += (o[0] * gw[0] + o[1] * gw[1]) + (o[2] * gw[2] + o[3] * gw[3]);
                }
                // values 8 c .. 8 c + 7 are piece c = 4 step + k-group; this thread's four are its lower or upper half
                h4 *piece = reinterpret_cast<h4 *>(&xrow[i >> 3]);
                piece[(i >> 2) & 1] = h4{static_cast<_Float16>(o[0]), static_cast<_Float16>(o[1]), static_cast<_Float16>(o[2]),
                                         static_cast<_Float16>(o[3])};
            }
        }
        if (first_tile) {  // (the same for the whole workgroup)
            for (int off = 32; off > 0; off >>= 1) dot += __shfl_xor(dot, off, 64);
            if (lane == 0) dot_part[wave] = dot;
        }
    }
    DFL_TRR(3);
    __syncthreads();  // the row, the weight rows and the gate's partial sums are in LDS
    DFL_TRR(4);
    if (first_tile && tid == 0) {
        float d = 0.0f;
        for (int k = 0; k < 4; k++) d += dot_part[k];
        gate_out[r] = 1.0f / (1.0f + expf(-d));
    }
    const uint8_t *rowp = ws + n * kQ8WRowStride;
    const half8_t zero = {0, 0, 0, 0, 0, 0, 0, 0};
    const int s0 = n_steps * wave / kMaxSplit, s1 = n_steps * (wave + 1) / kMaxSplit;
    float4_t acc = {0, 0, 0, 0};
    for (int st = s0; st < s1; st++) {
        const uint8_t *blk = rowp + st * DFL_Q8_0_BYTES;  // 2-byte aligned
        const uint16_t *q16 = reinterpret_cast<const uint16_t *>(blk + 2 + 8 * g);
        Raw8<DFLASH_TYPE_Q8_0> rw;
        rw.d = static_cast<float>(__builtin_bit_cast(_Float16, *reinterpret_cast<const uint16_t *>(blk)));
        rw.q = static_cast<uint64_t>(q16[0]) | (static_cast<uint64_t>(q16[1]) << 16) | (static_cast<uint64_t>(q16[2]) << 32) |
               (static_cast<uint64_t>(q16[3]) << 48);
        const half8_t piece = xrow[4 * st + g];
        acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(n == (r & 15) ? piece : zero, convert_raw8<DFLASH_TYPE_Q8_0>(rw), acc, 0, 0, 0);
    }
    // the row rides in MFMA row r % 16 (any one would do: the other fifteen are zeros): lane group (r % 16) / 4, element r % 4
    const int ri = r & 3;
    const float mine = ri == 0 ? acc[0] : ri == 1 ? acc[1] : ri == 2 ? acc[2] : acc[3];
    if (g == ((r & 15) >> 2)) red[wave][n] = mine;
    DFL_TRR(5);
    __syncthreads();
    DFL_TRR(6);
    if (tid < 16 && n0 + tid < n_out) {
        float sum = 0.0f;
        for (int wv = 0; wv < kMaxSplit; wv++) sum += red[wv][tid];
        y[static_cast<size_t>(r) * n_out + n0 + tid] = sum;
    }
    DFL_TRR(7);
}

// ----------------------------------------------------------------------------
// Q6_K kernel: half a super-block (128 weights of a row) per lane group and step
// ----------------------------------------------------------------------------
//
// A wave owns a 16-row tile and a run of half super-blocks; lane (n, g) serves weight row n and, in
// each of the half's four 32-element quarters, the eight weights 8 g .. 8 g + 7.  ggml's Q6_K packing
// (ql[128], qh[64], int8 scales[16], f16 d; metal/tests/q6_k_f32_tile.rs:46-71) makes those 32 weights
// come from just three 8-byte runs (two of ql, one of qh), eight scale bytes and d, so a lane issues
// five loads per four MFMAs.  Blocks are 210 bytes, so these loads are only 2-byte aligned; gfx950
// runs with unaligned vector memory access enabled and the compiler emits them as single loads.
// Activations are read from the caller's matrix and rounded to f16 on the fly (all tiles read the
// same rows: L2 hits).  Waves of a workgroup split K and add their tiles up in LDS in wave order.
// Up to three matrices that share the activations (the q, k and v projections of a layer) in one
// launch: workgroup b serves tile b - tile_begin[m] of the matrix m whose tile range holds b.
struct Q6KSet {
    const uint8_t *w[3];
    float *y[3];
    int n_out[3];
    int tile_begin[3];
    int n_mats;
};

template <typename XT>
__global__ void __launch_bounds__(64 * kMaxSplit)
    gemm_q6k_kernel(Q6KSet set, const XT *__restrict__ x, int nb, size_t row_bytes, int n_rows, int n_split) {
    extern __shared__ float red[];  // [n_split][256]
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int n = lane & 15, g = lane >> 4;
    int mat = 0;
    if (set.n_mats > 1 && static_cast<int>(blockIdx.x) >= set.tile_begin[1]) mat = 1;
    if (set.n_mats > 2 && static_cast<int>(blockIdx.x) >= set.tile_begin[2]) mat = 2;
    const uint8_t *__restrict__ w = set.w[mat];
    float *__restrict__ y = set.y[mat];
    const int n_out = set.n_out[mat];
    const int n0 = (blockIdx.x - set.tile_begin[mat]) * 16;
    const int row = min(n0 + n, n_out - 1);
    const uint8_t *rowp = w + static_cast<size_t>(row) * row_bytes;
    const int n_half = 2 * nb;
    const int h0 = n_half * wave / n_split, h1 = n_half * (wave + 1) / n_split;
    // lane (m = n, g) of the A operand: activation row n (lanes past n_rows repeat the last row: a
    // row of A only reaches the same row of the product, which is never stored for them)
    const XT *xrow = x + static_cast<size_t>(n < n_rows ? n : n_rows - 1) * (static_cast<size_t>(nb) * DFL_QK_K) + 8 * g;
    float4_t acc = {0, 0, 0, 0};
    for (int hb = h0; hb < h1; hb++) {
        const uint8_t *blk = rowp + static_cast<size_t>(hb >> 1) * DFL_Q6_K_BYTES;
        const int half = hb & 1;
        const uint64_t qa = load_u64_unaligned(blk + 64 * half + 8 * g);
        const uint64_t qb = load_u64_unaligned(blk + 64 * half + 32 + 8 * g);
        const uint64_t qh = load_u64_unaligned(blk + 128 + 32 * half + 8 * g);
        const uint64_t sc = load_u64_unaligned(blk + 192 + 8 * half);
        const float d = half_at(blk + 208);
        const XT *xk = xrow + static_cast<size_t>(hb) * 128;
#pragma unroll
        for (int kq = 0; kq < 4; kq++) {
            const int is = (g >> 1) + 2 * kq;
            const float ds = d * static_cast<float>(static_cast<int8_t>(sc >> (8 * is)));
            const float off = -32.0f * ds;
            const uint64_t src = (kq & 1) ? qb : qa;
            const uint64_t lo = ((kq & 2) ? (src >> 4) : src) & 0x0F0F0F0F0F0F0F0Full;
            const uint64_t hi = ((qh >> (2 * kq)) & 0x0303030303030303ull) << 4;
            const uint64_t q = lo | hi;
            const uint32_t q0 = static_cast<uint32_t>(q), q1 = static_cast<uint32_t>(q >> 32);
            half8_t b;
#pragma unroll
            for (int i = 0; i < 4; i++) {
                b[i] = static_cast<_Float16>(__builtin_fmaf(static_cast<float>((q0 >> (8 * i)) & 0xffu), ds, off));
                b[4 + i] = static_cast<_Float16>(__builtin_fmaf(static_cast<float>((q1 >> (8 * i)) & 0xffu), ds, off));
            }
            acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(convert_rawx8(load_rawx8(xk + 32 * kq)), b, acc, 0, 0, 0);
        }
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

}  // namespace

#ifdef DFLASH_TRACE
extern "C" void dflash_dbg_set_trace(uint64_t p) {
    unsigned long long *v = reinterpret_cast<unsigned long long *>(p);
    (void)hipMemcpyToSymbol(HIP_SYMBOL(g_trace), &v, sizeof(v));
}
extern "C" void dflash_dbg_set_trace2(uint64_t p) {
    unsigned long long *v = reinterpret_cast<unsigned long long *>(p);
    (void)hipMemcpyToSymbol(HIP_SYMBOL(g_trace2), &v, sizeof(v));
}
#endif

namespace {

// Tuning knobs from the environment, each read once per process (getenv walks the whole environment,
// and a launch-bound caller pays for that on every launch).
struct EnvInt {
    bool set;
    int value;
    explicit EnvInt(const char *name) {
        const char *v = getenv(name);
        set = v && *v;
        value = set ? atoi(v) : 0;
    }
    int get(int fallback) const { return set ? value : fallback; }
};
#define env_int(name, fallback) ([]() -> const EnvInt & { static const EnvInt e(name); return e; }().get(fallback))

int32_t launch_q6k(dflash_ctx *ctx, Q6KSet set, const void *x, int32_t x_type, int64_t n_in, int32_t n_rows, hipStream_t st) {
    if (reinterpret_cast<uintptr_t>(x) % (x_type == DFLASH_TYPE_F32 ? 16 : 8))
        return dfl_fail(ctx, DFLASH_ERR_ALIGNMENT, "gemm_fewrow: activations must be 16-byte (f32) / 8-byte (f16) aligned");
    const int nb = static_cast<int>(n_in / DFL_QK_K);
    const size_t row_bytes = static_cast<size_t>(nb) * DFL_Q6_K_BYTES;
    int tiles = 0;
    for (int m = 0; m < set.n_mats; m++) {
        set.tile_begin[m] = tiles;
        tiles += (set.n_out[m] + 15) / 16;
    }
    // waves of a workgroup split K: enough waves in total to fill the chip
    const int target_waves = 8 * ctx->n_cu;
    int split = (target_waves + tiles - 1) / tiles;
    split = env_int("DFLASH_GEMM_NSPLIT", split);
    if (split > 2 * nb) split = 2 * nb;
    if (split > kMaxSplit) split = kMaxSplit;
    if (split < 1) split = 1;
    const size_t lds = static_cast<size_t>(split) * 256 * sizeof(float);
    dfl_timed timer(ctx, st, DFL_T_GEMM);
    if (x_type == DFLASH_TYPE_F32)
        gemm_q6k_kernel<float><<<tiles, 64 * split, lds, st>>>(set, static_cast<const float *>(x), nb, row_bytes, n_rows, split);
    else
        gemm_q6k_kernel<_Float16><<<tiles, 64 * split, lds, st>>>(set, static_cast<const _Float16 *>(x), nb, row_bytes, n_rows, split);
    return DFLASH_OK;
}

}  // namespace

int32_t dfl_gemm_q6k_set(dflash_ctx *ctx, int n_mats, const void *const *w, float *const *y, const int64_t *n_out, const void *x,
                         int32_t x_type, int64_t n_in, int32_t n_rows, dflash_stream_t stream) {
    if (n_mats < 1 || n_mats > 3 || n_in <= 0 || n_in % DFL_QK_K || n_rows < 1 || n_rows > 16)
        return dfl_fail(ctx, DFLASH_ERR_BAD_SHAPE, "gemm_q6k_set: bad shape");
    Q6KSet set = {};
    set.n_mats = n_mats;
    for (int m = 0; m < n_mats; m++) {
        if (!w[m] || !y[m] || n_out[m] <= 0 || n_out[m] > 0x7fffffffll || reinterpret_cast<uintptr_t>(w[m]) % 2)
            return dfl_fail(ctx, DFLASH_ERR_INVALID_INPUT, "gemm_q6k_set: matrix %d", m);
        set.w[m] = static_cast<const uint8_t *>(w[m]);
        set.y[m] = y[m];
        set.n_out[m] = static_cast<int>(n_out[m]);
    }
    const int32_t rc = launch_q6k(ctx, set, x, x_type, n_in, n_rows, static_cast<hipStream_t>(stream));
    if (rc) return rc;
    DFL_HIP_CHECK(ctx, hipGetLastError());
    return DFLASH_OK;
}

namespace {

// The product for a Q4_K / Q6_K tensor that was not range-checked: every weight dequantised in f32 exactly as ggml does
// (dfl_dequant_elem), f32 activations (f16 ones widened), f32 sums.  Correct for every block the format can hold - the
// contract of the reference's seam, whose kernels scale in f32 after the MMA (mat_mat_fewrow_gen.metal:437-444) - and slow:
// one wave per weight row, no matrix cores.  Lanes stride over K, sixteen row sums per lane, a butterfly at the end.
template <typename XT>
__global__ void __launch_bounds__(256)
    gemm_safe_kernel(int type, const uint8_t *__restrict__ w, size_t row_bytes, const XT *__restrict__ x, float *__restrict__ y, int n_in,
                     int n_out, int n_rows) {
    const int row = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
    if (row >= n_out) return;
    const uint8_t *wr = w + static_cast<size_t>(row) * row_bytes;
    float acc[16];
#pragma unroll
    for (int m = 0; m < 16; m++) acc[m] = 0.0f;
    for (int k = lane; k < n_in; k += 64) {
        const float wv = dfl_dequant_elem(type, wr, k);
#pragma unroll
        for (int m = 0; m < 16; m++)
            if (m < n_rows) acc[m] += wv * static_cast<float>(x[static_cast<size_t>(m) * n_in + k]);
    }
#pragma unroll
    for (int m = 0; m < 16; m++) {
        float v = acc[m];
        for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
        if (lane == 0 && m < n_rows) y[static_cast<size_t>(m) * n_out + row] = v;
    }
}

// Launches the streaming Q4_K kernel (and its split-K reduction): one matrix (batch == nullptr) or the
// matrices a device-side list picks out of a stack (at most max_slots of them).
int32_t launch_q4k(dflash_ctx *ctx, const void *w, const void *x, int32_t x_type, float *y, int64_t n_in, int64_t n_out,
                   int32_t n_rows, hipStream_t st, const Q4KBatch *batch, int max_slots, bool tiled = false) {
    const int nb = static_cast<int>(n_in / DFL_QK_K);
    const size_t row_bytes = static_cast<size_t>(nb) * DFL_Q4_K_BYTES;
    const int tiles = static_cast<int>((n_out + 15) / 16);
    if (reinterpret_cast<uintptr_t>(x) % (x_type == DFLASH_TYPE_F32 ? 16 : 8))
        return dfl_fail(ctx, DFLASH_ERR_ALIGNMENT, "gemm_fewrow: activations must be 16-byte (f32) / 8-byte (f16) aligned");
    // whole-K batch over tiled matrices: one 16-row tile per wave (gemm_q4k_experts_kernel).  A plain product over a
    // shared x with less than two tiles per wave-slot of the chip (a drafter's five [wk; wv] pairs: 320 tiles) stays
    // with the streaming kernel: every workgroup of the expert kernel converts all of x for one or two tiles
    // (14.2 against 11.4 us for that launch).
    if (batch && dfl_q4k_batched_f16_out(ctx, tiled, batch->whole_groups, n_out) &&
        (batch->pair || batch->x_stride != 0 || batch->y_f16 || batch->route_logits || static_cast<int64_t>(max_slots) * tiles >= 2ll * ctx->n_cu)) {
        if (reinterpret_cast<uintptr_t>(x) % 16)
            return dfl_fail(ctx, DFLASH_ERR_ALIGNMENT, "gemm_q4k_batched: activations must be 16-byte aligned");
        const bool per_slot_x = batch->x_stride != 0;
        const int upm = per_slot_x ? (tiles + 15) / 16 : tiles;  // units per matrix
        int n_wg = env_int("DFLASH_MOE_WGS", ctx->batch_wgs > 0 ? ctx->batch_wgs : ctx->n_cu);
        if (n_wg < 1) n_wg = 1;
        if (static_cast<int64_t>(max_slots) * upm * (n_wg + 1) >= (int64_t(1) << 31) || nb > 4096)
            return dfl_fail(ctx, DFLASH_ERR_BAD_SHAPE, "gemm_fewrow: batch too large for 32-bit work indices");
        Q4KBatch bt = *batch;
        bt.by_wg = q4k_make_div(static_cast<uint32_t>(n_wg));
        const Q4KDiv by_upm = q4k_make_div(static_cast<uint32_t>(upm));
        // the first 64 list entries are loaded together with the slot count (0.5 us per down launch at light load)
        const int early_ids = env_int("DFLASH_EXP_EARLY_IDS", 1);
        const uint8_t *wb = static_cast<const uint8_t *>(w);
        const int no = static_cast<int>(n_out);
#define DFL_LAUNCH_EXPERTS(XT, YT, ROUTE)                                                                                   \
    do {                                                                                                                    \
        if (const int32_t rc_ = dfl_raise_lds_limit(ctx, reinterpret_cast<const void *>(gemm_q4k_experts_kernel<XT, YT, ROUTE>), kExpLdsBytes)) \
            return rc_;                                                                                                     \
        dfl_timed timer(ctx, st, DFL_T_GEMM);                                                                               \
        gemm_q4k_experts_kernel<XT, YT, ROUTE><<<n_wg, 64 * kSlabWaves, kExpLdsBytes, st>>>(wb, static_cast<const XT *>(x), reinterpret_cast<YT *>(y), \
                                                                                           no, nb, n_rows, bt, upm, by_upm, max_slots, early_ids); \
    } while (0)
        if (bt.route_logits) {
            if (x_type != DFLASH_TYPE_F32 || per_slot_x || bt.route_experts > 256 || bt.route_experts < 1 || bt.route_used < 1 ||
                bt.route_used > 64 || bt.route_used > bt.route_experts || max_slots + 0 > kExpRouteIds - 1)
                return dfl_fail(ctx, DFLASH_ERR_UNSUPPORTED, "gemm_q4k_batched: routing inside the launch needs f32 shared activations and at most 256 experts");
            if (bt.y_f16)
                DFL_LAUNCH_EXPERTS(float, _Float16, true);
            else
                DFL_LAUNCH_EXPERTS(float, float, true);
        } else if (x_type == DFLASH_TYPE_F32 && !bt.y_f16)
            DFL_LAUNCH_EXPERTS(float, float, false);
        else if (x_type == DFLASH_TYPE_F32)
            DFL_LAUNCH_EXPERTS(float, _Float16, false);
        else if (!bt.y_f16)
            DFL_LAUNCH_EXPERTS(_Float16, float, false);
        else
            DFL_LAUNCH_EXPERTS(_Float16, _Float16, false);
#undef DFL_LAUNCH_EXPERTS
        DFL_HIP_CHECK(ctx, hipGetLastError());
        return DFLASH_OK;
    }
    if (batch && (batch->y_f16 || batch->route_logits))
        return dfl_fail(ctx, DFLASH_ERR_UNSUPPORTED, "gemm_q4k_batched: f16 output and routing inside the launch need the tiled whole-K path");
    // A single matrix: 16-wave workgroups (256 weight rows per stage) when that still leaves every CU
    // a few stages of work, else 8-wave ones.  A batch is cut at tile-group boundaries only, so the
    // finer 8-wave groups balance it better (measured: the two expert launches of a 35B-A3B-shaped
    // layer take 50 us instead of 56 us).
    int waves = (!batch && static_cast<int64_t>((tiles + 15) / 16) * nb >= 2ll * ctx->n_cu) ? 16 : 8;
    waves = env_int("DFLASH_GEMM_WAVES", waves) == 16 ? 16 : 8;
    // A single matrix whose per-workgroup range is at most kSlabStages stages long takes the slab kernel (16-wave
    // groups): resident activation slab, wave-private weight rings, no per-stage barrier.
    bool slab = false;
    if (!batch && (tiled || env_int("DFLASH_Q4K_SLAB", 1)) && kSlabLdsBytes <= ctx->lds_bytes) {
        const int64_t total16 = static_cast<int64_t>((tiles + 15) / 16) * nb;
        const int64_t wgs = std::min<int64_t>(std::min<int64_t>(env_int("DFLASH_GEMM_WGS", ctx->n_cu), total16), ctx->n_partial_wgs / 2);
        // the longest range is ceil(total / wgs) stages
        slab = wgs >= 1 && (total16 + wgs - 1) / wgs <= kSlabStages;
        if (slab) waves = 16;
    }
    if (tiled && !batch) waves = 16;  // a single tiled matrix: whole 256-row tile groups (a batch may use their halves)
    const int gpm = (tiles + waves - 1) / waves;  // tile groups per matrix
    const int groups = gpm * max_slots * ((batch && batch->pair) ? 2 : 1);  // upper bound in batched mode (pair mode: virtual groups)
    int n_wg = batch ? env_int("DFLASH_MOE_WGS", ctx->batch_wgs > 0 ? ctx->batch_wgs : ctx->n_cu) : env_int("DFLASH_GEMM_WGS", ctx->n_cu);
    const int64_t total = static_cast<int64_t>(groups) * nb;
    const int max_wgs = ctx->n_partial_wgs * 8 / waves;
    if (n_wg > total) n_wg = static_cast<int>(total);
    if (n_wg > max_wgs) n_wg = max_wgs;
    if (n_wg < 1) n_wg = 1;
    if (total * (n_wg + 1) >= (int64_t(1) << 31) || row_bytes * 256 >= (size_t(1) << 32))
        return dfl_fail(ctx, DFLASH_ERR_BAD_SHAPE, "gemm_fewrow: problem too large for 32-bit work indices");
    float *partials = reinterpret_cast<float *>(ctx->partials);
    // a single matrix whose ranges are whole tile groups needs no reduction; a batch always may
    const bool split = (batch ? !batch->whole_groups : groups % n_wg != 0);
    const bool reduce = split;
    // a caller inside the library may ask for the SwiGLU of a fused gate | up product in place of the plain reduction
    float *swiglu_out = batch ? nullptr : ctx->swiglu_out;
    if (swiglu_out) ctx->swiglu_done = false;
    Q4KBatch bt = {};
    if (batch) bt = *batch;
    bt.groups_per_mat = gpm;
    bt.by_gpm = q4k_make_div(static_cast<uint32_t>(gpm));
    bt.by_nb = q4k_make_div(static_cast<uint32_t>(nb));
    bt.by_wg = q4k_make_div(static_cast<uint32_t>(n_wg));
    const uint8_t *wb = static_cast<const uint8_t *>(w);
    const int no = static_cast<int>(n_out);
#define DFL_LAUNCH_Q4K(WAVES, XT)                                                                                      \
    do {                                                                                                               \
        const size_t lds = static_cast<size_t>(Q4KGeom<WAVES>::kLdsPieces) * sizeof(half8_t);                      \
        if (lds > ctx->lds_bytes)                                                                                      \
            return dfl_fail(ctx, DFLASH_ERR_UNSUPPORTED, "gemm_fewrow: %zu bytes of LDS needed", lds);                 \
        if (const int32_t rc_ = dfl_raise_lds_limit(ctx, reinterpret_cast<const void *>(gemm_q4k_stream_kernel<WAVES, XT>), lds)) \
            return rc_;                                                                                                \
        {                                                                                                              \
            dfl_timed timer(ctx, st, DFL_T_GEMM);                                                                      \
            gemm_q4k_stream_kernel<WAVES, XT><<<n_wg, 64 * WAVES, lds, st>>>(wb, static_cast<const XT *>(x), y, partials, \
                                                                             no, nb, n_rows, groups, bt, tiled ? 1 : 0); \
        }                                                                                                              \
        if (reduce && swiglu_out) {                                                                                    \
            dfl_timed timer(ctx, st, DFL_T_REDUCE);                                                                    \
            q4k_reduce_swiglu_kernel<WAVES><<<no / 32, 256, 0, st>>>(partials, y, swiglu_out, no / 2, nb, n_rows, groups, n_wg); \
            ctx->swiglu_done = true;                                                                                   \
        } else if (reduce) {                                                                                           \
            dfl_timed timer(ctx, st, DFL_T_REDUCE);                                                                    \
            q4k_reduce_kernel<WAVES><<<groups * WAVES, 256, 0, st>>>(partials, y, no, nb, n_rows, groups, n_wg, bt);   \
        }                                                                                                              \
    } while (0)
    if (slab && tiled) {
        const void *fn = x_type == DFLASH_TYPE_F32 ? reinterpret_cast<const void *>(gemm_q4k_tiled_kernel<float>)
                                                   : reinterpret_cast<const void *>(gemm_q4k_tiled_kernel<_Float16>);
        if (const int32_t rc_ = dfl_raise_lds_limit(ctx, fn, kTiledLdsBytes)) return rc_;
        // weight stages issued ahead of the wait for the activations: two, or one when no range is longer than two
        // stages (measured on the 17.7 MB shape: 11.2 against 12.0 us per call; on the 50 MB shapes 19.1 against 18.7)
        const int k_pre = env_int("DFLASH_Q4K_PRE", (total + n_wg - 1) / n_wg <= 2 ? 1 : 2);
        // (while stamping is on, a dispatch carries start / stop stamps of its own: the kernel's duration as a trace reports it)
        {
            dfl_timed timer(ctx, st, DFL_T_GEMM);
            const dfl_stamp sp(ctx, DFL_T_KERNEL_Q4K_TILED);
            if (x_type == DFLASH_TYPE_F32)
                hipExtLaunchKernelGGL(gemm_q4k_tiled_kernel<float>, dim3(n_wg), dim3(64 * kSlabWaves), kTiledLdsBytes, st, sp.start, sp.stop, 0,
                                      wb, static_cast<const float *>(x), y, partials, no, nb, n_rows, groups, bt, k_pre);
            else
                hipExtLaunchKernelGGL(gemm_q4k_tiled_kernel<_Float16>, dim3(n_wg), dim3(64 * kSlabWaves), kTiledLdsBytes, st, sp.start, sp.stop, 0,
                                      wb, static_cast<const _Float16 *>(x), y, partials, no, nb, n_rows, groups, bt, k_pre);
        }
        if (reduce && swiglu_out) {
            dfl_timed timer(ctx, st, DFL_T_REDUCE);
            q4k_reduce_swiglu_kernel<16><<<no / 32, 256, 0, st>>>(partials, y, swiglu_out, no / 2, nb, n_rows, groups, n_wg);
            ctx->swiglu_done = true;
        } else if (reduce) {
            dfl_timed timer(ctx, st, DFL_T_REDUCE);
            const dfl_stamp sp(ctx, DFL_T_KERNEL_Q4K_REDUCE);
            hipExtLaunchKernelGGL(q4k_reduce_kernel<16>, dim3(groups * 16), dim3(256), 0, st, sp.start, sp.stop, 0, partials, y, no, nb, n_rows,
                                  groups, n_wg, bt);
        }
    } else if (slab) {
        const void *fn = x_type == DFLASH_TYPE_F32 ? reinterpret_cast<const void *>(gemm_q4k_slab_kernel<float>)
                                                   : reinterpret_cast<const void *>(gemm_q4k_slab_kernel<_Float16>);
        if (const int32_t rc_ = dfl_raise_lds_limit(ctx, fn, kSlabLdsBytes)) return rc_;
        {
            dfl_timed timer(ctx, st, DFL_T_GEMM);
            const dfl_stamp sp(ctx, DFL_T_KERNEL_Q4K_TILED);  // (the same slot as the tiled kernel: one of the two runs)
            if (x_type == DFLASH_TYPE_F32)
                hipExtLaunchKernelGGL(gemm_q4k_slab_kernel<float>, dim3(n_wg), dim3(64 * kSlabWaves), kSlabLdsBytes, st, sp.start, sp.stop, 0, wb,
                                      static_cast<const float *>(x), y, partials, no, nb, n_rows, groups, bt);
            else
                hipExtLaunchKernelGGL(gemm_q4k_slab_kernel<_Float16>, dim3(n_wg), dim3(64 * kSlabWaves), kSlabLdsBytes, st, sp.start, sp.stop, 0, wb,
                                      static_cast<const _Float16 *>(x), y, partials, no, nb, n_rows, groups, bt);
        }
        if (reduce && swiglu_out) {
            dfl_timed timer(ctx, st, DFL_T_REDUCE);
            q4k_reduce_swiglu_kernel<16><<<no / 32, 256, 0, st>>>(partials, y, swiglu_out, no / 2, nb, n_rows, groups, n_wg);
            ctx->swiglu_done = true;
        } else if (reduce) {
            dfl_timed timer(ctx, st, DFL_T_REDUCE);
            q4k_reduce_kernel<16><<<groups * 16, 256, 0, st>>>(partials, y, no, nb, n_rows, groups, n_wg, bt);
        }
    } else if (waves == 16 && x_type == DFLASH_TYPE_F32)
        DFL_LAUNCH_Q4K(16, float);
    else if (waves == 16)
        DFL_LAUNCH_Q4K(16, _Float16);
    else if (x_type == DFLASH_TYPE_F32)
        DFL_LAUNCH_Q4K(8, float);
    else
        DFL_LAUNCH_Q4K(8, _Float16);
#undef DFL_LAUNCH_Q4K
    DFL_HIP_CHECK(ctx, hipGetLastError());
    return DFLASH_OK;
}

}  // namespace

namespace {

// The streaming Q6_K kernel (and its split-K reduction) on one matrix.  (Measured and not kept: for the few-MB
// attention projections, workgroups of two waves that take the whole K of their 32 rows, as many as there are row
// groups (160 for a 5120-row q/k/v product, 64 for a 2048-row output projection): no partial tiles and no reduce
// launch, every test green, but a 40-layer verify took 4.88 instead of 4.71 ms: 8 or 16 dependent stages of one
// small workgroup are a longer chain than one or two stages on every CU plus the reduce launch.)
int32_t launch_q6k_stream(dflash_ctx *ctx, const void *w, const void *x, int32_t x_type, float *y, int64_t n_in,
                          int64_t n_out, int32_t n_rows, hipStream_t st) {
    const int nb = static_cast<int>(n_in / DFL_QK_K);
    const size_t row_bytes = static_cast<size_t>(nb) * DFL_Q6_K_BYTES;
    const int tiles = static_cast<int>((n_out + 15) / 16);
    if (reinterpret_cast<uintptr_t>(x) % (x_type == DFLASH_TYPE_F32 ? 16 : 8))
        return dfl_fail(ctx, DFLASH_ERR_ALIGNMENT, "gemm_fewrow: activations must be 16-byte (f32) / 8-byte (f16) aligned");
    int waves = (static_cast<int64_t>((tiles + 15) / 16) * nb >= 2ll * ctx->n_cu) ? 16 : 8;
    waves = env_int("DFLASH_GEMM_WAVES", waves) == 16 ? 16 : 8;
    const int groups = (tiles + waves - 1) / waves;
    int n_wg = env_int("DFLASH_GEMM_WGS", ctx->n_cu);
    const int64_t total = static_cast<int64_t>(groups) * nb;
    const int max_wgs = ctx->n_partial_wgs * 8 / waves;
    if (n_wg > total) n_wg = static_cast<int>(total);
    if (n_wg > max_wgs) n_wg = max_wgs;
    if (n_wg < 1) n_wg = 1;
    if (total * (n_wg + 1) >= (int64_t(1) << 31) || row_bytes * 256 >= (size_t(1) << 32))
        return dfl_fail(ctx, DFLASH_ERR_BAD_SHAPE, "gemm_fewrow: problem too large for 32-bit work indices");
    float *partials = reinterpret_cast<float *>(ctx->partials);
    const bool split = groups % n_wg != 0;
    Q4KBatch bt = {};
    bt.groups_per_mat = groups;
    bt.by_gpm = q4k_make_div(static_cast<uint32_t>(groups));
    bt.by_nb = q4k_make_div(static_cast<uint32_t>(nb));
    bt.by_wg = q4k_make_div(static_cast<uint32_t>(n_wg));
    const uint8_t *wb = static_cast<const uint8_t *>(w);
    const int no = static_cast<int>(n_out);
#define DFL_LAUNCH_Q6K(WAVES, XT)                                                                                      \
    do {                                                                                                               \
        const size_t lds = Q6KGeom<WAVES>::kLdsBytes;                                                                  \
        if (lds > ctx->lds_bytes)                                                                                      \
            return dfl_fail(ctx, DFLASH_ERR_UNSUPPORTED, "gemm_fewrow: %zu bytes of LDS needed", lds);                 \
        if (const int32_t rc_ = dfl_raise_lds_limit(ctx, reinterpret_cast<const void *>(gemm_q6k_stream_kernel<WAVES, XT>), lds)) \
            return rc_;                                                                                                \
        {                                                                                                              \
            dfl_timed timer(ctx, st, DFL_T_GEMM);                                                                      \
            gemm_q6k_stream_kernel<WAVES, XT><<<n_wg, 64 * WAVES, lds, st>>>(wb, static_cast<const XT *>(x), y, partials, \
                                                                             no, nb, n_rows, groups, bt);              \
        }                                                                                                              \
        if (split) {                                                                                                   \
            dfl_timed timer(ctx, st, DFL_T_REDUCE);                                                                    \
            q4k_reduce_kernel<WAVES><<<groups * WAVES, 256, 0, st>>>(partials, y, no, nb, n_rows, groups, n_wg, bt);   \
        }                                                                                                              \
    } while (0)
    if (waves == 16 && x_type == DFLASH_TYPE_F32)
        DFL_LAUNCH_Q6K(16, float);
    else if (waves == 16)
        DFL_LAUNCH_Q6K(16, _Float16);
    else if (x_type == DFLASH_TYPE_F32)
        DFL_LAUNCH_Q6K(8, float);
    else
        DFL_LAUNCH_Q6K(8, _Float16);
#undef DFL_LAUNCH_Q6K
    return DFLASH_OK;
}

}  // namespace

bool dfl_router_norm_fits(const dflash_ctx *ctx, int32_t router_type, const void *router_w, int64_t hidden, int32_t n_expert,
                          int32_t n_rows) {
    static const bool on = env_int("DFLASH_MOE_FUSED_NORM", 1) != 0;  // read once per process
    // (up to 128 tiles the separate router product runs 16 waves per workgroup as well: same bits)
    return on && router_type == DFLASH_TYPE_Q8_0 && hidden >= 256 && hidden % 256 == 0 && hidden <= 32 * kQ8ChunkSteps &&
           n_expert >= 1 && (n_expert + 15) / 16 <= 128 && n_rows >= 1 && n_rows <= 4096 &&
           reinterpret_cast<uintptr_t>(router_w) % 16 == 0 && ctx->lds_bytes >= 48 * 1024;
}

int32_t dfl_router_norm(dflash_ctx *ctx, const void *router_w, const float *x, const float *add, const float *norm_w,
                        const float *gate_w, float eps, float *cur, float *gate_out, float *logits, int64_t hidden,
                        int32_t n_expert, int32_t n_rows, hipStream_t st) {
    if (!router_w || !x || !add || !norm_w || !gate_w || !cur || !gate_out || !logits)
        return dfl_fail(ctx, DFLASH_ERR_INVALID_INPUT, "router_norm: null argument");
    if (!dfl_router_norm_fits(ctx, DFLASH_TYPE_Q8_0, router_w, hidden, n_expert, n_rows))
        return dfl_fail(ctx, DFLASH_ERR_UNSUPPORTED, "router_norm: hidden %lld / %d experts / %d rows", static_cast<long long>(hidden),
                        n_expert, n_rows);
    for (const void *p : {static_cast<const void *>(x), static_cast<const void *>(add), static_cast<const void *>(norm_w),
                          static_cast<const void *>(gate_w), static_cast<const void *>(cur)})
        if (reinterpret_cast<uintptr_t>(p) % 16)
            return dfl_fail(ctx, DFLASH_ERR_ALIGNMENT, "router_norm: rows and weights must be 16-byte aligned");
    const int n_steps = static_cast<int>(hidden / DFL_QK8_0);
    const int tiles = (n_expert + 15) / 16;
    dfl_timed timer(ctx, st, DFL_T_GEMM);
    q8_0_norm_router_kernel<<<dim3(tiles, n_rows), 64 * kMaxSplit, 0, st>>>(static_cast<const uint8_t *>(router_w), x, add, norm_w, gate_w, eps, cur,
                                                                 gate_out, logits, n_expert, n_steps,
                                                                 static_cast<size_t>(n_steps) * DFL_Q8_0_BYTES);
    DFL_HIP_CHECK(ctx, hipGetLastError());
    return DFLASH_OK;
}

int32_t dfl_router_rows(dflash_ctx *ctx, const void *router_w, const float *cur, float *logits, int64_t hidden, int32_t n_expert,
                        int32_t n_rows, hipStream_t st) {
    if (!router_w || !cur || !logits || n_rows < 1 || !dfl_router_norm_fits(ctx, DFLASH_TYPE_Q8_0, router_w, hidden, n_expert, 16) ||
        reinterpret_cast<uintptr_t>(cur) % 16)
        return dfl_fail(ctx, DFLASH_ERR_UNSUPPORTED, "router_rows: hidden %lld / %d experts / %d rows", static_cast<long long>(hidden), n_expert,
                        n_rows);
    if (const int32_t rc_ = dfl_raise_lds_limit(ctx, reinterpret_cast<const void *>(gemm_q8_0_staged_kernel<float>), kQ8StagedLds)) return rc_;
    const int n_steps = static_cast<int>(hidden / DFL_QK8_0);
    dfl_timed timer(ctx, st, DFL_T_GEMM);
    // sixteen waves split the 64 steps of a row, as the few-row product of a router does for one block
    gemm_q8_0_staged_kernel<float><<<dim3((n_expert + 15) / 16, (n_rows + 15) / 16), 64 * kMaxSplit, kQ8StagedLds, st>>>(
        static_cast<const uint8_t *>(router_w), cur, logits, n_expert, n_steps, static_cast<size_t>(n_steps) * DFL_Q8_0_BYTES, n_rows, kMaxSplit);
    DFL_HIP_CHECK(ctx, hipGetLastError());
    return DFLASH_OK;
}

bool dfl_q4k_batched_can_route(const dflash_ctx *ctx, int32_t tiled, int64_t n_out, int32_t n_expert, int32_t n_used) {
    return dfl_q4k_batched_f16_out(ctx, tiled, 1, n_out) && n_expert >= 1 && n_expert <= 256 && n_used >= 1 && n_used <= 64 &&
           n_used <= n_expert && env_int("DFLASH_MOE_FUSED_ROUTE", 1);
}

bool dfl_q4k_batched_f16_out(const dflash_ctx *ctx, int32_t tiled, int32_t whole_groups, int64_t n_out) {
    return tiled && whole_groups && n_out % 16 == 0 && kExpLdsBytes <= ctx->lds_bytes && env_int("DFLASH_MOE_EXPERTS_KERNEL", 1);
}

int32_t dfl_gemm_q4k_batched(dflash_ctx *ctx, const void *w_stack, size_t w_stride_bytes, const void *extra_w,
                             const int32_t *ids, const int32_t *n_slots, int max_slots, const void *x, int32_t x_type,
                             size_t x_stride,
                             void *y, int32_t y_type, size_t y_stride, int64_t n_in, int64_t n_out, int32_t n_rows,
                             int32_t whole_groups, const void *w_stack_up, const void *extra_w_up, int32_t tiled,
                             dflash_stream_t stream, const dfl_route_args *route) {
    if (y_type != DFLASH_TYPE_F32 && y_type != DFLASH_TYPE_F16)
        return dfl_fail(ctx, DFLASH_ERR_UNSUPPORTED, "gemm_q4k_batched: output type %d", y_type);
    if (n_in % DFL_QK_K || n_in <= 0 || n_out <= 0 || n_rows < 1 || n_rows > 16 || max_slots < 1)
        return dfl_fail(ctx, DFLASH_ERR_BAD_SHAPE, "gemm_q4k_batched: bad shape");
    if (reinterpret_cast<uintptr_t>(w_stack) % 16 || reinterpret_cast<uintptr_t>(extra_w) % 16 || w_stride_bytes % 16 || (x_stride * (x_type == DFLASH_TYPE_F32 ? 4 : 2)) % 16 ||
        reinterpret_cast<uintptr_t>(w_stack_up) % 16 || reinterpret_cast<uintptr_t>(extra_w_up) % 16)
        return dfl_fail(ctx, DFLASH_ERR_ALIGNMENT, "gemm_q4k_batched: operand alignment");
    if (w_stack_up && (!whole_groups || (extra_w != nullptr) != (extra_w_up != nullptr)))
        return dfl_fail(ctx, DFLASH_ERR_INVALID_INPUT, "gemm_q4k_batched: the gate/up pair needs whole groups and both or neither extra matrix");
    Q4KBatch bt = {};
    bt.pair = w_stack_up ? 1 : 0;
    bt.w2 = static_cast<const uint8_t *>(w_stack_up);
    bt.extra_w2 = static_cast<const uint8_t *>(extra_w_up);
    bt.ids = ids;
    bt.extra_w = static_cast<const uint8_t *>(extra_w);
    bt.n_slots = n_slots;
    bt.w_stride = w_stride_bytes;
    bt.x_stride = x_stride;
    bt.y_stride = y_stride;
    bt.whole_groups = whole_groups;
    bt.y_f16 = y_type == DFLASH_TYPE_F16;
    if (route) {
        if (!route->logits || !route->sel_e || !route->sel_w || !route->slot_of || x_stride != 0)
            return dfl_fail(ctx, DFLASH_ERR_INVALID_INPUT, "gemm_q4k_batched: routing inside the launch needs its buffers and shared activations");
        bt.route_logits = route->logits;
        bt.route_experts = route->n_expert;
        bt.route_used = route->n_used;
        bt.route_shared = route->with_shared;
        bt.route_sel_e = route->sel_e;
        bt.route_sel_w = route->sel_w;
        bt.route_slot_of = route->slot_of;
    }
    return launch_q4k(ctx, w_stack, x, x_type, static_cast<float *>(y), n_in, n_out, n_rows, static_cast<hipStream_t>(stream), &bt,
                      max_slots, tiled != 0);
}

namespace {
int32_t gemm_fewrow_impl(dflash_ctx *ctx, int32_t w_type, const void *w, const void *x, int32_t x_type, float *y, int64_t n_in,
                         int64_t n_out, int32_t n_rows, dflash_stream_t stream);
}

extern "C" size_t dflash_q4k_tiled_bytes(int64_t n_in, int64_t n_out) {
    if (n_in <= 0 || n_out <= 0 || n_in % DFL_QK_K) return 0;
    const size_t groups = (static_cast<size_t>(n_out) + 255) / 256;
    return groups * static_cast<size_t>(n_in / DFL_QK_K) * kTiledStageBytes;
}

extern "C" int32_t dflash_repack_q4k_tiled(dflash_ctx *ctx, const void *w, void *w_tiled, int64_t n_in, int64_t n_out,
                                           dflash_stream_t stream) {
    if (!ctx) return DFLASH_ERR_INVALID_INPUT;
    if (!w || !w_tiled) return dfl_fail(ctx, DFLASH_ERR_INVALID_INPUT, "repack_q4k_tiled: null pointer");
    if (n_in <= 0 || n_out <= 0 || n_in % DFL_QK_K || n_in > 0x7fffffffll || n_out > 0x7fffffffll)
        return dfl_fail(ctx, DFLASH_ERR_BAD_SHAPE, "repack_q4k_tiled: n_in %lld / n_out %lld", static_cast<long long>(n_in),
                        static_cast<long long>(n_out));
    if (reinterpret_cast<uintptr_t>(w) % 16 || reinterpret_cast<uintptr_t>(w_tiled) % 128)
        return dfl_fail(ctx, DFLASH_ERR_ALIGNMENT, "repack_q4k_tiled: source must be 16-byte, destination 128-byte aligned");
    const size_t out_bytes = dflash_q4k_tiled_bytes(n_in, n_out);
    const size_t in_bytes = static_cast<size_t>(n_out) * (n_in / DFL_QK_K) * DFL_Q4_K_BYTES;
    if (dfl_ranges_overlap(w_tiled, out_bytes, w, in_bytes)) return dfl_fail(ctx, DFLASH_ERR_ALIAS, "repack_q4k_tiled: buffers overlap");
    // a tiled tensor goes to the fast kernels unconditionally: it must be one they can take
    if (const int32_t rc = dflash_check_scale_range(ctx, DFLASH_TYPE_Q4_K, w, in_bytes / DFL_Q4_K_BYTES, nullptr, stream)) return rc;
    const int64_t n_pieces = static_cast<int64_t>(out_bytes / 16);
    const int64_t blocks = (n_pieces + 255) / 256;
    if (blocks > 0x7fffffffll) return dfl_fail(ctx, DFLASH_ERR_BAD_SHAPE, "repack_q4k_tiled: matrix too large");
    q4k_repack_tiled_kernel<<<static_cast<unsigned>(blocks), 256, 0, static_cast<hipStream_t>(stream)>>>(
        static_cast<const uint8_t *>(w), static_cast<uint8_t *>(w_tiled), static_cast<int>(n_out), static_cast<int>(n_in / DFL_QK_K), n_pieces);
    DFL_HIP_CHECK(ctx, hipGetLastError());
    return DFLASH_OK;
}

extern "C" int32_t dflash_gemm_fewrow(dflash_ctx *ctx, int32_t w_type, const void *w, const void *x, int32_t x_type,
                                      float *y, int64_t n_in, int64_t n_out, int32_t n_rows, dflash_stream_t stream) {
    if (!ctx) return DFLASH_ERR_INVALID_INPUT;
    return gemm_fewrow_impl(ctx, w_type, w, x, x_type, y, n_in, n_out, n_rows, stream);
}

int32_t dfl_gemm_fewrow_checked(dflash_ctx *ctx, int32_t w_type, const void *w, const void *x, int32_t x_type, float *y,
                                int64_t n_in, int64_t n_out, int32_t n_rows, dflash_stream_t stream) {
    return gemm_fewrow_impl(ctx, w_type | DFLASH_TYPE_RANGE_CHECKED, w, x, x_type, y, n_in, n_out, n_rows, stream);
}

namespace {

int32_t gemm_fewrow_impl(dflash_ctx *ctx, int32_t w_type, const void *w, const void *x, int32_t x_type, float *y, int64_t n_in,
                         int64_t n_out, int32_t n_rows, dflash_stream_t stream) {
    if (!w || !x || !y) return dfl_fail(ctx, DFLASH_ERR_INVALID_INPUT, "gemm_fewrow: null pointer");
    if (n_rows < 1 || n_rows > 16)
        return dfl_fail(ctx, DFLASH_ERR_BAD_SHAPE, "gemm_fewrow: n_rows %d outside 1..16", n_rows);
    if (n_in <= 0 || n_out <= 0 || n_in > 0x7fffffffll || n_out > 0x7fffffffll)
        return dfl_fail(ctx, DFLASH_ERR_BAD_SHAPE, "gemm_fewrow: n_in %lld / n_out %lld out of range",
                        static_cast<long long>(n_in), static_cast<long long>(n_out));
    if (x_type != DFLASH_TYPE_F32 && x_type != DFLASH_TYPE_F16)
        return dfl_fail(ctx, DFLASH_ERR_UNSUPPORTED, "gemm_fewrow: activations must be f32 or f16");
    // the fast Q4_K / Q6_K kernels scale in f16: only for a tensor tagged as range-checked (the tiled order is, by construction)
    const bool checked = (w_type & DFLASH_TYPE_RANGE_CHECKED) != 0 || w_type == DFLASH_TYPE_Q4_K_TILED;
    w_type &= ~DFLASH_TYPE_RANGE_CHECKED;
    const bool plain = w_type == DFLASH_TYPE_F32 || w_type == DFLASH_TYPE_F16;
    const bool tiled = w_type == DFLASH_TYPE_Q4_K_TILED;
    if (tiled) w_type = DFLASH_TYPE_Q4_K;
    if (w_type == DFLASH_TYPE_Q6_K_TILED)
        return dfl_fail(ctx, DFLASH_ERR_UNSUPPORTED,
                        "gemm_fewrow: a tiled Q6_K tensor is read by dflash_gemm_fewrow_xf (and the model-level calls) only");
    if (w_type != DFLASH_TYPE_Q4_K && w_type != DFLASH_TYPE_Q6_K && w_type != DFLASH_TYPE_Q8_0 && !plain)
        return dfl_fail(ctx, DFLASH_ERR_UNSUPPORTED, "gemm_fewrow: weight type %d has no few-row kernel", w_type);
    const int64_t blk = (w_type == DFLASH_TYPE_Q8_0 || plain) ? DFL_QK8_0 : DFL_QK_K;
    if (n_in % blk)
        return dfl_fail(ctx, DFLASH_ERR_BAD_SHAPE, "gemm_fewrow: n_in %lld is not a multiple of %lld",
                        static_cast<long long>(n_in), static_cast<long long>(blk));
    const size_t row_bytes = dflash_row_bytes(w_type, static_cast<size_t>(n_in));
    const size_t w_bytes = tiled ? dflash_q4k_tiled_bytes(n_in, n_out) : row_bytes * static_cast<size_t>(n_out);
    const size_t x_bytes = static_cast<size_t>(n_rows) * n_in * (x_type == DFLASH_TYPE_F32 ? 4 : 2);
    const size_t y_bytes = static_cast<size_t>(n_rows) * n_out * 4;
    if (reinterpret_cast<uintptr_t>(w) % ((w_type == DFLASH_TYPE_Q4_K || plain) ? 16 : 2) ||
        reinterpret_cast<uintptr_t>(x) % 4 || reinterpret_cast<uintptr_t>(y) % 4)
        return dfl_fail(ctx, DFLASH_ERR_ALIGNMENT, "gemm_fewrow: operand alignment");
    if (dfl_ranges_overlap(y, y_bytes, x, x_bytes) || dfl_ranges_overlap(y, y_bytes, w, w_bytes))
        return dfl_fail(ctx, DFLASH_ERR_ALIAS, "gemm_fewrow: y aliases an input");

    hipStream_t st = static_cast<hipStream_t>(stream);
    const int64_t n_steps = n_in / 32;
    const int tiles = static_cast<int>((n_out + 15) / 16);
    const int target_waves = 8 * ctx->n_cu;

    if ((w_type == DFLASH_TYPE_Q4_K || w_type == DFLASH_TYPE_Q6_K) && !checked) {
        // any block the format can hold: ggml's f32 dequantisation and f32 sums (gemm_safe_kernel)
        dfl_timed timer(ctx, st, DFL_T_GEMM);
        const unsigned grid = static_cast<unsigned>((n_out + 3) / 4);
        if (x_type == DFLASH_TYPE_F32)
            gemm_safe_kernel<float><<<grid, 256, 0, st>>>(w_type, static_cast<const uint8_t *>(w), row_bytes, static_cast<const float *>(x), y,
                                                       static_cast<int>(n_in), static_cast<int>(n_out), n_rows);
        else
            gemm_safe_kernel<_Float16><<<grid, 256, 0, st>>>(w_type, static_cast<const uint8_t *>(w), row_bytes,
                                                          static_cast<const _Float16 *>(x), y, static_cast<int>(n_in),
                                                          static_cast<int>(n_out), n_rows);
    } else if (w_type == DFLASH_TYPE_Q4_K) {
        if (tiled && reinterpret_cast<uintptr_t>(w) % 128)
            return dfl_fail(ctx, DFLASH_ERR_ALIGNMENT, "gemm_fewrow: tiled Q4_K weights must be 128-byte aligned");
        return launch_q4k(ctx, w, x, x_type, y, n_in, n_out, n_rows, st, nullptr, 1, tiled);
    } else if (w_type == DFLASH_TYPE_Q6_K && env_int("DFLASH_Q6K_STREAM", 1)) {
        const int32_t rc = launch_q6k_stream(ctx, w, x, x_type, y, n_in, n_out, n_rows, st);
        if (rc) return rc;
    } else if (w_type == DFLASH_TYPE_Q6_K) {
        Q6KSet set = {};
        set.n_mats = 1;
        set.w[0] = static_cast<const uint8_t *>(w);
        set.y[0] = y;
        set.n_out[0] = static_cast<int>(n_out);
        const int32_t rc = launch_q6k(ctx, set, x, x_type, n_in, n_rows, st);
        if (rc) return rc;
    } else {
        if (reinterpret_cast<uintptr_t>(x) % (x_type == DFLASH_TYPE_F32 ? 16 : 8))
            return dfl_fail(ctx, DFLASH_ERR_ALIGNMENT, "gemm_fewrow: activations must be 16-byte (f32) / 8-byte (f16) aligned");
        int split = (target_waves + tiles - 1) / tiles;
        split = env_int("DFLASH_GEMM_NSPLIT", split);
        if (split > n_steps) split = static_cast<int>(n_steps);
        if (split > kMaxSplit) split = kMaxSplit;
        if (split < 1) split = 1;
        size_t lds = static_cast<size_t>(split) * 256 * sizeof(float);
        const uint8_t *wb = static_cast<const uint8_t *>(w);
        dfl_timed timer(ctx, st, DFL_T_GEMM);
#define DFL_LAUNCH_GENERIC(TYPE)                                                                                         \
    do {                                                                                                                 \
        if (x_type == DFLASH_TYPE_F32)                                                                                   \
            gemm_generic_kernel<TYPE, float><<<tiles, 64 * split, lds, st>>>(                                            \
                wb, static_cast<const float *>(x), y, static_cast<int>(n_out), n_steps, row_bytes, n_rows, split);       \
        else                                                                                                             \
            gemm_generic_kernel<TYPE, _Float16><<<tiles, 64 * split, lds, st>>>(                                         \
                wb, static_cast<const _Float16 *>(x), y, static_cast<int>(n_out), n_steps, row_bytes, n_rows, split);    \
    } while (0)
        if (w_type == DFLASH_TYPE_F32)
            DFL_LAUNCH_GENERIC(DFLASH_TYPE_F32);
        else if (w_type == DFLASH_TYPE_F16)
            DFL_LAUNCH_GENERIC(DFLASH_TYPE_F16);
        else if (n_in % 256 == 0 && reinterpret_cast<uintptr_t>(w) % 16 == 0 && reinterpret_cast<uintptr_t>(x) % 16 == 0 &&
            env_int("DFLASH_Q8_STAGED", 1)) {
            if (const int32_t rc_ = dfl_raise_lds_limit(ctx, x_type == DFLASH_TYPE_F32
                                                                 ? reinterpret_cast<const void *>(gemm_q8_0_staged_kernel<float>)
                                                                 : reinterpret_cast<const void *>(gemm_q8_0_staged_kernel<_Float16>),
                                                        kQ8StagedLds))
                return rc_;
            // the waves of a workgroup split a 64-step chunk
            if (split > kQ8ChunkSteps) split = kQ8ChunkSteps;
            if (x_type == DFLASH_TYPE_F32)
                gemm_q8_0_staged_kernel<float><<<tiles, 64 * split, kQ8StagedLds, st>>>(
                    wb, static_cast<const float *>(x), y, static_cast<int>(n_out), static_cast<int>(n_steps), row_bytes, n_rows, split);
            else
                gemm_q8_0_staged_kernel<_Float16><<<tiles, 64 * split, kQ8StagedLds, st>>>(
                    wb, static_cast<const _Float16 *>(x), y, static_cast<int>(n_out), static_cast<int>(n_steps), row_bytes, n_rows,
                    split);
        } else
            DFL_LAUNCH_GENERIC(DFLASH_TYPE_Q8_0);
#undef DFL_LAUNCH_GENERIC
    }
    DFL_HIP_CHECK(ctx, hipGetLastError());
    return DFLASH_OK;
}

}  // namespace

// ----------------------------------------------------------------------------
// The same product for callers that may not allocate
// ----------------------------------------------------------------------------
//
// The streaming kernels keep split-K partial tiles in device memory between the GEMM kernel and its
// reduction.  dflash_gemm_fewrow takes that buffer from the context, which allocated it.  The entry
// below takes it from a fixed array in the library's device image instead and needs no context, so
// nothing on its path allocates: no hipMalloc / hipFree, no workspace, no stream or event creation.
// The array is sized for kNoAllocEntries partial-tile sets (one per 8-wave workgroup, two per 16-wave
// workgroup): launches are clamped to that many workgroups, which covers every CU of an MI355X.
// Every call on a GPU uses that GPU's one copy of the array: calls that overlap in time on the same
// GPU (two streams, two threads) race on it; calls on one stream are ordered and safe.  Nothing in
// the array has to start at zero: the reduction reads only the tiles the same launch wrote.
namespace {
constexpr int kNoAllocEntries = 512;
constexpr size_t kNoAllocScratchBytes = static_cast<size_t>(kNoAllocEntries) * 2 * 8 * 256 * sizeof(float);  // 8 MiB
constexpr int kNoAllocMaxDevices = 64;
}  // namespace

static __device__ __align__(256) unsigned char scratch[kNoAllocScratchBytes];

namespace {

struct NoAllocDevice {
    void *ptr = nullptr;  // this device's copy of `scratch` (hipGetSymbolAddress, once per device)
    int n_cu = 0;
    size_t lds_bytes = 0;
    // the context fields that remember per-device kernel attributes, carried from call to call
    const void *lds_attr_fn[96] = {nullptr};
    size_t lds_attr_bytes[96] = {0};
    int n_lds_attr = 0;
};
NoAllocDevice g_noalloc[kNoAllocMaxDevices];
std::mutex g_noalloc_mutex;  // guards the table above (the enqueue itself is short)
thread_local char g_noalloc_err[512] = "";

int32_t noalloc_fail(int32_t status, const char *msg) {
    snprintf(g_noalloc_err, sizeof(g_noalloc_err), "%s", msg);
    return status;
}

}  // namespace

extern "C" const char *dflash_gemm_fewrow_noalloc_error(void) { return g_noalloc_err; }

extern "C" int32_t dflash_gemm_fewrow_noalloc(int32_t w_type, const void *w, const void *x, int32_t x_type, float *y,
                                              int64_t n_in, int64_t n_out, int32_t n_rows, dflash_stream_t stream) {
    g_noalloc_err[0] = 0;
    if (n_in > DFLASH_NOALLOC_MAX_N_IN || n_out > DFLASH_NOALLOC_MAX_N_OUT)
        return noalloc_fail(DFLASH_ERR_BAD_SHAPE, "gemm_fewrow_noalloc: n_in / n_out beyond DFLASH_NOALLOC_MAX_N_IN / _N_OUT");
    int device = -1;
    if (hipGetDevice(&device) != hipSuccess || device < 0) return noalloc_fail(DFLASH_ERR_HIP, "gemm_fewrow_noalloc: no current device");
    if (device >= kNoAllocMaxDevices) return noalloc_fail(DFLASH_ERR_UNSUPPORTED, "gemm_fewrow_noalloc: device index beyond 63");
    std::lock_guard<std::mutex> lock(g_noalloc_mutex);
    NoAllocDevice &dev = g_noalloc[device];
    if (!dev.ptr) {
        // first call on this device, which is the current one: its own address of the array, and its shape
        void *ptr = nullptr;
        if (hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)) != hipSuccess || !ptr)
            return noalloc_fail(DFLASH_ERR_HIP, "gemm_fewrow_noalloc: hipGetSymbolAddress(scratch) failed");
        int n_cu = 0, lds = 0;
        if (hipDeviceGetAttribute(&n_cu, hipDeviceAttributeMultiprocessorCount, device) != hipSuccess ||
            hipDeviceGetAttribute(&lds, hipDeviceAttributeMaxSharedMemoryPerBlock, device) != hipSuccess || n_cu < 1)
            return noalloc_fail(DFLASH_ERR_HIP, "gemm_fewrow_noalloc: device attributes unavailable");
        dev.n_cu = n_cu;
        dev.lds_bytes = static_cast<size_t>(lds);
        dev.ptr = ptr;
    }
    // a context on the stack that owns nothing: the launch code reads its shape fields and the partial-tile buffer
    dflash_ctx local;
    local.device = device;
    local.n_cu = dev.n_cu;
    local.lds_bytes = dev.lds_bytes;
    local.partials = dev.ptr;
    local.n_partial_wgs = kNoAllocEntries;
    memcpy(local.lds_attr_fn, dev.lds_attr_fn, sizeof(dev.lds_attr_fn));
    memcpy(local.lds_attr_bytes, dev.lds_attr_bytes, sizeof(dev.lds_attr_bytes));
    local.n_lds_attr = dev.n_lds_attr;
    int32_t rc;
    if (!w || !x || !y)
        rc = dfl_fail(&local, DFLASH_ERR_INVALID_INPUT, "gemm_fewrow_noalloc: null pointer");
    else
        rc = gemm_fewrow_impl(&local, w_type, w, x, x_type, y, n_in, n_out, n_rows, stream);
    memcpy(dev.lds_attr_fn, local.lds_attr_fn, sizeof(dev.lds_attr_fn));
    memcpy(dev.lds_attr_bytes, local.lds_attr_bytes, sizeof(dev.lds_attr_bytes));
    dev.n_lds_attr = local.n_lds_attr;
    if (rc) snprintf(g_noalloc_err, sizeof(g_noalloc_err), "%s", local.err);
    return rc;
}
