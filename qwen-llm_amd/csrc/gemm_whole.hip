// Whole-K few-row GEMM for the small matrices of a verify or draft layer (a few MB each):
//   Y[n_rows][n_out] = X[n_rows][n_in] . W^T,  X handed over in MFMA fragment order (common.h, "XF").
// Same contraction as encode_mat_mat_dispatch_dflash_verify (metal_forward/dispatch.rs:365-378, kernel
// kernels/mat_mat_fewrow_gen.metal:374-474); used inside the layer loops where the kernel that produces X can
// write it in fragment order.
//
// Why a second kernel family.  The streaming kernels (gemm_fewrow.hip) give every CU a contiguous run of
// (tile group x super-block) stages; where a run cuts a tile group the K sum is split over workgroups and a second
// launch adds the partial tiles.  For a 50 MB matrix that is the right shape.  For the 6-9 MB projections of a
// 2048-wide model it is two dependent launches of 7-10 us + 4 us in which every wave sees one or two stages: the
// time is launch latency, the trip for the first bytes, and a reduction through memory.  Here every (tile, stage)
// of the matrix is one wave-slot of ONE round of the chip:
//   * a workgroup owns `tl` output units over the whole K; wave = (tile lane, K slice), a slice is one or two
//     super-blocks; every load of a wave (weights straight into registers, the stage's eight activation fragments
//     with eight coalesced 16-byte loads from the XF buffer, which sits in L2) is issued before anything is waited for;
//   * the slices' partial tiles are added in LDS in slice order (deterministic), by the wave of slice 0, which writes Y.
// No partial tiles in memory, no second launch, no loop.  A (row, column) result depends on nothing but its own
// activation row and weight row, so a 16-row block and a single row give the same bits.
//
// Arithmetic: that of the streaming kernels (exact f16 integers from the quant bits, one packed fma with
// s = d * scale, f32 accumulation on v_mfma_f32_16x16x32_f16; the Q4_K minima and the Q6_K offset through a twin MFMA
// of the same activation fragment into a second accumulator that is subtracted at the end).
#include "common.h"
#include "mfma_unpack.h"

#include <algorithm>
#include <cstdlib>

namespace {

struct WholeArgs {
    const uint8_t *w;
    const uint8_t *xf;
    float *y;
    uint8_t *y_xf;
    int y_xf_kind;
    int n_out;   // rows of w (pair mode: 2 * ffn)
    int nb;      // super-blocks per row
    int n_rows;
    int ksplit;  // K slices per unit; waves per workgroup = ksplit * tl
    int tl;      // units per workgroup
    int n_units; // plain: ceil(tiles / R) units of R consecutive tiles; pair: ffn / 16 units of (gate tile, up tile)
    int pair_off;  // pair mode: tiles between a gate tile and its up tile; 0 = plain
    uint32_t row_bytes;  // Q6_K (GGUF row order): bytes per weight row
    // several 16-row blocks against the same weights (a prefill): block i reads xf + i * xf_stride bytes and writes
    // y + i * y_stride floats (y_xf + i * y_xf_stride bytes); the last block has rows_last rows, the others 16
    int n_blocks, rows_last;
    uint32_t xf_stride, y_xf_stride;
    size_t y_stride;
};

// ---- Q4_K, tiled order: [tile group of 256 rows][super-block][tile][row][144-byte block] ----
struct Q4W {
    u32x4_t hdr, q0, q1;
};
__device__ __forceinline__ void load_w(Q4W &r, const WholeArgs &a, int tile, int b, int lane) {
    const int n = lane & 15, g = lane >> 4;
    const uint8_t *p = a.w + ((static_cast<size_t>(tile >> 4) * a.nb + b) * 16 + (tile & 15)) * (16 * DFL_Q4_K_BYTES) +
                       n * DFL_Q4_K_BYTES;
    r.hdr = *reinterpret_cast<const u32x4_t *>(p);
    r.q0 = *reinterpret_cast<const u32x4_t *>(p + 16 + 32 * g);
    r.q1 = *reinterpret_cast<const u32x4_t *>(p + 32 + 32 * g);
}
// One super-block of one tile: lane (n = weight row, g = 64-value chunk) against the eight activation fragments.
__device__ __forceinline__ void compute(const Q4W &r, const half8_t (&af)[8], int lane, uint8_t *, uint32_t sc_sel, Q4KMagic magic,
                                        float4_t &acc, float4_t &acc_sub) {
    const int g = lane >> 4;
    const u32x4_t hdr = r.hdr;
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
    const _Float16 m_lo = M[0], m_hi = M[1];
    const half8_t bml = {m_lo, m_lo, m_lo, m_lo, m_lo, m_lo, m_lo, m_lo};
    const half8_t bmh = {m_hi, m_hi, m_hi, m_hi, m_hi, m_hi, m_hi, m_hi};
    const uint32_t qw[8] = {r.q0.x, r.q0.y, r.q0.z, r.q0.w, r.q1.x, r.q1.y, r.q1.z, r.q1.w};
#pragma unroll
    for (int t = 0; t < 4; t++) {
        const half8_t bl = unpack_scale<false>(qw[2 * t], qw[2 * t + 1], s2l, c2l, magic.lo);
        acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(af[t], bl, acc, 0, 0, 0);
        acc_sub = __builtin_amdgcn_mfma_f32_16x16x32_f16(af[t], bml, acc_sub, 0, 0, 0);
    }
#pragma unroll
    for (int t = 0; t < 4; t++) {
        const half8_t bh = unpack_scale<true>(qw[2 * t], qw[2 * t + 1], s2h, c2h, magic.hi);
        acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(af[4 + t], bh, acc, 0, 0, 0);
        acc_sub = __builtin_amdgcn_mfma_f32_16x16x32_f16(af[4 + t], bmh, acc_sub, 0, 0, 0);
    }
}

// The same in two steps, for a launch that multiplies many row blocks with one set of weights: the B operands of a
// super-block's eight MFMAs once (unpack), then only the MFMAs per row block (mma), in compute()'s order.
struct Q4F {
    half8_t b[8];
    _Float16 m_lo, m_hi;
};
__device__ __forceinline__ void unpack(const Q4W &r, int lane, uint8_t *, uint32_t sc_sel, Q4KMagic magic, Q4F &f) {
    const int g = lane >> 4;
    const u32x4_t hdr = r.hdr;
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
    f.m_lo = M[0];
    f.m_hi = M[1];
    const uint32_t qw[8] = {r.q0.x, r.q0.y, r.q0.z, r.q0.w, r.q1.x, r.q1.y, r.q1.z, r.q1.w};
#pragma unroll
    for (int t = 0; t < 4; t++) {
        f.b[t] = unpack_scale<false>(qw[2 * t], qw[2 * t + 1], s2l, c2l, magic.lo);
        f.b[4 + t] = unpack_scale<true>(qw[2 * t], qw[2 * t + 1], s2h, c2h, magic.hi);
    }
}
__device__ __forceinline__ void mma(const Q4F &f, const half8_t (&af)[8], float4_t &acc, float4_t &acc_sub) {
    const half8_t bml = {f.m_lo, f.m_lo, f.m_lo, f.m_lo, f.m_lo, f.m_lo, f.m_lo, f.m_lo};
    const half8_t bmh = {f.m_hi, f.m_hi, f.m_hi, f.m_hi, f.m_hi, f.m_hi, f.m_hi, f.m_hi};
#pragma unroll
    for (int t = 0; t < 8; t++) {
        acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(af[t], f.b[t], acc, 0, 0, 0);
        acc_sub = __builtin_amdgcn_mfma_f32_16x16x32_f16(af[t], t < 4 ? bml : bmh, acc_sub, 0, 0, 0);
    }
}

// ---- Q6_K, GGUF row order: 210-byte blocks (ql[128], qh[64], scales[16], d), rows 2-byte aligned ----
// A tile's stage is 16 runs of 210 bytes a row stride apart.  They are loaded as 208 pieces of 16 bytes (13 per row,
// consecutive lanes taking consecutive pieces: row-contiguous requests) plus d, and pass through a wave-private LDS
// area with a 240-byte row stride, from which lane (n, g) picks its operands with aligned reads.  (Loading each lane's
// operands straight from memory, seven scattered unaligned loads, measured 8 us per launch against 4.8 us for the
// same bytes of Q4_K.)
constexpr int kQ6RowStride = 240;
constexpr int kQ6AreaBytes = 16 * kQ6RowStride;
typedef u32x4_t u32x4_unaligned_t __attribute__((aligned(2)));
struct Q6W {
    u32x4_t p[4];
    uint32_t d;
};
__device__ __forceinline__ void load_w(Q6W &r, const WholeArgs &a, int tile, int b, int lane) {
    const uint8_t *base = a.w + static_cast<size_t>(b) * DFL_Q6_K_BYTES;
    const int last = a.n_out - 1;  // rows past the matrix re-read its last row; never stored
#pragma unroll
    for (int j = 0; j < 4; j++) {
        const int i = min(lane + 64 * j, 207);
        const int row = min(tile * 16 + i / 13, last);
        r.p[j] = *reinterpret_cast<const u32x4_unaligned_t *>(base + static_cast<size_t>(row) * a.row_bytes + 16 * (i % 13));
    }
    r.d = *reinterpret_cast<const uint16_t *>(base + static_cast<size_t>(min(tile * 16 + (lane & 15), last)) * a.row_bytes + 208);
}
// A lane's operands of one super-block of one weight row (lane (n, g): half h = g / 2, quarters (g & 1) and 2 + (g & 1)):
// 32 bytes of ql, 32 of qh, the four scales of its two quarters and d.
struct Q6Ops {
    u32x4_t qa, qb, ha, hb;
    uint32_t sc4, sc4h;  // low 16 bits: the two int8 scales of the low (high) quarter
    float d;
};
// The lane's operands out of a wave-private LDS area that holds the tile's sixteen raw 210-byte blocks, rows 240 bytes apart.
__device__ __forceinline__ Q6Ops q6_stage_through_lds(const Q6W &r, int lane, uint8_t *area) {
    const int n = lane & 15, g = lane >> 4, h = g >> 1, odd = g & 1;
#pragma unroll
    for (int j = 0; j < 4; j++) {
        const int i = lane + 64 * j;
        if (i < 208) *reinterpret_cast<u32x4_t *>(area + (i / 13) * kQ6RowStride + 16 * (i % 13)) = r.p[j];
    }
    if (lane < 16) *reinterpret_cast<uint16_t *>(area + lane * kQ6RowStride + 208) = static_cast<uint16_t>(r.d);
    __builtin_amdgcn_wave_barrier();
    const uint8_t *rowp = area + n * kQ6RowStride;
    Q6Ops o;
    o.qa = *reinterpret_cast<const u32x4_t *>(rowp + 64 * h + 32 * odd);
    o.qb = *reinterpret_cast<const u32x4_t *>(rowp + 64 * h + 32 * odd + 16);
    o.ha = *reinterpret_cast<const u32x4_t *>(rowp + 128 + 32 * h);
    o.hb = *reinterpret_cast<const u32x4_t *>(rowp + 128 + 32 * h + 16);
    o.sc4 = (*reinterpret_cast<const uint32_t *>(rowp + 192 + 8 * h) >> (16 * odd)) & 0xffffu;
    o.sc4h = (*reinterpret_cast<const uint32_t *>(rowp + 192 + 8 * h + 4) >> (16 * odd)) & 0xffffu;
    o.d = __half2float(__ushort_as_half(*reinterpret_cast<const uint16_t *>(rowp + 208)));
    __builtin_amdgcn_wave_barrier();  // (the area is rewritten by this wave's next tile only after these reads: LDS runs a wave's accesses in order)
    return o;
}
__device__ __forceinline__ void q6_compute(const Q6Ops &o, const half8_t (&af)[8], int lane, Q4KMagic magic, float4_t &acc, float4_t &acc_sub) {
    const int odd = (lane >> 4) & 1;
    const int hs = 2 * odd;
    const uint32_t hq[8] = {o.ha.x >> hs, o.ha.y >> hs, o.ha.z >> hs, o.ha.w >> hs, o.hb.x >> hs, o.hb.y >> hs, o.hb.z >> hs, o.hb.w >> hs};
    const uint32_t ql[8] = {o.qa.x, o.qa.y, o.qa.z, o.qa.w, o.qb.x, o.qb.y, o.qb.z, o.qb.w};
    const float d = o.d;
    auto scale = [&](uint32_t pair, int j) { return static_cast<_Float16>(d * static_cast<float>(static_cast<int8_t>(pair >> (8 * j)))); };
    const _Float16 s_l0 = scale(o.sc4, 0), s_l1 = scale(o.sc4, 1), s_h0 = scale(o.sc4h, 0), s_h1 = scale(o.sc4h, 1);
#pragma unroll
    for (int t = 0; t < 4; t++) {
        const _Float16 sl = (t >> 1) ? s_l1 : s_l0;
        const half8_t bl = unpack6<false>(ql[2 * t], ql[2 * t + 1], hq[2 * t], hq[2 * t + 1], splat(sl),
                                          splat(sl * static_cast<_Float16>(-1024.0f)), magic.lo);
        acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(af[t], bl, acc, 0, 0, 0);
        const _Float16 of = sl * static_cast<_Float16>(32.0f);
        const half8_t bo = {of, of, of, of, of, of, of, of};
        acc_sub = __builtin_amdgcn_mfma_f32_16x16x32_f16(af[t], bo, acc_sub, 0, 0, 0);
    }
#pragma unroll
    for (int t = 0; t < 4; t++) {
        const _Float16 sh = (t >> 1) ? s_h1 : s_h0;
        const half8_t bh = unpack6<true>(ql[2 * t], ql[2 * t + 1], hq[2 * t] >> 4, hq[2 * t + 1] >> 4, splat(sh),
                                         splat(sh * static_cast<_Float16>(-64.0f)), magic.hi);
        acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(af[4 + t], bh, acc, 0, 0, 0);
        const _Float16 of = sh * static_cast<_Float16>(32.0f);
        const half8_t bo = {of, of, of, of, of, of, of, of};
        acc_sub = __builtin_amdgcn_mfma_f32_16x16x32_f16(af[4 + t], bo, acc_sub, 0, 0, 0);
    }
}
__device__ __forceinline__ void compute(const Q6W &r, const half8_t (&af)[8], int lane, uint8_t *area, uint32_t, Q4KMagic magic,
                                        float4_t &acc, float4_t &acc_sub) {
    q6_compute(q6_stage_through_lds(r, lane, area), af, lane, magic, acc, acc_sub);
}

// ---- Q6_K, tiled and field-planar: [tile group of 256 rows][super-block][tile 0..15][3360 bytes], a tile's sixteen
// blocks as four sections - ql [row][128], qh [row][64], scales [row][16], d [row] (f16) - every 16-byte piece aligned.
// The 16-byte pieces of a row's ql (qh) sit at piece index p ^ (row & 7) (p ^ ((row >> 1) & 3)): a layout that a wave
// can also read from LDS without bank conflicts.  Lane (n, g) fetches exactly its operands: four 16-byte loads, one of
// 8 bytes, one of 2, all aligned, a row's ql line shared by the four lanes of the row - no staging, no LDS.
constexpr int kQ6TileBytes = 16 * DFL_Q6_K_BYTES;  // 3360
constexpr int kQ6TQh = 2048, kQ6TSc = 3072, kQ6TD = 3328;
struct Q6T {
    u32x4_t qa, qb, ha, hb;
    uint32_t s0, s1;
    uint32_t d;
};
__host__ __device__ __forceinline__ int q6t_ql_piece(int row, int p) { return row * 128 + ((p ^ (row & 7)) << 4); }
__host__ __device__ __forceinline__ int q6t_qh_piece(int row, int p) { return kQ6TQh + row * 64 + ((p ^ ((row >> 1) & 3)) << 4); }
__device__ __forceinline__ void load_w(Q6T &r, const WholeArgs &a, int tile, int b, int lane) {
    const int n = lane & 15, g = lane >> 4, h = g >> 1, odd = g & 1;
    const uint8_t *p = a.w + ((static_cast<size_t>(tile >> 4) * a.nb + b) * 16 + (tile & 15)) * kQ6TileBytes;
    r.qa = *reinterpret_cast<const u32x4_t *>(p + q6t_ql_piece(n, 4 * h + 2 * odd));
    r.qb = *reinterpret_cast<const u32x4_t *>(p + q6t_ql_piece(n, 4 * h + 2 * odd + 1));
    r.ha = *reinterpret_cast<const u32x4_t *>(p + q6t_qh_piece(n, 2 * h));
    r.hb = *reinterpret_cast<const u32x4_t *>(p + q6t_qh_piece(n, 2 * h + 1));
    const uint2 sc = *reinterpret_cast<const uint2 *>(p + kQ6TSc + n * 16 + 8 * h);
    r.s0 = sc.x;
    r.s1 = sc.y;
    r.d = *reinterpret_cast<const uint16_t *>(p + kQ6TD + n * 2);
}
__device__ __forceinline__ Q6Ops q6_ops(const Q6T &r, int lane) {
    const int odd = (lane >> 4) & 1;
    Q6Ops o;
    o.qa = r.qa;
    o.qb = r.qb;
    o.ha = r.ha;
    o.hb = r.hb;
    o.sc4 = (r.s0 >> (16 * odd)) & 0xffffu;
    o.sc4h = (r.s1 >> (16 * odd)) & 0xffffu;
    o.d = __half2float(__ushort_as_half(static_cast<uint16_t>(r.d)));
    return o;
}
__device__ __forceinline__ void compute(const Q6T &r, const half8_t (&af)[8], int lane, uint8_t *, uint32_t, Q4KMagic magic, float4_t &acc,
                                        float4_t &acc_sub) {
    q6_compute(q6_ops(r, lane), af, lane, magic, acc, acc_sub);
}

struct Q6F {
    half8_t b[8];
    _Float16 o[4];  // 32 s of the four scale pairs: low quarter's two, high quarter's two
};
__device__ __forceinline__ void q6_unpack(const Q6Ops &o, int lane, Q4KMagic magic, Q6F &f) {
    const int odd = (lane >> 4) & 1;
    const int hs = 2 * odd;
    const uint32_t hq[8] = {o.ha.x >> hs, o.ha.y >> hs, o.ha.z >> hs, o.ha.w >> hs, o.hb.x >> hs, o.hb.y >> hs, o.hb.z >> hs, o.hb.w >> hs};
    const uint32_t ql[8] = {o.qa.x, o.qa.y, o.qa.z, o.qa.w, o.qb.x, o.qb.y, o.qb.z, o.qb.w};
    const float d = o.d;
    auto scale = [&](uint32_t pair, int j) { return static_cast<_Float16>(d * static_cast<float>(static_cast<int8_t>(pair >> (8 * j)))); };
    const _Float16 s_l0 = scale(o.sc4, 0), s_l1 = scale(o.sc4, 1), s_h0 = scale(o.sc4h, 0), s_h1 = scale(o.sc4h, 1);
    const _Float16 k32 = static_cast<_Float16>(32.0f);
    f.o[0] = s_l0 * k32;
    f.o[1] = s_l1 * k32;
    f.o[2] = s_h0 * k32;
    f.o[3] = s_h1 * k32;
#pragma unroll
    for (int t = 0; t < 4; t++) {
        const _Float16 sl = (t >> 1) ? s_l1 : s_l0, sh = (t >> 1) ? s_h1 : s_h0;
        f.b[t] = unpack6<false>(ql[2 * t], ql[2 * t + 1], hq[2 * t], hq[2 * t + 1], splat(sl), splat(sl * static_cast<_Float16>(-1024.0f)),
                                magic.lo);
        f.b[4 + t] = unpack6<true>(ql[2 * t], ql[2 * t + 1], hq[2 * t] >> 4, hq[2 * t + 1] >> 4, splat(sh),
                                   splat(sh * static_cast<_Float16>(-64.0f)), magic.hi);
    }
}
__device__ __forceinline__ void unpack(const Q6W &r, int lane, uint8_t *area, uint32_t, Q4KMagic magic, Q6F &f) {
    q6_unpack(q6_stage_through_lds(r, lane, area), lane, magic, f);
}
__device__ __forceinline__ void unpack(const Q6T &r, int lane, uint8_t *, uint32_t, Q4KMagic magic, Q6F &f) {
    q6_unpack(q6_ops(r, lane), lane, magic, f);
}
__device__ __forceinline__ void mma(const Q6F &f, const half8_t (&af)[8], float4_t &acc, float4_t &acc_sub) {
#pragma unroll
    for (int t = 0; t < 8; t++) {
        acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(af[t], f.b[t], acc, 0, 0, 0);
        const _Float16 o = f.o[t >> 1];
        const half8_t bo = {o, o, o, o, o, o, o, o};
        acc_sub = __builtin_amdgcn_mfma_f32_16x16x32_f16(af[t], bo, acc_sub, 0, 0, 0);
    }
}
template <typename W>
struct FragsOf;
template <>
struct FragsOf<Q4W> {
    typedef Q4F type;
};
template <>
struct FragsOf<Q6W> {
    typedef Q6F type;
};
template <>
struct FragsOf<Q6T> {
    typedef Q6F type;
};

__device__ __forceinline__ void load_xf(half8_t (&af)[8], const uint8_t *xf, int b, int lane) {
    const half8_t *p = reinterpret_cast<const half8_t *>(xf) + static_cast<size_t>(b) * 512 + lane;
#pragma unroll
    for (int t = 0; t < 8; t++) af[t] = p[t * 64];
}

// W: Q4W or Q6W.  R: tiles per wave and stage (they share the stage's activation fragments).
// kMulti: several 16-row blocks per launch (a.n_blocks): 1 = every wave has one stage (K of at most 16 super-blocks), 2 = one or
// two; the single-block instances (0) keep the registers of a kernel without the loop.
template <typename W, int R, int kMulti>
__global__ void __launch_bounds__(1024) gemm_whole_kernel(WholeArgs a) {
    // [16 waves][R] partial tiles; Q6_K: then a staging area per wave
    extern __shared__ float4_t red[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int tlane = wave / a.ksplit, kslice = wave - tlane * a.ksplit;
    const int unit = blockIdx.x * a.tl + tlane;
    const bool active = unit < a.n_units;
    const int n = lane & 15, g = lane >> 4;
    const int b0 = a.nb * kslice / a.ksplit, b1 = a.nb * (kslice + 1) / a.ksplit;  // one or two stages (host)
    const bool two = kMulti != 1 && b1 - b0 > 1;
    const int n_tiles = (a.n_out + 15) >> 4;
    int tile[R];
#pragma unroll
    for (int r = 0; r < R; r++) tile[r] = min(a.pair_off ? unit + r * a.pair_off : unit * R + r, n_tiles - 1);
    float4_t acc[R], acc_sub[R];
    const uint32_t sc_sel = (lane & 16) ? 0x04030402u : 0x04010400u;
    const Q4KMagic magic = q4k_magic();
    uint8_t *area = reinterpret_cast<uint8_t *>(red + 16 * R * 64) + wave * kQ6AreaBytes;
    // (every load in flight together where the registers hold them; else one tile at a time)
    constexpr bool kEarly = sizeof(W) * R <= 96;
    W w0[kEarly ? R : 1], w1[kEarly ? R : 1];
    if (kEarly && active) {
        // the weights come from HBM, the activations from L2: weights first; they stay in registers for every block
#pragma unroll
        for (int r = 0; r < (kEarly ? R : 1); r++) load_w(w0[r], a, tile[r], b0, lane);
        if (two) {
#pragma unroll
            for (int r = 0; r < (kEarly ? R : 1); r++) load_w(w1[r], a, tile[r], b0 + 1, lane);
        }
    }
    const int n_blocks = kMulti ? a.n_blocks : 1;
    half8_t af[8];
    if (kEarly && active) load_xf(af, a.xf, b0, lane);
    // many row blocks, one tile per wave: the B operands are unpacked once and stay in registers in place of the raw weights
    constexpr bool kFrags = kMulti != 0 && kEarly && R == 1;
    typename FragsOf<W>::type f0, f1;
    if (kFrags && active) {
        unpack(w0[0], lane, area, sc_sel, magic, f0);
        if (two) unpack(w1[0], lane, area, sc_sel, magic, f1);
    }
    for (int blk = 0; blk < n_blocks; blk++) {
        const uint8_t *xf = a.xf + static_cast<size_t>(blk) * a.xf_stride;
        const int n_rows = blk + 1 == n_blocks ? a.rows_last : 16;
#pragma unroll
        for (int r = 0; r < R; r++) acc[r] = acc_sub[r] = float4_t{0, 0, 0, 0};
        if (active) {
            if constexpr (kFrags) {
                mma(f0, af, acc[0], acc_sub[0]);
                if (two) {
                    load_xf(af, xf, b0 + 1, lane);
                    mma(f1, af, acc[0], acc_sub[0]);
                }
                if (blk + 1 < n_blocks) load_xf(af, xf + a.xf_stride, b0, lane);
            } else if constexpr (kEarly) {
                // (af holds this block's first stage: loaded above, or behind the previous block's products)
#pragma unroll
                for (int r = 0; r < R; r++) compute(w0[r], af, lane, area, sc_sel, magic, acc[r], acc_sub[r]);
                if (two) {
                    load_xf(af, xf, b0 + 1, lane);
#pragma unroll
                    for (int r = 0; r < R; r++) compute(w1[r], af, lane, area, sc_sel, magic, acc[r], acc_sub[r]);
                }
                // the next block's fragments travel while this block's partial tiles are summed and written
                if (kMulti != 0 && blk + 1 < n_blocks) load_xf(af, xf + a.xf_stride, b0, lane);
            } else {
                for (int b = b0; b < b1; b++) {
                    load_xf(af, xf, b, lane);
#pragma unroll
                    for (int r = 0; r < R; r++) {
                        W w;
                        load_w(w, a, tile[r], b, lane);
                        compute(w, af, lane, area, sc_sel, magic, acc[r], acc_sub[r]);
                    }
                }
            }
        }
        if (blk) __syncthreads();  // the previous block's partial tiles have been summed
#pragma unroll
        for (int r = 0; r < R; r++) red[(wave * R + r) * 64 + lane] = acc[r] - acc_sub[r];
        __syncthreads();
        if (kslice != 0 || !active) continue;
        float4_t sum[R];
#pragma unroll
        for (int r = 0; r < R; r++) {
            sum[r] = red[(wave * R + r) * 64 + lane];
            for (int s = 1; s < a.ksplit; s++) sum[r] += red[((wave + s) * R + r) * 64 + lane];
        }
        float *y = a.y ? a.y + static_cast<size_t>(blk) * a.y_stride : nullptr;
        if (!a.pair_off) {
#pragma unroll
            for (int r = 0; r < R; r++) {
                const int col = (unit * R + r) * 16 + n;
                if (col < a.n_out) {
#pragma unroll
                    for (int i = 0; i < 4; i++)
                        if (4 * g + i < n_rows) y[static_cast<size_t>(4 * g + i) * a.n_out + col] = sum[r][i];
                }
            }
            continue;
        }
        if constexpr (R == 2) {
            // SwiGLU of the (gate tile, up tile) pair: out[m][16 unit + n] = silu(gate) * up
            const int ffn = a.n_out >> 1;
            float4_t out;
#pragma unroll
            for (int i = 0; i < 4; i++) out[i] = sum[0][i] / (1.0f + expf(-sum[0][i])) * sum[1][i];
            const int col = unit * 16 + n;
            if (y && col < ffn) {
#pragma unroll
                for (int i = 0; i < 4; i++)
                    if (4 * g + i < n_rows) y[static_cast<size_t>(4 * g + i) * ffn + col] = out[i];
            }
            if (a.y_xf) {
                // the tile through this wave's own LDS slot: lane (m, octet) then holds eight consecutive columns of a row
                // (the slot's partial tile has been read: by this wave, above)
                float *f = reinterpret_cast<float *>(&red[wave * R * 64]);
                red[wave * R * 64 + lane] = out;
                __builtin_amdgcn_wave_barrier();
                if (lane < 32) {
                    const int m = lane >> 1, oct = lane & 1;
                    float v[8];
#pragma unroll
                    for (int i = 0; i < 8; i++) v[i] = f[((8 * oct + i) + 16 * (m >> 2)) * 4 + (m & 3)];
                    dfl_xf_store(a.y_xf + static_cast<size_t>(blk) * a.y_xf_stride, a.y_xf_kind, m, unit * 16 + 8 * oct, v[0], v[1], v[2],
                                 v[3], v[4], v[5], v[6], v[7]);
                }
            }
        }
    }
}

// The same product for a matrix of many more tiles than one round of the chip (an output head: 151936 rows), K of at
// most 16 super-blocks: a workgroup walks units blockIdx.x * tl + tlane, + gridDim.x * tl, ...  A wave's K slice is
// the same super-block in every unit, so its eight activation fragments are loaded ONCE and stay in registers; the
// weights of the next unit travel while the current one is unpacked and multiplied; the slices' partial tiles meet
// in one of two LDS buffers in turn (one barrier per unit: a buffer is rewritten two units later, behind the barrier
// of the unit in between).  Same sums, in the same order, as gemm_whole_kernel.
template <typename W>
__global__ void __launch_bounds__(1024) gemm_whole_loop_kernel(WholeArgs a) {
    extern __shared__ float4_t red[];  // [2][16 waves][64]; Q6_K in row order: then a staging area per wave
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int tlane = wave / a.ksplit, kslice = wave - tlane * a.ksplit;
    const int n = lane & 15, g = lane >> 4;
    const int b0 = a.nb * kslice / a.ksplit;  // one stage per wave (host: nb <= 16, so ksplit == nb and every slice is one super-block)
    const bool has_stage = a.nb * (kslice + 1) / a.ksplit > b0;
    const int n_tiles = (a.n_out + 15) >> 4;
    const int stride = static_cast<int>(gridDim.x) * a.tl;
    const uint32_t sc_sel = (lane & 16) ? 0x04030402u : 0x04010400u;
    const Q4KMagic magic = q4k_magic();
    uint8_t *area = reinterpret_cast<uint8_t *>(red + 2 * 16 * 64) + wave * kQ6AreaBytes;
    int unit = static_cast<int>(blockIdx.x) * a.tl + tlane;
    W w_cur, w_next;
    if (unit < n_tiles && has_stage) load_w(w_cur, a, unit, b0, lane);
    half8_t af[8];
    if (has_stage) load_xf(af, a.xf, b0, lane);
    for (int it = 0;; it++) {
        const int next = unit + stride;
        if (next < n_tiles && has_stage) load_w(w_next, a, next, b0, lane);
        float4_t acc = {0, 0, 0, 0}, acc_sub = {0, 0, 0, 0};
        if (unit < n_tiles && has_stage) compute(w_cur, af, lane, area, sc_sel, magic, acc, acc_sub);
        float4_t *buf = red + (it & 1) * (16 * 64);
        buf[wave * 64 + lane] = acc - acc_sub;
        __syncthreads();
        if (kslice == 0 && unit < n_tiles) {
            float4_t sum = buf[wave * 64 + lane];
            for (int s = 1; s < a.ksplit; s++) sum += buf[(wave + s) * 64 + lane];
            const int col = unit * 16 + n;
            if (col < a.n_out) {
#pragma unroll
                for (int i = 0; i < 4; i++)
                    if (4 * g + i < a.n_rows) a.y[static_cast<size_t>(4 * g + i) * a.n_out + col] = sum[i];
            }
        }
        // (the same decision in every wave of the workgroup: its first unit lane's next index)
        if (static_cast<int>(blockIdx.x) * a.tl + (it + 1) * stride >= n_tiles) break;
        unit = next;
        w_cur = w_next;
    }
}

// The looping kernel for the tiled Q6_K order with the weights brought in through LDS instead of registers: a wave
// streams its (tile, super-block) pieces - 3360 contiguous bytes, 210 pieces of 16 - with direct-to-LDS loads into a
// private ring of two buffers and picks its operands out of them with aligned, conflict-free reads (that is what the
// order's piece rotation is for).  No registers are tied up by bytes in flight, so two units travel per wave (the
// register version holds one and already spills); "landed" is an s_waitcnt vmcnt of the younger unit's four loads
// (loads return in order; a Y store of the previous unit that is still in flight only makes the wait stricter).
typedef const __attribute__((address_space(1))) void *gptr_t;
typedef __attribute__((address_space(3))) void *lptr_t;
constexpr int kQ6RingDepth = 2;
constexpr int kVmcnt4 = (4 & 0xF) | 0x0F70, kVmcnt0 = 0x0F70;  // s_waitcnt vmcnt(n), the other counters left alone (gfx9 encoding)
constexpr size_t kQ6LoopLds = static_cast<size_t>(2) * 16 * 64 * sizeof(float4_t) + static_cast<size_t>(16) * kQ6RingDepth * kQ6TileBytes;
__global__ void __launch_bounds__(1024) gemm_q6t_loop_kernel(WholeArgs a) {
    extern __shared__ float4_t red[];  // [2][16 waves][64], then the rings [16 waves][kQ6RingDepth][3360 bytes]
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int tlane = wave / a.ksplit, kslice = wave - tlane * a.ksplit;
    const int n = lane & 15, g = lane >> 4, h = g >> 1, odd = g & 1;
    const int b0 = kslice;  // (host: nb <= 16, so ksplit == nb and every slice is one super-block)
    const int n_tiles = (a.n_out + 15) >> 4;
    const int stride = static_cast<int>(gridDim.x) * a.tl;
    const Q4KMagic magic = q4k_magic();
    uint8_t *ring = reinterpret_cast<uint8_t *>(red + 2 * 16 * 64) + static_cast<size_t>(wave) * (kQ6RingDepth * kQ6TileBytes);
    auto issue = [&](int unit, int slot) {  // the unit's 210 pieces into ring buffer `slot`
        const uint8_t *src = a.w + ((static_cast<size_t>(unit >> 4) * a.nb + b0) * 16 + (unit & 15)) * kQ6TileBytes + lane * 16;
        uint8_t *dst = ring + slot * kQ6TileBytes;
        __builtin_amdgcn_global_load_lds((gptr_t)(src), (lptr_t)(dst), 16, 0, 0);
        __builtin_amdgcn_global_load_lds((gptr_t)(src + 1024), (lptr_t)(dst + 1024), 16, 0, 0);
        __builtin_amdgcn_global_load_lds((gptr_t)(src + 2048), (lptr_t)(dst + 2048), 16, 0, 0);
        // (the fourth load carries the last 18 pieces: a lane's 16 bytes land at the buffer address + 16 lane whatever it
        // reads, so the other lanes stay out of it; the wave still issues four loads, which is what the count below needs)
        if (lane < 18) __builtin_amdgcn_global_load_lds((gptr_t)(src + 3072), (lptr_t)(dst + 3072), 16, 0, 0);
    };
    int unit = static_cast<int>(blockIdx.x) * a.tl + tlane;
    half8_t af[8];
    load_xf(af, a.xf, b0, lane);
    __builtin_amdgcn_s_waitcnt(kVmcnt0);  // (the fragments are in registers: from here on only weight loads and Y stores are counted)
    if (unit < n_tiles) issue(unit, 0);
    for (int it = 0;; it++) {
        const int next = unit + stride;
        const int slot = it & 1;
        if (next < n_tiles) issue(next, slot ^ 1);  // (that buffer's unit was consumed one iteration ago: its reads are complete)
        float4_t acc = {0, 0, 0, 0}, acc_sub = {0, 0, 0, 0};
        if (unit < n_tiles) {
            if (next < n_tiles)
                __builtin_amdgcn_s_waitcnt(kVmcnt4);
            else
                __builtin_amdgcn_s_waitcnt(kVmcnt0);
            const uint8_t *t = ring + slot * kQ6TileBytes;
            Q6Ops o;
            o.qa = *reinterpret_cast<const u32x4_t *>(t + q6t_ql_piece(n, 4 * h + 2 * odd));
            o.qb = *reinterpret_cast<const u32x4_t *>(t + q6t_ql_piece(n, 4 * h + 2 * odd + 1));
            o.ha = *reinterpret_cast<const u32x4_t *>(t + q6t_qh_piece(n, 2 * h));
            o.hb = *reinterpret_cast<const u32x4_t *>(t + q6t_qh_piece(n, 2 * h + 1));
            const uint2 sc = *reinterpret_cast<const uint2 *>(t + kQ6TSc + n * 16 + 8 * h);
            o.sc4 = (sc.x >> (16 * odd)) & 0xffffu;
            o.sc4h = (sc.y >> (16 * odd)) & 0xffffu;
            o.d = __half2float(__ushort_as_half(*reinterpret_cast<const uint16_t *>(t + kQ6TD + n * 2)));
            q6_compute(o, af, lane, magic, acc, acc_sub);
        }
        float4_t *buf = red + slot * (16 * 64);
        buf[wave * 64 + lane] = acc - acc_sub;
        __syncthreads();
        if (kslice == 0 && unit < n_tiles) {
            float4_t sum = buf[wave * 64 + lane];
            for (int s = 1; s < a.ksplit; s++) sum += buf[(wave + s) * 64 + lane];
            const int col = unit * 16 + n;
            if (col < a.n_out) {
#pragma unroll
                for (int i = 0; i < 4; i++)
                    if (4 * g + i < a.n_rows) a.y[static_cast<size_t>(4 * g + i) * a.n_out + col] = sum[i];
            }
        }
        if (static_cast<int>(blockIdx.x) * a.tl + (it + 1) * stride >= n_tiles) break;
        unit = next;
    }
}

// Row-major activations -> XF: one thread per (row, eight consecutive values).
template <typename XT>
__global__ void __launch_bounds__(256) pack_xf_kernel(const XT *__restrict__ x, int n_rows, int n_in, int kind, uint8_t *__restrict__ xf) {
    const int oct = blockIdx.x * 256 + threadIdx.x, m = blockIdx.y;
    if (8 * oct >= n_in || m >= n_rows) return;
    const XT *p = x + static_cast<size_t>(m) * n_in + 8 * oct;
    dfl_xf_store(xf, kind, m, 8 * oct, static_cast<float>(p[0]), static_cast<float>(p[1]), static_cast<float>(p[2]), static_cast<float>(p[3]),
                 static_cast<float>(p[4]), static_cast<float>(p[5]), static_cast<float>(p[6]), static_cast<float>(p[7]));
}

struct EnvInt {
    const char *name;
    bool set;
    int value;
    explicit EnvInt(const char *n) : name(n), set(false), value(0) {
        if (const char *e = getenv(n)) {
            set = true;
            value = atoi(e);
        }
    }
    int get(int fallback) const { return set ? value : fallback; }
};
#define env_int(name, fallback) ([]() -> const EnvInt & { static const EnvInt e(name); return e; }().get(fallback))

struct WholePlan {
    int kind, ksplit, tl, R, n_units, n_wg;
    bool loop;  // more units than one round: gemm_whole_loop_kernel (one stage per wave, plain product)
};

// The split of a matrix over waves, or kind == DFL_XF_NONE where this path does not take it.
WholePlan whole_plan(const dflash_ctx *ctx, int32_t w_type, int64_t n_in, int64_t n_out, int64_t pair_ffn) {
    WholePlan p = {DFL_XF_NONE, 0, 0, 0, 0, 0, false};
    if (!env_int("DFLASH_GEMM_WHOLE", 1)) return p;
    const int kind = w_type == DFLASH_TYPE_Q4_K_TILED ? DFL_XF_Q4K
                     : (w_type == DFLASH_TYPE_Q6_K || w_type == DFLASH_TYPE_Q6_K_TILED) ? DFL_XF_Q6K
                                                                                       : DFL_XF_NONE;
    if (kind == DFL_XF_NONE || n_in <= 0 || n_in % DFL_QK_K || n_out <= 0 || n_out >= (1 << 24)) return p;
    const int nb = static_cast<int>(n_in / DFL_QK_K);
    if (nb > 32) return p;  // more than two stages per wave
    if (pair_ffn && (n_out != 2 * pair_ffn || pair_ffn % 16)) return p;
    const int ksplit = nb < 16 ? nb : 16, tl = 16 / ksplit;
    const int tiles = static_cast<int>((n_out + 15) / 16);
    int R = pair_ffn ? 2 : 1;
    int n_units = pair_ffn ? static_cast<int>(pair_ffn / 16) : tiles;
    // one round of the chip: at most one workgroup per CU (a wave's registers leave room for one)
    // (a quarter of a round more, 320 workgroups on 256 CUs, measured slower than two tiles per wave on 160: 10.1 -> 8.6 us
    // for 4096 -> 5120 Q4_K, 14.9 -> 14.0 us for 5120 -> 5120 Q6_K; DFLASH_WHOLE_TOL_PCT=25 for the former rule)
    static const int env_tol = env_int("DFLASH_WHOLE_TOL_PCT", 0);
    const int max_wg = ctx->n_cu + ctx->n_cu * env_tol / 100;
    if (!pair_ffn && (n_units + tl - 1) / tl > max_wg) {
        R = 2;
        n_units = (tiles + 1) / 2;
    }
    const int n_wg = (n_units + tl - 1) / tl;
    if (n_wg > max_wg) {
        // many rounds: the looping kernel, where every wave keeps one super-block of the activations (K <= 16 super-blocks)
        if (pair_ffn || nb > 16 || !env_int("DFLASH_GEMM_WHOLE_LOOP", 1)) return p;
        p = {kind, ksplit, tl, 1, tiles, std::min((tiles + tl - 1) / tl, ctx->n_cu), true};
        return p;
    }
    p = {kind, ksplit, tl, R, n_units, n_wg, false};
    return p;
}

}  // namespace

int dfl_whole_kind(const dflash_ctx *ctx, int32_t w_type, int64_t n_in, int64_t n_out, int64_t pair_ffn) {
    return whole_plan(ctx, w_type, n_in, n_out, pair_ffn).kind;
}

int32_t dfl_gemm_whole(dflash_ctx *ctx, int32_t w_type, const void *w, const void *xf, float *y, int64_t n_in, int64_t n_out,
                       int32_t n_rows, int64_t pair_ffn, void *y_xf, int y_xf_kind, hipStream_t st) {
    return dfl_gemm_whole_blocks(ctx, w_type, w, xf, y, n_in, n_out, n_rows, pair_ffn, y_xf, y_xf_kind, st);
}

int32_t dfl_gemm_whole_blocks(dflash_ctx *ctx, int32_t w_type, const void *w, const void *xf, float *y, int64_t n_in, int64_t n_out,
                              int32_t n_rows_total, int64_t pair_ffn, void *y_xf, int y_xf_kind, hipStream_t st) {
    const int32_t n_blocks = (n_rows_total + 15) / 16;
    const int32_t n_rows = n_rows_total - 16 * (n_blocks - 1);  // rows of the last block
    if (n_rows_total < 1 || n_blocks > 4096) return dfl_fail(ctx, DFLASH_ERR_BAD_SHAPE, "gemm_whole: %d rows", n_rows_total);
    const WholePlan p = whole_plan(ctx, w_type, n_in, n_out, pair_ffn);
    if (p.kind == DFL_XF_NONE) return dfl_fail(ctx, DFLASH_ERR_UNSUPPORTED, "gemm_whole: type %d, %lld -> %lld not taken", w_type,
                                               static_cast<long long>(n_in), static_cast<long long>(n_out));
    if (!w || !xf || n_rows < 1 || n_rows > 16 || (!y && !(pair_ffn && y_xf)))
        return dfl_fail(ctx, DFLASH_ERR_BAD_SHAPE, "gemm_whole: null operand or n_rows %d", n_rows);
    const bool q6_tiled = w_type == DFLASH_TYPE_Q6_K_TILED;
    if (reinterpret_cast<uintptr_t>(xf) % 16 || reinterpret_cast<uintptr_t>(w) % ((p.kind == DFL_XF_Q4K || q6_tiled) ? 16 : 2) ||
        (y_xf && reinterpret_cast<uintptr_t>(y_xf) % 16))
        return dfl_fail(ctx, DFLASH_ERR_ALIGNMENT, "gemm_whole: operand alignment");
    if (y_xf && (!pair_ffn || (y_xf_kind != DFL_XF_Q4K && y_xf_kind != DFL_XF_Q6K)))
        return dfl_fail(ctx, DFLASH_ERR_UNSUPPORTED, "gemm_whole: fragment-order output needs the SwiGLU pair mode and a kind");
    WholeArgs a;
    a.w = static_cast<const uint8_t *>(w);
    a.xf = static_cast<const uint8_t *>(xf);
    a.y = y;
    a.y_xf = static_cast<uint8_t *>(y_xf);
    a.y_xf_kind = y_xf_kind;
    a.n_out = static_cast<int>(n_out);
    a.nb = static_cast<int>(n_in / DFL_QK_K);
    a.n_rows = n_rows;
    a.ksplit = p.ksplit;
    a.tl = p.tl;
    a.n_units = p.n_units;
    a.pair_off = pair_ffn ? static_cast<int>(pair_ffn / 16) : 0;
    a.row_bytes = static_cast<uint32_t>(a.nb) * DFL_Q6_K_BYTES;
    a.n_blocks = n_blocks;
    a.rows_last = n_rows;
    a.xf_stride = static_cast<uint32_t>(dfl_xf_bytes(n_in));
    a.y_xf_stride = static_cast<uint32_t>(dfl_xf_bytes(pair_ffn ? pair_ffn : 256));
    a.y_stride = static_cast<size_t>(16) * (pair_ffn ? pair_ffn : n_out);
    const int threads = 64 * p.ksplit * p.tl;
    const size_t red_bytes = static_cast<size_t>(16) * p.R * 64 * sizeof(float4_t);
    const size_t lds = red_bytes + ((p.kind == DFL_XF_Q6K && !q6_tiled) ? static_cast<size_t>(16) * kQ6AreaBytes : 0);
    typedef void (*kernel_t)(WholeArgs);
    if (p.loop) {
        if (n_blocks > 1) return dfl_fail(ctx, DFLASH_ERR_UNSUPPORTED, "gemm_whole: a matrix of %d tiles takes one block of rows per call", p.n_units);
        const bool q6_ring = q6_tiled && kQ6LoopLds <= ctx->lds_bytes && env_int("DFLASH_Q6T_RING", 1);
        const kernel_t lf = p.kind == DFL_XF_Q4K ? gemm_whole_loop_kernel<Q4W>
                            : q6_ring            ? gemm_q6t_loop_kernel
                            : q6_tiled           ? gemm_whole_loop_kernel<Q6T>
                                                 : gemm_whole_loop_kernel<Q6W>;
        const size_t llds = q6_ring ? kQ6LoopLds
                                    : static_cast<size_t>(2) * 16 * 64 * sizeof(float4_t) +
                                          ((p.kind == DFL_XF_Q6K && !q6_tiled) ? static_cast<size_t>(16) * kQ6AreaBytes : 0);
        if (llds > ctx->lds_bytes) return dfl_fail(ctx, DFLASH_ERR_UNSUPPORTED, "gemm_whole: %zu bytes of LDS needed", llds);
        if (llds > 48 * 1024)
            if (const int32_t rc = dfl_raise_lds_limit(ctx, reinterpret_cast<const void *>(lf), llds)) return rc;
        dfl_timed timer(ctx, st, DFL_T_GEMM);
        lf<<<p.n_wg, 64 * p.ksplit * p.tl, llds, st>>>(a);
        DFL_HIP_CHECK(ctx, hipGetLastError());
        return DFLASH_OK;
    }
    const int multi = n_blocks > 1 ? (a.nb > p.ksplit ? 2 : 1) : 0;
#define DFL_WHOLE_PICK(WT, RR) (multi == 0 ? gemm_whole_kernel<WT, RR, 0> : multi == 1 ? gemm_whole_kernel<WT, RR, 1> : gemm_whole_kernel<WT, RR, 2>)
    const kernel_t fn = p.kind == DFL_XF_Q4K ? (p.R == 2 ? DFL_WHOLE_PICK(Q4W, 2) : DFL_WHOLE_PICK(Q4W, 1))
                        : q6_tiled           ? (p.R == 2 ? DFL_WHOLE_PICK(Q6T, 2) : DFL_WHOLE_PICK(Q6T, 1))
                                             : (p.R == 2 ? DFL_WHOLE_PICK(Q6W, 2) : DFL_WHOLE_PICK(Q6W, 1));
#undef DFL_WHOLE_PICK
    if (lds > ctx->lds_bytes) return dfl_fail(ctx, DFLASH_ERR_UNSUPPORTED, "gemm_whole: %zu bytes of LDS needed", lds);
    if (lds > 48 * 1024)
        if (const int32_t rc = dfl_raise_lds_limit(ctx, reinterpret_cast<const void *>(fn), lds)) return rc;
    dfl_timed timer(ctx, st, DFL_T_GEMM);
    fn<<<p.n_wg, threads, lds, st>>>(a);
    DFL_HIP_CHECK(ctx, hipGetLastError());
    return DFLASH_OK;
}

namespace {
// One thread per (row, super-block) of the tiled matrix: the row-order block's fields to their places (rows past the
// matrix: zero blocks, d = 0).
__global__ void __launch_bounds__(256)
    q6k_repack_tiled_kernel(const uint8_t *__restrict__ w, uint8_t *__restrict__ out, int n_out, int nb, int64_t n_items) {
    const int64_t i = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
    if (i >= n_items) return;
    const int b = static_cast<int>(i % nb);
    const int64_t row = i / nb;
    const int tile = static_cast<int>(row >> 4), r = static_cast<int>(row & 15);
    uint8_t *t = out + ((static_cast<size_t>(tile >> 4) * nb + b) * 16 + (tile & 15)) * kQ6TileBytes;
    const bool live = row < n_out;
    const uint8_t *src = w + (static_cast<size_t>(live ? row : 0) * nb + b) * DFL_Q6_K_BYTES;  // 2-byte aligned
    const uint16_t *s16 = reinterpret_cast<const uint16_t *>(src);
    auto put = [&](int dst_off, int src_off16) {  // one 16-byte piece
        uint16_t *d16 = reinterpret_cast<uint16_t *>(t + dst_off);
        for (int k = 0; k < 8; k++) d16[k] = live ? s16[src_off16 + k] : static_cast<uint16_t>(0);
    };
    for (int p = 0; p < 8; p++) put(q6t_ql_piece(r, p), 8 * p);
    for (int p = 0; p < 4; p++) put(q6t_qh_piece(r, p), 64 + 8 * p);
    put(kQ6TSc + r * 16, 96);
    *reinterpret_cast<uint16_t *>(t + kQ6TD + r * 2) = live ? s16[104] : static_cast<uint16_t>(0);
}
}  // namespace

extern "C" size_t dflash_q6k_tiled_bytes(int64_t n_in, int64_t n_out) {
    if (n_in <= 0 || n_out <= 0 || n_in % DFL_QK_K) return 0;
    const size_t groups = (static_cast<size_t>(n_out) + 255) / 256;
    return groups * static_cast<size_t>(n_in / DFL_QK_K) * 16 * kQ6TileBytes;
}

extern "C" int32_t dflash_repack_q6k_tiled(dflash_ctx *ctx, const void *w, void *w_tiled, int64_t n_in, int64_t n_out,
                                           dflash_stream_t stream) {
    if (!ctx) return DFLASH_ERR_INVALID_INPUT;
    if (!w || !w_tiled) return dfl_fail(ctx, DFLASH_ERR_INVALID_INPUT, "repack_q6k_tiled: null pointer");
    if (n_in <= 0 || n_out <= 0 || n_in % DFL_QK_K || n_in > 0x7fffffffll || n_out > 0x7fffffffll)
        return dfl_fail(ctx, DFLASH_ERR_BAD_SHAPE, "repack_q6k_tiled: n_in %lld / n_out %lld", static_cast<long long>(n_in),
                        static_cast<long long>(n_out));
    if (reinterpret_cast<uintptr_t>(w) % 2 || reinterpret_cast<uintptr_t>(w_tiled) % 128)
        return dfl_fail(ctx, DFLASH_ERR_ALIGNMENT, "repack_q6k_tiled: source must be 2-byte, destination 128-byte aligned");
    const size_t out_bytes = dflash_q6k_tiled_bytes(n_in, n_out);
    const int nb = static_cast<int>(n_in / DFL_QK_K);
    const size_t in_bytes = static_cast<size_t>(n_out) * nb * DFL_Q6_K_BYTES;
    if (dfl_ranges_overlap(w_tiled, out_bytes, w, in_bytes)) return dfl_fail(ctx, DFLASH_ERR_ALIAS, "repack_q6k_tiled: buffers overlap");
    // a tiled tensor goes to the fast kernels unconditionally: it must be one they can take
    if (const int32_t rc = dflash_check_scale_range(ctx, DFLASH_TYPE_Q6_K, w, in_bytes / DFL_Q6_K_BYTES, nullptr, stream)) return rc;
    const int64_t n_items = static_cast<int64_t>((static_cast<size_t>(n_out) + 255) / 256 * 256) * nb;
    const int64_t blocks = (n_items + 255) / 256;
    if (blocks > 0x7fffffffll) return dfl_fail(ctx, DFLASH_ERR_BAD_SHAPE, "repack_q6k_tiled: matrix too large");
    q6k_repack_tiled_kernel<<<static_cast<unsigned>(blocks), 256, 0, static_cast<hipStream_t>(stream)>>>(
        static_cast<const uint8_t *>(w), static_cast<uint8_t *>(w_tiled), static_cast<int>(n_out), nb, n_items);
    DFL_HIP_CHECK(ctx, hipGetLastError());
    return DFLASH_OK;
}

extern "C" size_t dflash_xf_bytes(int64_t n_in) { return n_in > 0 && n_in % DFL_QK_K == 0 ? dfl_xf_bytes(n_in) : 0; }

namespace {
// The public entries take a range-checked tensor only (there is no f32 kernel behind them): the tiled order, or
// DFLASH_TYPE_Q6_K | DFLASH_TYPE_RANGE_CHECKED.  Returns the bare type, or -1.
int32_t xf_public_type(int32_t w_type) {
    if (w_type == DFLASH_TYPE_Q4_K_TILED || w_type == DFLASH_TYPE_Q6_K_TILED) return w_type;
    if (w_type == (DFLASH_TYPE_Q6_K | DFLASH_TYPE_RANGE_CHECKED)) return DFLASH_TYPE_Q6_K;
    return -1;
}
}  // namespace

extern "C" int32_t dflash_gemm_fewrow_xf_kind(dflash_ctx *ctx, int32_t w_type, int64_t n_in, int64_t n_out) {
    const int32_t t = xf_public_type(w_type);
    return ctx && t >= 0 ? dfl_whole_kind(ctx, t, n_in, n_out, 0) : DFL_XF_NONE;
}

extern "C" int32_t dflash_pack_xf(dflash_ctx *ctx, const void *x, int32_t x_type, int32_t n_rows, int64_t n_in, int32_t kind,
                                  void *xf, dflash_stream_t stream) {
    if (!ctx) return DFLASH_ERR_INVALID_INPUT;
    if (!x || !xf || n_rows < 1 || n_rows > 16 || n_in <= 0 || n_in % DFL_QK_K || n_in > (1 << 24))
        return dfl_fail(ctx, DFLASH_ERR_BAD_SHAPE, "pack_xf: n_rows %d, n_in %lld", n_rows, static_cast<long long>(n_in));
    if (kind != DFL_XF_Q4K && kind != DFL_XF_Q6K) return dfl_fail(ctx, DFLASH_ERR_UNSUPPORTED, "pack_xf: kind %d", kind);
    if (x_type != DFLASH_TYPE_F32 && x_type != DFLASH_TYPE_F16) return dfl_fail(ctx, DFLASH_ERR_UNSUPPORTED, "pack_xf: x_type %d", x_type);
    if (reinterpret_cast<uintptr_t>(xf) % 16) return dfl_fail(ctx, DFLASH_ERR_ALIGNMENT, "pack_xf: xf must be 16-byte aligned");
    const size_t x_bytes = static_cast<size_t>(n_rows) * n_in * (x_type == DFLASH_TYPE_F32 ? 4 : 2);
    if (dfl_ranges_overlap(x, x_bytes, xf, dfl_xf_bytes(n_in))) return dfl_fail(ctx, DFLASH_ERR_ALIAS, "pack_xf: xf overlaps x");
    hipStream_t st = static_cast<hipStream_t>(stream);
    const dim3 grid(static_cast<unsigned>((n_in / 8 + 255) / 256), n_rows);
    if (x_type == DFLASH_TYPE_F32)
        pack_xf_kernel<float><<<grid, 256, 0, st>>>(static_cast<const float *>(x), n_rows, static_cast<int>(n_in), kind, static_cast<uint8_t *>(xf));
    else
        pack_xf_kernel<_Float16><<<grid, 256, 0, st>>>(static_cast<const _Float16 *>(x), n_rows, static_cast<int>(n_in), kind,
                                                     static_cast<uint8_t *>(xf));
    DFL_HIP_CHECK(ctx, hipGetLastError());
    return DFLASH_OK;
}

extern "C" int32_t dflash_gemm_fewrow_xf(dflash_ctx *ctx, int32_t w_type, const void *w, const void *xf, float *y, int64_t n_in,
                                         int64_t n_out, int32_t n_rows, dflash_stream_t stream) {
    if (!ctx) return DFLASH_ERR_INVALID_INPUT;
    const int32_t tagged = w_type;
    w_type = xf_public_type(tagged);
    if (w_type < 0)
        return dfl_fail(ctx, DFLASH_ERR_UNSUPPORTED,
                        "gemm_fewrow_xf: type tag %d: only DFLASH_TYPE_Q4_K_TILED, DFLASH_TYPE_Q6_K_TILED and DFLASH_TYPE_Q6_K | "
                        "DFLASH_TYPE_RANGE_CHECKED (a tensor that passed dflash_check_scale_range) are taken",
                        tagged);
    if (dfl_whole_kind(ctx, w_type, n_in, n_out, 0) == DFL_XF_NONE)
        return dfl_fail(ctx, DFLASH_ERR_UNSUPPORTED, "gemm_fewrow_xf: type %d, %lld -> %lld is not taken by the whole-K kernels", w_type,
                        static_cast<long long>(n_in), static_cast<long long>(n_out));
    if (n_in > 0 && n_out > 0 && y && xf && w) {
        const size_t wb = w_type == DFLASH_TYPE_Q4_K_TILED   ? dflash_q4k_tiled_bytes(n_in, n_out)
                          : w_type == DFLASH_TYPE_Q6_K_TILED ? dflash_q6k_tiled_bytes(n_in, n_out)
                                                             : dflash_row_bytes(w_type, n_in) * n_out;
        const size_t yb = static_cast<size_t>(n_rows > 0 ? n_rows : 1) * n_out * sizeof(float);
        if (dfl_ranges_overlap(y, yb, xf, dfl_xf_bytes(n_in)) || dfl_ranges_overlap(y, yb, w, wb))
            return dfl_fail(ctx, DFLASH_ERR_ALIAS, "gemm_fewrow_xf: y aliases an input");
    }
    return dfl_gemm_whole(ctx, w_type, w, xf, y, n_in, n_out, n_rows, 0, nullptr, DFL_XF_NONE, static_cast<hipStream_t>(stream));
}
