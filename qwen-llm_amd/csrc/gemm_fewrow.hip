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
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));

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

// Byte j of `v` (0..255) as an exact f16.
__device__ __forceinline__ _Float16 byte_to_half(uint32_t v, int j) {
    return static_cast<_Float16>(static_cast<float>((v >> (8 * j)) & 0xffu));
}

// One super-block of one output tile: 8 MFMAs.  hdr = {d|dmin, scales[0..3], [4..7], [8..11]},
// q0/q1 = the lane's 32 quant bytes (chunk g), a = this super-block's A fragments in LDS.
// A super-block slot past the end of a short stage (`live` false) holds a re-read of the last
// one; its scales are forced to zero so it adds nothing and the code stays straight-line.
// After every second MFMA the wave issues one load of a later stage (`next`, loads j0 ..): spread
// over the MFMAs, the loads never queue up behind each other in the address unit, which would
// otherwise stall all eight waves at once at the top of each stage.
struct Q4KIssue;
__device__ __forceinline__ void q4k_issue_one(const Q4KIssue &d, int j, int tid);

__device__ __forceinline__ float4_t q4k_block(u32x4_t hdr, u32x4_t q0, u32x4_t q1, const half8_t *a, int g,
                                              bool live, Q4KMagic magic, float4_t acc, const Q4KIssue &next, int j0,
                                              int tid) {
    // scales of sub-blocks 2g (low nibbles) and 2g+1 (high nibbles)
    uint32_t lo_sc = hdr.y & 0x3F3F3F3Fu;
    uint32_t hi_sc = (hdr.w & 0x0F0F0F0Fu) | ((hdr.y >> 2) & 0x30303030u);
    uint32_t sel = (g < 2 ? lo_sc : hi_sc) >> (16 * (g & 1));
    _Float16 d = live ? __builtin_bit_cast(half2_t, hdr.x)[0] : static_cast<_Float16>(0.0f);
    _Float16 s_lo = byte_to_half(sel, 0) * d;
    _Float16 s_hi = byte_to_half(sel, 1) * d;
    half2_t s2l = splat(s_lo), c2l = splat(s_lo * static_cast<_Float16>(-1024.0f));
    half2_t s2h = splat(s_hi), c2h = splat(s_hi * static_cast<_Float16>(-64.0f));
    uint32_t qw[8] = {q0.x, q0.y, q0.z, q0.w, q1.x, q1.y, q1.z, q1.w};
#pragma unroll
    for (int t = 0; t < 4; t++) {
        half8_t bl = unpack_scale<false>(qw[2 * t], qw[2 * t + 1], s2l, c2l, magic.lo);
        acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[t * 64], bl, acc, 0, 0, 0);
        if (t & 1) {
            q4k_issue_one(next, j0 + (t >> 1), tid);
            __builtin_amdgcn_sched_barrier(0);
        }
    }
#pragma unroll
    for (int t = 0; t < 4; t++) {
        half8_t bh = unpack_scale<true>(qw[2 * t], qw[2 * t + 1], s2h, c2h, magic.hi);
        acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[(4 + t) * 64], bh, acc, 0, 0, 0);
        if (t & 1) {
            q4k_issue_one(next, j0 + 2 + (t >> 1), tid);
            __builtin_amdgcn_sched_barrier(0);
        }
    }
    return acc;
}

// The eight dmin*m_j of one super-block as an MFMA B operand.
__device__ __forceinline__ half8_t q4k_mins(u32x4_t h, bool valid) {
    _Float16 dmin = valid ? __builtin_bit_cast(half2_t, h.x)[1] : static_cast<_Float16>(0.0f);
    uint32_t lo_m = h.z & 0x3F3F3F3Fu;
    uint32_t hi_m = ((h.w >> 4) & 0x0F0F0F0Fu) | ((h.z >> 2) & 0x30303030u);
    half8_t bm;
#pragma unroll
    for (int j = 0; j < 4; j++) {
        bm[j] = byte_to_half(lo_m, j) * dmin;
        bm[4 + j] = byte_to_half(hi_m, j) * dmin;
    }
    return bm;
}

// Streaming Q4_K kernel.
//
// Work split.  The iteration space is (tile group) x (super-block), flattened group-major; a
// tile group is kWavesQ4K consecutive output tiles, one per wave of a workgroup.  The grid is
// one workgroup per CU and workgroup i owns the contiguous range [T i / G, T (i+1) / G) of that
// space, so every CU streams the same number of weight bytes whatever the shape.
//
// Data path.  A workgroup walks its range in stages of up to kStage super-blocks that stay
// inside one tile group.  Per stage, the group's 128 weight rows (a row-contiguous slice of
// kStage*144 bytes each) and the prepared activations are copied global -> LDS by
// global_load_lds_dwordx4: consecutive lanes take consecutive 16-byte pieces, so HBM sees
// row-contiguous requests and no VGPR is held while a load is in flight.  The stages rotate
// through kBufs LDS buffers; the loads of stage j + kBufs - 1 are issued before stage j is
// computed, so HBM never idles.  Each wave issues exactly kLoadsPerStage load instructions per
// stage (surplus ones land in a spare LDS slot), which makes "stage j has landed" a constant
// s_waitcnt.  Waves then read their tile's quant bytes and A fragments with ds_read_b128.
//
// Split K.  When a range leaves a tile group, the accumulators are flushed: straight to Y if
// this workgroup covered the group's whole K, else as a partial tile whose every value carries
// the call's epoch tag in the same 8-byte store.  The highest-numbered workgroup that touches a
// group owns it: at the end of its own range it reads the group's partial tiles in workgroup
// order, polling each value until its tag is the current epoch, and writes Y.  No fences, no
// atomics, deterministic sums; a poll only ever waits for lower-numbered workgroups, which were
// dispatched first, and gives up (writing NaN) after a bounded number of tries.
constexpr int kStage = 2;
constexpr int kThreadsQ4K = 64 * kWavesQ4K;
constexpr int kGroupRows = 16 * kWavesQ4K;
constexpr int kRowPieces = 9 * kStage + 1;  // LDS row stride in pieces: one pad piece staggers the banks
constexpr int kStageWPieces = kGroupRows * kRowPieces;          // 16-byte pieces of weights per stage
constexpr int kStageXPieces = kStage * kQ4KBlockFrags;          // 16-byte pieces of activations per stage
constexpr int kBufPieces = kStageWPieces + kStageXPieces;       // one LDS buffer
constexpr int kWLoads = (kStageWPieces + kThreadsQ4K - 1) / kThreadsQ4K;
constexpr int kXLoads = (kStageXPieces + kThreadsQ4K - 1) / kThreadsQ4K;
constexpr int kLoadsPerStage = kWLoads + kXLoads;
constexpr uint32_t kSpinLimit = 1u << 22;

typedef const __attribute__((address_space(1))) void *gptr_t;
typedef __attribute__((address_space(3))) void *lptr_t;

// index of the workgroup whose range contains flattened iteration `it`
// (all of this index arithmetic fits 32 bits: the host checks total * n_wg < 2^31)
__device__ __forceinline__ int q4k_wg_of(int it, int total, int n_wg) {
    return static_cast<int>((static_cast<uint32_t>(it + 1) * n_wg + total - 1) / static_cast<uint32_t>(total)) - 1;
}

struct Q4KRange {
    int total, it_begin, it_end;
    int nb, n_wg, first_group;
};

__device__ __forceinline__ void q4k_stage_at(const Q4KRange &rg, int it, int &group, int &b, int &len) {
    group = static_cast<int>(static_cast<uint32_t>(it) / static_cast<uint32_t>(rg.nb));
    b = it - group * rg.nb;
    len = min(kStage, min(rg.nb - b, rg.it_end - it));
}

// Everything a wave needs to issue its kLoadsPerStage direct-to-LDS loads of one stage.
// `buf` is the stage's LDS buffer (kBufPieces pieces), `spare` a 1 KiB slot that absorbs the
// surplus loads of short stages.
struct Q4KIssue {
    const uint8_t *wbase;   // first super-block of the stage in weight row 0
    const half8_t *xsrc;    // the stage's prepared activations
    half8_t *buf, *spare;
    size_t row_bytes;
    int row0, n_out, ppr, n_x;
    bool on;
};

__device__ __forceinline__ Q4KIssue q4k_issue_desc(const uint8_t *__restrict__ w, const half8_t *__restrict__ xp,
                                                   half8_t *buf, half8_t *spare, int group, int b, int len,
                                                   int n_out, size_t row_bytes, bool on) {
    Q4KIssue d;
    d.wbase = w + static_cast<size_t>(b) * DFL_Q4_K_BYTES;
    d.xsrc = xp + static_cast<size_t>(b) * kQ4KBlockFrags;
    d.buf = buf;
    d.spare = spare;
    d.row_bytes = row_bytes;
    d.row0 = group * kGroupRows;
    d.n_out = n_out;
    d.ppr = 9 * len;  // real pieces per weight row; the rest of the row's kRowPieces re-read piece 0
    d.n_x = len * kQ4KBlockFrags;
    d.on = on;
    return d;
}

// Load number j (0 .. kLoadsPerStage-1) of the stage: kWLoads weight loads, then kXLoads
// activation loads.  Consecutive lanes take consecutive 16-byte pieces.
__device__ __forceinline__ void q4k_issue_one(const Q4KIssue &d, int j, int tid) {
    if (!d.on) return;
    const int lane = tid & 63, wave = tid >> 6;
    if (j < kWLoads) {
        const int p0 = (j * kWavesQ4K + wave) * 64;  // wave-uniform
        const int p = min(p0 + lane, kStageWPieces - 1);
        const int r = static_cast<int>(static_cast<uint32_t>(p) / static_cast<uint32_t>(kRowPieces));
        int o = p - r * kRowPieces;
        o = o < d.ppr ? o : 0;
        const int row = min(d.row0 + r, d.n_out - 1);
        const uint8_t *src = d.wbase + static_cast<size_t>(row) * d.row_bytes + o * 16;
        half8_t *dst = (p0 < kStageWPieces) ? d.buf + p0 : d.spare;
        __builtin_amdgcn_global_load_lds((gptr_t)(src), (lptr_t)(dst), 16, 0, 0);
    } else {
        const int p0 = ((j - kWLoads) * kWavesQ4K + wave) * 64;
        const int p = min(p0 + lane, d.n_x - 1);
        half8_t *dst = (p0 < d.n_x) ? d.buf + kStageWPieces + p0 : d.spare;
        __builtin_amdgcn_global_load_lds((gptr_t)(d.xsrc + p), (lptr_t)(dst), 16, 0, 0);
    }
}

__device__ __forceinline__ void q4k_issue_all(const Q4KIssue &d, int tid) {
#pragma unroll
    for (int j = 0; j < kLoadsPerStage; j++) q4k_issue_one(d, j, tid);
}

// One stage of MFMAs for this wave's tile, out of LDS buffer `buf`.
static_assert(kLoadsPerStage == 4 * kStage, "one load is issued after every second of a stage's 8*kStage MFMAs");

__device__ __forceinline__ void q4k_compute(const half8_t *buf, int len, int tid, Q4KMagic magic, float4_t &acc,
                                            float4_t &acc_min, const Q4KIssue &next) {
    const int lane = tid & 63, wave = tid >> 6, n = lane & 15, g = lane >> 4;
    const u32x4_t *wrow = reinterpret_cast<const u32x4_t *>(buf) + (wave * 16 + n) * kRowPieces;
    const half8_t *xbuf = buf + kStageWPieces;
#pragma unroll
    for (int u = 0; u < kStage; u++) {
        const int ub = min(u, len - 1);
        const u32x4_t *blk = wrow + ub * 9;
        acc = q4k_block(blk[0], blk[1 + 2 * g], blk[2 + 2 * g], xbuf + ub * kQ4KBlockFrags + lane, g, u < len, magic,
                        acc, next, 4 * u, tid);
    }
    // minima: lane (n, g) supplies super-block g of the stage
    const bool valid = g < len;
    const int gb = valid ? g : 0;
    half8_t bm = q4k_mins(wrow[gb * 9], valid);
    const half8_t *sums = xbuf + gb * kQ4KBlockFrags + 512 + n;
    acc_min = __builtin_amdgcn_mfma_f32_16x16x32_f16(sums[0], bm, acc_min, 0, 0, 0);
    acc_min = __builtin_amdgcn_mfma_f32_16x16x32_f16(sums[16], bm, acc_min, 0, 0, 0);
}

// s_waitcnt vmcnt(n) with the other counters left alone (gfx9 encoding: vmcnt low bits [3:0],
// high bits [15:14]; expcnt [6:4] and lgkmcnt [11:8] at their maxima)
constexpr int q4k_vmcnt(int n) { return ((n & 0xF) | ((n & 0x30) << 10)) | 0x0F70; }

struct Q4KTagged {
    float value;
    uint32_t tag;
};

// Ends a tile group's segment: Y directly if this workgroup covered the group's whole K, else a
// tagged partial tile.
__device__ __forceinline__ void q4k_flush(const Q4KRange &rg, int group, float4_t &acc, float4_t &acc_min,
                                          float *__restrict__ y, Q4KTagged *__restrict__ partials, uint32_t epoch,
                                          int n_out, int n_rows, int tid) {
    const int lane = tid & 63, wave = tid >> 6, n = lane & 15, g = lane >> 4;
    float4_t res = acc - acc_min;
    acc = float4_t{0, 0, 0, 0};
    acc_min = float4_t{0, 0, 0, 0};
    const int orow = (group * kWavesQ4K + wave) * 16 + n;
    const int wg_first = q4k_wg_of(group * rg.nb, rg.total, rg.n_wg);
    const int wg_last = q4k_wg_of((group + 1) * rg.nb - 1, rg.total, rg.n_wg);
    if (wg_first == wg_last) {
        if (orow < n_out) {
#pragma unroll
            for (int i = 0; i < 4; i++)
                if (4 * g + i < n_rows) y[static_cast<size_t>(4 * g + i) * n_out + orow] = res[i];
        }
        return;
    }
    const int slot = (group == rg.first_group) ? 0 : 1;
    Q4KTagged *p = partials + ((static_cast<size_t>(blockIdx.x) * 2 + slot) * kWavesQ4K + wave) * 256;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        Q4KTagged t = {res[i], epoch};
        __hip_atomic_store(reinterpret_cast<uint64_t *>(&p[(4 * g + i) * 16 + n]), __builtin_bit_cast(uint64_t, t),
                           __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
}

// Runs once, at the end of a workgroup's range: if its first tile group is split over several
// workgroups and this is the highest-numbered one, add the group's partial tiles in workgroup
// order and write Y.
__device__ __forceinline__ void q4k_reduce_owned(const Q4KRange &rg, float *__restrict__ y,
                                                 const Q4KTagged *__restrict__ partials, uint32_t epoch, int n_out,
                                                 int n_rows, int tid) {
    const int lane = tid & 63, wave = tid >> 6, n = lane & 15, g = lane >> 4;
    const int group = rg.first_group;
    const int wg_first = q4k_wg_of(group * rg.nb, rg.total, rg.n_wg);
    const int wg_last = q4k_wg_of((group + 1) * rg.nb - 1, rg.total, rg.n_wg);
    if (wg_first == wg_last || wg_last != static_cast<int>(blockIdx.x)) return;
    const int orow = (group * kWavesQ4K + wave) * 16 + n;
    if (orow >= n_out) return;
    float4_t sum = {0, 0, 0, 0};
    for (int wg = wg_first; wg <= wg_last; wg++) {
        const int wg_first_group = static_cast<int>(static_cast<uint32_t>(rg.total) * wg / rg.n_wg / rg.nb);
        const int slot = (group == wg_first_group) ? 0 : 1;
        const Q4KTagged *p = partials + ((static_cast<size_t>(wg) * 2 + slot) * kWavesQ4K + wave) * 256;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const uint64_t *src = reinterpret_cast<const uint64_t *>(&p[(4 * g + i) * 16 + n]);
            Q4KTagged t = __builtin_bit_cast(Q4KTagged, __hip_atomic_load(src, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
            for (uint32_t spin = 0; t.tag != epoch && spin < kSpinLimit; spin++) {
                __builtin_amdgcn_s_sleep(2);
                t = __builtin_bit_cast(Q4KTagged, __hip_atomic_load(src, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
            }
            sum[i] += (t.tag == epoch) ? t.value : __builtin_nanf("");
        }
    }
#pragma unroll
    for (int i = 0; i < 4; i++)
        if (4 * g + i < n_rows) y[static_cast<size_t>(4 * g + i) * n_out + orow] = sum[i];
}

template <int kBufs>
__global__ void __launch_bounds__(kThreadsQ4K)
    gemm_q4k_stream_kernel(const uint8_t *__restrict__ w, const half8_t *__restrict__ xp, float *__restrict__ y,
                           Q4KTagged *__restrict__ partials, uint32_t epoch, int n_out, int nb, int n_rows,
                           int n_groups) {
    extern __shared__ half8_t lds[];  // kBufs buffers of kBufPieces, then a 64-piece spare slot
    half8_t *spare = lds + kBufs * kBufPieces;

    const int tid = threadIdx.x;
    Q4KRange rg;
    rg.nb = nb;
    rg.n_wg = gridDim.x;
    rg.total = n_groups * nb;
    rg.it_begin = static_cast<int>(static_cast<uint32_t>(rg.total) * blockIdx.x / rg.n_wg);
    rg.it_end = static_cast<int>(static_cast<uint32_t>(rg.total) * (blockIdx.x + 1) / rg.n_wg);
    if (rg.it_begin >= rg.it_end) return;
    rg.first_group = static_cast<int>(static_cast<uint32_t>(rg.it_begin) / static_cast<uint32_t>(nb));
    const size_t row_bytes = static_cast<size_t>(nb) * DFL_Q4_K_BYTES;

    float4_t acc = {0, 0, 0, 0}, acc_min = {0, 0, 0, 0};
    const Q4KMagic magic = q4k_magic();

    // prologue: kBufs - 1 stages in flight
    int it_issue = rg.it_begin;  // next iteration to issue loads for
    int issued = 0;              // stages issued so far
#pragma unroll
    for (int s = 0; s < kBufs - 1; s++) {
        if (it_issue < rg.it_end) {
            int gi, bi, li;
            q4k_stage_at(rg, it_issue, gi, bi, li);
            q4k_issue_all(q4k_issue_desc(w, xp, lds + (issued % kBufs) * kBufPieces, spare, gi, bi, li, n_out,
                                         row_bytes, true),
                          tid);
            it_issue += li;
            issued++;
        }
    }
    int it = rg.it_begin;
    int done = 0;  // stages computed so far
    while (it < rg.it_end) {
        int gc, bc, lc;
        q4k_stage_at(rg, it, gc, bc, lc);
        // stage `done` has landed once at most (issued - done - 1) younger stages are in flight
        if (issued - done - 1 >= kBufs - 2 && kBufs > 2)
            __builtin_amdgcn_s_waitcnt(q4k_vmcnt((kBufs - 2) * kLoadsPerStage));
        else
            __builtin_amdgcn_s_waitcnt(q4k_vmcnt(0));
        // A bare barrier, not __syncthreads(): that one carries a workgroup-scope fence, which waits
        // for every load in flight and would undo the prefetch.  The s_waitcnt above is the only
        // ordering this needs: each wave's own pieces have landed before it arrives here.
        __builtin_amdgcn_s_barrier();  // the whole stage is in LDS; buffer (done-1) % kBufs is free
        // the stage kBufs-1 ahead is loaded into that free buffer while this one is computed
        const bool more = it_issue < rg.it_end;
        int gi = gc, bi = bc, li = lc;
        if (more) q4k_stage_at(rg, it_issue, gi, bi, li);
        const Q4KIssue next =
            q4k_issue_desc(w, xp, lds + (issued % kBufs) * kBufPieces, spare, gi, bi, li, n_out, row_bytes, more);
        q4k_compute(lds + (done % kBufs) * kBufPieces, lc, tid, magic, acc, acc_min, next);
        if (more) {
            it_issue += li;
            issued++;
        }
        it += lc;
        done++;
        int gn = gc;
        if (it < rg.it_end) gn = static_cast<int>(static_cast<uint32_t>(it) / static_cast<uint32_t>(nb));
        if (it >= rg.it_end || gn != gc) q4k_flush(rg, gc, acc, acc_min, y, partials, epoch, n_out, n_rows, tid);
    }
    q4k_reduce_owned(rg, y, partials, epoch, n_out, n_rows, tid);
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
        const int groups = (tiles + kWavesQ4K - 1) / kWavesQ4K;
        int n_wg = env_int("DFLASH_GEMM_WGS", ctx->n_cu);
        const int64_t total = static_cast<int64_t>(groups) * nb;
        if (n_wg > total) n_wg = static_cast<int>(total);
        if (n_wg > ctx->n_partial_wgs) n_wg = ctx->n_partial_wgs;
        if (n_wg < 1) n_wg = 1;
        if (total * (n_wg + 1) >= (int64_t(1) << 31))
            return dfl_fail(ctx, DFLASH_ERR_BAD_SHAPE, "gemm_fewrow: problem too large for 32-bit work indices");
        off = 0;
        xp = dfl_ws_take<half8_t>(ctx, &off, static_cast<size_t>(nb) * kQ4KBlockFrags * sizeof(half8_t));
        if (!xp) return dfl_fail(ctx, DFLASH_ERR_WORKSPACE, "gemm_fewrow: workspace too small");
        {
            dfl_timed timer(ctx, st, DFL_T_PREP);
            if (x_type == DFLASH_TYPE_F32)
                prep_x_q4k_kernel<float><<<nb, 256, 0, st>>>(static_cast<const float *>(x), xp, n_rows, n_in);
            else
                prep_x_q4k_kernel<_Float16><<<nb, 256, 0, st>>>(static_cast<const _Float16 *>(x), xp, n_rows, n_in);
        }
        // three LDS buffers when the device has the full 160 KiB per workgroup, else two
        const int bufs = env_int("DFLASH_GEMM_BUFS", ctx->lds_bytes >= (3 * kBufPieces + 64) * 16 ? 3 : 2);
        const size_t lds = static_cast<size_t>(bufs * kBufPieces + 64) * sizeof(half8_t);
        ctx->epoch += 1;
        if (ctx->epoch == 0) ctx->epoch = 1;
        Q4KTagged *partials = reinterpret_cast<Q4KTagged *>(ctx->tagged_partials);
        dfl_timed timer(ctx, st, DFL_T_GEMM);
        if (bufs == 3) {
            static bool attr3 = false;
            if (!attr3) {
                DFL_HIP_CHECK(ctx, hipFuncSetAttribute(reinterpret_cast<const void *>(gemm_q4k_stream_kernel<3>),
                                                       hipFuncAttributeMaxDynamicSharedMemorySize,
                                                       static_cast<int>(lds)));
                attr3 = true;
            }
            gemm_q4k_stream_kernel<3><<<n_wg, kThreadsQ4K, lds, st>>>(static_cast<const uint8_t *>(w), xp, y, partials,
                                                                      ctx->epoch, static_cast<int>(n_out), nb, n_rows,
                                                                      groups);
        } else {
            static bool attr2 = false;
            if (!attr2) {
                DFL_HIP_CHECK(ctx, hipFuncSetAttribute(reinterpret_cast<const void *>(gemm_q4k_stream_kernel<2>),
                                                       hipFuncAttributeMaxDynamicSharedMemorySize,
                                                       static_cast<int>(lds)));
                attr2 = true;
            }
            gemm_q4k_stream_kernel<2><<<n_wg, kThreadsQ4K, lds, st>>>(static_cast<const uint8_t *>(w), xp, y, partials,
                                                                      ctx->epoch, static_cast<int>(n_out), nb, n_rows,
                                                                      groups);
        }
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
