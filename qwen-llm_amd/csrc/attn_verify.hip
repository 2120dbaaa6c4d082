// Block-causal verify attention: the 16 draft rows of a block attend the whole prefix and
// each other causally, over an f16 KV cache, GQA.
//
// Replaces the reference's per-row loop (metal_dflash.rs:9963-10062: scatter one K/V row,
// then one single-query decode attention, sixteen times; kernels attn_v4.metal /
// attn.metal:266-336) with one pass that streams the KV cache once for all 16 rows:
//     o[i][h] = softmax(q[i][h] . K[0..L+i, kv(h)] * scale) . V[0..L+i, kv(h)]
//
// Mapping onto CDNA4 (split-KV flash decoding on MFMA):
//  * grid = (KV splits) x (KV heads); a workgroup owns one KV head and one contiguous chunk of
//    key positions; each of its waves owns one query head of the GQA group, i.e. a 16-row tile
//    (the block's rows are exactly the 16-wide side of v_mfma_f32_16x16x32_f16).
//  * K and V stream HBM -> LDS once per workgroup in stages of 32 keys (direct-to-LDS loads into a
//    ring of buffers, the next stages in flight while one is consumed), so the group's heads share
//    one copy; the K tile is bank-swizzled on the way in so that MFMA operand reads are conflict-free.
//  * scores are computed transposed, S^T = K . Q^T: K rows are the A operand, Q^T stays in
//    registers for the whole kernel (pre-multiplied by scale*log2(e), rounded to f16 as the
//    reference's decode kernel does, attn_v4.metal:20-31).  The result leaves every lane holding
//    one query row and eight consecutive keys of the stage, which is exactly the B operand of the
//    second product O^T = V^T . P^T, so probabilities never move between lanes.
//  * V is cached transposed, [kv head][dim][position]: the A operand of O^T wants 8 consecutive
//    positions of one dim, 16 contiguous bytes there.
//  * online softmax in base 2 on the lanes' own values; the running maximum is shared by the
//    four lanes of a row with two cross-lane exchanges per stage, the accumulator rescale is
//    skipped while no row's maximum moves, and stages every row sees in full skip the mask.
//  * each workgroup writes (m, l, O) partials; a second small kernel merges the splits.
#include "common.h"

#include <cmath>
#include <algorithm>
#include <cstdlib>

namespace {

typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
typedef float float4_t __attribute__((ext_vector_type(4)));

constexpr float kLog2e = 1.4426950408889634f;

// exchange with the lane 16 / 32 positions away (the other lanes that hold the same query row)
__device__ __forceinline__ float xor_lane(float v, int mask) {
    return __shfl_xor(v, mask, 64);
}

typedef const __attribute__((address_space(1))) void *gptr_t;
typedef __attribute__((address_space(3))) void *lptr_t;

constexpr int kAttnBufs = 3;  // LDS ring: stages in flight + the one being consumed (a fourth buffer measured the same)

// s_waitcnt vmcnt(n) with the other counters left alone (gfx9 encoding)
constexpr int attn_vmcnt(int n) { return ((n & 0xF) | ((n & 0x30) << 10)) | 0x0F70; }

// bank swizzle of the K tile: 16-byte chunk j of key row r sits at chunk j ^ swz(r), so that the
// eight key rows one MFMA operand read touches at a time land in eight different bank groups
__device__ __forceinline__ int attn_swz(int r) { return (r & 3) | ((r >> 1) & 4); }

// One workgroup = one KV head x one contiguous chunk of keys; wave w = query head w of the GQA
// group.  Stage = 32 keys: the K tile [32 keys][HD] and the V^T tile [HD dims][32 keys] are copied
// global -> LDS with direct-to-LDS loads into a ring of kAttnBufs buffers, so the whole group
// shares one copy and the loads of the next stages are in flight while this one is consumed.
// MAXW = most waves a workgroup may have; it sets the register budget.  HPW = query heads per wave:
// with two, every K and V^T fragment read from LDS feeds two MFMAs (half the LDS traffic per head,
// and two independent dependency chains per wave).
// Keys per KV split for n_pos visible positions: an even share of `want` splits, rounded up to
// whole 32-key stages, at least min_chunk.  Host and kernels use the same rule, so a launch whose
// context length is only known on the device (a captured graph) can size its grid for the largest
// context and let surplus workgroups leave.
__host__ __device__ __forceinline__ int64_t attn_chunk(int64_t n_pos, int64_t want, int64_t min_chunk) {
    int64_t chunk = (n_pos + want - 1) / want;
    chunk = (chunk + 31) / 32 * 32;
    return chunk < min_chunk ? min_chunk : chunk;
}

// eight consecutive query values (16-byte aligned) as floats
__device__ __forceinline__ void attn_load8(const float *p, float v[8]) {
    const float4_t a = *reinterpret_cast<const float4_t *>(p), b = *reinterpret_cast<const float4_t *>(p + 4);
#pragma unroll
    for (int i = 0; i < 4; i++) {
        v[i] = a[i];
        v[4 + i] = b[i];
    }
}
__device__ __forceinline__ void attn_load8(const _Float16 *p, float v[8]) {
    const half8_t a = *reinterpret_cast<const half8_t *>(p);
#pragma unroll
    for (int i = 0; i < 8; i++) v[i] = static_cast<float>(a[i]);
}

#ifdef DFLASH_TRACE
// Debug build only: per-workgroup time stamps (100 MHz constant clock).
__device__ unsigned long long *g_attn_trace = nullptr;  // [n_wg][16]
#define ATT_TR(i)                                                                                                   \
    do {                                                                                                            \
        if (threadIdx.x == 0 && g_attn_trace)                                                                       \
            g_attn_trace[(blockIdx.y * gridDim.x + blockIdx.x) * 16 + (i)] = wall_clock64();                        \
    } while (0)
#else
#define ATT_TR(i) \
    do {          \
    } while (0)
#endif

template <int HD, typename TQ, int MAXW, int HPW>
__global__ void __launch_bounds__(64 * MAXW)
    attn_split_kernel(const TQ *__restrict__ q, const _Float16 *__restrict__ k_cache,
                      const _Float16 *__restrict__ vt_cache, float *__restrict__ part_o, float *__restrict__ part_ml,
                      int64_t ctx_len, const int32_t *__restrict__ ctx_len_dev, int n_rows_total, int n_q, int n_kv,
                      int64_t vt_stride, int want, int min_chunk, float scale, int full_block, int64_t window,
                      int split_stride, int64_t part_slots) {
    // blockIdx.z: which block of sixteen query rows (a prefill group hands over many: block b's rows follow block
    // b - 1's in q and in the cache, its partial tiles sit part_slots slots further on)
    const int n_rows = min(16, n_rows_total - 16 * static_cast<int>(blockIdx.z));
    q += static_cast<int64_t>(blockIdx.z) * 16 * n_q * HD;
    part_o += static_cast<int64_t>(blockIdx.z) * part_slots * HD;
    part_ml += static_cast<int64_t>(blockIdx.z) * part_slots * 2;
    constexpr int KS = HD / 32;       // k-steps of the score product
    constexpr int DT = HD / 16;       // 16-dim tiles of the output
    constexpr int CH = HD / 8;        // 16-byte chunks per key row
    constexpr int kKPieces = 32 * CH; // pieces of the K tile; the V^T tile has as many
    constexpr int kWaveLoads = 2 * kKPieces / 64;
    extern __shared__ half8_t lds[];  // kAttnBufs x (K tile, V^T tile)
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int n_waves = blockDim.x >> 6;
    const int n = lane & 15, g = lane >> 4;
    const int group = n_q / n_kv;
    const int kvh = blockIdx.y;
    // blockIdx.x = split + split_stride * (part of the GQA group this workgroup serves); split_stride is a multiple
    // of 8, so the workgroups that read one chunk of keys are dispatched to the same XCD and share its L2 copy
    const int split = blockIdx.x % split_stride;
    const int head0 = kvh * group + ((blockIdx.x / split_stride) * n_waves + wave) * HPW;  // this wave serves heads head0 .. head0 + HPW - 1
    if (ctx_len_dev) ctx_len = *ctx_len_dev;
    ctx_len += 16 * static_cast<int64_t>(blockIdx.z);
    const int64_t n_pos = ctx_len + n_rows;
    const int64_t chunk = attn_chunk(n_pos, want, min_chunk);
    if (split * chunk >= n_pos) return;  // the grid is sized for the longest context
    const int64_t c0 = split * chunk;
    const int64_t c1 = min(n_pos, c0 + chunk);
    const int n_steps = static_cast<int>((c1 - c0 + 31) / 32);
    const int64_t kv_dim = static_cast<int64_t>(n_kv) * HD;
    const int per_wave = (kWaveLoads + n_waves - 1) / n_waves;  // loads each wave issues per stage
    ATT_TR(0);

    const uint8_t *kbytes = reinterpret_cast<const uint8_t *>(k_cache + static_cast<int64_t>(kvh) * HD);
    const uint8_t *vbytes = reinterpret_cast<const uint8_t *>(vt_cache + static_cast<int64_t>(kvh) * HD * vt_stride);
    // Stage `st` (keys c0 + 32 st ..) into ring buffer st % kAttnBufs: wave-load qd covers LDS pieces
    // 64 qd ..; this wave takes qd = j n_waves + wave, and loads past the end repeat earlier ones
    // (same bytes to the same place) so that every wave issues per_wave loads.  Key rows at or past
    // n_pos are never dereferenced: the last stage of the cache re-reads row n_pos - 1 instead (its
    // scores are masked and its V columns zeroed below).
    auto issue_stage = [&](int st) {
        const int64_t key0 = c0 + 32ll * st;
        half8_t *buf = lds + (st % kAttnBufs) * (2 * kKPieces);
        for (int j = 0; j < per_wave; j++) {
            const int qd = (j * n_waves + wave) % kWaveLoads;  // uniform
            const int p = qd * 64 + lane;
            const uint8_t *src;
            if (qd * 64 < kKPieces) {
                const int r = p / CH, jc = (p % CH) ^ attn_swz(r);
                const int64_t key = min(key0 + r, n_pos - 1);
                src = kbytes + key * kv_dim * 2 + jc * 16;
            } else {
                const int pv = p - kKPieces;
                src = vbytes + ((static_cast<int64_t>(pv >> 2) * vt_stride + key0 + 8 * (pv & 3)) * 2);
            }
            __builtin_amdgcn_global_load_lds((gptr_t)(src), (lptr_t)(buf + qd * 64), 16, 0, 0);
        }
    };

    // prologue: kAttnBufs - 1 stages in flight
    int issued = 0;
#pragma unroll
    for (int st = 0; st < kAttnBufs - 1; st++) {
        if (issued < n_steps) {
            issue_stage(issued);
            issued++;
        }
    }

    ATT_TR(1);
    // Q^T fragments: lane (row n, g) holds Q[n][head][32 s + 8 g ..+8] * scale * log2(e)
    // (rows at or past n_rows repeat the last row: they are never stored)
    half8_t qf[HPW][KS];
    {
        const float mult = scale * kLog2e;
        const int nq = min(n, n_rows - 1);
#pragma unroll
        for (int h = 0; h < HPW; h++) {
            const TQ *qrow = q + (static_cast<int64_t>(nq) * n_q + head0 + h) * HD + 8 * g;
#pragma unroll
            for (int s = 0; s < KS; s++) {
                float v[8];
                attn_load8(qrow + 32 * s, v);
#pragma unroll
                for (int i = 0; i < 8; i++) qf[h][s][i] = static_cast<_Float16>(v[i] * mult);
            }
        }
    }

    ATT_TR(2);
    float4_t acc[HPW][DT];
#pragma unroll
    for (int h = 0; h < HPW; h++)
#pragma unroll
        for (int t = 0; t < DT; t++) acc[h][t] = float4_t{0, 0, 0, 0};
    float m_run[HPW], l_run[HPW];  // running maximum of row n (base-2 logits, shared by its four lanes); this lane's share of the row sum
#pragma unroll
    for (int h = 0; h < HPW; h++) {
        m_run[h] = -INFINITY;
        l_run[h] = 0.0f;
    }
    // visible keys of row n, relative to c0: [lo, hi].  Block-causal: everything up to the row's own
    // position; full_block (drafter, non-causal): the whole block; a window keeps |distance| < window.
    const int64_t row_pos = ctx_len + n;
    int64_t hi64 = full_block ? n_pos - 1 : row_pos;
    int64_t lo64 = 0;
    if (window > 0) {
        lo64 = row_pos - window + 1;
        hi64 = min(hi64, row_pos + window - 1);
    }
    hi64 = min(hi64, c1 - 1);
    const int row_hi = static_cast<int>(max(min(hi64 - c0, static_cast<int64_t>(0x3fffffff)), static_cast<int64_t>(-1)));
    const int row_lo = static_cast<int>(max(min(lo64 - c0, static_cast<int64_t>(0x3fffffff)), static_cast<int64_t>(0)));
    // steps whose 32 keys are visible to every row need no masking: [all_lo, all_hi] in keys
    int all_hi = row_hi, all_lo = row_lo;
#pragma unroll
    for (int off = 1; off < 16; off <<= 1) {
        all_hi = min(all_hi, __shfl_xor(all_hi, off, 64));
        all_lo = max(all_lo, __shfl_xor(all_lo, off, 64));
    }
    all_hi = __builtin_amdgcn_readfirstlane(all_hi);
    all_lo = __builtin_amdgcn_readfirstlane(all_lo);

    const int rk0 = 8 * (n >> 2) + (n & 3);  // key row of S^T tile 0 this lane's A operand reads
    for (int st = 0; st < n_steps; st++) {
        if (issued - st - 1 >= kAttnBufs - 2) {
            // the loads of the kAttnBufs - 2 younger stages may still be in flight
            switch (per_wave * (kAttnBufs - 2)) {
                case 1: __builtin_amdgcn_s_waitcnt(attn_vmcnt(1)); break;
                case 2: __builtin_amdgcn_s_waitcnt(attn_vmcnt(2)); break;
                case 3: __builtin_amdgcn_s_waitcnt(attn_vmcnt(3)); break;
                case 4: __builtin_amdgcn_s_waitcnt(attn_vmcnt(4)); break;
                case 5: __builtin_amdgcn_s_waitcnt(attn_vmcnt(5)); break;
                case 6: __builtin_amdgcn_s_waitcnt(attn_vmcnt(6)); break;
                case 8: __builtin_amdgcn_s_waitcnt(attn_vmcnt(8)); break;
                case 10: __builtin_amdgcn_s_waitcnt(attn_vmcnt(10)); break;
                case 12: __builtin_amdgcn_s_waitcnt(attn_vmcnt(12)); break;
                case 16: __builtin_amdgcn_s_waitcnt(attn_vmcnt(16)); break;
                case 32: __builtin_amdgcn_s_waitcnt(attn_vmcnt(32)); break;
                default: __builtin_amdgcn_s_waitcnt(attn_vmcnt(0)); break;
            }
        } else {
            __builtin_amdgcn_s_waitcnt(attn_vmcnt(0));
        }
        __builtin_amdgcn_s_barrier();  // stage st is in LDS for everyone; buffer (st - 1) % kAttnBufs is free
        if (issued < n_steps) {
            issue_stage(issued);
            issued++;
        }
        const half8_t *kt = lds + (st % kAttnBufs) * (2 * kKPieces);
        const half8_t *vt = kt + kKPieces;
        const int key0 = 32 * st;  // relative to c0

        float4_t sc[HPW][2];
#pragma unroll
        for (int T = 0; T < 2; T++) {
            const int r = rk0 + 4 * T;
            const int sw = attn_swz(r);
#pragma unroll
            for (int h = 0; h < HPW; h++) sc[h][T] = float4_t{0, 0, 0, 0};
#pragma unroll
            for (int s = 0; s < KS; s++) {
                const half8_t kf = kt[r * CH + ((4 * s + g) ^ sw)];
#pragma unroll
                for (int h = 0; h < HPW; h++) sc[h][T] = __builtin_amdgcn_mfma_f32_16x16x32_f16(kf, qf[h][s], sc[h][T], 0, 0, 0);
            }
        }
        const bool masked = !(key0 >= all_lo && key0 + 31 <= all_hi);  // uniform: some key of this step is hidden from some row
        half8_t pf[HPW];
#pragma unroll
        for (int h = 0; h < HPW; h++) {
            float p[8];
#pragma unroll
            for (int i = 0; i < 8; i++) p[i] = (i < 4) ? sc[h][0][i] : sc[h][1][i - 4];
            if (masked) {
#pragma unroll
                for (int i = 0; i < 8; i++) {
                    const int key = key0 + 8 * g + i;
                    p[i] = (key >= row_lo && key <= row_hi) ? p[i] : -INFINITY;
                }
            }
            float mx = fmaxf(fmaxf(fmaxf(p[0], p[1]), fmaxf(p[2], p[3])), fmaxf(fmaxf(p[4], p[5]), fmaxf(p[6], p[7])));
            mx = fmaxf(mx, xor_lane(mx, 16));
            mx = fmaxf(mx, xor_lane(mx, 32));
            const float m_new = fmaxf(m_run[h], mx);
            // all keys of this step masked for this row and nothing seen before: keep the state
            const float m_safe = (m_new == -INFINITY) ? 0.0f : m_new;
            const float alpha = __builtin_amdgcn_exp2f(m_run[h] - m_safe);  // 0 when m_run = -inf
            float psum = 0.0f;
#pragma unroll
            for (int i = 0; i < 8; i++) {
                p[i] = __builtin_amdgcn_exp2f(p[i] - m_safe);
                psum += p[i];
            }
            l_run[h] = l_run[h] * alpha + psum;
            if (__builtin_amdgcn_ballot_w64(alpha != 1.0f) != 0) {
#pragma unroll
                for (int t = 0; t < DT; t++) acc[h][t] *= alpha;
            }
            m_run[h] = m_new;
#pragma unroll
            for (int i = 0; i < 8; i++) pf[h][i] = static_cast<_Float16>(p[i]);
        }
        // O^T tile t (dims 16 t ..): A = V^T[dim 16 t + n][keys key0 + 8 g ..+8].  Columns at or past
        // n_pos hold whatever the cache held before (possibly NaN patterns; 0 * NaN would poison
        // the accumulator): zero them in the last stage of the cache
        const int64_t vkey = c0 + key0 + 8 * g;
        const bool tail = c0 + key0 + 32 > n_pos;
#pragma unroll
        for (int t = 0; t < DT; t++) {
            half8_t vf = vt[(16 * t + n) * 4 + g];
            if (tail) {
#pragma unroll
                for (int i = 0; i < 8; i++)
                    if (vkey + i >= n_pos) vf[i] = static_cast<_Float16>(0.0f);
            }
#pragma unroll
            for (int h = 0; h < HPW; h++) acc[h][t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(vf, pf[h], acc[h][t], 0, 0, 0);
        }
        if (st < 8) ATT_TR(3 + st);
    }
    ATT_TR(12);

    // row sums over the four lanes of a row; partials: O^T tile t, lane (row n, g) holds dims 16 t + 4 g + i
#pragma unroll
    for (int h = 0; h < HPW; h++) {
        float l = l_run[h];
        l += xor_lane(l, 16);
        l += xor_lane(l, 32);
        if (n < n_rows) {
            const int64_t slot = (static_cast<int64_t>(split) * n_q + head0 + h) * 16 + n;
            float *po = part_o + slot * HD;
#pragma unroll
            for (int t = 0; t < DT; t++) *reinterpret_cast<float4_t *>(po + 16 * t + 4 * g) = acc[h][t];
            if (g == 0) {
                part_ml[slot * 2] = m_run[h];
                part_ml[slot * 2 + 1] = l;
            }
        }
    }
    ATT_TR(13);
}

#ifdef DFLASH_TRACE
}  // namespace
extern "C" void dflash_dbg_set_attn_trace(uint64_t p) {
    unsigned long long *v = reinterpret_cast<unsigned long long *>(p);
    (void)hipMemcpyToSymbol(HIP_SYMBOL(g_attn_trace), &v, sizeof(v));
}
namespace {
#endif

// out[row][head][:] = sum_s 2^(m_s - m*) O_s / sum_s 2^(m_s - m*) l_s
// One workgroup per (head, row): 256 threads = 8 split lanes x 32 dim lanes; a split lane adds up
// every eighth split (float4 per dim lane, all loads independent), then the eight are summed in LDS.
__global__ void __launch_bounds__(256)
    attn_combine_kernel(const float *__restrict__ part_o, const float *__restrict__ part_ml, float *__restrict__ out,
                        int n_rows_total, int n_q, int hd, int64_t ctx_len, const int32_t *__restrict__ ctx_len_dev, int want,
                        int min_chunk, void *__restrict__ out_xf, int out_xf_kind, int64_t part_slots, size_t xf_stride) {
    // blockIdx.z: which block of sixteen rows (see attn_split_kernel); rows past a short last block leave
    const int n_rows = min(16, n_rows_total - 16 * static_cast<int>(blockIdx.z));
    if (static_cast<int>(blockIdx.y) >= n_rows) return;
    part_o += static_cast<int64_t>(blockIdx.z) * part_slots * hd;
    part_ml += static_cast<int64_t>(blockIdx.z) * part_slots * 2;
    out += static_cast<int64_t>(blockIdx.z) * 16 * n_q * hd;
    if (out_xf) out_xf = static_cast<uint8_t *>(out_xf) + blockIdx.z * xf_stride;
    if (ctx_len_dev) ctx_len = *ctx_len_dev;
    ctx_len += 16 * static_cast<int64_t>(blockIdx.z);
    const int64_t n_pos = ctx_len + n_rows;
    const int64_t chunk = attn_chunk(n_pos, want, min_chunk);
    const int n_splits = static_cast<int>((n_pos + chunk - 1) / chunk);
    __shared__ float wgt[1024];          // 2^(m_s - m*) per split (n_splits <= 1024)
    __shared__ float red[8][256 + 4];    // partial outputs per split lane
    __shared__ float red_l[8];
    const int head = blockIdx.x, row = blockIdx.y;
    const int tid = threadIdx.x;
    const int64_t slot0 = static_cast<int64_t>(head) * 16 + row;
    const int64_t slot_stride = static_cast<int64_t>(n_q) * 16;
    // m* = max over splits (a thread keeps the maxima it loaded: n_splits <= 1024 = 4 per thread)
    float m_own[4];
#pragma unroll
    for (int j = 0; j < 4; j++) {
        const int s = tid + 256 * j;
        m_own[j] = s < n_splits ? part_ml[(slot0 + s * slot_stride) * 2] : -INFINITY;
    }
    // The partial outputs of the first kPre rounds of splits are asked for right behind the maxima, before those are
    // waited for: their addresses do not depend on the weights, so the two trips to memory are in flight together
    // instead of one behind the other across two barriers (the maxima first: loads return in the order of their issue,
    // and the maxima are what the first reduction needs).  The sums below take them in the order of the loop that follows.
    constexpr int kPre = 4;
    const int sl = tid >> 5, dl = tid & 31;  // split lane, dim lane
    const int n_vec = hd / 4;                // float4 per row: 16, 32 or 64
    float4_t pre0[kPre], pre1[kPre];
    float pre_l[kPre];
#pragma unroll
    for (int i = 0; i < kPre; i++) {
        const int s = sl + 8 * i;
        pre0[i] = float4_t{0, 0, 0, 0};
        pre1[i] = float4_t{0, 0, 0, 0};
        pre_l[i] = 0.0f;
        if (s < n_splits) {
            const float4_t *po = reinterpret_cast<const float4_t *>(part_o + (slot0 + s * slot_stride) * hd);
            if (dl < n_vec) pre0[i] = po[dl];
            if (dl + 32 < n_vec) pre1[i] = po[dl + 32];
            if (dl == 0) pre_l[i] = part_ml[(slot0 + s * slot_stride) * 2 + 1];
        }
    }
    float m_loc = fmaxf(fmaxf(m_own[0], m_own[1]), fmaxf(m_own[2], m_own[3]));
    for (int off = 32; off > 0; off >>= 1) m_loc = fmaxf(m_loc, __shfl_xor(m_loc, off, 64));
    if ((tid & 63) == 0) red_l[tid >> 6] = m_loc;
    __syncthreads();
    const float m_star = fmaxf(fmaxf(red_l[0], red_l[1]), fmaxf(red_l[2], red_l[3]));
#pragma unroll
    for (int j = 0; j < 4; j++) {
        const int s = tid + 256 * j;
        if (s < n_splits) wgt[s] = (m_own[j] == -INFINITY) ? 0.0f : exp2f(m_own[j] - m_star);
    }
    __syncthreads();  // (also: every thread has read red_l before the split lanes write their sums into it)
    float4_t acc0 = {0, 0, 0, 0}, acc1 = {0, 0, 0, 0};
    float l = 0.0f;
#pragma unroll
    for (int i = 0; i < kPre; i++) {
        const int s = sl + 8 * i;
        if (s < n_splits) {
            const float w = wgt[s];
            if (dl < n_vec) acc0 += w * pre0[i];
            if (dl + 32 < n_vec) acc1 += w * pre1[i];
            if (dl == 0) l += w * pre_l[i];
        }
    }
    for (int s = sl + 8 * kPre; s < n_splits; s += 8) {
        const float w = wgt[s];
        const float4_t *po = reinterpret_cast<const float4_t *>(part_o + (slot0 + s * slot_stride) * hd);
        if (dl < n_vec) acc0 += w * po[dl];
        if (dl + 32 < n_vec) acc1 += w * po[dl + 32];
        if (dl == 0) l += w * part_ml[(slot0 + s * slot_stride) * 2 + 1];
    }
#pragma unroll
    for (int i = 0; i < 4; i++) {
        red[sl][4 * dl + i] = acc0[i];
        red[sl][128 + 4 * dl + i] = acc1[i];
    }
    if (dl == 0) red_l[sl] = l;
    __syncthreads();
    float lsum = 0.0f;
#pragma unroll
    for (int k = 0; k < 8; k++) lsum += red_l[k];
    for (int d = tid; d < hd; d += 256) {
        float o = 0.0f;
#pragma unroll
        for (int k = 0; k < 8; k++) o += red[k][d];
        o /= lsum;
        out[(static_cast<int64_t>(row) * n_q + head) * hd + d] = o;
        if (out_xf) {
            // eight consecutive dims sit in eight consecutive lanes of one wave (hd is a multiple of 64)
            float v[8];
#pragma unroll
            for (int i = 0; i < 8; i++) v[i] = __shfl_down(o, i, 64);
            if ((d & 7) == 0) dfl_xf_store(out_xf, out_xf_kind, row, head * hd + d, v[0], v[1], v[2], v[3], v[4], v[5], v[6], v[7]);
        }
    }
}

// V [pos][n_kv][hd] -> V^T [n_kv][hd][stride]; one workgroup per (32 positions, kv head)
__global__ void __launch_bounds__(256) transpose_v_kernel(const _Float16 *__restrict__ v, _Float16 *__restrict__ vt,
                                                          int64_t n_pos, int n_kv, int hd, int64_t stride) {
    __shared__ _Float16 tile[32][256 + 2];
    const int64_t p0 = static_cast<int64_t>(blockIdx.x) * 32;
    const int kvh = blockIdx.y;
    for (int e = threadIdx.x; e < 32 * hd; e += blockDim.x) {
        int pl = e / hd, d = e - pl * hd;
        int64_t pos = p0 + pl;
        tile[pl][d] = pos < n_pos ? v[(pos * n_kv + kvh) * hd + d] : static_cast<_Float16>(0.0f);
    }
    __syncthreads();
    for (int e = threadIdx.x; e < 32 * hd; e += blockDim.x) {
        int d = e >> 5, pl = e & 31;
        int64_t pos = p0 + pl;
        if (pos < stride) vt[(static_cast<int64_t>(kvh) * hd + d) * stride + pos] = tile[pl][d];
    }
}

template <int HD, typename TQ>
int32_t launch_split(dflash_ctx *ctx, dim3 grid, int threads, hipStream_t st, const void *q, const _Float16 *k, const _Float16 *vt,
                  float *po, float *pml, int64_t ctx_len, const int32_t *ctx_len_dev, int n_rows, int n_q, int n_kv,
                  int64_t vt_stride, int want, int min_chunk, float scale, int full_block, int64_t window, int split_stride,
                  int64_t part_slots) {
    const size_t lds = static_cast<size_t>(kAttnBufs) * 2 * (32 * HD / 8) * sizeof(half8_t);
#define DFL_ATTN_LAUNCH(MAXW, HPW)                                                                                  \
    do {                                                                                                            \
        if (const int32_t rc_ = dfl_raise_lds_limit(ctx, reinterpret_cast<const void *>(attn_split_kernel<HD, TQ, MAXW, HPW>), lds)) \
            return rc_;                                                                                             \
        attn_split_kernel<HD, TQ, MAXW, HPW><<<grid, threads / HPW, lds, st>>>(static_cast<const TQ *>(q), k, vt, po, pml, \
                                                                              ctx_len, ctx_len_dev, n_rows, n_q, n_kv, \
                                                                              vt_stride, want, min_chunk, scale,    \
                                                                              full_block, window, split_stride, part_slots); \
    } while (0)
    // one head per wave: two (HPW = 2) halve the LDS reads per head but measured slower on MI355X
    // (fewer waves to hide the per-stage dependency chain)
    if (threads <= 512)
        DFL_ATTN_LAUNCH(8, 1);
    else
        DFL_ATTN_LAUNCH(16, 1);
#undef DFL_ATTN_LAUNCH
    return DFLASH_OK;
}

}  // namespace

extern "C" int32_t dflash_attn_verify_block(dflash_ctx *ctx, const void *q, int32_t q_type, const void *k_cache,
                                            const void *v_cache, int32_t v_layout, int64_t ctx_len, int32_t n_rows,
                                            int32_t n_q, int32_t n_kv, int32_t head_dim, int64_t kv_capacity,
                                            float scale, float *out, dflash_stream_t stream) {
    return dfl_attn_block(ctx, q, q_type, k_cache, v_cache, v_layout, ctx_len, n_rows, n_q, n_kv, head_dim, kv_capacity,
                          scale, out, stream, 0, 0, nullptr);
}

// n_rows_total rows, sixteen to a block (every block in the same bucket of context lengths: the caller's business);
// max_blocks_out: how many blocks the workspace holds partial tiles for (the caller launches the rest in further runs).
static int32_t attn_rows(dflash_ctx *ctx, const void *q, int32_t q_type, const void *k_cache, const void *v_cache,
                         int32_t v_layout, int64_t ctx_len, int32_t n_rows_total, int32_t n_q, int32_t n_kv, int32_t head_dim,
                         int64_t kv_capacity, float scale, float *out, dflash_stream_t stream, int32_t full_block,
                         int64_t window, const int32_t *ctx_len_dev, void *out_xf, int out_xf_kind, int32_t *blocks_done);

int32_t dfl_attn_block(dflash_ctx *ctx, const void *q, int32_t q_type, const void *k_cache, const void *v_cache,
                       int32_t v_layout, int64_t ctx_len, int32_t n_rows, int32_t n_q, int32_t n_kv, int32_t head_dim,
                       int64_t kv_capacity, float scale, float *out, dflash_stream_t stream, int32_t full_block,
                       int64_t window, const int32_t *ctx_len_dev, void *out_xf, int out_xf_kind) {
    if (!ctx) return DFLASH_ERR_INVALID_INPUT;
    if (n_rows < 1 || n_rows > 16) return dfl_fail(ctx, DFLASH_ERR_BAD_SHAPE, "attn_verify: n_rows %d outside 1..16", n_rows);
    return attn_rows(ctx, q, q_type, k_cache, v_cache, v_layout, ctx_len, n_rows, n_q, n_kv, head_dim, kv_capacity, scale, out, stream,
                     full_block, window, ctx_len_dev, out_xf, out_xf_kind, nullptr);
}

int32_t dfl_attn_blocks(dflash_ctx *ctx, const void *q, int32_t q_type, const void *k_cache, const void *vt_cache, int64_t ctx_len,
                        int32_t n_rows_total, int32_t n_q, int32_t n_kv, int32_t head_dim, int64_t kv_capacity, float scale,
                        float *out, dflash_stream_t stream, void *out_xf, int out_xf_kind) {
    if (!ctx) return DFLASH_ERR_INVALID_INPUT;
    if (n_rows_total < 1) return dfl_fail(ctx, DFLASH_ERR_BAD_SHAPE, "attn_verify: %d rows", n_rows_total);
    const size_t q_block = static_cast<size_t>(16) * n_q * head_dim;
    const size_t xf_block = dfl_xf_bytes(static_cast<int64_t>(n_q) * head_dim);
    const size_t q_el = q_type == DFLASH_TYPE_F16 ? 2 : 4;
    int32_t done = 0;
    const int32_t n_blocks = (n_rows_total + 15) / 16;
    while (done < n_blocks) {
        // a run: the blocks from `done` on that share its bucket (the split policy is a function of the bucket)
        const int64_t len0 = ctx_len + 16ll * done;
        const int64_t bucket = dfl_attn_bucket(len0 + std::min(16, n_rows_total - 16 * done));
        int32_t run = 1;
        while (done + run < n_blocks &&
               dfl_attn_bucket(ctx_len + 16ll * (done + run) + std::min(16, n_rows_total - 16 * (done + run))) == bucket)
            run++;
        const int32_t rows = std::min(n_rows_total - 16 * done, 16 * run);
        int32_t taken = 0;
        const int32_t rc = attn_rows(ctx, static_cast<const uint8_t *>(q) + done * q_block * q_el, q_type, k_cache, vt_cache, 1, len0, rows,
                                     n_q, n_kv, head_dim, kv_capacity, scale, out + done * q_block, stream, 0, 0, nullptr,
                                     out_xf ? static_cast<uint8_t *>(out_xf) + done * xf_block : nullptr, out_xf_kind, &taken);
        if (rc) return rc;
        done += taken;
    }
    return DFLASH_OK;
}

static int32_t attn_rows(dflash_ctx *ctx, const void *q, int32_t q_type, const void *k_cache, const void *v_cache,
                         int32_t v_layout, int64_t ctx_len, int32_t n_rows_total, int32_t n_q, int32_t n_kv, int32_t head_dim,
                         int64_t kv_capacity, float scale, float *out, dflash_stream_t stream, int32_t full_block,
                         int64_t window, const int32_t *ctx_len_dev, void *out_xf, int out_xf_kind, int32_t *blocks_done) {
    int32_t n_blocks = (n_rows_total + 15) / 16;
    const int32_t n_rows = std::min(16, n_rows_total);  // rows of the first block: what the split policy looks at
    if (n_blocks > 1 && (v_layout != 1 || ctx_len_dev))
        return dfl_fail(ctx, DFLASH_ERR_UNSUPPORTED, "attn_verify: several blocks need the transposed V cache and a host-side context length");
    if (out_xf && ((n_q * head_dim) % DFL_QK_K || reinterpret_cast<uintptr_t>(out_xf) % 16 ||
                   (out_xf_kind != DFL_XF_Q4K && out_xf_kind != DFL_XF_Q6K)))
        return dfl_fail(ctx, DFLASH_ERR_BAD_SHAPE, "attn_verify: fragment-order output needs n_q * head_dim %% 256 == 0 and a kind");
    if (!q || !k_cache || !v_cache || !out) return dfl_fail(ctx, DFLASH_ERR_INVALID_INPUT, "attn_verify: null pointer");
    if (n_q < 1 || n_kv < 1 || n_q % n_kv || n_q / n_kv > 16)
        return dfl_fail(ctx, DFLASH_ERR_BAD_SHAPE, "attn_verify: %d query heads over %d KV heads (group must be 1..16)",
                        n_q, n_kv);
    if (head_dim != 64 && head_dim != 128 && head_dim != 256)
        return dfl_fail(ctx, DFLASH_ERR_UNSUPPORTED, "attn_verify: head_dim %d (64, 128, 256 supported)", head_dim);
    if (ctx_len < 0 || ctx_len + n_rows_total > kv_capacity)
        return dfl_fail(ctx, DFLASH_ERR_STATE, "attn_verify: context %lld + %d rows exceeds the cache capacity %lld",
                        static_cast<long long>(ctx_len), n_rows_total, static_cast<long long>(kv_capacity));
    if (q_type != DFLASH_TYPE_F32 && q_type != DFLASH_TYPE_F16)
        return dfl_fail(ctx, DFLASH_ERR_UNSUPPORTED, "attn_verify: queries must be f32 or f16");
    if (v_layout != 0 && v_layout != 1) return dfl_fail(ctx, DFLASH_ERR_INVALID_INPUT, "attn_verify: v_layout");
    if (ctx_len_dev && v_layout != 1)
        return dfl_fail(ctx, DFLASH_ERR_UNSUPPORTED, "attn_verify: a device-side context length needs the transposed V cache");
    if (v_layout == 1 && kv_capacity % 32)
        return dfl_fail(ctx, DFLASH_ERR_ALIGNMENT, "attn_verify: transposed V needs a capacity that is a multiple of 32");
    if (reinterpret_cast<uintptr_t>(q) % 16 || reinterpret_cast<uintptr_t>(k_cache) % 16 ||
        reinterpret_cast<uintptr_t>(v_cache) % 16 || reinterpret_cast<uintptr_t>(out) % 16)
        return dfl_fail(ctx, DFLASH_ERR_ALIGNMENT, "attn_verify: Q, K, V and the output must be 16-byte aligned");

    hipStream_t st = static_cast<hipStream_t>(stream);
    const int group = n_q / n_kv;
    // with ctx_len_dev the context length is read on the device: everything sized here is then sized for the
    // largest context of the bucket
    const int64_t bucket = dfl_attn_bucket(ctx_len + n_rows);
    // (several blocks: sized for the last one, which sees the most keys)
    int64_t n_pos = ctx_len_dev ? std::min<int64_t>(kv_capacity, 2 * bucket - 1) : ctx_len + n_rows_total;

    // KV splits: enough workgroups to cover the chip once or twice, chunks a multiple of 32 keys and at least
    // min_chunk keys long (a split costs a partial tile per head and row).  The policy is a function of the
    // bucket alone.
    // Workgroups per CU the split aims at, in halves.  Short contexts: one (fewer splits, fewer partial tiles to merge).
    // Long contexts: two where two workgroups' LDS rings fit a CU side by side (heads of 64 or 128); with heads of 256 a
    // ring is 96 KB, a CU holds one workgroup, and a second round of them only halves the chunk: a workgroup's partial
    // tiles (16 rows x its heads x head_dim floats) are then as many bytes as the keys and values it read.  Half a
    // workgroup per CU there (16 q / 2 kv heads of 256, 40-layer verify: 5.25 -> 4.79 ms at 16 k of context with chunks
    // of 256 keys instead of 128, 6.21 -> 5.80 ms at 32 k with 512; a quarter measured slower again).
    const size_t ring_bytes = static_cast<size_t>(kAttnBufs) * 2 * 32 * head_dim * sizeof(_Float16);
    int per_cu_x2 = bucket >= 16384 ? (2 * ring_bytes <= static_cast<size_t>(ctx->lds_bytes) ? 4 : 1) : 2;
    int64_t min_chunk = bucket >= 8192 ? 128 : 64;
    // A workgroup serves hw heads of a GQA group (one wave each).  What a workgroup moves is its chunk of K and V,
    // its heads' queries and their partial outputs, and one CU takes in only 20-30 KB per microsecond: at short
    // contexts, where whole groups would leave most CUs without a workgroup, the group is divided until the chip
    // is covered (the chunk is then read by group / hw workgroups, of one XCD).
    // (Measured on the 16 q / 2 kv head shape of 256, 40-layer verify: covering half the chip is enough - 4 heads per
    // workgroup at 2 k of context, 2 at 1 k: 4.19 against 4.24 ms and 4.35 against 4.57 ms - but eight waves on one chunk
    // are too many - at 4-8 k, 4 heads per workgroup: 4.75 against 4.81 ms, 4.20 against 4.28 ms.)
    static const int env_cover_div = [] { const char *e = getenv("DFLASH_ATTN_COVER_DIV"); return e ? atoi(e) : 0; }();
    const int cover_div = env_cover_div > 0 ? env_cover_div : 2;
    int hw = group;
    if (cover_div > 1 && group % 4 == 0 && group > 4 && bucket < 16384) hw = 4;
    while (hw % 2 == 0 && static_cast<int64_t>(n_kv) * (group / hw) * ((bucket + min_chunk - 1) / min_chunk) < ctx->n_cu / cover_div) hw /= 2;
    // tuning knobs, read once per process
    static const int env_per_cu = [] { const char *e = getenv("DFLASH_ATTN_PER_CU"); return e ? atoi(e) : 0; }();
    static const int env_min_chunk = [] { const char *e = getenv("DFLASH_ATTN_MIN_CHUNK"); return e ? atoi(e) : 0; }();
    static const int env_hw = [] { const char *e = getenv("DFLASH_ATTN_HW"); return e ? atoi(e) : 0; }();
    if (env_per_cu > 0) per_cu_x2 = 2 * env_per_cu;
    if (env_min_chunk > 0) min_chunk = env_min_chunk;
    if (env_hw > 0 && group % env_hw == 0) hw = env_hw;
    if (per_cu_x2 < 1) per_cu_x2 = 1;
    if (min_chunk < 32) min_chunk = 32;
    int n_parts = group / hw;  // workgroups per (chunk, KV head)
    int want = static_cast<int>(std::max<int64_t>(
        1, (static_cast<int64_t>(per_cu_x2) * ctx->n_cu + 2 * n_kv * n_parts - 1) / (2 * n_kv * n_parts)));
    // (one workgroup per CU at most: beyond half the chip the chunks stay at 512 to 1024 keys - at 64 k of context 256
    // workgroups of 512 keys took 5.79 ms per 40-layer verify where 128 of 1024 took 6.70)
    static const int env_long_chunk = [] { const char *e = getenv("DFLASH_ATTN_LONG_CHUNK"); return e ? atoi(e) : 0; }();
    // (at most 256 splits, which two workgroups per CU would ask for as well: the partial tiles' share of the workspace stays what it was)
    if (per_cu_x2 == 1)
        want = std::max<int>(want, static_cast<int>(std::min<int64_t>(256, bucket / (env_long_chunk >= 32 ? env_long_chunk : 512))));
    // Several blocks in one launch cover the chip between them: a workgroup then serves the whole GQA group, so a chunk
    // of keys is staged once instead of group / hw times (a workgroup's LDS ring leaves no room for a second one on
    // its CU, whatever its size).  The split of the keys (want, min_chunk) stays the single block's, and a head is one
    // wave's work either way: the same bits.
    if (n_blocks > 1) {
        hw = group;
        n_parts = 1;
    }
    // most splits any context up to n_pos can have
    auto splits_for = [&](int64_t np) {
        return ctx_len_dev ? static_cast<int>(std::min<int64_t>(want, (np + min_chunk - 1) / min_chunk))
                           : static_cast<int>((np + attn_chunk(np, want, min_chunk) - 1) / attn_chunk(np, want, min_chunk));
    };
    int n_splits = splits_for(n_pos);
    // several blocks: as many as the workspace has room for partial tiles of (the caller comes back for the rest)
    const size_t slot_bytes = static_cast<size_t>(n_q) * 16 * (head_dim + 2) * sizeof(float);
    if (n_blocks > 1) {
        const size_t room = ctx->workspace_bytes > 4096 ? ctx->workspace_bytes - 4096 : 0;
        while (n_blocks > 1 && static_cast<size_t>(n_blocks) * n_splits * slot_bytes > room) {
            n_blocks--;
            n_rows_total = 16 * n_blocks;
            n_pos = ctx_len + n_rows_total;
            n_splits = splits_for(n_pos);
        }
    }
    if (blocks_done) *blocks_done = n_blocks;
    const int64_t part_slots = static_cast<int64_t>(n_splits) * n_q * 16;

    size_t off = 0;
    float *part_o = dfl_ws_take<float>(ctx, &off, static_cast<size_t>(n_blocks) * part_slots * head_dim * sizeof(float));
    float *part_ml = dfl_ws_take<float>(ctx, &off, static_cast<size_t>(n_blocks) * part_slots * 2 * sizeof(float));
    const _Float16 *vt = static_cast<const _Float16 *>(v_cache);
    int64_t vt_stride = kv_capacity;
    if (v_layout == 0) {
        vt_stride = (n_pos + 31) / 32 * 32;
        _Float16 *vt_ws = dfl_ws_take<_Float16>(ctx, &off, static_cast<size_t>(n_kv) * head_dim * vt_stride * 2);
        if (!vt_ws)
            return dfl_fail(ctx, DFLASH_ERR_WORKSPACE,
                            "attn_verify: transposing V needs %zu workspace bytes; pass the transposed cache instead",
                            static_cast<size_t>(n_kv) * head_dim * vt_stride * 2);
        transpose_v_kernel<<<dim3(static_cast<unsigned>(vt_stride / 32), n_kv), 256, 0, st>>>(
            static_cast<const _Float16 *>(v_cache), vt_ws, n_pos, n_kv, head_dim, vt_stride);
        vt = vt_ws;
    }
    if (!part_o || !part_ml) return dfl_fail(ctx, DFLASH_ERR_WORKSPACE, "attn_verify: workspace too small");

    if (n_splits > 1024) return dfl_fail(ctx, DFLASH_ERR_UNSUPPORTED, "attn_verify: %d KV splits", n_splits);
    const int split_stride = (n_splits + 7) / 8 * 8;
    const dim3 grid(split_stride * n_parts, n_kv, n_blocks);
    const int threads = 64 * hw;
    const _Float16 *k = static_cast<const _Float16 *>(k_cache);
    int32_t rc = DFLASH_OK;
    {
        dfl_timed timer(ctx, st, DFL_T_ATTN);
#define DFL_ATTN(HD)                                                                                              \
    if (q_type == DFLASH_TYPE_F32)                                                                                \
        rc = launch_split<HD, float>(ctx, grid, threads, st, q, k, vt, part_o, part_ml, ctx_len, ctx_len_dev, n_rows_total, n_q, n_kv, \
                                     vt_stride, want, static_cast<int>(min_chunk), scale, full_block, window,     \
                                     split_stride, part_slots);                                                   \
    else                                                                                                          \
        rc = launch_split<HD, _Float16>(ctx, grid, threads, st, q, k, vt, part_o, part_ml, ctx_len, ctx_len_dev, n_rows_total, n_q, \
                                        n_kv, vt_stride, want, static_cast<int>(min_chunk), scale, full_block, window, \
                                        split_stride, part_slots)
        if (head_dim == 64) {
            DFL_ATTN(64);
        } else if (head_dim == 128) {
            DFL_ATTN(128);
        } else {
            DFL_ATTN(256);
        }
#undef DFL_ATTN
    }
    if (rc) return rc;
    attn_combine_kernel<<<dim3(n_q, n_rows, n_blocks), 256, 0, st>>>(part_o, part_ml, out, n_rows_total, n_q, head_dim, ctx_len, ctx_len_dev,
                                                                    want, static_cast<int>(min_chunk), out_xf, out_xf_kind, part_slots,
                                                                    dfl_xf_bytes(static_cast<int64_t>(n_q) * head_dim));
    DFL_HIP_CHECK(ctx, hipGetLastError());
    return DFLASH_OK;
}
