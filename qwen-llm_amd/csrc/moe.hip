// Mixture-of-experts FFN of the packed verify: route on the device, then read every selected
// expert's weights ONCE for all block rows that picked it (the reference runs the experts per
// row after a packed route, metal_dflash.rs:10184-10403; CPU form ffn_moe, forward.rs:749-824).
//
//   probs   = softmax(router . x)                       over all experts
//   picks   = top-k by probability, ties to the lower expert id
//   weights = probs[pick] / max(sum(probs[picks]), 2^-14)
//   out     = sum_k weights[k] * down_e(silu(gate_e x) * up_e x)  +  sigmoid(x . w_shexp) * shared(x)
//
// Work items are "slots": slot = row * n_used + k.  The expert kernels run one workgroup column
// per expert; a workgroup first collects the slots that picked its expert and leaves at once
// if there are none, so HBM traffic is the distinct experts of the block, not rows x k.
#include "common.h"
#include "device_quant.h"
#include "moe_route.h"

#include <cstdlib>

namespace {

constexpr int kMaxSlots = 16;  // a row picks an expert at most once, and a block has at most 16 rows

// Maximum of a 64-bit key over the wave, in every lane: data-parallel-primitive moves within rows of
// 16 lanes (shift right by 1, 2, 4, 8: lane 15 of a row then holds the row's maximum), then lane 15
// of rows 0 and 2 broadcast into rows 1 and 3, then lane 31 into rows 2 and 3; lane 63 has the
// result.  Lanes without a source read 0, the identity.  No LDS round trips, unlike a shuffle.
__device__ __forceinline__ unsigned long long wave_max_u64(unsigned long long v) {
#define DFL_MAX_STEP(ctrl, row_mask)                                                                            \
    do {                                                                                                        \
        const unsigned lo = __builtin_amdgcn_update_dpp(0u, static_cast<unsigned>(v), ctrl, row_mask, 0xf, false);      \
        const unsigned hi = __builtin_amdgcn_update_dpp(0u, static_cast<unsigned>(v >> 32), ctrl, row_mask, 0xf, false); \
        const unsigned long long o = (static_cast<unsigned long long>(hi) << 32) | lo;                          \
        v = o > v ? o : v;                                                                                      \
    } while (0)
    DFL_MAX_STEP(0x111, 0xf);  // row_shr:1
    DFL_MAX_STEP(0x112, 0xf);  // row_shr:2
    DFL_MAX_STEP(0x114, 0xf);  // row_shr:4
    DFL_MAX_STEP(0x118, 0xf);  // row_shr:8
    DFL_MAX_STEP(0x142, 0xa);  // row_bcast:15 into rows 1 and 3
    DFL_MAX_STEP(0x143, 0xc);  // row_bcast:31 into rows 2 and 3
#undef DFL_MAX_STEP
    const unsigned lo = __builtin_amdgcn_readlane(static_cast<unsigned>(v), 63);
    const unsigned hi = __builtin_amdgcn_readlane(static_cast<unsigned>(v >> 32), 63);
    return (static_cast<unsigned long long>(hi) << 32) | lo;
}

// Routing of a whole block in one workgroup of sixteen waves (n_expert <= 1024, at most 16 rows).
// Wave w serves block row w: softmax, top-k (higher probability first, equal probabilities to the
// lower id), the renormalised weights in pick order, and the
// shared-expert gate; a row's arithmetic does not depend on how many rows the block has.  Then the
// whole workgroup lists the block's distinct experts in ascending id order: ids[0 .. n), then one
// slot with id -1 (the shared expert, which every row uses) if with_shared; *n_slots = n (+ 1); for
// every (row, k) pick, slot_of = the index of its expert in that list.
__global__ void __launch_bounds__(1024)
    moe_route_kernel(const float *__restrict__ logits, const float *__restrict__ x, const float *__restrict__ shexp_gate,
                     int n_rows, int n_expert, int n_used, int hidden, int with_shared, int32_t *__restrict__ sel_e,
                     float *__restrict__ sel_w, float *__restrict__ sg, int32_t *__restrict__ ids,
                     int32_t *__restrict__ n_slots, int32_t *__restrict__ slot_of) {
    typedef float f4 __attribute__((ext_vector_type(4)));
    extern __shared__ __attribute__((aligned(16))) float probs[];  // [16][n_expert], then int32 rank[n_expert]
    __shared__ float pick_w[16][64];
    __shared__ int32_t pick_e[16][64];
    __shared__ int wave_count[16];
    int32_t *rank = reinterpret_cast<int32_t *>(probs + 16 * n_expert);
    const int tid = threadIdx.x, lane = tid & 63, row = tid >> 6;
    const bool live = row < n_rows;
    float *pr = probs + row * n_expert;
    if (live) {
        // Everything this row reads from memory is requested before anything waits for it: its first
        // 256 router logits and (2048 elements at a time) the operands of the shared-expert gate
        // sigmoid(x . w); one memory latency instead of one per phase.
        const float *lg = logits + static_cast<size_t>(row) * n_expert;
        float lgv[4];
#pragma unroll
        for (int j = 0; j < 4; j++) lgv[j] = lane + 64 * j < n_expert ? lg[lane + 64 * j] : -INFINITY;
        const float *xr = x + static_cast<size_t>(row) * hidden;
        float dot = 0.0f;
        if (!shexp_gate) {
            // the gate was computed by the kernel that wrote x
        } else if (hidden % 4 == 0) {
            for (int base = 0; base < hidden; base += 2048) {
                f4 xa[8], gb[8];
#pragma unroll
                for (int j = 0; j < 8; j++) {
                    const int i = base + 4 * lane + 256 * j;
                    xa[j] = gb[j] = f4{0, 0, 0, 0};
                    if (i < hidden) {
                        xa[j] = *reinterpret_cast<const f4 *>(xr + i);
                        gb[j] = *reinterpret_cast<const f4 *>(shexp_gate + i);
                    }
                }
#pragma unroll
                for (int j = 0; j < 8; j++)
                    if (base + 4 * lane + 256 * j < hidden)
                        dot += (xa[j][0] * gb[j][0] + xa[j][1] * gb[j][1]) + (xa[j][2] * gb[j][2] + xa[j][3] * gb[j][3]);
            }
        } else {
            for (int i = lane; i < hidden; i += 64) dot += xr[i] * shexp_gate[i];
        }
        for (int off = 32; off > 0; off >>= 1) dot += __shfl_xor(dot, off, 64);
        if (shexp_gate && lane == 0) sg[row] = 1.0f / (1.0f + expf(-dot));

        float mx = -INFINITY;
#pragma unroll
        for (int j = 0; j < 4; j++) mx = fmaxf(mx, lgv[j]);
        for (int e = lane + 256; e < n_expert; e += 64) mx = fmaxf(mx, lg[e]);
        for (int off = 32; off > 0; off >>= 1) mx = fmaxf(mx, __shfl_xor(mx, off, 64));
        float sum = 0.0f;
#pragma unroll
        for (int j = 0; j < 4; j++) {
            if (lane + 64 * j < n_expert) {
                const float ex = expf(lgv[j] - mx);
                pr[lane + 64 * j] = ex;
                sum += ex;
            }
        }
        for (int e = lane + 256; e < n_expert; e += 64) {
            const float ex = expf(lg[e] - mx);
            pr[e] = ex;
            sum += ex;
        }
        for (int off = 32; off > 0; off >>= 1) sum += __shfl_xor(sum, off, 64);
        const float inv = 1.0f / sum;
        for (int e = lane; e < n_expert; e += 64) pr[e] *= inv;
    }
    if (tid < n_expert) rank[tid] = 0;
    __syncthreads();
    if (live) {
        // pick k = the best remaining expert: a wave-wide maximum over 64-bit keys (probability bits,
        // then ~id, so that equal probabilities go to the lower id); the winner's probability is
        // then marked taken (negative).  Same order as ranking every expert against all others, at
        // n_used * n_expert / 64 steps instead of n_expert^2 / 64.
        for (int k = 0; k < n_used; k++) {
            unsigned long long best = 0;
            for (int e = lane; e < n_expert; e += 64) {
                const float p = pr[e];
                const unsigned long long key = (static_cast<unsigned long long>(__float_as_uint(p)) << 32) | (0xffffffffu - static_cast<unsigned>(e));
                if (p >= 0.0f && key > best) best = key;
            }
            best = wave_max_u64(best);
            int e_win = static_cast<int>(0xffffffffu - static_cast<unsigned>(best));
            if (best == 0) e_win = k < n_expert ? k : n_expert - 1;  // nothing comparable left (NaN logits): stay in range
            if (lane == 0) {
                sel_e[row * n_used + k] = e_win;
                pick_e[row][k] = e_win;
                pick_w[row][k] = __uint_as_float(static_cast<unsigned>(best >> 32));
                rank[e_win] = 1;  // picked by some row
                pr[e_win] = -1.0f;
            }
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
        }
    }
    __syncthreads();
    if (live && lane == 0) {
        float wsum = 0.0f;
        for (int k = 0; k < n_used; k++) wsum += pick_w[row][k];  // in pick order, as the reference sums them
        wsum = fmaxf(wsum, 6.103515625e-05f);                     // 2^-14
        for (int k = 0; k < n_used; k++) sel_w[row * n_used + k] = pick_w[row][k] / wsum;
    }
    // distinct experts of the block
    const bool picked = tid < n_expert && rank[tid] != 0;
    const unsigned long long mask = __builtin_amdgcn_ballot_w64(picked);
    if (lane == 0) wave_count[row] = __popcll(mask);
    __syncthreads();
    int base = 0, total = 0;
    for (int w = 0; w < 16; w++) {
        if (w < row) base += wave_count[w];
        total += wave_count[w];
    }
    if (picked) {
        const int idx = base + __popcll(mask & ((1ull << lane) - 1));
        ids[idx] = tid;
        rank[tid] = idx;
    }
    if (tid == 0) {
        if (with_shared) ids[total] = -1;
        *n_slots = total + (with_shared ? 1 : 0);
    }
    __syncthreads();
    if (live && lane < n_used) slot_of[row * n_used + lane] = rank[pick_e[row][lane]];
}

// The same routing for n_expert <= 256, n_used <= 64, with a row's probabilities held in registers
// (four per lane) and one workgroup barrier in all: a row's picks stay in its wave (lane k keeps pick
// k), the row's picked experts go out as a 256-bit mask, and after the barrier every thread derives
// the block's ascending expert list and the slot of each pick from the union of the sixteen masks by
// population counts.  Same arithmetic, in the same order, as moe_route_kernel.
__global__ void __launch_bounds__(1024)
    moe_route_small_kernel(const float *__restrict__ logits, const float *__restrict__ x, const float *__restrict__ shexp_gate,
                           int n_rows, int n_expert, int n_used, int hidden, int with_shared, int32_t *__restrict__ sel_e,
                           float *__restrict__ sel_w, float *__restrict__ sg, int32_t *__restrict__ ids,
                           int32_t *__restrict__ n_slots, int32_t *__restrict__ slot_of) {
    typedef float f4 __attribute__((ext_vector_type(4)));
    __shared__ unsigned long long row_mask[16][4];
    const int tid = threadIdx.x, lane = tid & 63, row = tid >> 6;
    const bool live = row < n_rows;
    int my_e = 0;
    unsigned long long m[4] = {0, 0, 0, 0};
    if (live) {
        const float *lg = logits + static_cast<size_t>(row) * n_expert;
        const float *xr = x + static_cast<size_t>(row) * hidden;
        float dot = 0.0f;
        if (!shexp_gate) {
            // the gate was computed by the kernel that wrote x
        } else if (hidden % 4 == 0) {
            for (int base = 0; base < hidden; base += 2048) {
                f4 xa[8], gb[8];
#pragma unroll
                for (int j = 0; j < 8; j++) {
                    const int i = base + 4 * lane + 256 * j;
                    xa[j] = gb[j] = f4{0, 0, 0, 0};
                    if (i < hidden) {
                        xa[j] = *reinterpret_cast<const f4 *>(xr + i);
                        gb[j] = *reinterpret_cast<const f4 *>(shexp_gate + i);
                    }
                }
#pragma unroll
                for (int j = 0; j < 8; j++)
                    if (base + 4 * lane + 256 * j < hidden)
                        dot += (xa[j][0] * gb[j][0] + xa[j][1] * gb[j][1]) + (xa[j][2] * gb[j][2] + xa[j][3] * gb[j][3]);
            }
        } else {
            for (int i = lane; i < hidden; i += 64) dot += xr[i] * shexp_gate[i];
        }
        for (int off = 32; off > 0; off >>= 1) dot += __shfl_xor(dot, off, 64);
        if (shexp_gate && lane == 0) sg[row] = 1.0f / (1.0f + expf(-dot));

        const dfl_route::RowPicks pk = dfl_route::route_row(lg, n_expert, n_used, lane);
        my_e = pk.my_e;
#pragma unroll
        for (int j = 0; j < 4; j++) m[j] = pk.m[j];
        if (lane < n_used) {
            sel_e[row * n_used + lane] = my_e;
            sel_w[row * n_used + lane] = pk.my_w;
        }
    }
    if (lane < 4) row_mask[row][lane] = m[lane & 3];
    __syncthreads();
    unsigned long long un[4];
    dfl_route::union_of_rows(&row_mask[0][0], lane, un);
    auto slot = [&](int e) { return dfl_route::slot_below(un, e); };  // experts below e in the union
    if (tid < n_expert && ((un[tid >> 6] >> (tid & 63)) & 1)) ids[slot(tid)] = tid;
    if (tid == 0) {
        const int total = __popcll(un[0]) + __popcll(un[1]) + __popcll(un[2]) + __popcll(un[3]);
        if (with_shared) ids[total] = -1;
        *n_slots = total + (with_shared ? 1 : 0);
    }
    if (live && lane < n_used) slot_of[row * n_used + lane] = slot(my_e);
}

// Collects the slots whose pick is `expert`; returns the count (uniform over the workgroup).
__device__ int collect_slots(const int32_t *__restrict__ sel_e, int n_slots, int expert, int *list, int *count) {
    if (threadIdx.x == 0) *count = 0;
    __syncthreads();
    for (int s = threadIdx.x; s < n_slots; s += blockDim.x)
        if (sel_e[s] == expert) list[atomicAdd(count, 1)] = s;
    __syncthreads();
    return *count;
}

// y[slot][o] = W_expert[o][:] . xin[src(slot)][:]  for the slots of this expert.
// GATE_UP: two stacked matrices, y = silu(gate) * up, xin row = slot / n_used (the block row).
// Otherwise: one matrix, xin row = slot.
// A row of n_in/32 sub-blocks is spread over LPR lanes (32 or 64); a wave does 64/LPR rows at once.
template <bool GATE_UP, int LPR>
__global__ void __launch_bounds__(256)
    moe_expert_kernel(int type, const uint8_t *__restrict__ w0, const uint8_t *__restrict__ w1, size_t row_bytes,
                      const float *__restrict__ xin, const int32_t *__restrict__ sel_e, int n_slots, int n_used, int n_in,
                      int n_out, float *__restrict__ y) {
    __shared__ int list[kMaxSlots];
    __shared__ int count;
    const int expert = blockIdx.y;
    const int n = collect_slots(sel_e, n_slots, expert, list, &count);
    if (n == 0) return;
    constexpr int kRowsPerWave = 64 / LPR;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int sub_lane = lane % LPR, sub_row = lane / LPR;
    const int n_sub = n_in / 32;
    const int rows_per_wg = 4 * kRowsPerWave * 4;  // 4 waves x rows at once x 4 passes
    const int o0 = blockIdx.x * rows_per_wg;
    const size_t expert_off = static_cast<size_t>(expert) * n_out * row_bytes;
    for (int pass = 0; pass < 4; pass++) {
        const int o = o0 + (pass * 4 + wave) * kRowsPerWave + sub_row;
        const bool live = o < n_out;
        const uint8_t *r0 = w0 + expert_off + static_cast<size_t>(live ? o : 0) * row_bytes;
        const uint8_t *r1 = GATE_UP ? w1 + expert_off + static_cast<size_t>(live ? o : 0) * row_bytes : nullptr;
        for (int s0 = 0; s0 < n; s0 += 4) {  // up to 4 slots share one dequantisation
            float acc0[4] = {0, 0, 0, 0}, acc1[4] = {0, 0, 0, 0};
            for (int sb = sub_lane; sb < n_sub; sb += LPR) {
                float wa[32], wb[32];
                dfl_dequant_sub32(type, r0, sb, wa);
                if (GATE_UP) dfl_dequant_sub32(type, r1, sb, wb);
#pragma unroll
                for (int t = 0; t < 4; t++) {
                    if (s0 + t >= n) break;
                    const int slot = list[s0 + t];
                    const float4 *xr = reinterpret_cast<const float4 *>(
                        xin + static_cast<size_t>(GATE_UP ? slot / n_used : slot) * n_in + 32 * sb);
#pragma unroll
                    for (int v = 0; v < 8; v++) {
                        const float4 xv = xr[v];
                        acc0[t] += wa[4 * v] * xv.x + wa[4 * v + 1] * xv.y + wa[4 * v + 2] * xv.z + wa[4 * v + 3] * xv.w;
                        if (GATE_UP)
                            acc1[t] += wb[4 * v] * xv.x + wb[4 * v + 1] * xv.y + wb[4 * v + 2] * xv.z + wb[4 * v + 3] * xv.w;
                    }
                }
            }
#pragma unroll
            for (int t = 0; t < 4; t++) {
                float a = acc0[t], b = acc1[t];
                for (int off = LPR / 2; off > 0; off >>= 1) {
                    a += __shfl_xor(a, off, 64);
                    if (GATE_UP) b += __shfl_xor(b, off, 64);
                }
                if (sub_lane == 0 && live && s0 + t < n) {
                    const float r = GATE_UP ? a / (1.0f + expf(-a)) * b : a;
                    y[static_cast<size_t>(list[s0 + t]) * n_out + o] = r;
                }
            }
        }
    }
}

// x[row] += sum_k w[row][k] * eo[row*n_used + k]  +  sg[row] * shared[row]
__global__ void moe_combine_kernel(const float *__restrict__ eo, const float *__restrict__ sel_w, const float *__restrict__ sg,
                                   const float *__restrict__ shared, int n_used, int hidden, float *__restrict__ x) {
    const int row = blockIdx.y;
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= hidden) return;
    float out = 0.0f;
    for (int k = 0; k < n_used; k++)
        out += sel_w[row * n_used + k] * eo[(static_cast<size_t>(row) * n_used + k) * hidden + i];
    out += sg[row] * shared[static_cast<size_t>(row) * hidden + i];
    x[static_cast<size_t>(row) * hidden + i] += out;
}

__global__ void silu_mul_rows_kernel(float *__restrict__ g, const float *__restrict__ u, size_t n) {
    size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i < n) {
        const float v = g[i];
        g[i] = v / (1.0f + expf(-v)) * u[i];
    }
}

// x[row] += sum_k w[row][k] * eo[slot_of[row][k]][row]  +  sg[row] * shared[row]
// (shared == nullptr: the shared expert's output is the last slot of eo)
__global__ void moe_combine_slots_kernel(const float *__restrict__ eo, const int32_t *__restrict__ slot_of,
                                         const float *__restrict__ sel_w, const float *__restrict__ sg,
                                         const float *__restrict__ shared, const int32_t *__restrict__ n_slots, int n_used,
                                         int hidden, float *__restrict__ x) {
    const int row = blockIdx.y;
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= hidden) return;
    float out = 0.0f;
    for (int k = 0; k < n_used; k++) {
        const size_t slot = slot_of[row * n_used + k];
        out += sel_w[row * n_used + k] * eo[(slot * 16 + row) * hidden + i];
    }
    const float sh = shared ? shared[static_cast<size_t>(row) * hidden + i]
                            : eo[((static_cast<size_t>(*n_slots) - 1) * 16 + row) * hidden + i];
    out += sg[row] * sh;
    x[static_cast<size_t>(row) * hidden + i] += out;
}

// The same, followed in the same pass by the RMSNorm that consumes x next (the following layer's
// attention norm or the output norm): y = x * rsqrt(mean(x^2) + eps) * norm_w.  One workgroup per
// row, the row (hidden <= 4096, a multiple of 4) in registers; element sums and the sum of squares
// are taken in the order of moe_combine_slots_kernel followed by the norm kernel.
__global__ void __launch_bounds__(256)
    moe_combine_norm_kernel(const float *__restrict__ eo, const int32_t *__restrict__ slot_of, const float *__restrict__ sel_w,
                            const float *__restrict__ sg, const float *__restrict__ shared, const int32_t *__restrict__ n_slots,
                            int n_used, int hidden, float *__restrict__ x, const float *__restrict__ norm_w,
                            float *__restrict__ y, float eps, const float *__restrict__ pre_add, void *__restrict__ y_xf,
                            int y_xf_kind, int grouped = 0, size_t xf_stride = 0) {
    typedef float f4 __attribute__((ext_vector_type(4)));
    __shared__ float sh[4];
    __shared__ float w_k[64];
    __shared__ int32_t slot_k[64];  // row of eo that holds pick k of this row
    const int row = blockIdx.x, tid = threadIdx.x;
    // Everything whose address depends on nothing this kernel reads is asked for first (the slot count, the gate, the
    // residual row and the term to add to it), beside the picks: one trip to memory, then the picks' output rows.
    const size_t n_slots_now = static_cast<size_t>(*n_slots);
    const float gate = sg[row];
    f4 v[4];
#pragma unroll
    for (int j = 0; j < 4; j++) {
        const int i = 4 * (tid + 256 * j);
        v[j] = f4{0, 0, 0, 0};
        if (i < hidden) {
            v[j] = *reinterpret_cast<const f4 *>(x + static_cast<size_t>(row) * hidden + i);
            // (a residual term the norm before this layer's experts left out: it goes in first, as it would have there)
            if (pre_add) v[j] += *reinterpret_cast<const f4 *>(pre_add + static_cast<size_t>(row) * hidden + i);
        }
    }
    // grouped (rows of several 16-row blocks, moe_group_slots_kernel): slot_of is the eo row of a pick itself, and the
    // shared expert's slots are the last gridDim.x / 16 (rounded up) of the list, one per block of rows
    if (tid < n_used) {
        w_k[tid] = sel_w[row * n_used + tid];
        slot_k[tid] = grouped ? slot_of[row * n_used + tid] : slot_of[row * n_used + tid] * 16 + row;
    }
    __syncthreads();
    const size_t last = grouped ? (n_slots_now - (gridDim.x + 15) / 16 + (row >> 4)) * 16 + (row & 15) : (n_slots_now - 1) * 16 + row;
    float s = 0.0f;
#pragma unroll
    for (int j = 0; j < 4; j++) {
        const int i = 4 * (tid + 256 * j);
        if (i < hidden) {
            f4 out = {0, 0, 0, 0};
            for (int k = 0; k < n_used; k++)
                out += w_k[k] * *reinterpret_cast<const f4 *>(eo + static_cast<size_t>(slot_k[k]) * hidden + i);
            const f4 shv = shared ? *reinterpret_cast<const f4 *>(shared + static_cast<size_t>(row) * hidden + i)
                                  : *reinterpret_cast<const f4 *>(eo + last * hidden + i);
            out += gate * shv;
            v[j] += out;
            *reinterpret_cast<f4 *>(x + static_cast<size_t>(row) * hidden + i) = v[j];
        }
        s += (v[j][0] * v[j][0] + v[j][1] * v[j][1]) + (v[j][2] * v[j][2] + v[j][3] * v[j][3]);
    }
    // (the next norm's weights are asked for here, behind the picks' rows in the order of issue - loads return in that
    // order, and these come from further away than the rows the sum is waiting for - and ahead of the barrier)
    f4 nw[4];
#pragma unroll
    for (int j = 0; j < 4; j++) {
        const int i = 4 * (tid + 256 * j);
        nw[j] = i < hidden ? *reinterpret_cast<const f4 *>(norm_w + i) : f4{0, 0, 0, 0};
    }
    for (int off = 32; off > 0; off >>= 1) s += __shfl_xor(s, off, 64);
    if ((tid & 63) == 0) sh[tid >> 6] = s;
    __syncthreads();
    s = ((sh[0] + sh[1]) + sh[2]) + sh[3];
    const float scale = 1.0f / sqrtf(s / static_cast<float>(hidden) + eps);
#pragma unroll
    for (int j = 0; j < 4; j++) {
        const int i = 4 * (tid + 256 * j);
        if (i < hidden) {
            const f4 o = v[j] * scale * nw[j];
            *reinterpret_cast<f4 *>(y + static_cast<size_t>(row) * hidden + i) = o;
            // (hidden a multiple of 256 here: whole waves are inside or outside the row)
            if (y_xf)
                dfl_xf_store_pair(static_cast<uint8_t *>(y_xf) + (row >> 4) * xf_stride, y_xf_kind, row & 15, i & ~7, o[0], o[1], o[2], o[3]);
        }
    }
}

// ---- rows of several 16-row blocks through one pass over the experts (prefill) ----
//
// A block of 16 rows touches 60-80 of 128 experts, so block after block re-reads most of a layer's expert weights;
// 256 rows touch all of them about once.  The rows are therefore regrouped by expert: a slot is (expert, up to sixteen
// of the rows that picked it), the expert kernels run their per-slot-activations mode over gathered copies of those
// rows, and every row then sums its picks' outputs in pick order.  A (row, expert) product is one wave's whole-K sum
// over the row's own activations, so it has the bits it has when the row's block runs alone.

// Picks of every row: wave w of workgroup b routes row 16 b + w (dfl_route::route_row, as in the block kernels).
__global__ void __launch_bounds__(1024)
    moe_group_route_kernel(const float *__restrict__ logits, int n_rows, int n_expert, int n_used, int32_t *__restrict__ sel_e,
                           float *__restrict__ sel_w) {
    const int lane = threadIdx.x & 63, row = blockIdx.x * 16 + (threadIdx.x >> 6);
    if (row >= n_rows) return;
    const dfl_route::RowPicks pk = dfl_route::route_row(logits + static_cast<size_t>(row) * n_expert, n_expert, n_used, lane);
    if (lane < n_used) {
        sel_e[row * n_used + lane] = pk.my_e;
        sel_w[row * n_used + lane] = pk.my_w;
    }
}

// The slot list of a group of rows.  Expert e with c picks gets ceil(c / 16) consecutive slots, experts in ascending
// order; behind them one slot per block of sixteen rows for the shared expert (id -1, rows 16 b .. 16 b + 15).
//   ids[slot], *n_slots;  slot_rows[slot][16]: the rows whose activations the slot multiplies (unused places repeat
//   row 0: computed, never read);  pick_pos[row][k] = 16 slot + place of the pick's output row.
// Places inside an expert's slots are handed out by an atomic counter, so they vary from run to run; no sum does.
// One workgroup; n_rows * n_used <= 4096, n_expert <= 256.
constexpr int kGroupPicksPerThread = 4;
__global__ void __launch_bounds__(1024)
    moe_group_slots_kernel(const int32_t *__restrict__ sel_e, int n_rows, int n_used, int n_expert, int32_t *__restrict__ ids,
                           int32_t *__restrict__ n_slots, int32_t *__restrict__ slot_rows, int32_t *__restrict__ pick_pos,
                           int max_slots) {
    __shared__ int cnt[256], base[257];
    const int tid = threadIdx.x;
    if (tid < 256) cnt[tid] = 0;
    __syncthreads();
    const int n_picks = n_rows * n_used;
    int my_e[kGroupPicksPerThread], my_place[kGroupPicksPerThread];
#pragma unroll
    for (int j = 0; j < kGroupPicksPerThread; j++) {
        const int p = tid + 1024 * j;
        my_e[j] = -1;
        my_place[j] = 0;
        if (p < n_picks) {
            my_e[j] = min(max(sel_e[p], 0), n_expert - 1);
            my_place[j] = atomicAdd(&cnt[my_e[j]], 1);
        }
    }
    __syncthreads();
    if (tid == 0) {
        int b = 0;
        for (int e = 0; e < n_expert; e++) {
            base[e] = b;
            b += (cnt[e] + 15) >> 4;
        }
        base[n_expert] = b;
    }
    __syncthreads();
    const int total = base[n_expert], n_blocks = (n_rows + 15) >> 4;
    if (tid == 0) *n_slots = min(total + n_blocks, max_slots);  // (the host sizes max_slots for the worst case)
    if (tid < n_expert) {
        const int c = cnt[tid], b = base[tid];
        for (int t = 0; t < ((c + 15) >> 4); t++) ids[b + t] = tid;
        if (c & 15)
            for (int m = c & 15; m < 16; m++) slot_rows[(b + (c >> 4)) * 16 + m] = 0;
    }
    for (int r = tid; r < 16 * n_blocks; r += 1024) {
        slot_rows[total * 16 + r] = min(r, n_rows - 1);
        if ((r & 15) == 0) ids[total + (r >> 4)] = -1;
    }
#pragma unroll
    for (int j = 0; j < kGroupPicksPerThread; j++) {
        const int p = tid + 1024 * j;
        if (p < n_picks) {
            const int at = (base[my_e[j]] + (my_place[j] >> 4)) * 16 + (my_place[j] & 15);
            slot_rows[at] = p / n_used;
            pick_pos[p] = at;
        }
    }
}

// xg[slot][place][:] = f16(cur[slot_rows[slot][place]][:]): what the expert kernel would round the row to as it loads it.
__global__ void __launch_bounds__(256)
    moe_group_gather_kernel(const float *__restrict__ cur, const int32_t *__restrict__ slot_rows, const int32_t *__restrict__ n_slots,
                            int hidden, _Float16 *__restrict__ xg) {
    typedef float f4 __attribute__((ext_vector_type(4)));
    typedef _Float16 h8 __attribute__((ext_vector_type(8)));
    const int at = blockIdx.y;
    if ((at >> 4) >= *n_slots) return;
    const int i = 8 * (blockIdx.x * 256 + threadIdx.x);
    if (i >= hidden) return;
    const float *src = cur + static_cast<size_t>(slot_rows[at]) * hidden + i;
    const f4 a = *reinterpret_cast<const f4 *>(src), b = *reinterpret_cast<const f4 *>(src + 4);
    const h8 o = {static_cast<_Float16>(a[0]), static_cast<_Float16>(a[1]), static_cast<_Float16>(a[2]), static_cast<_Float16>(a[3]),
                  static_cast<_Float16>(b[0]), static_cast<_Float16>(b[1]), static_cast<_Float16>(b[2]), static_cast<_Float16>(b[3])};
    *reinterpret_cast<h8 *>(xg + static_cast<size_t>(at) * hidden + i) = o;
}

}  // namespace

namespace {
// whether the layer's expert stacks take the batched launches (one streaming GEMM per projection over the distinct experts)
bool moe_batched(const dflash_model_cfg &c, const dflash_layer &L) {
    static const bool per_slot_forced = getenv("DFLASH_MOE_PERSLOT") != nullptr;  // read once per process
    const int et = L.gate_exps.type, dt = L.down_exps.type;
    const bool tiled = et == DFLASH_TYPE_Q4_K_TILED;
    return (tiled || (et == DFLASH_TYPE_Q4_K && dt == DFLASH_TYPE_Q4_K)) && c.hidden % DFL_QK_K == 0 && c.ffn_expert % DFL_QK_K == 0 &&
           !per_slot_forced;
}
}  // namespace

bool dfl_moe_norm_fusable(const dflash_ctx *ctx, const dflash_model_cfg &c, const dflash_layer &L, int n) {
    // the residual term is added back by moe_combine_norm_kernel, which the batched path ends with
    return c.n_expert > 0 && L.shexp_gate && L.router.data && L.gate_exps.data && L.down_exps.data && moe_batched(c, L) &&
           c.hidden <= 4096 && c.hidden % 4 == 0 && dfl_router_norm_fits(ctx, L.router.type, L.router.data, c.hidden, c.n_expert, n);
}

int32_t dfl_moe_ffn(dflash_ctx *ctx, const dflash_model_cfg &c, const dflash_layer &L, float *cur, int n,
                    const dfl_moe_scratch &s, float *x_resid, bool gate_done, const float *next_norm_w, float *next_cur,
                    bool *next_done, hipStream_t st, const float *pre_add, const float *pre_norm_w, void *next_xf, int next_xf_kind) {
    if (next_done) *next_done = false;
    if ((pre_add != nullptr) != (pre_norm_w != nullptr) ||
        (pre_add && !(next_norm_w && next_cur && next_done && dfl_moe_norm_fusable(ctx, c, L, n))))
        return dfl_fail(ctx, DFLASH_ERR_INVALID_INPUT, "moe: the norm can ride in the router's launch only where dfl_moe_norm_fusable() holds");
    const int E = c.n_expert, used = c.n_expert_used < E ? c.n_expert_used : E;
    const int H = c.hidden, fe = c.ffn_expert, fs = c.ffn_shared;
    const int n_slots = n * used;
    if (used < 1 || used > 64 || E > 8192 || fe % 32 || H % 32)
        return dfl_fail(ctx, DFLASH_ERR_UNSUPPORTED, "moe: n_expert %d / n_expert_used %d / ffn_expert %d unsupported", E, used, fe);
    if (!L.router.data || !L.gate_exps.data || !L.up_exps.data || !L.down_exps.data || !L.shexp_gate || !L.gate.data ||
        !L.up.data || !L.down.data)
        return dfl_fail(ctx, DFLASH_ERR_INVALID_INPUT,
                        "moe: a mixture-of-experts layer needs router, gate/up/down_exps, shexp_gate and the shared expert's gate/up/down");
    const int et = L.gate_exps.type;
    const bool tiled = et == DFLASH_TYPE_Q4_K_TILED;  // every expert matrix repacked on its own (stack stride = tiled size)
    if (et != L.up_exps.type || (et != DFLASH_TYPE_Q4_K && et != DFLASH_TYPE_Q6_K && et != DFLASH_TYPE_Q8_0 && !tiled))
        return dfl_fail(ctx, DFLASH_ERR_UNSUPPORTED, "moe: expert weight type %d", et);
    const int dt = L.down_exps.type;
    if ((dt != DFLASH_TYPE_Q4_K && dt != DFLASH_TYPE_Q6_K && dt != DFLASH_TYPE_Q8_0 && dt != DFLASH_TYPE_Q4_K_TILED) ||
        (dt == DFLASH_TYPE_Q4_K_TILED) != tiled)
        return dfl_fail(ctx, DFLASH_ERR_UNSUPPORTED, "moe: expert weight types %d / %d (tiled stacks go together)", et, dt);
    const size_t rb_in = dflash_row_bytes(et, H), rb_dn = dflash_row_bytes(dt, fe);
    if (rb_in == 0 || rb_dn == 0) return dfl_fail(ctx, DFLASH_ERR_BAD_SHAPE, "moe: row sizes do not fit the block size");

    int32_t rc;
    if (pre_add) {
        rc = dfl_router_norm(ctx, L.router.data, x_resid, pre_add, pre_norm_w, L.shexp_gate, c.eps, cur, s.sg, s.probs, H, E, n, st);
        gate_done = true;
    } else {
        rc = dfl_gemm_fewrow_checked(ctx, L.router.type, L.router.data, cur, DFLASH_TYPE_F32, s.probs, H, E, n, st);
    }
    if (rc) return rc;
    if (E > 1024) return dfl_fail(ctx, DFLASH_ERR_UNSUPPORTED, "moe: %d experts (at most 1024)", E);
    const bool batched = moe_batched(c, L);
    if (tiled && !batched) return dfl_fail(ctx, DFLASH_ERR_UNSUPPORTED, "moe: tiled expert stacks need the batched path");
    // the shared expert rides along as one more slot of the batched GEMMs when it has the experts' shape (and order)
    const bool folded_shared = batched && fs == fe && L.gate.type == et && L.up.type == et && L.down.type == et;
    const size_t stride_in = tiled ? dflash_q4k_tiled_bytes(H, fe) : static_cast<size_t>(fe) * rb_in;
    const size_t stride_dn = tiled ? dflash_q4k_tiled_bytes(fe, H) : static_cast<size_t>(H) * rb_dn;
    const size_t route_lds = static_cast<size_t>(17) * E * sizeof(float);
    if (route_lds > 48 * 1024) {
        if (const int32_t rc_ = dfl_raise_lds_limit(ctx, reinterpret_cast<const void *>(moe_route_kernel), 17 * 1024 * sizeof(float)))
            return rc_;
    }
    const float *gate_w = gate_done ? nullptr : L.shexp_gate;  // null: sg is already there
    // the routing can ride in the gate/up launch (every workgroup derives the expert list itself): one launch fewer
    const bool route_inside = batched && tiled && !gate_w && n <= 16 &&
                              dfl_q4k_batched_can_route(ctx, 1, fe, E, used);
    if (route_inside) {
        // nothing to launch here
    } else if (E <= 256)
        moe_route_small_kernel<<<1, 1024, 0, st>>>(s.probs, cur, gate_w, n, E, used, H, folded_shared ? 1 : 0, s.sel_e,
                                                   s.sel_w, s.sg, s.ids, s.n_distinct, s.slot_of);
    else
        moe_route_kernel<<<1, 1024, route_lds, st>>>(s.probs, cur, gate_w, n, E, used, H, folded_shared ? 1 : 0,
                                                     s.sel_e, s.sel_w, s.sg, s.ids, s.n_distinct, s.slot_of);
    if (batched) {
        // the selected experts' matrices form one streaming GEMM each for gate, up and down: every
        // distinct expert's weights are read once, with all block rows riding along on the MFMA;
        // no split K, so a row's result is the same whichever other experts the block uses
        const bool fold = folded_shared;
        const int max_slots = (n_slots < E ? n_slots : E) + (fold ? 1 : 0);
        const size_t per_slot = static_cast<size_t>(16) * fe;
        // gate and up of every selected expert in one launch, silu(gate) * up applied to the tiles
        // while they are still in registers
        // (handed to the down product as f16 where the path writes it: the down kernel rounds its activations to f16
        // as it loads them, so the bits it computes with are the same and the hand-off is half the size)
        const int32_t mid_type = dfl_q4k_batched_f16_out(ctx, tiled ? 1 : 0, 1, fe) ? DFLASH_TYPE_F16 : DFLASH_TYPE_F32;
        const dfl_route_args route = {s.probs, E, used, folded_shared ? 1 : 0, s.sel_e, s.sel_w, s.slot_of};
        if ((rc = dfl_gemm_q4k_batched(ctx, L.gate_exps.data, stride_in, fold ? L.gate.data : nullptr, s.ids,
                                       s.n_distinct, max_slots, cur, DFLASH_TYPE_F32, 0, s.gate_out, mid_type, per_slot, H, fe, n, 1,
                                       L.up_exps.data, fold ? L.up.data : nullptr, tiled ? 1 : 0, st, route_inside ? &route : nullptr)))
            return rc;
        if ((rc = dfl_gemm_q4k_batched(ctx, L.down_exps.data, stride_dn, fold ? L.down.data : nullptr, s.ids,
                                       s.n_distinct, max_slots, s.gate_out, mid_type, per_slot, s.eo, DFLASH_TYPE_F32,
                                       static_cast<size_t>(16) * H, fe, H, n, 1, nullptr, nullptr, tiled ? 1 : 0, st)))
            return rc;
    } else {
        {
            dim3 grid(1, E);  // x: 16 * (64 / LPR) output rows per workgroup
            const int n_sub = H / 32;
            if (n_sub <= 32) {
                grid.x = (fe + 31) / 32;
                moe_expert_kernel<true, 32><<<grid, 256, 0, st>>>(et, static_cast<const uint8_t *>(L.gate_exps.data),
                                                                 static_cast<const uint8_t *>(L.up_exps.data), rb_in, cur, s.sel_e,
                                                                 n_slots, used, H, fe, s.act);
            } else {
                grid.x = (fe + 15) / 16;
                moe_expert_kernel<true, 64><<<grid, 256, 0, st>>>(et, static_cast<const uint8_t *>(L.gate_exps.data),
                                                                 static_cast<const uint8_t *>(L.up_exps.data), rb_in, cur, s.sel_e,
                                                                 n_slots, used, H, fe, s.act);
            }
        }
        {
            dim3 grid(1, E);
            const int n_sub = fe / 32;
            if (n_sub <= 32) {
                grid.x = (H + 31) / 32;
                moe_expert_kernel<false, 32><<<grid, 256, 0, st>>>(dt, static_cast<const uint8_t *>(L.down_exps.data), nullptr, rb_dn,
                                                                  s.act, s.sel_e, n_slots, used, fe, H, s.eo);
            } else {
                grid.x = (H + 15) / 16;
                moe_expert_kernel<false, 64><<<grid, 256, 0, st>>>(dt, static_cast<const uint8_t *>(L.down_exps.data), nullptr, rb_dn,
                                                                  s.act, s.sel_e, n_slots, used, fe, H, s.eo);
            }
        }
    }
    if (!folded_shared) {  // shared expert: plain dense SwiGLU through the few-row GEMM
        if ((rc = dfl_gemm_fewrow_checked(ctx, L.gate.type, L.gate.data, cur, DFLASH_TYPE_F32, s.g, H, fs, n, st))) return rc;
        if ((rc = dfl_gemm_fewrow_checked(ctx, L.up.type, L.up.data, cur, DFLASH_TYPE_F32, s.u, H, fs, n, st))) return rc;
        const size_t nf = static_cast<size_t>(n) * fs;
        silu_mul_rows_kernel<<<static_cast<unsigned>((nf + 255) / 256), 256, 0, st>>>(s.g, s.u, nf);
        if ((rc = dfl_gemm_fewrow_checked(ctx, L.down.type, L.down.data, s.g, DFLASH_TYPE_F32, s.shared, fs, H, n, st))) return rc;
    }
    if (batched && next_norm_w && next_cur && next_done && H <= 4096 && H % 4 == 0) {
        moe_combine_norm_kernel<<<n, 256, 0, st>>>(s.eo, s.slot_of, s.sel_w, s.sg, folded_shared ? nullptr : s.shared, s.n_distinct,
                                                   used, H, x_resid, next_norm_w, next_cur, c.eps, pre_add,
                                                   H % DFL_QK_K == 0 ? next_xf : nullptr, next_xf_kind);
        *next_done = true;
    } else if (batched)
        moe_combine_slots_kernel<<<dim3((H + 255) / 256, n), 256, 0, st>>>(s.eo, s.slot_of, s.sel_w, s.sg,
                                                                         folded_shared ? nullptr : s.shared, s.n_distinct, used,
                                                                         H, x_resid);
    else
        moe_combine_kernel<<<dim3((H + 255) / 256, n), 256, 0, st>>>(s.eo, s.sel_w, s.sg, s.shared, used, H, x_resid);
    DFL_HIP_CHECK(ctx, hipGetLastError());
    return DFLASH_OK;
}

int dfl_moe_group_max_slots(const dflash_model_cfg &c, int n_rows) {
    const int used = c.n_expert_used < c.n_expert ? c.n_expert_used : c.n_expert;
    const int picks = n_rows * used;
    // sum over experts of ceil(count / 16) <= distinct experts + picks / 16, and one shared-expert slot per block
    return (picks < c.n_expert ? picks : c.n_expert) + picks / 16 + (n_rows + 15) / 16;
}

bool dfl_moe_group_fits(const dflash_ctx *ctx, const dflash_model_cfg &c, const dflash_layer &L, int n_rows) {
    const int E = c.n_expert, used = c.n_expert_used < E ? c.n_expert_used : E;
    const bool tiled = L.gate_exps.type == DFLASH_TYPE_Q4_K_TILED && L.up_exps.type == DFLASH_TYPE_Q4_K_TILED &&
                       L.down_exps.type == DFLASH_TYPE_Q4_K_TILED;
    const bool folded = c.ffn_shared == c.ffn_expert && L.gate.type == DFLASH_TYPE_Q4_K_TILED && L.up.type == DFLASH_TYPE_Q4_K_TILED &&
                        L.down.type == DFLASH_TYPE_Q4_K_TILED;
    return E >= 1 && E <= 256 && used >= 1 && used <= 64 && n_rows >= 1 && n_rows * used <= 1024 * kGroupPicksPerThread && tiled && folded &&
           c.hidden % DFL_QK_K == 0 && c.ffn_expert % DFL_QK_K == 0 && c.hidden <= 4096 && L.shexp_gate && L.router.data &&
           dfl_router_norm_fits(ctx, L.router.type, L.router.data, c.hidden, E, 16) &&
           dfl_q4k_batched_f16_out(ctx, 1, 1, c.ffn_expert);
}

int32_t dfl_moe_ffn_group(dflash_ctx *ctx, const dflash_model_cfg &c, const dflash_layer &L, float *x_resid,
                          float *cur, int n_rows, const dfl_moe_group_scratch &s, const float *next_norm_w, void *next_xf,
                          int next_xf_kind, size_t next_xf_stride, hipStream_t st) {
    if (!dfl_moe_group_fits(ctx, c, L, n_rows) || !x_resid || !cur || !next_norm_w)
        return dfl_fail(ctx, DFLASH_ERR_UNSUPPORTED, "moe group: layer or row count (%d) not taken", n_rows);
    const int E = c.n_expert, used = c.n_expert_used < E ? c.n_expert_used : E, H = c.hidden, fe = c.ffn_expert;
    const int max_slots = dfl_moe_group_max_slots(c, n_rows);
    if (max_slots > s.max_slots) return dfl_fail(ctx, DFLASH_ERR_INVALID_INPUT, "moe group: scratch sized for %d slots, %d needed", s.max_slots, max_slots);
    int32_t rc;
    if ((rc = dfl_router_rows(ctx, L.router.data, cur, s.logits, H, E, n_rows, st))) return rc;
    moe_group_route_kernel<<<(n_rows + 15) / 16, 1024, 0, st>>>(s.logits, n_rows, E, used, s.sel_e, s.sel_w);
    moe_group_slots_kernel<<<1, 1024, 0, st>>>(s.sel_e, n_rows, used, E, s.ids, s.n_slots, s.slot_rows, s.pick_pos, max_slots);
    moe_group_gather_kernel<<<dim3((H / 8 + 255) / 256, max_slots * 16), 256, 0, st>>>(cur, s.slot_rows, s.n_slots, H, s.xg);
    const size_t stride_in = dflash_q4k_tiled_bytes(H, fe), stride_dn = dflash_q4k_tiled_bytes(fe, H);
    if ((rc = dfl_gemm_q4k_batched(ctx, L.gate_exps.data, stride_in, L.gate.data, s.ids, s.n_slots, max_slots, s.xg, DFLASH_TYPE_F16,
                                   static_cast<size_t>(16) * H, s.act, DFLASH_TYPE_F16, static_cast<size_t>(16) * fe, H, fe, 16, 1,
                                   L.up_exps.data, L.up.data, 1, st, nullptr)))
        return rc;
    if ((rc = dfl_gemm_q4k_batched(ctx, L.down_exps.data, stride_dn, L.down.data, s.ids, s.n_slots, max_slots, s.act, DFLASH_TYPE_F16,
                                   static_cast<size_t>(16) * fe, s.eo, DFLASH_TYPE_F32, static_cast<size_t>(16) * H, fe, H, 16, 1, nullptr,
                                   nullptr, 1, st, nullptr)))
        return rc;
    moe_combine_norm_kernel<<<n_rows, 256, 0, st>>>(s.eo, s.pick_pos, s.sel_w, s.sg, nullptr, s.n_slots, used, H, x_resid, next_norm_w,
                                                    cur, c.eps, nullptr, next_xf, next_xf_kind, 1, next_xf_stride);
    DFL_HIP_CHECK(ctx, hipGetLastError());
    return DFLASH_OK;
}
