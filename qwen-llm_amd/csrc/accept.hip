// Acceptance: row-wise argmax / top-k over logits, the sampler-v1 filter chain and the
// speculative couplings, and the accept-prefix block decision, on the GPU.
//
// Reference: kernels/elementwise.metal:1153-1359 (argmax family), kernels/dflash2.metal:73-170
// (top-16), crates/qwen-llm/src/sampling.rs (chain :1541-1615, couplings :692-790, ordering keys
// :1206-1235, RNG :1621-1670), crates/qwen-llm/src/metal_dflash/accept.rs:76-183 (block decision,
// CPU-only in the reference).
//
// Everything here is HBM-bound streaming over [rows][vocab] f32 plus O(top_k) arithmetic, and, at one block per
// call, a chain of latencies (a dependent launch, a trip to memory for what another XCD wrote, an LDS read) rather
// than a volume of work:
//  * a row is cut into chunks (8192 tokens for the argmax, 16384 for the top-k selection) so that rows x chunks
//    workgroups cover the chip in one round; each workgroup streams its chunk once with coalesced loads;
//  * order decisions use the reference's integer keys (descending f32 total order above ascending
//    token id), so the selected candidates and their order are exact, not approximately sorted;
//  * top-k of a chunk: the k-th best of the 1024 per-thread bests bounds every winner, so only the elements of the
//    k winning threads are ranked; ranks come from counting (keys are distinct), not from sorting networks in LDS,
//    whose every step is a workgroup barrier;
//  * everything that feeds a comparison with a uniform draw is f64 and added in the order of the reference's
//    loops; what is independent per candidate (conversions, exponentials) is done a candidate per lane;
//  * a block with dense draft proposals is three launches: selection of both logit tensors, the rows' chains
//    together with the draft rows' tile sums, the decision (written straight to pinned host memory).
#include "common.h"
#include "sampler_chain.h"
#include "accept_wide.h"

#include <cmath>
#include <cstring>

namespace {

constexpr int kChunk = 8192;       // tokens per workgroup of the argmax / top-2 kernel
// Tokens per workgroup of the top-k selection.  A 16-row block with dense draft proposals is 31 rows: at 8192 tokens
// per workgroup that is 589 workgroups of 1024 threads, more than the chip holds at once (two per CU), and the kernel
// takes two rounds of a workgroup whose time is mostly latency; at 16384 it is 310 and one round.
constexpr int kSelChunk = 16384;
constexpr int kSelThreads = 1024;  // 8 tokens per thread
constexpr int kMaxRows = 16;
constexpr uint64_t kNoKey = ~0ull;
constexpr int kNoNan = 0x7fffffff;

// Ascending bitonic sort of n (power of two, <= 2 * blockDim.x) keys in LDS.
__device__ void bitonic_sort(uint64_t *keys, int n) {
    for (int size = 2; size <= n; size <<= 1) {
        for (int stride = size >> 1; stride > 0; stride >>= 1) {
            __syncthreads();
            for (int i = threadIdx.x; i < n / 2; i += blockDim.x) {
                int lo = 2 * i - (i & (stride - 1));  // index with the `stride` bit clear
                int hi = lo + stride;
                bool up = (lo & size) == 0;
                uint64_t a = keys[lo], b = keys[hi];
                if ((a > b) == up) {
                    keys[lo] = b;
                    keys[hi] = a;
                }
            }
        }
    }
    __syncthreads();
}

// ------------------------------------------------------------------------------------------
// argmax_top2: IEEE comparisons, lowest index on ties, second value counts duplicates
// ------------------------------------------------------------------------------------------
struct Top2 {
    float v1;
    uint32_t i1;
    float v2;
};

__device__ __forceinline__ Top2 top2_merge(Top2 a, Top2 b) {
    if (b.v1 > a.v1 || (b.v1 == a.v1 && b.i1 < a.i1)) {
        Top2 t = a;
        a = b;
        b = t;
    }
    if (b.v1 > a.v2) a.v2 = b.v1;
    if (b.v2 > a.v2) a.v2 = b.v2;
    return a;
}

__global__ void __launch_bounds__(kSelThreads)
    top2_chunk_kernel(const float *__restrict__ logits, int64_t vocab, int64_t stride, Top2 *__restrict__ part) {
    __shared__ Top2 sh[kSelThreads];
    const int row = blockIdx.y, chunk = blockIdx.x;
    const float *x = logits + row * stride;
    Top2 t = {-INFINITY, 0xffffffffu, -INFINITY};
#pragma unroll
    for (int j = 0; j < kChunk / kSelThreads; j++) {
        int64_t i = static_cast<int64_t>(chunk) * kChunk + j * kSelThreads + threadIdx.x;
        if (i < vocab) {
            float v = x[i];
            if (v > t.v1) {
                t.v2 = t.v1;
                t.v1 = v;
                t.i1 = static_cast<uint32_t>(i);
            } else if (v == t.v1 && static_cast<uint32_t>(i) < t.i1) {
                t.v2 = t.v1;
                t.i1 = static_cast<uint32_t>(i);
            } else if (v > t.v2) {
                t.v2 = v;
            }
        }
    }
    sh[threadIdx.x] = t;
    for (int s = kSelThreads / 2; s > 0; s >>= 1) {
        __syncthreads();
        if (threadIdx.x < s) sh[threadIdx.x] = top2_merge(sh[threadIdx.x], sh[threadIdx.x + s]);
    }
    if (threadIdx.x == 0) part[row * gridDim.x + chunk] = sh[0];
}

__global__ void top2_final_kernel(const Top2 *__restrict__ part, int n_chunks, int32_t *__restrict__ idx,
                                  float *__restrict__ gap) {
    const int row = blockIdx.x;
    if (threadIdx.x != 0) return;
    Top2 t = part[row * n_chunks];
    for (int c = 1; c < n_chunks; c++) t = top2_merge(t, part[row * n_chunks + c]);
    idx[row] = static_cast<int32_t>(t.i1);
    gap[row] = t.v1 - t.v2;
}

// ------------------------------------------------------------------------------------------
// chunk selection: best K keys of a chunk (sorted), lowest NaN index, optional second row set
// ------------------------------------------------------------------------------------------
struct ChunkOut {
    uint64_t keys[kMaxK];
    int32_t nan_first;
    int32_t pad;
};

// min over the workgroup of a key / an int, result broadcast
__device__ uint64_t block_min_u64(uint64_t v, uint64_t *sh) {
    for (int off = 32; off > 0; off >>= 1) {
        uint64_t o = __shfl_xor(v, off, 64);
        v = o < v ? o : v;
    }
    __syncthreads();
    if ((threadIdx.x & 63) == 0) sh[threadIdx.x >> 6] = v;
    __syncthreads();
    uint64_t r = sh[0];
    for (int w = 1; w < static_cast<int>(blockDim.x >> 6); w++) r = sh[w] < r ? sh[w] : r;
    return r;
}

// Ascending sort of one key per lane over the wave (bitonic network of 21 compare-exchange steps between lanes: no
// LDS arrays, no barriers).
__device__ __forceinline__ uint64_t wave_sort_u64(uint64_t v) {
    const int lane = threadIdx.x & 63;
#pragma unroll
    for (int size = 2; size <= 64; size <<= 1) {
#pragma unroll
        for (int stride = size >> 1; stride > 0; stride >>= 1) {
            const uint32_t lo = __shfl_xor(static_cast<uint32_t>(v), stride, 64), hi = __shfl_xor(static_cast<uint32_t>(v >> 32), stride, 64);
            const uint64_t o = (static_cast<uint64_t>(hi) << 32) | lo;
            const bool lower = (lane & stride) == 0, ascending = (lane & size) == 0;
            const uint64_t mn = v < o ? v : o, mx = v < o ? o : v;
            v = (lower == ascending) ? mn : mx;
        }
    }
    return v;
}

// Minimum of a key over the wave, in every lane: data-parallel-primitive moves within rows of 16 lanes (shift right
// by 1, 2, 4, 8: lane 15 of a row then holds the row's minimum), then lane 15 of rows 0 and 2 into rows 1 and 3, then
// lane 31 into rows 2 and 3; lane 63 has the result.  Lanes without a source read the identity.  No LDS round trips.
__device__ __forceinline__ uint64_t wave_min_u64(uint64_t v) {
#define DFL_MIN_STEP(ctrl, row_mask)                                                                                     \
    do {                                                                                                                 \
        const unsigned lo = __builtin_amdgcn_update_dpp(0xffffffffu, static_cast<unsigned>(v), ctrl, row_mask, 0xf, false);       \
        const unsigned hi = __builtin_amdgcn_update_dpp(0xffffffffu, static_cast<unsigned>(v >> 32), ctrl, row_mask, 0xf, false); \
        const uint64_t o = (static_cast<uint64_t>(hi) << 32) | lo;                                                       \
        v = o < v ? o : v;                                                                                               \
    } while (0)
    DFL_MIN_STEP(0x111, 0xf);  // row_shr:1
    DFL_MIN_STEP(0x112, 0xf);  // row_shr:2
    DFL_MIN_STEP(0x114, 0xf);  // row_shr:4
    DFL_MIN_STEP(0x118, 0xf);  // row_shr:8
    DFL_MIN_STEP(0x142, 0xa);  // row_bcast:15 into rows 1 and 3
    DFL_MIN_STEP(0x143, 0xc);  // row_bcast:31 into rows 2 and 3
#undef DFL_MIN_STEP
    const unsigned lo = __builtin_amdgcn_readlane(static_cast<unsigned>(v), 63);
    const unsigned hi = __builtin_amdgcn_readlane(static_cast<unsigned>(v >> 32), 63);
    return (static_cast<uint64_t>(hi) << 32) | lo;
}

// The k smallest keys, in order, of n_lists <= 64 ascending lists of k keys each (list l at base + l * stride; missing
// keys are kNoKey, at the end), by ONE wave: lane l holds the head of list l, a step takes the minimum of the heads
// and advances the list it came from (keys are distinct).  Returns the k-th; with `out`, out[0 .. k) gets them all.
// (Measured in the selection kernel, k = 20: 3.3 us; every published key searching the sixteen lists instead, spread
// over all 1024 threads, 5.7 us: the waves of a workgroup share four instruction issuers, and the index arithmetic
// of 5120 searches costs more than twenty dependent steps of one wave.)
__device__ __forceinline__ uint64_t wave_merge_lists(const uint64_t *base, int n_lists, int stride, int k, uint64_t *out) {
    const int lane = threadIdx.x & 63;
    const bool own = lane < n_lists;
    const uint64_t *list = base + (own ? lane : 0) * stride;
    int pos = 0;
    uint64_t head = own ? list[0] : kNoKey;
    uint64_t next = (own && k > 1) ? list[1] : kNoKey;  // fetched one step ahead of its use
    uint64_t m = kNoKey;
    for (int step = 0; step < k; step++) {
        m = wave_min_u64(head);
        if (out && lane == 0) out[step] = m;
        if (own && head == m && m != kNoKey) {
            head = next;
            pos++;
            next = pos + 1 < k ? list[pos + 1] : kNoKey;
        }
    }
    return m;
}

// below[j] = number of keys below x[j] in the ascending list of 1 <= n <= kMaxK keys at base + off[j], four binary
// searches in lockstep: a probe is an LDS read the next one depends on, and a thread that runs its searches one
// after the other spends its time waiting for them.  step0 = the largest power of two <= n.
__device__ __forceinline__ void count_below4(const uint64_t *base, const int (&off)[4], int n, int step0, const uint64_t (&x)[4],
                                             int (&below)[4]) {
#pragma unroll
    for (int j = 0; j < 4; j++) below[j] = 0;
    for (int step = step0; step >= 1; step >>= 1) {
        uint64_t v[4];
        int probe[4];
#pragma unroll
        for (int j = 0; j < 4; j++) {
            probe[j] = below[j] + step;
            v[j] = base[off[j] + (probe[j] <= n ? probe[j] : n) - 1];
        }
#pragma unroll
        for (int j = 0; j < 4; j++) below[j] = (probe[j] <= n && v[j] < x[j]) ? probe[j] : below[j];
    }
}

// K == 1 fast path is the greedy / draft-max case: only the minimum key is needed.
//
// K > 1, without a sort over the workgroup (a bitonic network in LDS is one workgroup barrier per step, 91 steps
// here): every wave sorts its 64 per-thread bests between its lanes and publishes the first k; the k-th best of all
// 1024 per-thread bests (it bounds every winner of the chunk) is the k-th key of the merge of the sixteen published
// lists, which wave 0 runs; the at most 16 k elements at or below that bound are then ranked by counting the
// candidates below each, and a candidate of rank r < k is output r.  Keys are distinct (the token id is in the low
// bits), so ranks are too.
__device__ __forceinline__ void select_chunk_body(const float *__restrict__ logits, int64_t vocab, int64_t stride, int k,
                                                  ChunkOut *__restrict__ out, bool nan_is_candidate, int row) {
    __shared__ uint64_t sk[kSelThreads];  // k == 1: scratch of the minimum; else [16 waves][kMaxK] published bests
    __shared__ uint64_t cand[(kSelChunk / kSelThreads) * kMaxK];
    __shared__ uint64_t outk[kMaxK];
    __shared__ uint64_t tau_sh;
    __shared__ int rank_sh[kSelThreads];  // [16 waves][kMaxK] published bests, then the candidates (at most as many)
    __shared__ int cnt;
    __shared__ int nan_sh;
    const int chunk = blockIdx.x, tid = threadIdx.x;
    const float *x = logits + row * stride;
    uint64_t keys[kSelChunk / kSelThreads];
    uint64_t best = kNoKey;
    int nan_first = kNoNan;
    if (tid == 0) {
        cnt = 0;
        nan_sh = kNoNan;
    }
#pragma unroll
    for (int j = 0; j < kSelChunk / kSelThreads; j++) {
        int64_t i = static_cast<int64_t>(chunk) * kSelChunk + j * kSelThreads + tid;
        uint64_t key = kNoKey;
        if (i < vocab) {
            float v = x[i];
            if (v != v) {
                nan_first = nan_first < static_cast<int>(i) ? nan_first : static_cast<int>(i);
                if (nan_is_candidate) key = cand_key(static_cast<uint32_t>(i), v);
            } else {
                key = cand_key(static_cast<uint32_t>(i), v);
            }
        }
        keys[j] = key;
        best = key < best ? key : best;
    }
    __syncthreads();
    if (nan_first != kNoNan) atomicMin(&nan_sh, nan_first);
    ChunkOut *o = out + (row * gridDim.x + chunk);
    if (k == 1) {
        uint64_t m = block_min_u64(best, sk);
        if (tid == 0) {
            o->keys[0] = m;
            o->nan_first = nan_sh;
        }
        return;
    }
    // k-th best of the per-thread bests bounds every winner of the chunk
    const int lane = tid & 63, wave = tid >> 6;
    const uint64_t sorted = wave_sort_u64(best);
    if (lane < k) sk[wave * kMaxK + lane] = sorted;
    if (tid < kMaxK) outk[tid] = kNoKey;
    rank_sh[tid] = 0;
    __syncthreads();
    // the k-th best of the sixteen published lists: wave 0 merges them (fewer than k keys in all: kNoKey, and every
    // key of the chunk is a candidate)
    if (wave == 0) {
        const uint64_t kth = wave_merge_lists(sk, kSelThreads / 64, kMaxK, k, nullptr);
        if (lane == 0) tau_sh = kth;
    }
    __syncthreads();
    const uint64_t tau = tau_sh;
    if (best <= tau && best != kNoKey) {
#pragma unroll
        for (int j = 0; j < kSelChunk / kSelThreads; j++)
            if (keys[j] <= tau && keys[j] != kNoKey) cand[atomicAdd(&cnt, 1)] = keys[j];
    }
    __syncthreads();
    const int n_cand = cnt;  // <= 16 k <= kSelThreads
    if (n_cand > 0) {
        // candidate i = tid % n_cand counts the candidates below it in slice tid / n_cand of the list
        const int slices = kSelThreads / n_cand, i = tid % n_cand, sl = tid / n_cand;
        if (sl < slices) {
            const int per = (n_cand + slices - 1) / slices, j0 = sl * per, j1 = min(n_cand, j0 + per);
            const uint64_t key = cand[i];
            int c = 0;
            for (int j = j0; j < j1; j++) c += cand[j] < key;
            if (c) atomicAdd(&rank_sh[i], c);
        }
    }
    __syncthreads();
    if (tid < n_cand && rank_sh[tid] < k) outk[rank_sh[tid]] = cand[tid];
    __syncthreads();
    if (tid < k) o->keys[tid] = outk[tid];
    if (tid == 0) o->nan_first = nan_sh;
}

__global__ void __launch_bounds__(kSelThreads)
    select_chunk_kernel(const float *__restrict__ logits, int64_t vocab, int64_t stride, int k,
                        ChunkOut *__restrict__ out, bool nan_is_candidate) {
    select_chunk_body(logits, vocab, stride, k, out, nan_is_candidate, blockIdx.y);
}

// Two row sets in one launch: rows [0, n_a) of a (best k_a keys of every chunk), then the rows of b (best key).
__global__ void __launch_bounds__(kSelThreads)
    select_pair_kernel(const float *__restrict__ a, int n_a, int k_a, ChunkOut *__restrict__ out_a, const float *__restrict__ b,
                       ChunkOut *__restrict__ out_b, int64_t vocab, int64_t stride) {
    const int row = blockIdx.y;
    if (row < n_a)
        select_chunk_body(a, vocab, stride, k_a, out_a, false, row);
    else
        select_chunk_body(b, vocab, stride, 1, out_b, false, row - n_a);
}

// The dense proposal's side of a row: its largest draft logit (scaled) and NaN / no-candidate errors.
__device__ void merge_draft_side(const ChunkOut *__restrict__ draft_chunks, int n_chunks, int row, const ChainCfg &cfg, RowDist *d) {
    uint64_t best = kNoKey;
    int dn = kNoNan;
    for (int c = 0; c < n_chunks; c++) {
        const ChunkOut &dc = draft_chunks[row * n_chunks + c];
        best = dc.keys[0] < best ? dc.keys[0] : best;
        dn = dc.nan_first < dn ? dc.nan_first : dn;
    }
    d->d_err = 0;
    d->d_err_index = -1;
    d->d_max_scaled = static_cast<double>(key_logit(best)) / static_cast<double>(cfg.draft_temperature);
    if (dn != kNoNan) {
        d->d_err = DFLASH_ERR_NAN_LOGIT;
        d->d_err_index = dn;
    } else if (!isfinite(d->d_max_scaled)) {
        d->d_err = DFLASH_ERR_NO_CANDIDATES;
    }
}

// One workgroup per row: merge the chunk lists, order the best k, run the chain (wave 0, a candidate per lane).
__device__ __forceinline__ void row_merge_body(const ChunkOut *__restrict__ chunks, int n_chunks,
                                               const ChunkOut *__restrict__ draft_chunks, const ChainCfg &cfg,
                                               RowDist *__restrict__ rows, int32_t *__restrict__ greedy_out, bool draft_only,
                                               int row) {
    __shared__ uint64_t sk[2 * kSelThreads];
    const int tid = threadIdx.x;
    RowDist *d = rows + row;
    if (draft_only) {  // the target side of these rows was filled by the wide chain
        if (tid == 0) merge_draft_side(draft_chunks, n_chunks, row, cfg, d);
        return;
    }
    // The chunks' lists are ascending: the rank of a key among all of them is the sum, over the lists, of the keys
    // below it (binary searches); the keys of rank < k, in rank order, are the row's candidates, best first.
    const int k = cfg.k;
    const int n_in = n_chunks * k;  // <= 2048, checked on the host
    __shared__ uint64_t lists[2 * kSelThreads];
    __shared__ int rank_sh[2 * kSelThreads];
    __shared__ uint64_t red[kSelThreads / 64];
    if (tid < kMaxK) sk[tid] = kNoKey;
    uint64_t mine = kNoKey;
    for (int i = tid; i < n_in; i += kSelThreads) {
        const uint64_t key = chunks[row * n_chunks + i / k].keys[i % k];
        lists[i] = key;
        rank_sh[i] = 0;
        mine = key < mine ? key : mine;
    }
    if (k == 1) {
        mine = block_min_u64(mine, red);
        if (tid == 0) sk[0] = mine;
    } else {
        __syncthreads();
        // (key, list) pairs over all threads: a thread's searches are independent of each other
        // (consecutive threads: consecutive keys against the same list, so that a wave's probes fall on different
        // banks and its additions on different counters)
        const int step0 = 1 << (31 - __clz(k));
        for (int p0 = tid; p0 < n_in * n_chunks; p0 += 4 * kSelThreads) {
            int off[4], slot[4], below[4];
            uint64_t key[4];
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const int p = p0 + j * kSelThreads;
                const bool live = p < n_in * n_chunks;
                const int c = live ? p / n_in : 0;
                slot[j] = live ? p - c * n_in : 0;
                off[j] = c * k;
                key[j] = live ? lists[slot[j]] : 0;  // (nothing is below key 0)
            }
            count_below4(lists, off, k, step0, key, below);
#pragma unroll
            for (int j = 0; j < 4; j++)
                if (below[j] && key[j] != kNoKey) atomicAdd(&rank_sh[slot[j]], below[j]);
        }
        __syncthreads();
        for (int i = tid; i < n_in; i += kSelThreads)
            if (lists[i] != kNoKey && rank_sh[i] < k) sk[rank_sh[i]] = lists[i];
    }
    __syncthreads();
    if (tid >= 64) {
        // the dense proposal's side is independent of the target's: the first lane of the second wave takes it
        if (tid == 64 && draft_chunks) merge_draft_side(draft_chunks, n_chunks, row, cfg, d);
        return;
    }
    int nan_first = kNoNan;
    for (int c = tid; c < n_chunks; c += 64) {
        int nf = chunks[row * n_chunks + c].nan_first;
        nan_first = nf < nan_first ? nf : nan_first;
    }
    for (int off = 32; off > 0; off >>= 1) nan_first = min(nan_first, __shfl_xor(nan_first, off, 64));
    if (tid == 0) {
        d->n_keep = 0;
        d->err = 0;
        d->err_index = -1;
        d->total = 0.0;
        if (!draft_chunks) {
            d->d_err = 0;
            d->d_err_index = -1;
        }
        if (greedy_out) greedy_out[row] = nan_first != kNoNan ? ~nan_first : key_token(sk[0]);
    }
    if (nan_first != kNoNan) {
        if (tid == 0) {
            d->err = DFLASH_ERR_NAN_LOGIT;
            d->err_index = nan_first;
        }
    } else if (cfg.temperature == 0.0f) {
        // greedy target: one-hot on the total-order argmax (sampling.rs:391-400)
        if (tid == 0) {
            d->n_keep = 1;
            d->total = 1.0;
            d->tokens[0] = key_token(sk[0]);
            d->weights[0] = 1.0;
        }
    } else {
        const int len = __popcll(__builtin_amdgcn_ballot_w64(tid < k && sk[tid < k ? tid : 0] != kNoKey));  // (missing keys sort last)
        run_chain_wave(sk, len, cfg, d);
    }
}

__global__ void __launch_bounds__(kSelThreads)
    row_merge_kernel(const ChunkOut *__restrict__ chunks, int n_chunks, const ChunkOut *__restrict__ draft_chunks,
                     ChainCfg cfg, RowDist *__restrict__ rows, int32_t *__restrict__ greedy_out, bool draft_only) {
    row_merge_body(chunks, n_chunks, draft_chunks, cfg, rows, greedy_out, draft_only, blockIdx.x);
}

// top-16 output from the merged order
__global__ void __launch_bounds__(kSelThreads)
    top16_merge_kernel(const ChunkOut *__restrict__ chunks, int n_chunks, int32_t *__restrict__ ids,
                       float *__restrict__ vals) {
    __shared__ uint64_t sk[2 * kSelThreads];
    const int row = blockIdx.x, tid = threadIdx.x;
    const int n_in = n_chunks * 16;
    int n_sort = 16;
    while (n_sort < n_in) n_sort <<= 1;
    for (int i = tid; i < n_sort; i += kSelThreads) sk[i] = i < n_in ? chunks[row * n_chunks + i / 16].keys[i % 16] : kNoKey;
    bitonic_sort(sk, n_sort);
    if (tid < 16) {
        uint64_t key = sk[tid];
        ids[row * 16 + tid] = key == kNoKey ? -1 : key_token(key);
        vals[row * 16 + tid] = key == kNoKey ? -INFINITY : key_logit(key);
    }
}

// The rows' chains and the dense proposal's tile sums in one launch (neither needs the other; both need only the
// chunk selection): workgroups [0, n_rows) are row_merge_kernel's, the rest take eight 1024-token tiles each of draft
// row (workgroup - n_rows) / blocks_per_row.  A tile sum is the sum of exp(d/T - max/T) in a fixed shape: slot t of
// a tile holds ((e[4t]+e[4t+1])+e[4t+2])+e[4t+3], then a halving tree over the 256 slots; max is the row's largest
// draft logit, which every tile workgroup takes from the chunk minima itself.
__global__ void __launch_bounds__(kSelThreads)
    rows_and_tiles_kernel(const ChunkOut *__restrict__ chunks, int n_chunks, const ChunkOut *__restrict__ draft_chunks, ChainCfg cfg,
                          RowDist *__restrict__ rows, int n_rows, bool draft_only, const float *__restrict__ draft, int64_t vocab,
                          int64_t stride, int n_tiles, int blocks_per_row, double *__restrict__ tile_sums) {
    if (static_cast<int>(blockIdx.x) < n_rows) {
        row_merge_body(chunks, n_chunks, draft_chunks, cfg, rows, nullptr, draft_only, blockIdx.x);
        return;
    }
    __shared__ double slot[4][256];
    __shared__ uint64_t red[kSelThreads / 64];
    const int b = blockIdx.x - n_rows, row = b / blocks_per_row, q = threadIdx.x >> 8, t = threadIdx.x & 255;
    uint64_t best = kNoKey;
    for (int c = threadIdx.x; c < n_chunks; c += kSelThreads) {
        const uint64_t key = draft_chunks[row * n_chunks + c].keys[0];
        best = key < best ? key : best;
    }
    best = block_min_u64(best, red);
    const double T = static_cast<double>(cfg.draft_temperature);
    const double mx = static_cast<double>(key_logit(best)) / T;  // merge_draft_side's d_max_scaled
    const float *x = draft + row * stride;
    // (eight tiles per workgroup, two per quarter: with four, a 15-row block is more workgroups than the chip holds
    // at once)
    for (int half = 0; half < 2; half++) {
        const int tile = (b - row * blocks_per_row) * 8 + 4 * half + q;
        const int64_t base = static_cast<int64_t>(tile) * 1024 + 4 * t;
        double acc = 0.0;
#pragma unroll
        for (int e = 0; e < 4; e++) {
            int64_t i = base + e;
            double v = (tile < n_tiles && i < vocab) ? exp(static_cast<double>(x[i]) / T - mx) : 0.0;
            acc = (e == 0) ? v : acc + v;
        }
        __syncthreads();  // (the previous half's sums have been read)
        slot[q][t] = acc;
        for (int s = 128; s >= 1; s >>= 1) {
            __syncthreads();
            if (t < s) slot[q][t] += slot[q][t + s];
        }
        if (t == 0 && tile < n_tiles) tile_sums[row * n_tiles + tile] = slot[q][0];
    }
}

struct DecideArgs {
    int32_t n_tokens, n_stop, mode, vocab;
    int64_t budget;
    // The block's small host inputs travel by value, in the kernel arguments: a pageable host-to-device copy
    // of a few bytes costs several microseconds of idle GPU each.
    int32_t verified[kMaxRows];      // [n_tokens]
    double uniforms[kMaxRows + 2];   // [n_tokens + 1]
    int32_t prop_offsets[kMaxRows], prop_counts[kMaxRows];  // sparse proposals: row r's candidates in prop_cands
    const int32_t *stop_ids;   // [n_stop]
    const RowDist *rows;
    const dflash_weighted_candidate *prop_cands;
    // dense proposals
    const float *draft;
    int64_t draft_stride;
    const double *tile_sums;
    int32_t n_tiles;
    float temperature, draft_temperature;
    // wide candidate sets (effective top-k above kMaxK): row r's kept candidates are the first n_keep sorted keys
    // / weights at r * wide_stride of these arrays instead of the arrays inside RowDist; null otherwise
    const uint64_t *wide_keys;
    const double *wide_w;
    int64_t wide_stride;
};

// A row's kept candidates, wherever they live.
struct DistView {
    const RowDist *rd;
    const uint64_t *keys;  // null: inline arrays of rd
    const double *w;
    __device__ int32_t token(int i) const { return keys ? static_cast<int32_t>(keys[i] & kWideTokenMask) : rd->tokens[i]; }
    __device__ double weight(int i) const { return w ? w[i] : rd->weights[i]; }
};

// first candidate whose running sum exceeds x, else the last (sampling.rs:1587-1596)
__device__ int pick_index_view(const DistView &v, int n, double x) {
    double cumulative = 0.0;
    for (int i = 0; i < n; i++) {
        cumulative += v.weight(i);
        if (x < cumulative) return i;
    }
    return n - 1;
}

__device__ bool in_list(const int32_t *ids, int n, int32_t v) {
    for (int i = 0; i < n; i++)
        if (ids[i] == v) return true;
    return false;
}

// What one row of the walk comes to, given that every row before it accepted.
struct RowOutcome {
    int32_t acc;         // the draft is accepted (draft rows only)
    int32_t token;       // correction token (rejected draft row) or bonus token (last row)
    int32_t draws;       // random draws this row consumes
    int32_t err;         // DFLASH_ERR_* of this row, 0 if none
    int64_t err_index;
    // a rejected row under a stochastic proposal: its correction token is still to be drawn from the residual
    // distribution (residual_pick, by the whole wave, for the one row the walk stops at)
    int32_t need_residual;
    int32_t residual_draw;  // index of the uniform draw the pick uses
    double prop_total;
};

// One row of accept.rs:147-183 with the couplings of sampling.rs:692-790.  A row that is reached has seen only
// accepting rows before it, and an accepting row consumes exactly one draw (none when greedy): row r therefore
// starts at draw r whatever the rows before it held, which is what lets every row be evaluated at once.
__device__ RowOutcome decide_row(const DecideArgs &a, const RowDist *rows, int row, const double *p_total,
                                 const float *draft_tok_logit) {
    RowOutcome o = {0, 0, 0, 0, -1, 0, 0, 0.0};
    const int n_drafts = a.n_tokens - 1;
    const bool greedy = a.temperature == 0.0f;
    const RowDist &rd = rows[row];
    const DistView dv = {&rd, a.wide_keys ? a.wide_keys + row * a.wide_stride : nullptr,
                         a.wide_w ? a.wide_w + row * a.wide_stride : nullptr};
    int draws = greedy ? 0 : row;
    const int draws0 = draws;
    if (row == n_drafts) {  // bonus = sample(last reached row)
        if (rd.err) {
            o.err = rd.err;
            o.err_index = rd.err_index;
            return o;
        }
        int idx = 0;
        if (!greedy) idx = pick_index_view(dv, rd.n_keep, a.uniforms[draws++] * rd.total);
        o.token = dv.token(idx);
        o.draws = draws - draws0;
        return o;
    }
    const int32_t draft = a.verified[row + 1];
    if (a.mode == 0) {  // deterministic coupling: draw the target token, accept iff it is the draft
        if (rd.err) {
            o.err = rd.err;
            o.err_index = rd.err_index;
            return o;
        }
        int idx = 0;
        if (!greedy) idx = pick_index_view(dv, rd.n_keep, a.uniforms[draws++] * rd.total);
        o.token = dv.token(idx);
        o.acc = o.token == draft;
        o.draws = draws - draws0;
        return o;
    }
    // proposal probability q(draft) and, per target candidate, q(candidate)
    double prop_total = 0.0, prop_tok_w = 0.0;
    const dflash_weighted_candidate *pc = nullptr;
    int n_pc = 0;
    if (a.mode == 1) {
        pc = a.prop_cands + a.prop_offsets[row];
        n_pc = a.prop_counts[row];
        if (n_pc == 0) o.err = DFLASH_ERR_NO_CANDIDATES;
        for (int j = 0; j < n_pc && !o.err; j++) {
            if (!isfinite(pc[j].weight) || pc[j].weight < 0.0) {
                o.err = DFLASH_ERR_INVALID_PROPOSAL_WEIGHT;
                o.err_index = pc[j].token;
                break;
            }
            prop_total += pc[j].weight;
            if (pc[j].token == draft) prop_tok_w += pc[j].weight;
        }
        if (!o.err && !(isfinite(prop_total) && prop_total > 0.0)) o.err = DFLASH_ERR_NO_CANDIDATES;
        if (!o.err && !(isfinite(prop_tok_w) && prop_tok_w > 0.0)) {
            o.err = DFLASH_ERR_MISSING_PROPOSAL_TOKEN;
            o.err_index = draft;
        }
    } else {
        if (rd.d_err) {
            o.err = rd.d_err;
            o.err_index = rd.d_err_index;
        }
        prop_total = p_total[row];
        if (!o.err && !(isfinite(prop_total) && prop_total > 0.0)) o.err = DFLASH_ERR_NO_CANDIDATES;
        if (!o.err) {
            // (draft_tok_logit[row] = a.draft[row][draft], fetched ahead)
            prop_tok_w = exp(static_cast<double>(draft_tok_logit[row]) / static_cast<double>(a.draft_temperature) - rd.d_max_scaled);
            if (!(isfinite(prop_tok_w) && prop_tok_w > 0.0)) {
                o.err = DFLASH_ERR_MISSING_PROPOSAL_TOKEN;
                o.err_index = draft;
            }
        }
    }
    if (!o.err && rd.err) {
        o.err = rd.err;
        o.err_index = rd.err_index;
    }
    if (o.err) return o;
    double tp = -0.0;
    for (int i = 0; i < rd.n_keep; i++)
        if (dv.token(i) == draft) tp += dv.weight(i);
    const double target_probability = tp / rd.total;
    const double proposal_probability = prop_tok_w / prop_total;
    const double acceptance = fmin(target_probability / proposal_probability, 1.0);
    if (a.uniforms[draws++] < acceptance) {
        o.acc = 1;
    } else {
        // the correction token comes from the residual distribution: one more draw
        o.need_residual = 1;
        o.residual_draw = draws++;
        o.prop_total = prop_total;
    }
    o.draws = draws - draws0;
    return o;
}

// The correction token of rejected row `row`: residual weights max(p_i - q_i, 0) in the target's order
// (sampling.rs:752-790), summed first, then walked again for the pick; the second pass recomputes the same values,
// so no per-candidate array is needed.  By the whole wave: lane j computes the weight of candidate base + j (one f64
// exponential each under a dense proposal, the expensive part), and the sums add those values in candidate order,
// one addition after the other.
__device__ void residual_pick(const DecideArgs &a, const RowDist *rows, int row, RowOutcome &o, const float *draft_logit_of) {
    const int lane = threadIdx.x & 63;
    const RowDist &rd = rows[row];
    const DistView dv = {&rd, a.wide_keys ? a.wide_keys + row * a.wide_stride : nullptr,
                         a.wide_w ? a.wide_w + row * a.wide_stride : nullptr};
    const dflash_weighted_candidate *pc = a.mode == 1 ? a.prop_cands + a.prop_offsets[row] : nullptr;
    const int n_pc = a.mode == 1 ? a.prop_counts[row] : 0;
    const double prop_total = o.prop_total;
    auto residual_at = [&](int i) {
        const double p = dv.weight(i) / rd.total;
        double q;
        if (a.mode == 1) {
            const int32_t ti = dv.token(i);
            double qs = -0.0;
            for (int j = 0; j < n_pc; j++)
                if (pc[j].token == ti) qs += pc[j].weight;
            q = qs / prop_total;
        } else {
            // (draft_logit_of: the row's candidates' draft logits, fetched ahead; else they are read here)
            const float dl = draft_logit_of ? draft_logit_of[i] : a.draft[row * a.draft_stride + dv.token(i)];
            q = exp(static_cast<double>(dl) / static_cast<double>(a.draft_temperature) - rd.d_max_scaled) / prop_total;
        }
        return fmax(p - q, 0.0);
    };
    const int n_keep = rd.n_keep;
    double residual_total = 0.0;
    for (int base = 0; base < n_keep; base += 64) {
        const double r = base + lane < n_keep ? residual_at(base + lane) : 0.0;
        const int m = min(64, n_keep - base);
        for (int j = 0; j < m; j++) residual_total += chain_bcast(r, j);
    }
    if (!(isfinite(residual_total) && residual_total > 0.0)) {
        o.err = DFLASH_ERR_NO_CANDIDATES;
        return;
    }
    const double x = a.uniforms[o.residual_draw] * residual_total;
    int pick = n_keep - 1;
    double cumulative = 0.0;
    bool found = false;
    for (int base = 0; base < n_keep && !found; base += 64) {
        const double r = base + lane < n_keep ? residual_at(base + lane) : 0.0;
        const int m = min(64, n_keep - base);
        for (int j = 0; j < m; j++) {
            cumulative += chain_bcast(r, j);
            if (x < cumulative) {
                pick = base + j;
                found = true;
                break;
            }
        }
    }
    o.token = dv.token(pick);
}

// Thread r evaluates row r (all rows at once); thread 0 then walks the outcomes in order exactly as the serial
// loop of accept.rs:147-183 does: rows behind the first rejection, stop or error are never looked at.
__global__ void __launch_bounds__(64) decide_kernel(DecideArgs a, dflash_accept_decision *__restrict__ out) {
    constexpr int kStage = 256;  // tile sums per row and round
    __shared__ double p_total[kMaxRows];
    __shared__ RowOutcome outcome[kMaxRows + 1];
    // the rows' distributions are walked element by element: they are copied to LDS once, coalesced
    __shared__ RowDist rows_sh[kMaxRows];
    __shared__ double staged[kMaxRows][kStage];
    __shared__ float draft_tok_logit[kMaxRows];
    __shared__ float resid_logit[kMaxRows][kMaxK];
    static_assert(sizeof(RowDist) % 8 == 0, "copied as double words");
    const int tid = threadIdx.x;
    const int n_drafts = a.n_tokens - 1;
    const bool dense = a.mode == 2;
    // What the kernel reads from memory is written by other XCDs and comes from memory at about two microseconds a
    // trip: everything whose address is known is requested before anything is waited for (the first round of tile
    // sums, each draft row's logit of its own draft token, the rows), the candidates' draft logits as soon as the
    // rows are there, and the arithmetic runs on LDS copies.
    double tsum[kMaxRows - 1][kStage / 64];
    float my_logit = 0.0f;
    if (dense) {
#pragma unroll
        for (int r = 0; r < kMaxRows - 1; r++)
#pragma unroll
            for (int u = 0; u < kStage / 64; u++) {
                const int t = u * 64 + tid;
                tsum[r][u] = (r < n_drafts && t < a.n_tiles) ? a.tile_sums[r * a.n_tiles + t] : 0.0;
            }
        if (tid < n_drafts) my_logit = a.draft[tid * a.draft_stride + a.verified[tid + 1]];
    }
    {
        const uint64_t *src = reinterpret_cast<const uint64_t *>(a.rows);
        uint64_t *dst = reinterpret_cast<uint64_t *>(rows_sh);
        const int n_words = a.n_tokens * static_cast<int>(sizeof(RowDist) / 8);
        for (int base = 0; base < n_words; base += 64 * 8) {
            uint64_t v[8];
#pragma unroll
            for (int u = 0; u < 8; u++) v[u] = base + u * 64 + tid < n_words ? src[base + u * 64 + tid] : 0;
#pragma unroll
            for (int u = 0; u < 8; u++)
                if (base + u * 64 + tid < n_words) dst[base + u * 64 + tid] = v[u];
        }
    }
    if (dense) {
#pragma unroll
        for (int r = 0; r < kMaxRows - 1; r++)
#pragma unroll
            for (int u = 0; u < kStage / 64; u++) staged[r][u * 64 + tid] = tsum[r][u];
        if (tid < n_drafts) draft_tok_logit[tid] = my_logit;
    }
    __syncthreads();
    const bool prefetched = dense && !a.wide_keys;
    if (prefetched) {
        float v[kMaxRows - 1];
#pragma unroll
        for (int r = 0; r < kMaxRows - 1; r++)
            v[r] = (r < n_drafts && tid < rows_sh[r].n_keep) ? a.draft[r * a.draft_stride + rows_sh[r].tokens[tid]] : 0.0f;
#pragma unroll
        for (int r = 0; r < kMaxRows - 1; r++) resid_logit[r][tid] = v[r];
    }
    if (dense) {
        // P = sequential sum of a row's tile sums, in tile order, by thread r from the LDS copies
        double P = 0.0;
        for (int t0 = 0; t0 < a.n_tiles; t0 += kStage) {
            if (t0 > 0) {  // further rounds (vocabularies above 262144 tokens)
                __syncthreads();
                for (int r = 0; r < n_drafts; r++)
                    for (int u = 0; u < kStage / 64; u++) {
                        const int t = t0 + u * 64 + tid;
                        staged[r][u * 64 + tid] = t < a.n_tiles ? a.tile_sums[r * a.n_tiles + t] : 0.0;
                    }
                __syncthreads();
            }
            if (tid < n_drafts) {
                const int n = min(kStage, a.n_tiles - t0);
                for (int i = 0; i < n; i++) P += staged[tid][i];
            }
        }
        if (tid < n_drafts) p_total[tid] = P;
    }
    __syncthreads();
    if (tid <= n_drafts) outcome[tid] = decide_row(a, rows_sh, tid, p_total, draft_tok_logit);
    __syncthreads();
    // The walk, by every lane alike (the workgroup is one wave; everything it reads is uniform): at the row it stops
    // at, a rejected draft's correction token is drawn by the whole wave.  The decision is put together in LDS and
    // leaves as one coalesced store: `out` may be host memory, where every separate store is a transaction over the
    // bus.
    __shared__ dflash_accept_decision d_sh;
    static_assert(sizeof(dflash_accept_decision) % 4 == 0, "copied as words");
    int accepted = 0, draws = 0, carry_kind = DFLASH_CARRY_NONE, stop = DFLASH_STOP_NONE, carry_token = 0;
    int err = 0, err_row = -1;
    int64_t err_index = -1;
    for (;;) {
        const int row = accepted;
        RowOutcome o = outcome[row];
        if (!o.err && o.need_residual) residual_pick(a, rows_sh, row, o, prefetched ? resid_logit[row] : nullptr);
        if (o.err) {
            err = o.err;
            err_index = o.err_index;
            err_row = row;
            break;
        }
        draws += o.draws;
        if (row == n_drafts) {
            carry_kind = DFLASH_CARRY_BONUS;
            carry_token = o.token;
            break;
        }
        if (!o.acc) {
            carry_kind = DFLASH_CARRY_CORRECTION;
            carry_token = o.token;
            break;
        }
        const int32_t draft = a.verified[row + 1];
        accepted++;
        if (in_list(a.stop_ids, a.n_stop, draft)) {
            stop = DFLASH_STOP_EOS;
            break;
        }
        if (accepted == a.budget) {
            stop = DFLASH_STOP_TOKEN_LIMIT;
            break;
        }
    }
    if (threadIdx.x == 0) {
        dflash_accept_decision &d = d_sh;
        memset(&d, 0, sizeof(d));
        d.err_row = err_row;
        d.err_index = err_index;
        if (err) {
            d.err_code = err;
        } else {
            for (int i = 0; i < accepted; i++) d.accepted_drafts[i] = a.verified[i + 1];
            d.n_accepted = accepted;
            d.carry_kind = carry_kind;
            d.carry_token = carry_token;
            d.stop_reason = stop;
            d.retain_input_count = 1 + accepted - (stop != DFLASH_STOP_NONE ? 1 : 0);
            d.draws_used = draws;
        }
    }
    __syncthreads();
    {
        const uint32_t *src = reinterpret_cast<const uint32_t *>(&d_sh);
        uint32_t *dst = reinterpret_cast<uint32_t *>(out);
        for (int i = threadIdx.x; i < static_cast<int>(sizeof(dflash_accept_decision) / 4); i += blockDim.x) dst[i] = src[i];
    }
}

// ------------------------------------------------------------------------------------------
// host: random streams (sampling.rs:1621-1670; Philox4x32-10 after Salmon et al.)
// ------------------------------------------------------------------------------------------
uint64_t splitmix_next(uint64_t &state) {
    state += 0x9e3779b97f4a7c15ull;
    uint64_t v = state;
    v = (v ^ (v >> 30)) * 0xbf58476d1ce4e5b9ull;
    v = (v ^ (v >> 27)) * 0x94d049bb133111ebull;
    return v ^ (v >> 31);
}
uint64_t rotl64(uint64_t x, int k) { return (x << k) | (x >> (64 - k)); }
uint64_t xoshiro_next(uint64_t s[4]) {
    uint64_t result = rotl64(s[0] + s[3], 23) + s[0];
    uint64_t t = s[1] << 17;
    s[2] ^= s[0];
    s[3] ^= s[1];
    s[1] ^= s[2];
    s[0] ^= s[3];
    s[2] ^= t;
    s[3] = rotl64(s[3], 45);
    return result;
}
void philox4x32_10(const uint32_t ctr[4], const uint32_t key[2], uint32_t out[4]) {
    uint32_t c0 = ctr[0], c1 = ctr[1], c2 = ctr[2], c3 = ctr[3], k0 = key[0], k1 = key[1];
    for (int r = 0; r < 10; r++) {
        uint64_t p0 = static_cast<uint64_t>(0xD2511F53u) * c0;
        uint64_t p1 = static_cast<uint64_t>(0xCD9E8D57u) * c2;
        uint32_t n0 = static_cast<uint32_t>(p1 >> 32) ^ c1 ^ k0, n1 = static_cast<uint32_t>(p1);
        uint32_t n2 = static_cast<uint32_t>(p0 >> 32) ^ c3 ^ k1, n3 = static_cast<uint32_t>(p0);
        c0 = n0;
        c1 = n1;
        c2 = n2;
        c3 = n3;
        k0 += 0x9E3779B9u;
        k1 += 0xBB67AE85u;
    }
    out[0] = c0;
    out[1] = c1;
    out[2] = c2;
    out[3] = c3;
}
uint64_t sampler_raw_next(dflash_sampler *s) {
    if (s->cfg.rng_kind == 1) {
        uint64_t pos = s->s[0]++;
        uint32_t ctr[4] = {static_cast<uint32_t>(pos), static_cast<uint32_t>(pos >> 32), 0, 0};
        uint32_t key[2] = {static_cast<uint32_t>(s->cfg.seed), static_cast<uint32_t>(s->cfg.seed >> 32)};
        uint32_t out[4];
        philox4x32_10(ctr, key, out);
        return static_cast<uint64_t>(out[0]) | (static_cast<uint64_t>(out[1]) << 32);
    }
    return xoshiro_next(s->s);
}

int32_t status_of_hip(hipError_t e) { return e == hipSuccess ? DFLASH_OK : DFLASH_ERR_HIP; }

int32_t check_rows(dflash_ctx *ctx, const char *what, const float *logits, int32_t n_rows, int64_t vocab,
                   int64_t stride) {
    if (!logits) return dfl_fail(ctx, DFLASH_ERR_INVALID_INPUT, "%s: null pointer", what);
    if (n_rows < 1 || n_rows > 4096) return dfl_fail(ctx, DFLASH_ERR_BAD_SHAPE, "%s: n_rows %d", what, n_rows);
    if (vocab < 1) return dfl_fail(ctx, DFLASH_ERR_EMPTY_LOGITS, "%s: empty logits row", what);
    if (vocab > 0x7fffffffll) return dfl_fail(ctx, DFLASH_ERR_VOCAB_TOO_LARGE, "%s: vocabulary %lld", what, static_cast<long long>(vocab));
    if (stride < vocab) return dfl_fail(ctx, DFLASH_ERR_BAD_SHAPE, "%s: stride %lld < vocab", what, static_cast<long long>(stride));
    return DFLASH_OK;
}

}  // namespace

extern "C" {

int32_t dflash_argmax_top2(dflash_ctx *ctx, const float *logits, int32_t n_rows, int64_t vocab, int64_t stride,
                           int32_t *idx, float *gap, dflash_stream_t stream) {
    if (!ctx) return DFLASH_ERR_INVALID_INPUT;
    int32_t rc = check_rows(ctx, "argmax_top2", logits, n_rows, vocab, stride);
    if (rc) return rc;
    if (!idx || !gap) return dfl_fail(ctx, DFLASH_ERR_INVALID_INPUT, "argmax_top2: null output");
    hipStream_t st = static_cast<hipStream_t>(stream);
    const int n_chunks = static_cast<int>((vocab + kChunk - 1) / kChunk);
    size_t off = 0;
    Top2 *part = dfl_ws_take<Top2>(ctx, &off, sizeof(Top2) * n_rows * n_chunks);
    if (!part) return dfl_fail(ctx, DFLASH_ERR_WORKSPACE, "argmax_top2: workspace too small");
    dfl_timed timer(ctx, st, DFL_T_ARGMAX);
    top2_chunk_kernel<<<dim3(n_chunks, n_rows), kSelThreads, 0, st>>>(logits, vocab, stride, part);
    top2_final_kernel<<<n_rows, 64, 0, st>>>(part, n_chunks, idx, gap);
    DFL_HIP_CHECK(ctx, hipGetLastError());
    return DFLASH_OK;
}

int32_t dflash_argmax_greedy(dflash_ctx *ctx, const float *logits, int32_t n_rows, int64_t vocab, int64_t stride,
                             int32_t *idx, dflash_stream_t stream) {
    if (!ctx) return DFLASH_ERR_INVALID_INPUT;
    int32_t rc = check_rows(ctx, "argmax_greedy", logits, n_rows, vocab, stride);
    if (rc) return rc;
    if (!idx) return dfl_fail(ctx, DFLASH_ERR_INVALID_INPUT, "argmax_greedy: null output");
    hipStream_t st = static_cast<hipStream_t>(stream);
    const int n_chunks = static_cast<int>((vocab + kSelChunk - 1) / kSelChunk);
    if (n_chunks > 2 * kSelThreads) return dfl_fail(ctx, DFLASH_ERR_UNSUPPORTED, "argmax_greedy: vocabulary too large");
    size_t off = 0;
    ChunkOut *chunks = dfl_ws_take<ChunkOut>(ctx, &off, sizeof(ChunkOut) * n_rows * n_chunks);
    RowDist *rows = dfl_ws_take<RowDist>(ctx, &off, sizeof(RowDist) * n_rows);
    if (!chunks || !rows) return dfl_fail(ctx, DFLASH_ERR_WORKSPACE, "argmax_greedy: workspace too small");
    ChainCfg cfg = {};
    cfg.k = 1;
    dfl_timed timer(ctx, st, DFL_T_ARGMAX);
    select_chunk_kernel<<<dim3(n_chunks, n_rows), kSelThreads, 0, st>>>(logits, vocab, stride, 1, chunks, false);
    row_merge_kernel<<<n_rows, kSelThreads, 0, st>>>(chunks, n_chunks, nullptr, cfg, rows, idx, false);
    DFL_HIP_CHECK(ctx, hipGetLastError());
    return DFLASH_OK;
}

int32_t dflash_top16(dflash_ctx *ctx, const float *logits, int32_t n_rows, int64_t vocab, int64_t stride,
                     int32_t *ids, float *vals, dflash_stream_t stream) {
    if (!ctx) return DFLASH_ERR_INVALID_INPUT;
    int32_t rc = check_rows(ctx, "top16", logits, n_rows, vocab, stride);
    if (rc) return rc;
    if (!ids || !vals) return dfl_fail(ctx, DFLASH_ERR_INVALID_INPUT, "top16: null output");
    hipStream_t st = static_cast<hipStream_t>(stream);
    const int n_chunks = static_cast<int>((vocab + kSelChunk - 1) / kSelChunk);
    if (n_chunks * 16 > 2 * kSelThreads) return dfl_fail(ctx, DFLASH_ERR_UNSUPPORTED, "top16: vocabulary too large");
    size_t off = 0;
    ChunkOut *chunks = dfl_ws_take<ChunkOut>(ctx, &off, sizeof(ChunkOut) * n_rows * n_chunks);
    if (!chunks) return dfl_fail(ctx, DFLASH_ERR_WORKSPACE, "top16: workspace too small");
    dfl_timed timer(ctx, st, DFL_T_ARGMAX);
    select_chunk_kernel<<<dim3(n_chunks, n_rows), kSelThreads, 0, st>>>(logits, vocab, stride, 16, chunks, true);
    top16_merge_kernel<<<n_rows, kSelThreads, 0, st>>>(chunks, n_chunks, ids, vals);
    DFL_HIP_CHECK(ctx, hipGetLastError());
    return DFLASH_OK;
}

// sampling.rs:133-144, 346-366
int32_t dflash_sampler_init(dflash_sampler *s, const dflash_sampling_config *cfg) {
    if (!s || !cfg) return DFLASH_ERR_INVALID_INPUT;
    if (!std::isfinite(cfg->temperature) || cfg->temperature < 0.0f) return DFLASH_ERR_INVALID_TEMPERATURE;
    if (!std::isfinite(cfg->top_p) || !(0.0f < cfg->top_p && cfg->top_p <= 1.0f)) return DFLASH_ERR_INVALID_TOP_P;
    if (!std::isfinite(cfg->min_p) || !(0.0f <= cfg->min_p && cfg->min_p <= 1.0f)) return DFLASH_ERR_INVALID_MIN_P;
    s->cfg = *cfg;
    s->draws = 0;
    if (cfg->rng_kind == 1) {
        s->s[0] = s->s[1] = s->s[2] = s->s[3] = 0;
    } else {
        uint64_t sm = cfg->seed;
        for (int i = 0; i < 4; i++) s->s[i] = splitmix_next(sm);
    }
    return DFLASH_OK;
}

int32_t dflash_sampler_at_draw(dflash_sampler *s, const dflash_sampling_config *cfg, uint64_t draws) {
    int32_t rc = dflash_sampler_init(s, cfg);
    if (rc) return rc;
    dflash_sampler_advance(s, draws);
    return DFLASH_OK;
}

void dflash_sampler_peek(const dflash_sampler *s, int32_t n, double *out_host) {
    dflash_sampler copy = *s;
    for (int32_t i = 0; i < n; i++)
        out_host[i] = static_cast<double>(sampler_raw_next(&copy) >> 11) / 9007199254740992.0;
}

void dflash_sampler_advance(dflash_sampler *s, uint64_t draws) {
    for (uint64_t i = 0; i < draws; i++) sampler_raw_next(s);
    s->draws += draws;
}

int32_t dflash_accept_prefix(dflash_ctx *ctx, const int32_t *verified, int32_t n_tokens, const float *target_logits,
                             int64_t vocab, int32_t mode, int32_t n_proposals, const int32_t *prop_tokens,
                             const int32_t *prop_counts, const dflash_weighted_candidate *prop_cands,
                             const float *draft_logits, float draft_temperature, dflash_sampler *sampler,
                             int64_t budget, const int32_t *stop_ids, int32_t n_stop, dflash_accept_decision *out,
                             dflash_stream_t stream) {
    if (!ctx) return DFLASH_ERR_INVALID_INPUT;
    if (!out || !sampler) return dfl_fail(ctx, DFLASH_ERR_INVALID_INPUT, "accept_prefix: null sampler / output");
    memset(out, 0, sizeof(*out));
    out->err_row = -1;
    out->err_index = -1;
    // ---- whole-block validation before anything is drawn (accept.rs:85-130)
    if (n_tokens < 1 || !verified) return dfl_fail(ctx, DFLASH_ERR_INVALID_INPUT, "missing carry token");
    if (vocab <= 0 || vocab > 0x7fffffffll) return dfl_fail(ctx, DFLASH_ERR_INVALID_INPUT, "invalid vocabulary size");
    if (n_tokens > kMaxRows)
        return dfl_fail(ctx, DFLASH_ERR_BAD_SHAPE, "accept_prefix: %d verified tokens (at most %d)", n_tokens, kMaxRows);
    if (!target_logits) return dfl_fail(ctx, DFLASH_ERR_INVALID_INPUT, "target logits extent mismatch");
    if (mode < 0 || mode > 2) return dfl_fail(ctx, DFLASH_ERR_INVALID_INPUT, "accept_prefix: proposal mode %d", mode);
    if (n_stop < 0 || (n_stop > 0 && !stop_ids)) return dfl_fail(ctx, DFLASH_ERR_INVALID_INPUT, "accept_prefix: stop ids");
    for (int i = 0; i < n_tokens; i++) {
        if (verified[i] < 0 || verified[i] >= vocab) {
            out->err_row = i;
            out->err_index = verified[i];
            return dfl_fail(ctx, DFLASH_ERR_INVALID_TOKEN, "verified input token %d at index %d is outside vocabulary %lld",
                            verified[i], i, static_cast<long long>(vocab));
        }
    }
    const int n_drafts = n_tokens - 1;
    int prop_offsets[kMaxRows] = {0};
    int n_cands = 0;
    if (mode == 1) {
        if (n_proposals != n_drafts || (n_drafts > 0 && (!prop_tokens || !prop_counts)))
            return dfl_fail(ctx, DFLASH_ERR_INVALID_INPUT, "proposal row count mismatch");
        for (int r = 0; r < n_drafts; r++) {
            if (prop_tokens[r] != verified[r + 1]) {
                out->err_row = r;
                out->err_index = prop_tokens[r];
                return dfl_fail(ctx, DFLASH_ERR_PROPOSAL_MISMATCH, "proposal row %d sampled token %d, but verified draft is %d",
                                r, prop_tokens[r], verified[r + 1]);
            }
            if (prop_counts[r] < 0 || (prop_counts[r] > 0 && !prop_cands))
                return dfl_fail(ctx, DFLASH_ERR_INVALID_INPUT, "accept_prefix: proposal candidates");
            prop_offsets[r] = n_cands;
            for (int j = 0; j < prop_counts[r]; j++) {
                int32_t t = prop_cands[n_cands + j].token;
                if (t < 0 || t >= vocab) {
                    out->err_row = r;
                    out->err_code = DFLASH_ERR_PROPOSAL_TOKEN_OUT_OF_RANGE;
                    out->err_index = t;
                    return dfl_fail(ctx, DFLASH_ERR_PROPOSAL_TOKEN_OUT_OF_RANGE, "proposal token %d is outside the target vocabulary", t);
                }
            }
            n_cands += prop_counts[r];
        }
    }
    if (mode == 2) {
        if (!draft_logits) return dfl_fail(ctx, DFLASH_ERR_INVALID_INPUT, "accept_prefix: draft logits");
        if (!(std::isfinite(draft_temperature) && draft_temperature > 0.0f))
            return dfl_fail(ctx, DFLASH_ERR_INVALID_TEMPERATURE, "accept_prefix: draft temperature %f", draft_temperature);
    }
    // ---- terminal anchor / exhausted budget: no draw, nothing retained (accept.rs:131-145)
    bool anchor_eos = false;
    for (int i = 0; i < n_stop; i++) anchor_eos = anchor_eos || stop_ids[i] == verified[0];
    if (anchor_eos || budget == 0) {
        out->stop_reason = anchor_eos ? DFLASH_STOP_EOS : DFLASH_STOP_TOKEN_LIMIT;
        return DFLASH_OK;
    }
    const dflash_sampling_config &sc = sampler->cfg;
    int64_t k_eff = (sc.temperature == 0.0f) ? 1 : ((sc.top_k == 0 || static_cast<int64_t>(sc.top_k) >= vocab) ? vocab : static_cast<int64_t>(sc.top_k));
    const bool wide = k_eff > kMaxK;  // top_k = 0 or a large top_k: full order by radix sort (accept_wide.hip)
    const int n_chunks = static_cast<int>((vocab + kSelChunk - 1) / kSelChunk);
    if (!wide && n_chunks * k_eff > 2 * kSelThreads)
        return dfl_fail(ctx, DFLASH_ERR_UNSUPPORTED, "accept_prefix: vocabulary %lld x top_k %lld too large", static_cast<long long>(vocab), static_cast<long long>(k_eff));

    hipStream_t st = static_cast<hipStream_t>(stream);
    const int n_tiles = static_cast<int>((vocab + 1023) / 1024);
    size_t off = 0;
    ChunkOut *chunks = dfl_ws_take<ChunkOut>(ctx, &off, sizeof(ChunkOut) * n_tokens * n_chunks);
    ChunkOut *dchunks = dfl_ws_take<ChunkOut>(ctx, &off, sizeof(ChunkOut) * n_tokens * n_chunks);
    RowDist *rows = dfl_ws_take<RowDist>(ctx, &off, sizeof(RowDist) * n_tokens);
    double *tile_sums = dfl_ws_take<double>(ctx, &off, sizeof(double) * n_tokens * n_tiles);
    int32_t *d_stop = dfl_ws_take<int32_t>(ctx, &off, sizeof(int32_t) * (n_stop + 8));
    dflash_weighted_candidate *d_cands =
        dfl_ws_take<dflash_weighted_candidate>(ctx, &off, sizeof(dflash_weighted_candidate) * (n_cands + 1));
    dflash_accept_decision *d_out = dfl_ws_take<dflash_accept_decision>(ctx, &off, sizeof(dflash_accept_decision));
    if (!chunks || !dchunks || !rows || !tile_sums || !d_stop || !d_cands || !d_out)
        return dfl_fail(ctx, DFLASH_ERR_WORKSPACE, "accept_prefix: workspace too small");

    // small host inputs: by value in the decision kernel's arguments; only the variable-length lists are copied
    DecideArgs a;
    memset(&a, 0, sizeof(a));
    dflash_sampler_peek(sampler, n_tokens + 1, a.uniforms);
    for (int i = 0; i < n_tokens; i++) a.verified[i] = verified[i];
    for (int r = 0; r < n_drafts && mode == 1; r++) {
        a.prop_offsets[r] = prop_offsets[r];
        a.prop_counts[r] = prop_counts[r];
    }
    if (n_stop > 0)
        DFL_HIP_CHECK(ctx, hipMemcpyAsync(d_stop, stop_ids, sizeof(int32_t) * n_stop, hipMemcpyHostToDevice, st));
    if (n_cands > 0)
        DFL_HIP_CHECK(ctx, hipMemcpyAsync(d_cands, prop_cands, sizeof(dflash_weighted_candidate) * n_cands,
                                          hipMemcpyHostToDevice, st));

    ChainCfg cfg;
    cfg.temperature = sc.temperature;
    cfg.top_p = sc.top_p;
    cfg.min_p = sc.min_p;
    cfg.k = static_cast<int32_t>(k_eff);
    cfg.ln_min_p = sc.min_p > 0.0f ? std::log(static_cast<double>(sc.min_p)) : 0.0;
    cfg.draft_temperature = draft_temperature;
    cfg.mode = mode;
    {
        dfl_timed timer(ctx, st, DFL_T_ACCEPT);
        const bool dense = mode == 2 && n_drafts > 0;
        const uint64_t *wide_keys = nullptr;
        const double *wide_w = nullptr;
        if (wide) {
            if (const int32_t rc_ = dfl_accept_wide_rows(ctx, target_logits, n_tokens, vocab, vocab, cfg, rows, &off, &wide_keys, &wide_w, st))
                return rc_;
            if (dense) select_chunk_kernel<<<dim3(n_chunks, n_drafts), kSelThreads, 0, st>>>(draft_logits, vocab, vocab, 1, dchunks, false);
        } else if (dense) {
            select_pair_kernel<<<dim3(n_chunks, n_tokens + n_drafts), kSelThreads, 0, st>>>(target_logits, n_tokens, cfg.k, chunks,
                                                                                         draft_logits, dchunks, vocab, vocab);
        } else {
            select_chunk_kernel<<<dim3(n_chunks, n_tokens), kSelThreads, 0, st>>>(target_logits, vocab, vocab, cfg.k, chunks, false);
        }
        // the rows' chains and, for dense proposals, the tile sums of the draft rows: one launch
        if (dense) {
            const int blocks_per_row = (n_tiles + 7) / 8;
            const int n_row_wgs = wide ? n_drafts : n_tokens;  // (wide: the chain has run; only the draft side is merged)
            rows_and_tiles_kernel<<<n_row_wgs + n_drafts * blocks_per_row, kSelThreads, 0, st>>>(
                chunks, n_chunks, dchunks, cfg, rows, n_row_wgs, wide, draft_logits, vocab, vocab, n_tiles, blocks_per_row, tile_sums);
        } else if (!wide) {
            row_merge_kernel<<<n_tokens, kSelThreads, 0, st>>>(chunks, n_chunks, nullptr, cfg, rows, nullptr, false);
        }
        a.wide_keys = wide_keys;
        a.wide_w = wide_w;
        a.wide_stride = vocab;
        a.n_tokens = n_tokens;
        a.n_stop = n_stop;
        a.mode = mode;
        a.vocab = static_cast<int32_t>(vocab);
        a.budget = budget;
        a.stop_ids = d_stop;
        a.rows = rows;
        a.prop_cands = d_cands;
        a.draft = draft_logits;
        a.draft_stride = vocab;
        a.tile_sums = tile_sums;
        a.n_tiles = n_tiles;
        a.temperature = sc.temperature;
        a.draft_temperature = draft_temperature;
        // the decision goes straight to the context's pinned page when the device can address it (one copy less
        // between the last kernel and the host)
        static_assert(sizeof(dflash_accept_decision) <= DFL_PINNED_BYTES, "the decision is read back through the pinned page");
        void *pinned_dev = nullptr;
        const bool direct = ctx->pinned && hipHostGetDevicePointer(&pinned_dev, ctx->pinned, 0) == hipSuccess && pinned_dev;
        if (!direct) (void)hipGetLastError();
        decide_kernel<<<1, 64, 0, st>>>(a, direct ? static_cast<dflash_accept_decision *>(pinned_dev) : d_out);
        DFL_HIP_CHECK(ctx, hipGetLastError());
        if (!direct) DFL_HIP_CHECK(ctx, hipMemcpyAsync(ctx->pinned, d_out, sizeof(*out), hipMemcpyDeviceToHost, st));
    }
    DFL_HIP_CHECK(ctx, hipStreamSynchronize(st));
    memcpy(out, ctx->pinned, sizeof(*out));
    if (out->err_code) {
        int32_t code = out->err_code;
        return dfl_fail(ctx, code, "DFlash target row %d: %s (index %lld)", out->err_row, dflash_status_name(code),
                        static_cast<long long>(out->err_index));
    }
    dflash_sampler_advance(sampler, static_cast<uint64_t>(out->draws_used));  // committed only on success
    return DFLASH_OK;
}

}  // extern "C"
