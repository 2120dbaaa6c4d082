// Sampler chain for wide candidate sets: top_k = 0 (the whole vocabulary) or top_k above the 64
// candidates the selection kernels of accept.hip keep per row.
//
// Reference: sampling.rs:1198-1214 and 1273-1296 (full order: stable radix sort of the logit half of
// the (descending logit bits, token) keys; top_k < len: the top_k smallest keys, sorted), chain
// sampling.rs:1541-1615.
//
// All rows of the block are ordered by ONE device-wide radix sort: a key is
//   row << 60 | descending_logit_bits << 28 | token          (token < 2^28, row < 16)
// and ascending key order is (row, descending logit in f32 total order, ascending token id): row r's
// candidates end up, best first, at [r * vocab, (r + 1) * vocab).  All 64 bits are sorted (tokens are
// unique, so this is the reference's stable sort of the logit half; the library's sort over a sub-range of
// bits returned unsorted output for inputs of 4 k to 100 k keys on ROCm 7.2, checked against a host sort,
// while the full-width sort is correct at every size).  The sort itself is
// rocPRIM's radix_sort_keys (a plain library routine on a cold path; the streaming kernels of the hot
// path are in accept.hip).  The chain then runs per row on one workgroup: what is order-free (the
// min-p / +inf prefix lengths, the exponentials) is done by all threads, every sum that is compared
// with a uniform draw is the reference's sequential f64 fold, fed through LDS a tile at a time so
// that the one adding thread never waits on memory.
#include "common.h"
#include "sampler_chain.h"

#include <cstring>

#include <rocprim/device/device_radix_sort.hpp>

#include "accept_wide.h"

namespace {

constexpr int kWideThreads = 1024;
constexpr int kWideTile = 4096;  // doubles staged in LDS per step of a sequential fold
constexpr int kNoNanW = 0x7fffffff;

__device__ __forceinline__ float wide_key_logit(uint64_t key) {
    const uint32_t asc = ~static_cast<uint32_t>(key >> kWideTokenBits);
    const uint32_t bits = (asc & 0x80000000u) ? (asc & 0x7fffffffu) : ~asc;
    return __uint_as_float(bits);
}

__global__ void __launch_bounds__(256)
    wide_keys_kernel(const float *__restrict__ logits, int64_t vocab, int64_t stride, uint64_t *__restrict__ keys,
                     int32_t *__restrict__ nan_first) {
    const int row = blockIdx.y;
    const int64_t i = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
    if (i >= vocab) return;
    const float v = logits[row * stride + i];
    if (v != v) atomicMin(nan_first + row, static_cast<int32_t>(i));
    keys[row * vocab + i] = (static_cast<uint64_t>(row) << 60) |
                            (static_cast<uint64_t>(desc_bits(__float_as_uint(v))) << kWideTokenBits) | static_cast<uint64_t>(i);
}

__global__ void wide_init_kernel(int32_t *nan_first, int n) {
    if (static_cast<int>(threadIdx.x) < n) nan_first[threadIdx.x] = kNoNanW;
}

// workgroup-wide integer sum, result to every thread
__device__ int64_t block_sum_i64(int64_t v, int64_t *sh) {
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
    __syncthreads();
    if ((threadIdx.x & 63) == 0) sh[threadIdx.x >> 6] = v;
    __syncthreads();
    int64_t r = 0;
    for (int w = 0; w < static_cast<int>(blockDim.x >> 6); w++) r += sh[w];
    return r;
}

// The reference's `acc = start; for w in weights[..n] { acc += w }` by thread 0, weights staged through LDS.
// With stop_at >= 0 the fold stops after the first element that brings the sum to >= stop_at (top-p); *count is
// the number of elements added.  Returns the sum (to every thread).
__device__ double sequential_fold(const double *__restrict__ w, int64_t n, double start, bool use_stop, double stop_at,
                                  int64_t *count, double *tile, double *bcast, int64_t *bcast_n, int *done) {
    if (threadIdx.x == 0) {
        *bcast = start;
        *bcast_n = 0;
        *done = 0;
    }
    __syncthreads();
    for (int64_t base = 0; base < n; base += kWideTile) {
        const int m = static_cast<int>(n - base < kWideTile ? n - base : kWideTile);
        for (int i = threadIdx.x; i < m; i += blockDim.x) tile[i] = w[base + i];
        __syncthreads();
        if (threadIdx.x == 0) {
            double acc = *bcast;
            int i = 0;
            for (; i < m; i++) {
                acc += tile[i];
                if (use_stop && acc >= stop_at) {
                    i++;
                    *done = 1;
                    break;
                }
            }
            *bcast = acc;
            *bcast_n += i;
        }
        __syncthreads();
        if (*done) break;
    }
    const double result = *bcast;
    if (count) *count = *bcast_n;
    __syncthreads();  // everyone has read the result before the next fold resets it
    return result;
}

// sampling.rs:1541-1615 on the ordered candidates of one row; weights[row * vocab + i] receives candidate i's weight
__global__ void __launch_bounds__(kWideThreads)
    wide_chain_kernel(const uint64_t *__restrict__ keys_sorted, int64_t vocab, ChainCfg cfg, const int32_t *__restrict__ nan_first,
                      RowDist *__restrict__ rows, double *__restrict__ weights) {
    __shared__ double tile[kWideTile];
    __shared__ int64_t red[kWideThreads / 64];
    __shared__ double bcast;
    __shared__ int64_t bcast_n;
    __shared__ int done;
    const int row = blockIdx.x, tid = threadIdx.x;
    const uint64_t *keys = keys_sorted + static_cast<int64_t>(row) * vocab;
    double *w = weights + static_cast<int64_t>(row) * vocab;
    RowDist *d = rows + row;
    auto finish = [&](int32_t err, int64_t err_index, int64_t n_keep, double total) {
        if (tid == 0) {
            d->n_keep = static_cast<int32_t>(n_keep);
            d->err = err;
            d->err_index = err_index;
            d->total = total;
            d->d_err = 0;
            d->d_err_index = -1;
        }
    };
    if (nan_first[row] != kNoNanW) return finish(DFLASH_ERR_NAN_LOGIT, nan_first[row], 0, 0.0);
    int64_t len = cfg.k < vocab ? cfg.k : vocab;  // top-k
    const double l0 = static_cast<double>(wide_key_logit(keys[0]));
    if (cfg.min_p > 0.0f && isfinite(l0)) {  // min-p, before the temperature: a prefix of the descending order
        const double threshold = l0 + cfg.ln_min_p;
        int64_t c = 0;
        for (int64_t i = tid; i < len; i += kWideThreads) c += static_cast<double>(wide_key_logit(keys[i])) >= threshold;
        len = block_sum_i64(c, red);
    }
    if (len == 0) return finish(DFLASH_ERR_NO_CANDIDATES, -1, 0, 0.0);
    bool all_inf = false;
    if (l0 == INFINITY) {  // only the +inf logits stay, with weight one each
        int64_t c = 0;
        for (int64_t i = tid; i < len; i += kWideThreads) c += wide_key_logit(keys[i]) == INFINITY;
        len = block_sum_i64(c, red);
        all_inf = true;
    }
    const double temperature = static_cast<double>(cfg.temperature);
    if (all_inf) {
        for (int64_t i = tid; i < len; i += kWideThreads) w[i] = 1.0;
    } else {
        const double max_logit = l0 / temperature;
        if (max_logit == -INFINITY) return finish(DFLASH_ERR_NO_CANDIDATES, -1, 0, 0.0);
        int64_t bad = 0;
        for (int64_t i = tid; i < len; i += kWideThreads) {
            const double wi = exp(static_cast<double>(wide_key_logit(keys[i])) / temperature - max_logit);
            bad += !isfinite(wi);
            w[i] = wi;
        }
        if (block_sum_i64(bad, red) != 0) return finish(DFLASH_ERR_NO_CANDIDATES, -1, 0, 0.0);
    }
    __syncthreads();  // the weights are read back by other threads below
    if (cfg.top_p < 1.0f) {
        const double total = sequential_fold(w, len, -0.0, false, 0.0, nullptr, tile, &bcast, &bcast_n, &done);
        const double target = total * static_cast<double>(cfg.top_p);
        int64_t keep = 0;
        sequential_fold(w, len, 0.0, true, target, &keep, tile, &bcast, &bcast_n, &done);
        len = keep < 1 ? 1 : keep;
    }
    const double total_weight = sequential_fold(w, len, -0.0, false, 0.0, nullptr, tile, &bcast, &bcast_n, &done);
    if (!(isfinite(total_weight) && total_weight > 0.0)) return finish(DFLASH_ERR_NO_CANDIDATES, -1, 0, 0.0);
    finish(0, -1, len, total_weight);
}

}  // namespace

int32_t dfl_accept_wide_rows(dflash_ctx *ctx, const float *logits, int32_t n_rows, int64_t vocab, int64_t stride, const ChainCfg &cfg,
                             RowDist *rows, size_t *ws_off, const uint64_t **keys_out, const double **weights_out, hipStream_t st) {
    if (n_rows > 16 || vocab >= (int64_t(1) << kWideTokenBits))
        return dfl_fail(ctx, DFLASH_ERR_UNSUPPORTED, "accept_prefix: wide top-k needs <= 16 rows and a vocabulary below 2^28");
    const size_t n = static_cast<size_t>(n_rows) * static_cast<size_t>(vocab);
    uint64_t *keys_a = dfl_ws_take<uint64_t>(ctx, ws_off, n * sizeof(uint64_t));
    uint64_t *keys_b = dfl_ws_take<uint64_t>(ctx, ws_off, n * sizeof(uint64_t));
    double *weights = dfl_ws_take<double>(ctx, ws_off, n * sizeof(double));
    int32_t *nan_first = dfl_ws_take<int32_t>(ctx, ws_off, 16 * sizeof(int32_t));
    size_t tmp_bytes = 0;
    if (rocprim::radix_sort_keys(nullptr, tmp_bytes, keys_a, keys_b, n, 0, 64, st, false) != hipSuccess)
        return dfl_fail(ctx, DFLASH_ERR_HIP, "accept_prefix: radix sort size query failed");
    void *tmp = dfl_ws_take<char>(ctx, ws_off, tmp_bytes ? tmp_bytes : 1);
    if (!keys_a || !keys_b || !weights || !nan_first || !tmp)
        return dfl_fail(ctx, DFLASH_ERR_WORKSPACE,
                        "accept_prefix: top_k %lld over a vocabulary of %lld needs about %zu MB of context workspace",
                        static_cast<long long>(cfg.k), static_cast<long long>(vocab), (3 * n * 8 + tmp_bytes) >> 20);
    wide_init_kernel<<<1, 64, 0, st>>>(nan_first, n_rows);
    wide_keys_kernel<<<dim3(static_cast<unsigned>((vocab + 255) / 256), n_rows), 256, 0, st>>>(logits, vocab, stride, keys_a, nan_first);
    DFL_HIP_CHECK(ctx, rocprim::radix_sort_keys(tmp, tmp_bytes, keys_a, keys_b, n, 0, 64, st, false));
    wide_chain_kernel<<<n_rows, kWideThreads, 0, st>>>(keys_b, vocab, cfg, nan_first, rows, weights);
    DFL_HIP_CHECK(ctx, hipGetLastError());
    *keys_out = keys_b;
    *weights_out = weights;
    return DFLASH_OK;
}
