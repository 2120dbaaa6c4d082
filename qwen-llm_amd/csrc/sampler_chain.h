// The sampler-v1 filter chain on the device (sampling.rs:1541-1615), its ordering keys
// (sampling.rs:1206-1235) and the categorical pick (sampling.rs:1587-1596): shared by the
// accept-prefix kernels and the sampled DFlash-2 selector walk.  Everything that feeds a
// comparison with a uniform draw is f64 and sequential, in the order of the reference's loops.
#pragma once

#include "common.h"

#include <cmath>

// f64 arithmetic that is compared with uniform draws keeps the reference's separately rounded
// operations: no fused multiply-adds from here on in the including file.
#pragma clang fp contract(off)

constexpr int kMaxK = 64;  // most candidates a row keeps inline (wider sets live in device arrays, accept_wide.hip)

// ------------------------------------------------------------------------------------------
// per-row results
// ------------------------------------------------------------------------------------------
struct RowDist {
    int32_t n_keep;     // candidates after every filter (above kMaxK: tokens / weights are in the wide arrays instead)
    int32_t err;        // DFLASH_ERR_* or 0
    int64_t err_index;  // NaN index etc.
    double total;       // sum of the kept weights (sequential)
    int32_t tokens[kMaxK];
    double weights[kMaxK];
    // dense proposal side
    int32_t d_err;
    int32_t d_pad;
    int64_t d_err_index;
    double d_max_scaled;  // f64(max draft logit) / T
    double d_total;       // P
};

struct ChainCfg {
    float temperature, top_p, min_p;
    int32_t k;          // effective top-k
    double ln_min_p;    // ln(f64(min_p)), computed on the host
    float draft_temperature;
    int32_t mode;       // proposal mode
};

namespace {

// sampling.rs:1206-1220: a u32 whose ascending order is descending f32 total order
__device__ __host__ __forceinline__ uint32_t desc_bits(uint32_t bits) {
    uint32_t asc = (bits & 0x80000000u) ? ~bits : (bits | 0x80000000u);
    return ~asc;
}
__device__ __forceinline__ uint64_t cand_key(uint32_t token, float logit) {
    return (static_cast<uint64_t>(desc_bits(__float_as_uint(logit))) << 32) | token;
}
// sampling.rs:1223-1231
__device__ __forceinline__ float key_logit(uint64_t key) {
    uint32_t asc = ~static_cast<uint32_t>(key >> 32);
    uint32_t bits = (asc & 0x80000000u) ? (asc & 0x7fffffffu) : ~asc;
    return __uint_as_float(bits);
}
__device__ __forceinline__ int32_t key_token(uint64_t key) { return static_cast<int32_t>(static_cast<uint32_t>(key)); }

// sampling.rs:1541-1615 on the ordered candidates of one row (keys ascending = best first)
// Work arrays of the chain (kMaxK entries each): a caller that runs the chain on one thread of a workgroup
// keeps them in LDS; private arrays of this size live in scratch memory, where every access is a trip to memory.
struct ChainScratch {
    double *l, *w;
    int *tok;
};

__device__ void run_chain(const uint64_t *keys, int len, const ChainCfg &c, RowDist *d, const ChainScratch &scratch) {
    double *l = scratch.l;
    int *tok = scratch.tok;
    for (int i = 0; i < len; i++) {
        l[i] = static_cast<double>(key_logit(keys[i]));
        tok[i] = key_token(keys[i]);
    }
    if (c.min_p > 0.0f) {
        double max_logit = l[0];
        if (isfinite(max_logit)) {
            double threshold = max_logit + c.ln_min_p;
            int keep = 0;
            for (int i = 0; i < len; i++)
                if (l[i] >= threshold) {
                    l[keep] = l[i];
                    tok[keep] = tok[i];
                    keep++;
                }
            len = keep;
        }
    }
    if (len == 0) {
        d->err = DFLASH_ERR_NO_CANDIDATES;
        return;
    }
    if (l[0] == INFINITY) {
        int keep = 0;
        for (int i = 0; i < len; i++)
            if (l[i] == INFINITY) {
                l[keep] = l[i];
                tok[keep] = tok[i];
                keep++;
            }
        len = keep;
    }
    const double temperature = static_cast<double>(c.temperature);
    for (int i = 0; i < len; i++) l[i] /= temperature;
    double *w = scratch.w;
    int n_inf = 0;
    for (int i = 0; i < len; i++) n_inf += (l[i] == INFINITY);
    if (n_inf > 0) {
        for (int i = 0; i < len; i++) w[i] = (l[i] == INFINITY) ? 1.0 : 0.0;
    } else {
        double max_logit = l[0];
        if (max_logit == -INFINITY) {
            d->err = DFLASH_ERR_NO_CANDIDATES;
            return;
        }
        bool finite = true;
        for (int i = 0; i < len; i++) {
            w[i] = exp(l[i] - max_logit);
            finite = finite && isfinite(w[i]);
        }
        if (!finite) {
            d->err = DFLASH_ERR_NO_CANDIDATES;
            return;
        }
    }
    if (c.top_p < 1.0f) {
        double total = -0.0;
        for (int i = 0; i < len; i++) total += w[i];
        double target = total * static_cast<double>(c.top_p);
        double cumulative = 0.0;
        int keep = 0;
        for (int i = 0; i < len; i++) {
            cumulative += w[i];
            keep++;
            if (cumulative >= target) break;
        }
        len = keep < 1 ? 1 : keep;
    }
    double total_weight = -0.0;
    for (int i = 0; i < len; i++) total_weight += w[i];
    if (!(isfinite(total_weight) && total_weight > 0.0)) {
        d->err = DFLASH_ERR_NO_CANDIDATES;
        return;
    }
    d->n_keep = len;
    d->total = total_weight;
    for (int i = 0; i < len; i++) {
        d->tokens[i] = tok[i];
        d->weights[i] = w[i];
    }
}

// A lane's double in every lane (src uniform).
__device__ __forceinline__ double chain_bcast(double v, int src) {
    const unsigned long long b = static_cast<unsigned long long>(__double_as_longlong(v));
    const unsigned lo = __builtin_amdgcn_readlane(static_cast<unsigned>(b), src);
    const unsigned hi = __builtin_amdgcn_readlane(static_cast<unsigned>(b >> 32), src);
    return __longlong_as_double(static_cast<long long>((static_cast<unsigned long long>(hi) << 32) | lo));
}

// run_chain by one whole wave (len <= 64): lane i holds candidate i.  What the reference does element by element
// without carrying anything from one element to the next (the conversions, the division by the temperature, the
// exponentials, the filters' comparisons) is done by all lanes at once; every sum that is compared with something is
// still added in candidate order, one addition after the other, on values that are the same bits as run_chain's.
// The candidates are in descending logit order, so what min-p and the +inf rule keep is a prefix: its length is a
// population count.
__device__ void run_chain_wave(const uint64_t *keys, int len, const ChainCfg &c, RowDist *d) {
    const int lane = threadIdx.x & 63;
    double l = lane < len ? static_cast<double>(key_logit(keys[lane])) : 0.0;
    const int tok = lane < len ? key_token(keys[lane]) : 0;
    auto fail = [&]() {
        if (lane == 0) d->err = DFLASH_ERR_NO_CANDIDATES;
    };
    if (c.min_p > 0.0f && len > 0) {
        const double max_logit = chain_bcast(l, 0);
        if (isfinite(max_logit)) {
            const double threshold = max_logit + c.ln_min_p;
            len = __popcll(__builtin_amdgcn_ballot_w64(lane < len && l >= threshold));
        }
    }
    if (len == 0) return fail();
    if (chain_bcast(l, 0) == INFINITY) len = __popcll(__builtin_amdgcn_ballot_w64(lane < len && l == INFINITY));
    l = l / static_cast<double>(c.temperature);
    const int n_inf = __popcll(__builtin_amdgcn_ballot_w64(lane < len && l == INFINITY));
    double w;
    if (n_inf > 0) {
        w = (l == INFINITY) ? 1.0 : 0.0;
    } else {
        const double max_logit = chain_bcast(l, 0);
        if (max_logit == -INFINITY) return fail();
        w = lane < len ? exp(l - max_logit) : 0.0;
        if (__builtin_amdgcn_ballot_w64(lane < len && !isfinite(w)) != 0) return fail();
    }
    if (c.top_p < 1.0f) {
        double total = -0.0;
        for (int i = 0; i < len; i++) total += chain_bcast(w, i);
        const double target = total * static_cast<double>(c.top_p);
        double cumulative = 0.0;
        int keep = 0;
        for (int i = 0; i < len; i++) {
            cumulative += chain_bcast(w, i);
            keep++;
            if (cumulative >= target) break;
        }
        len = keep < 1 ? 1 : keep;
    }
    double total_weight = -0.0;
    for (int i = 0; i < len; i++) total_weight += chain_bcast(w, i);
    if (!(isfinite(total_weight) && total_weight > 0.0)) return fail();
    if (lane == 0) {
        d->n_keep = len;
        d->total = total_weight;
    }
    if (lane < len) {
        d->tokens[lane] = tok;
        d->weights[lane] = w;
    }
}

// the same with private work arrays
__device__ void run_chain(const uint64_t *keys, int len, const ChainCfg &c, RowDist *d) {
    double l[kMaxK], w[kMaxK];
    int tok[kMaxK];
    run_chain(keys, len, c, d, ChainScratch{l, w, tok});
}

// first candidate whose running sum exceeds x, else the last (sampling.rs:1587-1596)
__device__ int pick_index(const double *w, int n, double x) {
    double cumulative = 0.0;
    for (int i = 0; i < n; i++) {
        cumulative += w[i];
        if (x < cumulative) return i;
    }
    return n - 1;
}

}  // namespace
