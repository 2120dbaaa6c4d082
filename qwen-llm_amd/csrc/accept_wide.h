// Interface of the wide-candidate sampler chain (accept_wide.hip) to the accept-prefix decision (accept.hip).
#pragma once

#include "common.h"
#include "sampler_chain.h"

// A wide key is row << 60 | descending_logit_bits << 28 | token.
constexpr int kWideTokenBits = 28;
constexpr uint64_t kWideTokenMask = (uint64_t(1) << kWideTokenBits) - 1;

// Orders every row of logits [n_rows][stride] (n_rows <= 16, vocab < 2^28) and runs the sampler chain on it for
// an effective top-k above kMaxK.  rows[r] receives n_keep / err / err_index / total; row r's kept candidates
// are, best first, the tokens (key & kWideTokenMask) of (*keys_out)[r * vocab ..] with weights
// (*weights_out)[r * vocab ..].  Device arrays come from the context workspace at *ws_off.  Enqueue only.
int32_t dfl_accept_wide_rows(dflash_ctx *ctx, const float *logits, int32_t n_rows, int64_t vocab, int64_t stride, const ChainCfg &cfg,
                             RowDist *rows, size_t *ws_off, const uint64_t **keys_out, const double **weights_out, hipStream_t st);
