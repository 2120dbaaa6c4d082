// Adaptive speculation policy of the generation loop: host logic only (no device code).
//
// DflashAdaptiveState and the gate functions of crates/qwen-cli/src/qwen/dflash.rs:5-376: a trailing
// window of accepted-draft counts turns speculation off when the mean emitted tokens per step falls
// below break-even, off steps are counted and every so often one speculative probe step is allowed;
// in the long-context lane (positions at or past 16384 with a raised stop) dense exact-fallback
// replays back off too and re-entry needs sustained good probes.  The constants are the reference's
// (calibrated on its hardware); the mechanism is what a caller's loop shares with it.
#include "common.h"

#include <cstring>

namespace {

constexpr int kAlphaWindow = 16;                // DFLASH_ALPHA_WINDOW
constexpr int kSampledAlphaWindow = 8;          // DFLASH_SAMPLED_ALPHA_WINDOW
constexpr double kBreakevenBase = 3.1;          // DFLASH_BREAKEVEN_BASE (dflash_breakeven ignores the position)
constexpr double kAlphaOffMargin = 0.6;         // DFLASH_ALPHA_OFF_MARGIN
constexpr int kReprobeInterval = 8;             // DFLASH_REPROBE_INTERVAL
constexpr int kSampledReprobeInterval = 32;     // DFLASH_SAMPLED_REPROBE_INTERVAL
constexpr double kLongAlphaOffMean = 2.9;       // DFLASH_LONG_ALPHA_OFF_MEAN
constexpr int kLongFallbackEarlyWindow = 4;     // DFLASH_LONG_FALLBACK_EARLY_WINDOW
constexpr int kLongFallbackEarlyLimit = 2;      // DFLASH_LONG_FALLBACK_EARLY_LIMIT
constexpr int kLongFallbackWindow = 8;          // DFLASH_LONG_FALLBACK_WINDOW
constexpr int kLongFallbackLimit = 4;           // DFLASH_LONG_FALLBACK_LIMIT
constexpr int kLongReprobeInterval = 64;        // DFLASH_LONG_REPROBE_INTERVAL
constexpr int kLongFallbackReprobeInterval = 256;  // DFLASH_LONG_FALLBACK_REPROBE_INTERVAL
constexpr int kLongReentryProbes = 2;           // DFLASH_LONG_REENTRY_PROBES
constexpr double kLongReentryMean = 3.1;        // DFLASH_LONG_REENTRY_MEAN

static_assert(kAlphaWindow <= 16 && kLongFallbackWindow <= 8 && kLongReentryProbes <= 2, "window storage of dflash_adaptive_state");

// Vec::push followed by remove(0) once over the limit, on storage of exactly `limit` entries: a full
// window drops its oldest entry first
template <typename T>
void push_window(T *w, int32_t *n, int limit, T v) {
    if (*n >= limit) {
        for (int i = 1; i < *n; i++) w[i - 1] = w[i];
        *n = limit - 1;
    }
    w[(*n)++] = v;
}

void clear_windows(dflash_adaptive_state *s) { s->n_alpha = s->n_fallback = s->n_reentry = 0; }

void enter_long_backoff(dflash_adaptive_state *s, int32_t reason) {
    s->reason = reason;
    clear_windows(s);
}

}  // namespace

extern "C" {

void dflash_adaptive_init(dflash_adaptive_state *s) {
    if (s) memset(s, 0, sizeof(*s));
}

void dflash_adaptive_prepare_mode(dflash_adaptive_state *s, int32_t long_mode) {
    if (long_mode && !s->long_mode) {
        clear_windows(s);
        s->long_mode = 1;
    }
}

int32_t dflash_adaptive_backoff_active(const dflash_adaptive_state *s) { return s->reason != DFLASH_BACKOFF_NONE; }

int32_t dflash_adaptive_probe_due(const dflash_adaptive_state *s, int32_t sampled_mode, int32_t long_mode) {
    if (s->reason == DFLASH_BACKOFF_NONE) return 0;
    int64_t interval;
    if (long_mode)
        interval = s->reason == DFLASH_BACKOFF_ACCEPTANCE ? kLongReprobeInterval : kLongFallbackReprobeInterval;
    else
        interval = sampled_mode ? kSampledReprobeInterval : kReprobeInterval;
    return s->off_steps_since_probe > 0 && s->off_steps_since_probe % interval == 0;
}

void dflash_adaptive_record_off_step(dflash_adaptive_state *s) { s->off_steps_since_probe++; }

void dflash_adaptive_begin_spec_step(dflash_adaptive_state *s) { s->off_steps_since_probe = 0; }

void dflash_adaptive_record_spec_step(dflash_adaptive_state *s, int32_t n_accepted, int32_t fallback_ran, int32_t was_probe,
                                      int32_t reentry_eligible, int32_t sampled_mode, int32_t long_mode, int64_t position) {
    (void)position;  // dflash_breakeven takes it and ignores it (qwen/dflash.rs:146-148)
    if (long_mode) {
        if (was_probe) {
            if (fallback_ran) {
                s->reason = DFLASH_BACKOFF_FALLBACK;
                s->n_reentry = 0;
                return;
            }
            if (!reentry_eligible) {
                s->n_reentry = 0;
                return;
            }
            push_window(s->reentry_accepts, &s->n_reentry, kLongReentryProbes, n_accepted);
            if (s->n_reentry == kLongReentryProbes) {
                int64_t sum = 0;
                for (int i = 0; i < s->n_reentry; i++) sum += s->reentry_accepts[i];
                if (1.0 + static_cast<double>(sum) / kLongReentryProbes >= kLongReentryMean) {
                    s->reason = DFLASH_BACKOFF_NONE;
                    clear_windows(s);
                }
            }
            return;
        }
        push_window(s->alpha_window, &s->n_alpha, kAlphaWindow, n_accepted);
        push_window<uint8_t>(s->fallback_window, &s->n_fallback, kLongFallbackWindow, fallback_ran ? 1 : 0);
        int ran = 0;
        for (int i = 0; i < s->n_fallback; i++) ran += s->fallback_window[i];
        const bool fallback_losing = s->n_fallback == kLongFallbackWindow && ran >= kLongFallbackLimit;
        bool early_fallback_losing = false;
        if (s->n_fallback >= kLongFallbackEarlyWindow && s->n_alpha >= kLongFallbackEarlyWindow) {
            int early = 0;
            int64_t acc = 0;
            for (int i = s->n_fallback - kLongFallbackEarlyWindow; i < s->n_fallback; i++) early += s->fallback_window[i];
            // the acceptance window is at least as long as the fallback window (same pushes, larger limit)
            for (int i = s->n_alpha - kLongFallbackEarlyWindow; i < s->n_alpha; i++) acc += s->alpha_window[i];
            early_fallback_losing = early >= kLongFallbackEarlyLimit &&
                                    1.0 + static_cast<double>(acc) / kLongFallbackEarlyWindow < kLongAlphaOffMean;
        }
        int64_t sum = 0;
        for (int i = 0; i < s->n_alpha; i++) sum += s->alpha_window[i];
        const bool alpha_losing = s->n_alpha == kAlphaWindow && 1.0 + static_cast<double>(sum) / kAlphaWindow < kLongAlphaOffMean;
        if (early_fallback_losing || fallback_losing)
            enter_long_backoff(s, DFLASH_BACKOFF_FALLBACK);
        else if (alpha_losing)
            enter_long_backoff(s, DFLASH_BACKOFF_ACCEPTANCE);
        return;
    }
    const int window = sampled_mode ? kSampledAlphaWindow : kAlphaWindow;
    push_window(s->alpha_window, &s->n_alpha, window, n_accepted);
    if (s->n_alpha == window) {
        int64_t sum = 0;
        for (int i = 0; i < s->n_alpha; i++) sum += s->alpha_window[i];
        const double mean_emitted = 1.0 + static_cast<double>(sum) / window;
        if (mean_emitted < kBreakevenBase - kAlphaOffMargin)
            s->reason = DFLASH_BACKOFF_ACCEPTANCE;
        else if (s->reason != DFLASH_BACKOFF_NONE)
            s->reason = DFLASH_BACKOFF_NONE;
    }
}

int32_t dflash_speculation_enabled(int32_t spec_disabled, int64_t position, int64_t off_ctx, int64_t remaining_context_tokens,
                                   int32_t block_size, int32_t backoff_active, int32_t backoff_probe_due) {
    return !spec_disabled && position < off_ctx && remaining_context_tokens >= block_size && (!backoff_active || backoff_probe_due);
}

int32_t dflash_prefix_replay_allowed(int32_t spec_disabled, int64_t position, int64_t off_ctx, int64_t remaining_context_tokens,
                                     int32_t block_size, int32_t long_mode, int32_t backoff_active, int32_t backoff_probe_due) {
    return !spec_disabled && position < off_ctx && remaining_context_tokens >= block_size &&
           (!long_mode || !backoff_active || backoff_probe_due);
}

int32_t dflash_prefix_replay_drafts(const int32_t *history, int64_t n_history, const int32_t *emitted, int64_t n_emitted,
                                    int64_t draft_tokens, const int32_t **drafts) {
    if (drafts) *drafts = nullptr;
    if (!history || !emitted || n_emitted > n_history || draft_tokens < 0) return 0;
    for (int64_t i = 0; i < n_emitted; i++)
        if (history[i] != emitted[i]) return 0;
    if (n_emitted + draft_tokens > n_history) return 0;
    if (drafts) *drafts = history + n_emitted;
    return 1;
}

float dflash_verify_fallback_margin(int64_t n_pos) { return n_pos >= DFLASH_OFF_CTX_DEFAULT ? 0.75f : 0.1f; }

}  // extern "C"
