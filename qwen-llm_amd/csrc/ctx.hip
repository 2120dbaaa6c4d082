// Context lifetime, error reporting and block geometry of libdflash_hip.
#include "common.h"

#include <cstdlib>
#include <cstring>
#include <new>

int32_t dfl_fail(dflash_ctx *ctx, int32_t status, const char *fmt, ...) {
    if (ctx) {
        va_list ap;
        va_start(ap, fmt);
        vsnprintf(ctx->err, sizeof(ctx->err), fmt, ap);
        va_end(ap);
    }
    return status;
}

int32_t dfl_raise_lds_limit(dflash_ctx *ctx, const void *fn, size_t bytes) {
    constexpr int kCap = static_cast<int>(sizeof(ctx->lds_attr_fn) / sizeof(ctx->lds_attr_fn[0]));
    for (int i = 0; i < ctx->n_lds_attr; i++)
        if (ctx->lds_attr_fn[i] == fn) {
            if (ctx->lds_attr_bytes[i] >= bytes) return DFLASH_OK;
            DFL_HIP_CHECK(ctx, hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(bytes)));
            ctx->lds_attr_bytes[i] = bytes;
            return DFLASH_OK;
        }
    DFL_HIP_CHECK(ctx, hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(bytes)));
    if (ctx->n_lds_attr < kCap) {  // a full table only costs the repeated runtime call
        ctx->lds_attr_fn[ctx->n_lds_attr] = fn;
        ctx->lds_attr_bytes[ctx->n_lds_attr++] = bytes;
    }
    return DFLASH_OK;
}

extern "C" {

int32_t dflash_ctx_create(int32_t device, size_t workspace_bytes, dflash_ctx **out) {
    if (!out) return DFLASH_ERR_INVALID_INPUT;
    *out = nullptr;
    int count = 0;
    if (hipGetDeviceCount(&count) != hipSuccess || device < 0 || device >= count) return DFLASH_ERR_HIP;
    if (hipSetDevice(device) != hipSuccess) return DFLASH_ERR_HIP;
    dflash_ctx *ctx = new (std::nothrow) dflash_ctx();
    if (!ctx) return DFLASH_ERR_HIP;
    ctx->device = device;
    hipDeviceProp_t prop;
    if (hipGetDeviceProperties(&prop, device) == hipSuccess) {
        ctx->n_cu = prop.multiProcessorCount;
        ctx->lds_bytes = prop.sharedMemPerBlock;
    }
    ctx->workspace_bytes = workspace_bytes ? workspace_bytes : (size_t(128) << 20);
    if (hipMalloc(reinterpret_cast<void **>(&ctx->workspace), ctx->workspace_bytes) != hipSuccess) {
        delete ctx;
        return DFLASH_ERR_HIP;
    }
    ctx->n_partial_wgs = 1024;
    {
        // per workgroup: 2 partial tile sets of (8 waves x 256 floats); a 16-wave workgroup takes two entries
        const size_t bytes = static_cast<size_t>(ctx->n_partial_wgs) * 2 * 8 * 256 * sizeof(float);
        if (hipMalloc(&ctx->partials, bytes) != hipSuccess) {
            dflash_ctx_destroy(ctx);
            return DFLASH_ERR_HIP;
        }
    }
    if (hipEventCreate(&ctx->ev0) != hipSuccess || hipEventCreate(&ctx->ev1) != hipSuccess ||
        hipStreamCreateWithFlags(&ctx->gstream, hipStreamNonBlocking) != hipSuccess ||
        hipEventCreateWithFlags(&ctx->g_in, hipEventDisableTiming) != hipSuccess ||
        hipEventCreateWithFlags(&ctx->g_out, hipEventDisableTiming) != hipSuccess) {
        dflash_ctx_destroy(ctx);
        return DFLASH_ERR_HIP;
    }
    if (hipHostMalloc(&ctx->pinned, DFL_PINNED_BYTES, hipHostMallocDefault) != hipSuccess) {
        ctx->pinned = nullptr;
        dflash_ctx_destroy(ctx);
        return DFLASH_ERR_HIP;
    }
    if (const char *e = getenv("DFLASH_GRAPHS")) ctx->graphs = atoi(e) != 0;
    if (const char *e = getenv("DFLASH_DRAFT_GRAPH")) ctx->draft_graphs = atoi(e) != 0;
    *out = ctx;
    return DFLASH_OK;
}

void dflash_ctx_destroy(dflash_ctx *ctx) {
    if (!ctx) return;
    if (ctx->workspace) (void)hipFree(ctx->workspace);
    if (ctx->partials) (void)hipFree(ctx->partials);
    if (ctx->ev0) (void)hipEventDestroy(ctx->ev0);
    if (ctx->ev1) (void)hipEventDestroy(ctx->ev1);
    for (hipEvent_t e : ctx->stamp_events) (void)hipEventDestroy(e);
    if (ctx->g_in) (void)hipEventDestroy(ctx->g_in);
    if (ctx->g_out) (void)hipEventDestroy(ctx->g_out);
    if (ctx->gstream) (void)hipStreamDestroy(ctx->gstream);
    if (ctx->pinned) (void)hipHostFree(ctx->pinned);
    delete ctx;
}

void dflash_ctx_set_kernel_timing(dflash_ctx *ctx, int32_t enable) {
    if (!ctx) return;
    ctx->timing = enable == 1;
    ctx->stamping = enable == 2;
    ctx->stamps_used = 0;
    for (int i = 0; i < 8; i++) {
        ctx->timed_ms[i] = 0.0;
        ctx->timed_launches[i] = 0;
    }
}

void dflash_ctx_set_graphs(dflash_ctx *ctx, int32_t enable) {
    if (ctx) ctx->graphs = enable != 0;
}

void dflash_ctx_set_draft_graphs(dflash_ctx *ctx, int32_t enable) {
    if (ctx) ctx->draft_graphs = enable != 0;
}

int32_t dflash_ctx_kernel_timing(const dflash_ctx *ctx, int32_t slot, double *total_ms, int64_t *launches) {
    if (!ctx || slot < 0 || slot >= 8 || !total_ms || !launches) return DFLASH_ERR_INVALID_INPUT;
    if (ctx->stamps_used) {  // the stamped dispatches since the last query: wait for them and add their durations up
        dflash_ctx *c = const_cast<dflash_ctx *>(ctx);
        (void)hipDeviceSynchronize();
        for (size_t i = 0; i < c->stamps_used; i++) {
            float ms = 0.0f;
            if (hipEventElapsedTime(&ms, c->stamp_events[2 * i], c->stamp_events[2 * i + 1]) == hipSuccess) {
                c->timed_ms[c->stamp_slot[i]] += ms;
                c->timed_launches[c->stamp_slot[i]] += 1;
            }
        }
        c->stamps_used = 0;
    }
    *total_ms = ctx->timed_ms[slot];
    *launches = ctx->timed_launches[slot];
    return DFLASH_OK;
}

const char *dflash_last_error(const dflash_ctx *ctx) { return ctx ? ctx->err : "no context"; }

const char *dflash_status_name(int32_t s) {
    switch (s) {
    case DFLASH_OK: return "Ok";
    case DFLASH_ERR_BAD_SHAPE: return "BadShape";
    case DFLASH_ERR_UNSUPPORTED: return "Unsupported";
    case DFLASH_ERR_ALIAS: return "Alias";
    case DFLASH_ERR_ALIGNMENT: return "Alignment";
    case DFLASH_ERR_WORKSPACE: return "Workspace";
    case DFLASH_ERR_HIP: return "Hip";
    case DFLASH_ERR_INVALID_INPUT: return "InvalidInput";
    case DFLASH_ERR_INVALID_TOKEN: return "InvalidToken";
    case DFLASH_ERR_PROPOSAL_MISMATCH: return "ProposalMismatch";
    case DFLASH_ERR_STATE: return "State";
    case DFLASH_ERR_EMPTY_LOGITS: return "EmptyLogits";
    case DFLASH_ERR_INVALID_TEMPERATURE: return "InvalidTemperature";
    case DFLASH_ERR_INVALID_TOP_P: return "InvalidTopP";
    case DFLASH_ERR_INVALID_MIN_P: return "InvalidMinP";
    case DFLASH_ERR_NAN_LOGIT: return "NanLogit";
    case DFLASH_ERR_VOCAB_TOO_LARGE: return "VocabularyTooLarge";
    case DFLASH_ERR_NO_CANDIDATES: return "NoCandidates";
    case DFLASH_ERR_PROPOSAL_TOKEN_OUT_OF_RANGE: return "ProposalTokenOutOfRange";
    case DFLASH_ERR_INVALID_PROPOSAL_WEIGHT: return "InvalidProposalWeight";
    case DFLASH_ERR_MISSING_PROPOSAL_TOKEN: return "MissingProposalToken";
    default: return "Unknown";
    }
}

const char *dflash_version(void) { return "dflash_hip 0.1 (gfx950)"; }

// tensor.rs:164-208
size_t dflash_row_bytes(int32_t type, size_t n_in) {
    switch (type) {
    case DFLASH_TYPE_Q4_K:
    case DFLASH_TYPE_Q4_K_TILED:  // (a tiled matrix of a multiple of 256 rows is as long as its row-order original)
        return n_in % DFL_QK_K ? 0 : n_in / DFL_QK_K * DFL_Q4_K_BYTES;
    case DFLASH_TYPE_Q6_K:
    case DFLASH_TYPE_Q6_K_TILED:  // (likewise)
        return n_in % DFL_QK_K ? 0 : n_in / DFL_QK_K * DFL_Q6_K_BYTES;
    case DFLASH_TYPE_Q8_0: return n_in % DFL_QK8_0 ? 0 : n_in / DFL_QK8_0 * DFL_Q8_0_BYTES;
    case DFLASH_TYPE_F32: return n_in * 4;
    case DFLASH_TYPE_F16: return n_in * 2;
    default: return 0;
    }
}

}  // extern "C"
