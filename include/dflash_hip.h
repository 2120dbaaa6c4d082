/*
 * dflash_hip.h - C ABI of the MI355X (gfx950) DFlash speculative-decoding step.
 *
 * Plain C: pointers and sizes only.  Unless a parameter is suffixed `_host`, every
 * pointer is a caller-owned DEVICE pointer; the library never frees or retains
 * caller memory.  Every function returns a DFLASH_* status (0 = OK) and records a
 * message retrievable with dflash_last_error().  Calls enqueue work on the stream
 * passed in (a hipStream_t, given as void*; NULL = the default stream) and do not
 * synchronise unless their name ends in `_sync` or their comment says they return
 * host-side results.
 *
 * Each entry point cites the interface of the reference engine
 * (brittlewis12/qwen-llm, paths relative to its root) that it replaces.
 */
#ifndef DFLASH_HIP_H
#define DFLASH_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct dflash_ctx dflash_ctx;
typedef void *dflash_stream_t; /* hipStream_t */

/* status codes (the reference's Result enums: MetalError::BadShape, DFlashError
 * metal_dflash.rs:2698-2732, SamplingError sampling.rs:278-302, DFlashAcceptError
 * metal_dflash/accept.rs:34-52) */
enum {
    DFLASH_OK = 0,
    DFLASH_ERR_BAD_SHAPE = 1,       /* MetalError::BadShape */
    DFLASH_ERR_UNSUPPORTED = 2,     /* "decline": no kernel for this dtype / size */
    DFLASH_ERR_ALIAS = 3,           /* output aliases an input (dispatch.rs:221-225, 522-526) */
    DFLASH_ERR_ALIGNMENT = 4,
    DFLASH_ERR_WORKSPACE = 5,       /* context workspace too small for this call */
    DFLASH_ERR_HIP = 6,             /* a HIP runtime call failed */
    DFLASH_ERR_INVALID_INPUT = 7,   /* DFlashAcceptError::InvalidInput */
    DFLASH_ERR_INVALID_TOKEN = 8,   /* DFlashAcceptError::InvalidToken / ForwardError::BadToken */
    DFLASH_ERR_PROPOSAL_MISMATCH = 9,
    DFLASH_ERR_STATE = 10,          /* kv_n_pos != start_position and similar guard walls */
    DFLASH_ERR_IO = 11,             /* GgufError::Io: open / stat / mmap failed */
    DFLASH_ERR_FORMAT = 12,         /* GgufError::BadMagic / Decode: not a well-formed GGUF v3 file */
    DFLASH_ERR_METADATA = 13,       /* LoadError::BadMetadata / Missing / Shape / UnsupportedArch */
    /* sampling errors, numbered 32 + the sampler's own code */
    DFLASH_ERR_EMPTY_LOGITS = 33,
    DFLASH_ERR_INVALID_TEMPERATURE = 34,
    DFLASH_ERR_INVALID_TOP_P = 35,
    DFLASH_ERR_INVALID_MIN_P = 36,
    DFLASH_ERR_NAN_LOGIT = 37,
    DFLASH_ERR_VOCAB_TOO_LARGE = 38,
    DFLASH_ERR_NO_CANDIDATES = 39,
    DFLASH_ERR_PROPOSAL_TOKEN_OUT_OF_RANGE = 40,
    DFLASH_ERR_INVALID_PROPOSAL_WEIGHT = 41,
    DFLASH_ERR_MISSING_PROPOSAL_TOKEN = 42
};

/* ggml tensor type tags (crates/qwen-llm/src/tensor.rs:164-208) */
enum { DFLASH_TYPE_F32 = 0, DFLASH_TYPE_F16 = 1, DFLASH_TYPE_Q8_0 = 8, DFLASH_TYPE_Q4_K = 12, DFLASH_TYPE_Q6_K = 14 };
/* Not ggml types: Q4_K blocks in this library's tiled order (dflash_repack_q4k_tiled); Q6_K blocks in its tiled,
 * field-planar order (dflash_repack_q6k_tiled), which only dflash_gemm_fewrow_xf and the model-level calls take. */
enum { DFLASH_TYPE_Q4_K_TILED = 1012, DFLASH_TYPE_Q6_K_TILED = 1014 };

/* ---- context ------------------------------------------------------------------
 * Replaces MetalContext + the per-call scratch the reference keeps in
 * MetalDFlashVerifyScratch / MetalDFlashLayerMajorScratch (metal_dflash.rs:5863-5905,
 * 7240-7443).  `workspace_bytes` of device memory are allocated once here (0 = 128 MiB)
 * and reused by every call; calls on one context must not overlap. */
int32_t dflash_ctx_create(int32_t device, size_t workspace_bytes, dflash_ctx **out);
void dflash_ctx_destroy(dflash_ctx *ctx);
const char *dflash_last_error(const dflash_ctx *ctx);
const char *dflash_status_name(int32_t status);
const char *dflash_version(void);

/* Per-kernel GPU timers: enable_phase_timers / maybe_record (metal_dflash.rs:5181-5190, 5622).
 * While enabled, each call brackets its dominant kernel with events on the call's stream and
 * waits for it, accumulating into a slot: 0 few-row GEMM, 1 verify attention, 2 acceptance,
 * 3 argmax/top-k, 4 split-K reduction of the few-row GEMM.  enable == 2 instead: nothing waits; the single-matrix
 * Q4_K streaming kernel (slot 5) and its reduction (slot 6) are dispatched with start / stop stamps of their own - the
 * duration a kernel trace reports, without the dispatch latency an event pair around a launch includes, and with the
 * kernels still running back to back - which dflash_ctx_kernel_timing waits for and adds up when it is called.
 * Changing the mode clears the slots. */
void dflash_ctx_set_kernel_timing(dflash_ctx *ctx, int32_t enable);
int32_t dflash_ctx_kernel_timing(const dflash_ctx *ctx, int32_t slot, double *total_ms_host,
                                 int64_t *launches_host);
/* Graph replay of the packed verify (the counterpart of the reference's one command buffer per
 * verify block, encode_packed_verify_layer_major, metal_dflash.rs:10696-10719): a verify shape
 * (model tensors, row count, taps, output pointers) is run launch by launch the first time,
 * captured into a HIP graph the second time and replayed from then on, with the position read
 * from device memory.  Off by default (environment DFLASH_GRAPHS=1 or this call turn it on):
 * on ROCm 7.2 a replay measured slightly slower than the launches it replaces; results are
 * bit-identical either way.  Kernel timers switch it off while they are enabled. */
void dflash_ctx_set_graphs(dflash_ctx *ctx, int32_t enable);
/* The drafter's block forward (dflash_draft_block and the draft phase of dflash_spec_step: about 80 launches of
 * 4..8 us kernels) can be captured into a HIP graph on the second call with the same head / target / output pointers
 * and replayed from then on; ids, positions and the context length travel through device memory, so one graph serves
 * every step.  Off by default (environment DFLASH_DRAFT_GRAPH=1 or this call turn it on): on ROCm 7.2 a replayed
 * block measured 0.79 ms against 0.77 ms launched one by one; results are bit-identical either way.  Not used for the general
 * attention path (non-contiguous context positions), for a DFlash-2 selector walk that is not skipped, or while kernel
 * timers are enabled. */
void dflash_ctx_set_draft_graphs(dflash_ctx *ctx, int32_t enable);

/* ---- block dequantisation -------------------------------------------------------
 * codec::dequant_to_f32{,_into,_in_place} (codec.rs:256-302): ggml blocks -> f32,
 * bit-exact with ggml's dequantize_row_{q4_K,q6_K,q8_0}.  n_elems must be a multiple
 * of the block size (codec.rs:91-103). */
int32_t dflash_dequant(dflash_ctx *ctx, int32_t type, const void *blocks, size_t n_elems, float *out_f32,
                       dflash_stream_t stream);
size_t dflash_row_bytes(int32_t type, size_t n_in);

/* ---- scale range of a quantised tensor: the precondition of the fast kernels ------------------------
 * No counterpart in the reference: its kernels scale in f32 after the MMA (mat_mat_fewrow_gen.metal:437-444) and take
 * any ggml block.  The fast few-row Q4_K / Q6_K kernels here apply d * scale in f16 before the MFMA, which is finite
 * only while
 *   Q4_K: |d| <= DFLASH_Q4_K_MAX_D and |dmin| <= DFLASH_Q4_K_MAX_DMIN,   Q6_K: |d| <= DFLASH_Q6_K_MAX_D
 * (weight scales of real checkpoints are 1e-4 .. 1e-1).  The precondition is part of the tensor's tag:
 *   - dflash_check_scale_range scans a tensor's super-block headers on the device (once, when it is uploaded),
 *     returns the maxima in max_abs_host[2] (|d|, |dmin|; may be NULL) and DFLASH_ERR_UNSUPPORTED with a message for
 *     a tensor out of range or with a NaN / infinite scale, DFLASH_OK otherwise (and for types whose kernels have
 *     no such limit).  Blocking.
 *   - Only a tensor that passed may be tagged as checked: w_type | DFLASH_TYPE_RANGE_CHECKED where a call takes the
 *     type as an argument, flags = DFLASH_QT_RANGE_CHECKED in a dflash_qtensor.  dflash_repack_q4k_tiled runs the
 *     scan itself, so DFLASH_TYPE_Q4_K_TILED is checked by construction.
 *   - dflash_gemm_fewrow / dflash_gemm_fewrow_noalloc on an UNTAGGED Q4_K / Q6_K tensor run a kernel that dequantises
 *     in f32 exactly as ggml does and accumulates in f32: correct for every block a GGUF file can hold (what the
 *     reference's seam promises), about two orders of magnitude slower.  The model-level calls
 *     (dflash_verify_block, dflash_prefill_blocks, dflash_draft_block, dflash_draft_prepare_ctx, dflash_spec_step)
 *     decline a model that holds an untagged Q4_K / Q6_K tensor with DFLASH_ERR_UNSUPPORTED, naming it.
 * A result is therefore either correct or declined: never an infinity with status 0. */
#define DFLASH_Q4_K_MAX_D 1.0f
#define DFLASH_Q4_K_MAX_DMIN 32.0f
#define DFLASH_Q6_K_MAX_D 0.25f
enum {
    DFLASH_TYPE_RANGE_CHECKED = 65536, /* 0x10000, OR-ed into a w_type argument */
    DFLASH_QT_RANGE_CHECKED = 1        /* dflash_qtensor.flags */
};
int32_t dflash_check_scale_range(dflash_ctx *ctx, int32_t type, const void *blocks, size_t n_blocks, float *max_abs_host,
                                 dflash_stream_t stream);

/* ---- Q4_K weights in tiled order -------------------------------------------------
 * No counterpart in the reference (it streams GGUF row order, loader.rs tensors as mapped): a one-time
 * permutation of whole 144-byte blocks, done when a matrix is uploaded, into the order the M <= 16 GEMM reads it in:
 *   [tile group of 256 rows][super-block][tile 0..15][row 0..15][block],  last group padded with zero blocks.
 * dflash_q4k_tiled_bytes: size of the tiled matrix (0 for a bad shape).  dflash_repack_q4k_tiled: W in GGUF row
 * order (16-byte aligned) -> w_tiled (128-byte aligned, dflash_q4k_tiled_bytes long, not overlapping W).  The
 * result is passed to dflash_gemm_fewrow as w_type DFLASH_TYPE_Q4_K_TILED and gives bit-identical Y.  The source is
 * range-checked first (dflash_check_scale_range; DFLASH_ERR_UNSUPPORTED for a tensor out of range, nothing is written
 * then), so a tiled tensor is always one the fast kernels take.  Blocking. */
size_t dflash_q4k_tiled_bytes(int64_t n_in, int64_t n_out);
int32_t dflash_repack_q4k_tiled(dflash_ctx *ctx, const void *w, void *w_tiled, int64_t n_in, int64_t n_out,
                                dflash_stream_t stream);
/* The same idea for Q6_K matrices that only the one-launch GEMM below (dflash_gemm_fewrow_xf and the model-level
 * calls) reads - a 2048-wide model's attention projections: [tile group of 256 rows][super-block][tile 0..15][3360
 * bytes], a tile's sixteen 210-byte blocks stored field by field (ql [row][128], qh [row][64], scales [row][16],
 * d [row]) so that every 16-byte piece a lane fetches is aligned; same values, bit-identical Y.  w_type
 * DFLASH_TYPE_Q6_K_TILED.  dflash_gemm_fewrow does NOT take this type (DFLASH_ERR_UNSUPPORTED): tile a matrix only
 * where dflash_gemm_fewrow_xf_kind(ctx, DFLASH_TYPE_Q6_K_TILED, n_in, n_out) is not DFLASH_XF_NONE.  Source 2-byte,
 * destination 128-byte aligned; range-checked first, as above.  Blocking. */
size_t dflash_q6k_tiled_bytes(int64_t n_in, int64_t n_out);
int32_t dflash_repack_q6k_tiled(dflash_ctx *ctx, const void *w, void *w_tiled, int64_t n_in, int64_t n_out,
                                dflash_stream_t stream);

/* ---- few-row quantised GEMM ---------------------------------------------------
 * encode_mat_mat_dispatch_dflash_verify(ctx, enc, weight, x, y, n_in, n_out, n_query)
 * (metal_forward/dispatch.rs:365-378; kernel kernels/mat_mat_fewrow_gen.metal:374-474).
 *   Y[n_rows][n_out] = X[n_rows][n_in] . W^T,  W = quant blocks, row-major [n_out][n_in/blk]
 * x_type: DFLASH_TYPE_F32 (the reference's activations) or DFLASH_TYPE_F16; Y is f32.
 * w_type: a ggml tag (any block of that type is computed correctly), or tag | DFLASH_TYPE_RANGE_CHECKED /
 * DFLASH_TYPE_Q4_K_TILED for a tensor that passed dflash_check_scale_range (the fast kernels).
 * 1 <= n_rows <= 16; n_in % 256 == 0 (Q4_K, Q6_K) or % 32 == 0 (Q8_0, and plain F32 / F16 matrices
 * such as a router stored unquantised); W 16-byte aligned (2-byte for Q8_0 and Q6_K); Y must not
 * alias X or W.  Enqueue-only. */
int32_t dflash_gemm_fewrow(dflash_ctx *ctx, int32_t w_type, const void *w, const void *x, int32_t x_type, float *y,
                           int64_t n_in, int64_t n_out, int32_t n_rows, dflash_stream_t stream);

/* The same product for callers that cannot allocate: code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc.  No counterpart in the reference.  It takes no context and calls no
 * hipMalloc / hipFree or any allocating routine: the split-K partial tiles that dflash_gemm_fewrow keeps in
 * its context's buffer live in a fixed 8 MiB array of the library's device image (one copy per GPU, held until
 * the process ends).  Same arguments, guards, kernels and results (bit for bit) as dflash_gemm_fewrow on a
 * GPU of up to 256 compute units; the launch never uses more workgroups than the array has partial-tile
 * sets for.  Shapes beyond DFLASH_NOALLOC_MAX_N_IN / DFLASH_NOALLOC_MAX_N_OUT are refused with
 * DFLASH_ERR_BAD_SHAPE.  Runs on the CURRENT device (hipSetDevice): `stream` must belong to it, and the scratch
 * array and compute-unit count used are that device's.  Bit-identity with dflash_gemm_fewrow holds while both use the
 * same number of workgroups, i.e. with the environment knob DFLASH_GEMM_WGS unset (a debugging aid; the two entry
 * points cap it differently).  A type tag without DFLASH_TYPE_RANGE_CHECKED takes the f32 kernel, as in
 * dflash_gemm_fewrow.  All calls on one GPU share that GPU's array: calls
 * on one stream are ordered; calls that overlap in time on the same GPU (several streams or threads) race.
 * Enqueue-only.  dflash_gemm_fewrow_noalloc_error() returns the calling thread's last message. */
#define DFLASH_NOALLOC_MAX_N_IN 262144
#define DFLASH_NOALLOC_MAX_N_OUT 1048576
int32_t dflash_gemm_fewrow_noalloc(int32_t w_type, const void *w, const void *x, int32_t x_type, float *y,
                                   int64_t n_in, int64_t n_out, int32_t n_rows, dflash_stream_t stream);
const char *dflash_gemm_fewrow_noalloc_error(void);

/* ---- few-row GEMM over activations in fragment order -----------------------------------------
 * No counterpart in the reference (its kernels read row-major f32 activations, dispatch.rs:365-378).  The small
 * projections of a layer (a few MB: the q/k/v, output and drafter matrices of a 2048-wide model) are bound by launch
 * latency and by a split-K sum through memory, not by bytes.  Where the kernel that produces the 16 activation rows
 * can write them as f16 in the order the MFMA operands are read ("XF": per 256 values of K, 512 slots of 16 bytes;
 * slot (t, lane = 16 g + row) holds eight consecutive values of the row, the octet given by the consumer's type),
 * one launch computes the whole product with every output tile's K inside one workgroup: no partial tiles, no
 * second launch.  dflash_verify_block / dflash_draft_block use this hand-off between their own kernels; these three
 * calls expose it.
 *   dflash_xf_bytes: size of an XF buffer for n_in values per row (n_in % 256 == 0; 0 otherwise).
 *   dflash_gemm_fewrow_xf_kind: the XF kind (DFLASH_XF_Q4K / DFLASH_XF_Q6K) this (type, shape) reads, or
 *     DFLASH_XF_NONE where it is not taken: w_type must be DFLASH_TYPE_Q4_K_TILED, DFLASH_TYPE_Q6_K_TILED or
 *     DFLASH_TYPE_Q6_K | DFLASH_TYPE_RANGE_CHECKED (these kernels scale in f16: a range-checked tensor only), n_in at most 8192, and
 *     the matrix at most one round of the chip (about 320 workgroups of 16 or 32 rows).
 *   dflash_pack_xf: row-major x[n_rows][n_in] (f32 or f16) -> xf, rounding to f16 as every few-row kernel does.
 *   dflash_gemm_fewrow_xf: Y[n_rows][n_out] = X . W^T; same guards as dflash_gemm_fewrow; DFLASH_ERR_UNSUPPORTED
 *     where the kind is DFLASH_XF_NONE.  A (row, column) result depends on that activation row and weight row only.
 * All enqueue-only. */
enum { DFLASH_XF_NONE = 0, DFLASH_XF_Q4K = 1, DFLASH_XF_Q6K = 2 };
size_t dflash_xf_bytes(int64_t n_in);
int32_t dflash_gemm_fewrow_xf_kind(dflash_ctx *ctx, int32_t w_type, int64_t n_in, int64_t n_out);
int32_t dflash_pack_xf(dflash_ctx *ctx, const void *x, int32_t x_type, int32_t n_rows, int64_t n_in, int32_t kind, void *xf,
                       dflash_stream_t stream);
int32_t dflash_gemm_fewrow_xf(dflash_ctx *ctx, int32_t w_type, const void *w, const void *xf, float *y, int64_t n_in,
                              int64_t n_out, int32_t n_rows, dflash_stream_t stream);

/* ---- block-causal verify attention ------------------------------------------------
 * The reference verifies a block with a per-row loop: encode_scatter_offset_f32_to_f16_kv +
 * encode_attn_decode_v4_f32 / encode_attn_decode_f16kv_f32, once per row
 * (metal_dflash.rs:9963-10062; kernels/attn_v4.metal, kernels/attn.metal:266-336; CPU form
 * forward.rs:893-922).  This call is those n_rows launches in one: row i attends cache
 * positions [0, ctx_len + i].
 *   q        [n_rows][n_q][head_dim], f32 or f16 (q_type)
 *   k_cache  [kv_capacity][n_kv][head_dim] f16; rows ctx_len .. ctx_len+n_rows-1 hold the block
 *   v_cache  v_layout 0: same layout as k_cache (transposed into workspace first; small caches)
 *            v_layout 1: transposed [n_kv][head_dim][kv_capacity] f16 (native; capacity % 32 == 0)
 *   out      [n_rows][n_q][head_dim] f32
 * 1 <= n_rows <= 16; n_q % n_kv == 0 with at most 16 query heads per KV head; head_dim 64, 128
 * or 256.  Enqueue-only. */
int32_t dflash_attn_verify_block(dflash_ctx *ctx, const void *q, int32_t q_type, const void *k_cache,
                                 const void *v_cache, int32_t v_layout, int64_t ctx_len, int32_t n_rows, int32_t n_q,
                                 int32_t n_kv, int32_t head_dim, int64_t kv_capacity, float scale, float *out,
                                 dflash_stream_t stream);

/* ---- row-wise selection over logits -------------------------------------------------
 * logits [n_rows][stride] f32 (stride >= vocab).  All enqueue-only, outputs on the device.
 *
 * dflash_argmax_top2: kernel_argmax_top2_f32 (kernels/elementwise.metal:1231-1286, encoder
 *   metal/elementwise.rs:1196-1318): IEEE comparisons, lowest index on ties, gap = top1 - top2
 *   (0 when the maximum occurs twice, +inf for vocab == 1), an all-NaN row gives index -1.
 * dflash_argmax_greedy: kernel_argmax_f32_greedy (elementwise.metal:1300-1359) == greedy_token
 *   (sampling.rs:1159-1181): f32 total order, lowest index on ties, a row with a NaN gives
 *   ~(lowest NaN index).
 * dflash_top16: kernel_topk16_f32 (kernels/dflash2.metal:96-170): the 16 best (value, index)
 *   pairs by total order, ties to the lower index; unfilled slots are (-inf, -1). */
int32_t dflash_argmax_top2(dflash_ctx *ctx, const float *logits, int32_t n_rows, int64_t vocab, int64_t stride,
                           int32_t *idx, float *gap, dflash_stream_t stream);
int32_t dflash_argmax_greedy(dflash_ctx *ctx, const float *logits, int32_t n_rows, int64_t vocab, int64_t stride,
                             int32_t *idx, dflash_stream_t stream);
int32_t dflash_top16(dflash_ctx *ctx, const float *logits, int32_t n_rows, int64_t vocab, int64_t stride,
                     int32_t *ids, float *vals, dflash_stream_t stream);

/* ---- DFlash-2 extras ---------------------------------------------------------------------
 * dflash_dflash2_conv: kernel_dflash2_conv_f32 (kernels/dflash2.metal:40-69, encoder
 *   metal/dflash.rs:98-111): y[t][c] = sum_tap (base[side][tap][c] + dyn[t][side][tap][c / group_size])
 *   * x[t - tap][c], rows before the block read as zeros.  x, y [n_tokens][h] f32 (y must not alias
 *   x); dyn [n_tokens][2 * kernel_size * h / group_size] f32, (group, tap, side) fastest to slowest;
 *   base [2][kernel_size][h] f32.  Enqueue-only.
 * dflash_select_draft_path: select_draft_path (metal_dflash.rs:17176-17251) with
 *   DFlash2Codebook::dequant_row (:3275-3343), run on the device so that the top-16 and the
 *   selector hidden never leave it: out[0] = topk_ids[0]; for every later position the candidate b
 *   maximising topk_vals[pos][b] + sum_r (pred[r] * sel_h[pos][r]) * succ_b[r] (sums in rank order,
 *   products and additions rounded separately; strict >, so the first maximum wins and candidate 0
 *   when nothing compares greater; candidates below 0 or past the successor table are skipped);
 *   the winner's predecessor row conditions the next position.  Codebooks are [n_rows][rank] rows
 *   of F32, F16, Q8_0 or Q4_K in device memory (data on a 2-byte boundary); topk_ids/topk_vals [n][top_k], sel_h [n][rank] and
 *   out_tokens [n] are device pointers; top_k <= 16, rank <= 1024, n <= 16.  With out_tokens_host
 *   the call waits, copies the tokens and returns DFLASH_ERR_INVALID_TOKEN if a predecessor row was
 *   out of range (the reference's BadDrafter("selector codebook row out of range")); without it the
 *   call only enqueues. */
typedef struct {
    int32_t type; /* DFLASH_TYPE_F32 / F16 / Q8_0 / Q4_K */
    int32_t pad;
    int64_t n_rows;
    const void *data; /* device */
} dflash_codebook;

int32_t dflash_dflash2_conv(dflash_ctx *ctx, const float *x, const float *dyn, const float *base, float *y,
                            int32_t n_tokens, int32_t h, int32_t kernel_size, int32_t group_size, int32_t side,
                            dflash_stream_t stream);
int32_t dflash_select_draft_path(dflash_ctx *ctx, const dflash_codebook *predecessor, const dflash_codebook *successor,
                                 int32_t rank, int32_t top_k, int32_t carry_token, int32_t n, const int32_t *topk_ids,
                                 const float *topk_vals, const float *sel_h, int32_t *out_tokens,
                                 int32_t *out_tokens_host, dflash_stream_t stream);

/* ---- sampler state (host side) ------------------------------------------------------
 * SamplingConfig / Sampler (sampling.rs:18-145, 304-366): one request-local random stream.
 * rng_kind 0 = xoshiro256++ seeded by SplitMix64 (the reference's generator, sampling.rs:1621-1670),
 * 1 = Philox4x32-10 counter stream (key = seed, counter = draw index; u64 = word0 | word1 << 32).
 * A unit draw is (u64 >> 11) / 2^53. */
typedef struct {
    float temperature; /* 0 = greedy */
    float top_p;       /* (0, 1] */
    float min_p;       /* [0, 1] */
    int32_t rng_kind;
    uint64_t top_k;    /* 0 = off */
    uint64_t seed;
} dflash_sampling_config;

typedef struct {
    dflash_sampling_config cfg;
    uint64_t s[4];  /* xoshiro state, or s[0] = Philox stream position */
    uint64_t draws;
} dflash_sampler;

int32_t dflash_sampler_init(dflash_sampler *s, const dflash_sampling_config *cfg);             /* Sampler::new */
int32_t dflash_sampler_at_draw(dflash_sampler *s, const dflash_sampling_config *cfg, uint64_t draws); /* ::at_draw */
/* the next `n` unit draws of the stream, without advancing it (Sampler::gpu_uniform, sampling.rs:317-326) */
void dflash_sampler_peek(const dflash_sampler *s, int32_t n, double *out_host);
void dflash_sampler_advance(dflash_sampler *s, uint64_t draws);

/* ---- accept-prefix decision ---------------------------------------------------------
 * decide_dflash_accept_prefix (metal_dflash/accept.rs:76-183) with the Sampler's couplings
 * (sampling.rs:530-603, 692-790), evaluated on the GPU.  Row r of target_logits predicts
 * verified_tokens[r+1]; the last reached row supplies the bonus.
 *   proposal_mode 0: deterministic drafts (couple_deterministic_proposal)
 *                 1: sparse proposals: n_proposals (= n_tokens - 1) rows; row r has
 *                    prop_counts_host[r] (token, weight) candidates, stored back to back
 *                    (couple_sparse_proposal; prop_tokens_host[r] must equal verified_tokens[r+1])
 *                 2: vocabulary-wide draft distribution softmax(draft_logits / draft_temperature)
 *                    (sum order: 1024-token tiles, 256 four-element slots, halving tree, tiles
 *                    added in order)
 * The whole block is validated before anything is drawn; the sampler advances by the draws
 * actually consumed and only on DFLASH_OK.  Any top_k (sampling.rs:1198-1214, 1273-1296): up to 64
 * candidates per row stay on the streaming selection kernels; top_k = 0 (the whole vocabulary) and
 * top_k > 64 order the block's rows with one device-wide sort and need about 3 * 8 bytes per
 * (row, token) of context workspace (DFLASH_ERR_WORKSPACE names the figure).  Synchronises: the
 * decision is returned on the host. */
enum { DFLASH_CARRY_NONE = 0, DFLASH_CARRY_CORRECTION = 1, DFLASH_CARRY_BONUS = 2 };
enum { DFLASH_STOP_NONE = 0, DFLASH_STOP_EOS = 1, DFLASH_STOP_TOKEN_LIMIT = 2 };

typedef struct {
    int32_t n_accepted;
    int32_t accepted_drafts[16];
    int32_t carry_kind;
    int32_t carry_token;
    int32_t stop_reason;
    int32_t retain_input_count;
    int32_t draws_used;
    int32_t err_row;    /* row of a sampling error, else -1 */
    int32_t err_code;   /* DFLASH_ERR_* of that error */
    int64_t err_index;  /* offending token / NaN index, else -1 */
} dflash_accept_decision;

typedef struct {
    int32_t token;
    int32_t pad;
    double weight;
} dflash_weighted_candidate;

int32_t dflash_accept_prefix(dflash_ctx *ctx, const int32_t *verified_tokens_host, int32_t n_tokens,
                             const float *target_logits, int64_t vocab, int32_t proposal_mode, int32_t n_proposals,
                             const int32_t *prop_tokens_host, const int32_t *prop_counts_host,
                             const dflash_weighted_candidate *prop_cands_host, const float *draft_logits,
                             float draft_temperature, dflash_sampler *sampler, int64_t remaining_output_budget,
                             const int32_t *stop_ids_host, int32_t n_stop, dflash_accept_decision *out_host,
                             dflash_stream_t stream);

/* draft_block_sampled (metal_dflash.rs:17268-17415): the selector walk of dflash_select_draft_path,
 * but every position draws its token from softmax(score / T) over the top_k candidates with the
 * proposal sampler (sample_with_distribution, sampling.rs:439-453: one draw per position; skipped
 * candidates score -inf) and the sampled token conditions the next position.  The proposal sampler
 * must use temperature only (temperature > 0, top_k 0, top_p 1, min_p 0), as the reference demands.
 * Blocking; outputs on the host: out_tokens_host [n] (every slot pre-filled with the anchor's
 * top-1, slots 1.. the sampled tokens), and for position p >= 1 the sparse proposal
 * prop_cands_host[(p-1) * top_k ..][0 .. prop_counts_host[p-1]) = (token, weight) of the candidates
 * with positive weight in distribution order: what decide / dflash_accept_prefix take as
 * SparseProposal.  The sampler advances by the draws made; errors: DFLASH_ERR_INVALID_TOKEN (codebook
 * row out of range) or the sampler's own codes (NaN score, no candidate with finite score). */
int32_t dflash_select_draft_path_sampled(dflash_ctx *ctx, const dflash_codebook *predecessor,
                                         const dflash_codebook *successor, int32_t rank, int32_t top_k,
                                         int32_t carry_token, int32_t n, const int32_t *topk_ids, const float *topk_vals,
                                         const float *sel_h, dflash_sampler *proposal_sampler, int32_t *out_tokens_host,
                                         int32_t *prop_counts_host, dflash_weighted_candidate *prop_cands_host,
                                         dflash_stream_t stream);

/* ---- target model, session, packed verify -----------------------------------------------
 * Weights stay GGUF quant blocks used in place (crates/qwen-llm/src/lib.rs:17-18): a tensor is
 * a type tag and a device pointer to row-major [n_out][n_in/blk] blocks.  Norm weights are f32.
 * The block structure is the plain pre-norm decoder of forward.rs:96-163 with per-head q/k
 * RMSNorm and full-width NeoX RoPE (attn_step, forward.rs:834-932, without the q-gate and the
 * Gated-DeltaNet layers of the hybrid target, which the synthetic configurations do not have). */
typedef struct {
    int32_t type;
    int32_t flags; /* DFLASH_QT_RANGE_CHECKED: the tensor passed dflash_check_scale_range (Q4_K / Q6_K; see there) */
    const void *data; /* device */
} dflash_qtensor;

typedef struct {
    int32_t n_layers, hidden, n_q, n_kv, head_dim, ffn, vocab;
    int32_t n_expert, n_expert_used, ffn_expert, ffn_shared; /* n_expert == 0: dense FFN */
    float eps, rope_theta;
} dflash_model_cfg;

typedef struct {
    const float *attn_norm, *q_norm, *k_norm, *post_norm; /* device f32 */
    dflash_qtensor wq, wk, wv, wo, gate, up, down;        /* dense FFN, or the shared expert */
    dflash_qtensor router;                                /* [hidden -> n_expert] (MoE) */
    const float *shexp_gate;                              /* [hidden] f32 (MoE) */
    dflash_qtensor gate_exps, up_exps, down_exps;         /* n_expert stacked matrices (MoE) */
} dflash_layer;

typedef struct {
    dflash_model_cfg cfg;
    const dflash_layer *layers; /* host array of n_layers */
    dflash_qtensor token_embd, output;
    const float *output_norm;
} dflash_model;

/* MetalSession for the target (KV f16, kv_n_pos) plus MetalDFlashVerifyScratch /
 * MetalDFlashLayerMajorScratch (metal_dflash.rs:5863-5905, 7240-7443).  K is cached as
 * [layer][capacity][n_kv][head_dim], V transposed as [layer][n_kv][head_dim][capacity]; capacity
 * is rounded up to a multiple of 32. */
typedef struct dflash_session dflash_session;
int32_t dflash_session_create(dflash_ctx *ctx, const dflash_model_cfg *cfg, int64_t kv_capacity, int32_t n_taps,
                              dflash_session **out);
void dflash_session_destroy(dflash_session *s);
int64_t dflash_session_kv_n_pos(const dflash_session *s);
/* How many verify calls of this session were served by replaying a captured graph (see
 * dflash_ctx_set_graphs); no counterpart in the reference, used by tests and benchmarks. */
int64_t dflash_session_graph_replays(const dflash_session *session);

/* encode_packed_verify_layer_major_inner(base, target_layer_ids, tokens, start_position, ...,
 * debug_logits_dst, n_eff_override) (metal_dflash.rs:10696-10719): forward of tokens[n] at
 * positions start_position .. start_position+n-1, layer-major, K/V appended to the session.
 * Guards: kv_n_pos == start_position, start+n <= capacity, tokens in the vocabulary.
 * Outputs (device, may be NULL): argmax[n] i32 and gap[n] f32 (argmax_top2 of each row),
 * hidden_capture[n][n_taps][hidden] f32 (residual stream after the tapped layers, :10535-10551),
 * logits[n][vocab] f32.  If argmax_host is non-NULL the call waits and copies the n indices
 * there (the reference returns Vec<i32>).  With argmax, gap, logits and argmax_host all NULL the
 * output head (final norm, vocabulary projection, argmax) is not run: a prefill block, of which
 * only the K/V rows and the tapped hidden rows are wanted (the last layer then stops behind its
 * K/V rows unless its residual is tapped).  1 <= n <= 16. */
int32_t dflash_verify_block(dflash_ctx *ctx, const dflash_model *model, dflash_session *session,
                            const int32_t *tokens_host, int32_t n, int64_t start_position,
                            const int32_t *tap_layers_host, int32_t n_taps, int32_t *argmax, float *gap,
                            float *hidden_capture, float *logits, int32_t *argmax_host, dflash_stream_t stream);

/* encode_restore_after_partial_accept_inner (metal_dflash.rs:15649-15777): must directly follow
 * the matching verify; 1 <= n_keep <= n; sets kv_n_pos = start_position + n_keep (stale KV rows
 * stay in place and are overwritten by the next verify).  n_keep == 0 restores the pre-block
 * state (encode_restore_to_pre_block, :15789-15905). */
int32_t dflash_restore(dflash_ctx *ctx, dflash_session *session, int64_t start_position, int32_t n, int32_t n_keep);

/* The packed prefill with hidden capture (metal_dflash.rs:10779-15648; the reference walks the prompt in chunks of
 * layer_scratch.n rows, :10770-10778): tokens_host[n_tokens] at positions start_position .., through the same layers
 * as dflash_verify_block, without the output head; K/V rows are appended, the tapped hidden rows go to
 * hidden_capture[n_tokens][n_taps][hidden] (device; may be NULL with n_taps = 0).  Two schedules, same results:
 *   - a mixture-of-experts target whose expert stacks and shared expert are tiled Q4_K and whose q/k/v and output
 *     projections take the one-launch GEMM: the rows of up to 32 consecutive blocks (DFLASH_PREFILL_GROUP, 2..32;
 *     0 = never) pass through a layer together on the caller's stream - every projection once for all of them, the
 *     experts regrouped by expert - so a pass reads a layer's weights about once;
 *   - any other target: 16-row blocks, up to four in flight on as many streams (DFLASH_PREFILL_LANES, 1..8), ordered
 *     by per-layer events where a block reads the earlier blocks' K/V rows; the caller's stream continues behind all
 *     of them.
 * The scratch of both (group buffers; extra streams, scratch sets and contexts' workspaces) belongs to the session and
 * is made on the first call.  Results equal those of the same blocks through dflash_verify_block bit for bit.  Guards
 * as dflash_verify_block; on an error kv_n_pos is unchanged. */
/* Makes the group buffers, extra streams, scratch sets and contexts of dflash_prefill_blocks ahead of its first call (which makes
 * them otherwise): the allocations then stay out of the first prompt's latency.  No counterpart in the reference. */
int32_t dflash_prefill_prepare(dflash_ctx *ctx, dflash_session *session);
int32_t dflash_prefill_blocks(dflash_ctx *ctx, const dflash_model *model, dflash_session *session,
                              const int32_t *tokens_host, int32_t n_tokens, int64_t start_position,
                              const int32_t *tap_layers_host, int32_t n_taps, float *hidden_capture,
                              dflash_stream_t stream);

/* ---- block drafter ----------------------------------------------------------------------
 * DFlashConfig / DFlashHead / DFlashLayer (loader.rs:342-399), MetalDFlashSession
 * (metal_dflash.rs:5053-5191). */
typedef struct {
    int32_t n_layers, hidden, n_q, n_kv, head_dim, ffn, block_size, n_taps;
    int32_t causal;
    uint32_t swa_window; /* 0 = full */
    float eps, rope_theta;
    /* DFlash-2 (loader.rs:367-376, 1030-1056); all zero for a DFlash-1 drafter.  conv_kernel_size > 0:
     * every layer carries the two convolution pairs; selector_rank > 0: the head carries the
     * selector (selector_top_k must then be 16, the width of the top-16 kernel). */
    int32_t conv_kernel_size, conv_group_size, selector_rank, selector_top_k;
} dflash_draft_cfg;

typedef struct {
    const float *attn_norm, *q_norm, *k_norm, *post_norm;
    dflash_qtensor wq, wk, wv, wo, gate, up, down;
    int32_t is_swa;
    int32_t pad;
    /* DFlashConvTensors (loader.rs:305-323): blk.N.{attn,ffn}_conv_proj.weight
     * [hidden -> 2 * kernel * hidden / group] and blk.N.{attn,ffn}_conv_base, f32 [2][kernel][hidden] */
    dflash_qtensor conv_attn_proj, conv_ffn_proj;
    const float *conv_attn_base, *conv_ffn_base;
} dflash_draft_layer;

typedef struct {
    dflash_draft_cfg cfg;
    const dflash_draft_layer *layers; /* host array */
    dflash_qtensor fc;                /* [n_taps*hidden -> hidden] */
    const float *hidden_norm, *output_norm;
    /* DFlashSelectorTensors (loader.rs:325-340): selector_hidden.weight [hidden -> rank] and the
     * per-token predecessor / successor tables, [vocab][rank] */
    dflash_qtensor selector_hidden;
    dflash_codebook selector_predecessor, selector_successor;
} dflash_draft_head;

typedef struct dflash_draft_session dflash_draft_session;
int32_t dflash_draft_session_create(dflash_ctx *ctx, const dflash_draft_cfg *cfg, int64_t ctx_capacity,
                                    int64_t vocab, dflash_draft_session **out);
void dflash_draft_session_destroy(dflash_draft_session *s);
int64_t dflash_draft_session_ctx_len(const dflash_draft_session *s);
int64_t dflash_draft_session_graph_replays(const dflash_draft_session *s);

/* append_target_ctx_columns_now (metal_dflash.rs:5798-5860): append n_cols captured hidden rows
 * (hidden_capture layout [col][n_taps][hidden], device f32) with their positions. */
int32_t dflash_draft_append_ctx(dflash_ctx *ctx, dflash_draft_session *s, const float *hidden_capture, int32_t n_cols,
                                const int32_t *positions_host, dflash_stream_t stream);

/* The first phases of draft_block_inner alone (metal_dflash.rs:16045-16143 and the context K/V
 * projections that follow): fc + hidden_norm and every layer's K/V for the context columns appended
 * since they were last brought up to date.  dflash_draft_block does this itself for whatever is
 * pending; calling it after a prompt's columns were appended moves that work (one pass over the
 * whole prompt) out of the first speculative step.  Enqueue-only. */
int32_t dflash_draft_prepare_ctx(dflash_ctx *ctx, const dflash_draft_head *head, dflash_draft_session *s,
                                 dflash_stream_t stream);

/* MetalDFlashDraftDecoder::draft_block / draft_block_with_logits (metal_dflash.rs:17257-17513;
 * CPU oracle Forward::dflash_draft, forward.rs:380-662): noise ids [carry, mask x (block-1)] at
 * positions noise_start_pos.., attention over ctx || noise, shared embedding and lm_head of the
 * target.  Outputs (device, may be NULL): draft_argmax[block] i32 (slot 0 unused by callers),
 * draft_logits[block][vocab].  If argmax_host is non-NULL the call waits and copies.
 * A DFlash-2 head (cfg.conv_kernel_size / cfg.selector_rank) adds the per-layer convolutions
 * (metal_dflash.rs:16210-16262, 16795-16820, 16836-16885, 17003-17022) and replaces the argmax by
 * the top-16 + selector gate + lattice walk of :17098-17130 and select_draft_path (:17176-17251):
 * draft_argmax then holds the walk's tokens. */
int32_t dflash_draft_block(dflash_ctx *ctx, const dflash_model *target, const dflash_draft_head *head,
                           dflash_draft_session *s, int32_t carry_token, int32_t mask_token, int64_t noise_start_pos,
                           int32_t *draft_argmax, float *draft_logits, int32_t *argmax_host, dflash_stream_t stream);

/* The selector inputs the last draft block of a DFlash-2 head left in the session
 * (MetalDFlashSession::topk_ids / topk_vals / sel_h, metal_dflash.rs:5150-5155), copied to the
 * caller's device buffers: [block][16] i32, [block][16] f32, [block][selector_rank] f32 (any may be
 * NULL).  Enqueue-only.  DFLASH_ERR_STATE for a DFlash-1 session. */
int32_t dflash_draft_session_selector_inputs(dflash_ctx *ctx, const dflash_draft_session *s, int32_t *topk_ids,
                                             float *topk_vals, float *sel_h, dflash_stream_t stream);

/* ---- one speculative transition -----------------------------------------------------------
 * The body of the generation loop of crates/qwen-cli/src/qwen/dflash.rs:700-1241: draft a block
 * from `carry` at `position`, verify [carry, drafts...] in one packed pass, accept a prefix,
 * append the committed hidden columns to the drafter context, roll the target KV back.
 *
 * dflash_accept_greedy: the argmax accept loop (qwen/dflash.rs:838-858) in the decision format of
 * decide_dflash_accept_prefix: accept while verify_input[i+1] == verify_argmax[i]; stop on a stop
 * id or when `remaining_output_budget` accepted tokens are reached; otherwise the carry is
 * verify_argmax[n_accepted] (a correction, or the bonus when every draft was accepted). */
int32_t dflash_accept_greedy(const int32_t *verify_input_host, const int32_t *verify_argmax_host, int32_t n_tokens,
                             int64_t remaining_output_budget, const int32_t *stop_ids_host, int32_t n_stop,
                             dflash_accept_decision *out_host);

typedef struct {
    int32_t mask_token;
    int32_t sampled_mode;           /* 0: greedy argmax accept; 1: sampler-coupled accept of the drafter's greedy
                                       tokens (couple_deterministic_proposal), logits stay on the device; 2: a
                                       DFlash-2 head drafts by the sampled selector walk (draft_block_sampled,
                                       metal_dflash.rs:17268-17415) with proposal_sampler and the target's sampler
                                       is coupled to the walk's candidate distributions (couple_sparse_proposal;
                                       qwen/dflash.rs:508-519, 706-716) */
    float fallback_margin;          /* greedy only: replay when a committed row's packed top-2 gap is below this
                                       (DFLASH_VERIFY_FALLBACK_MARGIN_DEFAULT = 0.1); <= 0 disables */
    int32_t fallback_partial;       /* 1: keep rows before the first flagged row (QWEN_DFLASH_VERIFY_FALLBACK_PARTIAL) */
    float fallback_partial_min_gap; /* a partially replayed row below this gap escalates to a whole-block replay (0.15) */
    int32_t replay_only;            /* 1: a prefix-replay step (qwen/dflash.rs:700-712): draft_override_host supplies
                                       every draft and the drafter is not run (the context columns it leaves pending
                                       are taken up by the next draft); a missing entry is DFLASH_ERR_INVALID_INPUT */
} dflash_step_cfg;

typedef struct {
    dflash_accept_decision decision; /* accepted drafts, next carry, stop reason, n_keep = retain_input_count */
    int32_t n_block;
    int32_t draft_tokens[16];        /* slot 0 = carry */
    int32_t verify_argmax[16];       /* packed argmax; rows replayed by the fallback hold the replayed argmax */
    float verify_gap[16];            /* packed top-2 gaps */
    int32_t fallback_ran, fallback_rows_replayed, fallback_escalations, fallback_rows_kept;
    double draft_ms, verify_ms, accept_ms, fallback_ms, append_ms, restore_ms; /* host wall clock per phase */
} dflash_step_result;

/* draft_override_host (may be NULL): block_size-1 token ids replacing the drafter's proposals for slots
 * 1.. (entries < 0 keep the drafter's token): the loop's prefix-replay drafts (qwen/dflash.rs:700-712).
 * sampler is required when sampled_mode != 0, proposal_sampler (temperature only, its seed the
 * target's ^ 0x4446_4c41_5348_3251 in the reference) when sampled_mode == 2, which takes no override.
 * On ANY error nothing is committed: both samplers and the session's kv_n_pos are put back to what
 * they were on entry (the drafter session's watermarks only advance after a whole block), so the
 * caller may retry the step or fall back to a plain decode step at `position`.  Blocking. */
int32_t dflash_spec_step(dflash_ctx *ctx, const dflash_model *target, const dflash_draft_head *head,
                         dflash_session *session, dflash_draft_session *draft_session,
                         const int32_t *tap_layers_host, int32_t n_taps, int32_t carry_token, int64_t position,
                         const dflash_step_cfg *cfg, dflash_sampler *sampler, dflash_sampler *proposal_sampler,
                         int64_t remaining_output_budget, const int32_t *stop_ids_host, int32_t n_stop,
                         const int32_t *draft_override_host, dflash_step_result *out_host, dflash_stream_t stream);

/* ---- adaptive speculation policy (host logic only) ------------------------------------------
 * DflashAdaptiveState, dflash_speculation_enabled, dflash_prefix_replay_*, verify_fallback_margin
 * (crates/qwen-cli/src/qwen/dflash.rs:5-376): when the loop speculates, when it takes an exact
 * single-token step instead, and when it probes again.  The thresholds are the reference's own
 * (calibrated on its hardware).  A caller's loop: prepare_mode, backoff_active / probe_due ->
 * dflash_speculation_enabled; off step: record_off_step; speculative step: begin_spec_step before,
 * record_spec_step after. */
enum { DFLASH_BACKOFF_NONE = 0, DFLASH_BACKOFF_ACCEPTANCE = 1, DFLASH_BACKOFF_FALLBACK = 2 };
#define DFLASH_OFF_CTX_DEFAULT 16384 /* hard stop of speculation past the calibrated range */

typedef struct {
    int32_t alpha_window[16];   /* accepted drafts of the last speculative steps */
    int32_t n_alpha;
    uint8_t fallback_window[8]; /* whether the exact fallback ran (long-context lane) */
    int32_t n_fallback;
    int32_t reentry_accepts[2]; /* accepted drafts of the last probes (long-context lane) */
    int32_t n_reentry;
    int32_t reason;             /* DFLASH_BACKOFF_* */
    int32_t long_mode;
    int64_t off_steps_since_probe;
} dflash_adaptive_state;

void dflash_adaptive_init(dflash_adaptive_state *s);
void dflash_adaptive_prepare_mode(dflash_adaptive_state *s, int32_t long_mode);
int32_t dflash_adaptive_backoff_active(const dflash_adaptive_state *s);
int32_t dflash_adaptive_probe_due(const dflash_adaptive_state *s, int32_t sampled_mode, int32_t long_mode);
void dflash_adaptive_record_off_step(dflash_adaptive_state *s);
void dflash_adaptive_begin_spec_step(dflash_adaptive_state *s);
void dflash_adaptive_record_spec_step(dflash_adaptive_state *s, int32_t n_accepted, int32_t fallback_ran, int32_t was_probe,
                                      int32_t reentry_eligible, int32_t sampled_mode, int32_t long_mode, int64_t position);
int32_t dflash_speculation_enabled(int32_t spec_disabled, int64_t position, int64_t off_ctx, int64_t remaining_context_tokens,
                                   int32_t block_size, int32_t backoff_active, int32_t backoff_probe_due);
int32_t dflash_prefix_replay_allowed(int32_t spec_disabled, int64_t position, int64_t off_ctx, int64_t remaining_context_tokens,
                                     int32_t block_size, int32_t long_mode, int32_t backoff_active, int32_t backoff_probe_due);
/* 1 and *drafts = history + n_emitted if emitted is a prefix of history with draft_tokens more behind it, else 0 */
int32_t dflash_prefix_replay_drafts(const int32_t *history, int64_t n_history, const int32_t *emitted, int64_t n_emitted,
                                    int64_t draft_tokens, const int32_t **drafts);
/* verify_fallback_margin (qwen/dflash.rs:126-136): 0.1, or 0.75 at positions >= DFLASH_OFF_CTX_DEFAULT */
float dflash_verify_fallback_margin(int64_t n_pos);

/* ---- GGUF reader and drafter loader (host only) -----------------------------------------------
 * GgufFile (crates/qwen-llm/src/gguf.rs:129-740, layout :1320-1480): a read-only mapping of one
 * little-endian GGUF v3 file with its metadata and tensor table validated up front: counts and
 * lengths capped (:1303-1316), keys and tensor names unique, 1..4 dimensions, no zero or oversized
 * dimension, offsets aligned to general.alignment (default 32, at most 65536), every tensor inside
 * the file, no two tensors overlapping (:840-940).  Tensor bytes are NOT copied: data_host points
 * into the mapping and stays valid until dflash_gguf_close.  A failed call leaves its message in
 * dflash_gguf_last_error (for open: in `err`).
 * Split models (GgufFile::open, gguf.rs:154-228, :954-1095): a file whose split.count exceeds 1 must be
 * shard 0 (split.no = 0), carry split.tensors.count, and be named <prefix>-00001-of-<count, 5 digits>.gguf;
 * its siblings <prefix>-0000N-of-... are opened beside it (at most 1024), each checked for its own
 * split.no, the same split.count and, when present, the same split.tensors.count.  The handle then
 * holds the first shard's metadata and the tensors of all shards in shard order; a name may appear in
 * one shard only and the merged table must hold exactly the declared number of tensors.
 * dflash_gguf_alignment / dflash_gguf_data_start describe the first shard. */
typedef struct dflash_gguf dflash_gguf;

typedef struct {
    int32_t type;          /* ggml type id; DFLASH_TYPE_* for the types the kernels take */
    int32_t n_dims;        /* after dropping trailing 1s (gguf.rs:840-846) */
    uint64_t shape[4];     /* shape[0] = the fastest dimension (a matrix is [n_in, n_out]) */
    uint64_t n_bytes;      /* 0 = tensor absent (optional members of the structs below) */
    const void *data_host;
} dflash_gguf_tensor;

int32_t dflash_gguf_open(const char *path, dflash_gguf **out, char *err, size_t err_cap); /* GgufFile::open */
void dflash_gguf_close(dflash_gguf *g);
const char *dflash_gguf_last_error(const dflash_gguf *g);
int64_t dflash_gguf_tensor_count(const dflash_gguf *g);
int64_t dflash_gguf_shard_count(const dflash_gguf *g); /* GgufFile::shard_count: 1 for a single file */
int64_t dflash_gguf_kv_count(const dflash_gguf *g);
uint64_t dflash_gguf_alignment(const dflash_gguf *g);
uint64_t dflash_gguf_data_start(const dflash_gguf *g); /* file offset of the tensor data */
/* i-th tensor in file order; *name points into the handle */
int32_t dflash_gguf_tensor_at(const dflash_gguf *g, int64_t i, const char **name, dflash_gguf_tensor *out);
/* GgufFile::find (:474): 1 = found, 0 = no such tensor */
int32_t dflash_gguf_find(const dflash_gguf *g, const char *name, dflash_gguf_tensor *out);
/* Scalar getters (:514-545, :697): 1 = present with a usable type, 0 = absent or another type.
 * get_u64 takes any integer type with a non-negative value; get_f64 takes f32 / f64. */
int32_t dflash_gguf_get_u64(const dflash_gguf *g, const char *key, uint64_t *out);
int32_t dflash_gguf_get_f64(const dflash_gguf *g, const char *key, double *out);
int32_t dflash_gguf_get_bool(const dflash_gguf *g, const char *key, int32_t *out);
int32_t dflash_gguf_get_str(const dflash_gguf *g, const char *key, const char **out, uint64_t *len); /* not 0-terminated */
/* Array getters (:546-696): the array's length, or -1 if the key is absent, or -2 if it is not an
 * array of that kind (u64: any integer type, no negative element; bool; f64: f32 / f64); up to
 * `cap` elements are written to out (which may be NULL with cap 0). */
int64_t dflash_gguf_get_u64_array(const dflash_gguf *g, const char *key, uint64_t *out, int64_t cap);
int64_t dflash_gguf_get_bool_array(const dflash_gguf *g, const char *key, uint8_t *out, int64_t cap);
int64_t dflash_gguf_get_f64_array(const dflash_gguf *g, const char *key, double *out, int64_t cap);

/* open_dflash_drafter_for_target (crates/qwen-llm/src/loader.rs:832-1290): reads a drafter file of
 * either convention (arch "dflash-draft": keys dflash-draft.*, tensors dflash_fc / dflash_hidden_norm
 * / blk.N.post_attention_norm; arch "dflash": keys dflash.*, tensors fc / enc.output_norm /
 * blk.N.ffn_norm, target layers stored as layer-input indices and turned into post-block ids by
 * subtracting 1, :1010-1023), validates it against the target (hidden sizes equal, mask token inside
 * the vocabulary, tapped layers inside the target, n_target_features == taps * hidden, pattern length
 * == block_count, sliding-window layers need a window) and binds every tensor with its shape checked.
 * selector_hidden.weight present = DFlash-2: the four conv / selector keys and all conv and selector
 * tensors become mandatory (:1029-1056).  Norms and conv bases must be F32. */
typedef struct {
    uint32_t hidden_size, vocab_size, n_layer; /* DFlashTargetShape (loader.rs:849-856) */
} dflash_target_shape;

typedef struct {
    dflash_gguf_tensor attn_norm, wq, wk, wv, wo, q_norm, k_norm, post_norm, gate, up, down;
    dflash_gguf_tensor conv_attn_base, conv_attn_proj, conv_ffn_base, conv_ffn_proj; /* DFlash-2 only */
    int32_t is_swa, pad;
} dflash_gguf_draft_layer;

enum { DFLASH_GGUF_MAX_TAPS = 64 };
typedef struct {
    dflash_draft_cfg cfg;
    int32_t mask_token_id;
    int32_t convention;       /* 1 = "dflash-draft", 2 = "dflash" */
    int32_t n_target_layers;  /* == cfg.n_taps */
    int32_t target_layer_ids[DFLASH_GGUF_MAX_TAPS]; /* post-block layer ids of the target */
    dflash_gguf_tensor fc, hidden_norm, output_norm;
    dflash_gguf_tensor selector_hidden, selector_predecessor, selector_successor; /* DFlash-2 only */
} dflash_gguf_draft_head;

/* layers: caller's array of layer_cap entries; cfg.n_layers of them are filled. */
int32_t dflash_gguf_open_drafter(dflash_gguf *g, const dflash_target_shape *target, dflash_gguf_draft_head *out,
                                 dflash_gguf_draft_layer *layers, int32_t layer_cap);

/* =====================================================================================================
 * MEASUREMENT AID - not part of the drop-in surface.  No reference seam corresponds to it and no caller of the
 * engine needs them; bench.py uses it to find the ceiling of a read-only stream.  An integration can leave it unbound.
 * ===================================================================================================== */
/* Streaming-read probe: n_launches launches of a kernel that reads `bytes` (multiple of 16) of
 * bufs[k % n_bufs] (16-byte aligned) once with a grid-stride loop of 16-byte loads and stores a word per
 * workgroup into out_words[n_cu].  bench.py times it over the GEMM's own weight buffers (rotating, so that
 * nothing is found in a cache) as the practical ceiling of a read-only stream.  Enqueue-only. */
int32_t dflash_hbm_read_probe(dflash_ctx *ctx, const void *const *bufs, int32_t n_bufs, size_t bytes, int32_t n_launches,
                              void *out_words, dflash_stream_t stream);


#ifdef __cplusplus
}
#endif
#endif
