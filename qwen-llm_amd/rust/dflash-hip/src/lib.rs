//! The reference engine's `DFlashDecoder` surface (crates/qwen-llm/src/metal_dflash.rs:8328-8555, 15915-15925,
//! 17257-17415, 17519-17527) on top of `libdflash_hip.so`.
//!
//! What maps to what:
//!   MetalForward (target weights + device)        -> HipForward   { ctx, model }
//!   MetalDFlashHead (drafter weights, tap layers)   -> HipDFlashHead { head, target_layer_ids }
//!   MetalSession (target KV cache, kv_n_pos)        -> HipSession   (owns a dflash_session)
//!   MetalDFlashSession (drafter context + scratch)  -> HipDFlashSession (owns a dflash_draft_session)
//!   MetalDFlashVerifyScratch / LayerMajorScratch    -> HipVerifyScratch (device outputs of one block; the library
//!                                                      keeps its own layer-major scratch inside the session)
//!   DFlashError                                     -> DFlashError below, from the status codes
//! The methods keep the reference's names, argument order and error behaviour (guard walls before any launch,
//! nothing committed on error).  Everything is `unsafe` FFI underneath; this file is the only place that is.
//!
//! Shipped as source: the build image of this repository has no Rust toolchain, so the crate is checked against
//! the C header (every name it takes from the sys crate must be exported) but not compiled there.

use dflash_hip_sys as sys;
use std::ffi::{c_void, CStr};
use std::ptr;

/// `DFlashError` of the reference (metal_dflash.rs) as far as this path raises it, plus the sampling errors of
/// `DFlashAcceptError::Sampling { row, source }` (sampling.rs).
#[derive(Debug, Clone, PartialEq)]
pub enum DFlashError {
    /// MetalError::BadShape and the dimension guards at the top of packed verify
    BadShape(String),
    /// "decline": no kernel for this dtype / size; the caller keeps its incumbent path
    Declined(String),
    /// DFlashAcceptError::InvalidInput
    InvalidInput(String),
    /// DFlashAcceptError::InvalidToken / ForwardError::BadToken
    InvalidToken(String),
    /// DFlashAcceptError::ProposalMismatch
    ProposalMismatch(String),
    /// kv_n_pos != start_position, restore not directly after its verify, capacity walls
    State(String),
    /// DFlashError::BadDrafter
    BadDrafter(&'static str),
    /// DFlashAcceptError::Sampling { row, source }: `source` in the order of SamplingError
    Sampling { row: i32, source: i32, detail: String },
    /// workspace, alignment, aliasing, HIP runtime
    Device { status: i32, detail: String },
}

fn last_error(ctx: *const sys::dflash_ctx) -> String {
    unsafe {
        let p = sys::dflash_last_error(ctx);
        if p.is_null() { String::new() } else { CStr::from_ptr(p).to_string_lossy().into_owned() }
    }
}

/// Status code -> `DFlashError` (the table of the integration notes: 1 BadShape, 2 declined, 7 InvalidInput,
/// 8 InvalidToken, 9 ProposalMismatch, 10 State, 33.. Sampling with source = code - 32).
fn check(ctx: *const sys::dflash_ctx, rc: i32, err_row: i32) -> Result<(), DFlashError> {
    let detail = || last_error(ctx);
    match rc {
        0 => Ok(()),
        1 => Err(DFlashError::BadShape(detail())),
        2 => Err(DFlashError::Declined(detail())),
        7 => Err(DFlashError::InvalidInput(detail())),
        8 => Err(DFlashError::InvalidToken(detail())),
        9 => Err(DFlashError::ProposalMismatch(detail())),
        10 => Err(DFlashError::State(detail())),
        33..=42 => Err(DFlashError::Sampling { row: err_row, source: rc - 32, detail: detail() }),
        _ => Err(DFlashError::Device { status: rc, detail: detail() }),
    }
}

/// Device context + the bound target model (`MetalForward`).  `model` points at tensors the loader uploaded
/// (Q4_K matrices repacked with `dflash_repack_q4k_tiled`, every quantised tensor passed through
/// `dflash_check_scale_range`); it must outlive every decoder built on it.
pub struct HipForward {
    pub ctx: *mut sys::dflash_ctx,
    pub model: sys::dflash_model,
    pub stream: *mut c_void,
}

impl HipForward {
    pub fn new(device: i32, workspace_bytes: usize, model: sys::dflash_model) -> Result<Self, DFlashError> {
        let mut ctx = ptr::null_mut();
        let rc = unsafe { sys::dflash_ctx_create(device, workspace_bytes, &mut ctx) };
        if rc != 0 {
            return Err(DFlashError::Device { status: rc, detail: "dflash_ctx_create".into() });
        }
        Ok(Self { ctx, model, stream: ptr::null_mut() })
    }
}

impl Drop for HipForward {
    fn drop(&mut self) {
        unsafe { sys::dflash_ctx_destroy(self.ctx) }
    }
}

/// `MetalDFlashHead`: the drafter's tensors and the target layers whose hidden states it taps.
pub struct HipDFlashHead {
    pub head: sys::dflash_draft_head,
    pub target_layer_ids: Vec<i32>,
    pub mask_token: i32,
}

/// `MetalSession`: the target's f16 KV cache and `kv_n_pos`.
pub struct HipSession {
    raw: *mut sys::dflash_session,
}

impl HipSession {
    pub fn new(base: &HipForward, kv_capacity: i64, n_taps: i32) -> Result<Self, DFlashError> {
        let mut raw = ptr::null_mut();
        let rc = unsafe { sys::dflash_session_create(base.ctx, &base.model.cfg, kv_capacity, n_taps, &mut raw) };
        check(base.ctx, rc, -1)?;
        Ok(Self { raw })
    }
    pub fn kv_n_pos(&self) -> i64 {
        unsafe { sys::dflash_session_kv_n_pos(self.raw) }
    }
}

impl Drop for HipSession {
    fn drop(&mut self) {
        unsafe { sys::dflash_session_destroy(self.raw) }
    }
}

/// `MetalDFlashSession`: the drafter's accumulated context columns and their per-layer K/V.
pub struct HipDFlashSession {
    raw: *mut sys::dflash_draft_session,
}

impl HipDFlashSession {
    pub fn new(base: &HipForward, head: &HipDFlashHead, ctx_capacity: i64) -> Result<Self, DFlashError> {
        let mut raw = ptr::null_mut();
        let rc = unsafe {
            sys::dflash_draft_session_create(base.ctx, &head.head.cfg, ctx_capacity, base.model.cfg.vocab as i64, &mut raw)
        };
        check(base.ctx, rc, -1)?;
        Ok(Self { raw })
    }
    pub fn ctx_len(&self) -> i64 {
        unsafe { sys::dflash_draft_session_ctx_len(self.raw) }
    }
}

impl Drop for HipDFlashSession {
    fn drop(&mut self) {
        unsafe { sys::dflash_draft_session_destroy(self.raw) }
    }
}

/// Device outputs of one packed verify (`MetalDFlashVerifyScratch`: verify_argmax, the captured hidden rows;
/// `MetalDFlashDebugScratch` adds the logits).  The caller allocates them with its device allocator:
/// argmax [block] i32, gap [block] f32, hidden_capture [block][n_taps][hidden] f32, logits [block][vocab] f32 or null.
pub struct HipVerifyScratch {
    pub argmax: *mut i32,
    pub gap: *mut f32,
    pub hidden_capture: *mut f32,
    pub debug_logits: *mut f32,
    pub block_size: usize,
    pub n_taps: usize,
}

/// `DFlash2SparseProposalBlock` (metal_dflash.rs:17268-17415): the sampled walk's tokens and, per position, the
/// candidates it was drawn from.
pub struct DFlash2SparseProposalBlock {
    pub tokens: Vec<i32>,
    pub candidates: Vec<Vec<(i32, f64)>>,
}

pub struct DFlashDecoder<'a> {
    pub base: &'a HipForward,
    pub head: &'a HipDFlashHead,
    pub session: HipDFlashSession,
}

impl<'a> DFlashDecoder<'a> {
    /// metal_dflash.rs:8337-8349
    pub fn new(base: &'a HipForward, head: &'a HipDFlashHead, session: HipDFlashSession) -> Self {
        Self { base, head, session }
    }

    fn verify_inner(&self, tokens: &[i32], start_position: u32, scratch: &mut HipVerifyScratch, logits: *mut f32,
                    target_session: &mut HipSession) -> Result<Vec<i32>, DFlashError> {
        // the reference's entry guard (metal_dflash.rs:8367-8376): a scratch sized for another block / tap set
        if tokens.is_empty() || tokens.len() > scratch.block_size || scratch.n_taps != self.head.target_layer_ids.len() {
            return Err(DFlashError::BadShape(format!(
                "packed_verify: {} tokens / {} taps against a scratch of {} / {}",
                tokens.len(), self.head.target_layer_ids.len(), scratch.block_size, scratch.n_taps)));
        }
        let mut host = vec![0i32; tokens.len()];
        let rc = unsafe {
            sys::dflash_verify_block(self.base.ctx, &self.base.model, target_session.raw, tokens.as_ptr(), tokens.len() as i32,
                                     start_position as i64, self.head.target_layer_ids.as_ptr(),
                                     self.head.target_layer_ids.len() as i32, scratch.argmax, scratch.gap,
                                     scratch.hidden_capture, logits, host.as_mut_ptr(), self.base.stream)
        };
        check(self.base.ctx, rc, -1)?;
        Ok(host)
    }

    /// Default packed verify, layer-major (metal_dflash.rs:8397-8419): forwards `tokens` at
    /// `start_position..`, appends their K/V, captures the tapped hidden rows, returns the argmax per row.
    pub fn packed_verify(&self, tokens: &[i32], start_position: u32, verify_scratch: &mut HipVerifyScratch,
                         target_session: &mut HipSession) -> Result<Vec<i32>, DFlashError> {
        self.verify_inner(tokens, start_position, verify_scratch, ptr::null_mut(), target_session)
    }

    /// metal_dflash.rs:8427-8455: the same with the [n][vocab] logits kept (sampled acceptance reads them on the device).
    pub fn packed_verify_with_logits(&self, tokens: &[i32], start_position: u32, dbg_scratch: &mut HipVerifyScratch,
                                     target_session: &mut HipSession) -> Result<Vec<i32>, DFlashError> {
        if dbg_scratch.debug_logits.is_null() {
            return Err(DFlashError::BadShape("packed_verify_with_logits: scratch has no logits buffer".into()));
        }
        let logits = dbg_scratch.debug_logits;
        self.verify_inner(tokens, start_position, dbg_scratch, logits, target_session)
    }

    /// metal_dflash.rs:8539-8555.  `n_keep` = tokens of the verified block to retain (the carry + accepted drafts),
    /// not "accepted drafts"; must directly follow the matching verify of `n_block` tokens at `start_position`.
    pub fn restore_after_partial_accept(&self, n_block: u32, n_keep: u32, start_position: u32,
                                        target_session: &mut HipSession) -> Result<(), DFlashError> {
        let rc = unsafe { sys::dflash_restore(self.base.ctx, target_session.raw, start_position as i64, n_block as i32, n_keep as i32) };
        check(self.base.ctx, rc, -1)
    }

    /// Appends the hidden rows a verify captured for the committed positions to the drafter's context
    /// (the reference does this inside its session update after acceptance, qwen/dflash.rs:880-905).
    pub fn append_context(&mut self, hidden_capture: *const f32, positions: &[i32]) -> Result<(), DFlashError> {
        let rc = unsafe {
            sys::dflash_draft_append_ctx(self.base.ctx, self.session.raw, hidden_capture, positions.len() as i32,
                                         positions.as_ptr(), self.base.stream)
        };
        check(self.base.ctx, rc, -1)
    }

    /// The drafter's pass over pending context columns as part of the prefill (otherwise the next draft does it).
    pub fn prepare_context(&mut self) -> Result<(), DFlashError> {
        let rc = unsafe { sys::dflash_draft_prepare_ctx(self.base.ctx, &self.head.head, self.session.raw, self.base.stream) };
        check(self.base.ctx, rc, -1)
    }

    /// metal_dflash.rs:15915-15925, 17257-17263: one parallel draft of a block; slot 0 is the carry.
    pub fn draft_block(&mut self, carry_tok: i32, noise_start_pos: u32) -> Result<Vec<i32>, DFlashError> {
        let block = self.head.head.cfg.block_size as usize;
        let mut host = vec![0i32; block];
        let rc = unsafe {
            sys::dflash_draft_block(self.base.ctx, &self.base.model, &self.head.head, self.session.raw, carry_tok,
                                    self.head.mask_token, noise_start_pos as i64, ptr::null_mut(), ptr::null_mut(),
                                    host.as_mut_ptr(), self.base.stream)
        };
        check(self.base.ctx, rc, -1)?;
        Ok(host)
    }

    /// metal_dflash.rs:17268-17415, 17519-17527: DFlash-2 sampled selector walk.  The proposal sampler must apply
    /// positive temperature only (checked by the library, as by the reference).  `scratch_*` are device buffers of
    /// [block][16] i32, [block][16] f32 and [block][rank] f32 for the selector's inputs.
    pub fn draft_block_sampled(&mut self, carry_tok: i32, noise_start_pos: u32, proposal_sampler: &mut sys::dflash_sampler,
                               scratch_ids: *mut i32, scratch_vals: *mut f32, scratch_h: *mut f32)
                               -> Result<DFlash2SparseProposalBlock, DFlashError> {
        let cfg = &self.head.head.cfg;
        if cfg.selector_rank == 0 {
            return Err(DFlashError::BadDrafter("sampled path requires a DFlash 2 selector"));
        }
        let block = cfg.block_size as usize;
        let top_k = cfg.selector_top_k as usize;
        self.draft_block(carry_tok, noise_start_pos)?;
        let rc = unsafe {
            sys::dflash_draft_session_selector_inputs(self.base.ctx, self.session.raw, scratch_ids, scratch_vals, scratch_h,
                                                      self.base.stream)
        };
        check(self.base.ctx, rc, -1)?;
        let mut tokens = vec![0i32; block];
        let mut counts = vec![0i32; block - 1];
        let mut cands = vec![sys::dflash_weighted_candidate { token: 0, pad: 0, weight: 0.0 }; (block - 1) * top_k];
        let rc = unsafe {
            sys::dflash_select_draft_path_sampled(self.base.ctx, &self.head.head.selector_predecessor,
                                                  &self.head.head.selector_successor, cfg.selector_rank, cfg.selector_top_k,
                                                  carry_tok, block as i32, scratch_ids, scratch_vals, scratch_h,
                                                  proposal_sampler, tokens.as_mut_ptr(), counts.as_mut_ptr(),
                                                  cands.as_mut_ptr(), self.base.stream)
        };
        check(self.base.ctx, rc, -1)?;
        let candidates = (0..block - 1)
            .map(|p| cands[p * top_k..p * top_k + counts[p] as usize].iter().map(|c| (c.token, c.weight)).collect())
            .collect();
        Ok(DFlash2SparseProposalBlock { tokens, candidates })
    }

    /// One whole transition of the loop (qwen/dflash.rs:640-905: draft, packed verify, acceptance, margin fallback,
    /// KV rollback, context append) in one call.  On `Err` nothing is committed: samplers and kv_n_pos are back at
    /// their entry values.
    #[allow(clippy::too_many_arguments)]
    pub fn spec_step(&mut self, target_session: &mut HipSession, carry_token: i32, position: i64, cfg: &sys::dflash_step_cfg,
                     sampler: Option<&mut sys::dflash_sampler>, proposal_sampler: Option<&mut sys::dflash_sampler>,
                     remaining_output_budget: i64, stop_ids: &[i32], draft_override: Option<&[i32]>)
                     -> Result<sys::dflash_step_result, DFlashError> {
        let mut out: sys::dflash_step_result = unsafe { std::mem::zeroed() };
        let rc = unsafe {
            sys::dflash_spec_step(self.base.ctx, &self.base.model, &self.head.head, target_session.raw, self.session.raw,
                                  self.head.target_layer_ids.as_ptr(), self.head.target_layer_ids.len() as i32, carry_token,
                                  position, cfg, sampler.map_or(ptr::null_mut(), |s| s as *mut _),
                                  proposal_sampler.map_or(ptr::null_mut(), |s| s as *mut _), remaining_output_budget,
                                  stop_ids.as_ptr(), stop_ids.len() as i32,
                                  draft_override.map_or(ptr::null(), |d| d.as_ptr()), &mut out, self.base.stream)
        };
        check(self.base.ctx, rc, out.decision.err_row)?;
        Ok(out)
    }
}

/// metal_forward/dispatch.rs:365-378: the verifier's few-row mat-mat seam.  `Declined` keeps the caller on its
/// incumbent kernel, as the Metal route selection does.
#[allow(clippy::too_many_arguments)]
/// `weight_type`: the ggml tag of a tensor nobody checked (any block is computed correctly, by the f32 kernel), or
/// `tag | DFLASH_TYPE_RANGE_CHECKED` / `DFLASH_TYPE_Q4_K_TILED` for one `prepare_weight` accepted (the fast kernels).
pub fn encode_mat_mat_dispatch_dflash_verify(base: &HipForward, weight_type: i32, weight: *const c_void, x: *const c_void,
                                             x_type: i32, y: *mut f32, n_in: usize, n_out: usize, n_query: u32)
                                             -> Result<(), DFlashError> {
    let rc = unsafe {
        sys::dflash_gemm_fewrow(base.ctx, weight_type, weight, x, x_type, y, n_in as i64, n_out as i64, n_query as i32, base.stream)
    };
    check(base.ctx, rc, -1)
}

/// Loader step for one quantised tensor already in device memory: range guard, then (Q4_K matrices the few-row GEMM
/// alone reads) the one-time repack into tiled order.  Returns the descriptor to store in the model: the type tag and,
/// for a Q4_K / Q6_K tensor that passed the guard, `flags = DFLASH_QT_RANGE_CHECKED`, without which the model-level
/// calls decline the model and `dflash_gemm_fewrow` takes its slow f32 kernel.
pub fn prepare_weight(base: &HipForward, type_: i32, blocks: *const c_void, n_blocks: usize, tiled_dst: Option<*mut c_void>,
                      n_in: i64, n_out: i64) -> Result<sys::dflash_qtensor, DFlashError> {
    let rc = unsafe { sys::dflash_check_scale_range(base.ctx, type_, blocks, n_blocks, ptr::null_mut(), base.stream) };
    check(base.ctx, rc, -1)?;
    let flags = if type_ == 12 || type_ == 14 { sys::DFLASH_QT_RANGE_CHECKED } else { 0 };
    if let (12, Some(dst)) = (type_, tiled_dst) {
        debug_assert!(unsafe { sys::dflash_q4k_tiled_bytes(n_in, n_out) } > 0);
        let rc = unsafe { sys::dflash_repack_q4k_tiled(base.ctx, blocks, dst, n_in, n_out, base.stream) };
        check(base.ctx, rc, -1)?;
        return Ok(sys::dflash_qtensor { type_: sys::DFLASH_TYPE_Q4_K_TILED, flags, data: dst as *const c_void });
    }
    Ok(sys::dflash_qtensor { type_, flags, data: blocks })
}
