"""ctypes binding of libdflash_hip.so and a thin object layer over it.

The argument lists follow ``include/dflash_hip.h`` one to one.  Tensors are torch
device tensors; their ``data_ptr()`` is what crosses the C ABI.
"""
from __future__ import annotations

import ctypes as C
import os
import re

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(PKG_DIR, "libdflash_hip.so")
HEADER_PATH = os.path.join(PKG_DIR, "..", "include", "dflash_hip.h")

TYPE_F32, TYPE_F16, TYPE_Q8_0, TYPE_Q4_K, TYPE_Q6_K = 0, 1, 8, 12, 14
TYPE_Q4_K_TILED = 1012  # Q4_K blocks in the library's tiled order (Context.repack_q4k_tiled)
TYPE_Q6_K_TILED = 1014  # Q6_K blocks in the library's tiled, field-planar order (Context.repack_q6k_tiled): gemm_fewrow_xf only
XF_NONE, XF_Q4K, XF_Q6K = 0, 1, 2  # fragment orders of Context.pack_xf
TYPE_RANGE_CHECKED = 0x10000  # OR-ed into a w_type: the tensor passed Context.check_scale_range (fast Q4_K / Q6_K kernels)
QT_RANGE_CHECKED = 1  # the same fact in a dflash_qtensor's flags

STATUS = {
    0: "Ok", 1: "BadShape", 2: "Unsupported", 3: "Alias", 4: "Alignment", 5: "Workspace", 6: "Hip",
    7: "InvalidInput", 8: "InvalidToken", 9: "ProposalMismatch", 10: "State", 11: "Io", 12: "Format", 13: "Metadata", 33: "EmptyLogits",
    34: "InvalidTemperature", 35: "InvalidTopP", 36: "InvalidMinP", 37: "NanLogit", 38: "VocabularyTooLarge",
    39: "NoCandidates", 40: "ProposalTokenOutOfRange", 41: "InvalidProposalWeight", 42: "MissingProposalToken",
}


class DFlashError(RuntimeError):
    """A non-zero status from the library (the reference's Result::Err)."""

    def __init__(self, status: int, message: str):
        super().__init__(f"{STATUS.get(status, status)}: {message}")
        self.status = status
        self.kind = STATUS.get(status, str(status))
        self.message = message


class SamplingConfigC(C.Structure):
    _fields_ = [("temperature", C.c_float), ("top_p", C.c_float), ("min_p", C.c_float), ("rng_kind", C.c_int32),
                ("top_k", C.c_uint64), ("seed", C.c_uint64)]


class SamplerC(C.Structure):
    _fields_ = [("cfg", SamplingConfigC), ("s", C.c_uint64 * 4), ("draws", C.c_uint64)]


class WeightedCandidateC(C.Structure):
    _fields_ = [("token", C.c_int32), ("pad", C.c_int32), ("weight", C.c_double)]


class CodebookC(C.Structure):
    _fields_ = [("type", C.c_int32), ("pad", C.c_int32), ("n_rows", C.c_int64), ("data", C.c_void_p)]


class AcceptDecisionC(C.Structure):
    _fields_ = [("n_accepted", C.c_int32), ("accepted_drafts", C.c_int32 * 16), ("carry_kind", C.c_int32),
                ("carry_token", C.c_int32), ("stop_reason", C.c_int32), ("retain_input_count", C.c_int32),
                ("draws_used", C.c_int32), ("err_row", C.c_int32), ("err_code", C.c_int32), ("err_index", C.c_int64)]


RNG_XOSHIRO, RNG_PHILOX = 0, 1
CARRY_NONE, CARRY_CORRECTION, CARRY_BONUS = 0, 1, 2
STOP_NONE, STOP_EOS, STOP_TOKEN_LIMIT = 0, 1, 2


def declared_symbols() -> list[str]:
    """Every function name the public header declares."""
    text = open(HEADER_PATH).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(dflash_[a-z0-9_]+)\s*\(", text)))


_lib = None


def lib() -> C.CDLL:
    """Load the HIP library; raises if it has not been built (no fallback exists)."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(f"{LIB_PATH} is missing: run __graft_entry__.build() (hipcc, gfx950) first")
        _lib = C.CDLL(LIB_PATH)
        _declare(_lib)
    return _lib


def _declare(L):
    vp, sz, i32, i64, f32 = C.c_void_p, C.c_size_t, C.c_int32, C.c_int64, C.c_float
    L.dflash_ctx_create.restype = i32
    L.dflash_ctx_create.argtypes = [i32, sz, C.POINTER(vp)]
    L.dflash_ctx_destroy.restype = None
    L.dflash_ctx_destroy.argtypes = [vp]
    L.dflash_last_error.restype = C.c_char_p
    L.dflash_last_error.argtypes = [vp]
    L.dflash_status_name.restype = C.c_char_p
    L.dflash_status_name.argtypes = [i32]
    L.dflash_version.restype = C.c_char_p
    L.dflash_ctx_set_kernel_timing.restype = None
    L.dflash_ctx_set_kernel_timing.argtypes = [vp, i32]
    L.dflash_dflash2_conv.restype = i32
    L.dflash_dflash2_conv.argtypes = [vp, vp, vp, vp, vp, i32, i32, i32, i32, i32, vp]
    L.dflash_select_draft_path.restype = i32
    L.dflash_select_draft_path.argtypes = [vp, C.POINTER(CodebookC), C.POINTER(CodebookC), i32, i32, i32, i32, vp, vp, vp,
                                           vp, vp, vp]
    L.dflash_select_draft_path_sampled.restype = i32
    L.dflash_select_draft_path_sampled.argtypes = [vp, C.POINTER(CodebookC), C.POINTER(CodebookC), i32, i32, i32, i32, vp, vp,
                                                   vp, C.POINTER(SamplerC), vp, vp, C.POINTER(WeightedCandidateC), vp]
    L.dflash_ctx_set_draft_graphs.restype = None
    L.dflash_ctx_set_draft_graphs.argtypes = [vp, i32]
    L.dflash_ctx_set_graphs.restype = None
    L.dflash_ctx_set_graphs.argtypes = [vp, i32]
    L.dflash_ctx_kernel_timing.restype = i32
    L.dflash_ctx_kernel_timing.argtypes = [vp, i32, C.POINTER(C.c_double), C.POINTER(i64)]
    L.dflash_row_bytes.restype = sz
    L.dflash_row_bytes.argtypes = [i32, sz]
    L.dflash_dequant.restype = i32
    L.dflash_dequant.argtypes = [vp, i32, vp, sz, vp, vp]
    L.dflash_gemm_fewrow.restype = i32
    L.dflash_gemm_fewrow.argtypes = [vp, i32, vp, vp, i32, vp, i64, i64, i32, vp]
    L.dflash_check_scale_range.restype = i32
    L.dflash_check_scale_range.argtypes = [vp, i32, vp, sz, C.POINTER(f32), vp]
    L.dflash_hbm_read_probe.restype = i32
    L.dflash_hbm_read_probe.argtypes = [vp, C.POINTER(vp), i32, sz, i32, vp, vp]
    L.dflash_q4k_tiled_bytes.restype = sz
    L.dflash_q4k_tiled_bytes.argtypes = [i64, i64]
    L.dflash_repack_q4k_tiled.restype = i32
    L.dflash_repack_q4k_tiled.argtypes = [vp, vp, vp, i64, i64, vp]
    L.dflash_q6k_tiled_bytes.restype = sz
    L.dflash_q6k_tiled_bytes.argtypes = [i64, i64]
    L.dflash_repack_q6k_tiled.restype = i32
    L.dflash_repack_q6k_tiled.argtypes = [vp, vp, vp, i64, i64, vp]
    L.dflash_xf_bytes.restype = sz
    L.dflash_xf_bytes.argtypes = [i64]
    L.dflash_gemm_fewrow_xf_kind.restype = i32
    L.dflash_gemm_fewrow_xf_kind.argtypes = [vp, i32, i64, i64]
    L.dflash_pack_xf.restype = i32
    L.dflash_pack_xf.argtypes = [vp, vp, i32, i32, i64, i32, vp, vp]
    L.dflash_gemm_fewrow_xf.restype = i32
    L.dflash_gemm_fewrow_xf.argtypes = [vp, i32, vp, vp, vp, i64, i64, i32, vp]
    L.dflash_gemm_fewrow_noalloc.restype = i32
    L.dflash_gemm_fewrow_noalloc.argtypes = [i32, vp, vp, i32, vp, i64, i64, i32, vp]
    L.dflash_gemm_fewrow_noalloc_error.restype = C.c_char_p
    L.dflash_gemm_fewrow_noalloc_error.argtypes = []
    for name in ("dflash_argmax_top2", "dflash_top16"):
        getattr(L, name).restype = i32
        getattr(L, name).argtypes = [vp, vp, i32, i64, i64, vp, vp, vp]
    L.dflash_argmax_greedy.restype = i32
    L.dflash_argmax_greedy.argtypes = [vp, vp, i32, i64, i64, vp, vp]
    L.dflash_sampler_init.restype = i32
    L.dflash_sampler_init.argtypes = [C.POINTER(SamplerC), C.POINTER(SamplingConfigC)]
    L.dflash_sampler_at_draw.restype = i32
    L.dflash_sampler_at_draw.argtypes = [C.POINTER(SamplerC), C.POINTER(SamplingConfigC), C.c_uint64]
    L.dflash_sampler_peek.restype = None
    L.dflash_sampler_peek.argtypes = [C.POINTER(SamplerC), i32, C.POINTER(C.c_double)]
    L.dflash_sampler_advance.restype = None
    L.dflash_sampler_advance.argtypes = [C.POINTER(SamplerC), C.c_uint64]
    L.dflash_accept_prefix.restype = i32
    L.dflash_accept_prefix.argtypes = [vp, C.POINTER(i32), i32, vp, i64, i32, i32, C.POINTER(i32), C.POINTER(i32),
                                       C.POINTER(WeightedCandidateC), vp, f32, C.POINTER(SamplerC), i64,
                                       C.POINTER(i32), i32, C.POINTER(AcceptDecisionC), vp]
    L.dflash_attn_verify_block.restype = i32
    L.dflash_attn_verify_block.argtypes = [vp, vp, i32, vp, vp, i32, i64, i32, i32, i32, i32, i64, f32, vp, vp]


class Sampler:
    """Request-local sampler state (sampling.rs:304-366): config + random stream + draw count."""

    def __init__(self, temperature=0.0, top_k=0, top_p=1.0, min_p=0.0, seed=0, rng_kind=RNG_XOSHIRO, draws=0):
        self.c = SamplerC()
        cfg = SamplingConfigC(temperature, top_p, min_p, rng_kind, top_k, seed)
        rc = lib().dflash_sampler_at_draw(C.byref(self.c), C.byref(cfg), draws)
        if rc:
            raise DFlashError(rc, "invalid sampling configuration")

    @classmethod
    def at_draw(cls, other: "Sampler", draws: int) -> "Sampler":
        c = other.c.cfg
        return cls(c.temperature, c.top_k, c.top_p, c.min_p, c.seed, c.rng_kind, draws)

    def clone(self) -> "Sampler":
        t = Sampler.__new__(Sampler)
        t.c = SamplerC()
        C.memmove(C.byref(t.c), C.byref(self.c), C.sizeof(SamplerC))
        return t

    @property
    def draws(self) -> int:
        return int(self.c.draws)

    def state(self):
        return (tuple(self.c.s), int(self.c.draws))

    def peek(self, n: int):
        out = (C.c_double * n)()
        lib().dflash_sampler_peek(C.byref(self.c), n, out)
        return list(out)


class AcceptDecision:
    """DFlashAcceptDecision (metal_dflash/accept.rs:17-32)."""

    def __init__(self, c: AcceptDecisionC):
        self.accepted_drafts = list(c.accepted_drafts[: c.n_accepted])
        self.carry_kind = c.carry_kind
        self.carry_token = c.carry_token if c.carry_kind else 0
        self.stop_reason = c.stop_reason
        self.retain_input_count = c.retain_input_count
        self.draws_used = c.draws_used
        self.err_row, self.err_code, self.err_index = c.err_row, c.err_code, c.err_index

    def key(self):
        return (self.accepted_drafts, self.carry_kind, self.carry_token, self.stop_reason, self.retain_input_count)


def _torch():
    import torch

    return torch


def _empty(*args, **kwargs):
    """Every output tensor the host mirror allocates comes from here (tests swap it for an allocator that puts guard
    bands around the tensor)."""
    return _torch().empty(*args, **kwargs)


def _stream_ptr():
    torch = _torch()
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)


class Context:
    """Owns a ``dflash_ctx`` (device workspace + error slot) for one GPU."""

    def __init__(self, device: int = 0, workspace_bytes: int = 0):
        torch = _torch()
        if not torch.cuda.is_available():
            raise RuntimeError("no GPU visible: the DFlash step has no CPU fallback")
        self._lib = lib()
        self.device = device
        h = C.c_void_p()
        rc = self._lib.dflash_ctx_create(device, workspace_bytes, C.byref(h))
        if rc:
            raise DFlashError(rc, "dflash_ctx_create failed")
        self._h = h

    def close(self):
        if getattr(self, "_h", None):
            self._lib.dflash_ctx_destroy(self._h)
            self._h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def _check(self, rc: int):
        if rc:
            raise DFlashError(rc, self._lib.dflash_last_error(self._h).decode())

    # ---- enable_phase_timers (metal_dflash.rs:5181-5190)
    T_GEMM, T_ATTN, T_ACCEPT, T_ARGMAX, T_REDUCE = 0, 1, 2, 3, 4

    def set_kernel_timing(self, enable):
        """False / 0: off; True / 1: event pairs around the dominant kernels (each timed launch waits); 2: dispatch stamps
        of the Q4_K streaming kernel and its reduction (slots 5 and 6), read when kernel_timing() is called."""
        self._lib.dflash_ctx_set_kernel_timing(self._h, int(enable))

    def set_draft_graphs(self, enable: bool):
        """Graph replay of the drafter's block forward on or off (off by default; results are the same)."""
        self._lib.dflash_ctx_set_draft_graphs(self._h, int(enable))

    def set_graphs(self, enable: bool):
        """Graph replay of the packed verify on or off (off by default; results are the same)."""
        self._lib.dflash_ctx_set_graphs(self._h, int(enable))

    def kernel_timing(self, slot: int):
        ms, n = C.c_double(), C.c_int64()
        self._check(self._lib.dflash_ctx_kernel_timing(self._h, slot, C.byref(ms), C.byref(n)))
        return ms.value, n.value

    # ---- codec::dequant_to_f32 (codec.rs:256-302)
    def dequant_to_f32(self, qtype: int, blocks, n_elems: int, out=None):
        torch = _torch()
        if out is None:
            out = _empty(n_elems, dtype=torch.float32, device=blocks.device)
        self._check(self._lib.dflash_dequant(self._h, qtype, blocks.data_ptr(), n_elems, out.data_ptr(),
                                             _stream_ptr()))
        return out

    # ---- encode_mat_mat_dispatch_dflash_verify (metal_forward/dispatch.rs:365-378)
    def encode_mat_mat_dispatch_dflash_verify(self, weight, w_type: int, x, y, n_in: int, n_out: int, n_query: int):
        """y[n_query, n_out] = x[n_query, n_in] . W^T; enqueue only."""
        torch = _torch()
        if x.dtype == torch.float32:
            x_type = TYPE_F32
        elif x.dtype == torch.float16:
            x_type = TYPE_F16
        else:
            raise DFlashError(2, f"activation dtype {x.dtype} unsupported")
        self._check(self._lib.dflash_gemm_fewrow(self._h, w_type, weight.data_ptr(), x.data_ptr(), x_type,
                                                 y.data_ptr(), n_in, n_out, n_query, _stream_ptr()))
        return y

    def checked_type(self, qtype: int, blocks) -> int:
        """Range-checks a Q4_K / Q6_K tensor (raises DFlashError where the fast kernels cannot take it) and returns the
        type tag that selects them: ``qtype | TYPE_RANGE_CHECKED``.  Other types come back unchanged."""
        bb = {TYPE_Q4_K: 144, TYPE_Q6_K: 210}.get(int(qtype))
        if bb is None:
            return int(qtype)
        self.check_scale_range(int(qtype), blocks, blocks.numel() * blocks.element_size() // bb)
        return int(qtype) | TYPE_RANGE_CHECKED

    def check_scale_range(self, qtype: int, blocks, n_blocks: int):
        """Load-time guard: raises DFlashError (UNSUPPORTED) for a Q4_K / Q6_K tensor whose super-block scales are
        outside the few-row kernels' f16 range; returns (max |d|, max |dmin|)."""
        out = (C.c_float * 2)()
        self._check(self._lib.dflash_check_scale_range(self._h, int(qtype), blocks.data_ptr(), int(n_blocks), out, _stream_ptr()))
        return float(out[0]), float(out[1])

    def hbm_read_probe(self, bufs, n_launches: int, scratch):
        """``n_launches`` launches of a read-only streaming kernel over the equally sized uint8 tensors ``bufs``
        (in turn); ``scratch``: int32[n_cu]."""
        ptrs = (C.c_void_p * len(bufs))(*[b.data_ptr() for b in bufs])
        nbytes = bufs[0].numel() * bufs[0].element_size()
        self._check(self._lib.dflash_hbm_read_probe(self._h, ptrs, len(bufs), nbytes, n_launches, scratch.data_ptr(), _stream_ptr()))

    def repack_q4k_tiled(self, weight, n_in: int, n_out: int):
        """Q4_K blocks in GGUF row order -> a new tensor in tiled order (w_type TYPE_Q4_K_TILED): a one-time
        permutation of whole blocks at upload; the few-row GEMM on it gives bit-identical results."""
        torch = _torch()
        nbytes = self._lib.dflash_q4k_tiled_bytes(n_in, n_out)
        if nbytes == 0:
            raise DFlashError(2, f"bad Q4_K shape {n_out} x {n_in}")
        out = _empty(nbytes, dtype=torch.uint8, device=weight.device)
        self._check(self._lib.dflash_repack_q4k_tiled(self._h, weight.data_ptr(), out.data_ptr(), n_in, n_out, _stream_ptr()))
        return out

    def repack_q6k_tiled(self, weight, n_in: int, n_out: int):
        """Q6_K blocks in GGUF row order -> a new tensor in the tiled, field-planar order (w_type TYPE_Q6_K_TILED), which
        gemm_fewrow_xf (and the model-level calls) read with aligned loads; bit-identical results."""
        torch = _torch()
        nbytes = self._lib.dflash_q6k_tiled_bytes(n_in, n_out)
        if nbytes == 0:
            raise DFlashError(2, f"bad Q6_K shape {n_out} x {n_in}")
        out = _empty(nbytes, dtype=torch.uint8, device=weight.device)
        self._check(self._lib.dflash_repack_q6k_tiled(self._h, weight.data_ptr(), out.data_ptr(), n_in, n_out, _stream_ptr()))
        return out

    def gemm_fewrow(self, weight, w_type: int, x, n_in: int, n_out: int):
        torch = _torch()
        y = _empty((x.shape[0], n_out), dtype=torch.float32, device=x.device)
        return self.encode_mat_mat_dispatch_dflash_verify(weight, w_type, x, y, n_in, n_out, x.shape[0])

    # ---- the same product over activations handed over in MFMA fragment order (no counterpart in the reference)
    def xf_kind(self, w_type: int, n_in: int, n_out: int) -> int:
        """XF kind the whole-K kernel reads for this matrix (XF_Q4K / XF_Q6K), or XF_NONE where it does not take it."""
        return int(self._lib.dflash_gemm_fewrow_xf_kind(self._h, int(w_type), n_in, n_out))

    def pack_xf(self, x, kind: int):
        """x [n_rows, n_in] f32 / f16 -> a uint8 tensor holding the rows as f16 in fragment order `kind`."""
        torch = _torch()
        n_rows, n_in = x.shape
        nbytes = self._lib.dflash_xf_bytes(n_in)
        if nbytes == 0:
            raise DFlashError(1, f"n_in {n_in} is not a multiple of 256")
        xf = _empty(nbytes, dtype=torch.uint8, device=x.device)
        x_type = TYPE_F32 if x.dtype == torch.float32 else TYPE_F16
        self._check(self._lib.dflash_pack_xf(self._h, x.data_ptr(), x_type, n_rows, n_in, int(kind), xf.data_ptr(), _stream_ptr()))
        return xf

    def gemm_fewrow_xf(self, weight, w_type: int, xf, n_rows: int, n_in: int, n_out: int, y=None):
        torch = _torch()
        if y is None:
            y = _empty((n_rows, n_out), dtype=torch.float32, device=xf.device)
        self._check(self._lib.dflash_gemm_fewrow_xf(self._h, int(w_type), weight.data_ptr(), xf.data_ptr(), y.data_ptr(), n_in,
                                                     n_out, n_rows, _stream_ptr()))
        return y

    # ---- per-row scatter + decode attention loop of packed verify (metal_dflash.rs:9963-10062)
    def attn_verify_block(self, q, k_cache, v_cache, ctx_len: int, scale: float, v_transposed: bool = False,
                          out=None):
        """q [n_rows, n_q, hd] f32/f16; k_cache [cap, n_kv, hd] f16; v_cache the same, or
        [n_kv, hd, cap] when v_transposed.  Row i attends positions [0, ctx_len + i]."""
        torch = _torch()
        n_rows, n_q, hd = q.shape
        cap, n_kv = k_cache.shape[0], k_cache.shape[1]
        q_type = TYPE_F32 if q.dtype == torch.float32 else TYPE_F16
        if out is None:
            out = _empty((n_rows, n_q, hd), dtype=torch.float32, device=q.device)
        self._check(self._lib.dflash_attn_verify_block(self._h, q.data_ptr(), q_type, k_cache.data_ptr(),
                                                       v_cache.data_ptr(), 1 if v_transposed else 0, ctx_len, n_rows,
                                                       n_q, n_kv, hd, cap, scale, out.data_ptr(), _stream_ptr()))
        return out

    # ---- argmax family (metal/elementwise.rs:1196-1318) and top-16 (metal/elementwise.rs:1370-1386)
    def _rows(self, logits):
        if logits.dim() == 1:
            logits = logits.unsqueeze(0)
        return logits, logits.shape[0], logits.shape[1], logits.stride(0)

    def argmax_top2(self, logits):
        torch = _torch()
        logits, n, v, stride = self._rows(logits)
        idx = _empty(n, dtype=torch.int32, device=logits.device)
        gap = _empty(n, dtype=torch.float32, device=logits.device)
        self._check(self._lib.dflash_argmax_top2(self._h, logits.data_ptr(), n, v, stride, idx.data_ptr(),
                                                 gap.data_ptr(), _stream_ptr()))
        return idx, gap

    def argmax_greedy(self, logits):
        torch = _torch()
        logits, n, v, stride = self._rows(logits)
        idx = _empty(n, dtype=torch.int32, device=logits.device)
        self._check(self._lib.dflash_argmax_greedy(self._h, logits.data_ptr(), n, v, stride, idx.data_ptr(),
                                                   _stream_ptr()))
        return idx

    def top16(self, logits):
        torch = _torch()
        logits, n, v, stride = self._rows(logits)
        ids = _empty((n, 16), dtype=torch.int32, device=logits.device)
        vals = _empty((n, 16), dtype=torch.float32, device=logits.device)
        self._check(self._lib.dflash_top16(self._h, logits.data_ptr(), n, v, stride, ids.data_ptr(), vals.data_ptr(),
                                           _stream_ptr()))
        return ids, vals

    # ---- DFlash-2 extras (kernels/dflash2.metal:40-69; metal_dflash.rs:17176-17251)
    def dflash2_conv(self, x, dyn, base, kernel_size: int, group_size: int, side: int):
        """x [n_tokens, h], dyn [n_tokens, 2*kernel_size*h/group_size], base [2, kernel_size, h] (device f32) -> y."""
        torch = _torch()
        n, h = x.shape
        y = torch.empty_like(x)
        self._check(self._lib.dflash_dflash2_conv(self._h, x.data_ptr(), dyn.data_ptr(), base.data_ptr(), y.data_ptr(), n, h,
                                                  kernel_size, group_size, side, _stream_ptr()))
        return y

    def select_draft_path(self, predecessor, successor, rank: int, carry_token: int, topk_ids, topk_vals, sel_h):
        """predecessor / successor: (type, device tensor of rows); topk_ids/topk_vals [n, top_k], sel_h [n, rank]
        on the device.  Returns the n tokens of the greedy selector walk (host list)."""
        torch = _torch()
        n, top_k = topk_ids.shape

        def cb(pair):
            qtype, rows = pair
            return CodebookC(qtype, 0, rows.shape[0], rows.data_ptr())

        pc, sc = cb(predecessor), cb(successor)
        out = _empty(n, dtype=torch.int32, device=topk_ids.device)
        host = (C.c_int32 * n)()
        self._check(self._lib.dflash_select_draft_path(self._h, C.byref(pc), C.byref(sc), rank, top_k, carry_token, n,
                                                       topk_ids.data_ptr(), topk_vals.data_ptr(), sel_h.data_ptr(),
                                                       out.data_ptr(), host, _stream_ptr()))
        return list(host)

    def select_draft_path_sampled(self, predecessor, successor, rank: int, carry_token: int, topk_ids, topk_vals, sel_h,
                                  proposal_sampler: Sampler):
        """The sampled selector walk (draft_block_sampled, metal_dflash.rs:17268-17415).  Returns (tokens, proposals):
        tokens [n] on the host and, per position 1..n-1, (token, [(token, weight), ...]): the SparseProposal list that
        decide_dflash_accept_prefix takes.  Advances the proposal sampler by one draw per position."""
        torch = _torch()
        n, top_k = topk_ids.shape

        def cb(pair):
            qtype, rows = pair
            return CodebookC(qtype, 0, rows.shape[0], rows.data_ptr())

        pc, sc = cb(predecessor), cb(successor)
        toks = (C.c_int32 * n)()
        counts = (C.c_int32 * max(n - 1, 1))()
        cands = (WeightedCandidateC * (max(n - 1, 1) * top_k))()
        self._check(self._lib.dflash_select_draft_path_sampled(self._h, C.byref(pc), C.byref(sc), rank, top_k, carry_token, n,
                                                               topk_ids.data_ptr(), topk_vals.data_ptr(), sel_h.data_ptr(),
                                                               C.byref(proposal_sampler.c), toks, counts, cands, _stream_ptr()))
        props = [(toks[p + 1], [(cands[p * top_k + i].token, cands[p * top_k + i].weight) for i in range(counts[p])])
                 for p in range(n - 1)]
        return list(toks), props

    # ---- decide_dflash_accept_prefix (metal_dflash/accept.rs:76-84)
    def decide_dflash_accept_prefix(self, verified_tokens, target_logits, vocab, proposals, sampler: Sampler,
                                    remaining_output_budget, stop_ids, draft_logits=None, draft_temperature=0.0):
        """verified_tokens: [carry, drafts...] (host ints); target_logits: device f32 [len, vocab];
        proposals: None (deterministic drafts) or a list of (token, [(token, weight), ...]) per draft row;
        draft_logits: device f32 [len-1, vocab] selects the vocabulary-wide proposal instead.
        Returns an AcceptDecision; raises DFlashError (sampler unchanged) on any error."""
        n = len(verified_tokens)
        toks = (C.c_int32 * max(1, n))(*verified_tokens)
        stops = (C.c_int32 * max(1, len(stop_ids)))(*stop_ids)
        mode, n_props, ptoks, pcnts, pcands = 0, 0, None, None, None
        if draft_logits is not None:
            mode = 2
        elif proposals is not None:
            mode, n_props = 1, len(proposals)
            ptoks = (C.c_int32 * max(1, n_props))(*[p[0] for p in proposals])
            pcnts = (C.c_int32 * max(1, n_props))(*[len(p[1]) for p in proposals])
            flat = [c for p in proposals for c in p[1]]
            pcands = (WeightedCandidateC * max(1, len(flat)))()
            for i, (t, w) in enumerate(flat):
                pcands[i].token, pcands[i].weight = t, w
        if target_logits is not None and n > 0 and vocab > 0 and target_logits.numel() != n * vocab:
            raise DFlashError(7, "target logits extent mismatch")
        out = AcceptDecisionC()
        rc = self._lib.dflash_accept_prefix(
            self._h, toks, n, target_logits.data_ptr() if target_logits is not None else None, vocab, mode, n_props,
            ptoks, pcnts, pcands, draft_logits.data_ptr() if draft_logits is not None else None, draft_temperature,
            C.byref(sampler.c), remaining_output_budget, stops, len(stop_ids), C.byref(out), _stream_ptr())
        if rc:
            err = DFlashError(rc, self._lib.dflash_last_error(self._h).decode())
            err.decision = AcceptDecision(out)
            raise err
        return AcceptDecision(out)
