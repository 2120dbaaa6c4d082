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

STATUS = {
    0: "Ok", 1: "BadShape", 2: "Unsupported", 3: "Alias", 4: "Alignment", 5: "Workspace", 6: "Hip",
    7: "InvalidInput", 8: "InvalidToken", 9: "ProposalMismatch", 10: "State", 33: "EmptyLogits",
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
    L.dflash_ctx_kernel_timing.restype = i32
    L.dflash_ctx_kernel_timing.argtypes = [vp, i32, C.POINTER(C.c_double), C.POINTER(i64)]
    L.dflash_row_bytes.restype = sz
    L.dflash_row_bytes.argtypes = [i32, sz]
    L.dflash_dequant.restype = i32
    L.dflash_dequant.argtypes = [vp, i32, vp, sz, vp, vp]
    L.dflash_gemm_fewrow.restype = i32
    L.dflash_gemm_fewrow.argtypes = [vp, i32, vp, vp, i32, vp, i64, i64, i32, vp]
    L.dflash_attn_verify_block.restype = i32
    L.dflash_attn_verify_block.argtypes = [vp, vp, i32, vp, vp, i32, i64, i32, i32, i32, i32, i64, f32, vp, vp]


def _torch():
    import torch

    return torch


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
    T_GEMM, T_ATTN, T_ACCEPT, T_ARGMAX, T_PREP = 0, 1, 2, 3, 4

    def set_kernel_timing(self, enable: bool):
        self._lib.dflash_ctx_set_kernel_timing(self._h, int(enable))

    def kernel_timing(self, slot: int):
        ms, n = C.c_double(), C.c_int64()
        self._check(self._lib.dflash_ctx_kernel_timing(self._h, slot, C.byref(ms), C.byref(n)))
        return ms.value, n.value

    # ---- codec::dequant_to_f32 (codec.rs:256-302)
    def dequant_to_f32(self, qtype: int, blocks, n_elems: int, out=None):
        torch = _torch()
        if out is None:
            out = torch.empty(n_elems, dtype=torch.float32, device=blocks.device)
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

    def gemm_fewrow(self, weight, w_type: int, x, n_in: int, n_out: int):
        torch = _torch()
        y = torch.empty((x.shape[0], n_out), dtype=torch.float32, device=x.device)
        return self.encode_mat_mat_dispatch_dflash_verify(weight, w_type, x, y, n_in, n_out, x.shape[0])

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
            out = torch.empty((n_rows, n_q, hd), dtype=torch.float32, device=q.device)
        self._check(self._lib.dflash_attn_verify_block(self._h, q.data_ptr(), q_type, k_cache.data_ptr(),
                                                       v_cache.data_ptr(), 1 if v_transposed else 0, ctx_len, n_rows,
                                                       n_q, n_kv, hd, cap, scale, out.data_ptr(), _stream_ptr()))
        return out
