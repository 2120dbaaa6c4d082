"""Host mirror of the target session, packed verify, rollback and the block drafter.

Names follow the reference: ``MetalSession`` / ``encode_packed_verify_layer_major``
(metal_dflash.rs:10696-10719), ``encode_restore_after_partial_accept`` (:15649-15777),
``MetalDFlashSession`` / ``append_target_ctx_columns_now`` (:5053-5191, 5798-5860) and
``MetalDFlashDraftDecoder::draft_block`` (:17257-17513).  Weights are plain dictionaries of
numpy arrays (GGUF quant blocks as uint8 rows), uploaded once and used in place.
"""
from __future__ import annotations

import ctypes as C
import os
from dataclasses import asdict, dataclass

import numpy as np

from . import synth
from . import binding as _binding
from .binding import QT_RANGE_CHECKED, TYPE_Q4_K, TYPE_Q4_K_TILED, TYPE_Q6_K, TYPE_Q6_K_TILED, XF_NONE, CodebookC, Context, DFlashError, _stream_ptr, _torch, lib


@dataclass
class ModelConfig:
    n_layers: int
    hidden: int
    n_q: int
    n_kv: int
    head_dim: int
    ffn: int
    vocab: int
    n_expert: int = 0
    n_expert_used: int = 0
    ffn_expert: int = 0
    ffn_shared: int = 0
    eps: float = 1e-6
    rope_theta: float = 1e6

    def as_dict(self):
        return asdict(self)


@dataclass
class DraftConfig:
    n_layers: int
    hidden: int
    n_q: int
    n_kv: int
    head_dim: int
    ffn: int
    block_size: int = 16
    n_taps: int = 5
    causal: int = 0
    swa_window: int = 0
    eps: float = 1e-6
    rope_theta: float = 1e6
    # DFlash-2 (loader.rs:367-376): all zero for a DFlash-1 drafter
    conv_kernel_size: int = 0
    conv_group_size: int = 0
    selector_rank: int = 0
    selector_top_k: int = 0

    def as_dict(self):
        return asdict(self)


class QTensorC(C.Structure):
    _fields_ = [("type", C.c_int32), ("flags", C.c_int32), ("data", C.c_void_p)]


class ModelCfgC(C.Structure):
    _fields_ = [(n, C.c_int32) for n in ("n_layers", "hidden", "n_q", "n_kv", "head_dim", "ffn", "vocab", "n_expert",
                                          "n_expert_used", "ffn_expert", "ffn_shared")] + \
               [("eps", C.c_float), ("rope_theta", C.c_float)]


class LayerC(C.Structure):
    _fields_ = [("attn_norm", C.c_void_p), ("q_norm", C.c_void_p), ("k_norm", C.c_void_p), ("post_norm", C.c_void_p),
                ("wq", QTensorC), ("wk", QTensorC), ("wv", QTensorC), ("wo", QTensorC), ("gate", QTensorC),
                ("up", QTensorC), ("down", QTensorC), ("router", QTensorC), ("shexp_gate", C.c_void_p),
                ("gate_exps", QTensorC), ("up_exps", QTensorC), ("down_exps", QTensorC)]


class ModelC(C.Structure):
    _fields_ = [("cfg", ModelCfgC), ("layers", C.POINTER(LayerC)), ("token_embd", QTensorC), ("output", QTensorC),
                ("output_norm", C.c_void_p)]


class DraftCfgC(C.Structure):
    _fields_ = [(n, C.c_int32) for n in ("n_layers", "hidden", "n_q", "n_kv", "head_dim", "ffn", "block_size", "n_taps",
                                          "causal")] + \
               [("swa_window", C.c_uint32), ("eps", C.c_float), ("rope_theta", C.c_float)] + \
               [(n, C.c_int32) for n in ("conv_kernel_size", "conv_group_size", "selector_rank", "selector_top_k")]


class DraftLayerC(C.Structure):
    _fields_ = [("attn_norm", C.c_void_p), ("q_norm", C.c_void_p), ("k_norm", C.c_void_p), ("post_norm", C.c_void_p),
                ("wq", QTensorC), ("wk", QTensorC), ("wv", QTensorC), ("wo", QTensorC), ("gate", QTensorC),
                ("up", QTensorC), ("down", QTensorC), ("is_swa", C.c_int32), ("pad", C.c_int32),
                ("conv_attn_proj", QTensorC), ("conv_ffn_proj", QTensorC), ("conv_attn_base", C.c_void_p),
                ("conv_ffn_base", C.c_void_p)]


class DraftHeadC(C.Structure):
    _fields_ = [("cfg", DraftCfgC), ("layers", C.POINTER(DraftLayerC)), ("fc", QTensorC), ("hidden_norm", C.c_void_p),
                ("output_norm", C.c_void_p), ("selector_hidden", QTensorC), ("selector_predecessor", CodebookC),
                ("selector_successor", CodebookC)]


_declared = False


def _lib():
    global _declared
    L = lib()
    if not _declared:
        vp, i32, i64, f32 = C.c_void_p, C.c_int32, C.c_int64, C.c_float
        L.dflash_session_create.restype = i32
        L.dflash_session_create.argtypes = [vp, C.POINTER(ModelCfgC), i64, i32, C.POINTER(vp)]
        L.dflash_session_destroy.restype = None
        L.dflash_session_destroy.argtypes = [vp]
        L.dflash_session_kv_n_pos.restype = i64
        L.dflash_session_kv_n_pos.argtypes = [vp]
        L.dflash_session_graph_replays.restype = i64
        L.dflash_session_graph_replays.argtypes = [vp]
        L.dflash_verify_block.restype = i32
        L.dflash_verify_block.argtypes = [vp, C.POINTER(ModelC), vp, C.POINTER(i32), i32, i64, C.POINTER(i32), i32, vp,
                                          vp, vp, vp, C.POINTER(i32), vp]
        L.dflash_restore.restype = i32
        L.dflash_restore.argtypes = [vp, vp, i64, i32, i32]
        L.dflash_draft_session_create.restype = i32
        L.dflash_draft_session_create.argtypes = [vp, C.POINTER(DraftCfgC), i64, i64, C.POINTER(vp)]
        L.dflash_draft_session_destroy.restype = None
        L.dflash_draft_session_destroy.argtypes = [vp]
        L.dflash_draft_session_ctx_len.restype = i64
        L.dflash_draft_session_ctx_len.argtypes = [vp]
        L.dflash_draft_session_graph_replays.restype = i64
        L.dflash_draft_session_graph_replays.argtypes = [vp]
        L.dflash_draft_prepare_ctx.restype = i32
        L.dflash_draft_prepare_ctx.argtypes = [vp, vp, vp, vp]
        L.dflash_draft_append_ctx.restype = i32
        L.dflash_draft_append_ctx.argtypes = [vp, vp, vp, i32, C.POINTER(i32), vp]
        L.dflash_draft_block.restype = i32
        L.dflash_draft_block.argtypes = [vp, C.POINTER(ModelC), C.POINTER(DraftHeadC), vp, i32, i32, i64, vp, vp,
                                         C.POINTER(i32), vp]
        _declared = True
    return L


# ---- synthetic weights (numpy; the same dictionaries feed the CPU checker in the tests) ----

_ATTN_MATS = ("wq", "wk", "wv", "wo")


def _norm_w(rng, n):
    return (1.0 + 0.1 * rng.standard_normal(n)).astype(np.float32)


def _mat(qtype, n_out, n_in, seed):
    return (qtype, synth.random_weight(qtype, n_out, n_in, seed, std=1.0 / np.sqrt(n_in)))


def synth_target_weights(cfg: ModelConfig, seed: int, wtype: int = synth.Q4_K, embd_type: int = synth.Q6_K):
    """Random-init weights of the synthetic decoder: Q4_K projections, Q6_K embedding / lm_head."""
    rng = np.random.default_rng(seed)
    q_dim, kv_dim = cfg.n_q * cfg.head_dim, cfg.n_kv * cfg.head_dim
    s = seed * 1000003
    w = {"token_embd": (embd_type, synth.random_weight(embd_type, cfg.vocab, cfg.hidden, s + 1, std=1.0)),
         "output": _mat(embd_type, cfg.vocab, cfg.hidden, s + 2), "output_norm": _norm_w(rng, cfg.hidden), "layers": []}
    for il in range(cfg.n_layers):
        b = s + 100 * (il + 1)
        ffn = cfg.ffn_shared if cfg.n_expert else cfg.ffn
        L = {"attn_norm": _norm_w(rng, cfg.hidden), "q_norm": _norm_w(rng, cfg.head_dim),
             "k_norm": _norm_w(rng, cfg.head_dim), "post_norm": _norm_w(rng, cfg.hidden),
             "wq": _mat(wtype, q_dim, cfg.hidden, b + 1), "wk": _mat(wtype, kv_dim, cfg.hidden, b + 2),
             "wv": _mat(wtype, kv_dim, cfg.hidden, b + 3), "wo": _mat(wtype, cfg.hidden, q_dim, b + 4),
             "gate": _mat(wtype, ffn, cfg.hidden, b + 5), "up": _mat(wtype, ffn, cfg.hidden, b + 6),
             "down": _mat(wtype, cfg.hidden, ffn, b + 7)}
        if cfg.n_expert:
            fe = cfg.ffn_expert
            L["router"] = _mat(synth.Q8_0, cfg.n_expert, cfg.hidden, b + 8)
            L["shexp_gate"] = (rng.standard_normal(cfg.hidden) / np.sqrt(cfg.hidden)).astype(np.float32)
            L["gate_exps"] = _mat(wtype, cfg.n_expert * fe, cfg.hidden, b + 9)
            L["up_exps"] = _mat(wtype, cfg.n_expert * fe, cfg.hidden, b + 10)
            L["down_exps"] = _mat(wtype, cfg.n_expert * cfg.hidden, fe, b + 11)
        w["layers"].append(L)
    return w


def synth_target_weights_blocks(cfg: ModelConfig, seed: int, wtype: int = synth.Q4_K, attn_type: int = synth.Q6_K,
                                embd_type: int = synth.Q6_K):
    """The dictionary of synth_target_weights with every matrix made of random quant blocks at N(0, 1/n_in)-like
    magnitudes (synth.random_blocks_scaled) instead of quantised Gaussians: seconds instead of minutes for the
    128-expert shape, on the host, so that the same bytes feed the CPU checker."""
    rng = np.random.default_rng(seed)
    H, q_dim, kv_dim = cfg.hidden, cfg.n_q * cfg.head_dim, cfg.n_kv * cfg.head_dim

    def mat(qtype, n_out, n_in, std=None):
        return (qtype, synth.random_blocks_scaled(qtype, n_out, n_in, std if std is not None else n_in ** -0.5, rng))

    w = {"token_embd": mat(embd_type, cfg.vocab, H, 1.0), "output": mat(embd_type, cfg.vocab, H),
         "output_norm": _norm_w(rng, H), "layers": []}
    for _ in range(cfg.n_layers):
        ffn = cfg.ffn_shared if cfg.n_expert else cfg.ffn
        L = {"attn_norm": _norm_w(rng, H), "q_norm": _norm_w(rng, cfg.head_dim), "k_norm": _norm_w(rng, cfg.head_dim),
             "post_norm": _norm_w(rng, H), "wq": mat(attn_type, q_dim, H), "wk": mat(attn_type, kv_dim, H),
             "wv": mat(attn_type, kv_dim, H), "wo": mat(attn_type, H, q_dim), "gate": mat(wtype, ffn, H),
             "up": mat(wtype, ffn, H), "down": mat(wtype, H, ffn)}
        if cfg.n_expert:
            fe = cfg.ffn_expert
            L["router"] = mat(synth.Q8_0, cfg.n_expert, H)
            L["shexp_gate"] = (rng.standard_normal(H) * H ** -0.5).astype(np.float32)
            L["gate_exps"] = mat(wtype, cfg.n_expert * fe, H)
            L["up_exps"] = mat(wtype, cfg.n_expert * fe, H)
            L["down_exps"] = mat(wtype, cfg.n_expert * H, fe)
        w["layers"].append(L)
    return w


def synth_draft_weights(cfg: DraftConfig, seed: int, wtype: int = synth.Q4_K, swa_layers=(), vocab=None,
                        codebook_type: int = synth.Q4_K):
    rng = np.random.default_rng(seed + 7919)
    q_dim, kv_dim = cfg.n_q * cfg.head_dim, cfg.n_kv * cfg.head_dim
    s = seed * 1000003 + 500000
    w = {"fc": _mat(wtype, cfg.hidden, cfg.n_taps * cfg.hidden, s + 1), "hidden_norm": _norm_w(rng, cfg.hidden),
         "output_norm": _norm_w(rng, cfg.hidden), "layers": []}
    for il in range(cfg.n_layers):
        b = s + 100 * (il + 1)
        w["layers"].append({
            "attn_norm": _norm_w(rng, cfg.hidden), "q_norm": _norm_w(rng, cfg.head_dim),
            "k_norm": _norm_w(rng, cfg.head_dim), "post_norm": _norm_w(rng, cfg.hidden),
            "wq": _mat(wtype, q_dim, cfg.hidden, b + 1), "wk": _mat(wtype, kv_dim, cfg.hidden, b + 2),
            "wv": _mat(wtype, kv_dim, cfg.hidden, b + 3), "wo": _mat(wtype, cfg.hidden, q_dim, b + 4),
            "gate": _mat(wtype, cfg.ffn, cfg.hidden, b + 5), "up": _mat(wtype, cfg.ffn, cfg.hidden, b + 6),
            "down": _mat(wtype, cfg.hidden, cfg.ffn, b + 7), "is_swa": int(il in swa_layers)})
        if cfg.conv_kernel_size:
            dyn_dim = 2 * cfg.conv_kernel_size * (cfg.hidden // cfg.conv_group_size)
            L = w["layers"][-1]
            L["conv_attn_proj"] = _mat(wtype, dyn_dim, cfg.hidden, b + 8)
            L["conv_ffn_proj"] = _mat(wtype, dyn_dim, cfg.hidden, b + 9)
            # base kernels near the identity tap (tap 0 about 1, the others small), f32 [2][kernel][hidden]
            for name in ("conv_attn_base", "conv_ffn_base"):
                base = (0.1 * rng.standard_normal((2, cfg.conv_kernel_size, cfg.hidden))).astype(np.float32)
                base[:, 0, :] += 1.0
                L[name] = base
    if cfg.selector_rank:
        if vocab is None:
            raise ValueError("a DFlash-2 selector needs the target vocabulary size")
        w["selector_hidden"] = _mat(wtype, cfg.selector_rank, cfg.hidden, s + 2)
        # per-token predecessor / successor tables [vocab][rank]
        w["selector_predecessor"] = (codebook_type, synth.random_weight(codebook_type, vocab, cfg.selector_rank, s + 3, std=1.0))
        w["selector_successor"] = (codebook_type, synth.random_weight(codebook_type, vocab, cfg.selector_rank, s + 4, std=1.0))
    return w


def _dev_mat(qtype, n_out, n_in, std, gen, device):
    return (qtype, synth.random_blocks_device(qtype, n_out, n_in, std, gen, device))


def synth_target_weights_device(cfg: ModelConfig, seed: int, device, wtype: int = synth.Q4_K, attn_type: int = synth.Q6_K,
                                embd_type: int = synth.Q6_K):
    """The same dictionary as synth_target_weights, but every matrix is generated on the device as random
    quant blocks with scales chosen for N(0, 1/n_in)-like magnitudes (for timing large configurations: the host
    quantiser would take minutes on tens of GB).  Not reproducible by the CPU checker's quantiser; use only where
    results are compared between device paths."""
    torch = _torch()
    gen = torch.Generator(device=device)
    gen.manual_seed(seed)
    H, q_dim, kv_dim = cfg.hidden, cfg.n_q * cfg.head_dim, cfg.n_kv * cfg.head_dim

    def norm(n):
        return 1.0 + 0.1 * torch.randn(n, generator=gen, device=device)

    w = {"token_embd": _dev_mat(embd_type, cfg.vocab, H, 1.0, gen, device),
         "output": _dev_mat(embd_type, cfg.vocab, H, H ** -0.5, gen, device), "output_norm": norm(H), "layers": []}
    for _ in range(cfg.n_layers):
        ffn = cfg.ffn_shared if cfg.n_expert else cfg.ffn
        L = {"attn_norm": norm(H), "q_norm": norm(cfg.head_dim), "k_norm": norm(cfg.head_dim), "post_norm": norm(H),
             "wq": _dev_mat(attn_type, q_dim, H, H ** -0.5, gen, device), "wk": _dev_mat(attn_type, kv_dim, H, H ** -0.5, gen, device),
             "wv": _dev_mat(attn_type, kv_dim, H, H ** -0.5, gen, device), "wo": _dev_mat(attn_type, H, q_dim, q_dim ** -0.5, gen, device),
             "gate": _dev_mat(wtype, ffn, H, H ** -0.5, gen, device), "up": _dev_mat(wtype, ffn, H, H ** -0.5, gen, device),
             "down": _dev_mat(wtype, H, ffn, ffn ** -0.5, gen, device)}
        if cfg.n_expert:
            fe = cfg.ffn_expert
            L["router"] = _dev_mat(synth.Q8_0, cfg.n_expert, H, H ** -0.5, gen, device)
            L["shexp_gate"] = torch.randn(H, generator=gen, device=device) * H ** -0.5
            L["gate_exps"] = _dev_mat(wtype, cfg.n_expert * fe, H, H ** -0.5, gen, device)
            L["up_exps"] = _dev_mat(wtype, cfg.n_expert * fe, H, H ** -0.5, gen, device)
            L["down_exps"] = _dev_mat(wtype, cfg.n_expert * H, fe, fe ** -0.5, gen, device)
        w["layers"].append(L)
    return w


def synth_draft_weights_device(cfg: DraftConfig, seed: int, device, wtype: int = synth.Q4_K, vocab=None):
    """synth_draft_weights with every matrix generated on the device as random quant blocks (for timing; a DFlash-2
    configuration gets its convolution and selector tensors too and needs ``vocab`` for the codebooks)."""
    torch = _torch()
    gen = torch.Generator(device=device)
    gen.manual_seed(seed + 7919)
    H, q_dim, kv_dim = cfg.hidden, cfg.n_q * cfg.head_dim, cfg.n_kv * cfg.head_dim

    def norm(n):
        return 1.0 + 0.1 * torch.randn(n, generator=gen, device=device)

    w = {"fc": _dev_mat(wtype, H, cfg.n_taps * H, (cfg.n_taps * H) ** -0.5, gen, device), "hidden_norm": norm(H),
         "output_norm": norm(H), "layers": []}
    for _ in range(cfg.n_layers):
        w["layers"].append({
            "attn_norm": norm(H), "q_norm": norm(cfg.head_dim), "k_norm": norm(cfg.head_dim), "post_norm": norm(H),
            "wq": _dev_mat(wtype, q_dim, H, H ** -0.5, gen, device), "wk": _dev_mat(wtype, kv_dim, H, H ** -0.5, gen, device),
            "wv": _dev_mat(wtype, kv_dim, H, H ** -0.5, gen, device), "wo": _dev_mat(wtype, H, q_dim, q_dim ** -0.5, gen, device),
            "gate": _dev_mat(wtype, cfg.ffn, H, H ** -0.5, gen, device), "up": _dev_mat(wtype, cfg.ffn, H, H ** -0.5, gen, device),
            "down": _dev_mat(wtype, H, cfg.ffn, cfg.ffn ** -0.5, gen, device), "is_swa": 0})
        if cfg.conv_kernel_size:
            dyn_dim = 2 * cfg.conv_kernel_size * (H // cfg.conv_group_size)
            L = w["layers"][-1]
            L["conv_attn_proj"] = _dev_mat(wtype, dyn_dim, H, 0.1 * H ** -0.5, gen, device)
            L["conv_ffn_proj"] = _dev_mat(wtype, dyn_dim, H, 0.1 * H ** -0.5, gen, device)
            for name in ("conv_attn_base", "conv_ffn_base"):  # near the identity tap, f32 [2][kernel][hidden]
                base = 0.1 * torch.randn((2, cfg.conv_kernel_size, H), generator=gen, device=device)
                base[:, 0, :] += 1.0
                L[name] = base
    if cfg.selector_rank:
        if vocab is None:
            raise ValueError("a DFlash-2 selector needs the target vocabulary size")
        w["selector_hidden"] = _dev_mat(wtype, cfg.selector_rank, H, H ** -0.5, gen, device)
        w["selector_predecessor"] = _dev_mat(wtype, vocab, cfg.selector_rank, 1.0, gen, device)
        w["selector_successor"] = _dev_mat(wtype, vocab, cfg.selector_rank, 1.0, gen, device)
    return w


# ---- device-resident weights ----

class _Uploader:
    def __init__(self, device, ctx=None, tiled=True, tile_q6k=False):
        """``ctx``: when given, every Q4_K / Q6_K tensor's super-block scales are range-checked on upload (a tensor the
        few-row kernels cannot take is declined with DFlashError) and, with ``tiled``, Q4_K matrices uploaded with a
        tile shape are repacked into the tiled order.  ``tile_q6k``: Q6_K matrices uploaded with a tile shape that the
        one-launch GEMM takes (``Context.xf_kind``) go into the tiled Q6_K order as well (only that GEMM reads it: for
        tensors nothing else multiplies, i.e. a target's attention projections)."""
        self.torch = _torch()
        self.device = device
        self.ctx = ctx
        self.tiled = tiled and ctx is not None and not os.environ.get("DFLASH_NO_TILED")  # (the variable: for A/B runs)
        self.tile_q6k = tile_q6k and self.tiled and not os.environ.get("DFLASH_NO_TILED_Q6K")
        self.keep = []
        self.n_tiled = 0  # uploads that went into the tiled order

    _BLOCK_BYTES = {12: 144, 14: 210}

    def _guard(self, qtype, t) -> int:
        """Range check of a Q4_K / Q6_K tensor; returns the dflash_qtensor flags it has earned."""
        bb = self._BLOCK_BYTES.get(int(qtype))
        if self.ctx is not None and bb:
            self.ctx.check_scale_range(int(qtype), t, t.numel() * t.element_size() // bb)
            return QT_RANGE_CHECKED
        return 0

    def _from_numpy(self, a):
        """torch view of a host array; read-only arrays (views into a mapped GGUF file) are only ever copied from."""
        if a.flags.writeable:
            return self.torch.from_numpy(a)
        import warnings
        with warnings.catch_warnings():
            warnings.simplefilter("ignore")
            return self.torch.from_numpy(a)

    def f32(self, a):
        if isinstance(a, self.torch.Tensor):
            t = a.to(self.device, self.torch.float32).contiguous()
        else:
            t = self._from_numpy(np.ascontiguousarray(a, dtype=np.float32)).to(self.device)
        self.keep.append(t)
        return t.data_ptr()

    def q(self, pair, tile_shape=None, allow_q6k=False):
        """``tile_shape`` = (n_out, n_in): a Q4_K matrix that only the few-row GEMM reads is repacked into the
        library's tiled order (a permutation of whole blocks, bit-identical products, faster streaming)."""
        if pair is None:
            return QTensorC(0, 0, None)
        qtype, blocks = pair
        if isinstance(blocks, self.torch.Tensor):  # already resident (device-generated synthetic blocks)
            t = blocks.to(self.device).contiguous()
        else:
            t = self._from_numpy(np.ascontiguousarray(blocks)).to(self.device)
        flags = self._guard(qtype, t)
        if tile_shape is not None and self.tiled and int(qtype) == TYPE_Q4_K:
            t = self.ctx.repack_q4k_tiled(t, tile_shape[1], tile_shape[0])
            qtype = TYPE_Q4_K_TILED
            self.n_tiled += 1
        elif (tile_shape is not None and allow_q6k and self.tile_q6k and int(qtype) == TYPE_Q6_K
              and self.ctx.xf_kind(TYPE_Q6_K_TILED, tile_shape[1], tile_shape[0]) != XF_NONE):
            t = self.ctx.repack_q6k_tiled(t, tile_shape[1], tile_shape[0])
            qtype = TYPE_Q6_K_TILED
            self.n_tiled += 1
        self.keep.append(t)
        return QTensorC(int(qtype), flags, t.data_ptr())

    def q_adjacent(self, pairs, tile_shapes=None, allow_q6k=False):
        """Uploads matrices of one type and one row length back to back in a single allocation (rows of the
        first, then the second, ...): the library then runs a layer's wq/wk/wv (or gate/up) as ONE GEMM.
        Falls back to separate uploads when the types differ.  ``tile_shapes`` = [(n_out, n_in), ...]: Q4_K sets
        whose row counts are all multiples of 256 are repacked as one tiled matrix (tile groups are 256 rows, so
        every member still starts where its row-order address arithmetic says)."""
        if any(p is None for p in pairs) or len({int(p[0]) for p in pairs}) != 1:
            return [self.q(p, ts) for p, ts in zip(pairs, tile_shapes or [None] * len(pairs))]  # (never the tiled Q6_K order: separate launches)
        torch = self.torch
        flats = []
        for _, blocks in pairs:
            if isinstance(blocks, torch.Tensor):
                flats.append(blocks.to(self.device).contiguous().view(torch.uint8).reshape(-1))
            else:
                flats.append(self._from_numpy(np.ascontiguousarray(blocks).view(np.uint8).reshape(-1)).to(self.device))
        whole = torch.cat(flats)
        qtype = int(pairs[0][0])
        flags = self._guard(qtype, whole)
        if (tile_shapes is not None and self.tiled and qtype == TYPE_Q4_K
                and all(ts is not None and ts[0] % 256 == 0 for ts in tile_shapes)):
            whole = self.ctx.repack_q4k_tiled(whole, tile_shapes[0][1], sum(ts[0] for ts in tile_shapes))
            qtype = TYPE_Q4_K_TILED
            self.n_tiled += 1
        elif (tile_shapes is not None and allow_q6k and self.tile_q6k and qtype == TYPE_Q6_K
              and all(ts is not None and ts[0] % 256 == 0 for ts in tile_shapes)
              and self.ctx.xf_kind(TYPE_Q6_K_TILED, tile_shapes[0][1], sum(ts[0] for ts in tile_shapes)) != XF_NONE):
            whole = self.ctx.repack_q6k_tiled(whole, tile_shapes[0][1], sum(ts[0] for ts in tile_shapes))
            qtype = TYPE_Q6_K_TILED
            self.n_tiled += 1
        self.keep.append(whole)
        out, off = [], 0
        for f in flats:
            out.append(QTensorC(qtype, flags, whole.data_ptr() + off))
            off += f.numel()
        return out


class TargetModel:
    """Device copy of a weight dictionary plus the ``dflash_model`` descriptor."""

    def __init__(self, ctx: Context, cfg: ModelConfig, weights: dict, adjacent: bool = True, tiled: bool = True):
        """``adjacent``: place each layer's wq/wk/wv and gate/up back to back in device memory (one GEMM each).
        ``tiled``: repack the Q4_K matrices that only the few-row GEMM reads (attention projections, a dense layer's
        FFN, the output head; a mixture layer's expert stacks and shared expert when they are all Q4_K with row counts
        that are multiples of 256) into the library's tiled order at upload; the embedding table and the router stay
        in GGUF row order."""
        self.ctx, self.cfg = ctx, cfg
        # (Q6_K attention projections too, where the one-launch GEMM takes their shape: nothing else reads them)
        up = _Uploader(f"cuda:{ctx.device}", ctx, tiled, tile_q6k=adjacent)
        self._up = up
        self._layers = (LayerC * cfg.n_layers)()
        H, qd, kvd = cfg.hidden, cfg.n_q * cfg.head_dim, cfg.n_kv * cfg.head_dim
        dense = cfg.n_expert == 0
        shape = {"wq": (qd, H), "wk": (kvd, H), "wv": (kvd, H), "wo": (H, qd)}
        if dense:
            shape.update({"gate": (cfg.ffn, H), "up": (cfg.ffn, H), "down": (H, cfg.ffn)})
        elif cfg.ffn_expert % 256 == 0 and H % 256 == 0 and cfg.ffn_shared % 256 == 0:
            # a stack whose members have a multiple of 256 rows tiles as ONE matrix (tile groups never straddle
            # experts); the three stacks and the shared expert go together, or the batched kernel declines
            E, fe, fs = cfg.n_expert, cfg.ffn_expert, cfg.ffn_shared
            moe_shape = {"gate_exps": (E * fe, H), "up_exps": (E * fe, H), "down_exps": (E * H, fe),
                         "gate": (fs, H), "up": (fs, H), "down": (H, fs)}
            first = weights["layers"][0] if weights["layers"] else {}
            if all(first.get(k) is not None and int(first[k][0]) == TYPE_Q4_K for k in moe_shape):
                shape.update(moe_shape)
        for il, Lw in enumerate(weights["layers"]):
            L = self._layers[il]
            for k in ("attn_norm", "q_norm", "k_norm", "post_norm"):
                setattr(L, k, up.f32(Lw[k]))
            grouped = ()
            if adjacent:
                grouped = ("wq", "wk", "wv", "gate", "up")
                L.wq, L.wk, L.wv = up.q_adjacent([Lw.get("wq"), Lw.get("wk"), Lw.get("wv")], [shape["wq"], shape["wk"], shape["wv"]],
                                                 allow_q6k=True)
                L.gate, L.up = up.q_adjacent([Lw.get("gate"), Lw.get("up")], [shape.get("gate"), shape.get("up")])
            for k in ("wq", "wk", "wv", "wo", "gate", "up", "down", "router", "gate_exps", "up_exps", "down_exps"):
                if k not in grouped:
                    setattr(L, k, up.q(Lw.get(k), shape.get(k), allow_q6k=(k == "wo")))
            L.shexp_gate = up.f32(Lw["shexp_gate"]) if "shexp_gate" in Lw else None
        self.c = ModelC(ModelCfgC(**cfg.as_dict()), self._layers, up.q(weights["token_embd"]),
                        up.q(weights["output"], (cfg.vocab, H), allow_q6k=True), up.f32(weights["output_norm"]))

    def weight_bytes(self) -> int:
        return sum(t.numel() * t.element_size() for t in self._up.keep)

    @property
    def tiled_tensors(self) -> int:
        """Number of uploads (single matrices, fused sets, expert stacks) held in the tiled order."""
        return self._up.n_tiled


class VerifyOutput:
    def __init__(self, argmax, gap, hidden_capture, logits, argmax_host):
        self.argmax, self.gap, self.hidden_capture, self.logits, self.argmax_host = argmax, gap, hidden_capture, logits, argmax_host


class Session:
    """Target session: f16 KV cache and ``kv_n_pos``."""

    def __init__(self, ctx: Context, model: TargetModel, kv_capacity: int, tap_layers=()):
        self.ctx, self.model = ctx, model
        self.tap_layers = list(tap_layers)
        self.capacity = int(kv_capacity)
        self._L = _lib()
        h = C.c_void_p()
        cfgc = ModelCfgC(**model.cfg.as_dict())
        ctx._check(self._L.dflash_session_create(ctx._h, C.byref(cfgc), kv_capacity, len(self.tap_layers), C.byref(h)))
        self._h = h

    def close(self):
        if getattr(self, "_h", None):
            self._L.dflash_session_destroy(self._h)
            self._h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    @property
    def kv_n_pos(self) -> int:
        return self._L.dflash_session_kv_n_pos(self._h)

    def encode_packed_verify_layer_major(self, tokens, start_position: int, want_logits=False, want_hidden=True,
                                         sync=True, want_head=True) -> VerifyOutput:
        """Forward of ``tokens`` at positions start_position.. ; appends K/V; returns argmax, top-2
        gap, the tapped hidden rows [n][n_taps][hidden] and (optionally) the logits.  ``want_head=False`` (with
        ``want_logits=False``): no output of the head is asked for and the library does not run it (prefill blocks);
        argmax, gap and argmax_host of the result are then None."""
        torch = _torch()
        cfg = self.model.cfg
        n = len(tokens)
        dev = f"cuda:{self.ctx.device}"
        toks = (C.c_int32 * max(n, 1))(*[int(t) for t in tokens])
        n_taps = len(self.tap_layers) if want_hidden else 0
        taps = (C.c_int32 * max(n_taps, 1))(*self.tap_layers[:n_taps])
        want_head = want_head or want_logits
        argmax = _binding._empty(max(n, 1), dtype=torch.int32, device=dev) if want_head else None
        gap = _binding._empty(max(n, 1), dtype=torch.float32, device=dev) if want_head else None
        hidden = _binding._empty((n, n_taps, cfg.hidden), dtype=torch.float32, device=dev) if n_taps else None
        logits = _binding._empty((n, cfg.vocab), dtype=torch.float32, device=dev) if want_logits else None
        sync = sync and want_head
        host = (C.c_int32 * max(n, 1))() if sync else None
        self.ctx._check(self._L.dflash_verify_block(
            self.ctx._h, C.byref(self.model.c), self._h, toks, n, start_position, taps, n_taps,
            argmax.data_ptr() if want_head else None, gap.data_ptr() if want_head else None,
            hidden.data_ptr() if hidden is not None else None,
            logits.data_ptr() if logits is not None else None, host, _stream_ptr()))
        return VerifyOutput(argmax[:n] if want_head else None, gap[:n] if want_head else None, hidden, logits,
                            list(host[:n]) if sync else None)

    def prepare_prefill(self):
        """Sets up the scratch of prefill_blocks (group buffers, extra lanes) now instead of inside its first call."""
        self._L.dflash_prefill_prepare.restype = C.c_int32
        self._L.dflash_prefill_prepare.argtypes = [C.c_void_p, C.c_void_p]
        self.ctx._check(self._L.dflash_prefill_prepare(self.ctx._h, self._h))

    def prefill_blocks(self, tokens, start_position: int, want_hidden=True):
        """The prompt's blocks without the output head (dflash_prefill_blocks: a mixture-of-experts target takes the rows
        of many blocks per pass, any other target several blocks in flight on the library's lane streams); returns the
        tapped hidden rows [n_tokens][n_taps][hidden] (or None).  Enqueue only."""
        torch = _torch()
        cfg = self.model.cfg
        n = len(tokens)
        L = self._L
        L.dflash_prefill_blocks.restype = C.c_int32
        L.dflash_prefill_blocks.argtypes = [C.c_void_p, C.POINTER(ModelC), C.c_void_p, C.POINTER(C.c_int32), C.c_int32, C.c_int64,
                                            C.POINTER(C.c_int32), C.c_int32, C.c_void_p, C.c_void_p]
        toks = (C.c_int32 * max(n, 1))(*[int(t) for t in tokens])
        n_taps = len(self.tap_layers) if want_hidden else 0
        taps = (C.c_int32 * max(n_taps, 1))(*self.tap_layers[:n_taps])
        hidden = (_binding._empty((n, n_taps, cfg.hidden), dtype=torch.float32, device=f"cuda:{self.ctx.device}")
                  if n_taps else None)
        self.ctx._check(L.dflash_prefill_blocks(self.ctx._h, C.byref(self.model.c), self._h, toks, n, start_position, taps, n_taps,
                                                hidden.data_ptr() if hidden is not None else None, _stream_ptr()))
        return hidden

    @property
    def graph_replays(self) -> int:
        return int(self._L.dflash_session_graph_replays(self._h))

    def encode_restore_after_partial_accept(self, start_position: int, n: int, n_keep: int):
        self.ctx._check(self._L.dflash_restore(self.ctx._h, self._h, start_position, n, n_keep))


class DraftHead:
    def __init__(self, ctx: Context, cfg: DraftConfig, weights: dict, adjacent: bool = True, tiled: bool = True):
        """``adjacent`` / ``tiled``: as for TargetModel."""
        self.ctx, self.cfg = ctx, cfg
        up = _Uploader(f"cuda:{ctx.device}", ctx, tiled)
        self._up = up
        self._layers = (DraftLayerC * cfg.n_layers)()
        H, qd, kvd = cfg.hidden, cfg.n_q * cfg.head_dim, cfg.n_kv * cfg.head_dim
        shape = {"wq": (qd, H), "wk": (kvd, H), "wv": (kvd, H), "wo": (H, qd), "gate": (cfg.ffn, H), "up": (cfg.ffn, H),
                 "down": (H, cfg.ffn)}
        # every layer's wq / wk / wv in ONE allocation, layer after layer (same types throughout): each layer's three
        # are then adjacent (one GEMM for the block's q/k/v) and the layers' [wk; wv] pairs are an equal distance apart,
        # which lets the library project the context columns' K/V of all layers with one batched GEMM
        qkv_all = None
        lw = weights["layers"]
        if adjacent and len(lw) > 1 and len({int(Lw[k][0]) for Lw in lw for k in ("wq", "wk", "wv")}) == 1:
            qkv_all = up.q_adjacent([Lw[k] for Lw in lw for k in ("wq", "wk", "wv")],
                                    [shape[k] for _ in lw for k in ("wq", "wk", "wv")])
        for il, Lw in enumerate(weights["layers"]):
            L = self._layers[il]
            for k in ("attn_norm", "q_norm", "k_norm", "post_norm"):
                setattr(L, k, up.f32(Lw[k]))
            grouped = ()
            if adjacent:
                grouped = ("wq", "wk", "wv", "gate", "up")
                if qkv_all is not None:
                    L.wq, L.wk, L.wv = qkv_all[3 * il:3 * il + 3]
                else:
                    L.wq, L.wk, L.wv = up.q_adjacent([Lw["wq"], Lw["wk"], Lw["wv"]], [shape["wq"], shape["wk"], shape["wv"]])
                L.gate, L.up = up.q_adjacent([Lw["gate"], Lw["up"]], [shape["gate"], shape["up"]])
            for k in ("wq", "wk", "wv", "wo", "gate", "up", "down"):
                if k not in grouped:
                    setattr(L, k, up.q(Lw[k], shape[k]))
            L.is_swa = int(Lw.get("is_swa", 0))
            if cfg.conv_kernel_size:
                dyn_dim = 2 * cfg.conv_kernel_size * (H // cfg.conv_group_size)
                L.conv_attn_proj, L.conv_ffn_proj = up.q(Lw["conv_attn_proj"], (dyn_dim, H)), up.q(Lw["conv_ffn_proj"], (dyn_dim, H))
                L.conv_attn_base, L.conv_ffn_base = up.f32(Lw["conv_attn_base"]), up.f32(Lw["conv_ffn_base"])
        self.c = DraftHeadC(DraftCfgC(**cfg.as_dict()), self._layers, up.q(weights["fc"], (H, cfg.n_taps * H)), up.f32(weights["hidden_norm"]),
                            up.f32(weights["output_norm"]))
        if cfg.selector_rank:
            self.c.selector_hidden = up.q(weights["selector_hidden"])
            for name in ("selector_predecessor", "selector_successor"):
                qtype, rows = weights[name]
                t = up.q((qtype, rows))
                setattr(self.c, name, CodebookC(int(qtype), 0, int(rows.shape[0]), t.data))

    def weight_bytes(self) -> int:
        return sum(t.numel() * t.element_size() for t in self._up.keep)


class DraftSession:
    """Drafter session: accumulated target context columns and their per-layer K/V."""

    def __init__(self, ctx: Context, head: DraftHead, target: TargetModel, ctx_capacity: int):
        self.ctx, self.head, self.target = ctx, head, target
        self._L = _lib()
        h = C.c_void_p()
        cfgc = DraftCfgC(**head.cfg.as_dict())
        ctx._check(self._L.dflash_draft_session_create(ctx._h, C.byref(cfgc), ctx_capacity, target.cfg.vocab, C.byref(h)))
        self._h = h

    def close(self):
        if getattr(self, "_h", None):
            self._L.dflash_draft_session_destroy(self._h)
            self._h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    @property
    def ctx_len(self) -> int:
        return self._L.dflash_draft_session_ctx_len(self._h)

    @property
    def graph_replays(self) -> int:
        return int(self._L.dflash_draft_session_graph_replays(self._h))

    def append_target_ctx_columns(self, hidden_capture, positions):
        """hidden_capture: device f32 [n_cols][n_taps][hidden]; positions: their token positions."""
        n = len(positions)
        if n and tuple(hidden_capture.shape) != (n, self.head.cfg.n_taps, self.head.cfg.hidden):
            raise DFlashError(1, f"hidden_capture shape {tuple(hidden_capture.shape)}")
        pos = (C.c_int32 * max(n, 1))(*[int(p) for p in positions])
        hc = hidden_capture.contiguous() if n else None
        self.ctx._check(self._L.dflash_draft_append_ctx(self.ctx._h, self._h, hc.data_ptr() if n else None, n, pos,
                                                        _stream_ptr()))

    def selector_inputs(self):
        """(topk_ids [block, 16] i32, topk_vals [block, 16] f32, sel_h [block, rank] f32) of the last draft block of a
        DFlash-2 head, copied off the session's buffers."""
        torch = _torch()
        L = self._L
        L.dflash_draft_session_selector_inputs.restype = C.c_int32
        L.dflash_draft_session_selector_inputs.argtypes = [C.c_void_p] * 6
        n, rank = self.head.cfg.block_size, self.head.cfg.selector_rank
        dev = f"cuda:{self.ctx.device}"
        ids = _binding._empty((n, 16), dtype=torch.int32, device=dev)
        vals = _binding._empty((n, 16), dtype=torch.float32, device=dev)
        sel_h = _binding._empty((n, max(rank, 1)), dtype=torch.float32, device=dev)
        self.ctx._check(L.dflash_draft_session_selector_inputs(self.ctx._h, self._h, ids.data_ptr(), vals.data_ptr(),
                                                               sel_h.data_ptr(), _stream_ptr()))
        return ids, vals, sel_h

    def prepare_ctx(self):
        """Bring fc + hidden_norm and the per-layer context K/V up to date for the columns appended so far
        (draft_block does it lazily otherwise)."""
        self.ctx._check(self._L.dflash_draft_prepare_ctx(self.ctx._h, C.byref(self.head.c), self._h, _stream_ptr()))

    def draft_block(self, carry_token: int, mask_token: int, noise_start_pos: int, want_logits=False, sync=True, out=None):
        """``out`` = (argmax, logits) tensors to write into (the same output pointers from call to call let the
        library replay its captured graph of the block); fresh tensors otherwise."""
        torch = _torch()
        dev = f"cuda:{self.ctx.device}"
        N = self.head.cfg.block_size
        if out is not None:
            argmax, logits = out
        else:
            argmax = _binding._empty(N, dtype=torch.int32, device=dev)
            logits = _binding._empty((N, self.target.cfg.vocab), dtype=torch.float32, device=dev) if want_logits else None
        host = (C.c_int32 * N)() if sync else None
        self.ctx._check(self._L.dflash_draft_block(
            self.ctx._h, C.byref(self.target.c), C.byref(self.head.c), self._h, carry_token, mask_token, noise_start_pos,
            argmax.data_ptr(), logits.data_ptr() if logits is not None else None, host, _stream_ptr()))
        return argmax, logits, (list(host) if sync else None)


# ---- adaptive speculation policy (qwen/dflash.rs:5-376): host logic of the library ----

class AdaptiveStateC(C.Structure):
    _fields_ = [("alpha_window", C.c_int32 * 16), ("n_alpha", C.c_int32), ("fallback_window", C.c_uint8 * 8),
                ("n_fallback", C.c_int32), ("reentry_accepts", C.c_int32 * 2), ("n_reentry", C.c_int32),
                ("reason", C.c_int32), ("long_mode", C.c_int32), ("off_steps_since_probe", C.c_int64)]


_adaptive_declared = False


def adaptive_lib():
    """The library with the policy functions' signatures declared (they run on the host; no GPU needed)."""
    global _adaptive_declared
    L = lib()
    if not _adaptive_declared:
        i32, i64, sp = C.c_int32, C.c_int64, C.POINTER(AdaptiveStateC)
        for name, res, args in (
                ("dflash_adaptive_init", None, [sp]), ("dflash_adaptive_prepare_mode", None, [sp, i32]),
                ("dflash_adaptive_backoff_active", i32, [sp]), ("dflash_adaptive_probe_due", i32, [sp, i32, i32]),
                ("dflash_adaptive_record_off_step", None, [sp]), ("dflash_adaptive_begin_spec_step", None, [sp]),
                ("dflash_adaptive_record_spec_step", None, [sp, i32, i32, i32, i32, i32, i32, i64]),
                ("dflash_speculation_enabled", i32, [i32, i64, i64, i64, i32, i32, i32]),
                ("dflash_prefix_replay_allowed", i32, [i32, i64, i64, i64, i32, i32, i32, i32]),
                ("dflash_prefix_replay_drafts", i32, [C.POINTER(i32), i64, C.POINTER(i32), i64, i64,
                                                      C.POINTER(C.POINTER(i32))]),
                ("dflash_verify_fallback_margin", C.c_float, [i64])):
            f = getattr(L, name)
            f.restype, f.argtypes = res, args
        _adaptive_declared = True
    return L


# ---- one speculative transition and the generation loop (qwen/dflash.rs:700-1241) ----

from .binding import AcceptDecision, AcceptDecisionC, Sampler, SamplerC  # noqa: E402


class StepCfgC(C.Structure):
    _fields_ = [("mask_token", C.c_int32), ("sampled_mode", C.c_int32), ("fallback_margin", C.c_float),
                ("fallback_partial", C.c_int32), ("fallback_partial_min_gap", C.c_float), ("replay_only", C.c_int32)]


class StepResultC(C.Structure):
    _fields_ = [("decision", AcceptDecisionC), ("n_block", C.c_int32), ("draft_tokens", C.c_int32 * 16),
                ("verify_argmax", C.c_int32 * 16), ("verify_gap", C.c_float * 16), ("fallback_ran", C.c_int32),
                ("fallback_rows_replayed", C.c_int32), ("fallback_escalations", C.c_int32),
                ("fallback_rows_kept", C.c_int32), ("draft_ms", C.c_double), ("verify_ms", C.c_double),
                ("accept_ms", C.c_double), ("fallback_ms", C.c_double), ("append_ms", C.c_double),
                ("restore_ms", C.c_double)]


DFLASH_VERIFY_FALLBACK_MARGIN_DEFAULT = 0.1       # qwen/dflash.rs:104
DFLASH_VERIFY_FALLBACK_PARTIAL_MIN_GAP = 0.15     # qwen/dflash.rs:139


def accept_greedy(verify_input, verify_argmax, budget: int, stop_ids=()) -> AcceptDecision:
    L = _lib()
    n = len(verify_input)
    L.dflash_accept_greedy.restype = C.c_int32
    L.dflash_accept_greedy.argtypes = [C.POINTER(C.c_int32), C.POINTER(C.c_int32), C.c_int32, C.c_int64,
                                       C.POINTER(C.c_int32), C.c_int32, C.POINTER(AcceptDecisionC)]
    out = AcceptDecisionC()
    rc = L.dflash_accept_greedy((C.c_int32 * max(n, 1))(*verify_input), (C.c_int32 * max(n, 1))(*verify_argmax), n, budget,
                                (C.c_int32 * max(len(stop_ids), 1))(*stop_ids), len(stop_ids), C.byref(out))
    if rc:
        raise DFlashError(rc, "dflash_accept_greedy: invalid input")
    return AcceptDecision(out)


class SpeculativeDecoder:
    """Target + drafter sessions driven one packed-verify transition at a time."""

    def __init__(self, ctx: Context, target: TargetModel, head: DraftHead, tap_layers, kv_capacity: int,
                 mask_token: int, sampler: Sampler | None = None, fallback_margin: float = 0.0,
                 fallback_partial: bool = True, stop_ids=(), proposal_sampler: Sampler | None = None):
        """``proposal_sampler`` (with ``sampler`` and a DFlash-2 head): the drafter samples its tokens along the
        selector walk and the target's sampler is coupled to the walk's candidate distributions
        (qwen/dflash.rs:508-519: temperature of the target's sampler only, seed ^ 0x4446_4c41_5348_3251)."""
        self.ctx, self.target, self.head = ctx, target, head
        self.tap_layers = list(tap_layers)
        self.session = Session(ctx, target, kv_capacity, self.tap_layers)
        self.session.prepare_prefill()  # (the prompt's lanes are made with the decoder, not inside its first prefill)
        self.draft_session = DraftSession(ctx, head, target, kv_capacity)
        self.sampler = sampler
        self.proposal_sampler = proposal_sampler
        self.stop_ids = list(stop_ids)
        mode = 0 if sampler is None else (2 if proposal_sampler is not None else 1)
        self.cfg = StepCfgC(mask_token, mode, fallback_margin, int(fallback_partial),
                            DFLASH_VERIFY_FALLBACK_PARTIAL_MIN_GAP)
        self._L = _lib()
        self._L.dflash_spec_step.restype = C.c_int32
        self._L.dflash_spec_step.argtypes = [
            C.c_void_p, C.POINTER(ModelC), C.POINTER(DraftHeadC), C.c_void_p, C.c_void_p, C.POINTER(C.c_int32),
            C.c_int32, C.c_int32, C.c_int64, C.POINTER(StepCfgC), C.POINTER(SamplerC), C.POINTER(SamplerC), C.c_int64,
            C.POINTER(C.c_int32), C.c_int32, C.POINTER(C.c_int32), C.POINTER(StepResultC), C.c_void_p]
        self.position = 0

    def close(self):
        self.session.close()
        self.draft_session.close()

    def prefill(self, prompt):
        """Run the prompt through the packed verify in blocks of 16, feed the tapped hidden rows to
        the drafter context, and return the argmax after the last prompt token."""
        assert len(prompt) > 0 and self.position == 0
        # every block but the last: K/V and the tapped rows only (many blocks per pass, or several in flight); the last one with its head
        body = (len(prompt) - 1) // 16 * 16
        if body:
            hidden = self.session.prefill_blocks(list(prompt[:body]), 0)
            for s in range(0, body, 16):
                self.draft_session.append_target_ctx_columns(hidden[s:s + 16], list(range(s, s + 16)))
        blk = list(prompt[body:])
        last = self.session.encode_packed_verify_layer_major(blk, body)
        self.draft_session.append_target_ctx_columns(last.hidden_capture, list(range(body, body + len(blk))))
        # the drafter's pass over the prompt's columns belongs to the prefill, not to the first step
        self.draft_session.prepare_ctx()
        _torch().cuda.synchronize()
        self.position = len(prompt)
        return last.argmax_host[-1]

    def step(self, carry: int, budget: int, draft_override=None, replay_only: bool = False) -> StepResultC:
        """One speculative transition.  ``replay_only``: a prefix-replay step, ``draft_override`` holds every draft
        and the drafter is not run."""
        res = StepResultC()
        self.cfg.replay_only = int(replay_only)
        n = self.head.cfg.block_size
        ov = None
        if draft_override is not None:
            ov = (C.c_int32 * (n - 1))(*(list(draft_override) + [-1] * (n - 1))[: n - 1])
        # the constant argument arrays are built once (rebuilt if the lists change)
        key = (tuple(self.tap_layers), tuple(self.stop_ids))
        if getattr(self, "_arg_key", None) != key:
            self._arg_key = key
            self._taps_c = (C.c_int32 * len(self.tap_layers))(*self.tap_layers)
            self._stops_c = (C.c_int32 * max(len(self.stop_ids), 1))(*self.stop_ids)
        taps, stops = self._taps_c, self._stops_c
        self.ctx._check(self._L.dflash_spec_step(
            self.ctx._h, C.byref(self.target.c), C.byref(self.head.c), self.session._h, self.draft_session._h, taps,
            len(self.tap_layers), carry, self.position, C.byref(self.cfg),
            C.byref(self.sampler.c) if self.sampler is not None else None,
            C.byref(self.proposal_sampler.c) if self.proposal_sampler is not None else None, budget, stops,
            len(self.stop_ids), ov,
            C.byref(res), _stream_ptr()))
        self.position += res.decision.retain_input_count
        return res

    def _off_step(self, carry: int, append_ctx: bool) -> int:
        """One exact single-token step with hidden capture (the loop's off step, qwen/dflash.rs:617-690): the KV and
        the drafter context stay current; returns the next token (argmax, or a draw of the target's sampler)."""
        sampled = self.sampler is not None
        out = self.session.encode_packed_verify_layer_major([carry], self.position, want_logits=sampled)
        if append_ctx:
            self.draft_session.append_target_ctx_columns(out.hidden_capture, [self.position])
        self.position += 1
        if not sampled:
            return out.argmax_host[0]
        d = self.ctx.decide_dflash_accept_prefix([carry], out.logits, self.target.cfg.vocab, None, self.sampler, 1 << 30, [])
        return d.carry_token

    def generate(self, first_carry: int, max_tokens: int, on_step=None, draft_override_fn=None, adaptive: bool = False,
                 off_ctx: int = 16384, prefix_replay=None, position_margin: bool = False):
        """Emit up to max_tokens tokens starting with first_carry.  Returns (tokens, stats).
        ``adaptive``: run the reference loop's back-off policy (qwen/dflash.rs:566-612, 1218-1231): speculation turns
        off while the trailing acceptance window is below break-even (exact single-token steps keep the caches
        current), probes again every few off steps, and stops for good at ``off_ctx`` or when a block no longer fits.
        ``prefix_replay`` (with ``adaptive``, greedy only): a previous generation's tokens; while the emitted tokens
        are a prefix of it, its continuation replaces the drafter's tokens, also through back-off (:594-612, 700-712),
        and such steps do not count as re-entry evidence.  ``position_margin``: the greedy fallback margin follows the
        position (verify_fallback_margin, :126-136) instead of the constructor's value."""
        tokens = [first_carry]
        history = [int(t) for t in prefix_replay] if prefix_replay is not None else None
        hist_c = (C.c_int32 * max(len(history), 1))(*history) if history else None
        stats = {"spec_steps": 0, "accepted_drafts": 0, "drafts_scored": 0, "fallback_calls": 0, "draft_ms": 0.0,
                 "verify_ms": 0.0, "accept_ms": 0.0, "fallback_ms": 0.0, "append_ms": 0.0, "restore_ms": 0.0,
                 "stop_reason": None, "off_steps": 0, "backoff_probe_steps": 0, "backoff_reason": 0, "prefix_replay_steps": 0}
        carry = first_carry
        L = adaptive_lib() if adaptive else None
        state = AdaptiveStateC()
        if adaptive:
            L.dflash_adaptive_init(C.byref(state))
        spec_disabled = False
        sampled = int(self.sampler is not None)
        n_block = self.head.cfg.block_size
        while True:
            if carry in self.stop_ids:
                stats["stop_reason"] = "eos"
                break
            if len(tokens) >= max_tokens:
                stats["stop_reason"] = "token_limit"
                break
            was_probe, long_mode, replay = False, False, None
            if position_margin:
                self.cfg.fallback_margin = adaptive_lib().dflash_verify_fallback_margin(self.position + n_block)
            if adaptive:
                long_mode = off_ctx > 16384 and self.position >= 16384
                L.dflash_adaptive_prepare_mode(C.byref(state), int(long_mode))
                active = L.dflash_adaptive_backoff_active(C.byref(state))
                due = L.dflash_adaptive_probe_due(C.byref(state), sampled, int(long_mode))
                remaining = self.session.capacity - self.position
                if history and not sampled and L.dflash_prefix_replay_allowed(
                        int(spec_disabled), self.position, off_ctx, remaining, n_block, int(long_mode), active, due):
                    emitted = (C.c_int32 * len(tokens))(*tokens)
                    drafts = C.POINTER(C.c_int32)()
                    if L.dflash_prefix_replay_drafts(hist_c, len(history), emitted, len(tokens), n_block - 1, C.byref(drafts)):
                        replay = [drafts[i] for i in range(n_block - 1)]
                if replay is None and not L.dflash_speculation_enabled(int(spec_disabled), self.position, off_ctx, remaining,
                                                                       n_block, active, due):
                    if self.position >= off_ctx or remaining < n_block:
                        spec_disabled = True  # terminal: the drafter context is no longer fed
                    stats["off_steps"] += 1
                    L.dflash_adaptive_record_off_step(C.byref(state))
                    carry = self._off_step(carry, not spec_disabled)
                    tokens.append(carry)
                    continue
                was_probe = bool(active and due)
                stats["backoff_probe_steps"] += int(was_probe)
                L.dflash_adaptive_begin_spec_step(C.byref(state))
            ov = replay if replay is not None else (draft_override_fn(tokens, self.position) if draft_override_fn else None)
            stats["prefix_replay_steps"] += int(replay is not None)
            res = self.step(carry, max_tokens - len(tokens), ov, replay_only=replay is not None)
            d = res.decision
            stats["spec_steps"] += 1
            stats["accepted_drafts"] += d.n_accepted
            hist = stats.setdefault("accept_len_hist", [0] * 16)  # steps by number of accepted drafts (0..15)
            hist[min(d.n_accepted, 15)] += 1
            stats["drafts_scored"] += res.n_block - 1
            stats["fallback_calls"] += res.fallback_ran
            for k in ("draft_ms", "verify_ms", "accept_ms", "fallback_ms", "append_ms", "restore_ms"):
                stats[k] += getattr(res, k)
            tokens.extend(d.accepted_drafts[: d.n_accepted])
            if on_step:
                on_step(res)
            if d.stop_reason:
                stats["stop_reason"] = "eos" if d.stop_reason == 1 else "token_limit"
                break
            if adaptive:
                L.dflash_adaptive_record_spec_step(C.byref(state), d.n_accepted, res.fallback_ran, int(was_probe),
                                                   int(replay is None), sampled, int(long_mode), self.position)
                stats["backoff_reason"] = state.reason
            carry = d.carry_token
            tokens.append(carry)
        return tokens, stats
