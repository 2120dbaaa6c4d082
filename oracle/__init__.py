"""ctypes loader for the CPU oracle (test infrastructure only).

The oracle is a plain-C restatement of the reference engine's CPU algorithms for
the DFlash step; see ``dflash_oracle.h`` for what each function follows and how it
is pinned.  Only the test-suite, the smoke check and the benchmark's CPU-baseline
leg import this module.  The shipped library never does.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_DIR = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_DIR, "liboracle.so")

Q8_0, Q4_K, Q6_K = 8, 12, 14
RNG_XOSHIRO, RNG_PHILOX = 0, 1
CARRY_NONE, CARRY_CORRECTION, CARRY_BONUS = 0, 1, 2
STOP_NONE, STOP_EOS, STOP_TOKEN_LIMIT = 0, 1, 2

ERR = {
    0: "Ok", 1: "EmptyLogits", 2: "InvalidTemperature", 3: "InvalidTopP", 4: "InvalidMinP",
    5: "NanLogit", 6: "VocabularyTooLarge", 7: "NoCandidates", 8: "ProposalTokenOutOfRange",
    9: "InvalidProposalWeight", 10: "MissingProposalToken", 11: "InvalidInput", 12: "InvalidToken",
    13: "ProposalMismatch",
}


def build(force: bool = False) -> str:
    """Compile liboracle.so with gcc (a few seconds)."""
    srcs = [os.path.join(_DIR, f) for f in ("quant.c", "rng.c", "sampler.c", "forward.c", "dflash2.c", "dflash_oracle.h")]
    stale = force or not os.path.exists(_LIB_PATH) or any(
        os.path.getmtime(s) > os.path.getmtime(_LIB_PATH) for s in srcs)
    if stale:
        subprocess.run(["make", "-C", _DIR, "-B", "liboracle.so"], check=True, capture_output=True)
    return _LIB_PATH


class SamplingConfig(C.Structure):
    _fields_ = [("temperature", C.c_float), ("top_p", C.c_float), ("min_p", C.c_float),
                ("rng_kind", C.c_int32), ("top_k", C.c_uint64), ("seed", C.c_uint64)]


class Sampler(C.Structure):
    _fields_ = [("cfg", SamplingConfig), ("s", C.c_uint64 * 4), ("draws", C.c_uint64)]


class WeightedCandidate(C.Structure):
    _fields_ = [("token", C.c_int32), ("pad", C.c_int32), ("weight", C.c_double)]


class Codebook(C.Structure):
    _fields_ = [("type", C.c_int32), ("pad", C.c_int32), ("rank", C.c_size_t), ("n_rows", C.c_size_t),
                ("data", C.c_void_p)]


class AcceptDecision(C.Structure):
    _fields_ = [("n_accepted", C.c_int32), ("accepted_drafts", C.c_int32 * 64), ("carry_kind", C.c_int32),
                ("carry_token", C.c_int32), ("stop_reason", C.c_int32), ("retain_input_count", C.c_int32),
                ("err_row", C.c_int32), ("err_code", C.c_int32), ("err_index", C.c_int64)]

    def accepted(self):
        return list(self.accepted_drafts[: self.n_accepted])

    def key(self):
        return (self.accepted(), self.carry_kind, self.carry_token if self.carry_kind else 0, self.stop_reason,
                self.retain_input_count)


class ModelCfg(C.Structure):
    _fields_ = [(n, C.c_int32) for n in ("n_layers", "hidden", "n_q", "n_kv", "head_dim", "ffn", "vocab",
                                          "n_expert", "n_expert_used", "ffn_expert", "ffn_shared")] + \
               [("eps", C.c_float), ("rope_theta", C.c_float)]


class QTensor(C.Structure):
    _fields_ = [("type", C.c_int32), ("pad", C.c_int32), ("data", C.c_void_p)]


class Layer(C.Structure):
    _fields_ = [("attn_norm", C.c_void_p), ("q_norm", C.c_void_p), ("k_norm", C.c_void_p), ("post_norm", C.c_void_p),
                ("wq", QTensor), ("wk", QTensor), ("wv", QTensor), ("wo", QTensor), ("gate", QTensor), ("up", QTensor),
                ("down", QTensor), ("router", QTensor), ("shexp_gate", C.c_void_p), ("gate_exps", QTensor),
                ("up_exps", QTensor), ("down_exps", QTensor)]


class Model(C.Structure):
    _fields_ = [("cfg", ModelCfg), ("layers", C.POINTER(Layer)), ("token_embd", QTensor), ("output", QTensor),
                ("output_norm", C.c_void_p)]


class DraftCfg(C.Structure):
    _fields_ = [(n, C.c_int32) for n in ("n_layers", "hidden", "n_q", "n_kv", "head_dim", "ffn", "block_size",
                                          "n_taps", "causal")] + \
               [("swa_window", C.c_uint32), ("eps", C.c_float), ("rope_theta", C.c_float)]


class DraftLayer(C.Structure):
    _fields_ = [("attn_norm", C.c_void_p), ("q_norm", C.c_void_p), ("k_norm", C.c_void_p), ("post_norm", C.c_void_p),
                ("wq", QTensor), ("wk", QTensor), ("wv", QTensor), ("wo", QTensor), ("gate", QTensor), ("up", QTensor),
                ("down", QTensor), ("is_swa", C.c_int32), ("pad", C.c_int32)]


class DraftHead(C.Structure):
    _fields_ = [("cfg", DraftCfg), ("layers", C.POINTER(DraftLayer)), ("fc", QTensor), ("hidden_norm", C.c_void_p),
                ("output_norm", C.c_void_p)]


class DFlash2Ext(C.Structure):
    _fields_ = [("conv_kernel_size", C.c_int32), ("conv_group_size", C.c_int32), ("selector_rank", C.c_int32),
                ("pad", C.c_int32), ("conv_attn_proj", C.POINTER(QTensor)), ("conv_ffn_proj", C.POINTER(QTensor)),
                ("conv_attn_base", C.POINTER(C.c_void_p)), ("conv_ffn_base", C.POINTER(C.c_void_p)),
                ("selector_hidden", QTensor)]


_lib = None


def lib() -> C.CDLL:
    global _lib
    if _lib is None:
        build()
        _lib = C.CDLL(_LIB_PATH)
        _declare(_lib)
    return _lib


def _declare(L):
    vp, sz, i32, i64, u64, f32, f64 = C.c_void_p, C.c_size_t, C.c_int32, C.c_int64, C.c_uint64, C.c_float, C.c_double
    L.orc_f16_to_f32.restype = f32
    L.orc_f16_to_f32.argtypes = [C.c_uint16]
    L.orc_f32_to_f16.restype = C.c_uint16
    L.orc_f32_to_f16.argtypes = [f32]
    L.orc_dequant.restype = C.c_int
    L.orc_dequant.argtypes = [C.c_int, vp, sz, vp]
    L.orc_row_bytes.restype = sz
    L.orc_row_bytes.argtypes = [C.c_int, sz]
    L.orc_splitmix64_next.restype = u64
    L.orc_splitmix64_next.argtypes = [C.POINTER(u64)]
    L.orc_xoshiro_seed.argtypes = [u64, C.POINTER(u64)]
    L.orc_xoshiro_next.restype = u64
    L.orc_xoshiro_next.argtypes = [C.POINTER(u64)]
    L.orc_unit_f64.restype = f64
    L.orc_unit_f64.argtypes = [u64]
    L.orc_philox4x32_10.argtypes = [C.POINTER(C.c_uint32), C.POINTER(C.c_uint32), C.POINTER(C.c_uint32)]
    L.orc_sampler_init.argtypes = [C.POINTER(Sampler), C.POINTER(SamplingConfig)]
    L.orc_sampler_at_draw.argtypes = [C.POINTER(Sampler), C.POINTER(SamplingConfig), u64]
    L.orc_sampler_next_unit.restype = f64
    L.orc_sampler_next_unit.argtypes = [C.POINTER(Sampler)]
    L.orc_greedy_token.argtypes = [vp, sz, C.POINTER(i32), C.POINTER(i64)]
    L.orc_argmax_top2.argtypes = [vp, sz, C.POINTER(i32), C.POINTER(f32)]
    L.orc_top16.argtypes = [vp, sz, vp, vp]
    L.orc_sampler_diagnose.argtypes = [C.POINTER(Sampler), vp, sz, f64, C.POINTER(WeightedCandidate), sz,
                                       C.POINTER(sz), C.POINTER(f64), C.POINTER(i32), C.POINTER(sz), C.POINTER(i64)]
    L.orc_sampler_sample.argtypes = [C.POINTER(Sampler), vp, sz, C.POINTER(i32), C.POINTER(sz), C.POINTER(i64)]
    L.orc_couple_deterministic_proposal.argtypes = [C.POINTER(Sampler), vp, sz, i32, C.POINTER(C.c_int),
                                                    C.POINTER(i32), C.POINTER(i64)]
    L.orc_couple_sparse_proposal.argtypes = [C.POINTER(Sampler), vp, sz, i32, C.POINTER(WeightedCandidate), sz,
                                             C.POINTER(C.c_int), C.POINTER(i32), C.POINTER(i64)]
    L.orc_couple_dense_proposal.argtypes = [C.POINTER(Sampler), vp, vp, sz, f32, i32, C.POINTER(C.c_int),
                                            C.POINTER(i32), C.POINTER(i64)]
    L.orc_dense_proposal_total.restype = f64
    L.orc_dense_proposal_total.argtypes = [vp, sz, f32, C.POINTER(i64)]
    L.orc_decide_accept_prefix.argtypes = [vp, sz, vp, sz, sz, C.c_int, sz, vp, vp, vp, vp, C.POINTER(Sampler), sz,
                                           vp, sz, C.POINTER(AcceptDecision)]
    L.orc_decide_accept_prefix_dense.argtypes = [vp, sz, vp, vp, sz, f32, C.POINTER(Sampler), sz, vp, sz,
                                                 C.POINTER(AcceptDecision)]
    L.orc_decide_accept_prefix_batch.restype = None
    L.orc_decide_accept_prefix_batch.argtypes = [sz, vp, sz, vp, vp, sz, f32, vp, sz, vp, vp]
    L.orc_router_margin_take.restype = f32
    L.orc_router_margin_take.argtypes = []
    L.orc_rms_norm.argtypes = [vp, vp, sz, f32, vp]
    L.orc_silu.restype = f32
    L.orc_silu.argtypes = [f32]
    L.orc_softmax_in_place.argtypes = [vp, sz]
    L.orc_mat_vec.argtypes = [vp, sz, sz, vp, vp]
    L.orc_rope_in_place.argtypes = [vp, sz, sz, sz, C.c_uint32, f32]
    L.orc_gemm_fewrow.argtypes = [C.c_int, vp, vp, vp, sz, sz, sz]
    L.orc_attn_verify_block.argtypes = [vp, vp, vp, sz, sz, sz, sz, sz, f32, vp]
    L.orc_attn_draft.argtypes = [vp, vp, vp, vp, vp, vp, sz, sz, sz, sz, sz, C.c_uint32, C.c_int, C.c_uint32, vp]
    L.orc_target_verify.argtypes = [C.POINTER(Model), vp, sz, sz, vp, vp, sz, vp, vp, sz, vp]
    L.orc_dflash_draft.argtypes = [C.POINTER(Model), C.POINTER(DraftHead), vp, vp, sz, vp, C.c_uint32, vp]
    L.orc_dflash_draft_ex.restype = C.c_int
    L.orc_dflash_draft_ex.argtypes = [C.POINTER(Model), C.POINTER(DraftHead), C.POINTER(DFlash2Ext), vp, vp, sz, vp,
                                      C.c_uint32, vp, vp]
    L.orc_dflash2_conv.argtypes = [vp, vp, vp, vp, sz, sz, sz, sz, sz]
    L.orc_dflash2_conv.restype = None
    L.orc_codebook_row.argtypes = [C.POINTER(Codebook), sz, vp]
    L.orc_select_draft_path.argtypes = [C.POINTER(Codebook), C.POINTER(Codebook), sz, sz, i32, sz, vp, vp, vp, vp, vp, vp]
    L.orc_select_draft_path_sampled.argtypes = [C.POINTER(Codebook), C.POINTER(Codebook), sz, sz, i32, sz, vp, vp, vp,
                                                C.POINTER(Sampler), vp, vp, C.POINTER(WeightedCandidate), C.POINTER(sz)]


def _p(a: np.ndarray):
    return a.ctypes.data_as(C.c_void_p)


# ---------------------------------------------------------------- numpy-level helpers


def row_bytes(qtype: int, n_in: int) -> int:
    return int(lib().orc_row_bytes(qtype, n_in))


def dequant(qtype: int, blocks: np.ndarray, n_elems: int) -> np.ndarray:
    blocks = np.ascontiguousarray(blocks, dtype=np.uint8)
    out = np.empty(n_elems, dtype=np.float32)
    rc = lib().orc_dequant(qtype, _p(blocks), n_elems, _p(out))
    if rc:
        raise ValueError("orc_dequant: bad geometry")
    return out


def gemm_fewrow(qtype: int, w: np.ndarray, x: np.ndarray, n_in: int, n_out: int) -> np.ndarray:
    w = np.ascontiguousarray(w, dtype=np.uint8)
    x = np.ascontiguousarray(x, dtype=np.float32)
    n_rows = x.shape[0]
    y = np.empty((n_rows, n_out), dtype=np.float32)
    rc = lib().orc_gemm_fewrow(qtype, _p(w), _p(x), _p(y), n_in, n_out, n_rows)
    if rc:
        raise ValueError("orc_gemm_fewrow failed")
    return y


def attn_verify_block(q, k_cache, v_cache, ctx_len, scale):
    """q [n_rows,n_q,hd] f32; k/v cache [ctx_len+n_rows, n_kv, hd] float16."""
    q = np.ascontiguousarray(q, dtype=np.float32)
    k = np.ascontiguousarray(k_cache, dtype=np.float16)
    v = np.ascontiguousarray(v_cache, dtype=np.float16)
    n_rows, n_q, hd = q.shape
    n_kv = k.shape[1]
    out = np.empty_like(q)
    lib().orc_attn_verify_block(_p(q), _p(k), _p(v), ctx_len, n_rows, n_q, n_kv, hd, scale, _p(out))
    return out


def attn_draft(q, k_ctx, v_ctx, k_noise, v_noise, pos_ctx, noise_start_pos, causal, swa_window):
    q = np.ascontiguousarray(q, dtype=np.float32)
    n, n_q, hd = q.shape
    k_ctx = np.ascontiguousarray(k_ctx, dtype=np.float32)
    v_ctx = np.ascontiguousarray(v_ctx, dtype=np.float32)
    k_noise = np.ascontiguousarray(k_noise, dtype=np.float32)
    v_noise = np.ascontiguousarray(v_noise, dtype=np.float32)
    pos_ctx = np.ascontiguousarray(pos_ctx, dtype=np.int32)
    n_kv = k_noise.shape[1]
    out = np.empty_like(q)
    lib().orc_attn_draft(_p(q), _p(k_ctx), _p(v_ctx), _p(k_noise), _p(v_noise), _p(pos_ctx), len(pos_ctx), n, n_q,
                         n_kv, hd, noise_start_pos, int(causal), swa_window, _p(out))
    return out


def make_sampler(temperature=0.0, top_k=0, top_p=1.0, min_p=0.0, seed=0, rng_kind=RNG_XOSHIRO, draws=0):
    cfg = SamplingConfig(temperature, top_p, min_p, rng_kind, top_k, seed)
    s = Sampler()
    rc = lib().orc_sampler_at_draw(C.byref(s), C.byref(cfg), draws)
    if rc:
        raise ValueError(ERR[rc])
    return s


def clone_sampler(s: Sampler) -> Sampler:
    t = Sampler()
    C.memmove(C.byref(t), C.byref(s), C.sizeof(Sampler))
    return t


def sampler_state(s: Sampler):
    return (tuple(s.s), int(s.draws))


def greedy_token(logits):
    logits = np.ascontiguousarray(logits, dtype=np.float32)
    tok, err = C.c_int32(), C.c_int64(-1)
    rc = lib().orc_greedy_token(_p(logits), logits.size, C.byref(tok), C.byref(err))
    return rc, tok.value, err.value


def argmax_top2(logits):
    logits = np.ascontiguousarray(logits, dtype=np.float32)
    idx, gap = C.c_int32(), C.c_float()
    lib().orc_argmax_top2(_p(logits), logits.size, C.byref(idx), C.byref(gap))
    return idx.value, gap.value


def top16(logits):
    logits = np.ascontiguousarray(logits, dtype=np.float32)
    ids = np.empty(16, dtype=np.int32)
    vals = np.empty(16, dtype=np.float32)
    lib().orc_top16(_p(logits), logits.size, _p(ids), _p(vals))
    return ids, vals


def sample(s: Sampler, logits):
    logits = np.ascontiguousarray(logits, dtype=np.float32)
    tok, idx, err = C.c_int32(), C.c_size_t(), C.c_int64(-1)
    rc = lib().orc_sampler_sample(C.byref(s), _p(logits), logits.size, C.byref(tok), C.byref(idx), C.byref(err))
    return rc, tok.value, idx.value, err.value


def diagnose(s: Sampler, logits, uniform=0.0, cap=None):
    logits = np.ascontiguousarray(logits, dtype=np.float32)
    cap = cap or logits.size
    cands = (WeightedCandidate * cap)()
    n, total, tok, idx, err = C.c_size_t(), C.c_double(), C.c_int32(), C.c_size_t(), C.c_int64(-1)
    rc = lib().orc_sampler_diagnose(C.byref(s), _p(logits), logits.size, uniform, cands, cap, C.byref(n),
                                    C.byref(total), C.byref(tok), C.byref(idx), C.byref(err))
    if rc:
        return rc, [], 0.0, -1, err.value
    return rc, [(cands[i].token, cands[i].weight) for i in range(min(n.value, cap))], total.value, tok.value, idx.value


def _cands(pairs):
    arr = (WeightedCandidate * max(1, len(pairs)))()
    for i, (t, w) in enumerate(pairs):
        arr[i].token, arr[i].weight = t, w
    return arr


def couple_deterministic(s, logits, proposal):
    logits = np.ascontiguousarray(logits, dtype=np.float32)
    acc, corr, err = C.c_int(), C.c_int32(), C.c_int64(-1)
    rc = lib().orc_couple_deterministic_proposal(C.byref(s), _p(logits), logits.size, proposal, C.byref(acc),
                                                 C.byref(corr), C.byref(err))
    return rc, bool(acc.value), corr.value


def couple_sparse(s, logits, token, pairs):
    logits = np.ascontiguousarray(logits, dtype=np.float32)
    acc, corr, err = C.c_int(), C.c_int32(), C.c_int64(-1)
    rc = lib().orc_couple_sparse_proposal(C.byref(s), _p(logits), logits.size, token, _cands(pairs), len(pairs),
                                          C.byref(acc), C.byref(corr), C.byref(err))
    return rc, bool(acc.value), corr.value


def couple_dense(s, target_logits, draft_logits, draft_temperature, token):
    t = np.ascontiguousarray(target_logits, dtype=np.float32)
    d = np.ascontiguousarray(draft_logits, dtype=np.float32)
    acc, corr, err = C.c_int(), C.c_int32(), C.c_int64(-1)
    rc = lib().orc_couple_dense_proposal(C.byref(s), _p(t), _p(d), t.size, draft_temperature, token, C.byref(acc),
                                         C.byref(corr), C.byref(err))
    return rc, bool(acc.value), corr.value


def decide_accept_prefix(verified_tokens, target_logits, vocab, proposals, sampler, budget, stop_ids):
    """proposals: None or list of (token, [(token, weight), ...]) with one entry per draft row."""
    toks = np.ascontiguousarray(verified_tokens, dtype=np.int32)
    logits = np.ascontiguousarray(target_logits, dtype=np.float32)
    stops = np.ascontiguousarray(stop_ids, dtype=np.int32)
    out = AcceptDecision()
    if proposals is None:
        rc = lib().orc_decide_accept_prefix(_p(toks), toks.size, _p(logits), logits.size, vocab, 0, 0, None, None,
                                            None, None, C.byref(sampler), budget, _p(stops), stops.size,
                                            C.byref(out))
        return rc, out
    ptoks = np.array([p[0] for p in proposals], dtype=np.int32)
    counts = np.array([len(p[1]) for p in proposals], dtype=np.uint64)
    offsets = np.concatenate([[0], np.cumsum(counts)[:-1]]).astype(np.uint64) if len(proposals) else \
        np.zeros(0, dtype=np.uint64)
    flat = [c for p in proposals for c in p[1]]
    rc = lib().orc_decide_accept_prefix(_p(toks), toks.size, _p(logits), logits.size, vocab, 1, len(proposals),
                                        _p(ptoks), _p(offsets), _p(counts), _cands(flat), C.byref(sampler), budget,
                                        _p(stops), stops.size, C.byref(out))
    return rc, out


def decide_accept_prefix_dense(verified_tokens, target_logits, draft_logits, vocab, draft_temperature, sampler,
                               budget, stop_ids):
    toks = np.ascontiguousarray(verified_tokens, dtype=np.int32)
    t = np.ascontiguousarray(target_logits, dtype=np.float32)
    d = np.ascontiguousarray(draft_logits, dtype=np.float32)
    stops = np.ascontiguousarray(stop_ids, dtype=np.int32)
    out = AcceptDecision()
    rc = lib().orc_decide_accept_prefix_dense(_p(toks), toks.size, _p(t), _p(d), vocab, draft_temperature,
                                              C.byref(sampler), budget, _p(stops), stops.size, C.byref(out))
    return rc, out


def decide_accept_prefix_batch(verified_tokens, target_logits, draft_logits, draft_temperature, samplers, budget):
    """verified_tokens [trials, n]; target_logits [trials, n, vocab]; draft_logits [trials, n-1, vocab] or None;
    samplers: list of Sampler (advanced in place).  Returns (status list, list of AcceptDecision)."""
    toks = np.ascontiguousarray(verified_tokens, dtype=np.int32)
    t = np.ascontiguousarray(target_logits, dtype=np.float32)
    d = None if draft_logits is None else np.ascontiguousarray(draft_logits, dtype=np.float32)
    n_trials, n = toks.shape
    arr = (Sampler * n_trials)(*samplers)
    outs = (AcceptDecision * n_trials)()
    status = np.zeros(n_trials, np.int32)
    lib().orc_decide_accept_prefix_batch(n_trials, _p(toks), n, _p(t), _p(d) if d is not None else None, t.shape[2],
                                         draft_temperature, arr, budget, outs, _p(status))
    for i in range(n_trials):
        C.memmove(C.byref(samplers[i]), C.byref(arr[i]), C.sizeof(Sampler))
    return status.tolist(), list(outs)


# ---- synthetic decoder / drafter (plain dictionaries of numpy arrays in, numpy out) ----

class _Keep:
    """Owns the numpy buffers a ctypes descriptor points into."""

    def __init__(self):
        self.bufs = []

    def f32(self, a):
        a = np.ascontiguousarray(a, dtype=np.float32)
        self.bufs.append(a)
        return a.ctypes.data

    def q(self, pair):
        if pair is None:
            return QTensor(0, 0, None)
        qtype, blocks = pair
        b = np.ascontiguousarray(blocks, dtype=np.uint8)
        self.bufs.append(b)
        return QTensor(int(qtype), 0, b.ctypes.data)


def build_model(cfg: dict, weights: dict):
    """cfg: the dflash_model_cfg fields by name; weights: {'token_embd': (type, blocks), 'output', 'output_norm',
    'layers': [{'attn_norm', 'q_norm', 'k_norm', 'post_norm', 'wq', ... }]}.  Returns (Model, keepalive)."""
    keep = _Keep()
    layers = (Layer * cfg["n_layers"])()
    for il, Lw in enumerate(weights["layers"]):
        L = layers[il]
        for k in ("attn_norm", "q_norm", "k_norm", "post_norm"):
            setattr(L, k, keep.f32(Lw[k]))
        for k in ("wq", "wk", "wv", "wo", "gate", "up", "down", "router", "gate_exps", "up_exps", "down_exps"):
            setattr(L, k, keep.q(Lw.get(k)))
        L.shexp_gate = keep.f32(Lw["shexp_gate"]) if "shexp_gate" in Lw else None
    m = Model(ModelCfg(**cfg), layers, keep.q(weights["token_embd"]), keep.q(weights["output"]),
              keep.f32(weights["output_norm"]))
    keep.bufs.append(layers)
    return m, keep


def build_draft_head(cfg: dict, weights: dict):
    keep = _Keep()
    layers = (DraftLayer * cfg["n_layers"])()
    for il, Lw in enumerate(weights["layers"]):
        L = layers[il]
        for k in ("attn_norm", "q_norm", "k_norm", "post_norm"):
            setattr(L, k, keep.f32(Lw[k]))
        for k in ("wq", "wk", "wv", "wo", "gate", "up", "down"):
            setattr(L, k, keep.q(Lw[k]))
        L.is_swa = int(Lw.get("is_swa", 0))
    known = {n for n, _ in DraftCfg._fields_}
    h = DraftHead(DraftCfg(**{k: v for k, v in cfg.items() if k in known}), layers, keep.q(weights["fc"]),
                  keep.f32(weights["hidden_norm"]), keep.f32(weights["output_norm"]))
    keep.bufs.append(layers)
    return h, keep


def build_dflash2_ext(cfg: dict, weights: dict):
    """The DFlash-2 additions of a drafter: cfg carries conv_kernel_size / conv_group_size / selector_rank, every
    layer 'conv_attn_proj', 'conv_ffn_proj' ((type, blocks), [2*kernel*H/group rows][H]) and 'conv_attn_base',
    'conv_ffn_base' (f32 [2][kernel][H]); the head 'selector_hidden' ((type, blocks), [rank rows][H]).
    Returns (DFlash2Ext, keepalive)."""
    keep = _Keep()
    n = cfg["n_layers"]
    ap, fp = (QTensor * n)(), (QTensor * n)()
    ab, fb = (C.c_void_p * n)(), (C.c_void_p * n)()
    for il, Lw in enumerate(weights["layers"]):
        ap[il], fp[il] = keep.q(Lw["conv_attn_proj"]), keep.q(Lw["conv_ffn_proj"])
        ab[il], fb[il] = keep.f32(Lw["conv_attn_base"]), keep.f32(Lw["conv_ffn_base"])
    ext = DFlash2Ext(cfg["conv_kernel_size"], cfg["conv_group_size"], cfg["selector_rank"], 0, ap, fp, ab, fb,
                     keep.q(weights["selector_hidden"]))
    keep.bufs += [ap, fp, ab, fb]
    return ext, keep


def dflash_draft_ex(target: Model, head: DraftHead, ext: DFlash2Ext, noise_ids, ctx_stacked, pos_ctx, noise_start_pos: int):
    """The DFlash-2 drafter forward: returns (logits [block, V], sel_h [block, selector_rank])."""
    ids = np.asarray(noise_ids, np.int32)
    ctx_stacked = np.ascontiguousarray(ctx_stacked, dtype=np.float32)
    pos = np.asarray(pos_ctx if len(pos_ctx) else [0], np.int32)
    logits = np.zeros((head.cfg.block_size, target.cfg.vocab), np.float32)
    sel_h = np.zeros((head.cfg.block_size, max(ext.selector_rank, 1)), np.float32)
    rc = lib().orc_dflash_draft_ex(C.byref(target), C.byref(head), C.byref(ext), _p(ids), _p(ctx_stacked), len(pos_ctx),
                                   _p(pos), noise_start_pos, _p(logits), _p(sel_h))
    if rc:
        raise RuntimeError(f"orc_dflash_draft_ex failed: {rc}")
    return logits, sel_h


class TargetState:
    """KV cache of the CPU target: f16 bits [layer][capacity][n_kv*head_dim]."""

    def __init__(self, cfg: dict, capacity: int):
        kv_dim = cfg["n_kv"] * cfg["head_dim"]
        self.capacity = capacity
        self.k = np.zeros((cfg["n_layers"], capacity, kv_dim), np.uint16)
        self.v = np.zeros((cfg["n_layers"], capacity, kv_dim), np.uint16)


def target_verify(model: Model, state: TargetState, tokens, start_pos: int, tap_layers=()):
    """Token-by-token forward of tokens at start_pos..; returns (logits [n, V], hidden [n, n_taps, H])."""
    c = model.cfg
    n = len(tokens)
    toks = np.asarray(tokens, np.int32)
    taps = np.asarray(list(tap_layers) or [0], np.int32)
    logits = np.zeros((n, c.vocab), np.float32)
    hidden = np.zeros((n, max(len(tap_layers), 1), c.hidden), np.float32)
    rc = lib().orc_target_verify(C.byref(model), _p(toks), n, start_pos, _p(state.k), _p(state.v), state.capacity,
                                 _p(logits), _p(taps), len(tap_layers), _p(hidden))
    if rc:
        raise RuntimeError(f"orc_target_verify failed: {rc}")
    return logits, hidden[:, :len(tap_layers)]


def router_margin_take() -> float:
    """Smallest relative gap between the last expert picked and the best one left out over every routing decision
    since the previous call (inf if there was none)."""
    return float(lib().orc_router_margin_take())


def dflash_draft(target: Model, head: DraftHead, noise_ids, ctx_stacked, pos_ctx, noise_start_pos: int):
    """ctx_stacked [ctx_len, n_taps*hidden]; returns logits [block, V]."""
    ids = np.asarray(noise_ids, np.int32)
    ctx_stacked = np.ascontiguousarray(ctx_stacked, dtype=np.float32)
    pos = np.asarray(pos_ctx if len(pos_ctx) else [0], np.int32)
    logits = np.zeros((head.cfg.block_size, target.cfg.vocab), np.float32)
    rc = lib().orc_dflash_draft(C.byref(target), C.byref(head), _p(ids), _p(ctx_stacked), len(pos_ctx), _p(pos),
                                noise_start_pos, _p(logits))
    if rc:
        raise RuntimeError(f"orc_dflash_draft failed: {rc}")
    return logits


# ---- DFlash-2 extras ----
F32, F16 = 0, 1


def dflash2_conv(x, dyn, base, kernel_size: int, group_size: int, side: int) -> np.ndarray:
    """x [n_tokens][h], dyn [n_tokens][2*kernel_size*h/group_size], base [2][kernel_size][h] -> y [n_tokens][h]."""
    x = np.ascontiguousarray(x, np.float32)
    dyn = np.ascontiguousarray(dyn, np.float32)
    base = np.ascontiguousarray(base, np.float32)
    n, h = x.shape
    y = np.empty_like(x)
    lib().orc_dflash2_conv(x.ctypes.data, dyn.ctypes.data, base.ctypes.data, y.ctypes.data, n, h, kernel_size, group_size, side)
    return y


def make_codebook(qtype: int, rows: np.ndarray, rank: int):
    """rows: [n_rows][row bytes] uint8 (quantised types) or [n_rows][rank] float32/float16.  Returns (Codebook, keepalive)."""
    rows = np.ascontiguousarray(rows)
    return Codebook(qtype, 0, rank, rows.shape[0], rows.ctypes.data), rows


def codebook_row(cb, row: int) -> np.ndarray:
    out = np.empty(cb.rank, np.float32)
    if lib().orc_codebook_row(C.byref(cb), row, out.ctypes.data):
        raise ValueError("selector codebook row out of range")
    return out


def select_draft_path(pred_cb, succ_cb, top_k: int, rank: int, carry: int, n: int, ids, vals, sel_h):
    """Returns (tokens [n], scores [n][top_k], valid [n][top_k]); raises ValueError on an invalid predecessor row."""
    ids = np.ascontiguousarray(ids, np.int32)
    vals = np.ascontiguousarray(vals, np.float32)
    sel_h = np.ascontiguousarray(sel_h, np.float32)
    out = np.zeros(n, np.int32)
    scores = np.full((n, top_k), np.nan, np.float32)
    valid = np.zeros((n, top_k), np.uint8)
    rc = lib().orc_select_draft_path(C.byref(pred_cb), C.byref(succ_cb), top_k, rank, carry, n, ids.ctypes.data,
                                     vals.ctypes.data, sel_h.ctypes.data, out.ctypes.data, scores.ctypes.data,
                                     valid.ctypes.data)
    if rc:
        raise ValueError("selector codebook row out of range")
    return out, scores, valid


def select_draft_path_sampled(pred_cb, succ_cb, top_k: int, rank: int, carry: int, n: int, ids, vals, sel_h, proposal: Sampler):
    """Returns (rc, tokens [n], proposals: one [(token, weight), ...] per position 1..n-1, err_pos); advances `proposal`."""
    ids = np.ascontiguousarray(ids, np.int32)
    vals = np.ascontiguousarray(vals, np.float32)
    sel_h = np.ascontiguousarray(sel_h, np.float32)
    out = np.zeros(n, np.int32)
    counts = np.zeros(max(n - 1, 1), np.int32)
    cands = (WeightedCandidate * (max(n - 1, 1) * top_k))()
    err_pos = C.c_size_t(0)
    rc = lib().orc_select_draft_path_sampled(C.byref(pred_cb), C.byref(succ_cb), top_k, rank, carry, n, ids.ctypes.data,
                                             vals.ctypes.data, sel_h.ctypes.data, C.byref(proposal), out.ctypes.data,
                                             counts.ctypes.data, cands, C.byref(err_pos))
    props = [[(cands[p * top_k + i].token, cands[p * top_k + i].weight) for i in range(counts[p])] for p in range(n - 1)]
    return rc, out, props, err_pos.value
