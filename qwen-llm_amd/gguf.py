"""GGUF files: the reader of the library (``dflash_gguf_*``), the drafter and target loaders on top of it, and a
writer for exporting synthetic models.

Mirrors ``GgufFile`` (crates/qwen-llm/src/gguf.rs:129-740), ``open_dflash_drafter_for_target``
(crates/qwen-llm/src/loader.rs:832-1290) and the tensor naming of the target loader (loader.rs:436-500, 595-612).
Reading, validation and the drafter's binding run in the library; this module only wraps the handles, turns mapped
tensors into numpy views (no copy) and assembles the weight dictionaries ``TargetModel`` / ``DraftHead`` take.
"""
from __future__ import annotations

import ctypes as C
import struct

import numpy as np

from .binding import DFlashError, lib
from .model import DraftCfgC, DraftConfig, ModelConfig

GGUF_MAGIC = 0x46554747
# ggml type ids the kernels take (the same numbers as DFLASH_TYPE_*)
F32, F16, Q8_0, Q4_K, Q6_K = 0, 1, 8, 12, 14
KERNEL_TYPES = (F32, F16, Q8_0, Q4_K, Q6_K)
# metadata value types
_U8, _I8, _U16, _I16, _U32, _I32, _F32, _BOOL, _STR, _ARR, _U64, _I64, _F64 = range(13)
MAX_TAPS = 64


class GgufTensorC(C.Structure):
    _fields_ = [("type", C.c_int32), ("n_dims", C.c_int32), ("shape", C.c_uint64 * 4), ("n_bytes", C.c_uint64),
                ("data_host", C.c_void_p)]


class TargetShapeC(C.Structure):
    _fields_ = [("hidden_size", C.c_uint32), ("vocab_size", C.c_uint32), ("n_layer", C.c_uint32)]


_LAYER_TENSORS = ("attn_norm", "wq", "wk", "wv", "wo", "q_norm", "k_norm", "post_norm", "gate", "up", "down",
                  "conv_attn_base", "conv_attn_proj", "conv_ffn_base", "conv_ffn_proj")


class GgufDraftLayerC(C.Structure):
    _fields_ = [(n, GgufTensorC) for n in _LAYER_TENSORS] + [("is_swa", C.c_int32), ("pad", C.c_int32)]


class GgufDraftHeadC(C.Structure):
    _fields_ = [("cfg", DraftCfgC), ("mask_token_id", C.c_int32), ("convention", C.c_int32), ("n_target_layers", C.c_int32),
                ("target_layer_ids", C.c_int32 * MAX_TAPS), ("fc", GgufTensorC), ("hidden_norm", GgufTensorC),
                ("output_norm", GgufTensorC), ("selector_hidden", GgufTensorC), ("selector_predecessor", GgufTensorC),
                ("selector_successor", GgufTensorC)]


_declared = False


def gguf_lib():
    """The library with the reader's signatures declared (host code only; no GPU needed)."""
    global _declared
    L = lib()
    if not _declared:
        vp, cp, i32, i64, u64 = C.c_void_p, C.c_char_p, C.c_int32, C.c_int64, C.c_uint64
        tp = C.POINTER(GgufTensorC)
        for name, res, args in (
                ("dflash_gguf_open", i32, [cp, C.POINTER(vp), cp, C.c_size_t]), ("dflash_gguf_close", None, [vp]),
                ("dflash_gguf_last_error", cp, [vp]), ("dflash_gguf_tensor_count", i64, [vp]),
                ("dflash_gguf_shard_count", i64, [vp]),
                ("dflash_gguf_kv_count", i64, [vp]), ("dflash_gguf_alignment", u64, [vp]),
                ("dflash_gguf_data_start", u64, [vp]),
                ("dflash_gguf_tensor_at", i32, [vp, i64, C.POINTER(cp), tp]), ("dflash_gguf_find", i32, [vp, cp, tp]),
                ("dflash_gguf_get_u64", i32, [vp, cp, C.POINTER(u64)]),
                ("dflash_gguf_get_f64", i32, [vp, cp, C.POINTER(C.c_double)]),
                ("dflash_gguf_get_bool", i32, [vp, cp, C.POINTER(i32)]),
                ("dflash_gguf_get_str", i32, [vp, cp, C.POINTER(C.POINTER(C.c_char)), C.POINTER(u64)]),
                ("dflash_gguf_get_u64_array", i64, [vp, cp, C.POINTER(u64), i64]),
                ("dflash_gguf_get_bool_array", i64, [vp, cp, C.POINTER(C.c_uint8), i64]),
                ("dflash_gguf_get_f64_array", i64, [vp, cp, C.POINTER(C.c_double), i64]),
                ("dflash_gguf_open_drafter", i32, [vp, C.POINTER(TargetShapeC), C.POINTER(GgufDraftHeadC),
                                                   C.POINTER(GgufDraftLayerC), i32])):
            f = getattr(L, name)
            f.restype, f.argtypes = res, args
        _declared = True
    return L


class GgufTensor:
    """One tensor of an open file: ggml type, shape (fastest dimension first) and a view of its bytes."""

    def __init__(self, name: str, c: GgufTensorC, owner):
        self.name, self.type, self.n_bytes = name, int(c.type), int(c.n_bytes)
        self.shape = tuple(int(c.shape[i]) for i in range(c.n_dims))
        self._ptr, self._owner = c.data_host, owner

    def bytes(self) -> np.ndarray:
        """uint8 view into the mapping (valid while the file is open; copy before closing)."""
        if self._owner._h is None:
            raise DFlashError(10, f"tensor {self.name}: the file is closed")
        buf = (C.c_uint8 * self.n_bytes).from_address(self._ptr)
        a = np.frombuffer(buf, dtype=np.uint8)
        a.flags.writeable = False
        return a

    def f32(self) -> np.ndarray:
        if self.type != F32:
            raise DFlashError(2, f"tensor {self.name} is not F32 (type {self.type})")
        return self.bytes().view(np.float32).reshape(self.shape[::-1])


class GgufFile:
    """GgufFile::open (gguf.rs:154): a validated read-only mapping of one GGUF v3 file, or of all shards of a split
    model opened by its first shard (the metadata is the first shard's, the tensor table every shard's)."""

    def __init__(self, path: str):
        self._L = gguf_lib()
        self._h = None
        h = C.c_void_p()
        err = C.create_string_buffer(512)
        rc = self._L.dflash_gguf_open(str(path).encode(), C.byref(h), err, len(err))
        if rc:
            raise DFlashError(rc, err.value.decode(errors="replace"))
        self._h = h
        self.path = str(path)

    def close(self):
        if getattr(self, "_h", None):
            self._L.dflash_gguf_close(self._h)
            self._h = None

    __del__ = close

    def __enter__(self):
        return self

    def __exit__(self, *a):
        self.close()

    def _error(self, rc):
        return DFlashError(rc, self._L.dflash_gguf_last_error(self._h).decode(errors="replace"))

    @property
    def tensor_count(self) -> int:
        return int(self._L.dflash_gguf_tensor_count(self._h))

    @property
    def shard_count(self) -> int:
        return int(self._L.dflash_gguf_shard_count(self._h))

    @property
    def kv_count(self) -> int:
        return int(self._L.dflash_gguf_kv_count(self._h))

    @property
    def alignment(self) -> int:
        return int(self._L.dflash_gguf_alignment(self._h))

    @property
    def data_start(self) -> int:
        return int(self._L.dflash_gguf_data_start(self._h))

    def tensors(self):
        out = []
        for i in range(self.tensor_count):
            name, c = C.c_char_p(), GgufTensorC()
            rc = self._L.dflash_gguf_tensor_at(self._h, i, C.byref(name), C.byref(c))
            if rc:
                raise self._error(rc)
            out.append(GgufTensor(name.value.decode(), c, self))
        return out

    def find(self, name: str):
        c = GgufTensorC()
        if not self._L.dflash_gguf_find(self._h, name.encode(), C.byref(c)):
            return None
        return GgufTensor(name, c, self)

    def get_u64(self, key: str):
        v = C.c_uint64()
        return int(v.value) if self._L.dflash_gguf_get_u64(self._h, key.encode(), C.byref(v)) else None

    def get_f64(self, key: str):
        v = C.c_double()
        return float(v.value) if self._L.dflash_gguf_get_f64(self._h, key.encode(), C.byref(v)) else None

    def get_bool(self, key: str):
        v = C.c_int32()
        return bool(v.value) if self._L.dflash_gguf_get_bool(self._h, key.encode(), C.byref(v)) else None

    def get_str(self, key: str):
        p, n = C.POINTER(C.c_char)(), C.c_uint64()
        if not self._L.dflash_gguf_get_str(self._h, key.encode(), C.byref(p), C.byref(n)):
            return None
        return C.string_at(p, n.value).decode(errors="replace")

    def architecture(self):
        return self.get_str("general.architecture")

    def _array(self, fn, ctype, key):
        n = fn(self._h, key.encode(), None, 0)
        if n == -1:
            return None
        if n < 0:
            raise DFlashError(12, f"metadata key {key!r} is not an array of the requested kind")
        buf = (ctype * max(int(n), 1))()
        fn(self._h, key.encode(), buf, n)
        return list(buf[: int(n)])

    def get_u64_array(self, key: str):
        return self._array(self._L.dflash_gguf_get_u64_array, C.c_uint64, key)

    def get_bool_array(self, key: str):
        a = self._array(self._L.dflash_gguf_get_bool_array, C.c_uint8, key)
        return None if a is None else [bool(x) for x in a]

    def get_f64_array(self, key: str):
        return self._array(self._L.dflash_gguf_get_f64_array, C.c_double, key)


# ---- loaders ----

def _pair(t: GgufTensor, what: str):
    """(type, block bytes as [n_out][row bytes]) of a matrix the kernels can read."""
    if t.type not in KERNEL_TYPES:
        raise DFlashError(2, f"{what} ({t.name}): ggml type {t.type} has no kernel (F32, F16, Q8_0, Q4_K, Q6_K do)")
    rows = int(np.prod(t.shape[1:])) if len(t.shape) > 1 else 1
    return (t.type, t.bytes().reshape(rows, -1))


def _from_c(name: str, c: GgufTensorC, owner) -> GgufTensor:
    return GgufTensor(name, c, owner)


def open_dflash_drafter(gguf: GgufFile, target_hidden: int, target_vocab: int, target_n_layer: int):
    """open_dflash_drafter_for_target (loader.rs:832): returns (DraftConfig, weights, target_layer_ids, mask_token_id).
    ``weights`` is the dictionary ``DraftHead`` takes; its arrays are views into the mapping (``DraftHead`` copies them
    to the device, after which the file may be closed)."""
    L = gguf_lib()
    head = GgufDraftHeadC()
    cap = 4096
    layers = (GgufDraftLayerC * cap)()
    shape = TargetShapeC(target_hidden, target_vocab, target_n_layer)
    rc = L.dflash_gguf_open_drafter(gguf._h, C.byref(shape), C.byref(head), layers, cap)
    if rc:
        raise gguf._error(rc)
    cfg = DraftConfig(**{f: getattr(head.cfg, f) for f, _ in DraftCfgC._fields_})
    w = {"fc": _pair(_from_c("fc", head.fc, gguf), "fc"), "hidden_norm": _from_c("hidden_norm", head.hidden_norm, gguf).f32(),
         "output_norm": _from_c("output_norm", head.output_norm, gguf).f32(), "layers": []}
    for il in range(cfg.n_layers):
        Lc = layers[il]
        Lw = {"is_swa": int(Lc.is_swa)}
        for k in ("attn_norm", "q_norm", "k_norm", "post_norm"):
            Lw[k] = _from_c(f"blk.{il}.{k}", getattr(Lc, k), gguf).f32()
        for k in ("wq", "wk", "wv", "wo", "gate", "up", "down"):
            Lw[k] = _pair(_from_c(f"blk.{il}.{k}", getattr(Lc, k), gguf), k)
        if cfg.conv_kernel_size:
            for k in ("conv_attn_proj", "conv_ffn_proj"):
                Lw[k] = _pair(_from_c(f"blk.{il}.{k}", getattr(Lc, k), gguf), k)
            for k in ("conv_attn_base", "conv_ffn_base"):  # [hidden, kernel, 2] fastest-first = f32 [2][kernel][hidden]
                Lw[k] = _from_c(f"blk.{il}.{k}", getattr(Lc, k), gguf).f32()
        w["layers"].append(Lw)
    if cfg.selector_rank:
        for k in ("selector_hidden", "selector_predecessor", "selector_successor"):
            w[k] = _pair(_from_c(k, getattr(head, k), gguf), k)
    ids = [int(head.target_layer_ids[i]) for i in range(head.n_target_layers)]
    return cfg, w, ids, int(head.mask_token_id)


_TARGET_ARCHS = ("qwen3", "qwen3moe")


def open_target(gguf: GgufFile):
    """Binds a pure-attention Qwen3-style decoder (``general.architecture`` qwen3 or qwen3moe) with the tensor names
    and [in, out] shape checks of the target loader (loader.rs:436-500, 595-612): returns (ModelConfig, weights).
    The hybrid qwen35 / qwen35moe targets carry Gated-DeltaNet layers, for which this library has no kernels: they
    are refused, as the loader refuses architectures it does not know (loader.rs:1330-1337)."""
    arch = gguf.architecture()
    if arch not in _TARGET_ARCHS:
        raise DFlashError(13, f"unsupported architecture {arch!r} (targets: {', '.join(_TARGET_ARCHS)})")

    def need_u(key):
        v = gguf.get_u64(f"{arch}.{key}")
        if v is None or v == 0 or v > 0xFFFFFFFF:
            raise DFlashError(13, f"bad or missing metadata: {arch}.{key}")
        return v

    def need_t(name, shapes):
        t = gguf.find(name)
        if t is None:
            raise DFlashError(13, f"missing tensor {name}")
        if t.shape not in [tuple(s) for s in shapes]:
            raise DFlashError(13, f"tensor {name}: expected shape {list(shapes[0])}, got {list(t.shape)}")
        return t

    moe = arch == "qwen3moe"
    n_layers, hidden = need_u("block_count"), need_u("embedding_length")
    n_q, n_kv = need_u("attention.head_count"), need_u("attention.head_count_kv")
    head_dim = gguf.get_u64(f"{arch}.attention.key_length") or hidden // n_q
    if n_q % n_kv:
        raise DFlashError(13, f"{arch}.attention.head_count must be a multiple of head_count_kv")
    eps = gguf.get_f64(f"{arch}.attention.layer_norm_rms_epsilon") or 1e-6
    theta = gguf.get_f64(f"{arch}.rope.freq_base") or 1e6
    embd = gguf.find("token_embd.weight")
    if embd is None or len(embd.shape) != 2 or embd.shape[0] != hidden:
        raise DFlashError(13, "token_embd.weight missing or not [hidden, vocab]")
    vocab = embd.shape[1]
    kw = dict(n_layers=n_layers, hidden=hidden, n_q=n_q, n_kv=n_kv, head_dim=head_dim, vocab=vocab, eps=eps, rope_theta=theta)
    if moe:
        kw.update(ffn=0, n_expert=need_u("expert_count"), n_expert_used=need_u("expert_used_count"),
                  ffn_expert=need_u("expert_feed_forward_length"), ffn_shared=need_u("expert_shared_feed_forward_length"))
    else:
        kw.update(ffn=need_u("feed_forward_length"))
    cfg = ModelConfig(**kw)
    q_dim, kv_dim = n_q * head_dim, n_kv * head_dim
    out = gguf.find("output.weight")  # absent = tied embeddings (loader.rs:445-452)
    if out is not None and out.shape != (hidden, vocab):
        raise DFlashError(13, f"tensor output.weight: expected shape [{hidden}, {vocab}], got {list(out.shape)}")
    w = {"token_embd": _pair(embd, "token_embd"), "output": _pair(out if out is not None else embd, "output"),
         "output_norm": need_t("output_norm.weight", [(hidden,)]).f32(), "layers": []}
    for i in range(n_layers):
        b = f"blk.{i}."
        post = gguf.find(b + "post_attention_norm.weight") or need_t(b + "ffn_norm.weight", [(hidden,)])
        Lw = {"attn_norm": need_t(b + "attn_norm.weight", [(hidden,)]).f32(), "post_norm": post.f32(),
              "q_norm": need_t(b + "attn_q_norm.weight", [(head_dim,)]).f32(),
              "k_norm": need_t(b + "attn_k_norm.weight", [(head_dim,)]).f32(),
              "wq": _pair(need_t(b + "attn_q.weight", [(hidden, q_dim)]), "wq"),
              "wk": _pair(need_t(b + "attn_k.weight", [(hidden, kv_dim)]), "wk"),
              "wv": _pair(need_t(b + "attn_v.weight", [(hidden, kv_dim)]), "wv"),
              "wo": _pair(need_t(b + "attn_output.weight", [(q_dim, hidden)]), "wo")}
        if moe:
            E, fe, fs = cfg.n_expert, cfg.ffn_expert, cfg.ffn_shared
            Lw["router"] = _pair(need_t(b + "ffn_gate_inp.weight", [(hidden, E)]), "router")
            Lw["gate_exps"] = _pair(need_t(b + "ffn_gate_exps.weight", [(hidden, fe, E)]), "gate_exps")
            Lw["up_exps"] = _pair(need_t(b + "ffn_up_exps.weight", [(hidden, fe, E)]), "up_exps")
            Lw["down_exps"] = _pair(need_t(b + "ffn_down_exps.weight", [(fe, hidden, E)]), "down_exps")
            Lw["shexp_gate"] = need_t(b + "ffn_gate_inp_shexp.weight", [(hidden,)]).f32().reshape(-1)
            Lw["gate"] = _pair(need_t(b + "ffn_gate_shexp.weight", [(hidden, fs)]), "gate")
            Lw["up"] = _pair(need_t(b + "ffn_up_shexp.weight", [(hidden, fs)]), "up")
            Lw["down"] = _pair(need_t(b + "ffn_down_shexp.weight", [(fs, hidden)]), "down")
        else:
            f = cfg.ffn
            Lw["gate"] = _pair(need_t(b + "ffn_gate.weight", [(hidden, f)]), "gate")
            Lw["up"] = _pair(need_t(b + "ffn_up.weight", [(hidden, f)]), "up")
            Lw["down"] = _pair(need_t(b + "ffn_down.weight", [(f, hidden)]), "down")
        w["layers"].append(Lw)
    return cfg, w


# ---- writer ----

_BLOCK = {F32: (1, 4), F16: (1, 2), Q8_0: (32, 34), Q4_K: (256, 144), Q6_K: (256, 210)}


def _s(b: bytes) -> bytes:
    return struct.pack("<Q", len(b)) + b


def _value(v) -> bytes:
    """(type tag + payload) of one metadata value.  Python ints are written as u32 when they fit (u64 otherwise,
    i64 when negative), floats as f32, lists by their first element's kind; a (tag, value) tuple forces a type."""
    fmt = {_U8: "<B", _I8: "<b", _U16: "<H", _I16: "<h", _U32: "<I", _I32: "<i", _F32: "<f", _BOOL: "<?", _U64: "<Q",
           _I64: "<q", _F64: "<d"}

    def scalar(tag, x):
        return _s(x.encode() if isinstance(x, str) else x) if tag == _STR else struct.pack(fmt[tag], x)

    def tag_of(x):
        if isinstance(x, bool):
            return _BOOL
        if isinstance(x, int):
            return _I64 if x < 0 else (_U32 if x <= 0xFFFFFFFF else _U64)
        if isinstance(x, float):
            return _F32
        if isinstance(x, (str, bytes)):
            return _STR
        raise TypeError(f"no GGUF value type for {type(x)}")

    if isinstance(v, tuple):
        tag, x = v
        if isinstance(x, (list, np.ndarray)):
            return struct.pack("<IIQ", _ARR, tag, len(x)) + b"".join(scalar(tag, e) for e in x)
        return struct.pack("<I", tag) + scalar(tag, x)
    if isinstance(v, (list, np.ndarray)):
        v = list(v)
        tag = tag_of(v[0]) if v else _U32
        if tag in (_U32, _U64, _I64):
            tag = _I64 if any(e < 0 for e in v) else (_U64 if any(e > 0xFFFFFFFF for e in v) else _U32)
        return struct.pack("<IIQ", _ARR, tag, len(v)) + b"".join(scalar(tag, e) for e in v)
    tag = tag_of(v)
    return struct.pack("<I", tag) + scalar(tag, v)


def write_gguf(path, metadata: dict, tensors: dict, alignment: int = 32, version: int = 3):
    """Writes a little-endian GGUF v3 file.  ``tensors``: name -> float32 ndarray (written as F32 with its numpy
    shape reversed, fastest dimension first) or (ggml type, shape fastest-first, uint8 block bytes)."""
    infos, blobs, off = [], [], 0
    for name, t in tensors.items():
        if isinstance(t, np.ndarray):
            t = (F32, tuple(reversed(t.shape)), np.ascontiguousarray(t, dtype=np.float32).view(np.uint8).reshape(-1))
        ttype, shape, data = t
        data = np.ascontiguousarray(data).view(np.uint8).reshape(-1)
        be, bb = _BLOCK[ttype]
        if int(np.prod(shape)) // be * bb != data.size:
            raise ValueError(f"{name}: {data.size} bytes do not match shape {shape} of type {ttype}")
        infos.append(_s(name.encode()) + struct.pack("<I", len(shape)) + b"".join(struct.pack("<Q", d) for d in shape) +
                     struct.pack("<IQ", ttype, off))
        blobs.append((off, data))
        off = (off + data.size + alignment - 1) // alignment * alignment
    md = dict(metadata)
    if alignment != 32:
        md["general.alignment"] = alignment
    head = struct.pack("<IIQQ", GGUF_MAGIC, version, len(infos), len(md))
    head += b"".join(_s(k.encode()) + _value(v) for k, v in md.items()) + b"".join(infos)
    start = (len(head) + alignment - 1) // alignment * alignment
    with open(path, "wb") as f:
        f.write(head + b"\0" * (start - len(head)))
        for o, data in blobs:
            f.seek(start + o)
            f.write(data.tobytes())
        if blobs:  # pad the last tensor to the alignment, as converters do
            end = start + off
            f.seek(0, 2)
            f.write(b"\0" * (end - f.tell()))


def split_path(prefix, no: int, count: int) -> str:
    """File name of shard ``no`` (0-based) of ``count`` (split_suffix, gguf.rs:985: numbers in names start at 1)."""
    return f"{prefix}-{no + 1:05d}-of-{count:05d}.gguf"


def write_split_gguf(prefix, metadata: dict, shards: list, alignment: int = 32) -> list:
    """Writes a split model: ``shards`` is one tensor dictionary per file.  Every shard carries split.no (u16),
    split.count (u16) and split.tensors.count (i32) as converters write them; the model's own metadata goes into
    the first shard only.  Returns the paths, first shard first."""
    total = sum(len(t) for t in shards)
    paths = []
    for no, tensors in enumerate(shards):
        md = dict(metadata) if no == 0 else {}
        md.update({"split.no": (_U16, no), "split.count": (_U16, len(shards)), "split.tensors.count": (_I32, total)})
        paths.append(split_path(prefix, no, len(shards)))
        write_gguf(paths[-1], md, tensors, alignment=alignment)
    return paths


def _mat_entry(pair, n_in, rows_shape):
    qtype, blocks = pair
    if hasattr(blocks, "cpu"):
        blocks = blocks.cpu().numpy()
    return (int(qtype), (n_in,) + tuple(rows_shape), np.ascontiguousarray(blocks).view(np.uint8).reshape(-1))


def draft_head_tensors(cfg: DraftConfig, w: dict, convention: int = 1) -> dict:
    """Tensor table of a drafter file (names of the given convention) from a ``DraftHead`` weight dictionary."""
    fc, hn, post = (("dflash_fc.weight", "dflash_hidden_norm.weight", "post_attention_norm") if convention == 1 else
                    ("fc.weight", "enc.output_norm.weight", "ffn_norm"))
    H, q_dim, kv_dim = cfg.hidden, cfg.n_q * cfg.head_dim, cfg.n_kv * cfg.head_dim
    t = {fc: _mat_entry(w["fc"], cfg.n_taps * H, (H,)), hn: np.asarray(w["hidden_norm"], np.float32),
         "output_norm.weight": np.asarray(w["output_norm"], np.float32)}
    for i, Lw in enumerate(w["layers"]):
        b = f"blk.{i}."
        t[b + "attn_norm.weight"] = np.asarray(Lw["attn_norm"], np.float32)
        t[b + "attn_q.weight"] = _mat_entry(Lw["wq"], H, (q_dim,))
        t[b + "attn_k.weight"] = _mat_entry(Lw["wk"], H, (kv_dim,))
        t[b + "attn_v.weight"] = _mat_entry(Lw["wv"], H, (kv_dim,))
        t[b + "attn_output.weight"] = _mat_entry(Lw["wo"], q_dim, (H,))
        t[b + "attn_q_norm.weight"] = np.asarray(Lw["q_norm"], np.float32)
        t[b + "attn_k_norm.weight"] = np.asarray(Lw["k_norm"], np.float32)
        t[b + post + ".weight"] = np.asarray(Lw["post_norm"], np.float32)
        t[b + "ffn_gate.weight"] = _mat_entry(Lw["gate"], H, (cfg.ffn,))
        t[b + "ffn_up.weight"] = _mat_entry(Lw["up"], H, (cfg.ffn,))
        t[b + "ffn_down.weight"] = _mat_entry(Lw["down"], cfg.ffn, (H,))
        if cfg.conv_kernel_size:
            dyn = 2 * cfg.conv_kernel_size * (H // cfg.conv_group_size)
            t[b + "attn_conv_base"] = np.asarray(Lw["conv_attn_base"], np.float32)
            t[b + "attn_conv_proj.weight"] = _mat_entry(Lw["conv_attn_proj"], H, (dyn,))
            t[b + "ffn_conv_base"] = np.asarray(Lw["conv_ffn_base"], np.float32)
            t[b + "ffn_conv_proj.weight"] = _mat_entry(Lw["conv_ffn_proj"], H, (dyn,))
    if cfg.selector_rank:
        vocab = np.asarray(w["selector_predecessor"][1]).shape[0]
        t["selector_hidden.weight"] = _mat_entry(w["selector_hidden"], H, (cfg.selector_rank,))
        t["selector_predecessor.weight"] = _mat_entry(w["selector_predecessor"], cfg.selector_rank, (vocab,))
        t["selector_successor.weight"] = _mat_entry(w["selector_successor"], cfg.selector_rank, (vocab,))
    return t


def draft_head_metadata(cfg: DraftConfig, target_layer_ids, mask_token_id: int, swa_pattern=None, convention: int = 1) -> dict:
    """Metadata of a drafter file.  ``target_layer_ids`` are post-block ids; convention 2 stores them + 1."""
    swa = [bool(x) for x in (swa_pattern if swa_pattern is not None else [False] * cfg.n_layers)]
    p = "dflash-draft" if convention == 1 else "dflash"
    md = {"general.architecture": p, f"{p}.block_count": cfg.n_layers, f"{p}.embedding_length": cfg.hidden,
          f"{p}.feed_forward_length": cfg.ffn, f"{p}.attention.head_count": cfg.n_q,
          f"{p}.attention.head_count_kv": cfg.n_kv, f"{p}.attention.key_length": cfg.head_dim,
          f"{p}.rope.freq_base": float(cfg.rope_theta), f"{p}.attention.layer_norm_rms_epsilon": float(cfg.eps),
          f"{p}.attention.causal": bool(cfg.causal), f"{p}.attention.sliding_window": int(cfg.swa_window),
          f"{p}.attention.sliding_window_pattern": (_BOOL, swa)}
    if convention == 1:
        md.update({f"{p}.dflash.block_size": cfg.block_size, f"{p}.dflash.mask_token_id": mask_token_id,
                   f"{p}.dflash.target_layer_ids": [int(x) for x in target_layer_ids],
                   f"{p}.dflash.n_target_features": cfg.n_taps * cfg.hidden})
    else:
        md.update({"dflash.block_size": cfg.block_size, "tokenizer.ggml.mask_token_id": mask_token_id,
                   "dflash.target_layers": [int(x) + 1 for x in target_layer_ids]})
        if cfg.selector_rank:
            md.update({"dflash.conv_kernel_size": cfg.conv_kernel_size, "dflash.conv_group_size": cfg.conv_group_size,
                       "dflash.selector_rank": cfg.selector_rank, "dflash.selector_top_k": cfg.selector_top_k})
    return md


def target_tensors(cfg: ModelConfig, w: dict, tied: bool = False) -> dict:
    """Tensor table of a qwen3 / qwen3moe target file from a ``TargetModel`` weight dictionary."""
    H, q_dim, kv_dim = cfg.hidden, cfg.n_q * cfg.head_dim, cfg.n_kv * cfg.head_dim
    t = {"token_embd.weight": _mat_entry(w["token_embd"], H, (cfg.vocab,)),
         "output_norm.weight": np.asarray(w["output_norm"], np.float32)}
    if not tied:
        t["output.weight"] = _mat_entry(w["output"], H, (cfg.vocab,))
    for i, Lw in enumerate(w["layers"]):
        b = f"blk.{i}."
        t[b + "attn_norm.weight"] = np.asarray(Lw["attn_norm"], np.float32)
        t[b + "post_attention_norm.weight"] = np.asarray(Lw["post_norm"], np.float32)
        t[b + "attn_q_norm.weight"] = np.asarray(Lw["q_norm"], np.float32)
        t[b + "attn_k_norm.weight"] = np.asarray(Lw["k_norm"], np.float32)
        t[b + "attn_q.weight"] = _mat_entry(Lw["wq"], H, (q_dim,))
        t[b + "attn_k.weight"] = _mat_entry(Lw["wk"], H, (kv_dim,))
        t[b + "attn_v.weight"] = _mat_entry(Lw["wv"], H, (kv_dim,))
        t[b + "attn_output.weight"] = _mat_entry(Lw["wo"], q_dim, (H,))
        if cfg.n_expert:
            E, fe, fs = cfg.n_expert, cfg.ffn_expert, cfg.ffn_shared
            t[b + "ffn_gate_inp.weight"] = _mat_entry(Lw["router"], H, (E,))
            t[b + "ffn_gate_exps.weight"] = _mat_entry(Lw["gate_exps"], H, (fe, E))
            t[b + "ffn_up_exps.weight"] = _mat_entry(Lw["up_exps"], H, (fe, E))
            t[b + "ffn_down_exps.weight"] = _mat_entry(Lw["down_exps"], fe, (H, E))
            t[b + "ffn_gate_inp_shexp.weight"] = np.asarray(Lw["shexp_gate"], np.float32)
            t[b + "ffn_gate_shexp.weight"] = _mat_entry(Lw["gate"], H, (fs,))
            t[b + "ffn_up_shexp.weight"] = _mat_entry(Lw["up"], H, (fs,))
            t[b + "ffn_down_shexp.weight"] = _mat_entry(Lw["down"], fs, (H,))
        else:
            t[b + "ffn_gate.weight"] = _mat_entry(Lw["gate"], H, (cfg.ffn,))
            t[b + "ffn_up.weight"] = _mat_entry(Lw["up"], H, (cfg.ffn,))
            t[b + "ffn_down.weight"] = _mat_entry(Lw["down"], cfg.ffn, (H,))
    return t


def target_metadata(cfg: ModelConfig) -> dict:
    p = "qwen3moe" if cfg.n_expert else "qwen3"
    md = {"general.architecture": p, f"{p}.block_count": cfg.n_layers, f"{p}.embedding_length": cfg.hidden,
          f"{p}.attention.head_count": cfg.n_q, f"{p}.attention.head_count_kv": cfg.n_kv,
          f"{p}.attention.key_length": cfg.head_dim, f"{p}.rope.freq_base": float(cfg.rope_theta),
          f"{p}.attention.layer_norm_rms_epsilon": float(cfg.eps)}
    if cfg.n_expert:
        md.update({f"{p}.expert_count": cfg.n_expert, f"{p}.expert_used_count": cfg.n_expert_used,
                   f"{p}.expert_feed_forward_length": cfg.ffn_expert,
                   f"{p}.expert_shared_feed_forward_length": cfg.ffn_shared})
    else:
        md[f"{p}.feed_forward_length"] = cfg.ffn
    return md
