"""Synthetic inputs for the DFlash step: ggml block quantisers and random blocks.

The quantisers only manufacture weights: both the HIP kernels and the CPU checker
consume the bytes they produce, so their exact rounding is not part of any parity
claim.  They follow the simple min/max scheme (per sub-block minimum and range,
6-bit scales against an f16 super-block scale) rather than ggml's iterative search.
Block layouts: tensor.rs:164-208 of the reference; random-block recipe:
metal/mat_mat.rs:4154-4199.
"""
from __future__ import annotations

import numpy as np

Q8_0, Q4_K, Q6_K = 8, 12, 14
BLOCK_ELEMS = {Q8_0: 32, Q4_K: 256, Q6_K: 256}
BLOCK_BYTES = {Q8_0: 34, Q4_K: 144, Q6_K: 210}


def row_bytes(qtype: int, n_in: int) -> int:
    assert n_in % BLOCK_ELEMS[qtype] == 0
    return n_in // BLOCK_ELEMS[qtype] * BLOCK_BYTES[qtype]


def _f16_bytes(a: np.ndarray) -> np.ndarray:
    return a.astype(np.float16).view(np.uint8).reshape(a.shape + (2,))


def quantize_q4_k(w: np.ndarray) -> np.ndarray:
    """f32 [..., n_in] -> uint8 [..., n_in/256*144]"""
    w = np.ascontiguousarray(w, dtype=np.float32)
    lead, n_in = w.shape[:-1], w.shape[-1]
    x = w.reshape(-1, 8, 32)  # [blocks, sub, 32]
    nb = x.shape[0]
    mn = np.minimum(x.min(axis=2), 0.0)
    mx = x.max(axis=2)
    scale = (mx - mn) / 15.0
    d = (scale.max(axis=1) / 63.0).astype(np.float16).astype(np.float32)
    dmin = ((-mn).max(axis=1) / 63.0).astype(np.float16).astype(np.float32)
    with np.errstate(divide="ignore", invalid="ignore"):
        sc = np.where(d[:, None] > 0, np.rint(scale / d[:, None]), 0.0).clip(0, 63).astype(np.uint8)
        m = np.where(dmin[:, None] > 0, np.rint(-mn / dmin[:, None]), 0.0).clip(0, 63).astype(np.uint8)
        eff = d[:, None] * sc
        q = np.where(eff[:, :, None] > 0, np.rint((x + (dmin[:, None] * m)[:, :, None]) / eff[:, :, None]), 0.0)
    q = q.clip(0, 15).astype(np.uint8)
    out = np.zeros((nb, 144), np.uint8)
    out[:, 0:2] = _f16_bytes(d)
    out[:, 2:4] = _f16_bytes(dmin)
    out[:, 4:8] = sc[:, 0:4] | ((sc[:, 4:8] >> 4) << 6)
    out[:, 8:12] = m[:, 0:4] | ((m[:, 4:8] >> 4) << 6)
    out[:, 12:16] = (sc[:, 4:8] & 0x0F) | ((m[:, 4:8] & 0x0F) << 4)
    out[:, 16:144] = (q[:, 0::2, :] | (q[:, 1::2, :] << 4)).reshape(nb, 128)
    return out.reshape(lead + (n_in // 256 * 144,))


def quantize_q6_k(w: np.ndarray) -> np.ndarray:
    """f32 [..., n_in] -> uint8 [..., n_in/256*210]"""
    w = np.ascontiguousarray(w, dtype=np.float32)
    lead, n_in = w.shape[:-1], w.shape[-1]
    x = w.reshape(-1, 16, 16)
    nb = x.shape[0]
    amax = np.abs(x).max(axis=2)
    scale = amax / 31.0
    d = (scale.max(axis=1) / 127.0).astype(np.float16).astype(np.float32)
    with np.errstate(divide="ignore", invalid="ignore"):
        sc = np.where(d[:, None] > 0, np.rint(scale / d[:, None]), 0.0).clip(0, 127).astype(np.int8)
        eff = d[:, None] * sc
        q = np.where(eff[:, :, None] > 0, np.rint(x / eff[:, :, None]), 0.0)
    q = (q.clip(-32, 31) + 32).astype(np.uint8).reshape(nb, 2, 4, 32)  # [blk, half, quarter, l]
    out = np.zeros((nb, 210), np.uint8)
    ql = np.zeros((nb, 2, 64), np.uint8)
    ql[:, :, 0:32] = (q[:, :, 0] & 0xF) | ((q[:, :, 2] & 0xF) << 4)
    ql[:, :, 32:64] = (q[:, :, 1] & 0xF) | ((q[:, :, 3] & 0xF) << 4)
    qh = (q[:, :, 0] >> 4) | ((q[:, :, 1] >> 4) << 2) | ((q[:, :, 2] >> 4) << 4) | ((q[:, :, 3] >> 4) << 6)
    out[:, 0:128] = ql.reshape(nb, 128)
    out[:, 128:192] = qh.reshape(nb, 64)
    out[:, 192:208] = sc.view(np.uint8)
    out[:, 208:210] = _f16_bytes(d)
    return out.reshape(lead + (n_in // 256 * 210,))


def quantize_q8_0(w: np.ndarray) -> np.ndarray:
    w = np.ascontiguousarray(w, dtype=np.float32)
    lead, n_in = w.shape[:-1], w.shape[-1]
    x = w.reshape(-1, 32)
    nb = x.shape[0]
    d = (np.abs(x).max(axis=1) / 127.0).astype(np.float16).astype(np.float32)
    with np.errstate(divide="ignore", invalid="ignore"):
        q = np.where(d[:, None] > 0, np.rint(x / d[:, None]), 0.0).clip(-127, 127).astype(np.int8)
    out = np.zeros((nb, 34), np.uint8)
    out[:, 0:2] = _f16_bytes(d)
    out[:, 2:34] = q.view(np.uint8)
    return out.reshape(lead + (n_in // 32 * 34,))


def quantize(qtype: int, w: np.ndarray, chunk_rows: int = 2048) -> np.ndarray:
    """Quantise a 2-D weight [n_out, n_in] row-chunk by row-chunk (bounded memory)."""
    fn = {Q4_K: quantize_q4_k, Q6_K: quantize_q6_k, Q8_0: quantize_q8_0}[qtype]
    w = np.asarray(w)
    if w.ndim != 2:
        return fn(w)
    return np.concatenate([fn(w[i:i + chunk_rows]) for i in range(0, w.shape[0], chunk_rows)], axis=0)


def random_weight(qtype: int, n_out: int, n_in: int, seed: int, std: float = 0.02, chunk_rows: int = 2048):
    """Quantised N(0, std) weight [n_out, row_bytes] without holding the f32 matrix."""
    rng = np.random.default_rng(seed)
    fn = {Q4_K: quantize_q4_k, Q6_K: quantize_q6_k, Q8_0: quantize_q8_0}[qtype]
    parts = []
    for i in range(0, n_out, chunk_rows):
        rows = min(chunk_rows, n_out - i)
        parts.append(fn((rng.standard_normal((rows, n_in), dtype=np.float32) * np.float32(std))))
    return np.concatenate(parts, axis=0)


def random_blocks(qtype: int, n_blocks: int, seed: int) -> np.ndarray:
    """Blocks of random bytes with small fixed super-block scales (metal/mat_mat.rs:4154-4199)."""
    rng = np.random.default_rng(seed)
    out = rng.integers(0, 256, (n_blocks, BLOCK_BYTES[qtype]), dtype=np.uint8)
    d = _f16_bytes(np.full(n_blocks, 0.01, np.float32))
    if qtype == Q4_K:
        out[:, 0:2] = d
        out[:, 2:4] = _f16_bytes(np.full(n_blocks, 0.005, np.float32))
    elif qtype == Q6_K:
        out[:, 192:208] = (rng.integers(0, 15, (n_blocks, 16)) - 7).astype(np.int8).view(np.uint8)
        out[:, 208:210] = d
    else:
        out[:, 0:2] = d
    return out


def extreme_blocks(qtype: int, n_blocks: int, seed: int) -> np.ndarray:
    """Blocks that exercise the full range of every field: all scale/min codes, all quants,
    super-block scales across many binades (including negative ones)."""
    rng = np.random.default_rng(seed)
    out = rng.integers(0, 256, (n_blocks, BLOCK_BYTES[qtype]), dtype=np.uint8)
    # up to the limits the few-row kernels accept (dflash_check_scale_range): Q4_K |d| <= 1 and |dmin| <= 32, Q6_K
    # |d| <= 0.25; the reference's own extreme blocks (d = 0.001, dmin = 5, metal/mat_mat.rs:4228-4265) are inside
    top = {Q4_K: 0, Q6_K: -2}.get(qtype, 0)
    scales = (rng.choice([1.0, -1.0], n_blocks) * 2.0 ** rng.integers(-12, top + 1, n_blocks)).astype(np.float32)
    if qtype == Q4_K:
        out[:, 0:2] = _f16_bytes(scales)
        out[:, 2:4] = _f16_bytes((rng.choice([1.0, -1.0], n_blocks) * 2.0 ** rng.integers(-12, 6, n_blocks)))
        out[0::7, 4:16] = 0xFF
        out[1::7, 4:16] = 0x00
        out[2::7, 16:] = 0xFF
        out[3::7, 16:] = 0x00
    elif qtype == Q6_K:
        out[:, 208:210] = _f16_bytes(scales)
        out[0::5, 192:208] = 0x80  # -128
        out[1::5, 192:208] = 0x7F
        out[2::5, 0:192] = 0xFF
        out[3::5, 0:192] = 0x00
    else:
        out[:, 0:2] = _f16_bytes(scales)
        out[0::3, 2:] = 0x80
        out[1::3, 2:] = 0x7F
    return out


def reference_extreme_blocks(qtype: int, n_blocks: int) -> np.ndarray:
    """The reference's extreme few-row blocks (metal/mat_mat.rs:4228-4265): d = 0.001 (Q4_K: dmin = 5), every other
    byte 0x00 / 0xFF (Q6_K scales and Q8_0 quants 0x80 / 0x7F), the pattern shifted by one from block to block."""
    bb = BLOCK_BYTES[qtype]
    i = np.arange(bb)[None, :] + np.arange(n_blocks)[:, None]
    even = (i % 2 == 0)
    out = np.where(even, 0x00, 0xFF).astype(np.uint8)
    d = _f16_bytes(np.full(1, 0.001, np.float32))
    if qtype == Q4_K:
        out[:, 0:2] = d
        out[:, 2:4] = _f16_bytes(np.full(1, 5.0, np.float32))
    elif qtype == Q6_K:
        out[:, 192:208] = np.where(even[:, 192:208], 0x80, 0x7F)
        out[:, 208:210] = d
    else:
        out[:, 2:] = np.where(even[:, 2:], 0x80, 0x7F)
        out[:, 0:2] = d
    return out


def random_blocks_scaled(qtype: int, n_out: int, n_in: int, std: float, rng) -> np.ndarray:
    """[n_out, row_bytes] uint8 on the host: random quant codes with super-block scales chosen so that the dequantised
    weights have zero mean and roughly the standard deviation `std` (the host twin of random_blocks_device, for
    shapes too large for the quantisers; both the HIP kernels and the CPU checker consume the bytes as they are)."""
    nblk = n_out * (n_in // BLOCK_ELEMS[qtype])
    out = rng.integers(0, 256, (nblk, BLOCK_BYTES[qtype]), dtype=np.uint8)
    if qtype == Q4_K:
        d = std / 257.0
        out[:, 0:2] = _f16_bytes(np.full(1, d, np.float32))
        out[:, 2:4] = _f16_bytes(np.full(1, 7.5 * d, np.float32))
    elif qtype == Q6_K:
        out[:, 192:208] = rng.integers(-16, 16, (nblk, 16)).astype(np.int8).view(np.uint8)
        out[:, 208:210] = _f16_bytes(np.full(1, std / 170.0, np.float32))
    else:
        out[:, 0:2] = _f16_bytes(np.full(1, std / 74.0, np.float32))
    return out.reshape(n_out, -1)


def random_blocks_device(qtype: int, n_out: int, n_in: int, std: float, gen, device):
    """[n_out, row_bytes] uint8 on `device`: random quant codes with super-block scales set so that the
    dequantised weights have zero mean and roughly the standard deviation `std`.
      Q4_K: codes uniform; w = d sc q - dmin m with dmin = 7.5 d  -> std(w) ~ 257 d
      Q6_K: sub-block scales uniform in [-16, 16), q uniform      -> std(w) ~ 170 d
      Q8_0: q uniform in [-128, 128)                              -> std(w) ~ 74 d"""
    import torch

    nblk = n_out * (n_in // BLOCK_ELEMS[qtype])
    out = torch.randint(0, 256, (nblk, BLOCK_BYTES[qtype]), dtype=torch.uint8, device=device, generator=gen)

    def f16_bytes(v):
        return torch.tensor([v], dtype=torch.float16).view(torch.uint8).to(device)

    if qtype == Q4_K:
        d = std / 257.0
        out[:, 0:2] = f16_bytes(d)
        out[:, 2:4] = f16_bytes(7.5 * d)
    elif qtype == Q6_K:
        sc = torch.randint(-16, 16, (nblk, 16), dtype=torch.int8, device=device, generator=gen)
        out[:, 192:208] = sc.view(torch.uint8)
        out[:, 208:210] = f16_bytes(std / 170.0)
    else:
        out[:, 0:2] = f16_bytes(std / 74.0)
    return out.view(n_out, -1)
