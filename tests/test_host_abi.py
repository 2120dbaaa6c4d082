"""CPU-side checks: the C-ABI library loads and exports everything the public header
declares (no compute calls without a GPU), and the synthetic quantisers produce
blocks the oracle decodes back to within the format's step."""
import ctypes as C
import os

import numpy as np
import pytest

import qwen_llm_amd as dfl


def test_library_exports_every_declared_symbol():
    if not os.path.exists(dfl.LIB_PATH):
        pytest.skip("libdflash_hip.so not built yet (run __graft_entry__.build())")
    L = dfl.lib()
    names = dfl.declared_symbols()
    assert len(names) >= 8
    for name in names:
        assert hasattr(L, name), f"{name} declared in include/dflash_hip.h but not exported"
    assert b"gfx950" in L.dflash_version()
    assert L.dflash_status_name(1) == b"BadShape"


def test_row_bytes_matches_block_geometry():
    """tensor.rs:164-208"""
    if not os.path.exists(dfl.LIB_PATH):
        pytest.skip("library not built")
    L = dfl.lib()
    assert L.dflash_row_bytes(dfl.TYPE_Q4_K, 5120) == 5120 // 256 * 144
    assert L.dflash_row_bytes(dfl.TYPE_Q6_K, 512) == 420
    assert L.dflash_row_bytes(dfl.TYPE_Q8_0, 64) == 68
    assert L.dflash_row_bytes(dfl.TYPE_Q4_K, 100) == 0  # not block aligned (codec.rs:91-103)


def test_context_requires_gpu_or_fails_loudly():
    import torch

    if torch.cuda.is_available():
        pytest.skip("GPU present")
    with pytest.raises(RuntimeError):
        dfl.Context()


@pytest.mark.parametrize("qtype,step", [(dfl.synth.Q4_K, 1 / 15), (dfl.synth.Q6_K, 1 / 31), (dfl.synth.Q8_0, 1 / 127)])
def test_quantisers_round_trip_through_oracle(oracle, qtype, step):
    rng = np.random.default_rng(7)
    w = (rng.standard_normal((8, 1024)) * 0.02).astype(np.float32)
    blocks = dfl.synth.quantize(qtype, w)
    assert blocks.shape == (8, dfl.synth.row_bytes(qtype, 1024))
    back = oracle.dequant(qtype, blocks, w.size).reshape(w.shape)
    span = np.abs(w).max() * 2
    assert np.abs(back - w).max() <= span * step
    chunked = dfl.synth.random_weight(qtype, 8, 1024, seed=7, chunk_rows=3)
    assert np.array_equal(chunked, dfl.synth.random_weight(qtype, 8, 1024, seed=7, chunk_rows=8))
