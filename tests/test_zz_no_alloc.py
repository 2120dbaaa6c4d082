"""GPU test of dflash_gemm_fewrow_noalloc, the GEMM entry point for callers that may not allocate: called
through the C ABI with caller-owned buffers only, its output must equal dflash_gemm_fewrow's bit for bit
(same kernels, same launch shape, same order of the split-K sums), on two calls in a row, the second with
a smaller input (the fixed scratch array then still holds the first call's partial tiles)."""
import os

import numpy as np
import pytest

import qwen_llm_amd as dfl

pytestmark = pytest.mark.gpu


def _run_pair(ctx, L, qtype, n_in, n_out, n_rows, seed, x_f16):
    import torch

    w = torch.from_numpy(dfl.synth.random_weight(qtype, n_out, n_in, seed=seed)).cuda()
    x = torch.from_numpy(np.random.default_rng(seed).standard_normal((n_rows, n_in)).astype(np.float32)).cuda()
    if x_f16:
        x = x.half()
    x_type = dfl.TYPE_F16 if x_f16 else dfl.TYPE_F32
    qtype = ctx.checked_type(qtype, w)  # the tag of a range-checked tensor: both entry points then take the fast kernels
    want = ctx.gemm_fewrow(w, qtype, x, n_in, n_out)
    got = torch.full((n_rows, n_out), float("nan"), dtype=torch.float32, device="cuda")
    stream = torch.cuda.current_stream().cuda_stream
    rc = L.dflash_gemm_fewrow_noalloc(qtype, w.data_ptr(), x.data_ptr(), x_type, got.data_ptr(), n_in, n_out, n_rows, stream)
    assert rc == 0, L.dflash_gemm_fewrow_noalloc_error().decode()
    torch.cuda.synchronize()
    assert torch.equal(got.view(torch.int32), want.view(torch.int32)), (qtype, n_in, n_out, n_rows)


def test_noalloc_gemm_equals_context_gemm_twice_in_a_row():
    import torch

    torch.cuda.set_device(0)
    ctx = dfl.Context(0)
    L = dfl.lib()
    assert "DFLASH_GEMM_WGS" not in os.environ, "bit-identity of the two entry points holds with the workgroup knob unset"
    try:
        # nothing may be allocated by the entry point itself: a first call (symbol look-up, module load) aside, free
        # device memory must read the same before and after a call through the C ABI with caller-owned buffers
        w = torch.from_numpy(dfl.synth.random_weight(dfl.TYPE_Q4_K, 272, 1024, seed=9)).cuda()
        tag = ctx.checked_type(dfl.TYPE_Q4_K, w)
        x = torch.zeros((5, 1024), dtype=torch.float32, device="cuda")
        y = torch.empty((5, 272), dtype=torch.float32, device="cuda")
        stream = torch.cuda.current_stream().cuda_stream
        assert L.dflash_gemm_fewrow_noalloc(tag, w.data_ptr(), x.data_ptr(), dfl.TYPE_F32, y.data_ptr(), 1024, 272, 5, stream) == 0
        torch.cuda.synchronize()
        free_before = torch.cuda.mem_get_info(0)[0]
        for _ in range(3):
            assert L.dflash_gemm_fewrow_noalloc(tag, w.data_ptr(), x.data_ptr(), dfl.TYPE_F32, y.data_ptr(), 1024, 272, 5, stream) == 0
        torch.cuda.synchronize()
        assert torch.cuda.mem_get_info(0)[0] == free_before, "the no-allocation entry point allocated device memory"
        # split-K shapes (partial tiles go through the scratch array), larger then smaller, for both streaming kernels
        _run_pair(ctx, L, dfl.TYPE_Q4_K, 5120, 6144, 16, 1, True)
        _run_pair(ctx, L, dfl.TYPE_Q4_K, 1024, 272, 5, 2, False)
        _run_pair(ctx, L, dfl.TYPE_Q6_K, 2048, 4096, 16, 3, False)
        _run_pair(ctx, L, dfl.TYPE_Q6_K, 512, 48, 1, 4, True)
        _run_pair(ctx, L, dfl.TYPE_Q8_0, 1024, 128, 16, 5, False)  # a kernel without scratch: same entry point
    finally:
        ctx.close()


def test_noalloc_gemm_guards():
    import torch

    torch.cuda.set_device(0)
    L = dfl.lib()
    buf = torch.zeros(1 << 16, dtype=torch.uint8, device="cuda")
    y = torch.zeros(16 * 16, dtype=torch.float32, device="cuda")
    p = buf.data_ptr()
    assert L.dflash_gemm_fewrow_noalloc(dfl.TYPE_Q4_K, p, p + 32768, dfl.TYPE_F32, y.data_ptr(), (1 << 18) + 256, 16, 1, 0) == 1
    assert b"DFLASH_NOALLOC_MAX" in L.dflash_gemm_fewrow_noalloc_error()
    assert L.dflash_gemm_fewrow_noalloc(dfl.TYPE_Q4_K, p, p + 32768, dfl.TYPE_F32, y.data_ptr(), 256, (1 << 20) + 1, 1, 0) == 1
    assert L.dflash_gemm_fewrow_noalloc(dfl.TYPE_Q4_K, 0, p, dfl.TYPE_F32, y.data_ptr(), 256, 16, 1, 0) == 7
    assert L.dflash_gemm_fewrow_noalloc(dfl.TYPE_Q4_K, p, p + 32768, dfl.TYPE_F32, y.data_ptr(), 250, 16, 1, 0) == 1
    assert L.dflash_gemm_fewrow_noalloc(dfl.TYPE_Q4_K, p, p + 32768, dfl.TYPE_F32, y.data_ptr(), 256, 16, 17, 0) == 1
    assert L.dflash_gemm_fewrow_noalloc(dfl.TYPE_Q4_K, p, p + 32768, dfl.TYPE_F32, p + 16, 256, 16, 1, 0) == 3  # y aliases w
