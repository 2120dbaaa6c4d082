"""GPU parity of the whole-K few-row GEMM over activations in fragment order (dflash_pack_xf,
dflash_gemm_fewrow_xf): against float64 of the oracle's dequant (<= 1e-2 relative, f32 accumulation), and
against dflash_gemm_fewrow on the same weights (same operands rounded the same way: the two may differ only in
the order of the f32 sums)."""
import numpy as np
import pytest

import qwen_llm_amd as dfl

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ctx():
    c = dfl.Context(0)
    yield c
    c.close()


def dev(a):
    import torch

    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def check(y, ref, label):
    y = y.astype(np.float64)
    assert np.all(np.isfinite(y)), f"{label}: non-finite output"
    rel_l2 = np.linalg.norm(y - ref) / max(np.linalg.norm(ref), 1e-30)
    rms = np.sqrt(np.mean(ref ** 2))
    elem = np.max(np.abs(y - ref) / np.maximum(np.abs(ref), rms))
    assert rel_l2 <= 2e-3 and elem <= 1e-2, f"{label}: rel_l2 {rel_l2:.3e} elem {elem:.3e}"


# (n_in, n_out, rows): one stage per wave (n_in <= 4096), two (up to 8192), ragged tile and row counts, two tiles per wave
SHAPES = [(256, 16, 16), (256, 40, 1), (1024, 272, 16), (2048, 5120, 16), (2048, 1000, 7), (4096, 2048, 16), (6144, 2048, 16),
          (5120, 6144, 16), (2048, 12288, 16), (3072, 100, 3), (8192, 48, 16)]


def upload(ctx, qtype, n_in, n_out, seed, extreme=False):
    """(device weight, type tag for the GEMM, host blocks in GGUF row order)."""
    if extreme:
        blocks = dfl.synth.extreme_blocks(qtype, n_out * n_in // 256, seed=seed).reshape(n_out, -1)
    else:
        blocks = dfl.synth.random_weight(qtype, n_out, n_in, seed=seed)
    wd = dev(blocks)
    if qtype == dfl.synth.Q4_K:
        return ctx.repack_q4k_tiled(wd, n_in, n_out), dfl.TYPE_Q4_K_TILED, blocks, wd
    return wd, ctx.checked_type(dfl.TYPE_Q6_K, wd), blocks, wd


@pytest.mark.parametrize("qtype", [dfl.synth.Q4_K, dfl.synth.Q6_K])
@pytest.mark.parametrize("n_in,n_out,rows", SHAPES)
@pytest.mark.parametrize("x_dtype", [np.float32, np.float16])
def test_whole_k_gemm_matches_oracle_and_streaming_kernels(ctx, oracle, canaries, qtype, n_in, n_out, rows, x_dtype):
    w, w_type, blocks, w_rows = upload(ctx, qtype, n_in, n_out, seed=n_in + n_out)
    kind = ctx.xf_kind(w_type, n_in, n_out)
    assert kind == (dfl.XF_Q4K if qtype == dfl.synth.Q4_K else dfl.XF_Q6K)
    x = np.random.default_rng(rows).standard_normal((rows, n_in)).astype(x_dtype)
    xd = dev(x)
    xf = ctx.pack_xf(xd, kind)
    y = ctx.gemm_fewrow_xf(w, w_type, xf, rows, n_in, n_out).cpu().numpy()
    canaries.check()
    wf = oracle.dequant(qtype, blocks, n_in * n_out).reshape(n_out, n_in).astype(np.float64)
    ref = x.astype(np.float16).astype(np.float64) @ wf.T  # every few-row kernel rounds its activations to f16
    check(y, ref, f"{n_in}->{n_out} x{rows}")
    # the streaming kernels on the same operands: same products, other order of the f32 sums
    y2 = ctx.gemm_fewrow(w, w_type, xd, n_in, n_out).cpu().numpy()
    assert np.max(np.abs(y - y2)) <= 2e-5 * max(np.max(np.abs(ref)), 1.0) + 1e-4 * np.sqrt(np.mean(ref ** 2))


@pytest.mark.parametrize("qtype", [dfl.synth.Q4_K, dfl.synth.Q6_K])
def test_whole_k_gemm_extreme_blocks(ctx, oracle, qtype):
    """The reference's extreme blocks (metal/mat_mat.rs:4228-4265: largest scales and codes) within the kernels' range."""
    n_in, n_out, rows = 2048, 320, 16
    w, w_type, blocks, _ = upload(ctx, qtype, n_in, n_out, seed=5, extreme=True)
    x = np.random.default_rng(6).standard_normal((rows, n_in)).astype(np.float32)
    xf = ctx.pack_xf(dev(x), ctx.xf_kind(w_type, n_in, n_out))
    y = ctx.gemm_fewrow_xf(w, w_type, xf, rows, n_in, n_out).cpu().numpy()
    wf = oracle.dequant(qtype, blocks, n_in * n_out).reshape(n_out, n_in).astype(np.float64)
    check(y, x.astype(np.float16).astype(np.float64) @ wf.T, "extreme")


@pytest.mark.parametrize("n_in,n_out,rows", SHAPES)
def test_q6k_tiled_order_is_bit_identical(ctx, n_in, n_out, rows):
    """The tiled, field-planar Q6_K order holds the same blocks in other places: the one-launch GEMM on it equals the same
    GEMM on the GGUF row order bit for bit (ragged tile and row counts, one and two stages per wave, two tiles per wave)."""
    blocks = dfl.synth.random_weight(dfl.synth.Q6_K, n_out, n_in, seed=n_in * 3 + n_out)
    wd = dev(blocks)
    row_type = ctx.checked_type(dfl.TYPE_Q6_K, wd)
    kind = ctx.xf_kind(row_type, n_in, n_out)
    assert kind == dfl.XF_Q6K and ctx.xf_kind(dfl.TYPE_Q6_K_TILED, n_in, n_out) == dfl.XF_Q6K
    wt = ctx.repack_q6k_tiled(wd, n_in, n_out)
    x = dev(np.random.default_rng(rows + 1).standard_normal((rows, n_in)).astype(np.float32))
    xf = ctx.pack_xf(x, kind)
    a = ctx.gemm_fewrow_xf(wd, row_type, xf, rows, n_in, n_out).cpu().numpy()
    b = ctx.gemm_fewrow_xf(wt, dfl.TYPE_Q6_K_TILED, xf, rows, n_in, n_out).cpu().numpy()
    assert np.array_equal(a.view(np.uint32), b.view(np.uint32))


def test_q6k_tiled_guards(ctx):
    import torch

    n_in, n_out = 2048, 512
    blocks = dfl.synth.random_weight(dfl.synth.Q6_K, n_out, n_in, seed=3)
    wt = ctx.repack_q6k_tiled(dev(blocks), n_in, n_out)
    x = torch.zeros((16, n_in), device="cuda")
    with pytest.raises(dfl.DFlashError) as e:   # the streaming kernels do not read this order
        ctx.gemm_fewrow(wt, dfl.TYPE_Q6_K_TILED, x, n_in, n_out)
    assert e.value.kind == "Unsupported" and "gemm_fewrow_xf" in str(e.value)
    bad = dfl.synth.extreme_blocks(dfl.synth.Q6_K, n_out * n_in // 256, seed=1).reshape(n_out, -1).copy()
    bad.view(np.uint8).reshape(-1, 210)[0, 208:210] = np.array([np.float16(128.0)]).view(np.uint8)   # |d| = 128: outside the f16 range
    with pytest.raises(dfl.DFlashError) as e:
        ctx.repack_q6k_tiled(dev(bad), n_in, n_out)
    assert e.value.kind == "Unsupported"


@pytest.mark.parametrize("qtype,tiled", [(dfl.synth.Q4_K, True), (dfl.synth.Q6_K, True), (dfl.synth.Q6_K, False)])
@pytest.mark.parametrize("n_in,n_out,rows", [(2048, 20000, 16), (1024, 9001, 5), (4096, 6000, 16)])
def test_many_rounds_of_tiles_take_the_looping_kernel(ctx, oracle, qtype, tiled, n_in, n_out, rows):
    """A matrix of many more tiles than one round of the chip (an output head) with K of at most 16 super-blocks: the
    looping kernel against f64 of the oracle's dequant, and - the same sums in the same order - bit for bit against
    the one-round kernel on the matrix's first rows."""
    blocks = dfl.synth.random_weight(qtype, n_out, n_in, seed=n_out)
    wd = dev(blocks)
    if qtype == dfl.synth.Q4_K:
        w, w_type = ctx.repack_q4k_tiled(wd, n_in, n_out), dfl.TYPE_Q4_K_TILED
    elif tiled:
        w, w_type = ctx.repack_q6k_tiled(wd, n_in, n_out), dfl.TYPE_Q6_K_TILED
    else:
        w, w_type = wd, ctx.checked_type(dfl.TYPE_Q6_K, wd)
    kind = ctx.xf_kind(w_type, n_in, n_out)
    assert kind != dfl.XF_NONE
    x = np.random.default_rng(rows).standard_normal((rows, n_in)).astype(np.float32)
    xf = ctx.pack_xf(dev(x), kind)
    y = ctx.gemm_fewrow_xf(w, w_type, xf, rows, n_in, n_out).cpu().numpy()
    wf = oracle.dequant(qtype, blocks, n_in * n_out).reshape(n_out, n_in).astype(np.float64)
    check(y, x.astype(np.float16).astype(np.float64) @ wf.T, f"loop {n_in}->{n_out} x{rows}")
    head_rows = 2048   # a matrix of the first rows alone fits one round
    hb = np.ascontiguousarray(blocks[:head_rows])
    hd = dev(hb)
    if qtype == dfl.synth.Q4_K:
        hw, ht = ctx.repack_q4k_tiled(hd, n_in, head_rows), dfl.TYPE_Q4_K_TILED
    elif tiled:
        hw, ht = ctx.repack_q6k_tiled(hd, n_in, head_rows), dfl.TYPE_Q6_K_TILED
    else:
        hw, ht = hd, ctx.checked_type(dfl.TYPE_Q6_K, hd)
    y1 = ctx.gemm_fewrow_xf(hw, ht, xf, rows, n_in, head_rows).cpu().numpy()
    assert np.array_equal(y1.view(np.uint32), y[:, :head_rows].view(np.uint32))


def test_rows_are_independent(ctx):
    """A row of the product depends on its own activation row only: a 16-row block and each row alone agree bit for
    bit (what makes a packed verify equal to token-by-token decoding through the same kernel)."""
    n_in, n_out = 2048, 5120
    for qtype in (dfl.synth.Q4_K, dfl.synth.Q6_K):
        w, w_type, _, _ = upload(ctx, qtype, n_in, n_out, seed=9)
        kind = ctx.xf_kind(w_type, n_in, n_out)
        x = dev(np.random.default_rng(3).standard_normal((16, n_in)).astype(np.float32))
        y = ctx.gemm_fewrow_xf(w, w_type, ctx.pack_xf(x, kind), 16, n_in, n_out).cpu().numpy()
        for r in (0, 7, 15):
            y1 = ctx.gemm_fewrow_xf(w, w_type, ctx.pack_xf(x[r:r + 1].contiguous(), kind), 1, n_in, n_out).cpu().numpy()
            assert np.array_equal(y1[0].view(np.uint32), y[r].view(np.uint32))


def test_shapes_outside_the_path_are_declined(ctx):
    import torch

    assert ctx.xf_kind(dfl.TYPE_Q4_K_TILED, 17408, 5120) == dfl.XF_NONE      # more than two stages per wave
    assert ctx.xf_kind(dfl.TYPE_Q6_K | dfl.TYPE_RANGE_CHECKED, 5120, 151936) == dfl.XF_NONE  # many rounds of the chip and K over 16 super-blocks
    assert ctx.xf_kind(dfl.TYPE_Q6_K | dfl.TYPE_RANGE_CHECKED, 2048, 151936) == dfl.XF_Q6K   # many rounds, short K: the looping kernel
    assert ctx.xf_kind(dfl.TYPE_Q6_K | dfl.TYPE_RANGE_CHECKED, 2048, 2048) == dfl.XF_Q6K
    assert ctx.xf_kind(dfl.TYPE_Q6_K, 2048, 2048) == dfl.XF_NONE             # not range-checked: these kernels scale in f16
    assert ctx.xf_kind(dfl.TYPE_Q4_K, 2048, 2048) == dfl.XF_NONE             # GGUF row order Q4_K: streaming kernels only
    assert ctx.xf_kind(dfl.TYPE_Q8_0, 2048, 2048) == dfl.XF_NONE
    buf = torch.zeros(1 << 20, dtype=torch.uint8, device="cuda")
    y = torch.zeros((16, 5120), dtype=torch.float32, device="cuda")
    with pytest.raises(dfl.DFlashError) as e:
        ctx.gemm_fewrow_xf(buf, dfl.TYPE_Q4_K_TILED, buf, 16, 17408, 5120, y=y)
    assert e.value.kind == "Unsupported"
    with pytest.raises(dfl.DFlashError) as e:
        ctx.pack_xf(torch.zeros((16, 300), device="cuda"), dfl.XF_Q4K)
    assert e.value.kind == "BadShape"
