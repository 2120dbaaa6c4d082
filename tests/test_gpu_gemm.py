"""GPU parity: block dequantisation (bit-exact) and the few-row quantised GEMM
(<= 1e-2 relative, f32 accumulation) against the CPU oracle, through the C ABI."""
import numpy as np
import pytest

import qwen_llm_amd as dfl

pytestmark = pytest.mark.gpu

QTYPES = [dfl.synth.Q4_K, dfl.synth.Q6_K, dfl.synth.Q8_0]


@pytest.fixture(scope="module")
def ctx():
    c = dfl.Context(0)
    yield c
    c.close()


def dev(a):
    import torch

    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def gemm_fast(ctx, w, qtype, x, n_in, n_out):
    """The few-row GEMM through the fast kernels: the tensor is range-checked first, as a loader must, and tagged."""
    return ctx.gemm_fewrow(w, ctx.checked_type(qtype, w), x, n_in, n_out)


@pytest.mark.parametrize("qtype", QTYPES)
@pytest.mark.parametrize("kind", ["random", "extreme", "quantised"])
def test_dequant_bit_exact(ctx, oracle, qtype, kind):
    """codec.rs:474-577 / q6_k_f32_tile.rs:46-107: every element identical to ggml's value"""
    n_blocks = 1031
    be = dfl.synth.BLOCK_ELEMS[qtype]
    if kind == "random":
        blocks = dfl.synth.random_blocks(qtype, n_blocks, seed=1)
    elif kind == "extreme":
        blocks = dfl.synth.extreme_blocks(qtype, n_blocks, seed=2)
    else:
        w = (np.random.default_rng(3).standard_normal((n_blocks, be)) * 0.02).astype(np.float32)
        blocks = dfl.synth.quantize(qtype, w)
    want = oracle.dequant(qtype, blocks, n_blocks * be)
    got = ctx.dequant_to_f32(qtype, dev(blocks), n_blocks * be).cpu().numpy()
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


def test_dequant_rejects_bad_geometry(ctx):
    import torch

    buf = torch.zeros(144, dtype=torch.uint8, device="cuda")
    with pytest.raises(dfl.DFlashError) as e:
        ctx.dequant_to_f32(dfl.TYPE_Q4_K, buf, 100)
    assert e.value.kind == "BadShape"
    with pytest.raises(dfl.DFlashError) as e:
        ctx.dequant_to_f32(3, buf, 256)
    assert e.value.kind == "Unsupported"


def check_gemm(y, ref, label):
    """north-star bar: <= 1e-2 relative (norm-wise and element-wise against max(|ref|, rms));
    the reference's own bar (metal/mat_mat.rs:4285-4309) is reported alongside."""
    y = y.astype(np.float64)
    assert np.all(np.isfinite(y)), f"{label}: non-finite output"
    rel_l2 = np.linalg.norm(y - ref) / max(np.linalg.norm(ref), 1e-30)
    rms = np.sqrt(np.mean(ref ** 2))
    elem = np.max(np.abs(y - ref) / np.maximum(np.abs(ref), rms))
    assert rel_l2 <= 1e-2 and elem <= 1e-2, f"{label}: rel_l2 {rel_l2:.3e} elem {elem:.3e}"
    max_ref = np.max(np.abs(ref))
    atol, rtol = 1e-3 * max(max_ref, 1.0), 5e-3
    assert np.all(np.abs(y - ref) <= atol + rtol * np.abs(ref)), f"{label}: reference tolerance"
    if y.size >= 64:  # an RMS over a handful of outputs is a single-element bound, covered above
        assert rel_l2 <= 2e-3, f"{label}: RMS relative error {rel_l2:.3e}"
    return rel_l2


def f64_reference(oracle, qtype, w, x, n_in, n_out):
    wf = oracle.dequant(qtype, w, n_in * n_out).reshape(n_out, n_in).astype(np.float64)
    return x.astype(np.float64) @ wf.T


SHAPES = [(256, 16, 16), (256, 1, 1), (512, 17, 3), (1024, 33, 16), (2560, 100, 8), (5120, 64, 16), (768, 2049, 5),
          (4352, 130, 16), (256, 8, 9)]


@pytest.mark.parametrize("qtype", QTYPES)
@pytest.mark.parametrize("n_in,n_out,n_rows", SHAPES)
@pytest.mark.parametrize("x_dtype", ["f32", "f16"])
def test_gemm_fewrow_small_shapes(ctx, oracle, qtype, n_in, n_out, n_rows, x_dtype, canaries):
    """tile edges, ragged n_out, every row count class, random + extreme blocks"""
    rng = np.random.default_rng(n_in * 31 + n_out * 7 + n_rows)
    nblk = n_in // dfl.synth.BLOCK_ELEMS[qtype] * n_out
    w = dfl.synth.random_blocks(qtype, nblk, seed=n_out)
    x = rng.standard_normal((n_rows, n_in)).astype(np.float32)
    if x_dtype == "f16":
        x = x.astype(np.float16)
    ref = f64_reference(oracle, qtype, w, x.astype(np.float32), n_in, n_out)
    y = gemm_fast(ctx, dev(w), qtype, dev(x), n_in, n_out).cpu().numpy()
    check_gemm(y, ref, f"q{qtype} {n_in}x{n_out}x{n_rows} {x_dtype}")


@pytest.mark.parametrize("qtype", QTYPES)
def test_gemm_fewrow_extreme_blocks(ctx, oracle, qtype, canaries):
    """metal/mat_mat.rs:4228-4265: large minima / saturated codes must stay finite and accurate"""
    n_in, n_out, n_rows = 1024, 48, 16
    nblk = n_in // dfl.synth.BLOCK_ELEMS[qtype] * n_out
    w = dfl.synth.extreme_blocks(qtype, nblk, seed=5)
    x = np.random.default_rng(5).standard_normal((n_rows, n_in)).astype(np.float32)
    ref = f64_reference(oracle, qtype, w, x, n_in, n_out)
    y = gemm_fast(ctx, dev(w), qtype, dev(x), n_in, n_out).cpu().numpy()
    check_gemm(y, ref, f"extreme q{qtype}")


def test_gemm_matches_oracle_f32_path(ctx, oracle):
    """the oracle's own f32 dequant + mat_vec (forward.rs:1321-1334) on the same bytes"""
    n_in, n_out, n_rows = 2048, 96, 16
    w = dfl.synth.random_weight(dfl.synth.Q4_K, n_out, n_in, seed=1)
    x = np.random.default_rng(1).standard_normal((n_rows, n_in)).astype(np.float32)
    want = oracle.gemm_fewrow(dfl.synth.Q4_K, w, x, n_in, n_out)
    got = gemm_fast(ctx, dev(w), dfl.synth.Q4_K, dev(x), n_in, n_out).cpu().numpy()
    rms = np.sqrt(np.mean(want.astype(np.float64) ** 2))
    assert np.max(np.abs(got - want) / np.maximum(np.abs(want), rms)) <= 1e-2


def test_gemm_deterministic_and_linear(ctx):
    """size-independent properties at a full-size shape: run-to-run identical bits; linear in X"""
    import torch

    n_in, n_out = 5120, 6144
    w = dev(dfl.synth.random_weight(dfl.synth.Q4_K, n_out, n_in, seed=1))
    g = torch.Generator(device="cuda").manual_seed(1)
    x1 = torch.randn((16, n_in), device="cuda", generator=g, dtype=torch.float32).half()
    x2 = torch.randn((16, n_in), device="cuda", generator=g, dtype=torch.float32).half()
    y1 = gemm_fast(ctx, w, dfl.TYPE_Q4_K, x1, n_in, n_out)
    y1b = gemm_fast(ctx, w, dfl.TYPE_Q4_K, x1, n_in, n_out)
    assert torch.equal(y1, y1b)
    y2 = gemm_fast(ctx, w, dfl.TYPE_Q4_K, x2, n_in, n_out)
    xs = (x1.float() + x2.float())
    ys = gemm_fast(ctx, w, dfl.TYPE_Q4_K, xs, n_in, n_out)
    scale = ys.abs().max().item()
    assert (ys - (y1 + y2)).abs().max().item() <= 4e-3 * scale


@pytest.mark.parametrize("qtype", [dfl.synth.Q4_K, dfl.synth.Q6_K])
@pytest.mark.parametrize("n_in,n_out", [(2048, 5120), (4096, 2048), (2048, 12288), (6144, 2048)])
def test_gemm_small_split_k_repeats(ctx, oracle, qtype, n_in, n_out, canaries):
    """Products of a few MB (the projections of a decoder layer) are split over K across workgroups, their
    partial tiles living in a scratch buffer that every launch shares.  Forty launches in a row, alternating
    with another shape: every result bit-identical to the first and within the GEMM bar of the f64 reference."""
    import torch

    w = dev(dfl.synth.random_weight(qtype, n_out, n_in, seed=5))
    w2 = dev(dfl.synth.random_weight(qtype, 1024, 2048, seed=6))
    g = torch.Generator(device="cuda").manual_seed(2)
    x = torch.randn((16, n_in), device="cuda", generator=g, dtype=torch.float32)
    x2 = torch.randn((16, 2048), device="cuda", generator=g, dtype=torch.float32)
    first = gemm_fast(ctx, w, qtype, x, n_in, n_out).clone()
    other = gemm_fast(ctx, w2, qtype, x2, 2048, 1024).clone()
    for _ in range(20):
        assert torch.equal(gemm_fast(ctx, w, qtype, x, n_in, n_out), first)
        assert torch.equal(gemm_fast(ctx, w2, qtype, x2, 2048, 1024), other)
    ref = f64_reference(oracle, qtype, w.cpu().numpy(), x.cpu().numpy(), n_in, n_out)
    check_gemm(first.cpu().numpy(), ref, f"split-K {n_in}x{n_out}")


@pytest.mark.parametrize("n_in,n_out", [(5120, 17408), (17408, 5120), (5120, 6144)])
def test_gemm_fewrow_full_size_q4k(ctx, oracle, n_in, n_out):
    """the three production shapes, X f16 N(0,1), W = Q4_K(N(0,0.02)), seed 1; checked on a
    sample of output columns against the f64 reference (the oracle takes seconds per 256 rows)"""
    w = dfl.synth.random_weight(dfl.synth.Q4_K, n_out, n_in, seed=1)
    x = np.random.default_rng(1).standard_normal((16, n_in)).astype(np.float16)
    y = gemm_fast(ctx, dev(w), dfl.synth.Q4_K, dev(x), n_in, n_out).cpu().numpy()
    rows = np.unique(np.concatenate([np.arange(0, 64), np.arange(n_out - 64, n_out),
                                     np.random.default_rng(2).integers(0, n_out, 384)]))
    ref = f64_reference(oracle, dfl.synth.Q4_K, w[rows], x.astype(np.float32), n_in, len(rows))
    check_gemm(y[:, rows], ref, f"full {n_in}x{n_out}")


def test_gemm_guards(ctx):
    """dispatch.rs:256-327, 522-526: shape / alias / dtype refusals are errors, not crashes"""
    import torch

    w = torch.zeros(16 * 144, dtype=torch.uint8, device="cuda")
    x = torch.zeros((17, 256), device="cuda")
    y = torch.zeros((17, 16), device="cuda")
    with pytest.raises(dfl.DFlashError) as e:
        ctx.encode_mat_mat_dispatch_dflash_verify(w, dfl.TYPE_Q4_K, x, y, 256, 16, 17)
    assert e.value.kind == "BadShape"
    with pytest.raises(dfl.DFlashError) as e:
        ctx.encode_mat_mat_dispatch_dflash_verify(w, dfl.TYPE_Q4_K, x, y, 100, 16, 4)
    assert e.value.kind == "BadShape"
    with pytest.raises(dfl.DFlashError) as e:
        ctx.encode_mat_mat_dispatch_dflash_verify(w, 3, x, y, 256, 16, 4)
    assert e.value.kind == "Unsupported"
    xy = torch.zeros(4 * 256, device="cuda")
    with pytest.raises(dfl.DFlashError) as e:
        ctx.encode_mat_mat_dispatch_dflash_verify(w, dfl.TYPE_Q4_K, xy, xy, 256, 16, 4)
    assert e.value.kind == "Alias"


TILED_SHAPES = [(256, 16, 16), (256, 250, 3), (768, 257, 16), (1024, 4096, 7), (1280, 1000, 16), (2048, 5120, 1),
                (5120, 6144, 16), (5120, 17408, 16), (17408, 5120, 16),
                (2048, 50000, 16), (8192, 16384, 5)]  # the last two: ranges longer than six stages (the per-stage-barrier kernel)


@pytest.mark.parametrize("n_in,n_out,n_rows", TILED_SHAPES)
@pytest.mark.parametrize("x_dtype", ["f32", "f16"])
def test_gemm_q4k_tiled_order_is_bit_identical(ctx, n_in, n_out, n_rows, x_dtype, canaries):
    """The one-time repack into tiled order permutes whole blocks: the GEMM on it must give the very bits the GEMM on
    GGUF row order gives (ragged n_out, ranges that wrap over tile groups, every row count), and the padding rows of
    the last tile group must leave the output alone (guard bands around Y)."""
    import torch
    rng = np.random.default_rng(n_in + n_out + n_rows)
    w = dfl.synth.random_blocks(dfl.synth.Q4_K, n_out * n_in // 256, n_in + n_out)
    x = rng.standard_normal((n_rows, n_in)).astype(np.float32 if x_dtype == "f32" else np.float16)
    wd, xd = dev(w), dev(x)
    want = gemm_fast(ctx, wd, dfl.TYPE_Q4_K, xd, n_in, n_out)
    wt = ctx.repack_q4k_tiled(wd, n_in, n_out)
    guard = 64
    buf = torch.full((n_rows * n_out + 2 * guard,), float("nan"), dtype=torch.float32, device="cuda")
    y = buf[guard:guard + n_rows * n_out].view(n_rows, n_out)
    ctx.encode_mat_mat_dispatch_dflash_verify(wt, dfl.TYPE_Q4_K_TILED, xd, y, n_in, n_out, n_rows)
    torch.cuda.synchronize()
    assert torch.equal(y.view(torch.int32), want.view(torch.int32))
    assert torch.isnan(buf[:guard]).all() and torch.isnan(buf[-guard:]).all()


def test_q4k_tiled_repack_layout(ctx):
    """Block (row r, super-block b) of the row-order matrix sits at [r // 256][b][r % 256] of the tiled one; rows
    past n_out are zero blocks."""
    n_in, n_out = 768, 300
    nb = n_in // 256
    w = dfl.synth.random_blocks(dfl.synth.Q4_K, n_out * nb, 5)
    wt = ctx.repack_q4k_tiled(dev(w), n_in, n_out).cpu().numpy()
    groups = (n_out + 255) // 256
    assert wt.size == groups * nb * 256 * 144
    src = np.zeros((groups * 256, nb, 144), np.uint8)
    src[:n_out] = np.asarray(w).reshape(n_out, nb, 144)
    want = src.reshape(groups, 256, nb, 144).transpose(0, 2, 1, 3)
    assert np.array_equal(wt.reshape(groups, nb, 256, 144), want)


def test_q4k_tiled_guards(ctx):
    import torch
    n_in, n_out = 512, 64
    w = dev(dfl.synth.random_blocks(dfl.synth.Q4_K, n_out * n_in // 256, 1))
    with pytest.raises(dfl.DFlashError):
        ctx.repack_q4k_tiled(w, 500, n_out)
    wt = ctx.repack_q4k_tiled(w, n_in, n_out)
    x = torch.zeros((4, n_in), dtype=torch.float32, device="cuda")
    y = torch.empty((4, n_out), dtype=torch.float32, device="cuda")
    with pytest.raises(dfl.DFlashError):  # misaligned tiled weights
        ctx.encode_mat_mat_dispatch_dflash_verify(wt[16:], dfl.TYPE_Q4_K_TILED, x, y, n_in, n_out, 4)


@pytest.mark.parametrize("qtype", QTYPES)
def test_gemm_fewrow_reference_extreme_blocks(ctx, oracle, qtype, canaries):
    """The reference's own extreme blocks (metal/mat_mat.rs:4228-4265: d = 0.001, Q4_K dmin = 5, alternating 0x00 / 0xFF
    bytes, the pattern shifted from block to block) at a ragged shape, against the f64 product."""
    n_in, n_out, n_rows = 1024, 45, 13
    nblk = n_in // dfl.synth.BLOCK_ELEMS[qtype] * n_out
    w = dfl.synth.reference_extreme_blocks(qtype, nblk)
    x = np.random.default_rng(9).standard_normal((n_rows, n_in)).astype(np.float32)
    ref = f64_reference(oracle, qtype, w, x, n_in, n_out)
    y = gemm_fast(ctx, dev(w), qtype, dev(x), n_in, n_out).cpu().numpy()
    check_gemm(y, ref, f"reference extreme q{qtype}")


def _with_scales(qtype, n_blocks, d, dmin=None):
    w = dfl.synth.random_blocks(qtype, n_blocks, 3).copy()
    off = {dfl.synth.Q4_K: 0, dfl.synth.Q6_K: 208}[qtype]
    w[:, off:off + 2] = np.full(1, d, np.float16).view(np.uint8)
    if dmin is not None:
        w[:, 2:4] = np.full(1, dmin, np.float16).view(np.uint8)
    return w


def test_scale_range_guard(ctx, oracle):
    """A tensor whose super-block scales leave the f16 range of the few-row kernels is declined when it is uploaded
    (never computed to infinities); at the limits the product is still right."""
    n_in, n_out = 512, 32
    nblk = n_in // 256 * n_out
    x = np.random.default_rng(2).standard_normal((16, n_in)).astype(np.float32)
    # at the documented limits: accepted and accurate
    for qtype, d, dmin in ((dfl.synth.Q4_K, 1.0, 32.0), (dfl.synth.Q4_K, -1.0, -32.0), (dfl.synth.Q6_K, 0.25, None)):
        w = _with_scales(qtype, nblk, d, dmin)
        md, mm = ctx.check_scale_range(qtype, dev(w), nblk)
        assert md == abs(d) and (dmin is None or mm == abs(dmin))
        y = gemm_fast(ctx, dev(w), qtype, dev(x), n_in, n_out).cpu().numpy()
        assert np.all(np.isfinite(y))
        check_gemm(y, f64_reference(oracle, qtype, w, x, n_in, n_out), f"limit q{qtype} d={d}")
    # beyond them: declined with a message that names the figure
    for qtype, d, dmin in ((dfl.synth.Q4_K, 128.0, 0.5), (dfl.synth.Q4_K, 0.01, 64.0), (dfl.synth.Q6_K, 128.0, None),
                           (dfl.synth.Q4_K, np.inf, 0.5), (dfl.synth.Q4_K, np.nan, 0.5)):
        w = _with_scales(qtype, nblk, d, dmin)
        with pytest.raises(dfl.DFlashError) as e:
            ctx.check_scale_range(qtype, dev(w), nblk)
        assert e.value.status == 2 and "declined" in str(e.value)
    # one bad block among many is found
    w = _with_scales(dfl.synth.Q4_K, 4096, 0.01, 0.02)
    w[3071, 0:2] = np.full(1, 128.0, np.float16).view(np.uint8)
    with pytest.raises(dfl.DFlashError):
        ctx.check_scale_range(dfl.synth.Q4_K, dev(w), 4096)
    # types without the limit pass
    assert ctx.check_scale_range(dfl.synth.Q8_0, dev(dfl.synth.random_blocks(dfl.synth.Q8_0, 64, 1)), 64) == (0.0, 0.0)


def test_model_upload_declines_out_of_range_tensor(ctx):
    """The guard sits in the upload path of the host mirror: a model with one |d| = 128 block does not load."""
    cfg = dfl.ModelConfig(n_layers=1, hidden=256, n_q=4, n_kv=2, head_dim=64, ffn=512, vocab=512)
    w = dfl.synth_target_weights(cfg, seed=3)
    qtype, blocks = w["layers"][0]["wo"]
    blocks = np.array(blocks, copy=True)
    flat = blocks.reshape(-1, dfl.synth.BLOCK_BYTES[qtype])
    off = {dfl.synth.Q4_K: 0, dfl.synth.Q6_K: 208, dfl.synth.Q8_0: 0}[qtype]
    flat[5, off:off + 2] = np.full(1, 128.0, np.float16).view(np.uint8)
    w["layers"][0]["wo"] = (qtype, blocks)
    if qtype == dfl.synth.Q8_0:
        pytest.skip("synthetic wo is Q8_0: no f16-range limit")
    with pytest.raises(dfl.DFlashError):
        dfl.TargetModel(ctx, cfg, w)


def test_model_with_an_untagged_tensor_is_declined(ctx):
    """The model-level calls use the fast kernels only, so a Q4_K / Q6_K tensor whose descriptor lacks the
    range-checked flag (a loader that skipped dflash_check_scale_range) is declined by name, before any launch."""
    cfg = dfl.ModelConfig(n_layers=2, hidden=256, n_q=4, n_kv=2, head_dim=64, ffn=512, vocab=512)
    model = dfl.TargetModel(ctx, cfg, dfl.synth_target_weights(cfg, seed=3), tiled=False)
    sess = dfl.Session(ctx, model, 64, [0])
    try:
        sess.encode_packed_verify_layer_major([1, 2, 3], 0)  # as uploaded: fine
        sess.encode_restore_after_partial_accept(0, 3, 0)
        down = model._layers[1].down
        if down.type not in (dfl.TYPE_Q4_K, dfl.TYPE_Q6_K):
            pytest.skip("the synthetic down projection went into the tiled order (checked by construction)")
        down.flags = 0
        with pytest.raises(dfl.DFlashError) as e:
            sess.encode_packed_verify_layer_major([1, 2, 3], 0)
        assert e.value.kind == "Unsupported" and "down (layer 1)" in str(e.value)
    finally:
        sess.close()


@pytest.mark.parametrize("qtype", [dfl.synth.Q4_K, dfl.synth.Q6_K])
@pytest.mark.parametrize("x_dtype", [np.float32, np.float16])
def test_untagged_tensor_takes_the_f32_kernel_and_any_block(ctx, oracle, qtype, x_dtype, canaries):
    """The seam's contract (dispatch.rs:365-378; the reference scales in f32 after the MMA,
    mat_mat_fewrow_gen.metal:437-444): a tensor that nobody range-checked is computed correctly whatever its blocks
    hold - here super-block scales of +-128 and +-60000, far outside the fast kernels' f16 range - by ggml's f32
    dequantisation and f32 sums; never infinities with status OK."""
    n_in, n_out, n_rows = 1024, 77, 13
    nblk = n_in // 256 * n_out
    w = dfl.synth.random_blocks(qtype, nblk, 11).copy()
    off = {dfl.synth.Q4_K: 0, dfl.synth.Q6_K: 208}[qtype]
    d = np.where(np.arange(nblk) % 3 == 0, 128.0, np.where(np.arange(nblk) % 3 == 1, -60000.0, 0.03)).astype(np.float16)
    w[:, off:off + 2] = d.view(np.uint8).reshape(nblk, 2)
    if qtype == dfl.synth.Q4_K:
        w[:, 2:4] = np.full(nblk, 200.0, np.float16).view(np.uint8).reshape(nblk, 2)
    wd = dev(w)
    with pytest.raises(dfl.DFlashError):  # a loader that asks is told; the tag cannot be earned
        ctx.checked_type(qtype, wd)
    x = np.random.default_rng(4).standard_normal((n_rows, n_in)).astype(x_dtype)
    y = ctx.gemm_fewrow(wd, qtype, dev(x), n_in, n_out).cpu().numpy()
    canaries.check()
    ref = f64_reference(oracle, qtype, w, x.astype(np.float32), n_in, n_out)
    assert np.all(np.isfinite(y))
    assert np.max(np.abs(y - ref)) <= 2e-5 * np.max(np.abs(ref))
    # and on an ordinary tensor the two paths agree to the fast kernels' f16-operand tolerance
    w2 = dfl.synth.random_weight(qtype, n_out, n_in, seed=12)
    w2d = dev(w2)
    y_safe = ctx.gemm_fewrow(w2d, qtype, dev(x), n_in, n_out).cpu().numpy()
    y_fast = gemm_fast(ctx, w2d, qtype, dev(x), n_in, n_out).cpu().numpy()
    check_gemm(y_fast, y_safe.astype(np.float64), "fast against f32 kernel")


def test_repack_declines_a_tensor_out_of_range(ctx):
    """The tiled order goes to the fast kernels unconditionally, so the repack checks the range itself."""
    n_in, n_out = 512, 256
    w = _with_scales(dfl.synth.Q4_K, n_in // 256 * n_out, 128.0, 0.5)
    with pytest.raises(dfl.DFlashError) as e:
        ctx.repack_q4k_tiled(dev(w), n_in, n_out)
    assert e.value.status == 2
