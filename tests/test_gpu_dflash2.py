"""GPU parity of the DFlash-2 extras against the CPU oracle: the two-tap dynamic convolution
(kernels/dflash2.metal:40-69) bit for bit, and the greedy selector walk (metal_dflash.rs:17176-17251)
token for token: on the reference's own known-answer walks (metal_dflash/tests.rs:2978-3094) and on
seeded random lattices with Q4_K, Q8_0, F16 and F32 codebooks at the released drafters' shape
(rank 256, top-16, 8 and 16 positions), sentinels and out-of-range candidates included."""
import numpy as np
import pytest

import qwen_llm_amd as dfl

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ctx():
    c = dfl.Context(0)
    yield c
    c.close()


@pytest.mark.parametrize("n,h,ks,gs", [(16, 2048, 2, 16), (8, 1024, 2, 16), (5, 96, 3, 8), (1, 64, 2, 16)])
def test_conv_bit_exact(ctx, oracle, n, h, ks, gs):
    import torch

    rng = np.random.default_rng(n * 1000 + h)
    x = rng.standard_normal((n, h)).astype(np.float32)
    dyn = rng.standard_normal((n, 2 * ks * (h // gs))).astype(np.float32)
    base = rng.standard_normal((2, ks, h)).astype(np.float32)
    for side in (0, 1):
        want = oracle.dflash2_conv(x, dyn, base, ks, gs, side)
        got = ctx.dflash2_conv(torch.from_numpy(x).cuda(), torch.from_numpy(dyn).cuda(), torch.from_numpy(base).cuda(), ks, gs,
                               side).cpu().numpy()
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), f"side {side}"


def test_conv_rejects_aliasing_and_bad_groups(ctx):
    import torch

    x = torch.zeros((4, 64), device="cuda")
    dyn = torch.zeros((4, 2 * 2 * 4), device="cuda")
    base = torch.zeros((2, 2, 64), device="cuda")
    L = dfl.lib()
    rc = L.dflash_dflash2_conv(ctx._h, x.data_ptr(), dyn.data_ptr(), base.data_ptr(), x.data_ptr(), 4, 64, 2, 16, 0, None)
    L.dflash_status_name.restype = __import__("ctypes").c_char_p
    assert L.dflash_status_name(rc) == b"Alias"
    rc = L.dflash_dflash2_conv(ctx._h, x.data_ptr(), dyn.data_ptr(), base.data_ptr(), dyn.data_ptr(), 4, 64, 2, 24, 0, None)
    assert rc != 0


def walk_gpu(ctx, pred, succ, rank, carry, ids, vals, sel_h):
    import torch

    def dev(pair):
        return pair[0], torch.from_numpy(np.ascontiguousarray(pair[1])).cuda()

    return ctx.select_draft_path(dev(pred), dev(succ), rank, carry, torch.from_numpy(np.asarray(ids, np.int32)).cuda(),
                                 torch.from_numpy(np.asarray(vals, np.float32)).cuda(),
                                 torch.from_numpy(np.asarray(sel_h, np.float32)).cuda())


def test_walk_reference_known_answers(ctx):
    f32 = lambda rows: (dfl.TYPE_F32, np.asarray(rows, np.float32))
    got = walk_gpu(ctx, f32([[1, 2], [2, 0], [0, 3], [1, 1]]), f32([[0, 0], [1, 1], [2, 0], [0, 1]]), 2, 0,
                   np.array([0, 0, 1, 2, 3, 1]).reshape(3, 2), np.zeros((3, 2)), np.array([0, 0, 2, 0.5, 1, 2]).reshape(3, 2))
    assert got == [0, 2, 3]
    got = walk_gpu(ctx, f32([[1], [1]]), f32([[0], [1]]), 1, 0, np.array([0, 0, 0, 0, 1, 1, -1, 9]).reshape(2, 4),
                   np.zeros((2, 4)), np.array([0, 1]).reshape(2, 1))
    assert got == [0, 1]
    got = walk_gpu(ctx, f32([[1], [1], [1]]), f32([[0], [0], [0]]), 1, 0, np.array([0, 0, 1, 2, 1, 2]).reshape(3, 2),
                   np.array([0, 0, np.inf, 0, np.nan, -np.inf]).reshape(3, 2), np.array([0, 1, 1]).reshape(3, 1))
    assert got == [0, 1, 1]
    with pytest.raises(dfl.DFlashError):
        walk_gpu(ctx, f32([[1], [1]]), f32([[0], [0], [1]]), 1, 0, np.array([0, 2]).reshape(2, 1), np.array([0.0, 1.0]).reshape(2, 1),
                 np.array([0.0, 1.0]).reshape(2, 1))


@pytest.mark.parametrize("kind", ["q4_k", "q8_0", "f16", "f32"])
@pytest.mark.parametrize("n", [8, 16])
def test_walk_matches_oracle_on_random_lattices(ctx, oracle, kind, n):
    rank, top_k, vocab = 256, 16, 4096
    for seed in range(6):
        rng = np.random.default_rng(100 * seed + n)
        if kind in ("q4_k", "q8_0"):
            qt = dfl.synth.Q4_K if kind == "q4_k" else dfl.synth.Q8_0
            tt = dfl.TYPE_Q4_K if kind == "q4_k" else dfl.TYPE_Q8_0
            ot = oracle.Q4_K if kind == "q4_k" else oracle.Q8_0
            pred_rows = dfl.synth.random_weight(qt, vocab, rank, seed=2 * seed)
            succ_rows = dfl.synth.random_weight(qt, vocab, rank, seed=2 * seed + 1)
        else:
            dt = np.float16 if kind == "f16" else np.float32
            tt = dfl.TYPE_F16 if kind == "f16" else dfl.TYPE_F32
            ot = oracle.F16 if kind == "f16" else oracle.F32
            pred_rows = (rng.standard_normal((vocab, rank)) * 0.05).astype(dt)
            succ_rows = (rng.standard_normal((vocab, rank)) * 0.05).astype(dt)
        ids = rng.integers(0, vocab, (n, top_k)).astype(np.int32)
        ids[rng.random((n, top_k)) < 0.1] = -1           # unfilled top-k sentinels
        ids[rng.random((n, top_k)) < 0.05] = vocab + 7   # past the table
        ids[:, 0] = rng.integers(0, vocab, n)            # candidate 0 stays a valid predecessor
        vals = np.sort(rng.standard_normal((n, top_k)).astype(np.float32), axis=1)[:, ::-1].copy()
        vals[:, 1] = vals[:, 0]                          # a tie in the unary logits
        sel_h = rng.standard_normal((n, rank)).astype(np.float32)
        carry = int(rng.integers(0, vocab))
        pc, k1 = oracle.make_codebook(ot, pred_rows, rank)
        sc, k2 = oracle.make_codebook(ot, succ_rows, rank)
        want, _, _ = oracle.select_draft_path(pc, sc, top_k, rank, carry, n, ids, vals, sel_h)
        got = walk_gpu(ctx, (tt, pred_rows), (tt, succ_rows), rank, carry, ids, vals, sel_h)
        assert got == want.tolist(), f"{kind} n={n} seed={seed}"


@pytest.mark.parametrize("pred_kind,succ_kind,rank", [("q8_0", "q8_0", 32), ("q8_0", "f32", 96), ("f16", "q8_0", 160),
                                                      ("f16", "f16", 33), ("f32", "f16", 7), ("q4_k", "q8_0", 1024)])
def test_walk_with_rows_on_two_byte_boundaries_and_mixed_codebooks(ctx, oracle, pred_kind, succ_kind, rank):
    """Q8_0 rows of an odd number of blocks (34 bytes each) and F16 rows of an odd rank start on 2-byte boundaries only;
    the two codebooks may have different types; rank 1024 is the largest the walk takes."""
    top_k, vocab, n = 16, 512, 16

    def book(kind, seed, rng):
        if kind in ("q4_k", "q8_0"):
            qt = dfl.synth.Q4_K if kind == "q4_k" else dfl.synth.Q8_0
            return ((dfl.TYPE_Q4_K if kind == "q4_k" else dfl.TYPE_Q8_0), (oracle.Q4_K if kind == "q4_k" else oracle.Q8_0),
                    dfl.synth.random_weight(qt, vocab, rank, seed=seed))
        dt = np.float16 if kind == "f16" else np.float32
        return ((dfl.TYPE_F16 if kind == "f16" else dfl.TYPE_F32), (oracle.F16 if kind == "f16" else oracle.F32),
                (rng.standard_normal((vocab, rank)) * 0.05).astype(dt))

    for seed in range(3):
        rng = np.random.default_rng(7000 + 10 * seed + rank)
        pt, po, pred_rows = book(pred_kind, 2 * seed, rng)
        st, so, succ_rows = book(succ_kind, 2 * seed + 1, rng)
        ids = rng.integers(0, vocab, (n, top_k)).astype(np.int32)
        ids[rng.random((n, top_k)) < 0.1] = -1
        ids[:, 0] = rng.integers(0, vocab, n)
        vals = np.sort(rng.standard_normal((n, top_k)).astype(np.float32), axis=1)[:, ::-1].copy()
        sel_h = rng.standard_normal((n, rank)).astype(np.float32)
        carry = int(rng.integers(0, vocab))
        pc, k1 = oracle.make_codebook(po, pred_rows, rank)
        sc, k2 = oracle.make_codebook(so, succ_rows, rank)
        want, _, _ = oracle.select_draft_path(pc, sc, top_k, rank, carry, n, ids, vals, sel_h)
        got = walk_gpu(ctx, (pt, pred_rows), (st, succ_rows), rank, carry, ids, vals, sel_h)
        assert got == want.tolist(), f"{pred_kind}/{succ_kind} rank={rank} seed={seed}"


@pytest.mark.parametrize("kind", ["q4_k", "f32"])
def test_sampled_walk_matches_oracle(ctx, oracle, kind):
    """draft_block_sampled (metal_dflash.rs:17268-17415): tokens, the sparse proposals (candidate token ids in
    distribution order, weights to the last place of the f64 exponential) and the proposal sampler's stream position, against the oracle's
    restatement (its sampler chain is pinned by tests/test_oracle_pins.py), over seeded lattices with sentinels."""
    rank, top_k, vocab, n = 256, 16, 2048, 16
    for seed in range(8):
        rng = np.random.default_rng(7000 + seed)
        if kind == "q4_k":
            tt, ot = dfl.TYPE_Q4_K, oracle.Q4_K
            pred_rows = dfl.synth.random_weight(dfl.synth.Q4_K, vocab, rank, seed=2 * seed)
            succ_rows = dfl.synth.random_weight(dfl.synth.Q4_K, vocab, rank, seed=2 * seed + 1)
        else:
            tt, ot = dfl.TYPE_F32, oracle.F32
            pred_rows = (rng.standard_normal((vocab, rank)) * 0.05).astype(np.float32)
            succ_rows = (rng.standard_normal((vocab, rank)) * 0.05).astype(np.float32)
        ids = np.stack([rng.permutation(vocab)[:top_k] for _ in range(n)]).astype(np.int32)
        ids[rng.random((n, top_k)) < 0.1] = -1
        ids[:, 0] = rng.integers(0, vocab, n)
        vals = np.sort(rng.standard_normal((n, top_k)).astype(np.float32) * 2, axis=1)[:, ::-1].copy()
        sel_h = rng.standard_normal((n, rank)).astype(np.float32)
        carry = int(rng.integers(0, vocab))
        temperature = [0.7, 1.0, 0.3][seed % 3]
        osamp = oracle.make_sampler(temperature=temperature, top_k=0, top_p=1.0, min_p=0.0, seed=99 + seed)
        pc, k1 = oracle.make_codebook(ot, pred_rows, rank)
        sc, k2 = oracle.make_codebook(ot, succ_rows, rank)
        rc, want_tokens, want_props, _ = oracle.select_draft_path_sampled(pc, sc, top_k, rank, carry, n, ids, vals, sel_h, osamp)
        assert rc == 0
        gsamp = dfl.Sampler(temperature=temperature, top_k=0, top_p=1.0, min_p=0.0, seed=99 + seed)
        import torch

        got_tokens, got_props = ctx.select_draft_path_sampled(
            (tt, torch.from_numpy(pred_rows).cuda()), (tt, torch.from_numpy(succ_rows).cuda()), rank, carry,
            torch.from_numpy(ids).cuda(), torch.from_numpy(vals).cuda(), torch.from_numpy(sel_h).cuda(), gsamp)
        assert got_tokens == want_tokens.tolist(), f"{kind} seed {seed}"
        assert gsamp.draws == int(osamp.draws) == n - 1
        for p in range(n - 1):
            tok, cands = got_props[p]
            assert tok == want_tokens[p + 1]
            assert [t for t, _ in cands] == [t for t, _ in want_props[p]], f"{kind} seed {seed} position {p + 1}"
            # f64 exp on the device and in the host libm may differ in the last place
            gw, ww = np.array([w for _, w in cands]), np.array([w for _, w in want_props[p]])
            assert np.allclose(gw, ww, rtol=1e-12, atol=0.0), f"{kind} seed {seed} position {p + 1}: {np.max(np.abs(gw - ww) / ww)} {gw} {ww}"


def test_sampled_walk_rejects_target_filters(ctx):
    import torch

    rows = torch.zeros((4, 32), device="cuda")
    ids = torch.zeros((2, 2), dtype=torch.int32, device="cuda")
    vals = torch.zeros((2, 2), device="cuda")
    h = torch.zeros((2, 32), device="cuda")
    for bad in (dict(temperature=0.0), dict(temperature=0.7, top_k=20), dict(temperature=0.7, top_p=0.9),
                dict(temperature=0.7, min_p=0.1)):
        with pytest.raises(dfl.DFlashError):
            ctx.select_draft_path_sampled((dfl.TYPE_F32, rows), (dfl.TYPE_F32, rows), 32, 0, ids, vals, h, dfl.Sampler(seed=1, **bad))
