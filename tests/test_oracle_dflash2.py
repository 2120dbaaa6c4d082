"""Pins of the oracle's DFlash-2 extras before anything is compared against them.

Selector walk: the known-answer walks of the reference's own tests
(metal_dflash/tests.rs:2978-3094: scores and predecessor tracking, first-tie rule, sentinel and
out-of-range candidates, non-finite scores, invalid predecessor), restated here as data.
Convolution (kernels/dflash2.metal:40-69): the reference holds no value test for it, so it is
pinned by what the formula fixes: a one-tap kernel is a product, rows before the block are
zeros, and the (side, tap, group) indexing is checked against an independent numpy gather."""
import numpy as np
import pytest


def f32_codebook(oracle, rows):
    rows = np.asarray(rows, np.float32)
    return oracle.make_codebook(oracle.F32, rows, rows.shape[1])


def test_walk_scores_and_tracks_predecessors(oracle):
    pred, k1 = f32_codebook(oracle, [[1, 2], [2, 0], [0, 3], [1, 1]])
    succ, k2 = f32_codebook(oracle, [[0, 0], [1, 1], [2, 0], [0, 1]])
    ids = [0, 0, 1, 2, 3, 1]
    tokens, scores, valid = oracle.select_draft_path(pred, succ, 2, 2, 0, 3, ids, [0.0] * 6, [0, 0, 2, 0.5, 1, 2])
    assert tokens.tolist() == [0, 2, 3]
    assert scores[1].tolist() == [3.0, 4.0]
    assert scores[2].tolist() == [6.0, 6.0]  # a tie: the first candidate (token 3) is kept
    assert valid[1:].all()


def test_walk_keeps_first_tie_and_skips_sentinels(oracle):
    pred, k1 = f32_codebook(oracle, [[1], [1]])
    succ, k2 = f32_codebook(oracle, [[0], [1]])
    ids = [0, 0, 0, 0, 1, 1, -1, 9]
    tokens, scores, valid = oracle.select_draft_path(pred, succ, 4, 1, 0, 2, ids, [0.0] * 8, [0, 1])
    assert tokens.tolist() == [0, 1]
    assert valid[1].tolist() == [1, 1, 0, 0]  # -1 and 9 (past the successor table) are not scored
    assert scores[1][:2].tolist() == [1.0, 1.0]


def test_walk_nonfinite_scores_and_no_valid_choice(oracle):
    pred, k1 = f32_codebook(oracle, [[1], [1], [1]])
    succ, k2 = f32_codebook(oracle, [[0], [0], [0]])
    ids = [0, 0, 1, 2, 1, 2]
    unary = [0, 0, np.inf, 0, np.nan, -np.inf]
    tokens, scores, valid = oracle.select_draft_path(pred, succ, 2, 1, 0, 3, ids, unary, [0, 1, 1])
    assert tokens.tolist() == [0, 1, 1]  # +inf wins at depth 0; at depth 1 nothing compares greater: candidate 0
    assert np.isposinf(scores[1][0]) and np.isnan(scores[2][0]) and np.isneginf(scores[2][1])


def test_walk_rejects_invalid_predecessor(oracle):
    pred, k1 = f32_codebook(oracle, [[1], [1]])
    succ, k2 = f32_codebook(oracle, [[0], [0], [1]])
    with pytest.raises(ValueError):
        oracle.select_draft_path(pred, succ, 1, 1, 0, 2, [0, 2], [0.0, 1.0], [0.0, 1.0])


def test_codebook_rows_match_whole_tensor_dequant(oracle):
    """Q4_K / Q8_0 codebook row == the same row of the whole-tensor dequant, bit for bit
    (the property metal_dflash/tests.rs:2797-2822 checks)."""
    import qwen_llm_amd as dfl

    for qtype, oq in ((dfl.synth.Q4_K, oracle.Q4_K), (dfl.synth.Q8_0, oracle.Q8_0)):
        rank, n_rows = 256, 37
        w = dfl.synth.random_weight(qtype, n_rows, rank, seed=3)
        whole = oracle.dequant(oq, w, rank * n_rows).reshape(n_rows, rank)
        cb, keep = oracle.make_codebook(oq, w, rank)
        for r in (0, 5, 36):
            assert np.array_equal(oracle.codebook_row(cb, r).view(np.uint32), whole[r].view(np.uint32))
        with pytest.raises(ValueError):
            oracle.codebook_row(cb, n_rows)


def test_conv_closed_forms(oracle):
    rng = np.random.default_rng(0)
    n, h, ks, gs = 8, 64, 2, 16
    ng = h // gs
    x = rng.standard_normal((n, h)).astype(np.float32)
    dyn = rng.standard_normal((n, 2 * ks * ng)).astype(np.float32)
    base = rng.standard_normal((2, ks, h)).astype(np.float32)
    for side in (0, 1):
        y = oracle.dflash2_conv(x, dyn, base, ks, gs, side)
        # independent gather: dyn is (group, tap, side) fastest to slowest per token
        d = dyn.reshape(n, 2, ks, ng)[:, side]                      # [n][tap][group]
        coef = base[side][None, :, :] + np.repeat(d, gs, axis=2)     # [n][tap][h]
        want0 = coef[:, 0] * x                                       # tap 0
        xprev = np.vstack([np.zeros((1, h), np.float32), x[:-1]])    # zero row before the block
        ref = want0.astype(np.float64) + coef[:, 1].astype(np.float64) * xprev
        assert np.allclose(y, ref, rtol=1e-6, atol=1e-6)
        assert np.array_equal(y[0], want0[0])  # row 0 has only tap 0: a single rounded product
    # one tap: y = (base + dyn) * x exactly
    dyn1 = rng.standard_normal((n, 2 * ng)).astype(np.float32)
    base1 = rng.standard_normal((2, 1, h)).astype(np.float32)
    y1 = oracle.dflash2_conv(x, dyn1, base1, 1, gs, 1)
    want = (base1[1, 0][None, :] + np.repeat(dyn1.reshape(n, 2, 1, ng)[:, 1, 0], gs, axis=1)) * x
    assert np.array_equal(y1, want.astype(np.float32))
