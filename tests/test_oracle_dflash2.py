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


def test_dflash2_drafter_with_identity_convolutions_is_the_dflash1_drafter(oracle):
    """Pins the wiring of the DFlash-2 drafter restatement (orc_dflash_draft_ex; draft_block_inner with
    layer.conv, metal_dflash.rs:16210-16262, 16795-16885, 17003-17022) against the DFlash-1 forward
    (Forward::dflash_draft, forward.rs:380-662), which the drafter parity tests pin: with zero coefficient
    projections and base kernels that are the identity tap, every convolution returns its input bit for
    bit (fma(1, x, 0) and fma(0, x', acc)), so the logits must be bit-identical.  A second run with a
    non-trivial base kernel must differ (the convolutions are really on the path), and the selector gate
    must equal selector_hidden applied to the output-normed hidden."""
    import qwen_llm_amd as dfl

    C1 = dfl.ModelConfig(n_layers=1, hidden=256, n_q=4, n_kv=2, head_dim=64, ffn=512, vocab=512)
    D2 = dfl.DraftConfig(n_layers=2, hidden=256, n_q=4, n_kv=2, head_dim=64, ffn=512, block_size=8, n_taps=2,
                         conv_kernel_size=2, conv_group_size=32, selector_rank=64, selector_top_k=16)
    w = dfl.synth_target_weights(C1, seed=1)
    dw = dfl.synth_draft_weights(D2, seed=2, vocab=C1.vocab, codebook_type=dfl.synth.Q8_0)
    omodel, _k = oracle.build_model(C1.as_dict(), w)
    ohead, _k2 = oracle.build_draft_head(D2.as_dict(), dw)
    rng = np.random.default_rng(4)
    ctx_len = 5
    ctx = rng.standard_normal((ctx_len, D2.n_taps * D2.hidden)).astype(np.float32)
    ids = [7] + [C1.vocab - 1] * (D2.block_size - 1)
    plain = oracle.dflash_draft(omodel, ohead, ids, ctx, list(range(ctx_len)), ctx_len)

    ident = {**dw, "layers": []}
    for L in dw["layers"]:
        base = np.zeros((2, 2, D2.hidden), np.float32)
        base[:, 0, :] = 1.0
        zero = (L["conv_attn_proj"][0], np.zeros_like(L["conv_attn_proj"][1]))
        ident["layers"].append({**L, "conv_attn_proj": zero, "conv_ffn_proj": zero, "conv_attn_base": base,
                                "conv_ffn_base": base})
    ext, _k3 = oracle.build_dflash2_ext(D2.as_dict(), ident)
    got, sel_h = oracle.dflash_draft_ex(omodel, ohead, ext, ids, ctx, list(range(ctx_len)), ctx_len)
    assert np.array_equal(got.view(np.uint32), plain.view(np.uint32))
    assert sel_h.shape == (D2.block_size, 64) and np.all(np.isfinite(sel_h)) and np.abs(sel_h).max() > 0

    # Which side sits where: side 0 the identity, side 1 a per-channel scaling by 1 or 2.  Scaling a
    # sublayer's OUTPUT channel c by a power of two is exactly the DFlash-1 forward with row c of wo / down
    # scaled (d and dmin of its Q4_K blocks doubled: every product and sum doubles exactly); scaling the
    # sublayer's INPUT instead (sides swapped) is a different function.
    scale = np.where(np.arange(D2.hidden) % 3 == 0, 2.0, 1.0).astype(np.float32)
    sided = {**dw, "layers": []}
    doubled = {**dw, "layers": []}
    for L in dw["layers"]:
        base = np.zeros((2, 2, D2.hidden), np.float32)
        base[0, 0, :] = 1.0
        base[1, 0, :] = scale
        zero = (L["conv_attn_proj"][0], np.zeros_like(L["conv_attn_proj"][1]))
        sided["layers"].append({**L, "conv_attn_proj": zero, "conv_ffn_proj": zero, "conv_attn_base": base, "conv_ffn_base": base})
        mod = dict(L)
        for name in ("wo", "down"):
            qtype, blocks = L[name]
            assert qtype == dfl.synth.Q4_K
            b2 = blocks.copy().reshape(D2.hidden, -1, 144)
            dd = b2[:, :, :4].copy().view(np.float16)          # d, dmin of every block of every row
            dd[scale == 2.0] *= np.float16(2.0)
            assert np.all(np.isfinite(dd))
            b2[:, :, :4] = dd.view(np.uint8)
            mod[name] = (qtype, b2.reshape(blocks.shape))
        doubled["layers"].append(mod)
    ext_s, _k6 = oracle.build_dflash2_ext(D2.as_dict(), sided)
    got_s, _ = oracle.dflash_draft_ex(omodel, ohead, ext_s, ids, ctx, list(range(ctx_len)), ctx_len)
    ohead_d, _k7 = oracle.build_draft_head(D2.as_dict(), doubled)
    want_s = oracle.dflash_draft(omodel, ohead_d, ids, ctx, list(range(ctx_len)), ctx_len)
    assert np.array_equal(got_s.view(np.uint32), want_s.view(np.uint32))
    assert not np.array_equal(got_s, plain)

    ext2, _k4 = oracle.build_dflash2_ext(D2.as_dict(), dw)
    other, _ = oracle.dflash_draft_ex(omodel, ohead, ext2, ids, ctx, list(range(ctx_len)), ctx_len)
    assert not np.array_equal(other, plain)
    # a one-row-shift kernel on side 0 only (y[t] = x[t-1]) changes every row but row 0 of what q/k/v read;
    # with all taps zero the sublayers see zeros: the logits are then those of the embeddings alone
    dead = {**dw, "layers": []}
    for L in dw["layers"]:
        zero = (L["conv_attn_proj"][0], np.zeros_like(L["conv_attn_proj"][1]))
        dead["layers"].append({**L, "conv_attn_proj": zero, "conv_ffn_proj": zero,
                               "conv_attn_base": np.zeros((2, 2, D2.hidden), np.float32),
                               "conv_ffn_base": np.zeros((2, 2, D2.hidden), np.float32)})
    ext3, _k5 = oracle.build_dflash2_ext(D2.as_dict(), dead)
    bare, _ = oracle.dflash_draft_ex(omodel, ohead, ext3, ids, ctx, list(range(ctx_len)), ctx_len)
    # side-1 kernels of zero remove both residual branches: x stays the embedding, so rows 1.. (all the mask
    # token) are identical to each other
    assert np.array_equal(bare[1], bare[2]) and np.array_equal(bare[2], bare[7])
