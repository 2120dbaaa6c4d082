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


# ------------------------------------------------------------------ composed DFlash-2 forward, dynamic coefficients
#
# The reference holds no value test of the composed DFlash-2 forward that runs without model files
# (crates/qwen-llm/tests/dflash_correctness.rs:178-357 needs a checkpoint), so the wiring of the dynamic
# coefficients (metal_dflash.rs:16210-16262, 16795-16885, 17003-17022) is pinned by what the formula fixes,
# always with NON-ZERO coefficient projections:
#   * an independent vectorised float64 model of the whole layer,
#   * exact identities that hold only if (i) the coefficients come from the normed, pre-convolution input,
#     (ii) the attention pair and the FFN pair each use their own projection, (iii) both sides of a pair read
#     the two halves of ONE coefficient vector.


def np_conv(x, dyn, base, ks, gs, side):
    """y[t][c] = sum_tap (base[side][tap][c] + dyn[t][side][tap][c // gs]) * x[t - tap][c] in float64
    (kernels/dflash2.metal:40-69); rows before the block are zeros."""
    n, h = x.shape
    d = np.repeat(dyn.reshape(n, 2, ks, h // gs)[:, side], gs, axis=2)  # [n][tap][h]
    y = np.zeros((n, h))
    for tap in range(ks):
        shifted = np.zeros((n, h))
        shifted[tap:] = x[:n - tap]
        y += (base[side, tap][None, :] + d[:, tap]) * shifted
    return y


def np_draft2(c, m, emb, head_w, ids, ctx, pos_ctx, start, theta=1e6):
    """Float64 model of draft_block_inner with layer.conv (metal_dflash.rs:16195-17035): per sublayer the
    coefficients are one projection of the NORMED input; side 0 convolves that input before q/k/v (gate/up)
    read it, side 1 convolves the sublayer's output before the residual add.  The context columns' K/V come from
    ctx_h and see no convolution."""
    from test_oracle_forward import rms, rope, silu, softmax

    n, nq, nkv, hd, h = c["block_size"], c["n_q"], c["n_kv"], c["head_dim"], c["hidden"]
    ks, gs = c["conv_kernel_size"], c["conv_group_size"]
    group = nq // nkv
    ctx_len = len(pos_ctx)
    ctx_h = rms(np.asarray(ctx, np.float64) @ m["fc"].T, m["hidden_norm"]) if ctx_len else np.zeros((0, h))
    x = np.stack([emb[t] for t in ids])
    kpos = list(pos_ctx) + [start + i for i in range(n)]
    for L in m["layers"]:
        nn = rms(x, L["attn_norm"])
        dyn = nn @ L["conv_attn_proj"].T
        src = np_conv(nn, dyn, L["conv_attn_base"], ks, gs, 0)
        q = rms((src @ L["wq"].T).reshape(n, nq, hd), L["q_norm"])
        q = np.stack([rope(q[i], start + i, theta) for i in range(n)])
        kin = np.concatenate([ctx_h, src])
        k = rms((kin @ L["wk"].T).reshape(-1, nkv, hd), L["k_norm"])
        k = np.stack([rope(k[j], kpos[j], theta) for j in range(len(kpos))])
        v = (kin @ L["wv"].T).reshape(-1, nkv, hd)
        ao = np.zeros((n, nq, hd))
        for i in range(n):
            qp = start + i
            ok = np.array([(not c["causal"] or kp <= qp) for kp in kpos])
            for qh in range(nq):
                s = k[ok, qh // group] @ q[i, qh] / np.sqrt(hd)
                ao[i, qh] = softmax(s) @ v[ok, qh // group]
        x = x + np_conv(ao.reshape(n, -1) @ L["wo"].T, dyn, L["conv_attn_base"], ks, gs, 1)
        p = rms(x, L["post_norm"])
        dyn = p @ L["conv_ffn_proj"].T
        src = np_conv(p, dyn, L["conv_ffn_base"], ks, gs, 0)
        out = (silu(src @ L["gate"].T) * (src @ L["up"].T)) @ L["down"].T
        x = x + np_conv(out, dyn, L["conv_ffn_base"], ks, gs, 1)
    xn = rms(x, m["output_norm"])
    return xn @ head_w.T, xn @ m["selector_hidden"].T


def d2_cfg(**kw):
    from test_oracle_forward import draft_cfg

    return draft_cfg(conv_kernel_size=2, conv_group_size=8, selector_rank=12, selector_top_k=16, **kw)


def random_draft2(c, seed):
    """random_draft plus f32 DFlash-2 tensors with coefficients of order one."""
    from test_oracle_forward import random_draft

    m = random_draft(c, seed)
    rng = np.random.default_rng(seed + 1000)
    h, dd = c["hidden"], 2 * c["conv_kernel_size"] * (c["hidden"] // c["conv_group_size"])
    for L in m["layers"]:
        L["conv_attn_proj"] = (rng.standard_normal((dd, h)) * h ** -0.5).astype(np.float32)
        L["conv_ffn_proj"] = (rng.standard_normal((dd, h)) * h ** -0.5).astype(np.float32)
        L["conv_attn_base"] = rng.standard_normal((2, c["conv_kernel_size"], h)).astype(np.float32)
        L["conv_ffn_base"] = rng.standard_normal((2, c["conv_kernel_size"], h)).astype(np.float32)
    m["selector_hidden"] = (rng.standard_normal((c["selector_rank"], h)) * h ** -0.5).astype(np.float32)
    return m


BASES = ("conv_attn_base", "conv_ffn_base")


def d2_to_oracle(m):
    from test_oracle_forward import f32t

    w = {"fc": f32t(m["fc"]), "hidden_norm": m["hidden_norm"], "output_norm": m["output_norm"],
         "selector_hidden": f32t(m["selector_hidden"]), "layers": []}
    for L in m["layers"]:
        w["layers"].append({k: (v if isinstance(v, int) or v.ndim == 1 or k in BASES else f32t(v)) for k, v in L.items()})
    return w


def d2_f64(m):
    out = {k: np.asarray(v, np.float64) for k, v in m.items() if k != "layers"}
    out["layers"] = [{k: (v if isinstance(v, int) else np.asarray(v, np.float64)) for k, v in L.items()} for L in m["layers"]]
    return out


def run_d2(oracle, c, m, target, ids, ctx, pos_ctx, start):
    w = d2_to_oracle(m)
    head, k1 = oracle.build_draft_head(c, w)
    ext, k2 = oracle.build_dflash2_ext(c, w)
    return oracle.dflash_draft_ex(target, head, ext, ids, ctx, pos_ctx, start)


def bits(a):
    return np.ascontiguousarray(a, np.float32).view(np.uint32)


@pytest.mark.parametrize("causal,pos_ctx,start", [(0, [0, 1, 2, 3, 4], 5), (1, [2, 3, 7, 9], 11), (0, [], 3)])
def test_dflash2_drafter_matches_f64_model(oracle, causal, pos_ctx, start):
    """Random non-zero coefficient projections and base kernels against the float64 model.  A wiring mistake moves
    the logits by O(1) of their rms (checked below for the two nearest misreadings); f32-vs-f64 summation by 1e-6."""
    from test_oracle_forward import close, tiny_target

    c = d2_cfg(causal=causal)
    m = random_draft2(c, 51)
    target, keep, emb, head_w = tiny_target(oracle, 50, c["hidden"], 52)
    ctx = np.random.default_rng(53).standard_normal((len(pos_ctx), c["n_taps"] * c["hidden"])).astype(np.float32)
    ids = [7, 49, 49, 49, 49, 12]
    got, sel = run_d2(oracle, c, m, target, ids, ctx, pos_ctx, start)
    want, want_sel = np_draft2(c, d2_f64(m), emb, head_w, ids, ctx, pos_ctx, start)
    close(got, want, 5e-4, "logits")
    close(sel, want_sel, 5e-4, "selector gate")
    # the model itself tells the two nearest misreadings apart by far more than the tolerance
    shared = d2_f64(m)
    for L in shared["layers"]:
        L["conv_ffn_proj"] = L["conv_attn_proj"]
    other, _ = np_draft2(c, shared, emb, head_w, ids, ctx, pos_ctx, start)
    assert np.abs(other - want).max() / np.sqrt((want * want).mean()) > 1e-2


def constant_channel_target(oracle, vocab, hidden, seed):
    """Embedding rows of +-1 entries with channel 0 == +1: every row has mean square exactly 1, so channel 0 of the
    RMS-normed embedding is the same number for every token."""
    from test_oracle_forward import dense_cfg, f32t

    rng = np.random.default_rng(seed)
    emb = np.where(rng.random((vocab, hidden)) < 0.5, -1.0, 1.0).astype(np.float32)
    emb[:, 0] = 1.0
    head = (rng.standard_normal((vocab, hidden)) * hidden ** -0.5).astype(np.float32)
    model, keep = oracle.build_model(dense_cfg(n_layers=0, hidden=hidden, vocab=vocab),
                                     {"token_embd": f32t(emb), "output": f32t(head),
                                      "output_norm": np.ones(hidden, np.float32), "layers": []})
    return model, keep


def column0_projection(rng, dd, h):
    """A coefficient projection that reads channel 0 only, with power-of-two entries (exact products)."""
    p = np.zeros((dd, h), np.float32)
    p[:, 0] = np.ldexp(1.0, rng.integers(-3, 2, dd)) * np.where(rng.random(dd) < 0.5, -1.0, 1.0)
    return p


def test_attention_pair_reads_one_coefficient_vector_of_its_own_projection(oracle):
    """A projection that makes the coefficients a constant c must equal the static forward with base + c on BOTH sides.
    One layer; the embeddings' normed channel 0 is the same for every row (s = w0 / sqrt(1 + eps)), conv_attn_proj reads
    channel 0 only, so dyn[t] = c = p * s for every t.  The FFN pair keeps a random non-zero projection of its own in
    both runs.  Equality bit for bit fails if side 1 of the attention pair read another vector, if the FFN pair reused
    the attention pair's coefficients (its dyn would be c in one run and 0 in the other), or if dyn came from the
    un-normed x (channel 0 of x is 1, not s = 0.5 / sqrt(1 + eps))."""
    c = d2_cfg(n_layers=1)
    m = random_draft2(c, 61)
    h, dd = c["hidden"], m["layers"][0]["conv_attn_proj"].shape[0]
    target, keep = constant_channel_target(oracle, 50, h, 62)
    L = m["layers"][0]
    L["attn_norm"][0] = 0.5
    L["conv_attn_proj"] = column0_projection(np.random.default_rng(63), dd, h)
    s = np.float32(1.0) / np.sqrt(np.float32(1.0) + np.float32(c["eps"])) * np.float32(0.5)  # rms-normed channel 0
    const = (L["conv_attn_proj"][:, 0] * s).astype(np.float32)                               # [side][tap][group]
    ids, ctx, pos_ctx, start = [7, 49, 49, 49, 49, 12], np.zeros((0, c["n_taps"] * h), np.float32), [], 3
    dyn_run, _ = run_d2(oracle, c, m, target, ids, ctx, pos_ctx, start)

    static = {**m, "layers": [dict(L)]}
    static["layers"][0]["conv_attn_proj"] = np.zeros((dd, h), np.float32)
    static["layers"][0]["conv_attn_base"] = (L["conv_attn_base"] +
                                             np.repeat(const.reshape(2, 2, -1), c["conv_group_size"], axis=2)).astype(np.float32)
    static_run, _ = run_d2(oracle, c, static, target, ids, ctx, pos_ctx, start)
    assert np.array_equal(bits(dyn_run), bits(static_run))
    # the constant is really on the path: without it the logits differ
    plain = {**m, "layers": [dict(static["layers"][0], conv_attn_base=L["conv_attn_base"])]}
    assert not np.array_equal(bits(run_d2(oracle, c, plain, target, ids, ctx, pos_ctx, start)[0]), bits(dyn_run))


def test_ffn_pair_reads_one_coefficient_vector_of_its_own_projection(oracle):
    """The same identity for the FFN pair.  attn_output is zero, so the residual that post_norm reads is still the
    embedding and its normed channel 0 is constant; conv_ffn_proj reads channel 0 only.  The attention pair keeps a
    random non-zero projection in both runs: were its coefficients reused for the FFN pair, neither run would see
    the constant and the runs would differ by the base kernels."""
    c = d2_cfg(n_layers=1)
    m = random_draft2(c, 71)
    h, dd = c["hidden"], m["layers"][0]["conv_ffn_proj"].shape[0]
    target, keep = constant_channel_target(oracle, 50, h, 72)
    L = m["layers"][0]
    L["wo"] = np.zeros_like(L["wo"])
    L["post_norm"][0] = 0.25
    L["conv_ffn_proj"] = column0_projection(np.random.default_rng(73), dd, h)
    s = np.float32(1.0) / np.sqrt(np.float32(1.0) + np.float32(c["eps"])) * np.float32(0.25)
    const = (L["conv_ffn_proj"][:, 0] * s).astype(np.float32)
    ids, ctx, pos_ctx, start = [7, 49, 49, 49, 49, 12], np.zeros((0, c["n_taps"] * h), np.float32), [], 3
    dyn_run, _ = run_d2(oracle, c, m, target, ids, ctx, pos_ctx, start)
    static = {**m, "layers": [dict(L)]}
    static["layers"][0]["conv_ffn_proj"] = np.zeros((dd, h), np.float32)
    static["layers"][0]["conv_ffn_base"] = (L["conv_ffn_base"] +
                                            np.repeat(const.reshape(2, 2, -1), c["conv_group_size"], axis=2)).astype(np.float32)
    static_run, _ = run_d2(oracle, c, static, target, ids, ctx, pos_ctx, start)
    assert np.array_equal(bits(dyn_run), bits(static_run))
    plain = {**m, "layers": [dict(static["layers"][0], conv_ffn_base=L["conv_ffn_base"])]}
    assert not np.array_equal(bits(run_d2(oracle, c, plain, target, ids, ctx, pos_ctx, start)[0]), bits(dyn_run))


def test_coefficients_come_from_the_normed_input(oracle):
    """Doubling a norm's weights while halving the coefficient projection (exact in f32) leaves every coefficient
    bit-identical while the convolved input doubles exactly.
    FFN pair: with gate and up halved as well, g and u keep their bits, so no logit may change in a single bit.
    Attention pair (wk / wv also serve the context columns, which this norm does not feed, so they cannot be halved):
    the same function is reached with the ORIGINAL norm and a side-0 coefficient of 2 * (base + dyn) - side-0 base
    kernel and the side-0 rows of the projection doubled - and the two runs must agree bit for bit.
    Coefficients taken from the un-normed residual would halve in the first run of each pair and fail both."""
    from test_oracle_forward import tiny_target

    c = d2_cfg()
    m = random_draft2(c, 81)
    target, keep, emb, head_w = tiny_target(oracle, 50, c["hidden"], 82)
    pos_ctx, start = [0, 1, 2, 3], 4
    ctx = np.random.default_rng(83).standard_normal((len(pos_ctx), c["n_taps"] * c["hidden"])).astype(np.float32)
    ids = [7, 49, 49, 49, 49, 12]
    two, half = np.float32(2.0), np.float32(0.5)
    ref, ref_sel = run_d2(oracle, c, m, target, ids, ctx, pos_ctx, start)

    ffn = {**m, "layers": [dict(L, post_norm=L["post_norm"] * two, conv_ffn_proj=L["conv_ffn_proj"] * half,
                                gate=L["gate"] * half, up=L["up"] * half) for L in m["layers"]]}
    got, got_sel = run_d2(oracle, c, ffn, target, ids, ctx, pos_ctx, start)
    assert np.array_equal(bits(got), bits(ref)) and np.array_equal(bits(got_sel), bits(ref_sel))

    scaled = {**m, "layers": [dict(L, attn_norm=L["attn_norm"] * two, conv_attn_proj=L["conv_attn_proj"] * half)
                              for L in m["layers"]]}
    twin = {**m, "layers": []}
    for L in m["layers"]:
        p, b = L["conv_attn_proj"].copy(), L["conv_attn_base"].copy()
        p[:p.shape[0] // 2] *= two  # rows are [side][tap][group]: the first half feeds side 0
        b[0] *= two
        twin["layers"].append(dict(L, conv_attn_proj=p, conv_attn_base=b))
    got, _ = run_d2(oracle, c, scaled, target, ids, ctx, pos_ctx, start)
    want, _ = run_d2(oracle, c, twin, target, ids, ctx, pos_ctx, start)
    assert np.array_equal(bits(got), bits(want))
    assert not np.array_equal(bits(got), bits(ref))  # what q/k/v read did double
