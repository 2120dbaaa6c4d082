"""GPU parity: packed 16-row verify, KV rollback and the block drafter against the CPU oracle
(token-by-token attn_step / ffn of forward.rs:96-163, 834-932 and Forward::dflash_draft,
forward.rs:380-662) on the reference's own synthetic shape (metal_dflash.rs tests: 4 layers,
hidden 1024, 16 q / 8 kv heads of 128, FFN 3072, vocabulary 32000, Q4_K weights).

Tolerance: each GEMM and each attention call is held to 1e-2 by its own test; here the error of
4 layers x 8 such calls compounds, so the stack is held to a relative l2 error of 5e-3 and a
worst element (over ~10^6 values, relative to max(|ref|, rms)) of 3e-2; argmax identical wherever
the oracle's own top-2 gap exceeds the logit error bound."""
import numpy as np
import pytest

import qwen_llm_amd as dfl

pytestmark = pytest.mark.gpu

C1 = dfl.ModelConfig(n_layers=4, hidden=1024, n_q=16, n_kv=8, head_dim=128, ffn=3072, vocab=32000)
TAPS = [0, 1, 2, 3, 3]
D1 = dfl.DraftConfig(n_layers=2, hidden=1024, n_q=16, n_kv=8, head_dim=128, ffn=3072, block_size=16, n_taps=5)
PREFIX = 96


@pytest.fixture(scope="module")
def ctx():
    c = dfl.Context(0, workspace_bytes=256 << 20)
    yield c
    c.close()


@pytest.fixture(scope="module")
def target(ctx, oracle):
    w = dfl.synth_target_weights(C1, seed=11)
    return dfl.TargetModel(ctx, C1, w), oracle.build_model(C1.as_dict(), w)


def close(got, want, label, tol=3e-2, l2_tol=5e-3):
    got, want = np.asarray(got, np.float32), np.asarray(want, np.float32)
    assert got.shape == want.shape, f"{label}: shape {got.shape} vs {want.shape}"
    assert np.all(np.isfinite(got)), f"{label}: non-finite"
    rms = np.sqrt(np.mean(want.astype(np.float64) ** 2))
    err = np.max(np.abs(got - want) / np.maximum(np.abs(want), rms))
    l2 = np.linalg.norm(got.astype(np.float64) - want) / np.linalg.norm(want.astype(np.float64))
    print(f"{label}: max err {err:.3e} l2 {l2:.3e}")
    assert err <= tol, f"{label}: max err {err:.3e} (rms {rms:.3e})"
    assert l2 <= l2_tol, f"{label}: rel l2 {l2:.3e}"
    return err


def argmax_agrees(argmax, logits_ref, label):
    top = np.sort(logits_ref, axis=1)
    gap = top[:, -1] - top[:, -2]
    rms = np.sqrt(np.mean(logits_ref.astype(np.float64) ** 2))
    decided = gap > 2e-2 * rms
    assert decided.sum() >= len(gap) // 2, f"{label}: synthetic logits too flat to test the argmax"
    want = logits_ref.argmax(axis=1)
    assert np.array_equal(np.asarray(argmax)[decided], want[decided]), f"{label}: argmax differs on a decided row"


def prefill(sess, ostate, omodel, oracle, tokens):
    """Fill both caches with the prompt in blocks of 16 through the same verify path."""
    hid_g, hid_o = [], []
    for s in range(0, len(tokens), 16):
        blk = tokens[s:s + 16]
        out = sess.encode_packed_verify_layer_major(blk, s)
        hid_g.append(out.hidden_capture.cpu().numpy())
        hid_o.append(oracle.target_verify(omodel, ostate, blk, s, TAPS)[1])
    return np.concatenate(hid_g), np.concatenate(hid_o)


def test_verify_block_matches_oracle_and_restore(ctx, oracle, target):
    model, (omodel, _keep) = target
    rng = np.random.default_rng(5)
    cap = PREFIX + 64
    sess = dfl.Session(ctx, model, cap, TAPS)
    ostate = oracle.TargetState(C1.as_dict(), cap)
    prompt = rng.integers(0, C1.vocab, PREFIX).tolist()
    hg, ho = prefill(sess, ostate, omodel, oracle, prompt)
    close(hg, ho, "prefill hidden")
    assert sess.kv_n_pos == PREFIX

    pos = PREFIX
    for n, n_keep in ((16, 7), (16, 0), (1, 1), (5, 5), (16, 16), (3, 1)):
        blk = rng.integers(0, C1.vocab, n).tolist()
        out = sess.encode_packed_verify_layer_major(blk, pos, want_logits=True)
        lo, hid_o = oracle.target_verify(omodel, ostate, blk, pos, TAPS)
        close(out.logits.cpu().numpy(), lo, f"logits n={n} pos={pos}")
        close(out.hidden_capture.cpu().numpy(), hid_o, f"hidden n={n} pos={pos}")
        lg = out.logits.cpu().numpy()
        assert np.array_equal(out.argmax.cpu().numpy(), lg.argmax(axis=1)), "argmax is not the argmax of the logits"
        assert out.argmax_host == out.argmax.cpu().tolist()
        top = np.sort(lg, axis=1)
        np.testing.assert_array_equal(out.gap.cpu().numpy(), top[:, -1] - top[:, -2])
        if n >= 5:
            argmax_agrees(out.argmax.cpu().numpy(), lo, f"n={n}")
        assert sess.kv_n_pos == pos + n
        sess.encode_restore_after_partial_accept(pos, n, n_keep)
        assert sess.kv_n_pos == pos + n_keep
        pos += n_keep
    sess.close()


@pytest.mark.parametrize("taps", [TAPS, [0, 2]], ids=["last-layer-tapped", "last-layer-untapped"])
def test_a_block_without_head_outputs_leaves_the_same_state(ctx, target, taps):
    """A verify block whose caller asks for none of the head's outputs (a prefill block) does not run the head (nor,
    when the last layer's residual is not tapped, anything of that layer behind its K/V rows); its K/V rows and
    tapped hidden rows are those of the same block run in full: the next block's logits are equal bit for bit, for a
    16-row and a ragged block, and the guards still hold."""
    model, _ = target
    rng = np.random.default_rng(77)
    blocks = [rng.integers(0, C1.vocab, n).tolist() for n in (16, 5, 16)]
    full, lean = dfl.Session(ctx, model, 64, taps), dfl.Session(ctx, model, 64, taps)
    pos = 0
    for blk in blocks[:2]:
        a = full.encode_packed_verify_layer_major(blk, pos)
        b = lean.encode_packed_verify_layer_major(blk, pos, want_head=False)
        assert b.argmax is None and b.gap is None and b.argmax_host is None and b.logits is None
        assert np.array_equal(a.hidden_capture.cpu().numpy(), b.hidden_capture.cpu().numpy())
        pos += len(blk)
    assert lean.kv_n_pos == full.kv_n_pos == pos
    a = full.encode_packed_verify_layer_major(blocks[2], pos, want_logits=True)
    b = lean.encode_packed_verify_layer_major(blocks[2], pos, want_logits=True)
    assert np.array_equal(a.logits.cpu().numpy(), b.logits.cpu().numpy())
    assert a.argmax_host == b.argmax_host
    with pytest.raises(dfl.DFlashError) as e:
        lean.encode_packed_verify_layer_major([1, 2], 3, want_head=False)
    assert e.value.status == 10
    full.close()
    lean.close()


def test_pipelined_prefill_equals_block_by_block(ctx, target):
    """dflash_prefill_blocks (several blocks in flight on the lane streams, ordered by per-layer events) leaves the K/V rows and
    the tapped hidden rows of the same blocks run one by one through dflash_verify_block: the captured rows and the
    next block's logits are equal bit for bit, over a ragged token count, twice in a row on one session (the second
    lane's scratch and events are reused), and its guards hold."""
    model, _ = target
    rng = np.random.default_rng(78)
    first = rng.integers(0, C1.vocab, 16 * 5 + 7).tolist()   # five full blocks and a ragged one
    second = rng.integers(0, C1.vocab, 16 * 3).tolist()
    probe = rng.integers(0, C1.vocab, 9).tolist()
    ref, pipe = dfl.Session(ctx, model, 256, TAPS), dfl.Session(ctx, model, 256, TAPS)
    pos = 0
    for chunk in (first, second):
        got = pipe.prefill_blocks(chunk, pos)
        want = []
        for s0 in range(0, len(chunk), 16):
            out = ref.encode_packed_verify_layer_major(chunk[s0:s0 + 16], pos + s0, want_head=False)
            want.append(out.hidden_capture.cpu().numpy())
        assert np.array_equal(got.cpu().numpy(), np.concatenate(want, axis=0))
        pos += len(chunk)
        assert pipe.kv_n_pos == ref.kv_n_pos == pos
    a = ref.encode_packed_verify_layer_major(probe, pos, want_logits=True)
    b = pipe.encode_packed_verify_layer_major(probe, pos, want_logits=True)
    assert np.array_equal(a.logits.cpu().numpy(), b.logits.cpu().numpy())
    assert a.argmax_host == b.argmax_host
    with pytest.raises(dfl.DFlashError) as e:
        pipe.prefill_blocks([1, 2, 3], 0)
    assert e.value.status == 10
    with pytest.raises(dfl.DFlashError) as e:
        pipe.prefill_blocks([1, C1.vocab], pipe.kv_n_pos)
    assert e.value.status == 8
    ref.close()
    pipe.close()


def test_wide_hidden_verify_matches_oracle(ctx, oracle):
    """A 5120-wide dense layer pair (the width of the 27B-shaped benchmark matrices): rows wider than 4096 take the
    norm kernel's in-register path with eight vectors per thread, and the norms hand their rows to the one-launch
    projections in fragment order at that width too."""
    cfg = dfl.ModelConfig(n_layers=2, hidden=5120, n_q=8, n_kv=2, head_dim=128, ffn=2048, vocab=4096)
    w = dfl.synth_target_weights_blocks(cfg, 19)
    model = dfl.TargetModel(ctx, cfg, w)
    omodel, _keep = oracle.build_model(cfg.as_dict(), w)
    sess = dfl.Session(ctx, model, 64, [0, 1])
    ostate = oracle.TargetState(cfg.as_dict(), 64)
    rng = np.random.default_rng(4)
    pos = 0
    for n in (16, 5):
        blk = rng.integers(0, cfg.vocab, n).tolist()
        out = sess.encode_packed_verify_layer_major(blk, pos, want_logits=True)
        lo, hid = oracle.target_verify(omodel, ostate, blk, pos, [0, 1])
        close(out.hidden_capture.cpu().numpy(), hid, f"wide hidden n={n}")
        close(out.logits.cpu().numpy(), lo, f"wide logits n={n}")
        pos += n
    sess.close()


def test_verify_guard_walls(ctx, target):
    model, _ = target
    sess = dfl.Session(ctx, model, 64, TAPS)
    with pytest.raises(dfl.DFlashError) as e:
        sess.encode_packed_verify_layer_major([1, 2, 3], 5)
    assert e.value.status == 10 and "kv_n_pos" in str(e.value)
    with pytest.raises(dfl.DFlashError) as e:
        sess.encode_packed_verify_layer_major([1, C1.vocab], 0)
    assert e.value.status == 8
    with pytest.raises(dfl.DFlashError) as e:
        sess.encode_packed_verify_layer_major(list(range(17)), 0)
    assert e.value.status == 1
    with pytest.raises(dfl.DFlashError):
        sess.encode_packed_verify_layer_major([], 0)
    assert sess.kv_n_pos == 0
    sess.encode_packed_verify_layer_major(list(range(16)), 0)
    with pytest.raises(dfl.DFlashError) as e:
        sess.encode_restore_after_partial_accept(0, 16, 17)
    assert e.value.status == 1
    with pytest.raises(dfl.DFlashError) as e:
        sess.encode_restore_after_partial_accept(3, 16, 4)
    assert e.value.status == 10
    for s in range(16, 64, 16):
        sess.encode_packed_verify_layer_major(list(range(16)), s)
    with pytest.raises(dfl.DFlashError) as e:
        sess.encode_packed_verify_layer_major([1], 64)
    assert e.value.status == 10 and "capacity" in str(e.value)
    sess.close()


@pytest.mark.parametrize("causal,swa", [(0, 0), (1, 0), (0, 24), (1, 8)])
def test_draft_block_matches_oracle(ctx, oracle, target, causal, swa):
    model, (omodel, _keep) = target
    dcfg = dfl.DraftConfig(**{**D1.as_dict(), "causal": causal, "swa_window": swa})
    dw = dfl.synth_draft_weights(dcfg, seed=3, swa_layers=(1,) if swa else ())
    head = dfl.DraftHead(ctx, dcfg, dw)
    ohead, _k2 = oracle.build_draft_head(dcfg.as_dict(), dw)
    rng = np.random.default_rng(17 + causal + swa)
    cap = 128
    sess = dfl.Session(ctx, model, cap, TAPS)
    ostate = oracle.TargetState(C1.as_dict(), cap)
    dsess = dfl.DraftSession(ctx, head, model, cap)
    mask_token = C1.vocab - 1

    # incremental context: a 40-token prompt, then two accepted stretches of 5 and 16 columns
    all_hidden_o = []
    pos = 0
    for n_new in (40, 5, 16):
        toks = rng.integers(0, C1.vocab, n_new).tolist()
        for s in range(0, n_new, 16):
            blk = toks[s:s + 16]
            out = sess.encode_packed_verify_layer_major(blk, pos)
            dsess.append_target_ctx_columns(out.hidden_capture, list(range(pos, pos + len(blk))))
            all_hidden_o.append(oracle.target_verify(omodel, ostate, blk, pos, TAPS)[1])
            pos += len(blk)
        assert dsess.ctx_len == pos
        carry = int(rng.integers(0, C1.vocab))
        argmax, logits, host = dsess.draft_block(carry, mask_token, pos, want_logits=True)
        ctx_o = np.concatenate(all_hidden_o).reshape(pos, -1)
        want = oracle.dflash_draft(omodel, ohead, [carry] + [mask_token] * 15, ctx_o, list(range(pos)), pos)
        close(logits.cpu().numpy(), want, f"draft logits ctx={pos} causal={causal} swa={swa}")
        lg = logits.cpu().numpy()
        assert host == lg.argmax(axis=1).tolist() == argmax.cpu().tolist()
        argmax_agrees(host, want, f"draft ctx={pos}")
    with pytest.raises(dfl.DFlashError) as e:
        dsess.draft_block(C1.vocab, mask_token, pos)
    assert e.value.status == 8
    dsess.close()
    sess.close()


@pytest.mark.parametrize("wtype", [dfl.TYPE_Q4_K, dfl.TYPE_Q6_K])
def test_separate_and_adjacent_weight_layouts_agree(ctx, oracle, wtype):
    """A layer's wq/wk/wv and gate/up uploaded back to back run as one GEMM each (the default of the
    mirror); uploaded separately they run as three and two (Q6_K: the three projections in one launch of
    the set kernel).  Both layouts must match the oracle, and each other to GEMM tolerance (the split-K
    boundaries differ, so not bit for bit)."""
    w = dfl.synth_target_weights(C1, seed=11, wtype=wtype)
    omodel, _keep = oracle.build_model(C1.as_dict(), w)
    model_adj = dfl.TargetModel(ctx, C1, w)
    model_sep = dfl.TargetModel(ctx, C1, w, adjacent=False)
    L0a, L0s = model_adj.c.layers[0], model_sep.c.layers[0]
    rb = 1024 // 256 * (144 if wtype == dfl.TYPE_Q4_K else 210)
    assert L0a.wk.data == L0a.wq.data + 16 * 128 * rb and L0a.wv.data == L0a.wk.data + 8 * 128 * rb
    assert L0a.up.data == L0a.gate.data + 3072 * rb
    assert L0s.wk.data != L0s.wq.data + 16 * 128 * rb or L0s.wv.data != L0s.wk.data + 8 * 128 * rb
    dw = dfl.synth_draft_weights(D1, seed=3, wtype=wtype)
    ohead, _k2 = oracle.build_draft_head(D1.as_dict(), dw)
    rng = np.random.default_rng(23)
    cap = 64
    toks = rng.integers(0, C1.vocab, 32).tolist()
    carry = int(rng.integers(0, C1.vocab))
    outs = {}
    for name, model, adjacent in (("adjacent", model_adj, True), ("separate", model_sep, False)):
        head = dfl.DraftHead(ctx, D1, dw, adjacent=adjacent)
        sess = dfl.Session(ctx, model, cap, TAPS)
        dsess = dfl.DraftSession(ctx, head, model, cap)
        logits, hidden = [], []
        for s in range(0, 32, 16):
            out = sess.encode_packed_verify_layer_major(toks[s:s + 16], s, want_logits=True)
            dsess.append_target_ctx_columns(out.hidden_capture, list(range(s, s + 16)))
            logits.append(out.logits.cpu().numpy())
            hidden.append(out.hidden_capture.cpu().numpy())
        _, dl, _ = dsess.draft_block(carry, C1.vocab - 1, 32, want_logits=True)
        outs[name] = (np.concatenate(logits), np.concatenate(hidden), dl.cpu().numpy())
        dsess.close()
        sess.close()
    ostate = oracle.TargetState(C1.as_dict(), cap)
    lo, ho = [], []
    for s in range(0, 32, 16):
        l, h = oracle.target_verify(omodel, ostate, toks[s:s + 16], s, TAPS)
        lo.append(l)
        ho.append(h)
    lo, ho = np.concatenate(lo), np.concatenate(ho)
    want_d = oracle.dflash_draft(omodel, ohead, [carry] + [C1.vocab - 1] * 15, ho.reshape(32, -1), list(range(32)), 32)
    for name, (lg, hid, dl) in outs.items():
        close(lg, lo, f"{name}: verify logits")
        close(hid, ho, f"{name}: hidden")
        close(dl, want_d, f"{name}: draft logits")
    close(outs["adjacent"][0], outs["separate"][0], "adjacent vs separate verify logits")
    close(outs["adjacent"][2], outs["separate"][2], "adjacent vs separate draft logits")


@pytest.mark.parametrize("codebook_type", [dfl.TYPE_Q4_K, dfl.TYPE_Q8_0])
def test_dflash2_draft_block_matches_oracle(ctx, oracle, target, codebook_type):
    """A DFlash-2 head (two-tap dynamic convolutions around both sublayers, block of 8, selector of rank
    256 over the top-16 candidates; metal_dflash.rs:16210-16262, 16795-16885, 17003-17022, 17098-17251)
    against the oracle's restatement: logits to the stack tolerance; the tokens of the device-side walk
    are checked along the DEVICE's own path (each pick conditions the next): every pick is one of that
    row's top-16 and its score, recomputed from the oracle's selector gate and codebook rows, is the best
    of the row up to the logit error."""
    model, (omodel, _keep) = target
    dcfg = dfl.DraftConfig(**{**D1.as_dict(), "block_size": 8, "conv_kernel_size": 2, "conv_group_size": 64,
                              "selector_rank": 256, "selector_top_k": 16})
    dw = dfl.synth_draft_weights(dcfg, seed=9, vocab=C1.vocab, codebook_type=codebook_type)
    head = dfl.DraftHead(ctx, dcfg, dw)
    ohead, _k2 = oracle.build_draft_head(dcfg.as_dict(), dw)
    ext, _k3 = oracle.build_dflash2_ext(dcfg.as_dict(), dw)
    pred_cb, _k4 = oracle.make_codebook(codebook_type, dw["selector_predecessor"][1], 256)
    succ_cb, _k5 = oracle.make_codebook(codebook_type, dw["selector_successor"][1], 256)
    rng = np.random.default_rng(31)
    cap = 64
    sess = dfl.Session(ctx, model, cap, TAPS)
    ostate = oracle.TargetState(C1.as_dict(), cap)
    dsess = dfl.DraftSession(ctx, head, model, cap)
    mask_token = C1.vocab - 1
    hidden_o, pos = [], 0
    for n_new in (24, 5):
        toks = rng.integers(0, C1.vocab, n_new).tolist()
        for s0 in range(0, n_new, 16):
            blk = toks[s0:s0 + 16]
            out = sess.encode_packed_verify_layer_major(blk, pos)
            dsess.append_target_ctx_columns(out.hidden_capture, list(range(pos, pos + len(blk))))
            hidden_o.append(oracle.target_verify(omodel, ostate, blk, pos, TAPS)[1])
            pos += len(blk)
        carry = int(rng.integers(0, C1.vocab))
        tokens_dev, logits, host = dsess.draft_block(carry, mask_token, pos, want_logits=True)
        ctx_o = np.concatenate(hidden_o).reshape(pos, -1)
        want, sel_h = oracle.dflash_draft_ex(omodel, ohead, ext, [carry] + [mask_token] * 7, ctx_o, list(range(pos)), pos)
        lg = logits.cpu().numpy()
        # two more f16-operand GEMMs per sublayer (the coefficient projections) whose outputs multiply the
        # activations: the stack bound is widened accordingly (DFlash-1 on this shape: l2 about 3e-3)
        close(lg, want, f"dflash2 draft logits ctx={pos}", tol=5e-2, l2_tol=8e-3)
        assert host == tokens_dev.cpu().tolist()
        ids_d, vals_d = ctx.top16(logits)
        ids_d, vals_d = ids_d.cpu().numpy(), vals_d.cpu().numpy()
        assert host[0] == ids_d[0][0]
        rms = float(np.sqrt(np.mean(want.astype(np.float64) ** 2)))
        prev = carry
        for p in range(1, 8):
            gate = oracle.codebook_row(pred_cb, prev).astype(np.float64) * sel_h[p].astype(np.float64)
            scores = np.array([vals_d[p][b] + float(gate @ oracle.codebook_row(succ_cb, int(ids_d[p][b])).astype(np.float64))
                               for b in range(16)])
            assert host[p] in ids_d[p].tolist(), f"position {p}: pick {host[p]} is not a top-16 candidate"
            mine = scores[ids_d[p].tolist().index(host[p])]
            assert mine >= scores.max() - 4e-2 * rms, f"position {p}: pick scores {mine}, best {scores.max()}"
            prev = host[p]
    dsess.close()
    sess.close()


def test_dflash2_identity_convolutions_equal_dflash1_on_the_device(ctx, target):
    """With zero coefficient projections and identity base kernels every convolution returns its input bit
    for bit, so the DFlash-2 launches must reproduce the DFlash-1 drafter's logits exactly: the convolutions
    sit where the reference puts them and touch nothing else."""
    model, _ = target
    d1 = dfl.DraftConfig(**{**D1.as_dict(), "block_size": 8})
    d2 = dfl.DraftConfig(**{**d1.as_dict(), "conv_kernel_size": 2, "conv_group_size": 64})
    dw = dfl.synth_draft_weights(d2, seed=9)
    ident = {**dw, "layers": []}
    for L in dw["layers"]:
        base = np.zeros((2, 2, d2.hidden), np.float32)
        base[:, 0, :] = 1.0
        zero = (L["conv_attn_proj"][0], np.zeros_like(L["conv_attn_proj"][1]))
        ident["layers"].append({**L, "conv_attn_proj": zero, "conv_ffn_proj": zero, "conv_attn_base": base, "conv_ffn_base": base})
    rng = np.random.default_rng(2)
    toks = rng.integers(0, C1.vocab, 16).tolist()
    got = []
    for cfg, w in ((d1, dw), (d2, ident)):
        head = dfl.DraftHead(ctx, cfg, w)
        sess = dfl.Session(ctx, model, 64, TAPS)
        dsess = dfl.DraftSession(ctx, head, model, 64)
        out = sess.encode_packed_verify_layer_major(toks, 0)
        dsess.append_target_ctx_columns(out.hidden_capture, list(range(16)))
        _, logits, _ = dsess.draft_block(11, C1.vocab - 1, 16, want_logits=True)
        got.append(logits.cpu().numpy())
        dsess.close()
        sess.close()
    assert np.array_equal(got[0].view(np.uint32), got[1].view(np.uint32))


MOE_CASES = {
    # hidden 512: 16 sub-blocks per row (half-wave rows); hidden 2048 / F_exp 768: the end-to-end shape's widths
    "small": dfl.ModelConfig(n_layers=2, hidden=512, n_q=8, n_kv=2, head_dim=64, ffn=0, vocab=4096, n_expert=16,
                             n_expert_used=4, ffn_expert=256, ffn_shared=512),
    "wide": dfl.ModelConfig(n_layers=2, hidden=2048, n_q=16, n_kv=2, head_dim=256, ffn=0, vocab=8192, n_expert=32,
                            n_expert_used=8, ffn_expert=768, ffn_shared=768),
}


@pytest.mark.parametrize("name,wtype", [("small", dfl.TYPE_Q4_K), ("wide", dfl.TYPE_Q4_K), ("small", dfl.TYPE_Q8_0)])
def test_moe_verify_matches_oracle(ctx, oracle, name, wtype):
    """Q4_K experts run as one batched streaming GEMM per projection; other types through the per-expert
    f32 kernels.  Top-k routing is discontinuous: a row whose k-th and (k+1)-th expert probabilities are
    closer than the activation error (1e-3) may pick a different expert than the f32 oracle, which
    changes that whole row.  The seeds below have no such near tie in the rows compared."""
    cfg = MOE_CASES[name]
    w = dfl.synth_target_weights(cfg, seed={"small": 23, "wide": 31}[name], wtype=wtype)
    model = dfl.TargetModel(ctx, cfg, w)
    omodel, _keep = oracle.build_model(cfg.as_dict(), w)
    taps = [0, 1]
    sess = dfl.Session(ctx, model, 64, taps)
    ostate = oracle.TargetState(cfg.as_dict(), 64)
    rng = np.random.default_rng(29)
    pos = 0
    for n in (16, 16, 1, 7):
        blk = rng.integers(0, cfg.vocab, n).tolist()
        out = sess.encode_packed_verify_layer_major(blk, pos, want_logits=True)
        lo, hid = oracle.target_verify(omodel, ostate, blk, pos, taps)
        close(out.hidden_capture.cpu().numpy(), hid, f"moe {name} hidden n={n}")
        close(out.logits.cpu().numpy(), lo, f"moe {name} logits n={n}")
        pos += n
    sess.close()


def test_draft_block_general_positions(ctx, oracle, target):
    """Context columns at arbitrary positions and a block that does not start right behind them: the
    general f32 drafter attention (the MFMA path needs positions 0, 1, 2, ... and start == ctx_len)."""
    model, (omodel, _keep) = target
    dcfg = dfl.DraftConfig(**{**D1.as_dict(), "causal": 1, "swa_window": 12})
    dw = dfl.synth_draft_weights(dcfg, seed=4, swa_layers=(0,))
    head = dfl.DraftHead(ctx, dcfg, dw)
    ohead, _k2 = oracle.build_draft_head(dcfg.as_dict(), dw)
    rng = np.random.default_rng(41)
    sess = dfl.Session(ctx, model, 64, TAPS)
    ostate = oracle.TargetState(C1.as_dict(), 64)
    dsess = dfl.DraftSession(ctx, head, model, 64)
    toks = rng.integers(0, C1.vocab, 23).tolist()
    hidden_o = []
    for s in range(0, 23, 16):
        blk = toks[s:s + 16]
        out = sess.encode_packed_verify_layer_major(blk, s)
        # every second column is given a position shifted by 3
        dsess.append_target_ctx_columns(out.hidden_capture, [p + 3 * (p & 1) for p in range(s, s + len(blk))])
        hidden_o.append(oracle.target_verify(omodel, ostate, blk, s, TAPS)[1])
    pos_ctx = [p + 3 * (p & 1) for p in range(23)]
    carry, start = 77, 29
    argmax, logits, host = dsess.draft_block(carry, C1.vocab - 1, start, want_logits=True)
    want = oracle.dflash_draft(omodel, ohead, [carry] + [C1.vocab - 1] * 15, np.concatenate(hidden_o).reshape(23, -1),
                               pos_ctx, start)
    close(logits.cpu().numpy(), want, "draft logits, general positions")
    dsess.close()
    sess.close()


def test_graph_replay_is_bit_identical_to_launch_by_launch(ctx, target):
    """The packed verify replayed from a captured graph (second and later calls of a shape) against
    the same calls made launch by launch: logits, hidden capture, argmax and gap bit for bit, at
    moving positions, with a rollback and single-row calls in between and other GPU work and
    synchronisations between the replays.  The context grows past 256 positions on the way: the attention launches
    are cut by the power-of-two range of the context length, so a graph serves one such range and the next range
    captures its own."""
    import torch

    model, _ = target
    rng = np.random.default_rng(21)
    cap = 448
    blocks = [rng.integers(0, C1.vocab, 16).tolist() for _ in range(24)]
    singles = rng.integers(0, C1.vocab, 24).tolist()

    def run(graphs):
        ctx.set_graphs(graphs)
        sess = dfl.Session(ctx, model, cap, TAPS)
        outs, pos = [], 0
        scratch = torch.zeros(1 << 20, device="cuda")
        for i, blk in enumerate(blocks):
            o = sess.encode_packed_verify_layer_major(blk, pos, want_logits=True)
            outs.append((o.logits.cpu().numpy(), o.hidden_capture.cpu().numpy(), o.argmax.cpu().numpy(), o.gap.cpu().numpy()))
            del o
            scratch += float(i)  # the program's own eager work between replays
            torch.cuda.synchronize()
            keep = 16 if i % 3 else 5  # partial accept: roll the cache back
            sess.encode_restore_after_partial_accept(pos, 16, keep)
            pos += keep
            o = sess.encode_packed_verify_layer_major([singles[i]], pos, want_logits=True)
            outs.append((o.logits.cpu().numpy(), o.hidden_capture.cpu().numpy(), o.argmax.cpu().numpy(), o.gap.cpu().numpy()))
            del o
            pos += 1
        assert pos > 288
        replays = sess.graph_replays
        return outs, replays

    try:
        eager, r0 = run(False)
        replay, r1 = run(True)
    finally:
        ctx.set_graphs(False)
    assert r0 == 0
    assert r1 >= 36, f"only {r1} of 48 calls were graph replays"
    for i, (a, b) in enumerate(zip(eager, replay)):
        for x, y, name in zip(a, b, ("logits", "hidden", "argmax", "gap")):
            assert np.array_equal(x.view(np.uint32) if x.dtype == np.float32 else x,
                                  y.view(np.uint32) if y.dtype == np.float32 else y), f"call {i}: {name} differs under graph replay"
