"""GPU parity of one speculative transition and of the generation loop (qwen/dflash.rs:700-1241).

Invariant used as the oracle: whatever the drafter proposes, greedy speculative decoding emits the
target's own greedy continuation, and sampler-coupled decoding with deterministic proposals emits
the serial sampler's stream (sampling.rs:2837-2865).  The continuation itself comes from the CPU
oracle's token-by-token forward; rows whose oracle top-2 gap is within the logit error are not
compared (none occur for the seeds below)."""
import numpy as np
import pytest

import qwen_llm_amd as dfl

pytestmark = pytest.mark.gpu

C1 = dfl.ModelConfig(n_layers=4, hidden=1024, n_q=16, n_kv=8, head_dim=128, ffn=3072, vocab=32000)
TAPS = [0, 1, 2, 3, 3]
D1 = dfl.DraftConfig(n_layers=2, hidden=1024, n_q=16, n_kv=8, head_dim=128, ffn=3072, block_size=16, n_taps=5)
PROMPT_LEN = 40
MASK = C1.vocab - 1


@pytest.fixture(scope="module")
def ctx():
    c = dfl.Context(0, workspace_bytes=256 << 20)
    yield c
    c.close()


@pytest.fixture(scope="module")
def world(ctx, oracle):
    w = dfl.synth_target_weights(C1, seed=11)
    dw = dfl.synth_draft_weights(D1, seed=3)
    model, head = dfl.TargetModel(ctx, C1, w), dfl.DraftHead(ctx, D1, dw)
    omodel, keep = oracle.build_model(C1.as_dict(), w)
    prompt = np.random.default_rng(1).integers(0, C1.vocab - 1, PROMPT_LEN).tolist()
    # the oracle's serial greedy continuation and every row's logits
    ostate = oracle.TargetState(C1.as_dict(), 256)
    lo, _ = oracle.target_verify(omodel, ostate, prompt, 0, TAPS)
    cont, rows = [int(lo[-1].argmax())], []
    for i in range(72):
        lg, _ = oracle.target_verify(omodel, ostate, [cont[-1]], PROMPT_LEN + i, TAPS)
        rows.append(lg[0])
        cont.append(int(lg[0].argmax()))
    rows = np.stack(rows)
    top = np.sort(rows, axis=1)
    decided = (top[:, -1] - top[:, -2]) > 2e-2 * rows.std()
    return dict(model=model, head=head, omodel=omodel, keep=keep, prompt=prompt, cont=cont, rows=rows, decided=decided)


def new_decoder(ctx, world, **kw):
    dec = dfl.SpeculativeDecoder(ctx, world["model"], world["head"], TAPS, 256, MASK, **kw)
    first = dec.prefill(world["prompt"])
    return dec, first


@pytest.mark.parametrize("k", [0, 1, 7, 15])
def test_forced_prefix_is_accepted_exactly(ctx, world, k):
    cont = world["cont"]
    assert world["decided"][:16].all(), "seed gives an undecided row in the first block"
    dec, first = new_decoder(ctx, world)
    assert first == cont[0]
    wrong = [(t + 1) % (C1.vocab - 1) for t in cont[1:16]]
    override = cont[1:1 + k] + wrong[k:]
    res = dec.step(first, budget=1000, draft_override=override)
    d = res.decision
    assert d.n_accepted == k and list(d.accepted_drafts[:k]) == cont[1:1 + k]
    assert d.carry_token == cont[k + 1]
    assert d.carry_kind == (dfl.CARRY_BONUS if k == 15 else dfl.CARRY_CORRECTION)
    assert d.retain_input_count == k + 1 and d.stop_reason == dfl.STOP_NONE
    assert dec.session.kv_n_pos == PROMPT_LEN + k + 1 == dec.position
    assert dec.draft_session.ctx_len == PROMPT_LEN + k + 1
    assert list(res.verify_argmax[:k + 1]) == cont[1:k + 2]
    dec.close()


def test_step_stops_on_eos_and_budget(ctx, world):
    cont = world["cont"]
    dec, first = new_decoder(ctx, world, stop_ids=[cont[3]])
    res = dec.step(first, budget=1000, draft_override=cont[1:16])
    d = res.decision
    assert d.n_accepted == 3 and d.stop_reason == dfl.STOP_EOS and d.carry_kind == dfl.CARRY_NONE
    assert d.retain_input_count == 3 and dec.session.kv_n_pos == PROMPT_LEN + 3
    dec.close()
    dec, first = new_decoder(ctx, world)
    res = dec.step(first, budget=5, draft_override=cont[1:16])
    d = res.decision
    assert d.n_accepted == 5 and d.stop_reason == dfl.STOP_TOKEN_LIMIT and d.retain_input_count == 5
    dec.close()


@pytest.mark.parametrize("margin,partial", [(0.0, True), (1e9, False), (1e9, True), (0.5, True)])
def test_generate_greedy_equals_serial_greedy(ctx, world, margin, partial):
    cont = world["cont"]
    undecided = np.flatnonzero(~world["decided"])
    n_tok = int(min(60, undecided[0] if len(undecided) else 60))  # compare up to the first near-tie of the oracle
    assert n_tok >= 30
    dec, first = new_decoder(ctx, world, fallback_margin=margin, fallback_partial=partial)
    # every third step gets the true continuation as drafts so that long accepts and rollbacks mix
    def override(tokens, position):
        done = len(tokens)
        if (position // 3) % 2 == 0:
            return cont[done:done + 9] + [-1] * 6
        return None
    tokens, stats = dec.generate(first, n_tok, draft_override_fn=override)
    assert tokens == cont[:n_tok], f"diverged at {next(i for i, (a, b) in enumerate(zip(tokens, cont)) if a != b)}"
    assert stats["stop_reason"] == "token_limit"
    assert dec.session.kv_n_pos == PROMPT_LEN + n_tok - 1
    assert stats["accepted_drafts"] > 0
    if margin >= 1e9:
        assert stats["fallback_calls"] == stats["spec_steps"]
    dec.close()


def test_generate_with_a_dflash2_head_equals_serial_greedy(ctx, world):
    """The step loop with a DFlash-2 drafter (blocks of 8, convolutions, selector walk on the device): whatever
    the selector proposes, the emitted tokens are the target's serial greedy decode."""
    cont = world["cont"]
    undecided = np.flatnonzero(~world["decided"])
    n_tok = int(min(40, undecided[0] if len(undecided) else 40))
    d2 = dfl.DraftConfig(**{**D1.as_dict(), "block_size": 8, "conv_kernel_size": 2, "conv_group_size": 64,
                            "selector_rank": 64, "selector_top_k": 16})
    head = dfl.DraftHead(ctx, d2, dfl.synth_draft_weights(d2, seed=5, vocab=C1.vocab, codebook_type=dfl.TYPE_Q8_0))
    dec = dfl.SpeculativeDecoder(ctx, world["model"], head, TAPS, 256, MASK)
    first = dec.prefill(world["prompt"])

    def override(tokens, position):  # the block has 7 drafts
        done = len(tokens)
        if (position // 3) % 2 == 0:
            return cont[done:done + 4] + [-1] * 3
        return None
    tokens, stats = dec.generate(first, n_tok, draft_override_fn=override)
    assert tokens == cont[:n_tok]
    assert stats["accepted_drafts"] > 0 and stats["spec_steps"] >= n_tok // 8
    dec.close()


def test_sampled_dflash2_step_equals_its_parts(ctx, world, oracle):
    """sampled_mode 2 (draft_block_sampled + couple_sparse_proposal, qwen/dflash.rs:508-519, 706-716;
    metal_dflash.rs:17268-17415): a speculative step with a DFlash-2 head, a proposal sampler and the target's
    sampler must decide exactly what the parts decide when composed by hand on an identical second pair of
    sessions: the oracle's sampled walk over the drafter's selector inputs, a packed verify of those tokens,
    and the oracle's accept-prefix over the verify logits with the walk's sparse proposals.  Samplers advance
    identically.  Three consecutive steps, each continuing from the previous decision."""
    d2 = dfl.DraftConfig(**{**D1.as_dict(), "block_size": 8, "conv_kernel_size": 2, "conv_group_size": 64,
                            "selector_rank": 64, "selector_top_k": 16})
    dw = dfl.synth_draft_weights(d2, seed=5, vocab=C1.vocab, codebook_type=dfl.TYPE_Q8_0)
    head = dfl.DraftHead(ctx, d2, dw)
    pred_cb, _k1 = oracle.make_codebook(dfl.TYPE_Q8_0, dw["selector_predecessor"][1], 64)
    succ_cb, _k2 = oracle.make_codebook(dfl.TYPE_Q8_0, dw["selector_successor"][1], 64)
    tkw = dict(temperature=0.9, top_k=20, top_p=0.95, min_p=0.0, seed=77)
    pkw = dict(temperature=0.9, top_k=0, top_p=1.0, min_p=0.0, seed=77 ^ 0x4446_4c41_5348_3251)
    dec = dfl.SpeculativeDecoder(ctx, world["model"], head, TAPS, 256, MASK, sampler=dfl.Sampler(**tkw),
                                 proposal_sampler=dfl.Sampler(**pkw))
    first = dec.prefill(world["prompt"])
    # the by-hand twin
    sess = dfl.Session(ctx, world["model"], 256, TAPS)
    dsess = dfl.DraftSession(ctx, head, world["model"], 256)
    for s0 in range(0, PROMPT_LEN, 16):
        blk = world["prompt"][s0:s0 + 16]
        out = sess.encode_packed_verify_layer_major(blk, s0)
        dsess.append_target_ctx_columns(out.hidden_capture, list(range(s0, s0 + len(blk))))
    otarget, oprop = oracle.make_sampler(**tkw), oracle.make_sampler(**pkw)
    carry, pos = first, PROMPT_LEN
    for _ in range(3):
        res = dec.step(carry, 1000)
        got = dfl.AcceptDecision(res.decision)
        # by hand
        dsess.draft_block(carry, MASK, pos)
        ids, vals, sel_h = (t.cpu().numpy() for t in dsess.selector_inputs())
        rc, toks, props, _err = oracle.select_draft_path_sampled(pred_cb, succ_cb, 16, 64, carry, 8, ids, vals, sel_h, oprop)
        assert rc == 0
        block = [carry] + [int(t) for t in toks[1:]]
        assert list(res.draft_tokens[:8]) == block
        out = sess.encode_packed_verify_layer_major(block, pos, want_logits=True)
        proposals = [(block[r + 1], props[r]) for r in range(7)]
        rc, want = oracle.decide_accept_prefix(block, out.logits.cpu().numpy(), C1.vocab, proposals, otarget, 1000, [])
        assert rc == 0
        assert got.key() == want.key()
        assert dec.sampler.draws == oracle.sampler_state(otarget)[1]
        assert dec.proposal_sampler.draws == oracle.sampler_state(oprop)[1]
        n_keep = want.retain_input_count
        sess.encode_restore_after_partial_accept(pos, 8, n_keep)
        dsess.append_target_ctx_columns(out.hidden_capture[:n_keep], list(range(pos, pos + n_keep)))
        pos += n_keep
        carry = want.carry_token
        assert dec.position == pos
    # a draft override has no meaning when the drafts carry their proposal distributions
    with pytest.raises(dfl.DFlashError):
        dec.step(carry, 1000, draft_override=[1, 2, 3])
    dsess.close()
    sess.close()
    dec.close()


@pytest.mark.parametrize("kw", [
    dict(temperature=0.8, top_k=20, top_p=0.95, min_p=0.0, seed=1234),
    dict(temperature=0.7, top_k=200, top_p=1.0, min_p=0.05, seed=5),   # SamplingConfig::qwen_chat (sampling.rs:47-56)
    dict(temperature=1.0, top_k=0, top_p=0.9, min_p=0.0, seed=6),      # whole-vocabulary order
], ids=["top20", "qwen_chat", "top_k_off"])
def test_generate_sampled_equals_serial_sampler(ctx, world, oracle, kw):
    """Deterministic-proposal coupling == serial sampling with the same stream (sampling.rs:2837-2865).
    The serial stream is the CPU oracle's sampler applied to the logits of a token-by-token pass through
    the same device kernels: with random-init weights the top-20 logits are near ties, so a stream
    drawn from the oracle's own logits (1e-3 away) is not a usable expectation."""
    n_tok = 40
    osamp = oracle.make_sampler(**kw)
    serial = dfl.Session(ctx, world["model"], 256, TAPS)
    out = None
    for s in range(0, PROMPT_LEN, 16):
        out = serial.encode_packed_verify_layer_major(world["prompt"][s:s + 16], s)
    want = [out.argmax_host[-1]]
    while len(want) < n_tok:
        out = serial.encode_packed_verify_layer_major([want[-1]], PROMPT_LEN + len(want) - 1, want_logits=True)
        rc, tok, _idx, _err = oracle.sample(osamp, out.logits.cpu().numpy()[0])
        assert rc == 0
        want.append(tok)
    serial.close()
    dec, first = new_decoder(ctx, world, sampler=dfl.Sampler(**kw))
    tokens, stats = dec.generate(first, n_tok, draft_override_fn=lambda t, p: want[len(t):len(t) + 6] + [-1] * 9)
    assert tokens == want
    assert stats["accepted_drafts"] > 0
    assert dec.sampler.draws == n_tok - 1 == oracle.sampler_state(osamp)[1]
    dec.close()


def device_serial_greedy(ctx, world, n_tok):
    """Token-by-token greedy decode through the device kernels (the packed verify's rows are bit-identical to
    it), for comparisons that run past the first near-tie of the CPU oracle's logits."""
    serial = dfl.Session(ctx, world["model"], 256, TAPS)
    out = None
    for s in range(0, PROMPT_LEN, 16):
        out = serial.encode_packed_verify_layer_major(world["prompt"][s:s + 16], s)
    want = [out.argmax_host[-1]]
    while len(want) < n_tok:
        want.append(serial.encode_packed_verify_layer_major([want[-1]], PROMPT_LEN + len(want) - 1).argmax_host[0])
    serial.close()
    return want


def test_adaptive_generate_backs_off_probes_and_stays_exact(ctx, world):
    """The loop under the back-off policy (qwen/dflash.rs:566-690, 1218-1231): a drafter that never hits fills the
    acceptance window, speculation turns off, exact single-token steps carry on (the drafter context stays fed, so
    probes can run), and the emitted tokens are still the target's serial greedy decode."""
    n_tok = 70
    cont = device_serial_greedy(ctx, world, n_tok)
    assert cont[:30] == world["cont"][:30]
    dec, first = new_decoder(ctx, world)
    seen = []
    tokens, stats = dec.generate(first, n_tok, adaptive=True, on_step=lambda r: seen.append(r.decision.n_accepted))
    assert tokens == cont[:n_tok]
    # 16 speculative steps fill the window (random drafter: almost nothing accepted), then off steps with a probe
    # after every 8 of them
    assert stats["spec_steps"] >= 16 and stats["off_steps"] >= 16
    assert stats["backoff_probe_steps"] >= 1 and stats["backoff_reason"] == 1
    assert stats["spec_steps"] + stats["off_steps"] + stats["accepted_drafts"] in (n_tok - 1, n_tok)
    assert dec.session.kv_n_pos == PROMPT_LEN + n_tok - 1 == dec.draft_session.ctx_len
    dec.close()


def test_adaptive_generate_stops_speculating_at_off_ctx_and_near_capacity(ctx, world):
    """Past off_ctx (or with less than a block of room) every step is an exact single-token step and the drafter
    context is no longer appended (qwen/dflash.rs:617-624)."""
    cont = world["cont"]
    undecided = np.flatnonzero(~world["decided"])
    n_tok = int(min(40, undecided[0] if len(undecided) else 40))
    dec, first = new_decoder(ctx, world)
    off_ctx = PROMPT_LEN + 12
    tokens, stats = dec.generate(first, n_tok, adaptive=True, off_ctx=off_ctx,
                                 draft_override_fn=lambda t, p: cont[len(t):len(t) + 3] + [-1] * 12)
    assert tokens == cont[:n_tok]
    assert stats["spec_steps"] == 3 and stats["accepted_drafts"] == 9  # positions 40, 44, 48; 52 >= off_ctx
    assert stats["off_steps"] == n_tok - 1 - 12
    assert dec.draft_session.ctx_len == off_ctx and dec.session.kv_n_pos == PROMPT_LEN + n_tok - 1
    dec.close()


def test_adaptive_generate_sampled_equals_serial_sampler(ctx, world, oracle):
    """Off steps draw from the same sampler stream as speculative steps, so the emitted stream is the serial one."""
    n_tok = 48
    kw = dict(temperature=0.8, top_k=20, top_p=0.95, min_p=0.0, seed=77)
    osamp = oracle.make_sampler(**kw)
    serial = dfl.Session(ctx, world["model"], 256, TAPS)
    out = None
    for s in range(0, PROMPT_LEN, 16):
        out = serial.encode_packed_verify_layer_major(world["prompt"][s:s + 16], s)
    want = [out.argmax_host[-1]]
    while len(want) < n_tok:
        out = serial.encode_packed_verify_layer_major([want[-1]], PROMPT_LEN + len(want) - 1, want_logits=True)
        rc, tok, _idx, _err = oracle.sample(osamp, out.logits.cpu().numpy()[0])
        assert rc == 0
        want.append(tok)
    serial.close()
    dec, first = new_decoder(ctx, world, sampler=dfl.Sampler(**kw))
    tokens, stats = dec.generate(first, n_tok, adaptive=True)
    assert tokens == want
    assert stats["off_steps"] > 0 and dec.sampler.draws == n_tok - 1
    dec.close()


def test_prefix_replay_feeds_a_previous_generation_and_skips_the_drafter(ctx, world):
    """Prefix replay (qwen/dflash.rs:594-612, 700-712): with a previous generation as history, every step's drafts
    are its continuation (all accepted: 15 drafts + the bonus per step), the drafter is not run (no draft time is
    recorded for a step whose drafts are all given), and when the history runs out the loop drafts again."""
    cont = world["cont"]
    undecided = np.flatnonzero(~world["decided"])
    n_tok = int(min(60, undecided[0] if len(undecided) else 60))
    history = cont[:36]
    dec, first = new_decoder(ctx, world)
    seen = []
    tokens, stats = dec.generate(first, n_tok, adaptive=True, prefix_replay=history,
                                 on_step=lambda r: seen.append((r.decision.n_accepted, r.draft_ms)))
    assert tokens == cont[:n_tok]
    # 1 + 16 + 16 = 33 tokens after two replay steps; 36 - 33 = 3 < 15 drafts left: replay ends
    assert stats["prefix_replay_steps"] == 2 and [a for a, _ in seen[:2]] == [15, 15]
    assert stats["spec_steps"] > 2 and dec.draft_session.ctx_len == dec.session.kv_n_pos == PROMPT_LEN + n_tok - 1
    # a history that disagrees with what was emitted is never replayed
    dec2, first2 = new_decoder(ctx, world)
    wrong = [cont[0] + 1] + cont[1:40]
    tokens2, stats2 = dec2.generate(first2, 30, adaptive=True, prefix_replay=wrong)
    assert tokens2 == cont[:30] and stats2["prefix_replay_steps"] == 0
    dec.close()
    dec2.close()


def test_position_margin_follows_the_reference_rule(ctx, world):
    cont = world["cont"]
    dec, first = new_decoder(ctx, world, fallback_partial=True)
    tokens, stats = dec.generate(first, 24, position_margin=True)
    assert tokens == cont[:24]
    assert abs(dec.cfg.fallback_margin - 0.1) < 1e-7  # below 16384 positions (qwen/dflash.rs:126-136)
    dec.close()


@pytest.mark.parametrize("k", [0, 5, 15])
def test_baseline_plumbing_case_prefix_512(ctx, world, k):
    """The first BASELINE configuration at its own sizes: 4-layer decoder, a prefix of 512 uniform-random tokens
    (seed 0) prefilled into the f16 KV cache, one 16-token block whose first k drafts are copied from the target's
    own continuation: the accepted prefix is exactly k and the next token is the target's.  The expectation is the
    token-by-token decode through the same kernels (the CPU oracle pins those on the short prompt above)."""
    prompt = np.random.default_rng(0).integers(0, C1.vocab - 1, 512).tolist()
    serial = dfl.Session(ctx, world["model"], 640, TAPS)
    out = None
    for s in range(0, 512, 16):
        out = serial.encode_packed_verify_layer_major(prompt[s:s + 16], s)
    cont = [out.argmax_host[-1]]
    while len(cont) < 17:
        cont.append(serial.encode_packed_verify_layer_major([cont[-1]], 512 + len(cont) - 1).argmax_host[0])
    serial.close()
    dec = dfl.SpeculativeDecoder(ctx, world["model"], world["head"], TAPS, 640, MASK)
    first = dec.prefill(prompt)
    assert first == cont[0] and dec.session.kv_n_pos == 512 == dec.draft_session.ctx_len
    wrong = [(t + 1) % (C1.vocab - 1) for t in cont[1:16]]
    res = dec.step(first, budget=1000, draft_override=cont[1:1 + k] + wrong[k:])
    d = res.decision
    assert d.n_accepted == k and list(d.accepted_drafts[:k]) == cont[1:1 + k] and d.carry_token == cont[k + 1]
    assert dec.session.kv_n_pos == 512 + k + 1 == dec.position == dec.draft_session.ctx_len
    dec.close()


def test_draft_graph_replays_equal_eager_blocks(ctx, world):
    """The drafter's block forward replayed from its captured graph gives the very logits the launches give one by one:
    eight consecutive blocks on two sessions (graph on / off) as the context grows by a ragged number of columns per
    step, with eager work (verify, context append, read-backs) and synchronisations between the replays; then a whole
    generation with the graph on equals the one with it off."""
    import torch
    head = dfl.DraftHead(ctx, D1, dfl.synth_draft_weights(D1, seed=4))
    model = world["model"]
    sess = dfl.Session(ctx, model, 256, TAPS)
    ds = {True: dfl.DraftSession(ctx, head, model, 256), False: dfl.DraftSession(ctx, head, model, 256)}
    outs = {g: (torch.empty(D1.block_size, dtype=torch.int32, device="cuda"),
                torch.empty((D1.block_size, C1.vocab), dtype=torch.float32, device="cuda")) for g in ds}
    for s0 in range(0, PROMPT_LEN, 16):
        blk = world["prompt"][s0:s0 + 16]
        out = sess.encode_packed_verify_layer_major(blk, s0)
        for d in ds.values():
            d.append_target_ctx_columns(out.hidden_capture, list(range(s0, s0 + len(blk))))
    pos, carry = PROMPT_LEN, int(out.argmax_host[-1])
    rng = np.random.default_rng(3)
    try:
        for step in range(8):
            got = {}
            for g, d in ds.items():
                ctx.set_draft_graphs(g)
                d.draft_block(carry, MASK, pos, want_logits=True, out=outs[g])
                got[g] = (outs[g][0].cpu().numpy().copy(), outs[g][1].cpu().numpy().copy())
            assert np.array_equal(got[True][0], got[False][0]), f"step {step}: draft tokens differ"
            assert np.array_equal(got[True][1].view(np.uint32), got[False][1].view(np.uint32)), f"step {step}: logits differ"
            # eager work between replays: verify a block, keep a ragged prefix, append its columns to both drafters
            keep = int(rng.integers(1, 9))
            block = [carry] + [int(t) for t in got[True][0][1:]]
            v = sess.encode_packed_verify_layer_major(block, pos)
            sess.encode_restore_after_partial_accept(pos, len(block), keep)
            for d in ds.values():
                d.append_target_ctx_columns(v.hidden_capture[:keep], list(range(pos, pos + keep)))
            carry, pos = int(v.argmax_host[keep - 1]), pos + keep
        assert ds[True].graph_replays >= 6 and ds[False].graph_replays == 0
        results = {}
        for g in (True, False):
            ctx.set_draft_graphs(g)
            dec = dfl.SpeculativeDecoder(ctx, model, head, TAPS, 256, MASK)
            first = dec.prefill(world["prompt"])
            results[g] = dec.generate(first, 40)[0]
            if g:
                assert dec.draft_session.graph_replays > 0
            dec.close()
        assert results[True] == results[False]
    finally:
        ctx.set_draft_graphs(False)
        sess.close()
        for d in ds.values():
            d.close()
