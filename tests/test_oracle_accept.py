"""Accept-prefix decision of the CPU oracle against the value-specified cases of the
reference's own tests (crates/qwen-llm/src/metal_dflash/accept.rs:236-616)."""
import numpy as np

VOCAB = 6
INPUT = [0, 1, 2, 3]


def sampler(oracle, temperature, seed=17, **kw):
    return oracle.make_sampler(temperature, top_k=kw.pop("top_k", 1), seed=seed, **kw)


def logits(winners):
    v = np.full((len(winners), VOCAB), -10.0, np.float32)
    for r, t in enumerate(winners):
        v[r, t] = 10.0
    return v


def one_hot_proposals():
    return [(t, [(t, 1.0)]) for t in INPUT[1:]]


def same_rng(oracle, a, b):
    assert oracle.sampler_state(a) == oracle.sampler_state(b)


def at_draw(oracle, s, draws):
    c = s.cfg
    return oracle.make_sampler(c.temperature, c.top_k, c.top_p, c.min_p, c.seed, c.rng_kind, draws)


def test_every_rejection_position(oracle):
    """accept.rs:236-273"""
    for temperature in [0.0, 1.0]:
        for sparse in [False, True]:
            for rejected_row in range(3):
                winners = [1, 2, 3, 4]
                winners[rejected_row] = 5
                rows = logits(winners)
                rows[rejected_row + 1:] = np.nan
                req = sampler(oracle, temperature)
                rc, d = oracle.decide_accept_prefix(INPUT, rows, VOCAB, one_hot_proposals() if sparse else None, req,
                                                    4, [])
                assert rc == 0
                assert d.accepted() == INPUT[1:1 + rejected_row]
                assert (d.carry_kind, d.carry_token) == (oracle.CARRY_CORRECTION, 5)
                assert d.stop_reason == oracle.STOP_NONE
                assert d.retain_input_count == 1 + rejected_row
                draws = rejected_row + 2 if sparse else (rejected_row + 1 if temperature > 0 else 0)
                same_rng(oracle, req, at_draw(oracle, req, draws))


def test_all_accepted_samples_bonus(oracle):
    """accept.rs:275-313"""
    for temperature in [0.0, 1.0]:
        for sparse in [False, True]:
            req = sampler(oracle, temperature)
            rc, d = oracle.decide_accept_prefix(INPUT, logits([1, 2, 3, 4]), VOCAB,
                                                one_hot_proposals() if sparse else None, req, 4, [])
            assert rc == 0
            assert d.key() == ([1, 2, 3], oracle.CARRY_BONUS, 4, oracle.STOP_NONE, 4)
            draws = 4 if temperature > 0 else (3 if sparse else 0)
            same_rng(oracle, req, at_draw(oracle, req, draws))


def test_eos_and_cap_at_every_accepted_position(oracle):
    """accept.rs:315-361"""
    for sparse in [False, True]:
        for terminal_count in range(1, 4):
            for eos, cap in [(True, False), (False, True), (True, True)]:
                rows = logits([1, 2, 3, 4])
                rows[terminal_count:] = np.nan
                proposals = one_hot_proposals()
                for i in range(terminal_count, len(proposals)):
                    proposals[i] = (proposals[i][0], [(proposals[i][0], float("nan"))])
                stops = [INPUT[terminal_count]] if eos else []
                req = sampler(oracle, 1.0)
                rc, d = oracle.decide_accept_prefix(INPUT, rows, VOCAB, proposals if sparse else None, req,
                                                    terminal_count if cap else 4, stops)
                assert rc == 0
                assert d.accepted() == INPUT[1:terminal_count + 1]
                assert d.carry_kind == oracle.CARRY_NONE
                assert d.stop_reason == (oracle.STOP_EOS if eos else oracle.STOP_TOKEN_LIMIT)
                assert d.retain_input_count == terminal_count
                same_rng(oracle, req, at_draw(oracle, req, terminal_count))


def test_terminal_anchor_and_zero_budget(oracle):
    """accept.rs:363-395"""
    for inp in [INPUT[:1], INPUT]:
        for budget, stops, reason in [(0, [], oracle.STOP_TOKEN_LIMIT), (0, [0], oracle.STOP_EOS),
                                      (4, [0], oracle.STOP_EOS)]:
            req = sampler(oracle, 1.0)
            before = oracle.clone_sampler(req)
            rc, d = oracle.decide_accept_prefix(inp, np.full((len(inp), VOCAB), np.nan, np.float32), VOCAB, None,
                                                req, budget, stops)
            assert rc == 0
            assert d.key() == ([], oracle.CARRY_NONE, 0, reason, 0)
            same_rng(oracle, req, before)


def test_anchor_only_bonus_and_rejection_carry(oracle):
    """accept.rs:397-441"""
    for proposals in [None, []]:
        req = sampler(oracle, 1.0)
        rc, d = oracle.decide_accept_prefix([0], logits([4]), VOCAB, proposals, req, 1, [4])
        assert rc == 0
        assert d.key() == ([], oracle.CARRY_BONUS, 4, oracle.STOP_NONE, 1)
        assert req.draws == 1
    rc, d = oracle.decide_accept_prefix(INPUT, logits([5, 2, 3, 4]), VOCAB, None, sampler(oracle, 1.0), 1, [5])
    assert rc == 0
    assert d.key() == ([], oracle.CARRY_CORRECTION, 5, oracle.STOP_NONE, 1)


def test_sparse_coupling_uses_actual_q_and_target_filters(oracle):
    """accept.rs:443-535"""
    target_row = np.array([2.0, 1.9, 1.5, 0.5, -1.0, -2.0], np.float32)
    rows = np.concatenate([target_row[None], logits([4])])
    high_q = (0, [(0, 8.0), (1, 1.0), (5, 1.0)])
    low_q = (0, [(0, 1.0), (1, 99.0)])
    accepted = rejected = 0
    for seed in range(64):
        kw = dict(top_k=4, top_p=0.7, min_p=0.5, seed=seed)
        req = oracle.make_sampler(0.7, **kw)
        ref = oracle.clone_sampler(req)
        rc, acc, corr = oracle.couple_sparse(ref, target_row, *high_q)
        assert rc == 0
        if acc:
            accepted += 1
            bonus = oracle.sample(ref, rows[1])[1]
            expected = ([0], oracle.CARRY_BONUS, bonus, oracle.STOP_NONE, 2)
        else:
            rejected += 1
            assert corr == 1
            expected = ([], oracle.CARRY_CORRECTION, corr, oracle.STOP_NONE, 1)
        rc, d = oracle.decide_accept_prefix([3, 0], rows, VOCAB, [high_q], req, 2, [])
        assert rc == 0 and d.key() == expected
        same_rng(oracle, req, ref)

        rc, d = oracle.decide_accept_prefix([3, 0], rows, VOCAB, [low_q], oracle.make_sampler(0.7, **kw), 2, [])
        assert rc == 0 and d.accepted() == [0]

        # token 2 is removed by the target's top-p after top-k / min-p / temperature
        req = oracle.make_sampler(0.7, **kw)
        rc, d = oracle.decide_accept_prefix([3, 2], rows, VOCAB, [(2, [(2, 1.0), (0, 99.0)])], req, 2, [])
        assert rc == 0 and d.accepted() == []
        assert d.carry_kind == oracle.CARRY_CORRECTION and d.carry_token in (0, 1)
        assert req.draws == 2
    assert accepted > 0 and rejected > 0


def test_malformed_inputs_leave_rng_unchanged(oracle):
    """accept.rs:537-576"""
    rows = logits([1, 2, 3, 4])
    proposals = one_hot_proposals()
    mismatch = list(proposals)
    mismatch[2] = (4, mismatch[2][1])
    invalid_candidate = list(proposals)
    invalid_candidate[2] = (invalid_candidate[2][0], [(-1, 1.0)])
    flat = rows.reshape(-1)
    cases = [
        ([], np.zeros(0, np.float32), VOCAB, None),
        (INPUT, flat, 0, None),
        (INPUT, flat, 2 ** 63, None),
        (INPUT, flat[:-1], VOCAB, None),
        (INPUT[:3], flat, VOCAB, None),
        ([-1, 1, 2, 3], flat, VOCAB, None),
        ([0, 1, 2, 6], flat, VOCAB, None),
        (INPUT, flat, VOCAB, proposals[:2]),
        (INPUT, flat, VOCAB, mismatch),
        (INPUT, flat, VOCAB, invalid_candidate),
    ]
    for inp, r, vocab, props in cases:
        for budget in [0, 4]:
            req = sampler(oracle, 1.0)
            before = oracle.clone_sampler(req)
            rc, _ = oracle.decide_accept_prefix(inp, r, vocab, props, req, budget, [])
            assert rc != 0
            same_rng(oracle, req, before)


def test_errors_after_accepted_rows_roll_back_rng(oracle):
    """accept.rs:578-616"""
    for row in range(1, 4):
        rows = logits([1, 2, 3, 4])
        rows[row, 0] = np.nan
        req = sampler(oracle, 1.0)
        before = oracle.clone_sampler(req)
        rc, d = oracle.decide_accept_prefix(INPUT, rows, VOCAB, None, req, 4, [])
        assert rc == 5 and d.err_row == row  # NanLogit at that row
        same_rng(oracle, req, before)
    rows = logits([1, 2, 3, 4])
    for invalid in [(2, []), (2, [(2, -1.0)]), (2, [(2, float("nan"))]), (2, [(2, 0.0)]), (2, [(1, 1.0)])]:
        proposals = one_hot_proposals()
        proposals[1] = invalid
        req = sampler(oracle, 1.0)
        before = oracle.clone_sampler(req)
        rc, d = oracle.decide_accept_prefix(INPUT, rows, VOCAB, proposals, req, 4, [])
        assert rc != 0 and d.err_row == 1
        same_rng(oracle, req, before)


def test_dense_block_decision_equals_rowwise_couplings(oracle):
    """The dense block decision is the accept-prefix loop over dense couplings."""
    rng = np.random.default_rng(9)
    vocab, n = 500, 6
    for trial in range(50):
        tl = (rng.standard_normal((n, vocab)) * 3).astype(np.float32)
        dl = (tl + rng.standard_normal((n, vocab)) * 0.5).astype(np.float32)
        toks = [int(rng.integers(0, vocab))] + [int(np.argmax(dl[r])) for r in range(n - 1)]
        kw = dict(temperature=0.7, top_k=20, top_p=0.95, seed=trial, rng_kind=oracle.RNG_PHILOX)
        a, b = oracle.make_sampler(**kw), oracle.make_sampler(**kw)
        rc, d = oracle.decide_accept_prefix_dense(toks, tl, dl, vocab, 0.7, a, 100, [])
        assert rc == 0
        acc = []
        carry = None
        for r in range(n - 1):
            rc, ok, corr = oracle.couple_dense(b, tl[r], dl[r], 0.7, toks[r + 1])
            assert rc == 0
            if not ok:
                carry = (oracle.CARRY_CORRECTION, corr)
                break
            acc.append(toks[r + 1])
        if carry is None:
            carry = (oracle.CARRY_BONUS, oracle.sample(b, tl[n - 1])[1])
        assert (d.accepted(), d.carry_kind, d.carry_token) == (acc, carry[0], carry[1])
        same_rng(oracle, a, b)


def test_batched_decisions_equal_single_calls(oracle):
    """The OpenMP batch entry used by the long GPU runs is the per-block decision, trial by trial."""
    rng = np.random.default_rng(12)
    V, n, T, B = 3000, 6, 0.7, 9
    tl = (rng.standard_normal((B, n, V)) * 3).astype(np.float32)
    dl = tl[:, : n - 1] + rng.standard_normal((B, n - 1, V)).astype(np.float32) * 0.5
    toks = rng.integers(0, V, (B, n)).astype(np.int32)
    toks[:, 1:] = dl.argmax(axis=2)
    for dense in (True, False):
        for kind in (0, 1):
            a = [oracle.make_sampler(T, 20, 0.95, 0.0, 100 + b, kind) for b in range(B)]
            b_ = [oracle.make_sampler(T, 20, 0.95, 0.0, 100 + b, kind) for b in range(B)]
            status, outs = oracle.decide_accept_prefix_batch(toks, tl, dl if dense else None, T, a, 50)
            for t in range(B):
                if dense:
                    rc, od = oracle.decide_accept_prefix_dense(toks[t].tolist(), tl[t], dl[t], V, T, b_[t], 50, [])
                else:
                    rc, od = oracle.decide_accept_prefix(toks[t].tolist(), tl[t], V, None, b_[t], 50, [])
                assert rc == status[t] == 0 and od.key() == outs[t].key()
                assert oracle.sampler_state(a[t]) == oracle.sampler_state(b_[t])
