"""GPU parity, bit-exact: argmax / top-2 gap / top-16, and the accept-prefix decision (greedy
longest-prefix, deterministic coupling, sparse and vocabulary-wide rejection sampling) against
the CPU oracle on the same logits and the same random stream."""
import math

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


# ----------------------------------------------------------------------------- argmax family


def special_rows():
    rng = np.random.default_rng(0x5A17)
    specials = np.array([0.0, -0.0, np.inf, -np.inf, 1.17549435e-38, -1.17549435e-38, 1e-45, -1e-45, 3.4028235e38,
                         -3.4028235e38, 1.0, -1.0], np.float32)
    rows = []
    for n in [1, 2, 3, 31, 32, 33, 1023, 1025, 8191, 8192, 8193, 40000, 151936, 248320]:
        rows.append((rng.random(n) * 60 - 30).astype(np.float32))
        rows.append((rng.integers(0, 4, n) - 1.5).astype(np.float32))
        rows.append(specials[rng.integers(0, len(specials), n)])
        rows.append(np.full(n, 2.5, np.float32))
        r = np.full(n, -1.0, np.float32)
        r[n // 2] = 3.0
        r[n - 1] = 3.0
        rows.append(r)
        rows.append(np.full(n, -np.inf, np.float32))
    return rows


def test_argmax_top2_matches_oracle(ctx, oracle):
    """metal/elementwise.rs:3975-4231 cases + ties, signed zeros, infinities, boundary widths"""
    for row in special_rows():
        idx, gap = ctx.argmax_top2(dev(row))
        wi, wg = oracle.argmax_top2(row)
        assert int(idx[0]) == wi, f"n={len(row)}"
        g = float(gap[0])
        assert (math.isnan(g) and math.isnan(wg)) or g == wg, f"n={len(row)} gap {g} vs {wg}"
    assert int(ctx.argmax_top2(dev(np.full(1024, np.nan, np.float32)))[0][0]) == -1


def test_argmax_top2_batched_rows(ctx, oracle):
    rng = np.random.default_rng(1)
    x = (rng.standard_normal((16, 151936)) * 3).astype(np.float32)
    x[3, 777] = x[3].max()  # duplicate maximum -> gap 0
    idx, gap = ctx.argmax_top2(dev(x))
    for r in range(16):
        assert (int(idx[r]), float(gap[r])) == oracle.argmax_top2(x[r])


def test_argmax_greedy_total_order_and_nan(ctx, oracle):
    """sampling.rs:1159-1181, 1904-1909; NaN rows report ~(lowest NaN index)"""
    rows = special_rows() + [np.array(r, np.float32) for r in
                             ([1, 5, 5, 3], [2, 2, 2], [-0.0, 0.0, -0.0], [0.0, -0.0, 0.0], [1, 3, 3])]
    for row in rows:
        got = int(ctx.argmax_greedy(dev(row))[0])
        rc, tok, _ = oracle.greedy_token(row)
        assert rc == 0 and got == tok, f"n={len(row)}"
    row = np.random.default_rng(2).standard_normal(50000).astype(np.float32)
    row[[40000, 123, 9000]] = np.nan
    assert int(ctx.argmax_greedy(dev(row))[0]) == ~123
    assert oracle.greedy_token(row)[2] == 123


def test_top16_matches_oracle(ctx, oracle, canaries):
    for row in special_rows():
        ids, vals = ctx.top16(dev(row))
        wi, wv = oracle.top16(row)
        assert np.array_equal(ids[0].cpu().numpy(), wi), f"n={len(row)}"
        assert np.array_equal(vals[0].cpu().numpy().view(np.uint32), wv.view(np.uint32))
    x = (np.random.default_rng(3).integers(-50, 50, (16, 151936))).astype(np.float32)  # heavy ties
    ids, vals = ctx.top16(dev(x))
    for r in range(16):
        wi, wv = oracle.top16(x[r])
        assert np.array_equal(ids[r].cpu().numpy(), wi)
        assert np.array_equal(vals[r].cpu().numpy(), wv)


# ----------------------------------------------------------------------------- accept-prefix

VOCAB = 6
INPUT = [0, 1, 2, 3]


def logits(winners):
    v = np.full((len(winners), VOCAB), -10.0, np.float32)
    for r, t in enumerate(winners):
        v[r, t] = 10.0
    return v


def one_hot_proposals():
    return [(t, [(t, 1.0)]) for t in INPUT[1:]]


def both(ctx, oracle, toks, rows, vocab, proposals, budget, stops, draft=None, draft_T=0.0, **skw):
    """run the GPU decision and the oracle on identical inputs; return (gpu, oracle, samplers)"""
    gs = dfl.Sampler(**skw)
    os_ = oracle.make_sampler(skw.get("temperature", 0.0), skw.get("top_k", 0), skw.get("top_p", 1.0),
                              skw.get("min_p", 0.0), skw.get("seed", 0), skw.get("rng_kind", 0))
    rows = np.ascontiguousarray(rows, np.float32)
    if draft is not None:
        rc, od = oracle.decide_accept_prefix_dense(toks, rows, draft, vocab, draft_T, os_, budget, stops)
    else:
        rc, od = oracle.decide_accept_prefix(toks, rows, vocab, proposals, os_, budget, stops)
    try:
        gd = ctx.decide_dflash_accept_prefix(toks, dev(rows), vocab, proposals, gs, budget, stops,
                                             draft_logits=dev(draft) if draft is not None else None,
                                             draft_temperature=draft_T)
        grc = 0
    except dfl.DFlashError as e:
        gd, grc = e, e.status
    return grc, gd, rc, od, gs, os_


def assert_same(oracle, grc, gd, rc, od, gs, os_):
    assert (grc == 0) == (rc == 0), f"gpu status {grc} vs oracle {rc}"
    if rc == 0:
        assert gd.key() == od.key()
    else:
        assert grc == 32 + rc or grc in (7, 8, 9, 40), (grc, rc)
    assert gs.state() == oracle.sampler_state(os_)


def test_reference_accept_cases(ctx, oracle):
    """accept.rs:236-441: every rejection position, all accepted + bonus, EOS / cap at every
    position, terminal anchor, zero budget, anchor-only"""
    for temperature in [0.0, 1.0]:
        for sparse in [False, True]:
            for rejected_row in range(3):
                winners = [1, 2, 3, 4]
                winners[rejected_row] = 5
                rows = logits(winners)
                rows[rejected_row + 1:] = np.nan
                r = both(ctx, oracle, INPUT, rows, VOCAB, one_hot_proposals() if sparse else None, 4, [],
                         temperature=temperature, top_k=1, seed=17)
                assert_same(oracle, *r)
                gd = r[1]
                assert gd.accepted_drafts == INPUT[1:1 + rejected_row]
                assert (gd.carry_kind, gd.carry_token) == (dfl.CARRY_CORRECTION, 5)
                assert gd.retain_input_count == 1 + rejected_row
                want_draws = rejected_row + 2 if sparse else (rejected_row + 1 if temperature > 0 else 0)
                assert r[4].draws == want_draws
            r = both(ctx, oracle, INPUT, logits([1, 2, 3, 4]), VOCAB, one_hot_proposals() if sparse else None, 4, [],
                     temperature=temperature, top_k=1, seed=17)
            assert_same(oracle, *r)
            assert r[1].key() == ([1, 2, 3], dfl.CARRY_BONUS, 4, dfl.STOP_NONE, 4)
    for sparse in [False, True]:
        for terminal_count in range(1, 4):
            for eos, cap in [(True, False), (False, True), (True, True)]:
                rows = logits([1, 2, 3, 4])
                rows[terminal_count:] = np.nan
                props = one_hot_proposals()
                for i in range(terminal_count, len(props)):
                    props[i] = (props[i][0], [(props[i][0], float("nan"))])
                stops = [INPUT[terminal_count]] if eos else []
                r = both(ctx, oracle, INPUT, rows, VOCAB, props if sparse else None, terminal_count if cap else 4,
                         stops, temperature=1.0, top_k=1, seed=17)
                assert_same(oracle, *r)
                assert r[1].stop_reason == (dfl.STOP_EOS if eos else dfl.STOP_TOKEN_LIMIT)
                assert r[1].retain_input_count == terminal_count and r[4].draws == terminal_count
    for inp in [INPUT[:1], INPUT]:
        for budget, stops in [(0, []), (0, [0]), (4, [0])]:
            r = both(ctx, oracle, inp, np.full((len(inp), VOCAB), np.nan, np.float32), VOCAB, None, budget, stops,
                     temperature=1.0, top_k=1, seed=17)
            assert_same(oracle, *r)
            assert r[1].retain_input_count == 0 and r[4].draws == 0
    r = both(ctx, oracle, [0], logits([4]), VOCAB, None, 1, [4], temperature=1.0, top_k=1, seed=17)
    assert_same(oracle, *r)
    assert r[1].key() == ([], dfl.CARRY_BONUS, 4, dfl.STOP_NONE, 1)


def test_sparse_coupling_uses_actual_q_and_target_filters(ctx, oracle):
    """accept.rs:443-535"""
    target_row = np.array([2.0, 1.9, 1.5, 0.5, -1.0, -2.0], np.float32)
    rows = np.concatenate([target_row[None], logits([4])])
    accepted = rejected = 0
    for seed in range(64):
        kw = dict(temperature=0.7, top_k=4, top_p=0.7, min_p=0.5, seed=seed)
        for props, toks in [([(0, [(0, 8.0), (1, 1.0), (5, 1.0)])], [3, 0]), ([(0, [(0, 1.0), (1, 99.0)])], [3, 0]),
                            ([(2, [(2, 1.0), (0, 99.0)])], [3, 2])]:
            r = both(ctx, oracle, toks, rows, VOCAB, props, 2, [], **kw)
            assert_same(oracle, *r)
        accepted += len(r[1].accepted_drafts) == 0
    assert accepted > 0


def test_malformed_inputs_and_late_errors_leave_rng_unchanged(ctx, oracle):
    """accept.rs:537-616"""
    rows = logits([1, 2, 3, 4])
    props = one_hot_proposals()
    mismatch = list(props)
    mismatch[2] = (4, mismatch[2][1])
    bad_cand = list(props)
    bad_cand[2] = (bad_cand[2][0], [(-1, 1.0)])
    for toks, r_, vocab, p in [([-1, 1, 2, 3], rows, VOCAB, None), ([0, 1, 2, 6], rows, VOCAB, None),
                               (INPUT, rows, VOCAB, props[:2]), (INPUT, rows, VOCAB, mismatch),
                               (INPUT, rows, VOCAB, bad_cand)]:
        for budget in [0, 4]:
            s = dfl.Sampler(1.0, top_k=1, seed=17)
            before = s.state()
            with pytest.raises(dfl.DFlashError):
                ctx.decide_dflash_accept_prefix(toks, dev(r_), vocab, p, s, budget, [])
            assert s.state() == before
    s = dfl.Sampler(1.0, top_k=1, seed=17)
    with pytest.raises(dfl.DFlashError):
        ctx.decide_dflash_accept_prefix(INPUT[:3], dev(rows), VOCAB, None, s, 4, [])  # extent mismatch
    with pytest.raises(dfl.DFlashError):
        ctx.decide_dflash_accept_prefix([], dev(rows), VOCAB, None, s, 4, [])
    for row in range(1, 4):
        bad = logits([1, 2, 3, 4])
        bad[row, 0] = np.nan
        r = both(ctx, oracle, INPUT, bad, VOCAB, None, 4, [], temperature=1.0, top_k=1, seed=17)
        assert_same(oracle, *r)
        assert r[0] == 37 and r[1].decision.err_row == row and r[4].draws == 0
    for invalid in [(2, []), (2, [(2, -1.0)]), (2, [(2, float("nan"))]), (2, [(2, 0.0)]), (2, [(1, 1.0)])]:
        p = one_hot_proposals()
        p[1] = invalid
        r = both(ctx, oracle, INPUT, rows, VOCAB, p, 4, [], temperature=1.0, top_k=1, seed=17)
        assert_same(oracle, *r)
        assert r[0] != 0 and r[1].decision.err_row == 1


def block_inputs(rng, vocab, n, spread=0.5):
    tl = (rng.standard_normal((n, vocab)) * 3).astype(np.float32)
    dl = (tl[: n - 1] + rng.standard_normal((n - 1, vocab)) * spread).astype(np.float32)
    return tl, dl


def sample_drafts(dl, T, rng):
    """draft tokens drawn from softmax(draft / T) (input generation only)"""
    z = dl.astype(np.float64) / T
    p = np.exp(z - z.max(axis=1, keepdims=True))
    p /= p.sum(axis=1, keepdims=True)
    return [int(rng.choice(len(row), p=row)) for row in p]


@pytest.mark.parametrize("mode", ["deterministic", "sparse", "dense"])
@pytest.mark.parametrize("kind", [dfl.RNG_XOSHIRO, dfl.RNG_PHILOX])
def test_seeded_trials_small_vocab(ctx, oracle, mode, kind):
    """10000 seeded trials per stream over a 2048-token vocabulary: accepted length, tokens, carry,
    stop reason and draws identical to the oracle's (T 0.7, top-p 0.95, top-k 20)"""
    vocab, n = 2048, 16
    T = 0.7
    n_trials = 10000 if mode != "sparse" else 2000
    import torch

    lengths = np.zeros(n + 1, np.int64)
    for base in range(0, n_trials, 250):
        rng = np.random.default_rng(1000 + base)
        tls, dls = [], []
        for _ in range(250):
            tl, dl = block_inputs(rng, vocab, n)
            tls.append(tl)
            dls.append(dl)
        tl_dev = dev(np.stack(tls))
        dl_dev = dev(np.stack(dls))
        for t in range(250):
            seed = base + t
            tl, dl = tls[t], dls[t]
            drafts = sample_drafts(dl, T, rng) if mode != "deterministic" else \
                [int(np.argmax(tl[r])) if rng.random() < 0.8 else int(rng.integers(vocab)) for r in range(n - 1)]
            toks = [int(rng.integers(vocab))] + drafts
            skw = dict(temperature=T, top_k=20, top_p=0.95, seed=seed, rng_kind=kind)
            gs = dfl.Sampler(**skw)
            os_ = oracle.make_sampler(T, 20, 0.95, 0.0, seed, kind)
            if mode == "dense":
                rc, od = oracle.decide_accept_prefix_dense(toks, tl, dl, vocab, T, os_, 100, [])
                gd = ctx.decide_dflash_accept_prefix(toks, tl_dev[t], vocab, None, gs, 100, [], draft_logits=dl_dev[t],
                                                     draft_temperature=T)
            elif mode == "sparse":
                props = []
                for r in range(n - 1):
                    top = np.argsort(-dl[r])[:16]
                    if drafts[r] not in top:
                        top[-1] = drafts[r]
                    z = dl[r][top].astype(np.float64) / T
                    props.append((drafts[r], [(int(a), float(b)) for a, b in zip(top, np.exp(z - z.max()))]))
                rc, od = oracle.decide_accept_prefix(toks, tl, vocab, props, os_, 100, [])
                gd = ctx.decide_dflash_accept_prefix(toks, tl_dev[t], vocab, props, gs, 100, [])
            else:
                rc, od = oracle.decide_accept_prefix(toks, tl, vocab, None, os_, 100, [])
                gd = ctx.decide_dflash_accept_prefix(toks, tl_dev[t], vocab, None, gs, 100, [])
            assert rc == 0
            assert gd.key() == od.key(), f"trial {seed}"
            assert gs.state() == oracle.sampler_state(os_), f"trial {seed}"
            lengths[len(gd.accepted_drafts)] += 1
        del tl_dev, dl_dev
        torch.cuda.empty_cache()
    assert lengths[0] > 0 and lengths[1:].sum() > 0  # both outcomes exercised


@pytest.mark.parametrize("vocab", [16384 + 5, 2 * 16384 + 63, 3 * 16384])
@pytest.mark.parametrize("top_k", [2, 20, 64])
def test_selection_at_chunk_boundaries(ctx, oracle, vocab, top_k):
    """The top-k selection cuts a row into 16384-token chunks.  Vocabularies whose last chunk holds fewer tokens than
    k (every one of them is then a candidate of its chunk), exactly fills, or ends one short of a wave; rows whose
    winners all sit in one chunk, straddle a boundary, or are -inf but for a handful: decisions and sampler state
    equal the oracle's, dense and deterministic drafts, 40 seeds each."""
    n, T = 16, 0.7
    rng = np.random.default_rng(vocab * 131 + top_k)
    tl, dl = block_inputs(rng, vocab, n)
    tl[1, :] = -np.inf
    tl[1, rng.integers(0, vocab, 5)] = rng.standard_normal(5).astype(np.float32)      # fewer finite logits than k
    tl[2, 16384 - 3:16384 + 3] += 30.0                                                  # winners on both sides of a cut
    tl[3, vocab - 4:] += 30.0                                                           # winners at the ragged end
    tl[4, :16384] -= 50.0                                                               # one chunk out of the running
    dl = (tl[: n - 1] + rng.standard_normal((n - 1, vocab)) * 0.5).astype(np.float32)
    dl[~np.isfinite(dl)] = -30.0
    tl_dev, dl_dev = dev(tl), dev(dl)
    lengths = set()
    for seed in range(40):
        r2 = np.random.default_rng(seed)
        drafts = [int(np.argmax(tl[r])) if r2.random() < 0.8 else int(r2.integers(vocab)) for r in range(n - 1)]
        toks = [int(r2.integers(vocab))] + drafts
        for dense in (False, True):
            gs = dfl.Sampler(temperature=T, top_k=top_k, top_p=0.95, seed=seed, rng_kind=dfl.RNG_PHILOX)
            os_ = oracle.make_sampler(T, top_k, 0.95, 0.0, seed, dfl.RNG_PHILOX)
            if dense:
                rc, od = oracle.decide_accept_prefix_dense(toks, tl, dl, vocab, T, os_, 100, [])
                gd = ctx.decide_dflash_accept_prefix(toks, tl_dev, vocab, None, gs, 100, [], draft_logits=dl_dev, draft_temperature=T)
            else:
                rc, od = oracle.decide_accept_prefix(toks, tl, vocab, None, os_, 100, [])
                gd = ctx.decide_dflash_accept_prefix(toks, tl_dev, vocab, None, gs, 100, [])
            assert rc == 0
            assert gd.key() == od.key(), f"seed {seed} dense {dense}"
            assert gs.state() == oracle.sampler_state(os_), f"seed {seed} dense {dense}"
            lengths.add(len(gd.accepted_drafts))
    assert len(lengths) > 1


@pytest.mark.parametrize("kind,n_trials", [(dfl.RNG_PHILOX, 10000), (dfl.RNG_XOSHIRO, 2000)])
def test_seeded_trials_full_vocab_dense(ctx, oracle, kind, n_trials):
    """Stochastic acceptance at its benchmark size: vocabulary 151936, block 16, target logits N(0, 3), draft = target +
    N(0, 0.5), temperature 0.7 / top-p 0.95 / top-k 20, vocabulary-wide draft distribution; seeds 0 .. n_trials - 1:
    10000 trials on the Philox stream, 2000 on xoshiro256++.  Accepted length, tokens, carry, stop reason and
    draws used equal the oracle's in every trial.  Logits are generated on the device a batch at a time and copied
    to the host, where the oracle decides the batch's trials in parallel."""
    import torch

    vocab, n, T, batch = 151936, 16, 0.7, 32
    g = torch.Generator(device="cuda")
    acc_hist = np.zeros(n, np.int64)
    for b0 in range(0, n_trials, batch):
        nb = min(batch, n_trials - b0)
        g.manual_seed(1_000_003 * (kind + 1) + b0)
        tl = torch.randn((nb, n, vocab), device="cuda", generator=g) * 3
        dl = tl[:, : n - 1] + torch.randn((nb, n - 1, vocab), device="cuda", generator=g) * 0.5
        drafts = torch.multinomial(torch.softmax(dl.reshape(-1, vocab).double() / T, dim=1), 1, generator=g).reshape(nb, n - 1)
        toks = torch.cat([torch.arange(b0, b0 + nb, device="cuda").reshape(nb, 1) % vocab, drafts], dim=1).to(torch.int32).cpu().numpy()
        gpu = []
        for t in range(nb):
            gs = dfl.Sampler(T, top_k=20, top_p=0.95, seed=b0 + t, rng_kind=kind)
            gd = ctx.decide_dflash_accept_prefix(toks[t].tolist(), tl[t], vocab, None, gs, 100, [], draft_logits=dl[t],
                                                 draft_temperature=T)
            gpu.append((gd, gs))
        samplers = [oracle.make_sampler(T, 20, 0.95, 0.0, b0 + t, kind) for t in range(nb)]
        status, outs = oracle.decide_accept_prefix_batch(toks, tl.cpu().numpy(), dl.cpu().numpy(), T, samplers, 100)
        for t in range(nb):
            gd, gs = gpu[t]
            assert status[t] == 0 and gd.key() == outs[t].key(), f"trial {b0 + t}"
            assert gs.state() == oracle.sampler_state(samplers[t]), f"trial {b0 + t}"
            acc_hist[len(gd.accepted_drafts)] += 1
        del tl, dl
    assert acc_hist.sum() == n_trials and acc_hist[0] > 0 and acc_hist[1:].sum() > 0  # rejections at row 0 and later


def test_greedy_longest_prefix_full_vocab(ctx, oracle):
    """greedy acceptance == longest prefix with draft[i] == argmax(row i) (qwen/dflash.rs:838-858)"""
    rng = np.random.default_rng(4)
    vocab, n = 32000, 16
    tl = (rng.standard_normal((n, vocab)) * 3).astype(np.float32)
    am = tl.argmax(axis=1)
    for k in [0, 1, 7, 15]:
        drafts = [int(am[r]) if r < k else int((am[r] + 1) % vocab) for r in range(n - 1)]
        r = both(ctx, oracle, [5] + drafts, tl, vocab, None, 100, [], temperature=0.0)
        assert_same(oracle, *r)
        assert r[1].accepted_drafts == drafts[:k]
        want_kind = dfl.CARRY_BONUS if k == 15 else dfl.CARRY_CORRECTION
        assert (r[1].carry_kind, r[1].carry_token) == (want_kind, int(am[k]))


QWEN_CHAT = dict(temperature=0.7, top_k=200, top_p=1.0, min_p=0.05)  # SamplingConfig::qwen_chat, sampling.rs:47-56


def _wide_block(rng, vocab, n, spread=3.0):
    tl = (rng.standard_normal((n, vocab)) * spread).astype(np.float32)
    dl = (tl[: n - 1] + rng.standard_normal((n - 1, vocab)).astype(np.float32) * 0.5).astype(np.float32)
    return tl, dl


@pytest.mark.parametrize("top_k", [0, 64, 65, 200, 5000])
@pytest.mark.parametrize("filters", [dict(top_p=1.0, min_p=0.0), dict(top_p=0.9, min_p=0.0), dict(top_p=1.0, min_p=0.05),
                                     dict(top_p=0.97, min_p=0.02)])
def test_wide_top_k_matches_oracle(ctx, oracle, top_k, filters):
    """top_k = 0 (whole vocabulary, sampling.rs:1198-1214), the kMaxK boundary (64 inline, 65 through the sorted
    arrays), the reference's chat value 200 and top_k = vocabulary, with every filter combination, for the three
    couplings: decisions, tokens, draws and sampler state equal the oracle's."""
    vocab, n = 5000, 6
    rng = np.random.default_rng(1000 + top_k)
    for trial in range(12):
        tl, dl = _wide_block(rng, vocab, n)
        T = 0.7
        for mode in ("deterministic", "sparse", "dense"):
            if mode == "deterministic":
                drafts = [int(np.argmax(tl[r])) if rng.random() < 0.7 else int(rng.integers(vocab)) for r in range(n - 1)]
            else:
                drafts = sample_drafts(dl, T, rng)
            toks = [int(rng.integers(vocab))] + drafts
            skw = dict(temperature=T, top_k=top_k, seed=trial, **filters)
            props = None
            if mode == "sparse":
                props = []
                for r in range(n - 1):
                    top = np.argsort(-dl[r])[:16]
                    if drafts[r] not in top:
                        top[-1] = drafts[r]
                    z = dl[r][top].astype(np.float64) / T
                    props.append((drafts[r], [(int(a), float(b)) for a, b in zip(top, np.exp(z - z.max()))]))
            r = both(ctx, oracle, toks, tl, vocab, props, 100, [], draft=dl if mode == "dense" else None, draft_T=T, **skw)
            assert r[2] == 0
            assert_same(oracle, *r)


def test_wide_top_k_edge_rows(ctx, oracle):
    """NaN, +inf ties, all -inf but one, equal logits (ties go to the lower token id) and a -0.0 / +0.0 pair through
    the sorted path."""
    vocab = 3000
    rng = np.random.default_rng(7)
    base = (rng.standard_normal((2, vocab)) * 2).astype(np.float32)
    cases = []
    a = base.copy(); a[0, 1234] = np.nan; cases.append(a)
    a = base.copy(); a[0, [5, 2500]] = np.inf; cases.append(a)
    a = np.full((2, vocab), -np.inf, np.float32); a[:, 77] = 1.0; cases.append(a)
    a = np.zeros((2, vocab), np.float32); cases.append(a)
    a = base.copy(); a[0, 10] = -0.0; a[0, 11] = 0.0; a[0, 12:40] = 0.0; cases.append(a)
    a = np.full((2, vocab), -np.inf, np.float32); cases.append(a)
    for rows in cases:
        for seed in range(4):
            r = both(ctx, oracle, [1, int(np.nanargmax(np.where(np.isfinite(rows[0]), rows[0], -1e30)))], rows, vocab, None, 10, [],
                     temperature=0.9, top_k=0, top_p=0.95, min_p=0.01, seed=seed)
            assert_same(oracle, *r)


def test_qwen_chat_preset_full_vocabulary(ctx, oracle):
    """The reference's default chat sampler (temperature 0.7, top_k 200, min_p 0.05) at vocabulary 151936, block 16, both
    random streams, coupled to drafts sampled from the vocabulary-wide draft distribution and to deterministic drafts."""
    import torch

    vocab, n, T = 151936, 16, 0.7
    g = torch.Generator(device="cuda")
    for kind in (dfl.RNG_XOSHIRO, dfl.RNG_PHILOX):
        for seed in range(6):
            g.manual_seed(100 + seed)
            tl = torch.randn((n, vocab), device="cuda", generator=g) * 3
            dl = tl[: n - 1] + torch.randn((n - 1, vocab), device="cuda", generator=g) * 0.5
            drafts = torch.multinomial(torch.softmax(dl.double() / T, dim=1), 1, generator=g).flatten().tolist()
            toks = [seed] + drafts
            for dense in (True, False):
                gs = dfl.Sampler(seed=seed, rng_kind=kind, **QWEN_CHAT)
                os_ = oracle.make_sampler(QWEN_CHAT["temperature"], QWEN_CHAT["top_k"], QWEN_CHAT["top_p"], QWEN_CHAT["min_p"], seed, kind)
                if dense:
                    gd = ctx.decide_dflash_accept_prefix(toks, tl, vocab, None, gs, 100, [], draft_logits=dl, draft_temperature=T)
                    rc, od = oracle.decide_accept_prefix_dense(toks, tl.cpu().numpy(), dl.cpu().numpy(), vocab, T, os_, 100, [])
                else:
                    gd = ctx.decide_dflash_accept_prefix(toks, tl, vocab, None, gs, 100, [])
                    rc, od = oracle.decide_accept_prefix(toks, tl.cpu().numpy(), vocab, None, os_, 100, [])
                assert rc == 0 and gd.key() == od.key(), (kind, seed, dense)
                assert gs.state() == oracle.sampler_state(os_)


def test_full_vocabulary_order_top_k_zero(ctx, oracle):
    """top_k = 0 at vocabulary 151936 with top_p: the chain walks all 151936 ordered candidates."""
    import torch

    vocab, n = 151936, 4
    g = torch.Generator(device="cuda")
    g.manual_seed(9)
    tl = torch.randn((n, vocab), device="cuda", generator=g) * 2
    for seed in range(4):
        toks = [3] + [int(t) for t in torch.argmax(tl[: n - 1], dim=1).tolist()]
        gs = dfl.Sampler(1.0, top_k=0, top_p=0.9, seed=seed)
        os_ = oracle.make_sampler(1.0, 0, 0.9, 0.0, seed, 0)
        gd = ctx.decide_dflash_accept_prefix(toks, tl, vocab, None, gs, 100, [])
        rc, od = oracle.decide_accept_prefix(toks, tl.cpu().numpy(), vocab, None, os_, 100, [])
        assert rc == 0 and gd.key() == od.key(), seed
        assert gs.state() == oracle.sampler_state(os_)
