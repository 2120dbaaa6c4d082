"""Pins the CPU oracle against the vectors the reference's own tests hold and
against what the mathematics fixes, before anything else trusts it.

Each test names the reference test it restates (paths relative to the reference
root).  No GPU and no reference checkout are needed.
"""
import ctypes as C
import json
import math
import os

import numpy as np
import pytest

GOLD = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "reference_vectors.json")))


def f(v):
    return float(v) if isinstance(v, str) else v


# ----------------------------------------------------------------------------- RNG


def test_splitmix_xoshiro_unit_golden(oracle):
    """sampling.rs:1817-1864"""
    L = oracle.lib()
    st = C.c_uint64(0)
    got = [L.orc_splitmix64_next(C.byref(st)) for _ in range(4)]
    assert got == [int(v, 16) for v in GOLD["splitmix64_seed0"]["values"]]

    s = (C.c_uint64 * 4)()
    L.orc_xoshiro_seed(int(GOLD["xoshiro256pp"]["seed"], 16), s)
    got = [L.orc_xoshiro_next(s) for _ in range(4)]
    assert got == [int(v, 16) for v in GOLD["xoshiro256pp"]["values"]]

    L.orc_xoshiro_seed(0, s)
    bits = [np.float64(L.orc_unit_f64(L.orc_xoshiro_next(s))).view(np.uint64) for _ in range(4)]
    assert [int(b) for b in bits] == [int(v, 16) for v in GOLD["unit_f64_bits_seed0"]["values"]]


def test_philox_known_answers(oracle):
    L = oracle.lib()
    for case in GOLD["philox4x32_10"]["cases"]:
        ctr = (C.c_uint32 * 4)(*[int(v, 16) for v in case["ctr"]])
        key = (C.c_uint32 * 2)(*[int(v, 16) for v in case["key"]])
        out = (C.c_uint32 * 4)()
        L.orc_philox4x32_10(ctr, key, out)
        assert list(out) == [int(v, 16) for v in case["out"]]


def test_sample_stream_golden(oracle):
    """sampling.rs:1866-1877"""
    g = GOLD["sample_stream"]
    s = oracle.make_sampler(g["temperature"], g["top_k"], g["top_p"], g["min_p"], int(g["seed"], 16))
    toks = []
    for i in range(16):
        rc, tok, _, _ = oracle.sample(s, g["logits"])
        assert rc == 0
        toks.append(tok)
        assert s.draws == i + 1
    assert toks == g["tokens"]


def test_draw_count_reconstructs_stream(oracle):
    """sampling.rs:1880-1901"""
    logits = [1.0, 0.5, 0.0]
    a = oracle.make_sampler(1.0, seed=7)
    for _ in range(17):
        oracle.sample(a, logits)
    b = oracle.make_sampler(1.0, seed=7, draws=int(a.draws))
    for _ in range(32):
        assert oracle.sample(a, logits)[1:3] == oracle.sample(b, logits)[1:3]


# ----------------------------------------------------------------------------- greedy / ordering


def test_greedy_ties_lowest_index(oracle):
    """sampling.rs:1790-1796, 1904-1909"""
    for case in GOLD["greedy_ties"]["cases"]:
        logits = np.array([f(v) for v in case["logits"]], dtype=np.float32)
        rc, tok, _ = oracle.greedy_token(logits)
        assert rc == 0 and tok == case["token"]


def test_greedy_errors(oracle):
    """sampling.rs:1781-1787"""
    assert oracle.greedy_token(np.zeros(0, np.float32))[0] == 1  # EmptyLogits
    rc, _, err = oracle.greedy_token(np.array([0.0, np.nan], np.float32))
    assert rc == 5 and err == 1


def _comparator_order(logits):
    """descending f32 total order, ties ascending token (sampling.rs:1111-1116)"""
    bits = np.asarray(logits, np.float32).view(np.int32).astype(np.int64)
    key = bits ^ ((bits >> 31) & 0x7FFFFFFF)
    return sorted(range(len(logits)), key=lambda i: (-int(key[i]), i))


def test_full_and_partial_order_match_comparator(oracle):
    """sampling.rs:1929-1995, 2051-2110: radix/select order == comparator order on ties,
    signed zeros, infinities, subnormals, constant rows."""
    rng = np.random.default_rng(0x5A17)
    specials = np.array([0.0, -0.0, np.inf, -np.inf, 1.17549435e-38, -1.17549435e-38, 1e-45, -1e-45,
                         3.4028235e38, -3.4028235e38, 1.0, -1.0], dtype=np.float32)
    rows = []
    for n in [1, 2, 3, 17, 257, 2049]:
        rows.append((rng.random(n) * 60 - 30).astype(np.float32))
        rows.append((rng.integers(0, 4, n) - 1.5).astype(np.float32))
        rows.append(specials[rng.integers(0, len(specials), n)])
        rows.append(np.full(n, 2.5, np.float32))
    for row in rows:
        want = _comparator_order(row)
        for top_k in [0, 1, 2, 5, len(row)]:
            s = oracle.make_sampler(1.0, top_k=top_k, seed=1)
            rc, cands, total, _, _ = oracle.diagnose(s, row, 0.0)
            k = len(row) if top_k == 0 or top_k >= len(row) else top_k
            if rc != 0:
                # rows whose best logit is -inf hold no finite-probability candidate
                assert rc == 7
                continue
            got = [t for t, _ in cands]
            exp = want[:k]
            if row[exp[0]] == np.inf:
                exp = [i for i in exp if row[i] == np.inf]
            assert got == exp


def test_filtering_order_and_tie_boundaries(oracle):
    """sampling.rs:1997-2049"""
    s = oracle.make_sampler(2.0, top_k=0, top_p=1.0, min_p=0.5, seed=1)
    for _ in range(32):
        assert oracle.sample(s, [0.0, -1.0])[1] == 0
    s = oracle.make_sampler(2.0, top_p=0.7, seed=1)
    toks = [oracle.sample(s, [0.0, -1.0])[1] for _ in range(64)]
    assert 1 in toks  # top-p observes temperature scaling
    s = oracle.make_sampler(1.0, top_k=2, seed=9)
    for _ in range(64):
        _, tok, idx, _ = oracle.sample(s, [2.0, 2.0, 2.0])
        assert tok in (0, 1) and idx == tok
    s = oracle.make_sampler(1.0, min_p=1.0, seed=4)
    toks = [oracle.sample(s, [3.0, 3.0, 1.0])[1] for _ in range(64)]
    assert 0 in toks and 1 in toks and 2 not in toks


def test_top_k_one_draw_consumption(oracle):
    """sampling.rs:1911-1924"""
    s = oracle.make_sampler(1.0, top_k=1, seed=7)
    for draw in range(1, 33):
        assert oracle.sample(s, [0.0, 3.0, 1.0])[1] == 1
        assert s.draws == draw


def test_chain_matches_independent_numpy_model(oracle):
    """The whole chain against an independent float64 numpy statement of it
    (top-k -> min-p -> temperature -> top-p -> inverse CDF), on random rows."""
    rng = np.random.default_rng(11)
    for trial in range(200):
        n = int(rng.integers(2, 300))
        logits = (rng.standard_normal(n) * 3).astype(np.float32)
        T = np.float32(rng.choice([0.5, 0.7, 1.0, 1.3]))
        top_k = int(rng.choice([0, 1, 5, 20, 64]))
        top_p = np.float32(rng.choice([1.0, 0.95, 0.7, 0.2]))
        min_p = np.float32(rng.choice([0.0, 0.05, 0.5]))
        u = float(rng.random())
        s = oracle.make_sampler(float(T), top_k, float(top_p), float(min_p), seed=trial)
        rc, cands, total, tok, idx = oracle.diagnose(s, logits, u)
        assert rc == 0
        order = _comparator_order(logits)
        if 0 < top_k < n:
            order = order[:top_k]
        l = logits[order].astype(np.float64)
        if min_p > 0:
            keep = l >= l[0] + math.log(float(min_p))
            order = [o for o, k in zip(order, keep) if k]
            l = l[keep]
        sc = l / float(T)
        w = np.exp(sc - sc[0])
        cum = np.cumsum(w)  # sequential in numpy for 1-D float64
        if top_p < 1:
            keep_n = min(len(w), int(np.sum(cum < cum[-1] * float(top_p))) + 1)
            order, w, cum = order[:keep_n], w[:keep_n], cum[:keep_n]
        assert [t for t, _ in cands] == order
        np.testing.assert_allclose([x for _, x in cands], w, rtol=1e-15)
        pick = min(len(w) - 1, int(np.sum(cum <= u * cum[-1])))
        assert tok == order[pick] and idx == pick


# ----------------------------------------------------------------------------- couplings


def test_deterministic_coupling_preserves_serial_stream(oracle):
    """sampling.rs:2836-2865"""
    logits = [3.0, 2.0, 1.0, 0.0]
    kw = dict(temperature=0.7, top_k=4, top_p=0.9, min_p=0.0, seed=0x5EED)
    serial = oracle.make_sampler(**kw)
    expected = oracle.sample(serial, logits)[1]
    for proposal in [expected, (expected + 1) % 4]:
        spec = oracle.make_sampler(**kw)
        rc, acc, corr = oracle.couple_deterministic(spec, logits, proposal)
        assert rc == 0 and acc == (proposal == expected)
        if not acc:
            assert corr == expected
        assert oracle.sampler_state(spec) == oracle.sampler_state(serial)


def test_sparse_maximal_coupling_preserves_target_distribution(oracle):
    """sampling.rs:2888-2937"""
    tp = np.array([0.5, 0.3, 0.15, 0.05], np.float32)
    pp = np.array([0.1, 0.2, 0.3, 0.4], np.float32)
    tl, pl = np.log(tp), np.log(pp)
    target = oracle.make_sampler(1.0, seed=17)
    prop = oracle.make_sampler(1.0, seed=0xDFFA5202)
    counts = np.zeros(4)
    accepted = 0
    trials = 20000
    for _ in range(trials):
        u = oracle.lib().orc_sampler_next_unit(C.byref(prop))
        rc, cands, _, tok, _ = oracle.diagnose(prop, pl, u)
        rc, acc, corr = oracle.couple_sparse(target, tl, tok, cands)
        assert rc == 0
        accepted += acc
        counts[tok if acc else corr] += 1
    assert np.all(np.abs(counts / trials - tp) < 0.015)
    assert abs(accepted / trials - 0.5) < 0.015


def test_sparse_coupling_draw_counts(oracle):
    """sampling.rs:2939-2984"""
    s = oracle.make_sampler(1.0, top_k=1, seed=99)
    rc, acc, _ = oracle.couple_sparse(s, [4.0, 3.0], 0, [(0, 1.0)])
    assert rc == 0 and acc and s.draws == 1
    s = oracle.make_sampler(1.0, top_k=1, seed=99)
    rc, acc, corr = oracle.couple_sparse(s, [4.0, 3.0], 1, [(1, 1.0)])
    assert rc == 0 and not acc and corr == 0 and s.draws == 2


def test_sparse_coupling_rejects_invalid_proposals_without_advancing(oracle):
    """sampling.rs:2986-3050"""
    logits = [1.0, 0.0]
    for tok, pairs, code in [
        (2, [(2, 1.0)], 8),
        (0, [(2, 1.0)], 8),
        (0, [], 7),
        (0, [(0, -1.0)], 9),
        (0, [(0, float("nan"))], 9),
        (0, [(0, 0.0)], 7),
        (0, [(1, 1.0)], 10),
    ]:
        s = oracle.make_sampler(1.0, seed=7)
        before = oracle.sampler_state(s)
        rc, _, _ = oracle.couple_sparse(s, logits, tok, pairs)
        assert rc == code
        assert oracle.sampler_state(s) == before


def test_dense_coupling_reduces_to_sparse_on_small_vocab(oracle):
    """With one tile and <= 4 tokens the fixed-shape sum is the sequential sum, so
    the dense coupling must equal the sparse coupling fed the temperature-only
    proposal distribution (in token order)."""
    rng = np.random.default_rng(5)
    for trial in range(300):
        n = int(rng.integers(2, 5))
        tl = (rng.standard_normal(n) * 3).astype(np.float32)
        dl = (tl + rng.standard_normal(n) * 0.5).astype(np.float32)
        T = 0.7
        tok = int(rng.integers(0, n))
        kw = dict(temperature=T, top_k=3, top_p=0.95, seed=trial)
        a, b = oracle.make_sampler(**kw), oracle.make_sampler(**kw)
        T32 = float(np.float32(T))
        sc = dl.astype(np.float64) / T32
        w = np.exp(sc - sc.max())
        ra = oracle.couple_dense(a, tl, dl, T, tok)
        rb = oracle.couple_sparse(b, tl, tok, [(i, float(w[i])) for i in range(n)])
        assert ra == rb
        assert oracle.sampler_state(a) == oracle.sampler_state(b)


def test_dense_total_is_tree_sum_close_to_fsum(oracle):
    rng = np.random.default_rng(6)
    d = (rng.standard_normal(5000) * 3).astype(np.float32)
    err = C.c_int64(-1)
    P = oracle.lib().orc_dense_proposal_total(d.ctypes.data_as(C.c_void_p), d.size, 0.7, C.byref(err))
    T32 = float(np.float32(0.7))
    sc = d.astype(np.float64) / T32
    want = math.fsum(np.exp(sc - sc.max()))
    assert abs(P - want) / want < 1e-13


# ----------------------------------------------------------------------------- argmax_top2 / top16


def test_argmax_top2_reference_cases(oracle):
    """metal/elementwise.rs:4188-4230"""
    rows = [[1.0, 4.0, 2.0, 3.0, -1.0, -2.0, -3.0, -4.0], [5.0, 1.0, 5.0, 0.0, 5.0, 2.0, 5.0, 3.0], [7.0],
            [2.0, 2.0, 2.0, 2.0], [-8.0, -9.0, -7.0, -9.5], [-0.0, 0.0, -0.0, -1.0]]
    want = [(1, 1.0), (0, 0.0), (0, math.inf), (0, 0.0), (2, 1.0), (0, 0.0)]
    for row, (wi, wg) in zip(rows, want):
        assert oracle.argmax_top2(np.array(row, np.float32)) == (wi, wg)
    for width in [1, 31, 32, 33, 1023, 1025]:
        row = np.full(width, -1.0, np.float32)
        row[width // 2] = 3.0
        row[width - 1] = 3.0
        idx, gap = oracle.argmax_top2(row)
        assert idx == width // 2
        assert gap == (math.inf if width == 1 else 0.0)
    # metal/elementwise.rs:4080-4133: -inf rows, all-NaN rows
    x = np.full(1024, -np.inf, np.float32)
    assert oracle.argmax_top2(x)[0] == 0
    x[42], x[500] = -1e9, -1e10
    assert oracle.argmax_top2(x)[0] == 42
    assert oracle.argmax_top2(np.full(64, np.nan, np.float32))[0] == -1


def test_top16_is_bruteforce_sort(oracle):
    """kernels/dflash2.metal:73-170: (total-order value desc, index asc)"""
    rng = np.random.default_rng(3)
    for n in [1, 5, 16, 17, 1000, 40000]:
        x = (rng.integers(-8, 8, n)).astype(np.float32)  # heavy ties
        ids, vals = oracle.top16(x)
        want = _comparator_order(x)[:16]
        assert list(ids[: len(want)]) == want
        assert np.all(ids[len(want):] == -1)
        np.testing.assert_array_equal(vals[: len(want)], x[want])


# ----------------------------------------------------------------------------- dequant


def _f16_bytes(v):
    return np.array([v], np.float16).view(np.uint8)


def test_q4_k_known_block(oracle):
    """codec.rs:541-577"""
    g = GOLD["q4_k_known_block"]
    scales, mins = g["scales"], g["mins"]
    block = np.zeros(144, np.uint8)
    block[0:2] = _f16_bytes(g["d"])
    block[2:4] = _f16_bytes(g["dmin"])
    for j in range(4):
        block[4 + j] = scales[j] | ((scales[j + 4] >> 4) << 6)
        block[8 + j] = mins[j] | ((mins[j + 4] >> 4) << 6)
        block[12 + j] = (scales[j + 4] & 0x0F) | ((mins[j + 4] & 0x0F) << 4)
    expected = np.zeros(256, np.float32)
    for chunk in range(4):
        for lane in range(32):
            low = (chunk * 3 + lane) & 0x0F
            high = (15 + chunk * 5 - (lane & 0x0F)) & 0x0F
            block[16 + chunk * 32 + lane] = low | (high << 4)
            expected[chunk * 64 + lane] = np.float32(np.float32(0.5 * scales[2 * chunk]) * np.float32(low)) - \
                np.float32(0.25 * mins[2 * chunk])
            expected[chunk * 64 + 32 + lane] = np.float32(np.float32(0.5 * scales[2 * chunk + 1]) * np.float32(high)) \
                - np.float32(0.25 * mins[2 * chunk + 1])
    got = oracle.dequant(oracle.Q4_K, block, 256)
    assert np.array_equal(got.view(np.uint32), expected.view(np.uint32))


def test_q4_k_random_blocks_closed_form(oracle):
    """closed form y = (d*sc_j)*q - (dmin*m_j) with the 6-bit unpack, on random bytes"""
    rng = np.random.default_rng(1)
    nb = 64
    blocks = rng.integers(0, 256, (nb, 144), dtype=np.uint8)
    blocks[:, 0:2] = np.frombuffer(rng.standard_normal(nb).astype(np.float16).tobytes(), np.uint8).reshape(nb, 2)
    blocks[:, 2:4] = np.frombuffer(rng.standard_normal(nb).astype(np.float16).tobytes(), np.uint8).reshape(nb, 2)
    got = oracle.dequant(oracle.Q4_K, blocks, nb * 256).reshape(nb, 256)
    for b in range(nb):
        blk = blocks[b]
        d = np.float32(blk[0:2].view(np.float16)[0])
        dmin = np.float32(blk[2:4].view(np.float16)[0])
        s = blk[4:16].astype(np.int32)
        qs = blk[16:144]
        for j in range(8):
            if j < 4:
                sc, m = s[j] & 63, s[j + 4] & 63
            else:
                sc = (s[j + 4] & 0xF) | ((s[j - 4] >> 6) << 4)
                m = (s[j + 4] >> 4) | ((s[j] >> 6) << 4)
            q = qs[32 * (j // 2): 32 * (j // 2) + 32]
            q = (q >> 4) if j & 1 else (q & 0xF)
            want = np.float32(d * np.float32(sc)) * q.astype(np.float32) - np.float32(dmin * np.float32(m))
            assert np.array_equal(got[b, 32 * j: 32 * j + 32].view(np.uint32), want.astype(np.float32).view(np.uint32))


def _q6_k_block(d, scales, q):
    """metal/tests/q6_k_f32_tile.rs:27-44"""
    block = np.zeros(210, np.uint8)
    for n in range(2):
        for l in range(32):
            q1, q2, q3, q4 = (int(q[128 * n + l + o]) for o in (0, 32, 64, 96))
            block[64 * n + l] = (q1 & 0xF) | ((q3 & 0xF) << 4)
            block[64 * n + l + 32] = (q2 & 0xF) | ((q4 & 0xF) << 4)
            block[128 + 32 * n + l] = (q1 >> 4) | ((q2 >> 4) << 2) | ((q3 >> 4) << 4) | ((q4 >> 4) << 6)
    block[192:208] = np.array(scales, np.int8).view(np.uint8)
    block[208:210] = _f16_bytes(d)
    return block


def test_q6_k_layout_and_closed_form(oracle):
    """metal/tests/q6_k_f32_tile.rs:75-107: signed/extreme scales, every quant incl. 31..33"""
    rng = np.random.default_rng(2)
    for ordinal in range(24):
        d = [1.0 / 64.0, 3.0e-3, 0.25, 7.5e-4][ordinal % 4]
        scales = [[-128, 127, 0, -1][(ordinal + i) % 6] if (ordinal + i) % 6 < 4 else int(rng.integers(-128, 127))
                  for i in range(16)]
        q = [[31, 32, 33][(ordinal * 7 + i) % 9] if (ordinal * 7 + i) % 9 < 3 else int(rng.integers(0, 64))
             for i in range(256)]
        block = _q6_k_block(d, scales, q)
        got = oracle.dequant(oracle.Q6_K, block, 256)
        stored_d = np.float32(np.float16(d))
        want = np.array([np.float32(stored_d * np.float32(scales[i // 16])) * np.float32(q[i] - 32)
                         for i in range(256)], np.float32)
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


def test_q8_0_known_blocks(oracle):
    """codec.rs:474-538"""
    for case in GOLD["q8_0_blocks"]["cases"]:
        block = np.zeros(34, np.uint8)
        block[0:2] = _f16_bytes(case["d"])
        block[2:] = (np.arange(32) - case["offset"]).astype(np.int8).view(np.uint8)
        got = oracle.dequant(oracle.Q8_0, block, 32)
        want = ((np.arange(32, dtype=np.float32) - case["offset"]) * np.float32(case["d"])).astype(np.float32)
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


def test_block_geometry_and_alignment(oracle):
    """tensor.rs:164-208, codec.rs:91-103"""
    assert oracle.row_bytes(oracle.Q4_K, 256) == 144
    assert oracle.row_bytes(oracle.Q6_K, 256) == 210
    assert oracle.row_bytes(oracle.Q8_0, 32) == 34
    with pytest.raises(ValueError):
        oracle.dequant(oracle.Q8_0, np.zeros(34, np.uint8), 16)


def test_f16_conversions_match_numpy(oracle):
    L = oracle.lib()
    h = np.arange(0, 65536, dtype=np.uint16)
    ref = h.view(np.float16).astype(np.float32)
    got = np.array([L.orc_f16_to_f32(int(v)) for v in h[::37]], np.float32)
    ok = ~np.isnan(ref[::37])  # NaN payloads do not survive a float return value
    assert np.array_equal(got.view(np.uint32)[ok], ref[::37].view(np.uint32)[ok])
    assert np.all(np.isnan(got[~ok]))
    rng = np.random.default_rng(0)
    x = np.concatenate([rng.standard_normal(4000).astype(np.float32) * 10.0 ** rng.integers(-9, 6, 4000),
                        np.array([0.0, -0.0, 65504.0, 65520.0, 1e-8, 6e-8, np.inf, -np.inf], np.float32)])
    with np.errstate(over="ignore"):
        want = x.astype(np.float16).view(np.uint16)
    got = np.array([L.orc_f32_to_f16(float(v)) for v in x], np.uint16)
    assert np.array_equal(got, want)


# ----------------------------------------------------------------------------- f32 primitives / attention


def test_primitives_closed_forms(oracle):
    """forward.rs:1373-1397 + textbook forms in float64"""
    L = oracle.lib()
    assert abs(L.orc_silu(1.0) - GOLD["silu_1"]["value"]) < 1e-6
    rng = np.random.default_rng(0)
    x = rng.standard_normal(256).astype(np.float32)
    w = rng.standard_normal(256).astype(np.float32)
    out = np.empty_like(x)
    L.orc_rms_norm(x.ctypes.data, w.ctypes.data, 256, 1e-6, out.ctypes.data)
    want = x.astype(np.float64) / np.sqrt(np.mean(x.astype(np.float64) ** 2) + 1e-6) * w
    np.testing.assert_allclose(out, want, rtol=2e-6)
    sm = np.array([1.0, 2.0, 3.0], np.float32)
    L.orc_softmax_in_place(sm.ctypes.data, 3)
    np.testing.assert_allclose(sm, np.exp([1, 2, 3]) / np.sum(np.exp([1, 2, 3])), rtol=1e-6)
    # NeoX RoPE: pairs (i, i+half), angle = pos / theta^(2i/n_rot); a rotation preserves pair norms
    buf = rng.standard_normal(2 * 128).astype(np.float32)
    ref = buf.copy().astype(np.float64).reshape(2, 128)
    L.orc_rope_in_place(buf.ctypes.data, 2, 128, 128, 1234, 1e6)
    i = np.arange(64)
    ang = 1234.0 / (1e6 ** (2 * i / 128))
    want = np.concatenate([ref[:, :64] * np.cos(ang) - ref[:, 64:] * np.sin(ang),
                           ref[:, :64] * np.sin(ang) + ref[:, 64:] * np.cos(ang)], axis=1)
    np.testing.assert_allclose(buf.reshape(2, 128), want, atol=2e-4)


def test_draft_attention_sentinel(oracle):
    """metal/dflash.rs:1305-1317: strict window, future noise only when non-causal"""
    g = GOLD["dflash_attn_sentinel"]
    vals = np.array(g["v_values"], np.float32)
    n = 8
    q = np.zeros((n, 1, 1), np.float32)
    k_ctx = np.zeros((2, 1, 1), np.float32)
    k_noise = np.zeros((n, 1, 1), np.float32)
    v_ctx = vals[:2].reshape(2, 1, 1)
    v_noise = vals[2:].reshape(n, 1, 1)
    pos_ctx = np.array(g["positions"][:2], np.int32)
    for causal, want in [(True, g["causal"]), (False, g["noncausal"])]:
        out = oracle.attn_draft(q, k_ctx, v_ctx, k_noise, v_noise, pos_ctx, g["q_pos"], causal, g["window"])
        assert out[0, 0, 0] == want


def _attn_f64(q, k, v, ctx_len, scale):
    n_rows, n_q, hd = q.shape
    n_kv = k.shape[1]
    g = n_q // n_kv
    out = np.zeros((n_rows, n_q, hd))
    kd, vd = k.astype(np.float64), v.astype(np.float64)
    for r in range(n_rows):
        npos = ctx_len + r + 1
        for h in range(n_q):
            s = kd[:npos, h // g] @ q[r, h].astype(np.float64) * scale
            p = np.exp(s - s.max())
            out[r, h] = (p / p.sum()) @ vd[:npos, h // g]
    return out


def test_verify_attention_matches_f64_bruteforce(oracle):
    """16 independent causal single-query attentions over [0, L+i] (forward.rs:893-922)"""
    rng = np.random.default_rng(10)
    L, n_rows, n_q, n_kv, hd = 77, 16, 12, 4, 32
    q = rng.standard_normal((n_rows, n_q, hd)).astype(np.float32)
    k = rng.standard_normal((L + n_rows, n_kv, hd)).astype(np.float16)
    v = rng.standard_normal((L + n_rows, n_kv, hd)).astype(np.float16)
    scale = 1.0 / math.sqrt(hd)
    got = oracle.attn_verify_block(q, k, v, L, scale)
    want = _attn_f64(q, k, v, L, scale)
    np.testing.assert_allclose(got, want, atol=2e-5, rtol=1e-4)
    # block-causality: changing K/V of a later block row must not change earlier rows
    k2, v2 = k.copy(), v.copy()
    k2[L + 9:], v2[L + 9:] = 0, 7
    got2 = oracle.attn_verify_block(q, k2, v2, L, scale)
    assert np.array_equal(got[:9], got2[:9]) and not np.array_equal(got[9:], got2[9:])


def test_gemm_fewrow_matches_f64(oracle):
    """metal/mat_mat.rs:4285-4309 tolerances, f64 reference from the dequantised matrix"""
    rng = np.random.default_rng(4)
    for qt, blk_elems, blk_bytes in [(oracle.Q4_K, 256, 144), (oracle.Q6_K, 256, 210), (oracle.Q8_0, 32, 34)]:
        n_in, n_out, n_rows = 512, 24, 5
        nb = n_in // blk_elems * n_out
        w = rng.integers(0, 256, (nb, blk_bytes), dtype=np.uint8)
        dpos = {144: [0, 2], 210: [208], 34: [0]}[blk_bytes]
        for p in dpos:
            w[:, p:p + 2] = np.frombuffer(np.full(nb, 0.01, np.float16).tobytes(), np.uint8).reshape(nb, 2)
        x = rng.standard_normal((n_rows, n_in)).astype(np.float32)
        y = oracle.gemm_fewrow(qt, w, x, n_in, n_out)
        wf = oracle.dequant(qt, w, n_in * n_out).reshape(n_out, n_in).astype(np.float64)
        ref = x.astype(np.float64) @ wf.T
        assert np.max(np.abs(y - ref)) <= 1e-3 * max(1.0, np.max(np.abs(ref)))
