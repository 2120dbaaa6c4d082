"""Pins of the oracle's COMPOSED forwards (orc_target_verify with the dense and the MoE FFN,
orc_dflash_draft) before any device path is compared against them.  CPU only.

The operators are pinned one by one elsewhere; these tests pin the wiring around them (layer order,
where the q/k norms and RoPE sit, which residual feeds what, the tap point, GQA head mapping, the
MoE renormalisation and tie rule, the drafter's context columns and masks) through

  * the one value test the reference holds for the composed drafter
    (crates/qwen-llm/src/loader_dflash_tests.rs:212-241), restated with the same tiny model,
  * special cases that reduce a forward to a closed form computed here in float64 from the
    dequantised weights (single token at position 0, zeroed output projections, identical experts,
    all experts used, tied router rows, truncated models),
  * structural identities (packed rows == single-row steps, a context column == a noise row of a
    one-layer drafter),
  * an independent vectorised float64 model of the whole forward on small random models.

A wiring mistake (a dropped residual, norm after RoPE, a transposed head map, ctx columns run through
the layer norm, tap before the FFN residual ...) moves logits by O(1); float32-vs-float64 summation
moves them by about 1e-6.  Tolerances sit between the two.
"""
import numpy as np
import pytest

F32 = 0  # oracle.F32: unquantised tensor type


def f32t(a):
    """(type, bytes) pair of an unquantised f32 tensor [n_out, n_in] for oracle.build_model."""
    a = np.ascontiguousarray(a, np.float32)
    return (F32, a.view(np.uint8).reshape(a.shape[0], -1))


def rms(x, w, eps=1e-6):
    x = np.asarray(x, np.float64)
    return x / np.sqrt((x * x).mean(-1, keepdims=True) + eps) * np.asarray(w, np.float64)


def rope(v, pos, theta):
    """NeoX rotation of the last axis (pairs i, i + hd/2), angle pos / theta^(2i/hd)."""
    v = np.asarray(v, np.float64)
    hd = v.shape[-1]
    half = hd // 2
    freq = float(pos) / theta ** (2.0 * np.arange(half) / hd)
    c, s = np.cos(freq), np.sin(freq)
    a, b = v[..., :half], v[..., half:]
    return np.concatenate([a * c - b * s, a * s + b * c], -1)


def f16r(a):
    return np.asarray(a, np.float64).astype(np.float32).astype(np.float16).astype(np.float64)


def silu(x):
    return x / (1.0 + np.exp(-x))


def softmax(x):
    e = np.exp(x - x.max())
    return e / e.sum()


def close(got, want, tol, what=""):
    got, want = np.asarray(got, np.float64), np.asarray(want, np.float64)
    scale = max(np.sqrt((want * want).mean()), 1e-30)
    err = np.abs(got - want).max() / scale
    assert err <= tol, f"{what}: max |diff| / rms = {err:.3e} > {tol}"


# ----------------------------------------------------------------------------- f64 models


class NpTarget:
    """Vectorised float64 model of the synthetic decoder (forward.rs:96-163, 725-932 without the q-gate,
    full-width RoPE): weights as float64 matrices [n_out, n_in]."""

    def __init__(self, cfg, mats, theta=1e6):
        self.c, self.m, self.theta = cfg, mats, theta

    def ffn(self, L, p):
        c = self.c
        if not c["n_expert"]:
            return L["down"] @ (silu(L["gate"] @ p) * (L["up"] @ p))
        probs = softmax(L["router"] @ p)
        used = min(c["n_expert_used"], c["n_expert"])
        order = sorted(range(c["n_expert"]), key=lambda e: (-probs[e], e))[:used]
        wsum = max(sum(probs[e] for e in order), 2.0 ** -14)
        fe, h = c["ffn_expert"], c["hidden"]
        out = np.zeros(h)
        for e in order:
            g = L["gate_exps"][e * fe:(e + 1) * fe] @ p
            u = L["up_exps"][e * fe:(e + 1) * fe] @ p
            out += probs[e] / wsum * (L["down_exps"][e * h:(e + 1) * h] @ (silu(g) * u))
        sg = 1.0 / (1.0 + np.exp(-(p @ L["shexp_gate"])))
        return out + sg * (L["down"] @ (silu(L["gate"] @ p) * (L["up"] @ p)))

    def run(self, tokens, taps=()):
        """Tokens at positions 0..n-1 of an empty cache -> (logits [n, V], taps [n, len(taps), H], K cache, V cache)."""
        c, m = self.c, self.m
        nq, nkv, hd, h = c["n_q"], c["n_kv"], c["head_dim"], c["hidden"]
        group = nq // nkv
        kc = [[] for _ in range(c["n_layers"])]
        vc = [[] for _ in range(c["n_layers"])]
        logits, hid = [], []
        for pos, tok in enumerate(tokens):
            x = m["token_embd"][tok].copy()
            caps = {}
            for il, L in enumerate(m["layers"]):
                cur = rms(x, L["attn_norm"])
                q = rope(rms((L["wq"] @ cur).reshape(nq, hd), L["q_norm"]), pos, self.theta)
                k = rope(rms((L["wk"] @ cur).reshape(nkv, hd), L["k_norm"]), pos, self.theta)
                v = (L["wv"] @ cur).reshape(nkv, hd)
                kc[il].append(f16r(k))
                vc[il].append(f16r(v))
                K, V = np.stack(kc[il]), np.stack(vc[il])  # [pos+1, nkv, hd]
                ao = np.zeros((nq, hd))
                for qh in range(nq):
                    w = softmax(K[:, qh // group] @ q[qh] / np.sqrt(hd))
                    ao[qh] = w @ V[:, qh // group]
                x = x + L["wo"] @ ao.reshape(-1)
                x = x + self.ffn(L, rms(x, L["post_norm"]))
                if il in taps:
                    caps[il] = x.copy()
            hid.append([caps[t] for t in taps])
            logits.append(m["output"] @ rms(x, m["output_norm"]))
        return np.array(logits), np.array(hid), kc, vc


def np_draft(c, m, emb, head_w, ids, ctx, pos_ctx, start, theta=1e6):
    """Float64 model of Forward::dflash_draft (forward.rs:380-662)."""
    n, nq, nkv, hd, h = c["block_size"], c["n_q"], c["n_kv"], c["head_dim"], c["hidden"]
    group = nq // nkv
    ctx_len = len(pos_ctx)
    ctx_h = rms(np.asarray(ctx, np.float64) @ m["fc"].T, m["hidden_norm"]) if ctx_len else np.zeros((0, h))
    x = np.stack([emb[t] for t in ids])
    kpos = list(pos_ctx) + [start + i for i in range(n)]
    for L in m["layers"]:
        nn = rms(x, L["attn_norm"])
        q = rms((nn @ L["wq"].T).reshape(n, nq, hd), L["q_norm"])
        q = np.stack([rope(q[i], start + i, theta) for i in range(n)])
        src = np.concatenate([ctx_h, nn])  # context columns are NOT run through the layer's attn_norm
        k = rms((src @ L["wk"].T).reshape(-1, nkv, hd), L["k_norm"])
        k = np.stack([rope(k[j], kpos[j], theta) for j in range(len(kpos))])
        v = (src @ L["wv"].T).reshape(-1, nkv, hd)
        window = c["swa_window"] if L["is_swa"] else 0
        ao = np.zeros((n, nq, hd))
        for i in range(n):
            qp = start + i
            ok = np.array([(not c["causal"] or kp <= qp) and (window == 0 or abs(qp - kp) < window) for kp in kpos])
            for qh in range(nq):
                s = k[ok, qh // group] @ q[i, qh] / np.sqrt(hd)
                ao[i, qh] = softmax(s) @ v[ok, qh // group]
        x = x + ao.reshape(n, -1) @ L["wo"].T
        p = rms(x, L["post_norm"])
        x = x + (silu(p @ L["gate"].T) * (p @ L["up"].T)) @ L["down"].T
    return rms(x, m["output_norm"]) @ head_w.T


# ----------------------------------------------------------------------------- random small models


def dense_cfg(**kw):
    c = dict(n_layers=2, hidden=64, n_q=4, n_kv=2, head_dim=16, ffn=96, vocab=40, n_expert=0, n_expert_used=0,
             ffn_expert=0, ffn_shared=0, eps=1e-6, rope_theta=1e6)
    c.update(kw)
    return c


def random_target(c, seed):
    """f32 weights of a small decoder: (oracle weight dictionary, float64 matrices)."""
    rng = np.random.default_rng(seed)
    h, qd, kvd = c["hidden"], c["n_q"] * c["head_dim"], c["n_kv"] * c["head_dim"]

    def mat(n_out, n_in, std=None):
        return (rng.standard_normal((n_out, n_in)) * (std or n_in ** -0.5)).astype(np.float32)

    def norm(n):
        return (1.0 + 0.2 * rng.standard_normal(n)).astype(np.float32)

    mats = {"token_embd": mat(c["vocab"], h, 1.0), "output": mat(c["vocab"], h), "output_norm": norm(h), "layers": []}
    for _ in range(c["n_layers"]):
        f = c["ffn_shared"] if c["n_expert"] else c["ffn"]
        L = {"attn_norm": norm(h), "q_norm": norm(c["head_dim"]), "k_norm": norm(c["head_dim"]), "post_norm": norm(h),
             "wq": mat(qd, h), "wk": mat(kvd, h), "wv": mat(kvd, h), "wo": mat(h, qd), "gate": mat(f, h), "up": mat(f, h),
             "down": mat(h, f)}
        if c["n_expert"]:
            fe, ne = c["ffn_expert"], c["n_expert"]
            L.update(router=mat(ne, h, 1.0), shexp_gate=(rng.standard_normal(h) * h ** -0.5).astype(np.float32),
                     gate_exps=mat(ne * fe, h), up_exps=mat(ne * fe, h), down_exps=mat(ne * h, fe))
        mats["layers"].append(L)
    return mats


def to_oracle(mats):
    w = {"token_embd": f32t(mats["token_embd"]), "output": f32t(mats["output"]), "output_norm": mats["output_norm"], "layers": []}
    for L in mats["layers"]:
        o = {k: (v if v.ndim == 1 else f32t(v)) for k, v in L.items()}
        w["layers"].append(o)
    return w


def f64(mats):
    out = {k: (np.asarray(v, np.float64) if not isinstance(v, list) else v) for k, v in mats.items()}
    out["layers"] = [{k: np.asarray(v, np.float64) for k, v in L.items()} for L in mats["layers"]]
    return out


def run_oracle(oracle, c, mats, tokens, taps=(), start=0, state=None):
    model, keep = oracle.build_model(c, to_oracle(mats))
    state = state or oracle.TargetState(c, 32)
    logits, hidden = oracle.target_verify(model, state, tokens, start, taps)
    return logits, hidden, state


# ----------------------------------------------------------------------------- target verify


@pytest.mark.parametrize("seed", [0, 1])
def test_target_dense_matches_f64_model(oracle, seed):
    c = dense_cfg(n_layers=3)
    mats = random_target(c, seed)
    tokens = [3, 17, 3, 39, 0, 8]
    taps = (0, 2)
    got, hid, st = run_oracle(oracle, c, mats, tokens, taps)
    want, whid, kc, vc = NpTarget(c, f64(mats)).run(tokens, taps)
    close(got, want, 2e-4, "logits")
    close(hid, whid, 2e-4, "captured hiddens")
    # the cache holds, per layer and position, the normed + rotated K and the plain V, rounded to f16
    for il in range(c["n_layers"]):
        kgot = st.k[il, :len(tokens)].view(np.float16).astype(np.float64)
        vgot = st.v[il, :len(tokens)].view(np.float16).astype(np.float64)
        close(kgot, np.array(kc[il]).reshape(len(tokens), -1), 2e-3, f"K cache layer {il}")
        close(vgot, np.array(vc[il]).reshape(len(tokens), -1), 2e-3, f"V cache layer {il}")
    assert not st.k[:, len(tokens):].any() and not st.v[:, len(tokens):].any()


def test_target_single_token_closed_form(oracle):
    """One token at position 0: RoPE is the identity and the softmax has one term, so attention returns the
    (f16-rounded) V row of each q head's group, whatever q and k are."""
    c = dense_cfg(n_layers=1)
    mats = random_target(c, 5)
    m = f64(mats)
    L = m["layers"][0]
    for tok in (0, 7, 39):
        got, _, _ = run_oracle(oracle, c, mats, [tok])
        x = m["token_embd"][tok]
        v = f16r(L["wv"] @ rms(x, L["attn_norm"])).reshape(c["n_kv"], c["head_dim"])
        ao = np.concatenate([v[qh // (c["n_q"] // c["n_kv"])] for qh in range(c["n_q"])])
        x = x + L["wo"] @ ao
        p = rms(x, L["post_norm"])
        x = x + L["down"] @ (silu(L["gate"] @ p) * (L["up"] @ p))
        close(got[0], m["output"] @ rms(x, m["output_norm"]), 1e-4, f"token {tok}")


def test_target_packed_rows_equal_single_row_steps(oracle):
    c = dense_cfg()
    mats = random_target(c, 2)
    tokens = [5, 1, 30, 30, 12]
    packed, hp, sp = run_oracle(oracle, c, mats, tokens, (1,))
    model, keep = oracle.build_model(c, to_oracle(mats))
    st = oracle.TargetState(c, 32)
    rows, hids = [], []
    for i, t in enumerate(tokens):
        lg, hd = oracle.target_verify(model, st, [t], i, (1,))
        rows.append(lg[0])
        hids.append(hd[0])
    assert np.array_equal(np.array(rows).view(np.uint32), packed.view(np.uint32))
    assert np.array_equal(np.array(hids).view(np.uint32), hp.view(np.uint32))
    assert np.array_equal(st.k, sp.k) and np.array_equal(st.v, sp.v)
    # a block appended after a prefix reads the prefix rows it finds in the cache
    st2 = oracle.TargetState(c, 32)
    oracle.target_verify(model, st2, tokens[:3], 0, (1,))
    tail, _ = oracle.target_verify(model, st2, tokens[3:], 3, (1,))
    assert np.array_equal(tail.view(np.uint32), packed[3:].view(np.uint32))


def test_target_zero_output_projections_leave_the_embedding(oracle):
    """wo = 0 and down = 0 on quantised weights: both residual branches add exact zeros, so the logits are
    head(output_norm(embed(token))) at every position, computed here from the dequantised blocks."""
    import qwen_llm_amd as dfl

    cfg = dfl.ModelConfig(n_layers=2, hidden=256, n_q=4, n_kv=2, head_dim=64, ffn=256, vocab=64)
    w = dfl.synth_target_weights(cfg, seed=3)
    for L in w["layers"]:
        for name in ("wo", "down"):
            L[name] = (L[name][0], np.zeros_like(L[name][1]))
    model, keep = oracle.build_model(cfg.as_dict(), w)
    tokens = [9, 63, 9, 1]
    got, _ = oracle.target_verify(model, oracle.TargetState(cfg.as_dict(), 16), tokens, 0)
    emb = oracle.dequant(w["token_embd"][0], w["token_embd"][1], cfg.vocab * cfg.hidden).reshape(cfg.vocab, -1).astype(np.float64)
    head = oracle.dequant(w["output"][0], w["output"][1], cfg.vocab * cfg.hidden).reshape(cfg.vocab, -1).astype(np.float64)
    for r, t in enumerate(tokens):
        close(got[r], head @ rms(emb[t], w["output_norm"]), 2e-5, f"row {r}")
    assert np.array_equal(got[0], got[2])  # same token, different position and history: nothing may leak in


def test_tap_is_the_residual_after_the_layer(oracle):
    """The hidden captured at layer k is what a model truncated after layer k hands to its output norm."""
    c = dense_cfg(n_layers=3)
    mats = random_target(c, 4)
    tokens = [2, 11, 25]
    _, hid, _ = run_oracle(oracle, c, mats, tokens, (0, 1, 2))
    for k in range(3):
        ck = dict(c, n_layers=k + 1)
        mk = dict(mats, layers=mats["layers"][:k + 1])
        lg, _, _ = run_oracle(oracle, ck, mk, tokens)
        want = rms(hid[:, k], mats["output_norm"]) @ np.asarray(mats["output"], np.float64).T
        close(lg, want, 2e-5, f"tap {k}")


# ----------------------------------------------------------------------------- MoE FFN


def moe_cfg(**kw):
    c = dense_cfg(n_layers=1, ffn=0, n_expert=8, n_expert_used=2, ffn_expert=48, ffn_shared=32)
    c.update(kw)
    return c


def decisive(c, mats, tokens, margin=1e-4):
    """True when no router decision of this run sits on a near-tie (f32 and f64 must then agree on the picks)."""
    model = NpTarget(c, f64(mats))
    ok = [True]
    orig = model.ffn

    def spy(L, p):
        probs = np.sort(softmax(L["router"] @ p))[::-1]
        used = min(c["n_expert_used"], c["n_expert"])
        if used < c["n_expert"] and probs[used - 1] - probs[used] < margin:
            ok[0] = False
        return orig(L, p)

    model.ffn = spy
    model.run(tokens)
    return ok[0]


@pytest.mark.parametrize("used", [1, 2, 8])
def test_target_moe_matches_f64_model(oracle, used):
    c = moe_cfg(n_layers=2, n_expert_used=used)
    mats = random_target(c, 10 + used)
    tokens = [1, 2, 3, 33]
    assert decisive(c, mats, tokens)
    got, hid, _ = run_oracle(oracle, c, mats, tokens, (1,))
    want, whid, _, _ = NpTarget(c, f64(mats)).run(tokens, (1,))
    close(got, want, 2e-4, "logits")
    close(hid, whid, 2e-4, "captured hiddens")


def test_moe_all_experts_used_is_the_softmax_weighted_sum(oracle):
    """n_expert_used = n_expert: the picked probabilities sum to one, the renormalisation is a no-op and the routed
    part is sum_e softmax(router x)_e expert_e(x); written out here without any ranking."""
    c = moe_cfg(n_expert=4, n_expert_used=4)
    mats = random_target(c, 21)
    m = f64(mats)
    L = m["layers"][0]
    got, _, _ = run_oracle(oracle, c, mats, [6])
    x = m["token_embd"][6]
    v = f16r(L["wv"] @ rms(x, L["attn_norm"])).reshape(c["n_kv"], c["head_dim"])
    x = x + L["wo"] @ np.concatenate([v[qh // 2] for qh in range(c["n_q"])])
    p = rms(x, L["post_norm"])
    probs = softmax(L["router"] @ p)
    fe, h = c["ffn_expert"], c["hidden"]
    routed = sum(probs[e] * (L["down_exps"][e * h:(e + 1) * h] @ (silu(L["gate_exps"][e * fe:(e + 1) * fe] @ p) *
                                                                  (L["up_exps"][e * fe:(e + 1) * fe] @ p))) for e in range(4))
    shared = (L["down"] @ (silu(L["gate"] @ p) * (L["up"] @ p))) / (1.0 + np.exp(-(p @ L["shexp_gate"])))
    close(got[0], m["output"] @ rms(x + routed + shared, m["output_norm"]), 1e-4)


def test_moe_identical_experts_reduce_to_one_expert_plus_gated_shared(oracle):
    """All experts equal: the renormalised weights sum to one, so the routed part is that expert's FFN whatever the
    router says (a missing renormalisation would scale it by the picked probability mass, about 2/8 here)."""
    c = moe_cfg()
    mats = random_target(c, 22)
    L = mats["layers"][0]
    fe, h = c["ffn_expert"], c["hidden"]
    for name, rows in (("gate_exps", fe), ("up_exps", fe), ("down_exps", h)):
        L[name] = np.tile(L[name][:rows], (c["n_expert"], 1))
    tokens = [4, 19]
    a, _, _ = run_oracle(oracle, c, mats, tokens)
    other = dict(mats, layers=[dict(L, router=np.random.default_rng(9).standard_normal(L["router"].shape).astype(np.float32))])
    b, _, _ = run_oracle(oracle, c, other, tokens)
    close(a, b, 1e-5, "router independence")
    # the same function written as a dense model whose FFN is [expert ; shared] stacked, the shared half scaled by
    # its sigmoid gate: only possible per token, so check the first token through the closed form instead
    m = f64(mats)
    Lm = m["layers"][0]
    x = m["token_embd"][tokens[0]]
    v = f16r(Lm["wv"] @ rms(x, Lm["attn_norm"])).reshape(c["n_kv"], c["head_dim"])
    x = x + Lm["wo"] @ np.concatenate([v[qh // 2] for qh in range(c["n_q"])])
    p = rms(x, Lm["post_norm"])
    expert = Lm["down_exps"][:h] @ (silu(Lm["gate_exps"][:fe] @ p) * (Lm["up_exps"][:fe] @ p))
    shared = (Lm["down"] @ (silu(Lm["gate"] @ p) * (Lm["up"] @ p))) / (1.0 + np.exp(-(p @ Lm["shexp_gate"])))
    close(a[0], m["output"] @ rms(x + expert + shared, m["output_norm"]), 1e-4, "closed form")


def test_moe_router_ties_go_to_the_lower_expert(oracle):
    """A zero router gives every expert the same probability: the ranking (probability descending, then id
    ascending, forward.rs:769-775) must pick experts 0 .. used-1 with equal weights."""
    c = moe_cfg(n_expert_used=3)
    mats = random_target(c, 23)
    mats["layers"][0]["router"][:] = 0.0
    m = f64(mats)
    L = m["layers"][0]
    got, _, _ = run_oracle(oracle, c, mats, [12])
    x = m["token_embd"][12]
    v = f16r(L["wv"] @ rms(x, L["attn_norm"])).reshape(c["n_kv"], c["head_dim"])
    x = x + L["wo"] @ np.concatenate([v[qh // 2] for qh in range(c["n_q"])])
    p = rms(x, L["post_norm"])
    fe, h = c["ffn_expert"], c["hidden"]

    def logits_for(picks):
        routed = sum((L["down_exps"][e * h:(e + 1) * h] @ (silu(L["gate_exps"][e * fe:(e + 1) * fe] @ p) *
                                                          (L["up_exps"][e * fe:(e + 1) * fe] @ p))) / len(picks) for e in picks)
        shared = (L["down"] @ (silu(L["gate"] @ p) * (L["up"] @ p))) / (1.0 + np.exp(-(p @ L["shexp_gate"])))
        return m["output"] @ rms(x + routed + shared, m["output_norm"])

    close(got[0], logits_for([0, 1, 2]), 1e-4, "lowest ids")
    wrong = logits_for([5, 6, 7])
    assert np.abs(got[0] - wrong).max() > 1e-2 * np.sqrt((wrong * wrong).mean())


# ----------------------------------------------------------------------------- drafter


def draft_cfg(**kw):
    c = dict(n_layers=2, hidden=64, n_q=4, n_kv=2, head_dim=16, ffn=96, block_size=6, n_taps=2, causal=0, swa_window=0,
             eps=1e-6, rope_theta=1e6)
    c.update(kw)
    return c


def random_draft(c, seed, swa_layers=()):
    rng = np.random.default_rng(seed)
    h, qd, kvd = c["hidden"], c["n_q"] * c["head_dim"], c["n_kv"] * c["head_dim"]

    def mat(n_out, n_in):
        return (rng.standard_normal((n_out, n_in)) * n_in ** -0.5).astype(np.float32)

    def norm(n):
        return (1.0 + 0.2 * rng.standard_normal(n)).astype(np.float32)

    m = {"fc": mat(h, c["n_taps"] * h), "hidden_norm": norm(h), "output_norm": norm(h), "layers": []}
    for il in range(c["n_layers"]):
        m["layers"].append({"attn_norm": norm(h), "q_norm": norm(c["head_dim"]), "k_norm": norm(c["head_dim"]),
                            "post_norm": norm(h), "wq": mat(qd, h), "wk": mat(kvd, h), "wv": mat(kvd, h), "wo": mat(h, qd),
                            "gate": mat(c["ffn"], h), "up": mat(c["ffn"], h), "down": mat(h, c["ffn"]),
                            "is_swa": int(il in swa_layers)})
    return m


def draft_to_oracle(m):
    w = {"fc": f32t(m["fc"]), "hidden_norm": m["hidden_norm"], "output_norm": m["output_norm"], "layers": []}
    for L in m["layers"]:
        w["layers"].append({k: (v if isinstance(v, int) or v.ndim == 1 else f32t(v)) for k, v in L.items()})
    return w


def draft_f64(m):
    out = {k: np.asarray(v, np.float64) for k, v in m.items() if k != "layers"}
    out["layers"] = [{k: (v if isinstance(v, int) else np.asarray(v, np.float64)) for k, v in L.items()} for L in m["layers"]]
    return out


def tiny_target(oracle, vocab, hidden, seed):
    """A target that only lends its embedding and output head to the drafter."""
    rng = np.random.default_rng(seed)
    emb = rng.standard_normal((vocab, hidden)).astype(np.float32)
    head = (rng.standard_normal((vocab, hidden)) * hidden ** -0.5).astype(np.float32)
    c = dense_cfg(n_layers=0, hidden=hidden, vocab=vocab)
    model, keep = oracle.build_model(c, {"token_embd": f32t(emb), "output": f32t(head),
                                         "output_norm": np.ones(hidden, np.float32), "layers": []})
    return model, keep, emb.astype(np.float64), head.astype(np.float64)


@pytest.mark.parametrize("causal,window,swa_layers,pos_ctx,start", [
    (0, 0, (), [0, 1, 2, 3, 4], 5),          # full block attention, contiguous context
    (1, 0, (), [0, 1, 2, 3, 4], 5),          # causal drafter
    (0, 4, (1,), [0, 1, 2, 3, 4], 5),        # sliding window on the second layer only
    (1, 3, (0, 1), [2, 3, 7, 9], 11),        # causal + window, context positions with gaps
    (0, 0, (), [], 3),                        # no context columns at all
])
def test_drafter_matches_f64_model(oracle, causal, window, swa_layers, pos_ctx, start):
    c = draft_cfg(causal=causal, swa_window=window)
    m = random_draft(c, 31, swa_layers)
    target, keep, emb, head_w = tiny_target(oracle, 50, c["hidden"], 32)
    ohead, keep2 = oracle.build_draft_head(c, draft_to_oracle(m))
    rng = np.random.default_rng(33)
    ctx = rng.standard_normal((len(pos_ctx), c["n_taps"] * c["hidden"])).astype(np.float32)
    ids = [7, 49, 49, 49, 49, 12]
    got = oracle.dflash_draft(target, ohead, ids, ctx, pos_ctx, start)
    want = np_draft(c, draft_f64(m), emb, head_w, ids, ctx, pos_ctx, start)
    close(got, want, 2e-4)


def test_drafter_visibility_reference_case(oracle):
    """crates/qwen-llm/src/loader_dflash_tests.rs:212-241 with its fixture (:10-190): hidden 32, one head of 32,
    vocabulary 2 with embedding rows e0 / e1 tied to the head, unit norms, v and o the identity, every other matrix
    zero, block 8, window 4, no context, block at position 10.  A changed token at block index 1, 3 or 4 moves the
    first row's logit for token 1 by more than 0.1 iff the drafter is not causal and (the layer is not
    sliding-window or the index is inside the window); otherwise the first row is bit-identical."""
    h = 32
    emb = np.zeros((2, h), np.float32)
    emb[0, 0] = emb[1, 1] = 1.0
    target, keep = oracle.build_model(dense_cfg(n_layers=0, hidden=h, vocab=2),
                                      {"token_embd": f32t(emb), "output": f32t(emb), "output_norm": np.ones(h, np.float32),
                                       "layers": []})
    ones, zero, eye = np.ones(h, np.float32), np.zeros((h, h), np.float32), np.eye(h, dtype=np.float32)
    for causal in (0, 1):
        for swa in (0, 1):
            c = draft_cfg(n_layers=1, hidden=h, n_q=1, n_kv=1, head_dim=h, ffn=h, block_size=8, n_taps=1, causal=causal,
                          swa_window=4)
            w = {"fc": f32t(zero), "hidden_norm": ones, "output_norm": ones,
                 "layers": [{"attn_norm": ones, "q_norm": ones, "k_norm": ones, "post_norm": ones, "wq": f32t(zero),
                             "wk": f32t(zero), "wv": f32t(eye), "wo": f32t(eye), "gate": f32t(zero), "up": f32t(zero),
                             "down": f32t(zero), "is_swa": swa}]}
            head, keep2 = oracle.build_draft_head(c, w)

            def run(ids):
                return oracle.dflash_draft(target, head, ids, np.zeros((0, h), np.float32), [], 10)

            base = run([0] * 8)
            for future in (1, 3, 4):
                ids = [0] * 8
                ids[future] = 1
                changed = run(ids)
                visible = (not causal) and (not swa or future < 4)
                if visible:
                    assert abs(changed[0, 1] - base[0, 1]) > 0.1, (causal, swa, future)
                else:
                    assert np.array_equal(changed[0].view(np.uint32), base[0].view(np.uint32)), (causal, swa, future)


def test_context_column_acts_like_a_noise_row(oracle):
    """One-layer, non-causal drafter whose context projection is the identity and whose hidden_norm equals the layer's
    attn_norm: a context column holding embed(t) at position p then offers the other rows exactly the key and value
    a noise row with token t at p would (k-norm and RoPE at pos_ctx, no norm on V).  So rows 0..n-1 of a block of n
    rows plus that column equal rows 0..n-1 of a block of n+1 rows."""
    n = 5
    c1 = draft_cfg(n_layers=1, block_size=n, n_taps=1)
    m = random_draft(c1, 41)
    m["fc"] = np.eye(c1["hidden"], dtype=np.float32)
    m["hidden_norm"] = m["layers"][0]["attn_norm"].copy()
    target, keep, emb, head_w = tiny_target(oracle, 30, c1["hidden"], 42)
    ids = [3, 29, 29, 29, 29, 17]
    start = 8
    h_small, k1 = oracle.build_draft_head(c1, draft_to_oracle(m))
    h_big, k2 = oracle.build_draft_head(dict(c1, block_size=n + 1), draft_to_oracle(m))
    big = oracle.dflash_draft(target, h_big, ids, np.zeros((0, c1["hidden"]), np.float32), [], start)
    col = emb[ids[n]][None, :].astype(np.float32)
    small = oracle.dflash_draft(target, h_small, ids[:n], col, [start + n], start)
    close(small, big[:n], 1e-5)
    # and the column's position matters: moved elsewhere, the rows change
    moved = oracle.dflash_draft(target, h_small, ids[:n], col, [start + n + 3], start)
    assert np.abs(moved - big[:n]).max() > 1e-3


# ----------------------------------------------------------------------------- dense coupling, distribution


def test_dense_coupling_reproduces_the_target_distribution_across_tiles(oracle):
    """Vocabulary of 2600 tokens (three 1024-token tiles of the proposal's sum): draft tokens drawn from
    q = softmax(draft / T_d), coupled against the filtered target chain; the marginal of the emitted token
    (accepted draft or residual correction) must be the target's own distribution, and the acceptance rate
    sum_i min(p_i, q_i)."""
    V, trials = 2600, 30000
    rng = np.random.default_rng(50)
    target = (rng.standard_normal(V) * 3.0).astype(np.float32)
    draft = (target + rng.standard_normal(V) * 0.7).astype(np.float32)
    td = 0.9
    cfg = dict(temperature=0.8, top_k=12, top_p=0.97, min_p=0.0)
    rc, cands, total, _, _ = oracle.diagnose(oracle.make_sampler(**cfg, seed=0), target)
    assert rc == 0 and 3 <= len(cands) <= 12
    p = {t: w / total for t, w in cands}
    assert len({t // 1024 for t in p}) >= 2  # the target's support really spans tiles
    q = np.exp((draft.astype(np.float64) - float(draft.max())) / np.float64(np.float32(td)))
    q /= q.sum()
    drafts = rng.choice(V, size=trials, p=q)
    s = oracle.make_sampler(**cfg, seed=1234)
    counts, accepted = {}, 0
    for d in drafts:
        rc, acc, corr = oracle.couple_dense(s, target, draft, td, int(d))
        assert rc == 0
        tok = int(d) if acc else corr
        accepted += acc
        counts[tok] = counts.get(tok, 0) + 1
    assert set(counts) <= set(p)
    for t, pt in p.items():
        sigma = np.sqrt(pt * (1 - pt) / trials)
        assert abs(counts.get(t, 0) / trials - pt) <= 4 * sigma + 1e-4, (t, pt, counts.get(t, 0) / trials)
    rate = sum(min(pt, q[t]) for t, pt in p.items())
    assert abs(accepted / trials - rate) <= 4 * np.sqrt(rate * (1 - rate) / trials) + 1e-4
