"""GPU parity at the end-to-end configuration's own widths, at reduced depth: a 35B-A3B-shaped mixture-of-experts
target (hidden 2048, 16 q / 2 kv heads of 256, 128 experts top-8 with F_exp 768 plus a shared expert, Q4_K experts,
Q6_K attention, vocabulary 151936; 2 layers instead of 40) and a 5-layer-shaped drafter (2 layers here) in one
generation loop.  The 128-expert routing kernel, the batched expert GEMMs at their real expert count and the
151936-wide output head are compared with the CPU oracle; the loop is compared with the serial greedy decode.

Weights are random quant blocks (synth.random_blocks_scaled): the quantisers would take minutes at this size, and
both sides consume the same bytes.  Top-8-of-128 routing is discontinuous: the seeds are chosen so that no routing
decision of the compared rows is a near tie (the oracle reports its smallest relative gap; asserted below)."""
import numpy as np
import pytest

import qwen_llm_amd as dfl

pytestmark = pytest.mark.gpu

C5 = dfl.ModelConfig(n_layers=2, hidden=2048, n_q=16, n_kv=2, head_dim=256, ffn=0, vocab=151936, n_expert=128,
                     n_expert_used=8, ffn_expert=768, ffn_shared=768)
D5 = dfl.DraftConfig(n_layers=2, hidden=2048, n_q=16, n_kv=2, head_dim=256, ffn=6144, block_size=16, n_taps=2)
TAPS = [0, 1]


@pytest.fixture(scope="module")
def ctx():
    c = dfl.Context(0, workspace_bytes=256 << 20)
    yield c
    c.close()


@pytest.fixture(scope="module")
def weights():
    return dfl.synth_target_weights_blocks(C5, 41)


def close(got, want, label, tol=3e-2, l2_tol=5e-3):
    got, want = np.asarray(got, np.float32), np.asarray(want, np.float32)
    assert got.shape == want.shape and np.all(np.isfinite(got)), label
    rms = np.sqrt(np.mean(want.astype(np.float64) ** 2))
    err = np.max(np.abs(got - want) / np.maximum(np.abs(want), rms))
    l2 = np.linalg.norm(got.astype(np.float64) - want) / np.linalg.norm(want.astype(np.float64))
    print(f"{label}: max err {err:.3e} l2 {l2:.3e}")
    assert err <= tol and l2 <= l2_tol, f"{label}: max err {err:.3e}, rel l2 {l2:.3e}"


def test_moe_128_experts_verify_matches_oracle(ctx, oracle, weights):
    model = dfl.TargetModel(ctx, C5, weights)
    omodel, _keep = oracle.build_model(C5.as_dict(), weights)
    sess = dfl.Session(ctx, model, 64, TAPS)
    ostate = oracle.TargetState(C5.as_dict(), 64)
    rng = np.random.default_rng(52)
    pos = 0
    oracle.router_margin_take()
    for n in (16, 3):
        blk = rng.integers(0, C5.vocab, n).tolist()
        out = sess.encode_packed_verify_layer_major(blk, pos, want_logits=True)
        lo, hid = oracle.target_verify(omodel, ostate, blk, pos, TAPS)
        margin = oracle.router_margin_take()
        assert margin > 5e-3, f"seed no longer decisive: smallest relative router gap {margin:.2e}"
        close(out.hidden_capture.cpu().numpy(), hid, f"C5-shape hidden n={n}")
        close(out.logits.cpu().numpy(), lo, f"C5-shape logits n={n}")
        top = np.sort(lo, axis=1)
        decided = (top[:, -1] - top[:, -2]) > 2e-2 * lo.std()
        assert np.array_equal(np.asarray(out.argmax_host)[decided], lo.argmax(axis=1)[decided])
        pos += n
    sess.close()


def test_more_slots_than_one_round_of_the_expert_kernel(ctx, oracle):
    """Top-12 routing over 128 experts: a 16-row block then touches about 99 distinct experts (128 (1 - e^-1.5); more
    than 85 with near certainty), i.e. more than 4096 (slot, tile) units for the gate/up launch, so its workgroups
    run two rounds of sixteen units (slab refilled four times, ring streaming across the round boundary), and the
    expert list is longer than one 64-entry window for the down launch.  Compared with the CPU oracle like the top-8
    shape."""
    cfg = dfl.ModelConfig(n_layers=2, hidden=2048, n_q=16, n_kv=2, head_dim=256, ffn=0, vocab=8192, n_expert=128,
                          n_expert_used=12, ffn_expert=768, ffn_shared=768)
    w = dfl.synth_target_weights_blocks(cfg, 43)
    model = dfl.TargetModel(ctx, cfg, w)
    assert model.tiled_tensors > 0
    omodel, _keep = oracle.build_model(cfg.as_dict(), w)
    sess = dfl.Session(ctx, model, 64, TAPS)
    ostate = oracle.TargetState(cfg.as_dict(), 64)
    rng = np.random.default_rng(128)  # (of seeds 100..159 the one whose 384 routing decisions are furthest from a tie)
    oracle.router_margin_take()
    blk = rng.integers(0, cfg.vocab, 16).tolist()
    out = sess.encode_packed_verify_layer_major(blk, 0, want_logits=True)
    lo, hid = oracle.target_verify(omodel, ostate, blk, 0, TAPS)
    margin = oracle.router_margin_take()
    assert margin > 5e-3, f"seed no longer decisive: smallest relative router gap {margin:.2e}"
    close(out.hidden_capture.cpu().numpy(), hid, "top-12 hidden")
    close(out.logits.cpu().numpy(), lo, "top-12 logits")
    sess.close()


def test_tiled_expert_stacks_agree_with_row_order(ctx, weights):
    """The expert stacks and the shared expert of this shape (768 and 2048 rows per expert: multiples of 256) are
    uploaded in the tiled order and run through the expert kernel (one 16-row tile per wave, minima through the
    activations' sub-block sums); the row-order upload of the same bytes runs the streaming kernel's batched mode.
    Same weights, same f16 rounding of the activations, different order of the f32 sums: the two agree far inside the
    tolerance either has against the CPU restatement, for a full block and for ragged ones."""
    tiled = dfl.TargetModel(ctx, C5, weights)
    rows = dfl.TargetModel(ctx, C5, weights, tiled=False)
    assert tiled.tiled_tensors > 0 and rows.tiled_tensors == 0
    rng = np.random.default_rng(3)
    s_t, s_r = dfl.Session(ctx, tiled, 64, TAPS), dfl.Session(ctx, rows, 64, TAPS)
    pos = 0
    for n in (16, 5, 1):
        blk = rng.integers(0, C5.vocab, n).tolist()
        a = s_t.encode_packed_verify_layer_major(blk, pos, want_logits=True)
        b = s_r.encode_packed_verify_layer_major(blk, pos, want_logits=True)
        close(a.hidden_capture.cpu().numpy(), b.hidden_capture.cpu().numpy(), f"tiled vs row order, hidden n={n}", tol=5e-3, l2_tol=1e-3)
        close(a.logits.cpu().numpy(), b.logits.cpu().numpy(), f"tiled vs row order, logits n={n}", tol=5e-3, l2_tol=1e-3)
        pos += n
    s_t.close()
    s_r.close()


def test_expert_kernel_rows_do_not_depend_on_the_rest_of_the_block(ctx, weights):
    """A row verified alone and the same row at the head of a 16-row block (other rows, so other experts, around it)
    give the same result: every (row, expert) product of the expert kernel is one wave's whole-K sum in a fixed order,
    and rows past the block's end are never stored.  (Compared to 1e-4: the attention kernel splits the keys by the
    block's last position, so its f32 sums are not ordered identically in the two calls.)"""
    model = dfl.TargetModel(ctx, C5, weights)
    rng = np.random.default_rng(11)
    blk = rng.integers(0, C5.vocab, 16).tolist()
    s_blk, s_one = dfl.Session(ctx, model, 64, TAPS), dfl.Session(ctx, model, 64, TAPS)
    a = s_blk.encode_packed_verify_layer_major(blk, 0, want_logits=True)
    hid, lo = a.hidden_capture.cpu().numpy(), a.logits.cpu().numpy()
    b = s_one.encode_packed_verify_layer_major(blk[:1], 0, want_logits=True)
    close(b.hidden_capture.cpu().numpy()[:1], hid[:1], "row alone vs in a block, hidden", tol=1e-4, l2_tol=1e-5)
    close(b.logits.cpu().numpy()[:1], lo[:1], "row alone vs in a block, logits", tol=1e-4, l2_tol=1e-5)
    assert b.argmax_host[0] == a.argmax_host[0]
    s_blk.close()
    s_one.close()


def test_pipelined_prefill_on_the_moe_shape_equals_block_by_block(ctx, weights):
    """Four blocks in flight through the mixture-of-experts layers (each lane routes and runs its experts in its own
    scratch and context): captured rows and the following block's logits equal block-by-block execution bit for bit."""
    model = dfl.TargetModel(ctx, C5, weights)
    rng = np.random.default_rng(21)
    toks = rng.integers(0, C5.vocab, 16 * 6 + 3).tolist()
    probe = rng.integers(0, C5.vocab, 16).tolist()
    ref, pipe = dfl.Session(ctx, model, 256, TAPS), dfl.Session(ctx, model, 256, TAPS)
    got = pipe.prefill_blocks(toks, 0)
    want = []
    for s0 in range(0, len(toks), 16):
        want.append(ref.encode_packed_verify_layer_major(toks[s0:s0 + 16], s0, want_head=False).hidden_capture.cpu().numpy())
    assert np.array_equal(got.cpu().numpy(), np.concatenate(want, axis=0))
    a = ref.encode_packed_verify_layer_major(probe, len(toks), want_logits=True)
    b = pipe.encode_packed_verify_layer_major(probe, len(toks), want_logits=True)
    assert np.array_equal(a.logits.cpu().numpy(), b.logits.cpu().numpy())
    ref.close()
    pipe.close()


@pytest.mark.parametrize("n_head,n_toks", [(5, 512 + 16 * 2 + 5), (0, 17), (250, 16 * 3), (9, 512)])
def test_grouped_prefill_over_several_groups_equals_block_by_block(ctx, weights, n_head, n_toks):
    """A prompt longer than one group of the grouped prefill (512 rows a pass: every projection once for all of them, the
    experts regrouped by expert) with a ragged tail, started at a position that is not a multiple of 16; one block and
    a row; blocks on both sides of a boundary between attention's context-length buckets; exactly one full pass: captured
    rows, and the logits of a block that follows (which read every K/V row written), equal block-by-block execution bit
    for bit."""
    model = dfl.TargetModel(ctx, C5, weights)
    rng = np.random.default_rng(23)
    head = rng.integers(0, C5.vocab, n_head).tolist()
    toks = rng.integers(0, C5.vocab, n_toks).tolist()
    probe = rng.integers(0, C5.vocab, 16).tolist()
    ref, pipe = dfl.Session(ctx, model, 1024, TAPS), dfl.Session(ctx, model, 1024, TAPS)
    for s in (ref, pipe):
        for h0 in range(0, len(head), 16):
            s.encode_packed_verify_layer_major(head[h0:h0 + 16], h0, want_head=False)
    got = pipe.prefill_blocks(toks, len(head))
    want = []
    for s0 in range(0, len(toks), 16):
        want.append(ref.encode_packed_verify_layer_major(toks[s0:s0 + 16], len(head) + s0, want_head=False).hidden_capture.cpu().numpy())
    want = np.concatenate(want, axis=0)
    got = got.cpu().numpy()
    bad = np.flatnonzero(np.any(got.reshape(len(toks), -1) != want.reshape(len(toks), -1), axis=1))
    assert bad.size == 0, f"rows that differ: {bad[:16].tolist()} of {len(toks)}"
    a = ref.encode_packed_verify_layer_major(probe, len(head) + len(toks), want_logits=True)
    b = pipe.encode_packed_verify_layer_major(probe, len(head) + len(toks), want_logits=True)
    assert np.array_equal(a.logits.cpu().numpy(), b.logits.cpu().numpy())
    ref.close()
    pipe.close()


_ROUTE_PROBE = r"""
import sys
import numpy as np
import qwen_llm_amd as dfl
cfg = dfl.ModelConfig(n_layers=2, hidden=2048, n_q=16, n_kv=2, head_dim=256, ffn=0, vocab=8192, n_expert=128,
                      n_expert_used=8, ffn_expert=768, ffn_shared=768)
ctx = dfl.Context(0, workspace_bytes=64 << 20)
model = dfl.TargetModel(ctx, cfg, dfl.synth_target_weights_blocks(cfg, 47))
sess = dfl.Session(ctx, model, 64, [0, 1])
rng = np.random.default_rng(9)
outs = []
pos = 0
for n in (16, 4, 1):
    out = sess.encode_packed_verify_layer_major(rng.integers(0, cfg.vocab, n).tolist(), pos, want_logits=True)
    outs.append(np.concatenate([out.logits.cpu().numpy(), out.hidden_capture.cpu().numpy().reshape(n, -1)], axis=1))
    pos += n
np.save(sys.argv[1], np.concatenate(outs, axis=0))
"""


def _probe_under(tmp_path, knob):
    """Logits and captured rows of three blocks (16, 4 and 1 rows) with the environment switch `knob` at 1 and at 0.  The
    switches are read once per process, so each setting runs in a process of its own (two short-lived ones, one after
    the other)."""
    import os
    import subprocess
    import sys

    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    got = {}
    for flag in ("1", "0"):
        path = str(tmp_path / f"out_{flag}.npy")
        env = dict(os.environ, PYTHONPATH=root + os.pathsep + os.environ.get("PYTHONPATH", ""))
        env[knob] = flag
        r = subprocess.run([sys.executable, "-c", _ROUTE_PROBE, path], env=env, cwd=root, capture_output=True, text=True, timeout=240)
        assert r.returncode == 0, r.stderr[-2000:]
        got[flag] = np.load(path)
    assert got["1"].shape == got["0"].shape == (21, 8192 + 2 * 2048)
    assert np.all(np.isfinite(got["1"]))
    return got["1"], got["0"]


def test_routing_inside_the_expert_launch_equals_the_routing_kernel(tmp_path):
    """The expert list, the weights and the slots come out of the same row arithmetic (moe_route.h) whether the
    gate/up launch derives them in its prologue or moe_route_small_kernel does in a launch of its own: logits and
    captured rows are equal bit for bit."""
    on, off = _probe_under(tmp_path, "DFLASH_MOE_FUSED_ROUTE")
    assert np.array_equal(on, off)


def test_norm_inside_the_router_launch_equals_the_norm_kernel(tmp_path):
    """Residual add, RMSNorm and shared-expert gate computed by every workgroup of the router's launch (the residual
    term added to x later, with the experts' sum) against rms_norm_kernel followed by the Q8_0 product: the sums are
    taken in the same order, so logits and captured rows are equal bit for bit."""
    on, off = _probe_under(tmp_path, "DFLASH_MOE_FUSED_NORM")
    assert np.array_equal(on, off)


_LANES_PROBE = r"""
import sys
import numpy as np
import qwen_llm_amd as dfl
cfg = dfl.ModelConfig(n_layers=2, hidden=2048, n_q=16, n_kv=2, head_dim=256, ffn=0, vocab=8192, n_expert=128,
                      n_expert_used=8, ffn_expert=768, ffn_shared=768)
ctx = dfl.Context(0, workspace_bytes=64 << 20)
model = dfl.TargetModel(ctx, cfg, dfl.synth_target_weights_blocks(cfg, 47))
rng = np.random.default_rng(13)
toks = rng.integers(0, cfg.vocab, 16 * 6 + 3).tolist()
probe = rng.integers(0, cfg.vocab, 16).tolist()
sess = dfl.Session(ctx, model, 256, [0, 1])
hid = sess.prefill_blocks(toks, 0).cpu().numpy().reshape(len(toks), -1)
out = sess.encode_packed_verify_layer_major(probe, len(toks), want_logits=True)
np.save(sys.argv[1], np.concatenate([hid.reshape(-1), out.logits.cpu().numpy().reshape(-1)]))
"""


def test_prefill_with_blocks_in_flight_on_lanes_equals_grouped_prefill(tmp_path):
    """The two prefill schedules of a mixture-of-experts target - rows of many blocks per pass (the default) and, with
    DFLASH_PREFILL_GROUP=0, four blocks in flight on lane streams, each routing and running its experts in its own
    scratch - leave the same captured rows and the same logits for a block that follows, bit for bit.  (The switch is
    read once per process: each setting runs in a short-lived process of its own, one after the other.)"""
    import os
    import subprocess
    import sys

    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    got = {}
    for flag in ("32", "0"):
        path = str(tmp_path / f"prefill_{flag}.npy")
        env = dict(os.environ, PYTHONPATH=root + os.pathsep + os.environ.get("PYTHONPATH", ""), DFLASH_PREFILL_GROUP=flag)
        r = subprocess.run([sys.executable, "-c", _LANES_PROBE, path], env=env, cwd=root, capture_output=True, text=True, timeout=240)
        assert r.returncode == 0, r.stderr[-2000:]
        got[flag] = np.load(path)
    assert got["32"].shape == got["0"].shape and np.all(np.isfinite(got["32"]))
    assert np.array_equal(got["32"], got["0"])


def test_generate_on_the_moe_shape_equals_serial_greedy(ctx, weights):
    """MoE target + drafter in one loop at the end-to-end widths: every emitted token is the target's serial greedy
    decode through the same kernels, through full accepts, partial accepts and rollbacks."""
    model = dfl.TargetModel(ctx, C5, weights)
    rng = np.random.default_rng(7)

    def mat(n_out, n_in):
        return (dfl.synth.Q4_K, dfl.synth.random_blocks_scaled(dfl.synth.Q4_K, n_out, n_in, n_in ** -0.5, rng))

    def norm(n):
        return (1.0 + 0.1 * rng.standard_normal(n)).astype(np.float32)

    H, qd, kvd = D5.hidden, D5.n_q * D5.head_dim, D5.n_kv * D5.head_dim
    dw = {"fc": mat(H, D5.n_taps * H), "hidden_norm": norm(H), "output_norm": norm(H), "layers": []}
    for _ in range(D5.n_layers):
        dw["layers"].append({"attn_norm": norm(H), "q_norm": norm(D5.head_dim), "k_norm": norm(D5.head_dim), "post_norm": norm(H),
                             "wq": mat(qd, H), "wk": mat(kvd, H), "wv": mat(kvd, H), "wo": mat(H, qd), "gate": mat(D5.ffn, H),
                             "up": mat(D5.ffn, H), "down": mat(H, D5.ffn), "is_swa": 0})
    head = dfl.DraftHead(ctx, D5, dw)
    prompt = rng.integers(0, C5.vocab - 1, 37).tolist()
    n_tok = 30
    serial = dfl.Session(ctx, model, 128, TAPS)
    out = None
    for s in range(0, len(prompt), 16):
        out = serial.encode_packed_verify_layer_major(prompt[s:s + 16], s)
    want = [out.argmax_host[-1]]
    while len(want) < n_tok + 16:
        want.append(serial.encode_packed_verify_layer_major([want[-1]], len(prompt) + len(want) - 1).argmax_host[0])
    serial.close()
    dec = dfl.SpeculativeDecoder(ctx, model, head, TAPS, 128, C5.vocab - 1)
    first = dec.prefill(prompt)
    assert first == want[0]

    def override(tokens, position):
        done = len(tokens)
        k = (0, 15, 3, 7)[(position // 2) % 4]
        return want[done:done + k] + [-1] * (15 - k)

    tokens, stats = dec.generate(first, n_tok, draft_override_fn=override)
    assert tokens == want[:n_tok], f"diverged at {next(i for i, (a, b) in enumerate(zip(tokens, want)) if a != b)}"
    assert stats["accepted_drafts"] > 0 and stats["spec_steps"] >= 2
    assert dec.session.kv_n_pos == len(prompt) + n_tok - 1
    dec.close()


def test_full_depth_generation_equals_serial_greedy(ctx):
    """The end-to-end configuration at its own size: all 40 layers (15 GB of Q4_K / Q6_K weights generated on the
    device), the 5-layer drafter fed by three tapped layers, a prompt of 2048 seeded tokens through the pipelined
    prefill, then 256 tokens by speculative steps with greedy acceptance.  Random-init models never agree, so the
    number of accepted drafts is forced block by block on the schedule 7, 3, 15, 0, 1 (the target's own serial
    continuation supplies the first k drafts, wrong tokens the rest; the drafter runs all the same).  Property, which
    does not depend on the size: every emitted token equals the serial greedy decode through the same kernels, the
    accept lengths are the forced ones."""
    import torch

    cfg = dfl.ModelConfig(n_layers=40, hidden=2048, n_q=16, n_kv=2, head_dim=256, ffn=0, vocab=151936, n_expert=128,
                          n_expert_used=8, ffn_expert=768, ffn_shared=768)
    dcfg = dfl.DraftConfig(n_layers=5, hidden=2048, n_q=16, n_kv=2, head_dim=256, ffn=6144, block_size=16, n_taps=3)
    taps, prompt_len, n_generate = [1, 19, 38], 2048, 256
    cap = prompt_len + n_generate + 64
    target = dfl.TargetModel(ctx, cfg, dfl.synth_target_weights_device(cfg, 0, "cuda"))
    head = dfl.DraftHead(ctx, dcfg, dfl.synth_draft_weights_device(dcfg, 0, "cuda"))
    prompt = np.random.default_rng(0).integers(0, cfg.vocab - 1, prompt_len).tolist()
    serial = dfl.Session(ctx, target, cap, taps)
    body = (prompt_len - 1) // 16 * 16
    serial.prefill_blocks(prompt[:body], 0, want_hidden=False)
    out = serial.encode_packed_verify_layer_major(prompt[body:], body, want_hidden=False)
    cont = [out.argmax_host[-1]]
    while len(cont) < n_generate + 16:
        out = serial.encode_packed_verify_layer_major([cont[-1]], prompt_len + len(cont) - 1, want_hidden=False)
        cont.append(out.argmax_host[0])
    serial.close()

    schedule, forced = [7, 3, 15, 0, 1], []
    dec = dfl.SpeculativeDecoder(ctx, target, head, taps, cap, cfg.vocab - 1)
    first = dec.prefill(prompt)
    assert first == cont[0]

    def override(tokens, position):
        k = schedule[len(forced) % len(schedule)]
        forced.append(k)
        done = len(tokens)
        return cont[done:done + k] + [(t + 1) % (cfg.vocab - 1) for t in cont[done + k:done + 15]]

    tokens, st = dec.generate(first, n_generate, draft_override_fn=override)
    torch.cuda.synchronize()
    assert n_generate - 16 <= len(tokens) <= n_generate + 16 and tokens == cont[:len(tokens)]
    # a block accepts exactly its forced drafts (a wrong draft is the target's token + 1, never the target's token),
    # except the last one, which the token budget may cut short
    hist = st["accept_len_hist"]
    want = [0] * 16
    for k in forced[:-1]:
        want[k] += 1
    assert all(h >= w for h, w in zip(hist, want)) and sum(hist) == len(forced)
    dec.close()
