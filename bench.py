#!/usr/bin/env python3
"""Benchmark of the DFlash verify hot path on one MI355X.

A step is one pass of the few-row Q4_K dequant-GEMM over the three Qwen3.6-27B-shaped
projections of a 16-row verify block (gate/up 5120->17408, down 17408->5120, fused QKV
5120->6144), synthetic inputs resident in HBM.  Prints ONE JSON line.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

METRIC = "accepted tokens/s @ batch1 block16; verify Q4_K GEMM HBM GB/s (% of peak)"
SHAPES = [(5120, 17408), (17408, 5120), (5120, 6144)]  # (n_in, n_out)
HBM_PEAK_GBS = 8000.0
# HBM bytes per launch of the dominant kernel, averaged over the three shapes of a step: FETCH_SIZE + WRITE_SIZE from
# two rocprofv3 --pmc runs of this file, each scaled by what the same counter reads for a plain 256 MiB copy.  A
# counter figure, not measured by this run: read from the line "traffic_bytes_per_launch: N" of the summary below.
TRAFFIC_PROFILE = os.path.join(ROOT, "profiles", "gemm_q4k_tiled_kernel__hbm_traffic.txt")


def measured_traffic():
    try:
        with open(TRAFFIC_PROFILE) as f:
            for line in f:
                if line.startswith("traffic_bytes_per_launch:"):
                    return float(line.split(":", 1)[1])
    except OSError:
        pass
    return None


def cpu_baseline(shapes, weights, xs):
    """The oracle's dequant + f32 GEMM (OpenMP over output rows) on the same weights: a bounded
    sample of the workload (the first `rows` output rows of every shape), scaled to GB/s."""
    import numpy as np

    import oracle

    cores = min(os.cpu_count() or 1, int(os.environ.get("OMP_NUM_THREADS", "16")))
    rows_frac = 0.25
    total_bytes, total_s = 0, 0.0
    for (n_in, n_out), w, x in zip(shapes, weights, xs):
        rows = max(16, int(n_out * rows_frac))
        ws = np.ascontiguousarray(w[:rows])
        xf = x.astype(np.float32)
        oracle.gemm_fewrow(oracle.Q4_K, ws, xf, n_in, rows)  # warm-up
        best = 1e30
        for _ in range(3):
            t0 = time.perf_counter()
            oracle.gemm_fewrow(oracle.Q4_K, ws, xf, n_in, rows)
            best = min(best, time.perf_counter() - t0)
        total_bytes += ws.size
        total_s += best
    return {"value": total_bytes / total_s / 1e9, "unit": "GB/s", "cores": cores, "kind": "port",
            "sample": f"first {int(rows_frac * 100)}% of the output rows of each of the 3 GEMMs, best of 3"}


def attention_section(ctx, with_cpu=True):
    """Block-causal verify attention, 16 query rows after L keys, 48 q / 8 kv heads of 128, f16 K/V resident in HBM
    (V in the transposed cache layout): microseconds per call and KV-stream GB/s = (L + 16) * 8 * 128 * 2 * 2 B / time.
    cpu_baseline: the oracle's per-(row, head) f32 attention (OpenMP) on the same tensors at the shortest context."""
    import math

    import torch

    out = []
    n_rows, n_q, n_kv, hd = 16, 48, 8, 128
    for L in (4096, 32768, 131072):
        cap = (L + n_rows + 31) // 32 * 32
        g = torch.Generator(device="cuda")
        g.manual_seed(10)
        q = torch.randn((n_rows, n_q, hd), device="cuda", generator=g).half()
        k = torch.randn((cap, n_kv, hd), device="cuda", generator=g).half()
        vt = torch.randn((n_kv, hd, cap), device="cuda", generator=g).half()
        o = torch.empty((n_rows, n_q, hd), device="cuda")
        scale = 1.0 / math.sqrt(hd)
        for _ in range(5):
            ctx.attn_verify_block(q, k, vt, L, scale, v_transposed=True, out=o)
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(30):
            ctx.attn_verify_block(q, k, vt, L, scale, v_transposed=True, out=o)
        e1.record()
        torch.cuda.synchronize()
        us = e0.elapsed_time(e1) / 30 * 1e3
        kv_bytes = (L + n_rows) * n_kv * hd * 2 * 2
        out.append({"context": L, "us_per_call": us, "kv_bytes": kv_bytes, "GBps": kv_bytes / (us * 1e-6) / 1e9,
                    "frac_of_hbm_peak": kv_bytes / (us * 1e-6) / 1e9 / HBM_PEAK_GBS})
        if with_cpu and L == 4096:
            import oracle
            qn = q.float().cpu().numpy()
            kn = k[:L + n_rows].float().cpu().numpy()
            vn = vt[:, :, :L + n_rows].permute(2, 0, 1).contiguous().float().cpu().numpy()
            oracle.attn_verify_block(qn, kn, vn, L, scale)
            best = 1e30
            for _ in range(3):
                t0 = time.perf_counter()
                oracle.attn_verify_block(qn, kn, vn, L, scale)
                best = min(best, time.perf_counter() - t0)
            out[-1]["cpu_baseline"] = {"value": kv_bytes / best / 1e9, "unit": "GB/s", "us_per_call": best * 1e6,
                                       "cores": min(os.cpu_count() or 1, int(os.environ.get("OMP_NUM_THREADS", "16"))),
                                       "kind": "port", "sample": "the context-4096 call, best of 3 (f32 K/V on the host)"}
        del q, k, vt, o
    return out


def q6k_section(ctx):
    """Few-row Q6_K GEMM, M=16: the output head of the end-to-end model (2048 -> 151936, 255 MB) and a 5120 -> 5120
    projection (21.5 MB); weights rotate over enough copies to stay out of the memory-side cache.  Microseconds per
    call and weight GB/s, two ways: through dflash_gemm_fewrow on GGUF row order with f32 activations (the streaming
    kernel and its split-K reduction launch), and - what the model-level calls run - through dflash_gemm_fewrow_xf on the
    tiled Q6_K order with the activations already in fragment order (one launch; `tiled_xf_*`)."""
    import torch

    import qwen_llm_amd as dfl

    def timed(fn, n_sets, reps=3):
        for i in range(n_sets):
            fn(i)
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(reps):
            for i in range(n_sets):
                fn(i)
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / (reps * n_sets) * 1e3

    out = []
    g = torch.Generator(device="cuda")
    g.manual_seed(3)
    for n_in, n_out in ((2048, 151936), (5120, 5120)):
        nbytes = n_in * n_out * 210 // 256
        n_sets = min(24, max(2, int(400e6 // nbytes) + 1))
        ws = [dfl.synth.random_blocks_device(dfl.synth.Q6_K, n_out, n_in, 0.02, g, "cuda") for _ in range(n_sets)]
        x = torch.randn((16, n_in), device="cuda", generator=g)
        y = torch.empty((16, n_out), device="cuda")
        tag = ctx.checked_type(dfl.TYPE_Q6_K, ws[0])  # (every set comes from the same generator: one range check speaks for all)
        us = timed(lambda i: ctx.encode_mat_mat_dispatch_dflash_verify(ws[i], tag, x, y, n_in, n_out, 16), n_sets)
        row = {"n_in": n_in, "n_out": n_out, "weight_bytes": nbytes, "us_per_call": us,
               "GBps": nbytes / (us * 1e-6) / 1e9, "frac_of_hbm_peak": nbytes / (us * 1e-6) / 1e9 / HBM_PEAK_GBS,
               "rotating_copies": n_sets}
        kind = ctx.xf_kind(dfl.TYPE_Q6_K_TILED, n_in, n_out)
        if kind != dfl.XF_NONE:
            wts = [ctx.repack_q6k_tiled(w, n_in, n_out) for w in ws]
            del ws
            xf = ctx.pack_xf(x, kind)
            us_t = timed(lambda i: ctx.gemm_fewrow_xf(wts[i], dfl.TYPE_Q6_K_TILED, xf, 16, n_in, n_out, y=y), n_sets)
            row.update({"tiled_xf_us_per_call": us_t, "tiled_xf_GBps": nbytes / (us_t * 1e-6) / 1e9,
                        "tiled_xf_frac_of_hbm_peak": nbytes / (us_t * 1e-6) / 1e9 / HBM_PEAK_GBS})
            del wts
        out.append(row)
    return out


def acceptance_section(ctx, with_cpu=True):
    """Stochastic acceptance of one block: vocabulary 151936, 15 drafts + bonus, target logits N(0,3), draft = target +
    N(0,0.5), T 0.7 / top-p 0.95 / top-k 20, vocabulary-wide draft distribution (temperature 0.7), Philox stream.
    Time per block (device kernels + the host-side decision read-back) and logits bytes / time."""
    import torch

    import qwen_llm_amd as dfl

    vocab, n = 151936, 16
    g = torch.Generator(device="cuda")
    g.manual_seed(4)
    target = torch.randn((n, vocab), device="cuda", generator=g) * 3.0
    draft = target[: n - 1] + 0.5 * torch.randn((n - 1, vocab), device="cuda", generator=g)
    toks = [int(t) for t in torch.argmax(target, dim=1).tolist()]
    verified = [toks[0]] + [int(t) for t in torch.argmax(draft, dim=1).tolist()]
    times, accepted = [], 0
    for trial in range(24):
        samp = dfl.Sampler(temperature=0.7, top_k=20, top_p=0.95, min_p=0.0, seed=trial, rng_kind=dfl.RNG_PHILOX)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        d = ctx.decide_dflash_accept_prefix(verified, target, vocab, None, samp, 1000, [], draft_logits=draft,
                                            draft_temperature=0.7)
        times.append(time.perf_counter() - t0)
        accepted += len(d.accepted_drafts)
    times = sorted(times[4:])
    us = times[len(times) // 2] * 1e6
    logits_bytes = (2 * n - 1) * vocab * 4
    res = {"vocab": vocab, "block": n, "us_per_block": us, "logits_bytes": logits_bytes,
           "GBps": logits_bytes / (us * 1e-6) / 1e9, "mean_accepted": accepted / 24}
    # the same block between two HIP events around its kernels (the library's own timer slot for acceptance): without
    # the launch from an idle GPU and the host's wait for the decision
    ctx.set_kernel_timing(True)
    for trial in range(8):
        samp = dfl.Sampler(temperature=0.7, top_k=20, top_p=0.95, min_p=0.0, seed=100 + trial, rng_kind=dfl.RNG_PHILOX)
        ctx.decide_dflash_accept_prefix(verified, target, vocab, None, samp, 1000, [], draft_logits=draft, draft_temperature=0.7)
    ms, count = ctx.kernel_timing(2)
    ctx.set_kernel_timing(False)
    if count:
        res["us_between_events"] = ms * 1e3 / count
    # the wide path (top_k 0 or above 64: one device-wide sort of the block's rows, then the chain per row) with the
    # reference's chat preset (temperature 0.7, top-k 200, top-p 1.0, min-p 0.05), deterministic drafts
    wide = []
    for trial in range(10):
        samp = dfl.Sampler(temperature=0.7, top_k=200, top_p=1.0, min_p=0.05, seed=trial, rng_kind=dfl.RNG_PHILOX)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        ctx.decide_dflash_accept_prefix(verified, target, vocab, None, samp, 1000, [])
        wide.append(time.perf_counter() - t0)
    wide = sorted(wide[2:])
    res["top_k_200_us_per_block"] = wide[len(wide) // 2] * 1e6
    if with_cpu:
        # the oracle's restatement of decide_dflash_accept_prefix + Sampler (one thread per block, as the reference's
        # host code runs it) on the same logits, same samplers
        import oracle
        tn, dn = target.cpu().numpy(), draft.cpu().numpy()
        cpu_times, cpu_accepted = [], 0
        for trial in range(8):
            so = oracle.make_sampler(temperature=0.7, top_k=20, top_p=0.95, min_p=0.0, seed=trial, rng_kind=oracle.RNG_PHILOX)
            t0 = time.perf_counter()
            rc, d = oracle.decide_accept_prefix_dense(verified, tn, dn, vocab, 0.7, so, 1000, [])
            cpu_times.append(time.perf_counter() - t0)
            cpu_accepted += int(d.n_accepted) if hasattr(d, "n_accepted") else 0
        cpu_times.sort()
        cpu_us = cpu_times[len(cpu_times) // 2] * 1e6
        res["cpu_baseline"] = {"value": logits_bytes / (cpu_us * 1e-6) / 1e9, "unit": "GB/s", "us_per_block": cpu_us, "cores": 1,
                               "kind": "port", "sample": "8 of the 24 blocks, median"}
    return res


def c1_section(ctx, with_cpu=True):
    """The CPU-runnable plumbing case: greedy verify of one 16-token draft block on a 4-layer dense decoder (hidden 1024,
    16 q / 8 kv heads of 128, SwiGLU 3072, vocabulary 32000; Q4_K projections, Q6_K embedding and output head, random
    blocks) after a 512-token prefix; the first 7 drafts are the target's own greedy continuation, so the accepted
    prefix is known.  GPU: verify + greedy accept + rollback per block.  cpu_baseline: the oracle's forward (OpenMP)
    and acceptance on the same weights and tokens, the one verify block timed after an untimed prefill."""
    import numpy as np
    import torch

    import qwen_llm_amd as dfl

    cfg = dfl.ModelConfig(n_layers=4, hidden=1024, n_q=16, n_kv=8, head_dim=128, ffn=3072, vocab=32000)
    weights = dfl.synth_target_weights_blocks(cfg, 0, attn_type=dfl.synth.Q4_K)
    model = dfl.TargetModel(ctx, cfg, weights)
    prompt = np.random.default_rng(0).integers(0, cfg.vocab, 512).tolist()
    sess = dfl.Session(ctx, model, 640, [])
    for s0 in range(0, 512, 16):
        out = sess.encode_packed_verify_layer_major(prompt[s0:s0 + 16], s0, want_hidden=False)
    cont = [out.argmax_host[-1]]
    for i in range(8):
        cont.append(sess.encode_packed_verify_layer_major([cont[-1]], 512 + i, want_hidden=False).argmax_host[0])
    sess.encode_restore_after_partial_accept(512, 8, 0)
    k = 7
    rng = np.random.default_rng(1)
    block = cont[:1 + k] + [int((cont[1 + k] + 1 + rng.integers(0, 100)) % cfg.vocab)] + rng.integers(0, cfg.vocab, 15 - k - 1).tolist()

    def one():
        o = sess.encode_packed_verify_layer_major(block, 512, want_hidden=False)
        acc = 0
        while acc < 15 and block[1 + acc] == o.argmax_host[acc]:
            acc += 1
        sess.encode_restore_after_partial_accept(512, 16, 0)
        return acc, o.argmax_host[acc]

    for _ in range(3):
        acc, bonus = one()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    reps = 20
    for _ in range(reps):
        one()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) / reps * 1e3
    sess.close()
    res = {"config": "4 layers, hidden 1024, 16q/8kv x 128, ffn 3072, vocab 32000, prefix 512, block 16, forced k=7",
           "ms_per_verify_block": ms, "accepted_drafts": acc, "bonus_token": int(bonus),
           "blocks_per_s": 1e3 / ms, "accepted_tokens_per_s": (acc + 1) * 1e3 / ms}
    if with_cpu:
        import oracle
        omodel, _keep = oracle.build_model(cfg.as_dict(), weights)
        ostate = oracle.TargetState(cfg.as_dict(), 640)
        for s0 in range(0, 512, 16):
            oracle.target_verify(omodel, ostate, prompt[s0:s0 + 16], s0, [])
        t0 = time.perf_counter()
        lo, _ = oracle.target_verify(omodel, ostate, block, 512, [])
        am = lo.argmax(axis=1)
        oacc = 0
        while oacc < 15 and block[1 + oacc] == int(am[oacc]):
            oacc += 1
        cpu_ms = (time.perf_counter() - t0) * 1e3
        res["cpu_baseline"] = {"value": 1e3 / cpu_ms, "unit": "blocks/s", "ms_per_verify_block": cpu_ms,
                               "cores": min(os.cpu_count() or 1, int(os.environ.get("OMP_NUM_THREADS", "16"))), "kind": "port",
                               "sample": "the one 16-token verify block after an untimed 512-token prefill, single run",
                               "accepted_drafts": oacc, "bonus_token": int(am[oacc])}
        res["matches_cpu"] = bool(oacc == acc and int(am[oacc]) == int(bonus))
    return res


def acceptance_table(hist):
    """Per-position acceptance of the draft block from the histogram of accepted lengths: position i (1-based) is
    accepted in the steps that accepted at least i drafts.  alpha_pos1 is the first position's rate."""
    steps = max(sum(hist), 1)
    at_least = [sum(hist[i:]) / steps for i in range(1, 16)]
    return {"alpha_pos1": at_least[0], "per_position_acceptance": at_least, "accept_len_hist": list(hist)}


def e2e_speculative(ctx, n_generate, sweep, log, prompt_len=2048, dflash2=True):
    """End-to-end DFlash speculative decode on the 35B-A3B-shaped synthetic MoE target (40 layers, hidden 2048,
    16 q / 2 kv heads of 256, 128 experts top-8 with F_exp 768 plus a shared expert; experts Q4_K, attention Q6_K,
    vocabulary 151936) with a 5-layer drafter fed by 3 tapped layers, batch 1, block 16, prompt 2048, greedy accept.
    Random-init weights: the drafter never agrees with the target by itself, so acceptance is forced: the target's
    own serial greedy continuation replaces the first k drafts of every block, wrong tokens the rest (the drafter
    still runs and is timed).  Margin fallback off (random-init logits are all near ties).  The decoder's prefill
    (timed separately, prefill_with_drafter_tokens_per_s) includes the drafter's pass over the prompt's captured
    columns; the speculative loop is timed from the first draft block."""
    import numpy as np
    import torch

    import qwen_llm_amd as dfl

    cfg = dfl.ModelConfig(n_layers=40, hidden=2048, n_q=16, n_kv=2, head_dim=256, ffn=0, vocab=151936, n_expert=128,
                          n_expert_used=8, ffn_expert=768, ffn_shared=768)
    dcfg = dfl.DraftConfig(n_layers=5, hidden=2048, n_q=16, n_kv=2, head_dim=256, ffn=6144, block_size=16, n_taps=3)
    taps = [1, 19, 38]
    cap = prompt_len + n_generate + 64
    t0 = time.perf_counter()
    target = dfl.TargetModel(ctx, cfg, dfl.synth_target_weights_device(cfg, 0, "cuda"))
    head = dfl.DraftHead(ctx, dcfg, dfl.synth_draft_weights_device(dcfg, 0, "cuda"))
    torch.cuda.synchronize()
    log(f"e2e: weights on device in {time.perf_counter() - t0:.1f} s "
        f"({(target.weight_bytes() + head.weight_bytes()) / 1e9:.2f} GB)")
    prompt = np.random.default_rng(0).integers(0, cfg.vocab - 1, prompt_len).tolist()
    mask = cfg.vocab - 1

    # the target's serial greedy continuation (token by token through the same kernels)
    serial = dfl.Session(ctx, target, cap, taps)
    serial.prepare_prefill()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    # every block but the last without the output head (dflash_prefill_blocks: the rows of up to 32 blocks per pass); the last with it
    body = (prompt_len - 1) // 16 * 16
    serial.prefill_blocks(prompt[:body], 0, want_hidden=False)
    out = serial.encode_packed_verify_layer_major(prompt[body:], body, want_hidden=False)
    prefill_s = time.perf_counter() - t0
    cont = [out.argmax_host[-1]]
    t0 = time.perf_counter()
    while len(cont) < n_generate + 16:
        out = serial.encode_packed_verify_layer_major([cont[-1]], prompt_len + len(cont) - 1, want_hidden=False)
        cont.append(out.argmax_host[0])
    serial_s = time.perf_counter() - t0
    serial.close()
    res = {"prompt": prompt_len, "generated": n_generate, "prefill_tokens_per_s": prompt_len / prefill_s,
           "serial_tokens_per_s": (len(cont) - 1) / serial_s, "weights_GB": (target.weight_bytes() + head.weight_bytes()) / 1e9,
           "sweep": []}
    log(f"e2e: prefill {res['prefill_tokens_per_s']:.0f} tok/s, serial decode {res['serial_tokens_per_s']:.1f} tok/s")
    for k in sweep:
        dec = dfl.SpeculativeDecoder(ctx, target, head, taps, cap, mask)
        dec.session.prepare_prefill()  # the prefill's scratch is set-up, as for the serial session above: not timed
        torch.cuda.synchronize()
        tp = time.perf_counter()
        first = dec.prefill(prompt)  # target prefill with hidden capture + the drafter's pass over the prompt's columns
        torch.cuda.synchronize()
        spec_prefill_s = time.perf_counter() - tp

        def override(tokens, position, k=k):
            done = len(tokens)
            good = cont[done:done + k]
            bad = [(t + 1) % (cfg.vocab - 1) for t in cont[done + k:done + 15]]
            return good + bad

        torch.cuda.synchronize()
        t0 = time.perf_counter()
        tokens, st = dec.generate(first, n_generate, draft_override_fn=override)
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        dec.close()
        agree = sum(int(a == b) for a, b in zip(tokens, cont))
        res["sweep"].append({
            "forced_k": k, "accepted_tokens_per_s": (len(tokens) - 1) / dt, "steps": st["spec_steps"],
            "prefill_with_drafter_tokens_per_s": prompt_len / spec_prefill_s,
            "mean_accept_len": st["accepted_drafts"] / max(st["spec_steps"], 1),
            "mean_emitted_per_step": (len(tokens) - 1) / max(st["spec_steps"], 1),
            "ms_per_step": dt * 1e3 / max(st["spec_steps"], 1),
            "draft_ms": st["draft_ms"] / st["spec_steps"], "verify_ms": st["verify_ms"] / st["spec_steps"],
            "accept_ms": st["accept_ms"] / st["spec_steps"], "append_ms": st["append_ms"] / st["spec_steps"],
            "tokens_equal_serial_greedy": agree, "tokens": len(tokens)})
        res["sweep"][-1].update(acceptance_table(st.get("accept_len_hist", [0] * 16)))
        log(f"e2e: forced k={k}: {res['sweep'][-1]}")

    # The same run with a DFlash-2 drafter of that shape (what current drafters ship: a dynamic two-tap convolution
    # before and after both sublayers of every layer, top-16 of the head's logits and the selector's walk over rank-256
    # Q4_K codebooks in place of the argmax), greedy, forced k = 7.
    if dflash2:
        k = 7
        d2cfg = dfl.DraftConfig(n_layers=5, hidden=2048, n_q=16, n_kv=2, head_dim=256, ffn=6144, block_size=16, n_taps=3,
                                conv_kernel_size=2, conv_group_size=64, selector_rank=256, selector_top_k=16)
        head2 = dfl.DraftHead(ctx, d2cfg, dfl.synth_draft_weights_device(d2cfg, 1, "cuda", vocab=cfg.vocab))
        dec = dfl.SpeculativeDecoder(ctx, target, head2, taps, cap, mask)
        first = dec.prefill(prompt)

        def override2(tokens, position):
            done = len(tokens)
            return cont[done:done + k] + [(t + 1) % (cfg.vocab - 1) for t in cont[done + k:done + 15]]

        torch.cuda.synchronize()
        t0 = time.perf_counter()
        tokens, st = dec.generate(first, n_generate, draft_override_fn=override2)
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        dec.close()
        res["dflash2"] = {
            "drafter": "DFlash-2: 5 layers, conv kernel 2 / group 64, selector rank 256 over Q4_K codebooks, top-16",
            "forced_k": k, "accepted_tokens_per_s": (len(tokens) - 1) / dt, "steps": st["spec_steps"],
            "ms_per_step": dt * 1e3 / max(st["spec_steps"], 1), "draft_ms": st["draft_ms"] / st["spec_steps"],
            "verify_ms": st["verify_ms"] / st["spec_steps"],
            "tokens_equal_serial_greedy": sum(int(a == b) for a, b in zip(tokens, cont)), "tokens": len(tokens)}
        log(f"e2e: DFlash-2 drafter, forced k={k}: {res['dflash2']}")
        del head2
        # ... and at the block size the released DFlash-2 drafters use, 8: all seven drafts of a block accepted
        d8cfg = dfl.DraftConfig(n_layers=5, hidden=2048, n_q=16, n_kv=2, head_dim=256, ffn=6144, block_size=8, n_taps=3,
                                conv_kernel_size=2, conv_group_size=64, selector_rank=256, selector_top_k=16)
        head8 = dfl.DraftHead(ctx, d8cfg, dfl.synth_draft_weights_device(d8cfg, 1, "cuda", vocab=cfg.vocab))
        dec = dfl.SpeculativeDecoder(ctx, target, head8, taps, cap, mask)
        first = dec.prefill(prompt)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        tokens, st = dec.generate(first, n_generate, draft_override_fn=lambda tokens, position: cont[len(tokens):len(tokens) + 7])
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        dec.close()
        res["dflash2_block8"] = {
            "drafter": "the same DFlash-2 drafter with blocks of 8", "forced_k": 7,
            "accepted_tokens_per_s": (len(tokens) - 1) / dt, "steps": st["spec_steps"],
            "mean_accept_len": st["accepted_drafts"] / max(st["spec_steps"], 1),
            "ms_per_step": dt * 1e3 / max(st["spec_steps"], 1), "draft_ms": st["draft_ms"] / st["spec_steps"],
            "verify_ms": st["verify_ms"] / st["spec_steps"],
            "tokens_equal_serial_greedy": sum(int(a == b) for a, b in zip(tokens, cont)), "tokens": len(tokens)}
        log(f"e2e: DFlash-2 drafter, blocks of 8: {res['dflash2_block8']}")
        del head8

    # Stochastic acceptance (sampler coupled to deterministic drafts), forced the same way: the serial sampler's own
    # stream (temperature 0.7, top-k 20, top-p 0.95, one draw per token, through the same kernels) supplies the first
    # k drafts of every block.  Shorter run: the serial stream costs one full decode step per token.
    n_s, k = min(n_generate, 256), 7
    kw = dict(temperature=0.7, top_k=20, top_p=0.95, min_p=0.0, seed=1)
    samp = dfl.Sampler(**kw)
    serial = dfl.Session(ctx, target, cap, taps)
    for s0 in range(0, prompt_len, 16):
        out = serial.encode_packed_verify_layer_major(prompt[s0:s0 + 16], s0, want_hidden=False)
    stream = [out.argmax_host[-1]]
    while len(stream) < n_s + 16:
        out = serial.encode_packed_verify_layer_major([stream[-1]], prompt_len + len(stream) - 1, want_logits=True,
                                                       want_hidden=False)
        stream.append(ctx.decide_dflash_accept_prefix([stream[-1]], out.logits, cfg.vocab, None, samp, 1 << 30, []).carry_token)
    serial.close()
    dec = dfl.SpeculativeDecoder(ctx, target, head, taps, cap, mask, sampler=dfl.Sampler(**kw))
    first = dec.prefill(prompt)

    def override_s(tokens, position):
        done = len(tokens)
        return stream[done:done + k] + [(t + 1) % (cfg.vocab - 1) for t in stream[done + k:done + 15]]

    torch.cuda.synchronize()
    t0 = time.perf_counter()
    tokens, st = dec.generate(first, n_s, draft_override_fn=override_s)
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    dec.close()
    res["sampled"] = {
        "forced_k": k, "sampling": kw, "accepted_tokens_per_s": (len(tokens) - 1) / dt, "steps": st["spec_steps"],
        "mean_accept_len": st["accepted_drafts"] / max(st["spec_steps"], 1), "ms_per_step": dt * 1e3 / max(st["spec_steps"], 1),
        "draft_ms": st["draft_ms"] / st["spec_steps"], "verify_ms": st["verify_ms"] / st["spec_steps"],
        "accept_ms": st["accept_ms"] / st["spec_steps"],
        "tokens_equal_serial_sampler": sum(int(a == b) for a, b in zip(tokens, stream)), "tokens": len(tokens)}
    res["sampled"].update(acceptance_table(st.get("accept_len_hist", [0] * 16)))
    log(f"e2e: sampled, forced k={k}: {res['sampled']}")
    return res


def dense_verify_section(ctx, n_layers=64, context=2048, blocks=40):
    """The 16-token verify step of a 27B-shaped dense Q4_K target as a whole: hidden 5120, 32 q / 8 kv heads of 128
    (fused q|k|v 5120 -> 6144), SwiGLU FFN 17408 (the three matrix shapes of the headline are this layer's), `n_layers`
    layers, output head 5120 -> 151936 in Q6_K; random quant blocks generated on the device.  Reports the time of one
    packed verify of 16 rows at `context` (every layer's GEMMs with their reductions, norms, RoPE, attention, SwiGLU;
    head and argmax included) and the rate at which it streams the model's weights."""
    import numpy as np
    import torch

    import qwen_llm_amd as dfl

    cfg = dfl.ModelConfig(n_layers=n_layers, hidden=5120, n_q=32, n_kv=8, head_dim=128, ffn=17408, vocab=151936)
    target = dfl.TargetModel(ctx, cfg, dfl.synth_target_weights_device(cfg, 3, "cuda", attn_type=dfl.synth.Q4_K))
    sess = dfl.Session(ctx, target, context + 64, [1])
    prompt = np.random.default_rng(2).integers(0, cfg.vocab - 1, context + 16).tolist()
    sess.prefill_blocks(prompt[:context], 0, want_hidden=False)
    torch.cuda.synchronize()
    for _ in range(3):
        sess.encode_packed_verify_layer_major(prompt[context:], context, want_hidden=False)
        sess.encode_restore_after_partial_accept(context, 16, 0)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(blocks):
        sess.encode_packed_verify_layer_major(prompt[context:], context, want_hidden=False)
        sess.encode_restore_after_partial_accept(context, 16, 0)
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) / blocks * 1e3
    sess.close()
    H, F, qkv = cfg.hidden, cfg.ffn, (cfg.n_q + 2 * cfg.n_kv) * cfg.head_dim
    layer_bytes = (3 * H * F + H * qkv + cfg.n_q * cfg.head_dim * H) * 144 // 256
    head_bytes = H * cfg.vocab * 210 // 256
    streamed = n_layers * layer_bytes + head_bytes
    return {"model": f"27B-shaped dense Q4_K target: {n_layers} layers, hidden 5120, 32 q / 8 kv heads of 128, FFN 17408, Q6_K head 151936",
            "context": context, "rows": 16, "ms_per_verify": ms, "weight_bytes_per_verify": streamed,
            "GBps": streamed / (ms * 1e-3) / 1e9, "frac_of_hbm_peak": streamed / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS,
            "us_per_layer": (ms * 1e3) / n_layers, "weights_GB": target.weight_bytes() / 1e9}


def moe_layer_probe(nd, blocks=60):
    """Verify blocks on a 4-layer 35B-A3B-shaped mixture-of-experts target (random quant blocks) whose 16 tokens are
    drawn from `nd` distinct ones: 16 distinct random tokens touch about 80 of the 128 experts per layer, 4 about 30,
    1 exactly 8 (+ the shared expert).  Every block of the run (the 2048-token context included) is drawn that way,
    so under `rocprofv3 --kernel-trace --stats` the per-kernel averages are those of one load: the expert launches
    show up per kernel instance (gate/up: f32 in, f16 out; down: f16 in, f32 out).  Prints wall-clock per block."""
    import numpy as np
    import torch

    import qwen_llm_amd as dfl

    cfg = dfl.ModelConfig(n_layers=4, hidden=2048, n_q=16, n_kv=2, head_dim=256, ffn=0, vocab=32000, n_expert=128,
                          n_expert_used=8, ffn_expert=768, ffn_shared=768)
    ctx = dfl.Context(0, workspace_bytes=256 << 20)
    model = dfl.TargetModel(ctx, cfg, dfl.synth_target_weights_blocks(cfg, 41))
    sess = dfl.Session(ctx, model, 4096, [0, 1])
    rng = np.random.default_rng(5)

    def draw():
        base = rng.integers(0, cfg.vocab, nd)
        return [int(base[i % nd]) for i in range(16)]

    pos = 0
    for _ in range(128):  # a 2048-token context
        sess.encode_packed_verify_layer_major(draw(), pos)
        pos += 16
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(blocks):
        sess.encode_packed_verify_layer_major(draw(), pos)
        sess.encode_restore_after_partial_accept(pos, 16, 0)
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) / blocks * 1e3
    sess.close()
    print(json.dumps({"moe_layer_probe": {"distinct_tokens": nd, "layers": cfg.n_layers, "blocks": 128 + blocks,
                                          "ms_per_block_from_the_host": ms}}))


def rocprof_summary(directory):
    """Text summary of a rocprofv3 CSV output directory: per-kernel durations from *_kernel_trace.csv and
    per-kernel counter averages from *_counter_collection.csv (whichever exist)."""
    import collections
    import csv
    import glob

    def short(name):
        name = name.replace("(anonymous namespace)::", "").replace("void ", "")
        return name.split("(")[0]

    for path in sorted(glob.glob(os.path.join(directory, "**", "*_kernel_trace.csv"), recursive=True)):
        per = collections.defaultdict(list)
        for r in csv.DictReader(open(path)):
            name = short(r["Kernel_Name"])
            per[(name, r["Grid_Size_X"], r["Workgroup_Size_X"])].append(int(r["End_Timestamp"]) - int(r["Start_Timestamp"]))
        print(f"# {os.path.basename(path)}: kernel, grid, workgroup, launches, avg / min / median / max duration (us)")
        for (name, grid, wg), d in sorted(per.items(), key=lambda kv: -sum(kv[1])):
            d.sort()
            print(f"{name[:72]:72s} grid {grid:>8s} wg {wg:>5s} n {len(d):5d}  avg {sum(d) / len(d) / 1e3:8.2f}  "
                  f"min {d[0] / 1e3:8.2f}  med {d[len(d) // 2] / 1e3:8.2f}  max {d[-1] / 1e3:8.2f}")
    for path in sorted(glob.glob(os.path.join(directory, "**", "*_counter_collection.csv"), recursive=True)):
        per = collections.defaultdict(lambda: collections.defaultdict(list))
        for r in csv.DictReader(open(path)):
            name = short(r["Kernel_Name"])
            per[(name, r.get("Grid_Size", r.get("Grid_Size_X", "")))][r["Counter_Name"]].append(float(r["Counter_Value"]))
        print(f"# {os.path.basename(path)}: kernel, grid, dispatches, average counter value per dispatch")
        for (name, grid), ctrs in sorted(per.items()):
            vals = "  ".join(f"{c} {sum(v) / len(v):.1f}" for c, v in sorted(ctrs.items()))
            n = max(len(v) for v in ctrs.values())
            print(f"{name[:72]:72s} grid {grid:>8s} n {n:4d}  {vals}")


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run a plain 256 MiB read + 256 MiB write kernel (an int32 add) a few times, outside the timed "
                         "region: the reference dispatch for scaling FETCH_SIZE / WRITE_SIZE counter readings")
    ap.add_argument("--rocprof-summary", metavar="DIR", help="print a text summary of a rocprofv3 CSV output directory and exit")
    ap.add_argument("--no-e2e", action="store_true", help="skip the end-to-end speculative decode measurement")
    ap.add_argument("--e2e-tokens", type=int, default=1024)
    ap.add_argument("--e2e-prompt", type=int, default=2048, help="prompt length of the end-to-end section (the headline uses 2048)")
    ap.add_argument("--weight-sets", type=int, default=3,
                    help="copies of the three weight matrices the timed loops rotate over; 3 x 118 MB exceeds the 256 MB "
                         "memory-side cache, so weights come from HBM as they do in a real model (1 = cache-resident)")
    ap.add_argument("--gemm-only", action="store_true", help="skip the attention, acceptance and end-to-end sections")
    ap.add_argument("--moe-layer", metavar="N", type=int, help="only run the mixture-of-experts layer probe with blocks of N "
                                                               "distinct tokens (16, 4, 1 ...) and exit; for kernel traces")
    ap.add_argument("--dense-verify", action="store_true", help="only run the 27B-shaped dense verify-step probe and print its result")
    ap.add_argument("--shapes", default="0,1,2", help="which of the three GEMM shapes take part (for per-shape profiles; the "
                                                      "metric is defined on all three)")
    args = ap.parse_args()
    if args.rocprof_summary:
        rocprof_summary(args.rocprof_summary)
        return
    if args.gpus != 1:
        print("bench.py measures one GPU: the DFlash step is batch-1 and this build has no multi-GPU path; "
              "run with --gpus 1", file=sys.stderr)
        sys.exit(2)

    if args.moe_layer:
        moe_layer_probe(max(1, min(16, args.moe_layer)))
        return
    if args.dense_verify:
        import qwen_llm_amd as dfl

        print(json.dumps({"dense_verify_27b": dense_verify_section(dfl.Context(0, workspace_bytes=256 << 20))}))
        return

    import numpy as np
    import torch

    import qwen_llm_amd as dfl

    global SHAPES
    SHAPES = [SHAPES[int(i)] for i in args.shapes.split(",")]
    torch.cuda.set_device(0)
    ctx = dfl.Context(0)
    rng = np.random.default_rng(1)
    weights, xs, wd, xd, yd = [], [], [], [], []
    # The weights are uploaded the way a model's are: Q4_K blocks repacked once into the library's tiled order
    # (a permutation of whole 144-byte blocks; same bytes streamed, bit-identical products).  One copy of each matrix
    # stays in GGUF row order so that the same kernel family can be timed on it beside the headline.
    wrow = []
    for n_in, n_out in SHAPES:
        w = dfl.synth.random_weight(dfl.synth.Q4_K, n_out, n_in, seed=1)
        x = rng.standard_normal((16, n_in)).astype(np.float16)
        weights.append(w)
        xs.append(x)
        w0 = torch.from_numpy(w).cuda()
        wrow.append(w0)
        t0 = ctx.repack_q4k_tiled(w0, n_in, n_out)
        wd.append([t0] + [t0.clone() for _ in range(max(1, args.weight_sets) - 1)])
        xd.append(torch.from_numpy(x).cuda())
        yd.append(torch.empty((16, n_out), dtype=torch.float32, device="cuda"))
    w_bytes = [int(w.size) for w in weights]
    w_type = dfl.TYPE_Q4_K_TILED

    n_sets = len(wd[0])
    turn = [0]

    # the launches go straight through the C ABI with arguments marshalled once: a call then costs the host about a
    # microsecond, well under the kernels' time, so the GPU never waits for Python
    from qwen_llm_amd.binding import _stream_ptr
    gemm_c = ctx._lib.dflash_gemm_fewrow

    def bound_call(w, wt, i):
        n_in, n_out = SHAPES[i]
        a = (ctx._h, wt, w.data_ptr(), xd[i].data_ptr(), dfl.TYPE_F16, yd[i].data_ptr(), n_in, n_out, 16, _stream_ptr())
        return a

    step_args = [[bound_call(wd[i][k], w_type, i) for i in range(len(SHAPES))] for k in range(n_sets)]

    def step():
        k = turn[0] = (turn[0] + 1) % n_sets
        for a in step_args[k]:
            if gemm_c(*a):
                raise RuntimeError(ctx._lib.dflash_last_error(ctx._h).decode())

    if args.calibrate_copy:
        # a plain streaming kernel of known traffic: reads 256 MiB, writes 256 MiB (an int32 add, so that its name
        # differs from the device copies that made the weight sets)
        src = torch.ones(64 << 20, dtype=torch.int32, device="cuda")
        dst = torch.empty_like(src)
        for _ in range(5):
            torch.add(src, 1, out=dst)
        torch.cuda.synchronize()
        del src, dst
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record()
    for _ in range(args.steps):
        step()
    e1.record()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3
    ms_per_step = e0.elapsed_time(e1) / args.steps

    # Dominant kernel alone.  Every timed loop below rotates over enough copies of ITS matrix to exceed the 256 MB
    # memory-side cache by a margin (kernel_footprint bytes: 8 copies of a 50 MB matrix, 23 of the 17.7 MB one), so that
    # every launch streams from HBM, as the whole-step loop above does with its three shapes x weight sets.
    reps = max(20, args.steps // 4)
    kernel_footprint = 400e6

    def copies(base, nbytes):
        n = max(len(base), int(kernel_footprint // nbytes) + 1)
        return list(base) + [base[0].clone() for _ in range(n - len(base))]

    n_per_shape = 8 * max(reps, 3)  # the same number of launches for every shape: a trace's average then weighs them equally

    def kernel_times(sets, wt):
        """Per shape: (the streaming kernel's own duration, the whole call's time), both in microseconds.
        Kernel: the library's timer slot 5, i.e. the start / stop stamps of that one dispatch (what a kernel trace reports
        as its duration; an event pair recorded around a launch would add the dispatch latency, about 2.5 us).  Whole
        call (streaming kernel + split-K reduction): back-to-back calls between two events on the stream they run on."""
        kern, call = [], []
        for i, w in enumerate(sets):
            calls = [bound_call(wk, wt, i) for wk in w]
            for a in calls:
                gemm_c(*a)
            torch.cuda.synchronize()
            ctx.set_kernel_timing(2)  # stamps on the dispatches; the launches still follow each other without a wait
            for k in range(n_per_shape):
                gemm_c(*calls[k % len(calls)])
            ms, count = ctx.kernel_timing(5)
            ctx.set_kernel_timing(0)
            kern.append(ms / max(count, 1) * 1e3)
            k0, k1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            k0.record()
            for k in range(n_per_shape):
                gemm_c(*calls[k % len(calls)])
            k1.record()
            torch.cuda.synchronize()
            call.append(k0.elapsed_time(k1) / n_per_shape * 1e3)
        return kern, call

    big = [copies(wd[i], w_bytes[i]) for i in range(len(SHAPES))]
    tiled_us, call_us = kernel_times(big, w_type)
    # a read-only stream over the same buffers with the same launch shape: the practical ceiling of such a kernel
    probe_out = torch.zeros(1024, dtype=torch.int32, device="cuda")
    probe_us = []
    for i in range(len(SHAPES)):
        ctx.hbm_read_probe(big[i], len(big[i]), probe_out)
        torch.cuda.synchronize()
        p0, p1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        n_probe = 4 * len(big[i])
        p0.record()
        ctx.hbm_read_probe(big[i], n_probe, probe_out)
        p1.record()
        torch.cuda.synchronize()
        probe_us.append(p0.elapsed_time(p1) / n_probe * 1e3)
    n_kernel_sets = [len(b) for b in big]
    del big
    # the same launches on GGUF row order, rotating over as many copies (the same blocks the repack range-checked)
    row_sets = [copies([w], nb_) for w, nb_ in zip(wrow, w_bytes)]
    row_us, _ = kernel_times(row_sets, dfl.TYPE_Q4_K | dfl.TYPE_RANGE_CHECKED)
    del row_sets
    per_shape = [{"n_in": n_in, "n_out": n_out, "weight_bytes": nbytes, "kernel_us": us, "GBps": nbytes / (us * 1e-6) / 1e9,
                  "call_us_with_reduction": cus, "row_order_kernel_us": rus, "read_probe_us": pus, "rotating_copies": nk}
                 for (n_in, n_out), nbytes, us, cus, rus, pus, nk in zip(SHAPES, w_bytes, tiled_us, call_us, row_us, probe_us,
                                                                         n_kernel_sets)]
    k_bytes = sum(p["weight_bytes"] for p in per_shape) / len(per_shape)
    k_us = sum(p["kernel_us"] for p in per_shape) / len(per_shape)
    achieved = k_bytes / (k_us * 1e-6) / 1e9
    ceiling = sum(w_bytes) / (sum(probe_us) * 1e-6) / 1e9

    out = {
        "metric": METRIC,
        "value": sum(w_bytes) / (ms_per_step * 1e-3) / 1e9,
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f16",
        "data": "synthetic",
        "config": {"workload": "few-row Q4_K dequant GEMM, M=16, (K,N) in {(5120,17408),(17408,5120),(5120,6144)}, "
                               "X f16 N(0,1), W Q4_K from N(0,0.02) seed 1 (blocks in the library's tiled order, "
                               "repacked once at upload), f32 accumulation",
                   "shapes_in_this_run": args.shapes,
                   "weight_bytes_per_step": sum(w_bytes), "block": 16, "batch": 1, "weight_sets": n_sets,
                   "weight_footprint_bytes": n_sets * sum(w_bytes)},
        "roofline": {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": achieved / HBM_PEAK_GBS, "traffic": measured_traffic(),
                     "kernel": "gemm_q4k_tiled_kernel", "bytes_per_launch": k_bytes, "us_per_launch": k_us,
                     "read_probe_GBps": ceiling, "frac_of_read_probe": achieved / ceiling,
                     "note": "the streaming kernel's own duration (start / stop stamps of the dispatch, as a kernel trace reports "
                             "it), mean over the three shapes; its split-K reduction is another kernel; every launch streams "
                             "from HBM (each shape rotates over more than 256 MB of copies); the whole call is "
                             "shapes[].call_us_with_reduction, the whole step is `value`",
                     "whole_call_frac": k_bytes / (sum(call_us) / len(call_us) * 1e-6) / 1e9 / HBM_PEAK_GBS},
        "shapes": per_shape,
        "pct_of_hbm_peak": 100.0 * sum(w_bytes) / (ms_per_step * 1e-3) / 1e9 / HBM_PEAK_GBS,
        "accepted_tokens_per_s": None,
        "wall_ms_per_step": wall_ms / args.steps,
    }
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(SHAPES, weights, xs)
    del wd, xd, yd, wrow
    if not args.gemm_only:
        try:
            with_cpu = not args.no_cpu_baseline
            out["gemm_q6k"] = q6k_section(ctx)
            out["attention"] = attention_section(ctx, with_cpu)
            out["acceptance"] = acceptance_section(ctx, with_cpu)
            out["c1_verify"] = c1_section(ctx, with_cpu)
            out["dense_verify_27b"] = dense_verify_section(ctx)
        except Exception as e:  # the GEMM line above stays valid
            out["sections_error"] = f"{type(e).__name__}: {e}"
    if not args.no_e2e and not args.gemm_only:
        try:
            e2e = e2e_speculative(ctx, args.e2e_tokens, [7, 3, 15], lambda m: print(m, file=sys.stderr, flush=True),
                                  prompt_len=args.e2e_prompt)
            out["e2e"] = e2e
            out["accepted_tokens_per_s"] = e2e["sweep"][0]["accepted_tokens_per_s"]
            out["config"]["e2e"] = ("35B-A3B-shaped MoE target (40 layers, 128 experts top-8, Q4_K experts, Q6_K attention, V 151936) "
                                    f"+ 5-layer drafter, prompt {args.e2e_prompt}, greedy accept, forced acceptance k=7 of 15 drafts")
        except Exception as e:  # the GEMM line above stays valid
            out["e2e_error"] = f"{type(e).__name__}: {e}"
    print(json.dumps(out))


if __name__ == "__main__":
    main()
