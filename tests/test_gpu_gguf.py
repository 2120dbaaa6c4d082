"""GPU: models bound from GGUF files run the hot path exactly like models built from the same weights in memory, and
the few-row GEMM takes the unquantised (F32 / F16) matrices real files carry (routers, small projections)."""
import numpy as np
import pytest

import qwen_llm_amd as dfl
from qwen_llm_amd import gguf as G

pytestmark = pytest.mark.gpu

TAPS = [0, 1, 1]


@pytest.fixture(scope="module")
def ctx():
    c = dfl.Context(0, workspace_bytes=256 << 20)
    yield c
    c.close()


def dev(a):
    import torch

    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


@pytest.mark.parametrize("wtype,n_in,n_out,n_rows,x_dtype", [
    (G.F32, 2048, 128, 16, np.float32), (G.F32, 256, 40, 3, np.float16), (G.F16, 1024, 256, 16, np.float32),
    (G.F16, 96, 17, 1, np.float16), (G.F32, 32, 16, 16, np.float32)])
def test_gemm_fewrow_plain_matrices(ctx, oracle, wtype, n_in, n_out, n_rows, x_dtype):
    """Y = X . W^T for an F32 / F16 weight matrix, against the CPU oracle's dequantise-and-dot (<= 1e-2 relative to
    max(|ref|, rms); f16 operands, f32 accumulation) and, for the plain case, against numpy's own matmul."""
    rng = np.random.default_rng(n_in + n_out)
    w = (rng.standard_normal((n_out, n_in)) / np.sqrt(n_in)).astype(np.float32 if wtype == G.F32 else np.float16)
    x = rng.standard_normal((n_rows, n_in)).astype(x_dtype)
    y = ctx.gemm_fewrow(dev(w.view(np.uint8)), wtype, dev(x), n_in, n_out).cpu().numpy()
    ref = oracle.gemm_fewrow(wtype, w.view(np.uint8), x.astype(np.float32), n_in, n_out)
    np.testing.assert_allclose(ref, x.astype(np.float64) @ w.astype(np.float64).T, rtol=0, atol=1e-4)
    tol = 1e-2 * np.maximum(np.abs(ref), np.sqrt(np.mean(ref ** 2)))
    assert np.all(np.abs(y - ref) <= tol), float(np.max(np.abs(y - ref) / tol))
    import torch

    with pytest.raises(dfl.DFlashError) as e:  # rows of 8-element steps: n_in must be a multiple of 32
        ctx.gemm_fewrow(dev(w.view(np.uint8)), wtype, torch.zeros((1, 48), device="cuda"), 48, 4)
    assert e.value.kind == "BadShape"


def test_dense_target_and_drafter_from_files_equal_the_in_memory_models(ctx, tmp_path):
    cfg = dfl.ModelConfig(n_layers=2, hidden=256, n_q=4, n_kv=2, head_dim=64, ffn=512, vocab=2048)
    dcfg = dfl.DraftConfig(n_layers=2, hidden=256, n_q=4, n_kv=2, head_dim=64, ffn=512, block_size=16, n_taps=3, swa_window=32)
    w = dfl.synth_target_weights(cfg, seed=21)
    dw = dfl.synth_draft_weights(dcfg, seed=22, swa_layers=[1])
    dfl.write_gguf(tmp_path / "t.gguf", G.target_metadata(cfg), G.target_tensors(cfg, w))
    dfl.write_gguf(tmp_path / "d.gguf", G.draft_head_metadata(dcfg, TAPS, 2047, swa_pattern=[False, True], convention=1),
                   G.draft_head_tensors(dcfg, dw, 1))
    with dfl.GgufFile(tmp_path / "t.gguf") as g:
        fcfg, fw = dfl.open_target(g)
        model_f = dfl.TargetModel(ctx, fcfg, fw)
    with dfl.GgufFile(tmp_path / "d.gguf") as g:
        fdcfg, fdw, ids, mask = dfl.open_dflash_drafter(g, cfg.hidden, cfg.vocab, cfg.n_layers)
        head_f = dfl.DraftHead(ctx, fdcfg, fdw)
    assert ids == TAPS and mask == 2047
    # the mappings are gone: everything the device needs was copied at construction
    model_m, head_m = dfl.TargetModel(ctx, cfg, w), dfl.DraftHead(ctx, dcfg, dw)
    prompt = np.random.default_rng(5).integers(0, cfg.vocab - 1, 24).tolist()
    outs = []
    for model, head in ((model_f, head_f), (model_m, head_m)):
        dec = dfl.SpeculativeDecoder(ctx, model, head, ids, 128, mask)
        first = dec.prefill(prompt)
        tokens, stats = dec.generate(first, 24)
        draft = dec.draft_session.draft_block(tokens[-1], mask, dec.position, want_logits=True)
        outs.append((first, tokens, stats["accepted_drafts"], draft[1].cpu().numpy()))
        dec.close()
    assert outs[0][:3] == outs[1][:3]
    assert np.array_equal(outs[0][3], outs[1][3])  # same bytes on the device -> bit-identical drafter logits


def test_moe_target_from_a_file_with_an_unquantised_router(ctx, oracle, tmp_path):
    """Real MoE files keep ffn_gate_inp as F32.  The verify of a model bound from such a file is checked against the
    CPU oracle's token-by-token forward over the same bytes."""
    cfg = dfl.ModelConfig(n_layers=2, hidden=256, n_q=4, n_kv=2, head_dim=64, ffn=0, vocab=2048, n_expert=8, n_expert_used=2,
                          ffn_expert=256, ffn_shared=256)
    w = dfl.synth_target_weights(cfg, seed=31)
    rng = np.random.default_rng(32)
    for Lw in w["layers"]:
        Lw["router"] = (G.F32, (rng.standard_normal((cfg.n_expert, cfg.hidden)) * 0.5).astype(np.float32).view(np.uint8))
    dfl.write_gguf(tmp_path / "moe.gguf", G.target_metadata(cfg), G.target_tensors(cfg, w))
    with dfl.GgufFile(tmp_path / "moe.gguf") as g:
        assert g.find("blk.0.ffn_gate_inp.weight").type == G.F32
        fcfg, fw = dfl.open_target(g)
        model = dfl.TargetModel(ctx, fcfg, fw)
        omodel, keep = oracle.build_model(fcfg.as_dict(), fw)
        tokens = rng.integers(0, cfg.vocab, 12).tolist()
        sess = dfl.Session(ctx, model, 64, [1])
        out = sess.encode_packed_verify_layer_major(tokens, 0, want_logits=True)
        ostate = oracle.TargetState(fcfg.as_dict(), 64)
        want, want_h = oracle.target_verify(omodel, ostate, tokens, 0, [1])
    got = out.logits.cpu().numpy()
    rel = np.linalg.norm(got - want) / np.linalg.norm(want)
    assert rel <= 5e-3, rel
    hid = out.hidden_capture.cpu().numpy()
    assert np.linalg.norm(hid - want_h) / np.linalg.norm(want_h) <= 5e-3
    top = np.sort(want, axis=1)
    decided = (top[:, -1] - top[:, -2]) > 2e-2 * want.std()
    assert decided.sum() >= 8 and np.array_equal(np.asarray(out.argmax_host)[decided], want.argmax(1)[decided])
    sess.close()
