"""GPU parity: block-causal verify attention against the CPU oracle (per-row f32 softmax
attention over the f16 cache, forward.rs:893-922) and an f64 brute force; <= 1e-2."""
import math

import numpy as np
import pytest

import qwen_llm_amd as dfl

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ctx():
    c = dfl.Context(0, workspace_bytes=256 << 20)
    yield c
    c.close()


def dev(a):
    import torch

    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def make_case(seed, L, n_rows, n_q, n_kv, hd, cap=None):
    rng = np.random.default_rng(seed)
    cap = cap or (L + n_rows + 31) // 32 * 32
    q = rng.standard_normal((n_rows, n_q, hd)).astype(np.float32)
    k = np.full((cap, n_kv, hd), np.nan, np.float16)  # rows past the block are never read as values
    v = np.full((cap, n_kv, hd), np.nan, np.float16)
    k[: L + n_rows] = rng.standard_normal((L + n_rows, n_kv, hd)).astype(np.float16)
    v[: L + n_rows] = rng.standard_normal((L + n_rows, n_kv, hd)).astype(np.float16)
    return q, k, v, cap


def check(got, want, label):
    assert np.all(np.isfinite(got)), f"{label}: non-finite output"
    err = np.max(np.abs(got - want))
    rms = np.sqrt(np.mean(want.astype(np.float64) ** 2))
    rel = np.linalg.norm(got - want) / np.linalg.norm(want)
    # north-star bar: within 1e-2 of the f32 CPU reference (element-wise against max(|ref|, rms))
    assert np.max(np.abs(got - want) / np.maximum(np.abs(want), rms)) <= 1e-2, f"{label}: max abs err {err:.3e}"
    assert rel <= 5e-3, f"{label}: rel l2 {rel:.3e}"


CASES = [
    # (L, n_rows, n_q, n_kv, hd)
    (0, 16, 4, 2, 128), (1, 1, 2, 2, 64), (5, 3, 16, 8, 128), (31, 16, 6, 1, 128), (32, 16, 8, 8, 64),
    (257, 16, 48, 8, 128), (1000, 7, 16, 2, 256), (4096, 16, 48, 8, 128), (777, 16, 32, 2, 128), (300, 16, 16, 8, 128),
]


@pytest.mark.parametrize("L,n_rows,n_q,n_kv,hd", CASES)
@pytest.mark.parametrize("transposed", [False, True])
@pytest.mark.parametrize("q_f16", [False, True])
def test_attn_matches_oracle(ctx, oracle, L, n_rows, n_q, n_kv, hd, transposed, q_f16, canaries):
    q, k, v, cap = make_case(L * 7 + n_q, L, n_rows, n_q, n_kv, hd)
    scale = 1.0 / math.sqrt(hd)
    if q_f16:
        q = q.astype(np.float16).astype(np.float32)
    want = oracle.attn_verify_block(q, k[: L + n_rows], v[: L + n_rows], L, scale)
    qd = dev(q.astype(np.float16) if q_f16 else q)
    vd = dev(np.ascontiguousarray(v.transpose(1, 2, 0))) if transposed else dev(v)
    got = ctx.attn_verify_block(qd, dev(k), vd, L, scale, v_transposed=transposed).cpu().numpy()
    check(got, want, f"L={L} rows={n_rows} q={n_q} kv={n_kv} hd={hd}")


def test_block_causality_and_prefix_visibility(ctx, canaries):
    """row i must not see block rows > i, and must see the whole prefix: perturbing a later block
    row leaves earlier rows bit-identical; perturbing prefix position 0 changes every row"""
    L, n_rows, n_q, n_kv, hd = 200, 16, 8, 4, 128
    q, k, v, cap = make_case(3, L, n_rows, n_q, n_kv, hd)
    scale = 1.0 / math.sqrt(hd)
    base = ctx.attn_verify_block(dev(q), dev(k), dev(v), L, scale).cpu().numpy()
    k2, v2 = k.copy(), v.copy()
    k2[L + 9], v2[L + 9] = 0.5, 3.0
    pert = ctx.attn_verify_block(dev(q), dev(k2), dev(v2), L, scale).cpu().numpy()
    assert np.array_equal(base[:9], pert[:9])
    assert not np.array_equal(base[9], pert[9])
    v3 = v.copy()
    v3[0] += 4.0
    pert = ctx.attn_verify_block(dev(q), dev(k), dev(v3), L, scale).cpu().numpy()
    assert np.all(np.any(pert != base, axis=(1, 2)))


def test_equals_sixteen_single_query_attentions(ctx, canaries):
    """the packed call == n_rows separate one-row calls over growing prefixes (the reference's loop)"""
    L, n_q, n_kv, hd = 333, 12, 4, 128
    q, k, v, cap = make_case(5, L, 16, n_q, n_kv, hd)
    scale = 1.0 / math.sqrt(hd)
    kd, vd = dev(k), dev(v)
    packed = ctx.attn_verify_block(dev(q), kd, vd, L, scale).cpu().numpy()
    for i in [0, 5, 15]:
        one = ctx.attn_verify_block(dev(q[i:i + 1]), kd, vd, L + i, scale).cpu().numpy()
        np.testing.assert_allclose(one[0], packed[i], atol=2e-3, rtol=2e-3)


@pytest.mark.parametrize("L", [32768, 131072])
def test_attn_long_context(ctx, oracle, L, canaries):
    """production shape: 48 q / 8 kv heads, hd 128; checked on a few heads against the oracle
    (the oracle is O(L) per row and head) and through linearity in V over all heads"""
    import torch

    n_rows, n_q, n_kv, hd = 16, 48, 8, 128
    cap = L + 32
    g = torch.Generator(device="cuda").manual_seed(10)
    q = torch.randn((n_rows, n_q, hd), device="cuda", generator=g).half()
    k = torch.randn((cap, n_kv, hd), device="cuda", generator=g).half()
    vt = torch.randn((n_kv, hd, cap), device="cuda", generator=g).half()
    scale = 1.0 / math.sqrt(hd)
    got = ctx.attn_verify_block(q, k, vt, L, scale, v_transposed=True)
    assert torch.isfinite(got).all()
    # oracle on KV head 3 only (its 6 query heads)
    h0 = 3
    qn = q[:, 6 * h0: 6 * h0 + 6].float().cpu().numpy()
    kn = k[: L + n_rows, h0: h0 + 1].cpu().numpy()
    vn = vt[h0, :, : L + n_rows].t().contiguous().unsqueeze(1).cpu().numpy()
    want = oracle.attn_verify_block(qn, kn, vn, L, scale)
    check(got[:, 6 * h0: 6 * h0 + 6].cpu().numpy(), want, f"long L={L}")
    # softmax weights sum to one: with V == const the output is that constant
    ones = torch.full_like(vt, 0.75)
    out1 = ctx.attn_verify_block(q, k, ones, L, scale, v_transposed=True)
    assert (out1 - 0.75).abs().max().item() < 2e-3


@pytest.mark.gpu
@pytest.mark.parametrize("L", [16500, 40000, 70001])
def test_attn_long_context_wide_heads(ctx, oracle, L, canaries):
    """the end-to-end model's shape, 16 q / 2 kv heads of 256, at contexts where one LDS ring fits a CU and the split
    aims at half a workgroup per CU with chunks of 512 to 1024 keys; oracle on one KV head, constant V over all"""
    import torch

    n_rows, n_q, n_kv, hd = 16, 16, 2, 256
    cap = (L + n_rows + 31) // 32 * 32
    g = torch.Generator(device="cuda").manual_seed(11)
    q = torch.randn((n_rows, n_q, hd), device="cuda", generator=g).half()
    k = torch.randn((cap, n_kv, hd), device="cuda", generator=g).half()
    vt = torch.randn((n_kv, hd, cap), device="cuda", generator=g).half()
    scale = 1.0 / math.sqrt(hd)
    got = ctx.attn_verify_block(q, k, vt, L, scale, v_transposed=True)
    assert torch.isfinite(got).all()
    h0 = 1
    qn = q[:, 8 * h0: 8 * h0 + 8].float().cpu().numpy()
    kn = k[: L + n_rows, h0: h0 + 1].cpu().numpy()
    vn = vt[h0, :, : L + n_rows].t().contiguous().unsqueeze(1).cpu().numpy()
    want = oracle.attn_verify_block(qn, kn, vn, L, scale)
    check(got[:, 8 * h0: 8 * h0 + 8].cpu().numpy(), want, f"wide heads L={L}")
    ones = torch.full_like(vt, -1.25)
    out1 = ctx.attn_verify_block(q, k, ones, L, scale, v_transposed=True)
    assert (out1 + 1.25).abs().max().item() < 2e-3
    # a single row at the block's last position sees the same keys through the same split: the same bits
    one = ctx.attn_verify_block(q[15:16].contiguous(), k, vt, L + 15, scale, v_transposed=True)
    if (L + 16).bit_length() == (L + 15 + 1).bit_length():
        assert torch.equal(one[0], got[15])


def test_attn_guards(ctx, canaries):
    import torch

    q = torch.zeros((17, 4, 128), device="cuda")
    k = torch.zeros((64, 2, 128), device="cuda", dtype=torch.float16)
    with pytest.raises(dfl.DFlashError) as e:
        ctx.attn_verify_block(q, k, k, 0, 1.0)
    assert e.value.kind == "BadShape"
    with pytest.raises(dfl.DFlashError) as e:
        ctx.attn_verify_block(q[:16], k, k, 60, 1.0)  # 60 + 16 > capacity 64
    assert e.value.kind == "State"
    k96 = torch.zeros((64, 2, 96), device="cuda", dtype=torch.float16)
    with pytest.raises(dfl.DFlashError) as e:
        ctx.attn_verify_block(torch.zeros((4, 4, 96), device="cuda"), k96, k96, 0, 1.0)
    assert e.value.kind == "Unsupported"
