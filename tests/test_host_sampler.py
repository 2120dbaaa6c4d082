"""Host-side sampler state of the library (no GPU): the random streams must be the
reference's (golden vectors, sampling.rs:1817-1864) and the oracle's, draw for draw."""
import json
import os

import numpy as np
import pytest

import qwen_llm_amd as dfl

GOLD = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "reference_vectors.json")))
pytestmark = pytest.mark.skipif(not os.path.exists(dfl.LIB_PATH), reason="library not built")


def bits(u):
    return int(np.float64(u).view(np.uint64))


def test_xoshiro_unit_draws_golden():
    s = dfl.Sampler(1.0, seed=0)
    assert [bits(u) for u in s.peek(4)] == [int(v, 16) for v in GOLD["unit_f64_bits_seed0"]["values"]]
    s = dfl.Sampler(1.0, seed=int(GOLD["xoshiro256pp"]["seed"], 16))
    raw = [int(v, 16) for v in GOLD["xoshiro256pp"]["values"]]
    assert s.peek(4) == [(r >> 11) / 2.0 ** 53 for r in raw]
    # peeking does not advance; at_draw does
    assert s.peek(2) == s.peek(2) and s.draws == 0
    t = dfl.Sampler.at_draw(s, 2)
    assert t.draws == 2 and t.peek(2) == s.peek(4)[2:]


def test_philox_stream_known_answer():
    case = GOLD["philox4x32_10"]["cases"][0]  # counter 0, key 0
    out = [int(v, 16) for v in case["out"]]
    s = dfl.Sampler(1.0, seed=0, rng_kind=dfl.RNG_PHILOX)
    assert s.peek(1)[0] == ((out[0] | (out[1] << 32)) >> 11) / 2.0 ** 53


@pytest.mark.parametrize("kind", [dfl.RNG_XOSHIRO, dfl.RNG_PHILOX])
def test_streams_match_oracle(oracle, kind):
    import ctypes as C

    for seed in [0, 1, 17, 0x5EED, 2 ** 63 + 12345]:
        s = dfl.Sampler(0.7, top_k=20, top_p=0.95, seed=seed, rng_kind=kind, draws=3)
        o = oracle.make_sampler(0.7, 20, 0.95, 0.0, seed, kind, draws=3)
        want = [oracle.lib().orc_sampler_next_unit(C.byref(o)) for _ in range(40)]
        assert s.peek(40) == want


def test_config_validation():
    """sampling.rs:133-144"""
    for kw, kind in [({"temperature": -1.0}, "InvalidTemperature"), ({"temperature": float("nan")}, "InvalidTemperature"),
                     ({"top_p": 0.0}, "InvalidTopP"), ({"top_p": 1.5}, "InvalidTopP"), ({"min_p": -0.1}, "InvalidMinP"),
                     ({"min_p": 1.1}, "InvalidMinP")]:
        with pytest.raises(dfl.DFlashError) as e:
            dfl.Sampler(**kw)
        assert e.value.kind == kind
