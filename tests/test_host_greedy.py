"""dflash_accept_greedy (host-only): the argmax accept loop of qwen/dflash.rs:838-858 in the decision
format of decide_dflash_accept_prefix; checked against the oracle's accept-prefix with a greedy
sampler on one-hot logits, and against the by-value cases of accept.rs:236-330."""
import numpy as np
import pytest

import qwen_llm_amd as dfl


def one_hot_logits(argmax, vocab):
    lg = np.zeros((len(argmax), vocab), np.float32)
    for r, t in enumerate(argmax):
        lg[r, t] = 5.0
    return lg


def test_by_value_cases():
    d = dfl.accept_greedy([7, 1, 2, 3], [1, 2, 9, 4], budget=100)
    assert d.key() == ([1, 2], dfl.CARRY_CORRECTION, 9, dfl.STOP_NONE, 3)
    d = dfl.accept_greedy([7, 1, 2, 3], [1, 2, 3, 4], budget=100)
    assert d.key() == ([1, 2, 3], dfl.CARRY_BONUS, 4, dfl.STOP_NONE, 4)
    d = dfl.accept_greedy([7, 1, 2, 3], [1, 2, 3, 4], budget=2)
    assert d.key() == ([1, 2], dfl.CARRY_NONE, 0, dfl.STOP_TOKEN_LIMIT, 2)
    d = dfl.accept_greedy([7, 1, 2, 3], [1, 2, 3, 4], budget=100, stop_ids=[2])
    assert d.key() == ([1, 2], dfl.CARRY_NONE, 0, dfl.STOP_EOS, 2)
    d = dfl.accept_greedy([7, 1, 2, 3], [1, 2, 3, 4], budget=100, stop_ids=[7])
    assert d.key() == ([], dfl.CARRY_NONE, 0, dfl.STOP_EOS, 0)
    d = dfl.accept_greedy([7, 1], [1, 2], budget=0)
    assert d.key() == ([], dfl.CARRY_NONE, 0, dfl.STOP_TOKEN_LIMIT, 0)
    d = dfl.accept_greedy([7], [3], budget=4)
    assert d.key() == ([], dfl.CARRY_BONUS, 3, dfl.STOP_NONE, 1)
    with pytest.raises(dfl.DFlashError):
        dfl.accept_greedy([], [], budget=1)
    with pytest.raises(dfl.DFlashError):
        dfl.accept_greedy(list(range(17)), list(range(17)), budget=1)


def test_matches_oracle_accept_prefix_on_random_blocks(oracle):
    rng = np.random.default_rng(0)
    vocab = 12
    for trial in range(400):
        n = int(rng.integers(1, 17))
        verify_input = rng.integers(0, vocab, n).tolist()
        argmax = rng.integers(0, vocab, n).tolist()
        for i in range(n - 1):  # make long accepted prefixes likely
            if rng.random() < 0.8:
                argmax[i] = verify_input[i + 1]
        budget = int(rng.integers(0, 20))
        stops = rng.integers(0, vocab, int(rng.integers(0, 3))).tolist()
        got = dfl.accept_greedy(verify_input, argmax, budget, stops)
        samp = oracle.make_sampler(temperature=0.0)
        rc, want = oracle.decide_accept_prefix(verify_input, one_hot_logits(argmax, vocab), vocab, None, samp, budget, stops)
        assert rc == 0
        assert got.key() == want.key(), (trial, verify_input, argmax, budget, stops)
